// A scripted executor for tests of the code above the executor interface: it
// checks that Prefill receives the expected ids and hands out a fixed list of
// decode tokens, counting steps the way the reference's fake does
// (runtime/executor/fake_llm_executor.h:31-91, fake_llm_executor.cc:60-170:
// a prefill advances the step by the number of ids, a decode by one; calling
// either more often than scripted is kInvalidArgument; max_num_tokens 1024).
#ifndef LITERT_LM_AMD_EXECUTOR_FAKE_LLM_EXECUTOR_H_
#define LITERT_LM_AMD_EXECUTOR_FAKE_LLM_EXECUTOR_H_

#include <limits>
#include <string>
#include <utility>
#include <vector>

#include "llm_executor_base.h"

namespace litert::lm {

class FakeLlmExecutor : public LlmExecutorBase {
 public:
  FakeLlmExecutor(int vocab_size, std::vector<std::vector<int>> prefill_tokens_set,
                  std::vector<std::vector<int>> decode_tokens_set, int batch_size = 1)
      : vocab_size_(vocab_size),
        prefill_tokens_set_(std::move(prefill_tokens_set)),
        decode_tokens_set_(std::move(decode_tokens_set)),
        batch_size_(batch_size),
        settings_(*LlmExecutorSettings::CreateDefault(Backend::GPU_HIP)) {
    settings_.SetMaxNumTokens(1024);
  }

  Status Prefill(const ExecutorInputs& inputs) override {
    if (prefill_times_ >= prefill_tokens_set_.size())
      return InvalidArgumentError("Prefill function has been called more times than the number of expected prefill tokens." +
                                  std::to_string(prefill_times_));
    ASSIGN_OR_RETURN(const TensorBuffer* ids, inputs.GetTextTokenIdsPtr());
    RETURN_IF_ERROR(CheckEquivalent(prefill_tokens_set_[prefill_times_], ids->as<int32_t>(), ids->NumElements()));
    ++prefill_times_;
    current_step_ += static_cast<int>(ids->NumElements());
    return OkStatus();
  }
  Status Prefill(const ExecutorInputs& inputs, const ExecutorPrefillParams& params) override {
    last_wait_for_completion_ = params.GetWaitForCompletion();
    return Prefill(inputs);
  }

  Status Decode(TensorBuffer& output_tokens) override {
    RETURN_IF_ERROR(CheckDecodeBudget());
    const std::vector<int>& tokens = decode_tokens_set_[decode_times_];
    for (size_t i = 0; i < tokens.size(); ++i) output_tokens.as<int32_t>()[i] = tokens[i];
    ++decode_times_;
    ++current_step_;
    return OkStatus();
  }

  Status Decode(const ExecutorInputs& inputs, TensorBuffer& output_logits) override {
    RETURN_IF_ERROR(CheckDecodeBudget());
    if (decode_times_ > 0) {  // the caller must feed back what the last step produced
      ASSIGN_OR_RETURN(const TensorBuffer* ids, inputs.GetTextTokenIdsPtr());
      RETURN_IF_ERROR(CheckEquivalent(decode_tokens_set_[decode_times_ - 1], ids->as<int32_t>(), ids->NumElements()));
    }
    FillLogits(decode_tokens_set_[decode_times_], output_logits.as<float>());
    ++decode_times_;
    ++current_step_;
    return OkStatus();
  }

  StatusOr<TensorBuffer> DecodeLogits(const ExecutorInputs& inputs) override {
    TensorBuffer logits = TensorBuffer::Create(ElementType::kFloat32, {batch_size_, 1, vocab_size_});
    RETURN_IF_ERROR(Decode(inputs, logits));
    return logits;
  }

  string_view ExecutorBackendName() const override { return "FakeLlmExecutorBackend"; }
  StatusOr<int> GetVocabSize() override { return vocab_size_; }
  StatusOr<int> GetCurrentStep() const override { return current_step_; }
  StatusOr<LlmExecutorSettings> GetExecutorSettings() const override { return settings_; }
  LlmExecutorSettings* GetMutableExecutorSettings() { return &settings_; }
  bool last_wait_for_completion() const { return last_wait_for_completion_; }

 private:
  Status CheckDecodeBudget() const {
    if (decode_times_ >= decode_tokens_set_.size())
      return InvalidArgumentError("Decode function has been called more times than the number of expected decode tokens." +
                                  std::to_string(decode_times_));
    return OkStatus();
  }
  static Status CheckEquivalent(const std::vector<int>& expected, const int32_t* actual, size_t count) {
    if (expected.size() != count)
      return InvalidArgumentError("Expected token size is " + std::to_string(expected.size()) + " but got " +
                                  std::to_string(count));
    for (size_t i = 0; i < count; ++i)
      if (expected[i] != actual[i])
        return InvalidArgumentError("Expected token at index " + std::to_string(i) + " is " +
                                    std::to_string(expected[i]) + " but got " + std::to_string(actual[i]));
    return OkStatus();
  }
  // The scripted id gets the largest float, every other entry the lowest.
  void FillLogits(const std::vector<int>& ids, float* logits) const {
    for (size_t i = 0; i < ids.size(); ++i)
      for (int j = 0; j < vocab_size_; ++j)
        logits[i * vocab_size_ + j] = ids[i] == j ? std::numeric_limits<float>::max() : std::numeric_limits<float>::lowest();
  }

  int vocab_size_;
  std::vector<std::vector<int>> prefill_tokens_set_, decode_tokens_set_;
  int batch_size_;
  size_t prefill_times_ = 0, decode_times_ = 0;
  int current_step_ = 0;
  bool last_wait_for_completion_ = false;
  LlmExecutorSettings settings_;
};

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_FAKE_LLM_EXECUTOR_H_
