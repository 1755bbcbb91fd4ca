#include "pipeline.h"

#include <string>
#include <utility>

namespace litert::lm {
namespace {

constexpr int kDefaultMaxNumTokens = 4096;  // when the executor has no settings to ask (pipeline.cc:50-62)

int TryGetMaxNumTokens(const LlmExecutor& executor) {
  auto settings = executor.GetExecutorSettings();
  return settings.ok() ? settings->GetMaxNumTokens() : kDefaultMaxNumTokens;
}

// (true, cache_full): the loop ends; cache_full tells why.
std::pair<bool, bool> ShouldStop(bool hit_stop_tokens, int benchmark_decode_token_count, int num_decoded_steps,
                                 int current_step, int max_num_tokens) {
  if (hit_stop_tokens && benchmark_decode_token_count == 0) return {true, false};
  if (benchmark_decode_token_count > 0 && num_decoded_steps >= benchmark_decode_token_count) return {true, false};
  if (current_step >= max_num_tokens) return {true, true};
  return {false, false};
}

// One decode step with sampling inside the executor (pipeline.cc:160-227).
class DecodeInternalSamplingOneStep {
 public:
  DecodeInternalSamplingOneStep(LlmExecutor& executor, const StopTokenDetector& detector,
                                std::optional<BenchmarkInfo>& benchmark_info)
      : executor_(executor), benchmark_info_(benchmark_info), detector_(detector) {
    output_tokens_ = TensorBuffer::Create(ElementType::kInt32, {1, 1});
  }
  StatusOr<bool> Run() {
    if (benchmark_info_.has_value()) RETURN_IF_ERROR(benchmark_info_->TimeMarkDelta("executor_decode_and_sample"));
    RETURN_IF_ERROR(executor_.Decode(output_tokens_));
    if (benchmark_info_.has_value()) RETURN_IF_ERROR(benchmark_info_->TimeMarkDelta("executor_decode_and_sample"));
    if (output_tokens_.NumElements() != 1) return InternalError("Unexpected number of decoded tokens.");
    RETURN_IF_ERROR(detector_.ProcessTokens(output_tokens_.as<int32_t>(), 1));
    return detector_.AllDone();
  }
  int token() const { return output_tokens_.as<int32_t>()[0]; }

 private:
  LlmExecutor& executor_;
  std::optional<BenchmarkInfo>& benchmark_info_;
  StopTokenDetector detector_;
  TensorBuffer output_tokens_;
};

}  // namespace

StatusOr<int> Prefill(LlmExecutor& executor, std::vector<int> ids, int bos_token_id, bool wait_for_completion,
                      std::optional<BenchmarkInfo>& benchmark_info) {
  int benchmark_prefill_token_count = 0;
  if (benchmark_info.has_value()) {
    benchmark_prefill_token_count = benchmark_info->GetBenchmarkParams().num_prefill_tokens;
    RETURN_IF_ERROR(benchmark_info->TimePrefillTurnStart());
  }
  if (benchmark_prefill_token_count > 0) ids.resize(benchmark_prefill_token_count);
  else ids.insert(ids.begin(), bos_token_id);
  const int max_num_tokens = TryGetMaxNumTokens(executor);
  if (static_cast<int>(ids.size()) >= max_num_tokens)
    return InvalidArgumentError("Input token ids are too long. Exceeding the maximum number of tokens allowed: " +
                                std::to_string(ids.size()) + " >= " + std::to_string(max_num_tokens));
  if (ids.empty()) return InternalError("Input token ids are empty.");
  const int last_token_id = ids.back();
  const int count = static_cast<int>(ids.size());
  ExecutorPrefillParams params;
  params.SetWaitForCompletion(wait_for_completion);
  RETURN_IF_ERROR(executor.Prefill(
      ExecutorInputs(ExecutorTextData(TensorBuffer::CopyFrom(ElementType::kInt32, {1, count}, ids.data()))), params));
  if (benchmark_info.has_value()) RETURN_IF_ERROR(benchmark_info->TimePrefillTurnEnd(ids.size()));
  return last_token_id;
}

Status DecodeStreaming(LlmExecutor& executor, const StopTokenDetector& stop_token_detector,
                       std::optional<BenchmarkInfo>& benchmark_info, const std::function<void(int)>& on_next,
                       const std::function<void(const Status&)>& on_error) {
  int benchmark_decode_token_count = 0;
  if (benchmark_info.has_value()) {
    benchmark_decode_token_count = benchmark_info->GetBenchmarkParams().num_decode_tokens;
    RETURN_IF_ERROR(benchmark_info->TimeDecodeTurnStart());
  }
  int num_decoded_steps = 0;
  const int max_num_tokens = TryGetMaxNumTokens(executor);
  DecodeInternalSamplingOneStep run_one_step(executor, stop_token_detector, benchmark_info);
  while (true) {
    StatusOr<bool> hit_stop_tokens = run_one_step.Run();
    if (!hit_stop_tokens.ok()) {
      if (on_error) on_error(hit_stop_tokens.status());
      return hit_stop_tokens.status();
    }
    ++num_decoded_steps;
    if (on_next) on_next(run_one_step.token());
    ASSIGN_OR_RETURN(const int current_step, executor.GetCurrentStep());
    const auto stop = ShouldStop(*hit_stop_tokens, benchmark_decode_token_count, num_decoded_steps, current_step,
                                 max_num_tokens);
    if (stop.second && on_error) on_error(InternalError("Maximum kv-cache size reached."));
    if (stop.first) break;
  }
  if (benchmark_info.has_value()) RETURN_IF_ERROR(benchmark_info->TimeDecodeTurnEnd(num_decoded_steps));
  return OkStatus();
}

StatusOr<std::vector<int>> Decode(LlmExecutor& executor, const StopTokenDetector& stop_token_detector,
                                  std::optional<BenchmarkInfo>& benchmark_info) {
  std::vector<int> tokens;
  RETURN_IF_ERROR(DecodeStreaming(executor, stop_token_detector, benchmark_info,
                                  [&](int id) { tokens.push_back(id); }, nullptr));
  return tokens;
}

}  // namespace litert::lm
