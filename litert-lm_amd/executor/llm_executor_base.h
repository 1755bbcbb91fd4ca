// The executor interface this build plugs into: same methods, argument meaning
// and default behaviour (UnimplementedError naming the backend) as
// LlmExecutorBase in runtime/executor/llm_executor_base.h:33-121, so that a
// class derived from this one compiles against the reference's header once the
// stand-in types (Status, string_view, TensorBuffer) are swapped for absl's and
// LiteRT's.
#ifndef LITERT_LM_AMD_EXECUTOR_LLM_EXECUTOR_BASE_H_
#define LITERT_LM_AMD_EXECUTOR_LLM_EXECUTOR_BASE_H_

#include <string>

#include "llm_executor_io_types.h"
#include "llm_executor_settings.h"
#include "status.h"
#include "tensor_buffer.h"

namespace litert::lm {

class LlmExecutorBase {
 public:
  virtual ~LlmExecutorBase() = default;

  // Token ids `[batch, sequence_length]`.
  virtual Status Prefill(const ExecutorInputs& inputs) = 0;
  virtual Status Prefill(const ExecutorInputs& inputs, const ExecutorPrefillParams& params) {
    (void)inputs;
    (void)params;
    return Unimplemented("Prefill with prefill params");
  }
  // Fills `[batch, sequence_length]` int32 output tokens.
  virtual Status Decode(TensorBuffer& output_tokens) = 0;
  // Logits `[batch, sequence_length, vocab_size]` float32, no sampling.
  virtual Status Decode(const ExecutorInputs& inputs, TensorBuffer& output_logits) {
    (void)inputs;
    (void)output_logits;
    return Unimplemented("Decode for logits output");
  }
  virtual StatusOr<TensorBuffer> DecodeLogits(const ExecutorInputs& inputs) {
    (void)inputs;
    return Unimplemented("Decode for logits output");
  }
  virtual string_view ExecutorBackendName() const = 0;
  virtual StatusOr<int> GetVocabSize() { return Unimplemented("GetVocabSize"); }
  virtual StatusOr<int> GetCurrentStep() const { return Unimplemented("GetCurrentStep"); }
  virtual StatusOr<LlmExecutorSettings> GetExecutorSettings() const { return Unimplemented("GetExecutorSettings"); }
  // Vision embeddings of image `image_index` for the prefill that follows (llm_executor_base.h:108).
  virtual Status FillVisionEmbeddings(const ExecutorVisionData& vision_input, int image_index) {
    (void)vision_input;
    (void)image_index;
    return Unimplemented("FillVisionEmbeddings");
  }
  virtual Status Reset() { return Unimplemented("Reset"); }

 private:
  Status Unimplemented(const char* what) const {
    return UnimplementedError(std::string(what) + " not implemented for backend: " + std::string(ExecutorBackendName()));
  }
};

using LlmExecutor = LlmExecutorBase;  // runtime/executor/llm_executor.h:8

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_LLM_EXECUTOR_BASE_H_
