// Argument types of the executor interface, text path only. Mirrors the parts
// of runtime/executor/llm_executor_io_types.h that the hot path reads:
// ExecutorInputs::GetTextTokenIdsPtr (:172-213) and ExecutorPrefillParams
// (:217-250). Vision data is carried as a type only (the executor interface names
// it); audio inputs are outside this build.
#ifndef LITERT_LM_AMD_EXECUTOR_LLM_EXECUTOR_IO_TYPES_H_
#define LITERT_LM_AMD_EXECUTOR_LLM_EXECUTOR_IO_TYPES_H_

#include <atomic>
#include <optional>
#include <utility>

#include "status.h"
#include "tensor_buffer.h"

namespace litert::lm {

class ExecutorTextData {
 public:
  ExecutorTextData() = default;
  // token_ids: int32 `[batch_size, tokens_per_batch]`.
  explicit ExecutorTextData(TensorBuffer&& token_ids) : token_ids_(std::move(token_ids)) {}
  const TensorBuffer& GetTokenIds() const { return token_ids_; }
  TensorBuffer& GetMutableTokenIds() { return token_ids_; }
  void SetTokenIds(TensorBuffer&& token_ids) { token_ids_ = std::move(token_ids); }

 private:
  TensorBuffer token_ids_;
};

// Vision embeddings `[vision_tokens, model_dim]` and per-layer embeddings `[layers, vision_tokens, dim]`
// (llm_executor_io_types.h:81-116). No executor of this build consumes them: the type exists so that
// LlmExecutorBase::FillVisionEmbeddings has the reference's signature.
class ExecutorVisionData {
 public:
  static constexpr int kSpecialToken = -1;
  ExecutorVisionData() = default;
  ExecutorVisionData(std::optional<TensorBuffer>&& embeddings, std::optional<TensorBuffer>&& per_layer_embeddings)
      : embeddings_(std::move(embeddings)), per_layer_embeddings_(std::move(per_layer_embeddings)) {}
  StatusOr<const TensorBuffer*> GetEmbeddingsPtr() const {
    if (!embeddings_.has_value()) return NotFoundError("ExecutorVisionData::embeddings_ is not set.");
    return &*embeddings_;
  }
  StatusOr<const TensorBuffer*> GetPerLayerEmbeddingsPtr() const {
    if (!per_layer_embeddings_.has_value())
      return NotFoundError("ExecutorVisionData::per_layer_embeddings_ is not set.");
    return &*per_layer_embeddings_;
  }

 private:
  std::optional<TensorBuffer> embeddings_;
  std::optional<TensorBuffer> per_layer_embeddings_;
};

class ExecutorInputs {
 public:
  ExecutorInputs() = default;
  explicit ExecutorInputs(std::optional<ExecutorTextData> text) : text_data_(std::move(text)) {}

  StatusOr<const ExecutorTextData*> GetTextDataPtr() const {
    if (!text_data_.has_value()) return NotFoundError("ExecutorInputs::text_data_ is not set.");
    return &*text_data_;
  }
  StatusOr<const TensorBuffer*> GetTextTokenIdsPtr() const {
    ASSIGN_OR_RETURN(const ExecutorTextData* text, GetTextDataPtr());
    return &text->GetTokenIds();
  }
  void SetTextData(ExecutorTextData&& text) { text_data_ = std::move(text); }

 private:
  std::optional<ExecutorTextData> text_data_;
};

class ExecutorPrefillParams {
 public:
  ExecutorPrefillParams() = default;
  ExecutorPrefillParams(int current_step, bool wait_for_completion, const std::atomic_bool* cancel)
      : current_step_(current_step), wait_for_completion_(wait_for_completion), cancel_(cancel) {}
  int GetCurrentStep() const { return current_step_; }
  void SetCurrentStep(int s) { current_step_ = s; }
  bool GetWaitForCompletion() const { return wait_for_completion_; }
  void SetWaitForCompletion(bool w) { wait_for_completion_ = w; }
  const std::atomic_bool* GetCancelFlag() const { return cancel_; }
  void SetCancelFlag(const std::atomic_bool* c) { cancel_ = c; }

 private:
  int current_step_ = -1;
  bool wait_for_completion_ = false;
  const std::atomic_bool* cancel_ = nullptr;
};

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_LLM_EXECUTOR_IO_TYPES_H_
