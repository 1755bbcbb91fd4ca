// HipLlmExecutor: an LlmExecutor whose attention and KV cache live on an
// MI355X behind the C ABI of libmi355_attn.so. It takes the seat of
// LlmLiteRtCompiledModelExecutor
// (runtime/executor/llm_litert_compiled_model_executor.h) and keeps its
// observable behaviour: prefill chunking over static runner lengths, the
// "last token of a prefill is executed by the next call" rule, positions,
// GetCurrentStep, Reset and the status codes of the error paths.
#ifndef LITERT_LM_AMD_EXECUTOR_HIP_LLM_EXECUTOR_H_
#define LITERT_LM_AMD_EXECUTOR_HIP_LLM_EXECUTOR_H_

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "attention_backend.h"
#include "decoder_layers.h"
#include "llm_executor_base.h"
#include "prefill_planner.h"

namespace litert::lm {

struct HipExecutorOptions {
  // Static sequence lengths of the prefill runners; stands in for the
  // prefill_* signatures found in the model
  // (runtime/executor/litert_compiled_model_executor_utils.cc:262-298).
  std::vector<int> prefill_runner_lengths = {1024};
  // The reference loop never runs for a one-id chunk, so a token left pending
  // by an earlier call is overwritten and lost
  // (llm_litert_compiled_model_executor.cc:187,244). false (default): the
  // reference behaviour, step counts and positions included; true: execute the
  // pending token first (opt-in fix: GetCurrentStep then reads one higher than
  // the reference's after such a call).
  bool execute_pending_on_single_id_chunk = false;
  // Where activations live. kDevice: q / k / v / attention output, logits and the sampled id stay in device memory
  // for the whole forward pass, every layer is queued on the attention backend's stream without a wait in between,
  // Decode(tokens) samples on the device (libmi355_sampler.so) and only the id comes back; Prefill returns after
  // queueing unless the prefill parameters ask to wait. This is the reference's GPU arrangement
  // (llm_litert_compiled_model_executor.cc:536-566,753-755). kHost: float32 host rows staged through the boundary
  // per call. kAuto: kDevice when the decoder layers have a device form and no backend was injected, else kHost.
  enum class Residency { kAuto, kHost, kDevice };
  Residency residency = Residency::kAuto;
  // Device-resident one-token passes over layers with a transform: true (default) queues the step before
  // attention and the attention as one call per layer where the backend has one (same results); false keeps
  // the two calls (comparisons).
  bool single_call_decode_step = true;
};

// One forward pass as the executor issued it (kept for tests and debugging).
struct ExecutorRunRecord {
  bool is_decode;
  std::vector<int32_t> tokens;
  std::vector<int32_t> positions;
};

class HipLlmExecutor : public LlmExecutorBase {
 public:
  // `backend` may be null: then an MI355X backend is created from the layers'
  // shape and the settings (fp16 activations -> fp16 cache, else fp32).
  static StatusOr<std::unique_ptr<HipLlmExecutor>> Create(LlmExecutorSettings settings,
                                                          std::unique_ptr<DecoderLayers> layers,
                                                          HipExecutorOptions options = {},
                                                          std::unique_ptr<AttentionBackend> backend = nullptr);

  Status Prefill(const ExecutorInputs& inputs) override { return Prefill(inputs, ExecutorPrefillParams()); }
  Status Prefill(const ExecutorInputs& inputs, const ExecutorPrefillParams& params) override;
  Status Decode(TensorBuffer& output_tokens) override;
  Status Decode(const ExecutorInputs& inputs, TensorBuffer& output_logits) override;
  StatusOr<TensorBuffer> DecodeLogits(const ExecutorInputs& inputs) override;
  string_view ExecutorBackendName() const override { return "MI355X HIP attention"; }
  StatusOr<int> GetVocabSize() override { return layers_->VocabSize(); }
  // What the caller expects: tokens handed in so far, the deferred one included
  // (llm_litert_compiled_model_executor.h:95-97).
  StatusOr<int> GetCurrentStep() const override { return current_step_ + (next_input_token_id_ == -1 ? 0 : 1); }
  StatusOr<LlmExecutorSettings> GetExecutorSettings() const override { return settings_; }
  Status Reset() override;

  ~HipLlmExecutor() override;
  const std::vector<ExecutorRunRecord>& run_records() const { return records_; }
  AttentionBackend* attention_backend() { return backend_.get(); }
  bool device_resident() const { return device_ != nullptr; }
  // Waits for everything this executor has queued (a no-op when host-staged).
  Status WaitForCompletion();

 private:
  HipLlmExecutor(LlmExecutorSettings settings, std::unique_ptr<DecoderLayers> layers, HipExecutorOptions options,
                 std::unique_ptr<AttentionBackend> backend);
  Status PrefillInternal(const int32_t* ids, int count);
  // Picks the id of a decode step, runs it and leaves the logits in logits_.
  Status DecodeStep(const ExecutorInputs& inputs);
  // Runs all layers for `tokens` at `positions` (consecutive, starting at the
  // cache row of the first one); logits of the last token if asked for.
  Status RunTokens(const std::vector<int32_t>& tokens, const std::vector<int32_t>& positions, bool is_decode,
                   bool want_logits);
  Status RunTokensOnDevice(const std::vector<int32_t>& tokens, const std::vector<int32_t>& positions, bool is_decode,
                           bool want_logits);
  // Device-resident decode step: logits stay in device memory (copied to logits_ only when `fetch_logits`).
  Status FetchLogits();
  struct DeviceState;  // device buffers, sampler handle, pinned id slot
  Status InitDeviceState();

  LlmExecutorSettings settings_;
  std::unique_ptr<DecoderLayers> layers_;
  HipExecutorOptions options_;
  std::unique_ptr<AttentionBackend> backend_;
  SortedPrefillSignatureMap prefill_signature_map_;
  int current_step_ = 0;
  int next_input_token_id_ = -1;
  TensorBuffer logits_;  // [1, 1, vocab] float32
  std::vector<float> q_, k_, v_, attn_;
  std::vector<ExecutorRunRecord> records_;
  std::unique_ptr<DeviceState> device_;  // null: host-staged
};

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_HIP_LLM_EXECUTOR_H_
