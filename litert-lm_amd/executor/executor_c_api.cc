// C test surface of HipLlmExecutor for the Python tests (ctypes): create an
// executor over the synthetic decoder layers, drive Prefill / Decode, read the
// trace of forward passes. Status codes are absl::StatusCode integers; error
// text is malloc'd for the caller to free().
#include <cstdlib>
#include <cstring>
#include <memory>

#include "hip_llm_executor.h"

using namespace litert::lm;

namespace {
int Finish(const Status& s, char** err) {
  if (!s.ok() && err) {
    *err = static_cast<char*>(malloc(s.message().size() + 1));
    if (*err) memcpy(*err, s.message().c_str(), s.message().size() + 1);
  }
  return static_cast<int>(s.code());
}
ExecutorInputs IdsInput(const int32_t* ids, int batch, int n) {
  return ExecutorInputs(ExecutorTextData(TensorBuffer::CopyFrom(ElementType::kInt32, {batch, n}, ids)));
}
}  // namespace

extern "C" {

struct hle_config {
  int32_t num_layers, num_q_heads, num_kv_heads, vocab, max_num_tokens;
  const int32_t* layer_window;       // [num_layers] or null
  const int32_t* runner_lengths;     // [num_runners]
  int32_t num_runners;
  int32_t fp16_activations;          // 0: float32, 1: float16
  int32_t recording_backend;         // 1: no GPU, attention returns zeros and records calls
  int32_t execute_pending_on_single_id_chunk;
  float softcap;
  int32_t pre_attention;             // 1: the layers hand over raw projections; Gemma-3-like norm + rotary constants
};

int hle_create(const hle_config* c, void** out, char** err) {
  *out = nullptr;
  AttentionShape shape;
  shape.num_layers = c->num_layers;
  shape.num_q_heads = c->num_q_heads;
  shape.num_kv_heads = c->num_kv_heads;
  shape.head_dim = 256;
  shape.max_tokens = c->max_num_tokens;
  shape.softcap = c->softcap;
  if (c->layer_window) shape.layer_window.assign(c->layer_window, c->layer_window + c->num_layers);
  if (c->pre_attention) shape.transforms = SyntheticDecoderLayers::Transforms(shape);
  auto settings = LlmExecutorSettings::CreateDefault(Backend::GPU_HIP);
  if (!settings.ok()) return Finish(settings.status(), err);
  settings->SetMaxNumTokens(c->max_num_tokens);
  settings->SetActivationDataType(c->fp16_activations ? ActivationDataType::FLOAT16 : ActivationDataType::FLOAT32);
  HipExecutorOptions options;
  options.prefill_runner_lengths.assign(c->runner_lengths, c->runner_lengths + c->num_runners);
  options.execute_pending_on_single_id_chunk = c->execute_pending_on_single_id_chunk != 0;
  std::unique_ptr<AttentionBackend> backend;
  if (c->recording_backend) backend = std::make_unique<RecordingAttentionBackend>(shape);
  auto ex = HipLlmExecutor::Create(*settings, std::make_unique<SyntheticDecoderLayers>(shape, c->vocab), options,
                                   std::move(backend));
  if (!ex.ok()) return Finish(ex.status(), err);
  *out = ex->release();
  return 0;
}

void hle_destroy(void* h) { delete static_cast<HipLlmExecutor*>(h); }

int hle_prefill(void* h, const int32_t* ids, int32_t batch, int32_t n, char** err) {
  return Finish(static_cast<HipLlmExecutor*>(h)->Prefill(IdsInput(ids, batch, n)), err);
}

int hle_decode(void* h, int32_t* out_token, char** err) {
  TensorBuffer out = TensorBuffer::Create(ElementType::kInt32, {1, 1});
  Status s = static_cast<HipLlmExecutor*>(h)->Decode(out);
  if (s.ok()) *out_token = out.as<int32_t>()[0];
  return Finish(s, err);
}

// explicit_id < 0: use the pending token.
int hle_decode_logits(void* h, int32_t explicit_id, float* logits, char** err) {
  auto* ex = static_cast<HipLlmExecutor*>(h);
  ExecutorInputs inputs = explicit_id >= 0 ? IdsInput(&explicit_id, 1, 1) : ExecutorInputs();
  auto r = ex->DecodeLogits(inputs);
  if (!r.ok()) return Finish(r.status(), err);
  memcpy(logits, r->as<float>(), r->PackedSize());
  return 0;
}

int hle_current_step(void* h) { return *static_cast<HipLlmExecutor*>(h)->GetCurrentStep(); }
int hle_vocab_size(void* h) { return *static_cast<HipLlmExecutor*>(h)->GetVocabSize(); }
int hle_max_num_tokens(void* h) { return static_cast<HipLlmExecutor*>(h)->GetExecutorSettings()->GetMaxNumTokens(); }
int hle_reset(void* h, char** err) { return Finish(static_cast<HipLlmExecutor*>(h)->Reset(), err); }
const char* hle_backend_name(void* h) {
  static thread_local std::string name;
  name = static_cast<HipLlmExecutor*>(h)->ExecutorBackendName();
  return name.c_str();
}

int hle_num_runs(void* h) { return static_cast<int>(static_cast<HipLlmExecutor*>(h)->run_records().size()); }
// Copies run `i`: returns its token count; is_decode, tokens and positions are filled (capacity `cap`).
int hle_get_run(void* h, int i, int32_t* is_decode, int32_t* tokens, int32_t* positions, int cap) {
  const auto& r = static_cast<HipLlmExecutor*>(h)->run_records()[i];
  *is_decode = r.is_decode ? 1 : 0;
  const int n = static_cast<int>(r.tokens.size());
  for (int j = 0; j < n && j < cap; ++j) {
    tokens[j] = r.tokens[j];
    positions[j] = r.positions[j];
  }
  return n;
}

int hle_backend_from_string(const char* s) {
  auto b = GetBackendFromString(s);
  return b.ok() ? static_cast<int>(*b) : -static_cast<int>(b.status().code());
}

// Chunk plan for `n` ids over the given runner lengths: fills lens[] with the
// runner length and counts[] with the ids of each call; returns the number of calls.
int hle_plan(const int32_t* runner_lengths, int num_runners, int n, int32_t* lens, int32_t* counts, int cap) {
  SortedPrefillSignatureMap m;
  for (int i = 0; i < num_runners; ++i) m[runner_lengths[i]] = std::to_string(runner_lengths[i]);
  auto g = GetOptimizedPrefillWorkGroups(m, n);
  if (!g.ok()) return -static_cast<int>(g.status().code());
  int k = 0;
  for (const auto& e : *g) {
    if (k < cap) {
      lens[k] = std::stoi(e.first);
      counts[k] = e.second;
    }
    ++k;
  }
  return k;
}

}  // extern "C"
