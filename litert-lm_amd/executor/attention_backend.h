// What the executor needs from an attention implementation: a KV cache it can
// append rows to, and prefill / decode attention over it. Mi355AttentionBackend
// forwards to the C ABI of libmi355_attn.so (include/mi355_attn.h);
// RecordingAttentionBackend keeps only the call trace and returns zeros, so the
// executor's host logic can be tested on a machine without a GPU (the same
// role FakeLlmExecutor plays for the reference's callers,
// runtime/executor/fake_llm_executor.h:31-91).
#ifndef LITERT_LM_AMD_EXECUTOR_ATTENTION_BACKEND_H_
#define LITERT_LM_AMD_EXECUTOR_ATTENTION_BACKEND_H_

#include <memory>
#include <string>
#include <vector>

#include "status.h"

struct mi355_attn;

namespace litert::lm {

// Constants of the step right before attention for one layer: RMS norm of the
// query / key (/ value) heads and the rotary embedding (in the reference part of
// the model graph; the NPU flow runs the rotary tables and the cache update as
// signatures of their own, llm_litert_npu_compiled_model_executor.cc:82-110).
struct LayerTransform {
  bool norm_q = false, norm_k = false, norm_v = false;
  std::vector<float> q_weight, k_weight;  // [head_dim] or empty: no learned scale
  float eps = 1e-6f;
  float weight_offset = 1.f;              // learned scale = weight_offset + weight
  std::vector<float> rope_inv_freq;       // [head_dim / 2] or empty: no rotation
};

struct AttentionShape {
  int num_layers = 0;
  int num_q_heads = 0;
  int num_kv_heads = 0;
  int head_dim = 256;
  int max_tokens = 0;
  std::vector<int> layer_window;  // per layer, 0 = global
  float scale = 0.f;              // 0 => head_dim^-0.5
  float softcap = 0.f;
  std::vector<LayerTransform> transforms;  // per layer; empty = the layers hand over finished q / k / v rows
};

class AttentionBackend {
 public:
  virtual ~AttentionBackend() = default;
  // k, v: [n][kv_heads][head_dim] float32 host rows written at pos .. pos+n-1.
  virtual Status Append(int layer, int pos, int n, const float* k, const float* v) = 0;
  // The same with the layer's transform applied first: q [n][q_heads][head_dim] is
  // normalised and rotated in place, k / v go through norm / rotation into the cache.
  virtual Status PreAttention(int layer, int pos, int n, float* q, const float* k, const float* v) = 0;
  // q, out: [n][q_heads][head_dim] float32 host; rows at positions q_pos0 .. q_pos0+n-1.
  virtual Status Prefill(int layer, int q_pos0, int n, const float* q, float* out) = 0;
  // One row at position kv_len - 1.
  virtual Status Decode(int layer, int kv_len, const float* q, float* out) = 0;
  virtual Status Reset() = 0;
  virtual std::string Name() const = 0;

  // Device-resident form: the rows are device buffers in the activation type of the backend (float32, or IEEE half
  // for fp16 activations), every call is queued on Stream() and returns without waiting, results are ordered by the
  // stream. This is how the reference's GPU branch runs: cache and activations stay in device buffers across
  // signatures (llm_litert_compiled_model_executor.cc:753-755). A backend is either host-staged (the calls above) or
  // device-resident (the calls below); the other set answers kFailedPrecondition.
  virtual bool DeviceResident() const { return false; }
  virtual void* Stream() const { return nullptr; }  // hipStream_t
  virtual Status AppendOnDevice(int, int, int, const void*, const void*) { return NotDeviceResident(); }
  virtual Status PreAttentionOnDevice(int, int, int, void*, const void*, const void*) { return NotDeviceResident(); }
  virtual Status PrefillOnDevice(int, int, int, const void*, void*) { return NotDeviceResident(); }
  virtual Status DecodeOnDevice(int, int, const void*, void*) { return NotDeviceResident(); }
  // PreAttentionOnDevice for the one row at kv_len - 1 and DecodeOnDevice in one queued call (same results); q, k, v
  // are the raw projections of that row. A backend without such a call answers kUnimplemented and the executor
  // makes the two calls.
  virtual Status DecodeStepOnDevice(int, int, const void*, const void*, const void*, void*) {
    return UnimplementedError("attention backend '" + Name() + "' has no single-call decode step.");
  }
  virtual bool HasDecodeStep() const { return false; }
  virtual Status Sync() { return OkStatus(); }  // waits for everything queued on Stream()

 protected:
  Status NotDeviceResident() const {
    return FailedPreconditionError("attention backend '" + Name() + "' is not device-resident.");
  }
};

struct AttentionCall {
  enum Kind { kAppend, kPrefill, kDecode, kReset } kind;
  int layer, pos, n;
};

class RecordingAttentionBackend : public AttentionBackend {
 public:
  explicit RecordingAttentionBackend(AttentionShape shape) : shape_(std::move(shape)) {}
  Status Append(int layer, int pos, int n, const float*, const float*) override {
    if (pos + n > shape_.max_tokens) return OutOfRangeError("KV cache is full.");
    calls.push_back({AttentionCall::kAppend, layer, pos, n});
    return OkStatus();
  }
  Status PreAttention(int layer, int pos, int n, float*, const float* k, const float* v) override {
    return Append(layer, pos, n, k, v);
  }
  Status Prefill(int layer, int q_pos0, int n, const float*, float* out) override {
    calls.push_back({AttentionCall::kPrefill, layer, q_pos0, n});
    Zero(out, n);
    return OkStatus();
  }
  Status Decode(int layer, int kv_len, const float*, float* out) override {
    calls.push_back({AttentionCall::kDecode, layer, kv_len - 1, 1});
    Zero(out, 1);
    return OkStatus();
  }
  Status Reset() override {
    calls.push_back({AttentionCall::kReset, 0, 0, 0});
    return OkStatus();
  }
  std::string Name() const override { return "recording"; }
  std::vector<AttentionCall> calls;

 private:
  void Zero(float* out, int n) const {
    for (size_t i = 0; i < (size_t)n * shape_.num_q_heads * shape_.head_dim; ++i) out[i] = 0.f;
  }
  AttentionShape shape_;
};

// fp32 activations: fp32 cache and I/O. fp16 activations: fp16 cache and I/O (converted on the host at this
// boundary when host-staged). device_resident: the handle takes device pointers and runs on a stream of its own.
StatusOr<std::unique_ptr<AttentionBackend>> CreateMi355AttentionBackend(const AttentionShape& shape, bool fp16,
                                                                         int device, bool device_resident = false);

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_ATTENTION_BACKEND_H_
