// AttentionBackend over the C ABI of libmi355_attn.so, in one of two forms.
// Host-staged: host float32 rows cross the boundary as they are (fp32 cache) or
// as fp16 (fp16 cache); the library stages them to the device (host_io = 1) and
// returns with results in place. Device-resident: the handle takes device
// pointers (host_io = 0) and queues every call on its own stream without
// waiting, so a forward pass over all layers runs without a host round trip,
// as the reference's GPU branch does with its device-side cache and activation
// buffers (runtime/executor/llm_litert_compiled_model_executor.cc:753-755).
#include <cstdlib>
#include <string>
#include <vector>

#include "../../include/mi355_attn.h"
#include "attention_backend.h"

namespace litert::lm {
namespace {

Status FromCode(int rc, char* err, const char* what) {
  if (rc == MI355_ATTN_OK) return OkStatus();
  std::string msg = std::string(what) + ": " + (err ? err : "(no message)");
  free(err);
  return Status(static_cast<StatusCode>(rc), msg);
}

class Mi355AttentionBackend : public AttentionBackend {
 public:
  Mi355AttentionBackend(mi355_attn* h, AttentionShape shape, bool fp16, bool device_resident)
      : h_(h), shape_(std::move(shape)), fp16_(fp16), device_resident_(device_resident) {}
  ~Mi355AttentionBackend() override { mi355_attn_destroy(h_); }

  bool DeviceResident() const override { return device_resident_; }
  void* Stream() const override { return mi355_attn_stream(h_); }
  Status AppendOnDevice(int layer, int pos, int n, const void* k, const void* v) override {
    if (!device_resident_) return NotDeviceResident();
    char* err = nullptr;
    return FromCode(mi355_attn_kv_append(h_, layer, 0, pos, n, k, v, &err), err, "kv_append");
  }
  Status PreAttentionOnDevice(int layer, int pos, int n, void* q, const void* k, const void* v) override {
    if (!device_resident_) return NotDeviceResident();
    char* err = nullptr;
    return FromCode(mi355_attn_pre_attention(h_, layer, 0, pos, n, q, k, v, q, &err), err, "pre_attention");
  }
  Status PrefillOnDevice(int layer, int q_pos0, int n, const void* q, void* out) override {
    if (!device_resident_) return NotDeviceResident();
    char* err = nullptr;
    return FromCode(mi355_attn_prefill(h_, layer, 0, q_pos0, n, q, out, &err), err, "prefill");
  }
  Status DecodeOnDevice(int layer, int kv_len, const void* q, void* out) override {
    if (!device_resident_) return NotDeviceResident();
    char* err = nullptr;
    const int32_t len = kv_len;
    return FromCode(mi355_attn_decode(h_, layer, nullptr, &len, 1, q, out, 0, &err), err, "decode");
  }
  bool HasDecodeStep() const override { return device_resident_; }
  Status DecodeStepOnDevice(int layer, int kv_len, const void* q, const void* k, const void* v, void* out) override {
    if (!device_resident_) return NotDeviceResident();
    char* err = nullptr;
    const int32_t len = kv_len;
    return FromCode(mi355_attn_decode_step(h_, layer, nullptr, &len, 1, q, k, v, out, 0, &err), err, "decode_step");
  }
  Status Sync() override {
    char* err = nullptr;
    return FromCode(mi355_attn_sync(h_, &err), err, "sync");
  }

  Status Append(int layer, int pos, int n, const float* k, const float* v) override {
    if (device_resident_) return HostStagedOnly();
    char* err = nullptr;
    const size_t count = (size_t)n * shape_.num_kv_heads * shape_.head_dim;
    int rc;
    if (fp16_) {
      ToHalf(k, count, &ha_);
      ToHalf(v, count, &hb_);
      rc = mi355_attn_kv_append(h_, layer, 0, pos, n, ha_.data(), hb_.data(), &err);
    } else {
      rc = mi355_attn_kv_append(h_, layer, 0, pos, n, k, v, &err);
    }
    return FromCode(rc, err, "kv_append");
  }

  Status PreAttention(int layer, int pos, int n, float* q, const float* k, const float* v) override {
    if (device_resident_) return HostStagedOnly();
    char* err = nullptr;
    const size_t qn = (size_t)n * shape_.num_q_heads * shape_.head_dim;
    const size_t kn = (size_t)n * shape_.num_kv_heads * shape_.head_dim;
    int rc;
    if (fp16_) {
      ToHalf(q, qn, &hq_);
      ToHalf(k, kn, &ha_);
      ToHalf(v, kn, &hb_);
      rc = mi355_attn_pre_attention(h_, layer, 0, pos, n, hq_.data(), ha_.data(), hb_.data(), hq_.data(), &err);
      if (rc == MI355_ATTN_OK) FromHalf(hq_, qn, q);
    } else {
      rc = mi355_attn_pre_attention(h_, layer, 0, pos, n, q, k, v, q, &err);
    }
    return FromCode(rc, err, "pre_attention");
  }

  Status Prefill(int layer, int q_pos0, int n, const float* q, float* out) override {
    if (device_resident_) return HostStagedOnly();
    char* err = nullptr;
    const size_t count = (size_t)n * shape_.num_q_heads * shape_.head_dim;
    int rc;
    if (fp16_) {
      ToHalf(q, count, &ha_);
      hb_.resize(count);
      rc = mi355_attn_prefill(h_, layer, 0, q_pos0, n, ha_.data(), hb_.data(), &err);
      if (rc == MI355_ATTN_OK) FromHalf(hb_, count, out);
    } else {
      rc = mi355_attn_prefill(h_, layer, 0, q_pos0, n, q, out, &err);
    }
    return FromCode(rc, err, "prefill");
  }

  Status Decode(int layer, int kv_len, const float* q, float* out) override {
    if (device_resident_) return HostStagedOnly();
    char* err = nullptr;
    const size_t count = (size_t)shape_.num_q_heads * shape_.head_dim;
    const int32_t len = kv_len;
    int rc;
    if (fp16_) {
      ToHalf(q, count, &ha_);
      hb_.resize(count);
      rc = mi355_attn_decode(h_, layer, nullptr, &len, 1, ha_.data(), hb_.data(), 0, &err);
      if (rc == MI355_ATTN_OK) FromHalf(hb_, count, out);
    } else {
      rc = mi355_attn_decode(h_, layer, nullptr, &len, 1, q, out, 0, &err);
    }
    return FromCode(rc, err, "decode");
  }

  Status Reset() override {
    char* err = nullptr;
    return FromCode(mi355_attn_reset(h_, -1, &err), err, "reset");
  }

  std::string Name() const override { return mi355_attn_version(); }

 private:
  Status HostStagedOnly() const {
    return FailedPreconditionError("this attention backend is device-resident: it takes device buffers.");
  }
  static void ToHalf(const float* src, size_t n, std::vector<_Float16>* dst) {
    dst->resize(n);
    for (size_t i = 0; i < n; ++i) (*dst)[i] = static_cast<_Float16>(src[i]);
  }
  static void FromHalf(const std::vector<_Float16>& src, size_t n, float* dst) {
    for (size_t i = 0; i < n; ++i) dst[i] = static_cast<float>(src[i]);
  }
  mi355_attn* h_;
  AttentionShape shape_;
  bool fp16_;
  bool device_resident_;
  std::vector<_Float16> ha_, hb_, hq_;
};

}  // namespace

StatusOr<std::unique_ptr<AttentionBackend>> CreateMi355AttentionBackend(const AttentionShape& shape, bool fp16,
                                                                         int device, bool device_resident) {
  mi355_attn_config cfg{};
  cfg.struct_size = sizeof(cfg);
  cfg.num_layers = shape.num_layers;
  cfg.num_q_heads = shape.num_q_heads;
  cfg.num_kv_heads = shape.num_kv_heads;
  cfg.head_dim = shape.head_dim;
  cfg.max_tokens = shape.max_tokens;
  cfg.max_seqs = 1;  // the reference executor is batch 1 (llm_litert_compiled_model_executor.cc:798-800)
  cfg.kv_dtype = fp16 ? MI355_ATTN_F16 : MI355_ATTN_F32;
  cfg.io_dtype = cfg.kv_dtype;
  cfg.scale = shape.scale;
  cfg.softcap = shape.softcap;
  cfg.layer_window = shape.layer_window.empty() ? nullptr : shape.layer_window.data();
  cfg.device = device;
  cfg.host_io = device_resident ? 0 : 1;
  cfg.own_stream = 1;
  mi355_attn* h = nullptr;
  char* err = nullptr;
  const int rc = mi355_attn_create(&cfg, &h, &err);
  if (rc != MI355_ATTN_OK) return FromCode(rc, err, "mi355_attn_create");
  if (!shape.transforms.empty() && (int)shape.transforms.size() != shape.num_layers) {
    mi355_attn_destroy(h);
    return InvalidArgumentError("transforms needs one entry per layer.");
  }
  for (int layer = 0; layer < (int)shape.transforms.size(); ++layer) {
    const LayerTransform& lt = shape.transforms[layer];
    const size_t d = (size_t)shape.head_dim;
    if ((!lt.q_weight.empty() && lt.q_weight.size() != d) || (!lt.k_weight.empty() && lt.k_weight.size() != d) ||
        (!lt.rope_inv_freq.empty() && lt.rope_inv_freq.size() != d / 2)) {
      mi355_attn_destroy(h);
      return InvalidArgumentError("transform of layer " + std::to_string(layer) + ": wrong array length.");
    }
    mi355_attn_layer_transform t{};
    t.struct_size = sizeof(t);
    t.norm_q = lt.norm_q;
    t.norm_k = lt.norm_k;
    t.norm_v = lt.norm_v;
    t.q_weight = lt.q_weight.empty() ? nullptr : lt.q_weight.data();
    t.k_weight = lt.k_weight.empty() ? nullptr : lt.k_weight.data();
    t.eps = lt.eps;
    t.weight_offset = lt.weight_offset;
    t.rope_inv_freq = lt.rope_inv_freq.empty() ? nullptr : lt.rope_inv_freq.data();
    const int trc = mi355_attn_set_layer_transform(h, layer, &t, &err);
    if (trc != MI355_ATTN_OK) {
      mi355_attn_destroy(h);
      return FromCode(trc, err, "mi355_attn_set_layer_transform");
    }
  }
  return std::unique_ptr<AttentionBackend>(new Mi355AttentionBackend(h, shape, fp16, device_resident));
}

}  // namespace litert::lm
