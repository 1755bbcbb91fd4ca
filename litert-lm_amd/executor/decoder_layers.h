// Everything of the transformer that is NOT attention, as the executor sees
// it. In the reference all of it (embedding, projections, RoPE, norms, MLP,
// logits) sits inside the .tflite graph behind compiled_model_.Run
// (runtime/executor/llm_litert_compiled_model_executor.cc:271,407,522); this
// build accelerates the attention between ProjectQkv and ConsumeAttention and
// leaves the rest to whoever implements this interface.
//
// SyntheticDecoderLayers is a deterministic, seed-free toy stack (hash-derived
// embeddings and element-wise weights, RMS norm, a small logits projection)
// used to drive the executor end to end in tests; it is test scaffolding for
// the cache / position / step plumbing, not a model.
#ifndef LITERT_LM_AMD_EXECUTOR_DECODER_LAYERS_H_
#define LITERT_LM_AMD_EXECUTOR_DECODER_LAYERS_H_

#include <cstdint>
#include <vector>

#include "attention_backend.h"
#include "status.h"

namespace litert::lm {

class DecoderLayers {
 public:
  virtual ~DecoderLayers() = default;
  virtual const AttentionShape& Shape() const = 0;
  virtual int VocabSize() const = 0;
  // Starts a forward pass over n tokens at the given absolute positions.
  virtual Status Begin(const std::vector<int32_t>& tokens, const std::vector<int32_t>& positions) = 0;
  // q [n][Hq][D], k and v [n][Hkv][D] of `layer` for the tokens of this pass.
  virtual Status ProjectQkv(int layer, float* q, float* k, float* v) = 0;
  // attn [n][Hq][D]: the attention output of `layer`.
  virtual Status ConsumeAttention(int layer, const float* attn) = 0;
  // Logits [vocab] of the last token of this pass.
  virtual Status Logits(float* logits) = 0;

  // Device-resident form of the same pass. The buffers are device memory in the activation type of the executor
  // (`fp16`: IEEE half, else float32), sized for `n` tokens; all work is queued on `stream` (a hipStream_t) and no
  // call waits. The graph between two attention ops is one segment: what follows attention of layer l (output
  // projection, MLP, norms) and what precedes attention of layer l + 1 (its q / k / v projections).
  struct DeviceActivations {
    void* q = nullptr;     // [n][Hq][D]
    void* k = nullptr;     // [n][Hkv][D]
    void* v = nullptr;     // [n][Hkv][D]
    void* attn = nullptr;  // [n][Hq][D]
    bool fp16 = false;
    void* stream = nullptr;
  };
  virtual bool HasDeviceForm() const { return false; }
  // Starts a pass (tokens and positions are host arrays, consumed before the call returns) and fills q / k / v of layer 0.
  virtual Status BeginOnDevice(const std::vector<int32_t>& tokens, const std::vector<int32_t>& positions,
                               const DeviceActivations& io) {
    (void)tokens, (void)positions, (void)io;
    return UnimplementedError("these decoder layers have no device-resident form.");
  }
  // Consumes io.attn of `layer` and, unless it was the last layer, fills q / k / v of layer + 1.
  virtual Status NextLayerOnDevice(int layer, const DeviceActivations& io) {
    (void)layer, (void)io;
    return UnimplementedError("these decoder layers have no device-resident form.");
  }
  // Logits [vocab] float32 (device memory) of the last token of this pass.
  virtual Status LogitsOnDevice(float* logits, void* stream) {
    (void)logits, (void)stream;
    return UnimplementedError("these decoder layers have no device-resident form.");
  }
};

class SyntheticDecoderLayers : public DecoderLayers {
 public:
  SyntheticDecoderLayers(AttentionShape shape, int vocab) : shape_(std::move(shape)), vocab_(vocab) {}
  const AttentionShape& Shape() const override { return shape_; }
  int VocabSize() const override { return vocab_; }
  Status Begin(const std::vector<int32_t>& tokens, const std::vector<int32_t>& positions) override;
  Status ProjectQkv(int layer, float* q, float* k, float* v) override;
  Status ConsumeAttention(int layer, const float* attn) override;
  Status Logits(float* logits) override;

  // The same arithmetic as kernels (synthetic_decoder_layers_device.hip).
  ~SyntheticDecoderLayers() override;
  bool HasDeviceForm() const override { return true; }
  Status BeginOnDevice(const std::vector<int32_t>& tokens, const std::vector<int32_t>& positions,
                       const DeviceActivations& io) override;
  Status NextLayerOnDevice(int layer, const DeviceActivations& io) override;
  Status LogitsOnDevice(float* logits, void* stream) override;

  // Deterministic norm weights and rotary frequencies in the pattern of Gemma 3
  // (query / key norm with a (1 + weight) scale, theta 10,000 on windowed layers
  // and 1,000,000 on global ones) for tests of the fused step before attention.
  static std::vector<LayerTransform> Transforms(const AttentionShape& shape);

  static uint32_t Mix(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7feb352dU;
    x ^= x >> 15;
    x *= 0x846ca68bU;
    x ^= x >> 16;
    return x;
  }
  // Uniform in [-1, 1) from a 32-bit key.
  static float Unit(uint32_t key) { return static_cast<float>(Mix(key) >> 8) * (1.0f / 16777216.0f) * 2.0f - 1.0f; }

 private:
  int Hidden() const { return shape_.num_q_heads * shape_.head_dim; }
  AttentionShape shape_;
  int vocab_;
  int n_ = 0;
  std::vector<float> state_;  // [n][hidden]
  // device-resident pass: state [capacity][hidden] float32 and the token ids of a long pass, in device memory
  float* d_state_ = nullptr;
  int32_t* d_tokens_ = nullptr;
  int d_capacity_ = 0;
  int d_n_ = 0;
  // pinned host slots the ids of long passes are copied from, each with the event that says its copy has run
  static constexpr int kTokenStages = 4;
  int32_t* stage_ids_[kTokenStages] = {};
  void* stage_done_[kTokenStages] = {};  // hipEvent_t
  int stage_next_ = 0;
};

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_DECODER_LAYERS_H_
