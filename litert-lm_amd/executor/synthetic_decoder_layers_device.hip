// Device-resident form of SyntheticDecoderLayers: the same arithmetic as
// synthetic_decoder_layers.cc, one workgroup per token, the token's state row
// held in LDS. Like the host form it is scaffolding for the executor's cache /
// position / step plumbing, not a model: it lets HipLlmExecutor run a whole
// forward pass without a host round trip between layers, the way the reference's
// GPU branch keeps activations in device buffers between signatures
// (runtime/executor/llm_litert_compiled_model_executor.cc:753-755).
//
// Built with -ffp-contract=off so that every float operation rounds as in the
// host form; the sums of squares and the logits are reduced in double by a
// tree instead of in sequence, which is the only difference in rounding.
#include <hip/hip_runtime.h>

#include <string>

#include "decoder_layers.h"

namespace litert::lm {
namespace {

constexpr int kThreads = 256;
constexpr int kInlineTokens = 16;  // passes up to this long carry their ids as kernel arguments

struct PassTokens {
  int32_t inline_ids[kInlineTokens];
  const int32_t* ids;  // device array, used when n > kInlineTokens
  int32_t pos0;
  int32_t n;
};

__device__ __forceinline__ uint32_t mix(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352dU;
  x ^= x >> 15;
  x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}
__device__ __forceinline__ float unit(uint32_t key) {
  return static_cast<float>(mix(key) >> 8) * (1.0f / 16777216.0f) * 2.0f - 1.0f;
}

template <class T>
__device__ __forceinline__ float load(const T* p, size_t i) { return static_cast<float>(p[i]); }
template <class T>
__device__ __forceinline__ void store(T* p, size_t i, float x) { p[i] = static_cast<T>(x); }

__device__ double block_sum(double x, double* scratch) {
  const int tid = threadIdx.x;
  scratch[tid] = x;
  __syncthreads();
  for (int s = kThreads / 2; s > 0; s >>= 1) {
    if (tid < s) scratch[tid] += scratch[tid + s];
    __syncthreads();
  }
  const double total = scratch[0];
  __syncthreads();
  return total;
}

// q / k / v of `layer` from the state row `s` (LDS) of token t.
template <class T>
__device__ void project(const float* s, int layer, int t, int hq, int hkv, int d, T* q, T* k, T* v) {
  const int hidden = hq * d, group = hq / hkv;
  const uint32_t ul = static_cast<uint32_t>(layer);
  const float inv_group = 1.0f / static_cast<float>(group);
  for (int i = threadIdx.x; i < hidden; i += kThreads)
    store(q, (size_t)t * hidden + i, s[i] * (1.0f + 0.5f * unit(ul * 0x165667B1U + (uint32_t)i * 0x9E3779B1U + 3U)));
  for (int e = threadIdx.x; e < hkv * d; e += kThreads) {
    const int kh = e / d, c = e - kh * d;
    float sum = 0.f;
    for (int j = 0; j < group; ++j) sum += s[(kh * group + j) * d + c];
    const float mean = sum * inv_group;
    const uint32_t idx = static_cast<uint32_t>(e);
    store(k, (size_t)t * hkv * d + e, mean * (1.0f + 0.5f * unit(ul * 0x27D4EB2FU + idx * 0x165667B1U + 5U)));
    store(v, (size_t)t * hkv * d + e,
          mean * unit(ul * 0x85EBCA77U + idx * 0xC2B2AE3DU + 6U) + 0.25f * unit(idx * 0x9E3779B1U + ul + 7U));
  }
}

template <class T>
__global__ void __launch_bounds__(kThreads) begin_kernel(PassTokens p, int hq, int hkv, int d, float* state, T* q, T* k,
                                                         T* v) {
  extern __shared__ float s[];
  const int t = blockIdx.x, hidden = hq * d;
  const uint32_t tok = static_cast<uint32_t>(p.n <= kInlineTokens ? p.inline_ids[t] : p.ids[t]);
  const uint32_t pos = static_cast<uint32_t>(p.pos0 + t);
  for (int i = threadIdx.x; i < hidden; i += kThreads) {
    const uint32_t ui = static_cast<uint32_t>(i);
    const float x = unit(tok * 0x9E3779B1U + ui * 0x85EBCA77U + 1U) + 0.5f * unit(pos * 0xC2B2AE3DU + ui * 0x27D4EB2FU + 2U);
    s[i] = x;
    state[(size_t)t * hidden + i] = x;
  }
  __syncthreads();
  project(s, 0, t, hq, hkv, d, q, k, v);
}

// Residual add of the attention output of `layer`, RMS norm of the row, then q / k / v of layer + 1.
template <class T>
__global__ void __launch_bounds__(kThreads) next_layer_kernel(int layer, bool project_next, int hq, int hkv, int d,
                                                              float* state, const T* attn, T* q, T* k, T* v) {
  extern __shared__ float s[];
  __shared__ double scratch[kThreads];
  const int t = blockIdx.x, hidden = hq * d;
  const uint32_t ul = static_cast<uint32_t>(layer);
  double sq = 0.0;
  for (int i = threadIdx.x; i < hidden; i += kThreads) {
    const float x = state[(size_t)t * hidden + i] +
                    load(attn, (size_t)t * hidden + i) * unit(ul * 0xC2B2AE3DU + (uint32_t)i * 0x27D4EB2FU + 8U);
    s[i] = x;
    sq += static_cast<double>(x) * static_cast<double>(x);
  }
  const double total = block_sum(sq, scratch);
  const float inv_rms = static_cast<float>(1.0 / sqrt(total / hidden + 1e-6));
  for (int i = threadIdx.x; i < hidden; i += kThreads) {
    const float x = s[i] * inv_rms;
    s[i] = x;
    state[(size_t)t * hidden + i] = x;
  }
  __syncthreads();
  if (project_next) project(s, layer + 1, t, hq, hkv, d, q, k, v);
}

// One workgroup per vocabulary entry, over the state row of the pass's last token.
__global__ void __launch_bounds__(kThreads) logits_kernel(const float* row, int hidden, float* logits) {
  __shared__ double scratch[kThreads];
  const uint32_t vtok = blockIdx.x;
  double acc = 0.0;
  for (int i = threadIdx.x; i < hidden; i += kThreads)
    acc += static_cast<double>(row[i]) * static_cast<double>(unit(vtok * 0x2545F491U + (uint32_t)i * 0x61C88647U + 4U));
  const double total = block_sum(acc, scratch);
  if (threadIdx.x == 0) logits[vtok] = static_cast<float>(total * (1.0 / sqrt(static_cast<double>(hidden))));
}

Status HipStatus(hipError_t e, const char* what) {
  if (e == hipSuccess) return OkStatus();
  return InternalError(std::string(what) + ": " + hipGetErrorString(e));
}

}  // namespace

SyntheticDecoderLayers::~SyntheticDecoderLayers() {
  if (d_state_) (void)hipFree(d_state_);
  if (d_tokens_) (void)hipFree(d_tokens_);
  for (int i = 0; i < kTokenStages; ++i) {
    if (stage_done_[i]) (void)hipEventDestroy(static_cast<hipEvent_t>(stage_done_[i]));
    if (stage_ids_[i]) (void)hipHostFree(stage_ids_[i]);
  }
}

Status SyntheticDecoderLayers::BeginOnDevice(const std::vector<int32_t>& tokens, const std::vector<int32_t>& positions,
                                             const DeviceActivations& io) {
  RET_CHECK_EQ(tokens.size(), positions.size());
  RET_CHECK_GT(tokens.size(), 0u);
  const int n = static_cast<int>(tokens.size());
  for (int t = 1; t < n; ++t) RET_CHECK_EQ(positions[t], positions[0] + t) << "positions of a pass must be consecutive.";
  RET_CHECK(io.q && io.k && io.v && io.attn);
  hipStream_t stream = static_cast<hipStream_t>(io.stream);
  const int hidden = Hidden();
  if (n > d_capacity_) {
    // Grows only between passes of different length: wait for the passes that still read the old buffers.
    RETURN_IF_ERROR(HipStatus(hipStreamSynchronize(stream), "hipStreamSynchronize"));
    if (d_state_) (void)hipFree(d_state_);
    if (d_tokens_) (void)hipFree(d_tokens_);
    d_state_ = nullptr, d_tokens_ = nullptr, d_capacity_ = 0;
    for (int i = 0; i < kTokenStages; ++i) {
      if (stage_ids_[i]) (void)hipHostFree(stage_ids_[i]);
      stage_ids_[i] = nullptr;
    }
    RETURN_IF_ERROR(HipStatus(hipMalloc(&d_state_, sizeof(float) * (size_t)n * hidden), "hipMalloc(state)"));
    RETURN_IF_ERROR(HipStatus(hipMalloc(&d_tokens_, sizeof(int32_t) * (size_t)n), "hipMalloc(tokens)"));
    for (int i = 0; i < kTokenStages; ++i) {
      RETURN_IF_ERROR(HipStatus(hipHostMalloc(&stage_ids_[i], sizeof(int32_t) * (size_t)n), "hipHostMalloc(token stage)"));
      if (!stage_done_[i]) {
        hipEvent_t ev;
        RETURN_IF_ERROR(HipStatus(hipEventCreateWithFlags(&ev, hipEventDisableTiming), "hipEventCreate"));
        stage_done_[i] = ev;
      }
    }
    d_capacity_ = n;
  }
  PassTokens p{};
  p.ids = d_tokens_;
  p.pos0 = positions[0];
  p.n = n;
  if (n <= kInlineTokens) {
    for (int t = 0; t < n; ++t) p.inline_ids[t] = tokens[t];
  } else {
    // Through a pinned slot, so that the copy is a plain stream operation (ordered behind the kernels that still
    // read the previous ids) and the call does not wait for it; a slot is reused once its own copy has run.
    const int slot = stage_next_;
    stage_next_ = (stage_next_ + 1) % kTokenStages;
    hipEvent_t done = static_cast<hipEvent_t>(stage_done_[slot]);
    RETURN_IF_ERROR(HipStatus(hipEventSynchronize(done), "hipEventSynchronize"));
    for (int t = 0; t < n; ++t) stage_ids_[slot][t] = tokens[t];
    RETURN_IF_ERROR(HipStatus(hipMemcpyAsync(d_tokens_, stage_ids_[slot], sizeof(int32_t) * (size_t)n,
                                             hipMemcpyHostToDevice, stream),
                              "hipMemcpyAsync(tokens)"));
    RETURN_IF_ERROR(HipStatus(hipEventRecord(done, stream), "hipEventRecord"));
  }
  d_n_ = n;
  const size_t lds = sizeof(float) * (size_t)hidden;
  if (io.fp16)
    hipLaunchKernelGGL(begin_kernel<_Float16>, dim3(n), dim3(kThreads), lds, stream, p, shape_.num_q_heads,
                       shape_.num_kv_heads, shape_.head_dim, d_state_, static_cast<_Float16*>(io.q),
                       static_cast<_Float16*>(io.k), static_cast<_Float16*>(io.v));
  else
    hipLaunchKernelGGL(begin_kernel<float>, dim3(n), dim3(kThreads), lds, stream, p, shape_.num_q_heads,
                       shape_.num_kv_heads, shape_.head_dim, d_state_, static_cast<float*>(io.q),
                       static_cast<float*>(io.k), static_cast<float*>(io.v));
  return HipStatus(hipGetLastError(), "begin_kernel");
}

Status SyntheticDecoderLayers::NextLayerOnDevice(int layer, const DeviceActivations& io) {
  RET_CHECK_GT(d_n_, 0) << "NextLayerOnDevice before BeginOnDevice.";
  RET_CHECK(layer >= 0 && layer < shape_.num_layers);
  hipStream_t stream = static_cast<hipStream_t>(io.stream);
  const bool next = layer + 1 < shape_.num_layers;
  const size_t lds = sizeof(float) * (size_t)Hidden();
  if (io.fp16)
    hipLaunchKernelGGL(next_layer_kernel<_Float16>, dim3(d_n_), dim3(kThreads), lds, stream, layer, next,
                       shape_.num_q_heads, shape_.num_kv_heads, shape_.head_dim, d_state_,
                       static_cast<const _Float16*>(io.attn), static_cast<_Float16*>(io.q), static_cast<_Float16*>(io.k),
                       static_cast<_Float16*>(io.v));
  else
    hipLaunchKernelGGL(next_layer_kernel<float>, dim3(d_n_), dim3(kThreads), lds, stream, layer, next, shape_.num_q_heads,
                       shape_.num_kv_heads, shape_.head_dim, d_state_, static_cast<const float*>(io.attn),
                       static_cast<float*>(io.q), static_cast<float*>(io.k), static_cast<float*>(io.v));
  return HipStatus(hipGetLastError(), "next_layer_kernel");
}

Status SyntheticDecoderLayers::LogitsOnDevice(float* logits, void* stream) {
  RET_CHECK_GT(d_n_, 0) << "LogitsOnDevice before BeginOnDevice.";
  const int hidden = Hidden();
  hipLaunchKernelGGL(logits_kernel, dim3(vocab_), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                     d_state_ + (size_t)(d_n_ - 1) * hidden, hidden, logits);
  return HipStatus(hipGetLastError(), "logits_kernel");
}

}  // namespace litert::lm
