// The step right before attention, in one pass over the new rows: per-head RMS
// norm of the query / key (/ value) projections, rotary position embedding of
// query and key, the query written out for the attention kernels and the key /
// value rows written straight into the cache planes in MFMA operand order
// (quantised with the plane's fixed scales for an int8 cache).
//
// Replaces, in the reference's NPU flow, the RoPE signature that turns
// `input_pos` into cos / sin tables and the cache-update signature that merges
// the new `kv_slice_{k,v}_i` rows at `input_pos`
// (runtime/executor/llm_litert_npu_compiled_model_executor.cc:82-110,1209-1219,
// 1294-1333); in the CPU/GPU executor the same work sits inside the graph behind
// compiled_model_.Run (llm_litert_compiled_model_executor.cc:271,407,522). The
// int8 write follows the quantise idiom of
// llm_litert_npu_compiled_model_executor.cc:116-148 (reciprocal scale,
// std::round, clamp).
//
// Bound: HBM. Each row of 256 channels is read once and written once; one wave
// owns one (token, head) row, a lane the channel pairs (2l, 2l+1) and
// (128+2l, 128+2l+1), so both members of every rotated pair (d, d+128) are in
// the same lane and the only cross-lane step is the sum of squares of the norm.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include "attn_params.h"
#include "kernels.h"
#include "mfma_util.h"

namespace mi355 {
namespace {

constexpr int kD = 256;
constexpr int kRowsPerWg = 4;  // waves per workgroup

template <int DT>
__device__ __forceinline__ void load_pair(const void* base, int64_t elem, float& a, float& b) {
  if constexpr (DT == kF32) {
    const float2 x = *reinterpret_cast<const float2*>(reinterpret_cast<const float*>(base) + elem);
    a = x.x; b = x.y;
  } else if constexpr (DT == kF16) {
    const h2 x = *reinterpret_cast<const h2*>(reinterpret_cast<const _Float16*>(base) + elem);
    a = (float)x[0]; b = (float)x[1];
  } else {
    const uint32_t x = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint16_t*>(base) + elem);
    a = __uint_as_float(x << 16); b = __uint_as_float(x & 0xffff0000u);
  }
}

// Two consecutive elements of type DT at byte address p (4- or 8-byte aligned).
template <int DT>
__device__ __forceinline__ void store_pair(uint8_t* p, float a, float b) {
  if constexpr (DT == kF32) {
    *reinterpret_cast<float2*>(p) = make_float2(a, b);
  } else if constexpr (DT == kF16) {
    h2 x = {(_Float16)a, (_Float16)b};
    *reinterpret_cast<h2*>(p) = x;
  } else {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    bf2 x = {(__bf16)a, (__bf16)b};
    *reinterpret_cast<bf2*>(p) = x;
  }
}

template <int DT>
__device__ __forceinline__ void store_one(uint8_t* p, float a) {
  if constexpr (DT == kF32) *reinterpret_cast<float*>(p) = a;
  else if constexpr (DT == kF16) *reinterpret_cast<_Float16*>(p) = (_Float16)a;
  else *reinterpret_cast<__bf16*>(p) = (__bf16)a;
}

// A value-plane element: like store_one, except that a bfloat16 cache keeps its V planes as IEEE
// half values (attn_params.h): the value is rounded to bfloat16 first, so that the cache holds
// exactly what a bfloat16 row appended through the copy kernel would leave.
template <int DT>
__device__ __forceinline__ void store_value(uint8_t* p, float a) {
  if constexpr (DT == kBF16) *reinterpret_cast<uint16_t*>(p) = bf16_bits_to_half_bits(bit_cast<uint16_t>((__bf16)a));
  else store_one<DT>(p, a);
}

// round-half-away of x / scale, clamped to +-127; scale 0 stores 0
__device__ __forceinline__ int quantise(float x, float scale) {
  const float inv = scale != 0.f ? 1.0f / scale : 0.f;
  const float r = roundf(x * inv);
  return (int)fminf(fmaxf(r, -127.f), 127.f);
}

template <int IO, int KV>
__global__ void __launch_bounds__(64 * kRowsPerWg) pre_attention_kernel(const PreAttentionArgs a) {
  constexpr int ESZ = KV == kF32 ? 4 : (KV == kI8 ? 1 : 2);
  constexpr int EPC = 16 / ESZ;
  const int lane = threadIdx.x & 63;
  const int rows_per_token = a.hq + 2 * a.geom.hkv;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerWg + (threadIdx.x >> 6);
  if (row >= (int64_t)a.n * rows_per_token) return;  // whole waves leave; no barrier below
  const int i = (int)(row / rows_per_token);
  const int j = (int)(row % rows_per_token);
  const int kind = j < a.hq ? 0 : (j < a.hq + a.geom.hkv ? 1 : 2);  // 0 = query, 1 = key, 2 = value
  const int head = kind == 0 ? j : (kind == 1 ? j - a.hq : j - a.hq - a.geom.hkv);
  const void* src = kind == 0 ? a.q : (kind == 1 ? a.k : a.v);
  const int heads = kind == 0 ? a.hq : a.geom.hkv;
  const int64_t base = ((int64_t)i * heads + head) * kD;
  const int d0 = 2 * lane, d1 = kD / 2 + 2 * lane;  // the lane's channels: d0, d0+1, d1, d1+1

  float x[4];
  load_pair<IO>(src, base + d0, x[0], x[1]);
  load_pair<IO>(src, base + d1, x[2], x[3]);

  // sine / cosine of the lane's two angles first: they depend on the position
  // only, so their ~200 instructions run while the row's loads are in flight
  const int t = a.pos + i;
  const bool rotate = a.rope && kind != 2;
  float s0 = 0.f, c0 = 1.f, s1 = 0.f, c1 = 1.f;
  if (rotate) {
    const float2 f = *reinterpret_cast<const float2*>(a.constants + d0);  // frequencies of pairs d0, d0+1
    sincosf((float)t * f.x, &s0, &c0);
    sincosf((float)t * f.y, &s1, &c1);
  }

  const bool norm = kind == 0 ? a.norm_q != 0 : (kind == 1 ? a.norm_k != 0 : a.norm_v != 0);
  if (norm) {
    float ss = (x[0] * x[0] + x[1] * x[1]) + (x[2] * x[2] + x[3] * x[3]);
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) ss += __shfl_xor(ss, off, 64);
    const float r = 1.0f / sqrtf(ss * (1.0f / kD) + a.eps);
    const bool scaled = kind == 0 ? a.q_scaled != 0 : (kind == 1 ? a.k_scaled != 0 : false);
    if (scaled) {
      const float* w = a.constants + kD / 2 + (kind == 1 ? kD : 0);
      const float2 w0 = *reinterpret_cast<const float2*>(w + d0);
      const float2 w1 = *reinterpret_cast<const float2*>(w + d1);
      x[0] = x[0] * r * (a.weight_offset + w0.x);
      x[1] = x[1] * r * (a.weight_offset + w0.y);
      x[2] = x[2] * r * (a.weight_offset + w1.x);
      x[3] = x[3] * r * (a.weight_offset + w1.y);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] *= r;
    }
  }
  if (rotate) {
    const float lo0 = x[0], lo1 = x[1], hi0 = x[2], hi1 = x[3];
    x[0] = lo0 * c0 - hi0 * s0;
    x[2] = hi0 * c0 + lo0 * s0;
    x[1] = lo1 * c1 - hi1 * s1;
    x[3] = hi1 * c1 + lo1 * s1;
  }

  if (kind == 0) {
    uint8_t* out = reinterpret_cast<uint8_t*>(a.q_out);
    constexpr int IOSZ = IO == kF32 ? 4 : 2;
    store_pair<IO>(out + (base + d0) * IOSZ, x[0], x[1]);
    store_pair<IO>(out + (base + d1) * IOSZ, x[2], x[3]);
    return;
  }
  uint8_t* plane = a.cache + a.geom.plane_offset(a.layer, a.seq, head, kind == 2 ? 1 : 0);
  if constexpr (KV == kI8) {
    const float* sc = a.scales + a.geom.scale_offset(a.layer, a.seq, kind == 2 ? 1 : 0, head);
    const float2 s0 = *reinterpret_cast<const float2*>(sc + d0);
    const float2 s1 = *reinterpret_cast<const float2*>(sc + d1);
    const int qv[4] = {quantise(x[0], s0.x), quantise(x[1], s0.y), quantise(x[2], s1.x), quantise(x[3], s1.y)};
    if (kind == 1) {
      *reinterpret_cast<uint16_t*>(plane + k_chunk_offset(t, d0 / EPC, kD, ESZ) + d0 % EPC) =
          (uint16_t)((qv[0] & 0xff) | ((qv[1] & 0xff) << 8));
      *reinterpret_cast<uint16_t*>(plane + k_chunk_offset(t, d1 / EPC, kD, ESZ) + d1 % EPC) =
          (uint16_t)((qv[2] & 0xff) | ((qv[3] & 0xff) << 8));
    } else {
      plane[v_elem_offset(t, d0, kD, ESZ)] = (uint8_t)qv[0];
      plane[v_elem_offset(t, d0 + 1, kD, ESZ)] = (uint8_t)qv[1];
      plane[v_elem_offset(t, d1, kD, ESZ)] = (uint8_t)qv[2];
      plane[v_elem_offset(t, d1 + 1, kD, ESZ)] = (uint8_t)qv[3];
    }
  } else {
    if (kind == 1) {
      store_pair<KV>(plane + k_chunk_offset(t, d0 / EPC, kD, ESZ) + (d0 % EPC) * ESZ, x[0], x[1]);
      store_pair<KV>(plane + k_chunk_offset(t, d1 / EPC, kD, ESZ) + (d1 % EPC) * ESZ, x[2], x[3]);
    } else {
      store_value<KV>(plane + v_elem_offset(t, d0, kD, ESZ), x[0]);
      store_value<KV>(plane + v_elem_offset(t, d0 + 1, kD, ESZ), x[1]);
      store_value<KV>(plane + v_elem_offset(t, d1, kD, ESZ), x[2]);
      store_value<KV>(plane + v_elem_offset(t, d1 + 1, kD, ESZ), x[3]);
    }
  }
}

template <int IO, int KV>
hipError_t launch_typed(const PreAttentionArgs& a, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  const int64_t rows = (int64_t)a.n * (a.hq + 2 * a.geom.hkv);
  const dim3 grid((unsigned)((rows + kRowsPerWg - 1) / kRowsPerWg));
  hipExtLaunchKernelGGL((pre_attention_kernel<IO, KV>), grid, dim3(64 * kRowsPerWg), 0, stream, ev0, ev1, 0, a);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_pre_attention(const PreAttentionArgs& a, int kv_dtype, int io_dtype, hipStream_t stream,
                                hipEvent_t ev0, hipEvent_t ev1) {
  if (a.n <= 0) return hipSuccess;
  if (a.geom.head_dim != kD) return hipErrorInvalidValue;
  if (kv_dtype == kI8 && io_dtype == kF16) return launch_typed<kF16, kI8>(a, stream, ev0, ev1);
  if (kv_dtype != io_dtype) return hipErrorInvalidValue;
  switch (io_dtype) {
    case kF32: return launch_typed<kF32, kF32>(a, stream, ev0, ev1);
    case kF16: return launch_typed<kF16, kF16>(a, stream, ev0, ev1);
    case kBF16: return launch_typed<kBF16, kBF16>(a, stream, ev0, ev1);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace mi355
