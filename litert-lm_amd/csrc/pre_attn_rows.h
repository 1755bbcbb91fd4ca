// The arithmetic of the step before attention for one row of head_dim 256 held by one wave: per-head
// RMS norm, rotary position embedding, and the stores of a key / value row into the cache planes.
// Shared by pre_attention_kernel (pre_attn.hip) and by the decode kernel that runs the step for its
// one new token itself (decode_attn.hip), so that both leave the same bits.
//
// A lane owns the channel pairs (2l, 2l+1) and (128+2l, 128+2l+1): both members of every rotated
// pair (d, d+128) are in the same lane and the only cross-lane step is the sum of squares of the norm.
//
// The arithmetic is compiled without contraction of multiplies and adds into FMAs: which of two
// products the compiler fuses depends on the code around it, and the two kernels would then round
// differently now and then (seen: a value row's norm, one ulp apart, in one of some hundred rows).
#ifndef LITERT_LM_AMD_CSRC_PRE_ATTN_ROWS_H_
#define LITERT_LM_AMD_CSRC_PRE_ATTN_ROWS_H_

#include <hip/hip_runtime.h>

#include "attn_params.h"
#include "mfma_util.h"

namespace mi355 {

constexpr int kRowD = 256;

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
#pragma clang fp contract(off)
  const float inv = scale != 0.f ? 1.0f / scale : 0.f;
  const float r = roundf(x * inv);
  return (int)fminf(fmaxf(r, -127.f), 127.f);
}

// Sine / cosine of the lane's two angles at position t (they depend on the position only);
// inv_freq: the layer's [128] rotary frequencies, nullptr: no rotation.
struct RowAngles {
  float s0, c0, s1, c1;
};
__device__ __forceinline__ RowAngles row_angles(const float* inv_freq, int t, int lane) {
#pragma clang fp contract(off)
  RowAngles r{0.f, 1.f, 0.f, 1.f};
  if (inv_freq) {
    const float2 f = *reinterpret_cast<const float2*>(inv_freq + 2 * lane);  // frequencies of pairs 2l, 2l+1
    sincosf((float)t * f.x, &r.s0, &r.c0);
    sincosf((float)t * f.y, &r.s1, &r.c1);
  }
  return r;
}

// x = the lane's channels 2l, 2l+1, 128+2l, 128+2l+1 of one row. norm: RMS-normalise the row (eps inside the
// root), then scale channel d by weight_offset + weights[d] when weights != nullptr; rotate: apply `ang`.
// (Flags and pointers come as plain values: picked out of a struct by the row's kind, the struct ends up in
// memory and the kernel several times slower.)
__device__ __forceinline__ void transform_row(float (&x)[4], bool norm, const float* weights, float weight_offset,
                                              float eps, bool rotate, const RowAngles& ang, int lane) {
#pragma clang fp contract(off)
  const int d0 = 2 * lane, d1 = kRowD / 2 + 2 * lane;
  if (norm) {
    float ss = (x[0] * x[0] + x[1] * x[1]) + (x[2] * x[2] + x[3] * x[3]);
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) ss += __shfl_xor(ss, off, 64);
    const float r = 1.0f / sqrtf(ss * (1.0f / kRowD) + eps);
    if (weights) {
      const float2 w0 = *reinterpret_cast<const float2*>(weights + d0);
      const float2 w1 = *reinterpret_cast<const float2*>(weights + d1);
      x[0] = x[0] * r * (weight_offset + w0.x);
      x[1] = x[1] * r * (weight_offset + w0.y);
      x[2] = x[2] * r * (weight_offset + w1.x);
      x[3] = x[3] * r * (weight_offset + w1.y);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] *= r;
    }
  }
  if (rotate) {
    const float lo0 = x[0], lo1 = x[1], hi0 = x[2], hi1 = x[3];
    x[0] = lo0 * ang.c0 - hi0 * ang.s0;
    x[2] = hi0 * ang.c0 + lo0 * ang.s0;
    x[1] = lo1 * ang.c1 - hi1 * ang.s1;
    x[3] = hi1 * ang.c1 + lo1 * ang.s1;
  }
}

// The layer's constants: [128] rotary frequencies, [256] query norm weights, [256] key norm weights.
__device__ __forceinline__ const float* row_weights(const float* constants, int kind, bool q_scaled, bool k_scaled) {
  if (kind == 0) return q_scaled ? constants + kRowD / 2 : nullptr;
  if (kind == 1) return k_scaled ? constants + kRowD / 2 + kRowD : nullptr;
  return nullptr;
}

// The transformed key (is_v 0) or value (is_v 1) row of token t into its plane; `scales` = the plane's
// [256] dequantisation scales (int8 cache only). LINEAR: `plane` is a buffer of 256 elements instead and
// element d of the row goes to element d of the buffer, in the same element format.
template <int KV, bool LINEAR = false>
__device__ __forceinline__ void store_cache_row(uint8_t* plane, const float* scales, int is_v, int t,
                                                const float (&x)[4], int lane) {
  constexpr int ESZ = KV == kF32 ? 4 : (KV == kI8 ? 1 : 2);
  constexpr int EPC = 16 / ESZ;
  const int d0 = 2 * lane, d1 = kRowD / 2 + 2 * lane;
  auto k_chunk_offset = [](int tt, int c, int, int) -> int64_t {
    return LINEAR ? (int64_t)c * 16 : mi355::k_chunk_offset(tt, c, kRowD, ESZ);
  };
  auto v_elem_offset = [](int tt, int d, int, int) -> int64_t {
    return LINEAR ? (int64_t)d * ESZ : mi355::v_elem_offset(tt, d, kRowD, ESZ);
  };
  if constexpr (KV == kI8) {
    const float2 s0 = *reinterpret_cast<const float2*>(scales + d0);
    const float2 s1 = *reinterpret_cast<const float2*>(scales + d1);
    const int qv[4] = {quantise(x[0], s0.x), quantise(x[1], s0.y), quantise(x[2], s1.x), quantise(x[3], s1.y)};
    if (!is_v) {
      *reinterpret_cast<uint16_t*>(plane + k_chunk_offset(t, d0 / EPC, kRowD, ESZ) + d0 % EPC) =
          (uint16_t)((qv[0] & 0xff) | ((qv[1] & 0xff) << 8));
      *reinterpret_cast<uint16_t*>(plane + k_chunk_offset(t, d1 / EPC, kRowD, ESZ) + d1 % EPC) =
          (uint16_t)((qv[2] & 0xff) | ((qv[3] & 0xff) << 8));
    } else {
      plane[v_elem_offset(t, d0, kRowD, ESZ)] = (uint8_t)qv[0];
      plane[v_elem_offset(t, d0 + 1, kRowD, ESZ)] = (uint8_t)qv[1];
      plane[v_elem_offset(t, d1, kRowD, ESZ)] = (uint8_t)qv[2];
      plane[v_elem_offset(t, d1 + 1, kRowD, ESZ)] = (uint8_t)qv[3];
    }
  } else {
    if (!is_v) {
      store_pair<KV>(plane + k_chunk_offset(t, d0 / EPC, kRowD, ESZ) + (d0 % EPC) * ESZ, x[0], x[1]);
      store_pair<KV>(plane + k_chunk_offset(t, d1 / EPC, kRowD, ESZ) + (d1 % EPC) * ESZ, x[2], x[3]);
    } else {
      store_value<KV>(plane + v_elem_offset(t, d0, kRowD, ESZ), x[0]);
      store_value<KV>(plane + v_elem_offset(t, d0 + 1, kRowD, ESZ), x[1]);
      store_value<KV>(plane + v_elem_offset(t, d1, kRowD, ESZ), x[2]);
      store_value<KV>(plane + v_elem_offset(t, d1 + 1, kRowD, ESZ), x[3]);
    }
  }
}

}  // namespace mi355
#endif  // LITERT_LM_AMD_CSRC_PRE_ATTN_ROWS_H_
