// Vector types, MFMA wrappers and small device helpers for gfx950 (wave64).
//
// Operand layouts relied on (each verified on hardware by the parity tests):
//   mfma 16x16xK: A lane l supplies row l%16, K-slice group l/16;
//                 B lane l supplies column l%16, the same K-slice group;
//                 D lane l holds rows 4*(l/16)+i (i=0..3) of column l%16.
//   mfma 32x32xK: A lane l supplies row l%32, K-slice group l/32; B likewise
//                 for column l%32; D lane l holds rows 8*(i/4)+4*(l/32)+i%4
//                 (i=0..15) of column l%32.
#ifndef LITERT_LM_AMD_CSRC_MFMA_UTIL_H_
#define LITERT_LM_AMD_CSRC_MFMA_UTIL_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355 {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef __bf16 b4 __attribute__((ext_vector_type(4)));
typedef unsigned u4 __attribute__((ext_vector_type(4)));
typedef unsigned u2 __attribute__((ext_vector_type(2)));

// Streaming 16-byte load: K/V rows are read once per call, so they bypass
// cache retention (measured: ~7.1 TB/s against ~6.0 TB/s for plain loads).
__device__ __forceinline__ u4 load_stream16(const uint8_t* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u4*>(p));
}

__device__ __forceinline__ f4 mfma16_f16(h8 a, h8 b, f4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f4 mfma16_bf16(b8 a, b8 b, f4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f4 mfma16_f32(float a, float b, f4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f16v mfma32_f16(h8 a, h8 b, f16v c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f16v mfma32_bf16(b8 a, b8 b, f16v c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

template <class To, class From>
__device__ __forceinline__ To bit_cast(const From& f) {
  static_assert(sizeof(To) == sizeof(From), "size mismatch");
  return __builtin_bit_cast(To, f);
}

// 16 two's-complement int8 (one 16-byte chunk) -> two h8, element order kept.
// byte ^ 0x80 = value + 128; 0x6400 | that = fp16(1024 + value + 128).
__device__ __forceinline__ void cvt_i8x16_to_h8x2(u4 w, h8& lo, h8& hi) {
  unsigned o[8];
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const unsigned x = w[d] ^ 0x80808080u;
    o[2 * d] = __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u);      // bytes 0,1
    o[2 * d + 1] = __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u);  // bytes 2,3
  }
  const h8 bias = {1152, 1152, 1152, 1152, 1152, 1152, 1152, 1152};
  u4 a = {o[0], o[1], o[2], o[3]}, b = {o[4], o[5], o[6], o[7]};
  lo = bit_cast<h8>(a) - bias;
  hi = bit_cast<h8>(b) - bias;
}

// 8 two's-complement int8 (8 bytes) -> one h8, element order kept (half of cvt_i8x16_to_h8x2).
__device__ __forceinline__ h8 cvt_i8x8_to_h8(u2 w) {
  unsigned o[4];
#pragma unroll
  for (int d = 0; d < 2; ++d) {
    const unsigned x = w[d] ^ 0x80808080u;
    o[2 * d] = __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u);
    o[2 * d + 1] = __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u);
  }
  const h8 bias = {1152, 1152, 1152, 1152, 1152, 1152, 1152, 1152};
  const u4 a = {o[0], o[1], o[2], o[3]};
  return bit_cast<h8>(a) - bias;
}

// bfloat16 bits -> the IEEE half that a V plane of a bfloat16 cache stores (exact for
// 2^-17 <= |v| <= 65504, finite values above saturate, nearest multiple of 2^-24 below), and back.
// NaN and +-infinity pass through as NaN and +-infinity (fminf / fmaxf would turn a NaN into a bound).
__device__ __forceinline__ uint16_t bf16_bits_to_half_bits(uint16_t b) {
  const float f = __uint_as_float((uint32_t)b << 16);
  const bool finite = (b & 0x7F80u) != 0x7F80u;
  const _Float16 h = (_Float16)(finite ? fminf(fmaxf(f, -65504.f), 65504.f) : f);
  return bit_cast<uint16_t>(h);
}
__device__ __forceinline__ uint16_t half_bits_to_bf16_bits(uint16_t hb) {
  const float f = (float)bit_cast<_Float16>(hb);  // at most 11 significant bits; what came from a bfloat16 has 8
  return bit_cast<uint16_t>((__bf16)f);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// tanh(y) = sign(y) * (1 - t) / (1 + t), t = exp(-2|y|): no overflow, no branch.
__device__ __forceinline__ float fast_tanh(float y) {
  const float t = __builtin_amdgcn_exp2f(-2.8853900817779268f * fabsf(y));
  const float r = (1.f - t) * __builtin_amdgcn_rcpf(1.f + t);
  return copysignf(r, y);
}

__device__ __forceinline__ float wave_xor_max(float v, int mask) { return fmaxf(v, __shfl_xor(v, mask, 64)); }
__device__ __forceinline__ float wave_xor_add(float v, int mask) { return v + __shfl_xor(v, mask, 64); }

}  // namespace mi355
#endif  // LITERT_LM_AMD_CSRC_MFMA_UTIL_H_
