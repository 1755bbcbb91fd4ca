// Causal / sliding-window prefill attention over the KV cache (gfx950, MFMA).
//
// Grid: x = tile of query positions, y = KV head x head block, z = layer.
// A workgroup of 4 waves covers HPB query heads of one KV head times PT tiles
// of 32 consecutive positions (HPB * PT = 4); all its waves walk the same
// 32-key blocks, so each K/V block is brought from HBM/L2 into LDS once per
// workgroup and read from there as MFMA operands. The key loop starts at the
// first block the window still reaches and stops at the diagonal.
//
// Per wave and key block (32x32x16 MFMA, transposed formulation so that one
// lane owns one query):
//   S^T[key][query] = K . Q^T        16 MFMAs (head_dim 256), Q^T in registers
//   online softmax on the 16 scores a lane holds for its query
//   O^T[d][query]  += V^T . P^T      16 MFMAs, P^T taken from S^T's registers
// The row order in which K is fed to the first MFMA is chosen so that the
// probabilities already sit in the token order of the V plane.
//
// Replaces the prefill-time attention the reference reaches through
// compiled_model_.Run(prefill_signature, ...)
// (runtime/executor/llm_litert_compiled_model_executor.cc:271) and the
// [1,1,S,ctx] mask built for it
// (runtime/executor/litert_compiled_model_executor_utils.cc:332-397).
#include <hip/hip_runtime.h>
#include <math.h>

#include "attn_params.h"
#include "kernels.h"
#include <hip/hip_ext.h>

#include "mfma_util.h"

namespace mi355 {
namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kKeysPerBlock = 32;  // one V block of a 16-bit cache = two K tiles

template <int T>
struct El;
template <>
struct El<kF16> {
  using type = _Float16;
  using vec8 = h8;
  static __device__ __forceinline__ f16v mfma(vec8 a, vec8 b, f16v c) { return mfma32_f16(a, b, c); }
};
template <>
struct El<kBF16> {
  using type = __bf16;
  using vec8 = b8;
  static __device__ __forceinline__ f16v mfma(vec8 a, vec8 b, f16v c) { return mfma32_bf16(a, b, c); }
};

// Key (0..31, within a block) that MFMA row m of S^T stands for.
__device__ __forceinline__ int key_of_row(int m) { return 16 * ((m >> 3) & 1) + 8 * (m >> 4) + (m & 7); }

template <int DT, int D, int HPB>
__global__ void __launch_bounds__(256) prefill_attn_kernel(const PrefillArgs a) {
  using E = El<DT>;
  using elem_t = typename E::type;
  using vec8 = typename E::vec8;
  constexpr int PT = 4 / HPB;            // position tiles per workgroup
  constexpr int NJ = D / 16;             // K-slices of the QK^T product
  constexpr int NDP = D / 32;            // 32-channel tiles of O^T
  constexpr int kBlockBytes = 64 * D;    // one 32-key block of a 16-bit plane
  constexpr int kChunksPerThread = kBlockBytes / 16 / 256;

  __shared__ __attribute__((aligned(16))) uint8_t sm_k[kBlockBytes];
  __shared__ __attribute__((aligned(16))) uint8_t sm_v[kBlockBytes];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 31, hh = lane >> 5;
  const int hblocks = a.group / HPB;
  const int kvh = blockIdx.y / hblocks, hb = blockIdx.y - kvh * hblocks;
  const int li = blockIdx.z, layer = a.layer_begin + li;
  const int window = a.layer_window[layer];
  const int head = kvh * a.group + hb * HPB + (wave % HPB);
  const int wg_pos0 = a.q_pos0 + blockIdx.x * (32 * PT);  // first position of the workgroup
  const int pos_end = a.q_pos0 + a.n;                     // one past the last query position
  const int my_pos0 = wg_pos0 + (wave / HPB) * 32;        // first position of this wave's tile
  const int row = my_pos0 - a.q_pos0 + n;                 // query row in q / out
  const int my_pos = my_pos0 + n;
  const bool row_ok = row < a.n;

  const uint8_t* kplane = a.cache + a.geom.plane_offset(layer, a.seq, kvh, 0);
  const uint8_t* vplane = kplane + a.geom.plane_bytes;

  // Q^T operand: lane (n, hh) holds channels 16*j + 8*hh .. +7 of its query.
  vec8 qreg[NJ];
  {
    const elem_t* qrow =
        reinterpret_cast<const elem_t*>(a.q) + (((int64_t)li * a.n + (row_ok ? row : 0)) * a.hq + head) * D;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const u4 w = *reinterpret_cast<const u4*>(qrow + 16 * j + 8 * hh);
      qreg[j] = bit_cast<vec8>(row_ok ? w : u4{0, 0, 0, 0});
    }
  }

  f16v acc[NDP];
#pragma unroll
  for (int i = 0; i < NDP; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // Key blocks the workgroup walks: from the first one the window of its first
  // row reaches to the one holding the diagonal of its last valid row.
  const int last_pos = min(wg_pos0 + 32 * PT, pos_end) - 1;
  int kb_lo = 0;
  if (window > 0 && wg_pos0 - window + 1 > 0) kb_lo = (wg_pos0 - window + 1) / kKeysPerBlock;
  const int kb_hi = last_pos / kKeysPerBlock;  // inclusive
  // Blocks this wave needs (others are skipped without touching its state).
  int my_lo = 0;
  if (window > 0 && my_pos0 - window + 1 > 0) my_lo = (my_pos0 - window + 1) / kKeysPerBlock;
  const int my_hi = (my_pos0 + 31) / kKeysPerBlock;

  const float sc = a.scale, softcap = a.softcap;

  u4 pre_k[kChunksPerThread], pre_v[kChunksPerThread];
  auto prefetch = [&](int kb) {
    const uint8_t* kg = kplane + (int64_t)kb * kBlockBytes;
    const uint8_t* vg = vplane + (int64_t)kb * kBlockBytes;
#pragma unroll
    for (int i = 0; i < kChunksPerThread; ++i) {
      pre_k[i] = *reinterpret_cast<const u4*>(kg + (tid + 256 * i) * 16);
      pre_v[i] = *reinterpret_cast<const u4*>(vg + (tid + 256 * i) * 16);
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int i = 0; i < kChunksPerThread; ++i) {
      *reinterpret_cast<u4*>(sm_k + (tid + 256 * i) * 16) = pre_k[i];
      *reinterpret_cast<u4*>(sm_v + (tid + 256 * i) * 16) = pre_v[i];
    }
  };

  if (kb_lo <= kb_hi) prefetch(kb_lo);
  for (int kb = kb_lo; kb <= kb_hi; ++kb) {
    __syncthreads();  // everyone finished reading the previous block
    commit();
    __syncthreads();
    if (kb + 1 <= kb_hi) prefetch(kb + 1);
    if (kb < my_lo || kb > my_hi) continue;

    // ---- S^T = K . Q^T
    f16v s;
#pragma unroll
    for (int e = 0; e < 16; ++e) s[e] = 0.f;
    {
      const int key = key_of_row(n);
      const uint8_t* kb_base = sm_k + (key >> 4) * (16 * D * 2) + (key & 15) * 16;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const vec8 kop = *reinterpret_cast<const vec8*>(kb_base + (2 * j + hh) * 256);
        s = E::mfma(kop, qreg[j], s);
      }
    }

    // ---- online softmax; this lane holds 16 keys of query n
    const int key0 = kb * kKeysPerBlock;
    const bool interior = (key0 + 31 <= my_pos0) && (window <= 0 || my_pos0 + 31 - key0 < window);
    float bm = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float x = s[i] * sc;
      if (softcap > 0.f) x = softcap * tanhf(x / softcap);
      x *= kLog2e;
      if (!interior) {
        const int key = key0 + key_of_row(8 * (i >> 2) + 4 * hh + (i & 3));
        const bool vis = key <= my_pos && (window <= 0 || my_pos - key < window);
        x = vis ? x : -INFINITY;
      }
      s[i] = x;
      bm = fmaxf(bm, x);
    }
    bm = wave_xor_max(bm, 32);
    const float m_new = fmaxf(m_run, bm);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_use);
    float lsum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float p = fast_exp2(s[i] - m_use);
      s[i] = p;
      lsum += p;
    }
    l_run = l_run * alpha + lsum;
    m_run = m_new;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int dp = 0; dp < NDP; ++dp) acc[dp] *= alpha;
    }

    // ---- O^T += V^T . P^T
    const uint8_t* vb_base = sm_v + (n >> 4) * 1024 + hh * 256 + (n & 15) * 16;
    if constexpr (DT == kBF16) {
      // bf16 keeps 8 significant bits; feeding P as hi + lo parts keeps ~16 of
      // them, otherwise P.V alone carries ~1e-3 of relative error.
      vec8 p0, p1, q0, q1;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        p0[e] = (elem_t)s[e];
        p1[e] = (elem_t)s[8 + e];
        q0[e] = (elem_t)(s[e] - (float)p0[e]);
        q1[e] = (elem_t)(s[8 + e] - (float)p1[e]);
      }
#pragma unroll
      for (int dp = 0; dp < NDP; ++dp) {
        const vec8 v0 = *reinterpret_cast<const vec8*>(vb_base + dp * 2048);
        const vec8 v1 = *reinterpret_cast<const vec8*>(vb_base + dp * 2048 + 512);
        acc[dp] = E::mfma(v0, p0, acc[dp]);
        acc[dp] = E::mfma(v1, p1, acc[dp]);
        acc[dp] = E::mfma(v0, q0, acc[dp]);
        acc[dp] = E::mfma(v1, q1, acc[dp]);
      }
    } else {
      vec8 p0, p1;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        p0[e] = (elem_t)s[e];
        p1[e] = (elem_t)s[8 + e];
      }
#pragma unroll
      for (int dp = 0; dp < NDP; ++dp) {
        const vec8 v0 = *reinterpret_cast<const vec8*>(vb_base + dp * 2048);
        const vec8 v1 = *reinterpret_cast<const vec8*>(vb_base + dp * 2048 + 512);
        acc[dp] = E::mfma(v0, p0, acc[dp]);
        acc[dp] = E::mfma(v1, p1, acc[dp]);
      }
    }
  }

  // ---- normalise and store: lane (n, hh) holds channels 32*dp + 8*a + 4*hh + b
  const float l_tot = wave_xor_add(l_run, 32);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (row_ok) {
    elem_t* orow = reinterpret_cast<elem_t*>(a.out) + (((int64_t)li * a.n + row) * a.hq + head) * D;
#pragma unroll
    for (int dp = 0; dp < NDP; ++dp) {
#pragma unroll
      for (int aa = 0; aa < 4; ++aa) {
        elem_t o[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) o[b] = (elem_t)(acc[dp][4 * aa + b] * inv);
        *reinterpret_cast<u2*>(orow + 32 * dp + 8 * aa + 4 * hh) = *reinterpret_cast<const u2*>(o);
      }
    }
  }
}

template <int DT, int D>
hipError_t launch_typed(const PrefillArgs& a, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  const int G = a.group;
  const int hpb = (G % 4 == 0) ? 4 : ((G % 2 == 0) ? 2 : 1);
  const int pt = 4 / hpb;
  const dim3 grid((a.n + 32 * pt - 1) / (32 * pt), a.geom.hkv * (G / hpb), a.n_layers);
  // ev0/ev1 ride on the dispatch: the kernel's own begin / end timestamps
  if (hpb == 4) hipExtLaunchKernelGGL((prefill_attn_kernel<DT, D, 4>), grid, dim3(256), 0, stream, ev0, ev1, 0, a);
  else if (hpb == 2) hipExtLaunchKernelGGL((prefill_attn_kernel<DT, D, 2>), grid, dim3(256), 0, stream, ev0, ev1, 0, a);
  else hipExtLaunchKernelGGL((prefill_attn_kernel<DT, D, 1>), grid, dim3(256), 0, stream, ev0, ev1, 0, a);
  return hipGetLastError();
}

}  // namespace

bool prefill_supported(int kv_dtype, int io_dtype, int head_dim) {
  return head_dim == 256 && kv_dtype == io_dtype && (kv_dtype == kF16 || kv_dtype == kBF16);
}

hipError_t launch_prefill(const PrefillArgs& a, int kv_dtype, int io_dtype, hipStream_t stream, hipEvent_t ev0,
                          hipEvent_t ev1) {
  (void)io_dtype;
  if (kv_dtype == kF16) return launch_typed<kF16, 256>(a, stream, ev0, ev1);
  if (kv_dtype == kBF16) return launch_typed<kBF16, 256>(a, stream, ev0, ev1);
  return hipErrorInvalidValue;
}

}  // namespace mi355
