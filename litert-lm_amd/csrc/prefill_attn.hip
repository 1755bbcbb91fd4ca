// Causal / sliding-window prefill attention over the KV cache (gfx950, MFMA).
//
// Grid: x = (layer, KV head, head block), y = tile of query positions, longest
// key loops first. A workgroup of 4 waves covers HPB query heads of one KV head
// times PT tiles of 32 consecutive positions (HPB * PT = 4); all its waves walk
// the same 32-key blocks, so each K/V block is brought from HBM/L2 into a
// three-stage LDS ring once per workgroup (global_load ... lds, no registers
// in between, two iterations ahead) and read from there as MFMA operands, the
// K operands one block ahead of their use. The key loop starts at the first block the window still reaches
// and stops at the diagonal.
//
// Per wave and key block (32x32x16 MFMA, transposed formulation so that one
// lane owns one query):
//   S^T[key][query] = K . Q^T        16 MFMAs (head_dim 256), Q^T in a per-wave LDS slice
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
constexpr float kRescaleSlack = 8.f;  // log2 units a score may exceed the reference max before it is moved

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

// LDS plan (dynamic): a ring of three K blocks, a ring of three V blocks and
// the Q^T operands of the four waves: (3 + 3) * 64*D + 4 * (D/16) KiB = 160 KiB
// at head_dim 256, the whole LDS of a CU.
constexpr int kStages = 3;
template <int D>
constexpr int prefill_lds_bytes() { return 2 * kStages * 64 * D + 4 * (D / 16) * 1024; }

// s_waitcnt immediates (gfx9 encoding: vmcnt[3:0], expcnt[6:4], lgkmcnt[11:8],
// vmcnt[15:14]) that wait on vector-memory operations only.
constexpr int kWaitVm0 = 0x0F70;  // all of this wave's transfers have landed
constexpr int kWaitVm4 = 0x0F74;  // all but the 4 most recent ones
constexpr int kWaitVm8 = 0x0F78;  // all but the 8 most recent ones

template <int DT, int D, int HPB>
__global__ void __launch_bounds__(256) prefill_attn_kernel(const PrefillArgs a) {
  using E = El<DT>;
  using elem_t = typename E::type;
  using vec8 = typename E::vec8;
  constexpr int PT = 4 / HPB;            // position tiles per workgroup
  constexpr int NJ = D / 16;             // K-slices of the QK^T product
  constexpr int NDP = D / 32;            // 32-channel tiles of O^T
  constexpr int kBlockBytes = 64 * D;    // one 32-key block of a 16-bit plane

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint8_t* const sm_k = smem;                              // [kStages][K block]
  uint8_t* const sm_v = smem + kStages * kBlockBytes;      // [kStages][V block]
  vec8* const sm_q_all = reinterpret_cast<vec8*>(smem + 2 * kStages * kBlockBytes);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, hh = lane >> 5;
  // x = (layer, KV head, head block), y = position tile, heaviest tiles first:
  // workgroups are dispatched x-fastest, so every layer's longest key loops
  // start before any short one.
  const int hblocks = a.group / HPB;
  const int per_layer = a.geom.hkv * hblocks;
  const int li = blockIdx.x / per_layer, rem = blockIdx.x - li * per_layer;
  const int kvh = rem / hblocks, hb = rem - kvh * hblocks;
  const int tile = gridDim.y - 1 - blockIdx.y;
  const int layer = a.layer_begin + li;
  const int window = a.layer_window[layer];
  const int head = kvh * a.group + hb * HPB + (wave % HPB);
  const int wg_pos0 = a.q_pos0 + tile * (32 * PT);   // first position of the workgroup
  const int pos_end = a.q_pos0 + a.n;                // one past the last query position
  const int my_pos0 = wg_pos0 + (wave / HPB) * 32;   // first position of this wave's tile
  const int row = my_pos0 - a.q_pos0 + n;            // query row in q / out
  const int my_pos = my_pos0 + n;
  const bool row_ok = row < a.n;

  const uint8_t* kplane = a.cache + a.geom.plane_offset(layer, a.seq, kvh, 0);
  const uint8_t* vplane = kplane + a.geom.plane_bytes;

  // Key blocks the workgroup walks: from the first one the window of its first
  // row reaches to the one holding the diagonal of its last valid row. Every
  // wave walks all of them (blocks outside its own tile's range are masked).
  const int last_pos = min(wg_pos0 + 32 * PT, pos_end) - 1;
  int kb_lo = 0;
  if (window > 0 && wg_pos0 - window + 1 > 0) kb_lo = (wg_pos0 - window + 1) / kKeysPerBlock;
  const int nblk = last_pos / kKeysPerBlock - kb_lo + 1;

  // A K or V block travels HBM/L2 -> LDS without touching registers: every
  // wave issues 4 of the 16 wave-wide 1 KiB transfers of a block; the data of
  // lane l lands at the stage offset of the transfer + 16 * l.
  auto fetch = [&](const uint8_t* plane, uint8_t* ring, int i) {
    const uint8_t* g = plane + (int64_t)(kb_lo + i) * kBlockBytes + lane * 16;
    uint8_t* dst = ring + (i % kStages) * kBlockBytes;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int off = (wave + 4 * t) * 1024;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(g + off),
                                       (__attribute__((address_space(3))) void*)(dst + off), 16, 0, 0);
    }
  };
  // Ring protocol. Iteration i requests K block i+3 and V block i+2: the stage
  // of K(i+3) held K(i), whose operands went to registers during iteration
  // i-1; the stage of V(i+2) held V(i-1). At the bottom of iteration i every
  // wave waits for its share of K(i+2) and V(i+1) (requested one iteration
  // earlier), so after the barrier iteration i+1 finds V(i+1) and K(i+2)
  // resident: every transfer has two iterations to land.
  fetch(kplane, sm_k, 0);
  fetch(vplane, sm_v, 0);
  if (nblk > 1) { fetch(kplane, sm_k, 1); fetch(vplane, sm_v, 1); }
  if (nblk > 2) fetch(kplane, sm_k, 2);

  // Q^T operand in this wave's LDS slice: entry (j, lane) with lane = (n, hh)
  // holds channels 16*j + 8*hh .. +7 of the lane's query. A lane reads back only
  // what it wrote itself.
  vec8* const sm_q = sm_q_all + wave * (NJ * 64) + lane;
  {
    const elem_t* qrow =
        reinterpret_cast<const elem_t*>(a.q) + (((int64_t)li * a.n + (row_ok ? row : 0)) * a.hq + head) * D;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const u4 w = *reinterpret_cast<const u4*>(qrow + 16 * j + 8 * hh);
      sm_q[j * 64] = bit_cast<vec8>(row_ok ? w : u4{0, 0, 0, 0});
    }
  }

  f16v acc[NDP];
#pragma unroll
  for (int i = 0; i < NDP; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const float sc = a.scale, softcap = a.softcap;

  // LDS offsets of this lane's operands inside a block
  const int key_row = key_of_row(n);
  const int k_off = (key_row >> 4) * (16 * D * 2) + (key_row & 15) * 16 + hh * 256;
  const int v_off = (n >> 4) * 1024 + hh * 256 + (n & 15) * 16;

  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();  // the first blocks are resident

  // Operand registers: all K slices of the coming block and the first half of
  // the Q slices are read one phase ahead of their MFMAs.
  vec8 kop[NJ], qa[NJ / 2], qb[NJ / 2], vop[2 * NDP];
#pragma unroll
  for (int j = 0; j < NJ; ++j) kop[j] = *reinterpret_cast<const vec8*>(sm_k + k_off + j * 512);
#pragma unroll
  for (int j = 0; j < NJ / 2; ++j) qa[j] = sm_q[j * 64];

  for (int i = 0; i < nblk; ++i) {
    const bool fetch_k = i + 3 < nblk, fetch_v = i + 2 < nblk;
    if (fetch_k) fetch(kplane, sm_k, i + 3);
    if (fetch_v) fetch(vplane, sm_v, i + 2);

    // ---- S^T = K . Q^T; the second half of the Q slices arrives under the
    // first eight MFMAs
#pragma unroll
    for (int j = 0; j < NJ / 2; ++j) qb[j] = sm_q[(NJ / 2 + j) * 64];
    f16v s;
#pragma unroll
    for (int e = 0; e < 16; ++e) s[e] = 0.f;
#pragma unroll
    for (int j = 0; j < NJ / 2; ++j) s = E::mfma(kop[j], qa[j], s);
#pragma unroll
    for (int j = 0; j < NJ / 2; ++j) s = E::mfma(kop[NJ / 2 + j], qb[j], s);
    __builtin_amdgcn_sched_barrier(0);

    // V operands of this block are requested now and arrive while the softmax runs
    {
      const uint8_t* vb = sm_v + (i % kStages) * kBlockBytes + v_off;
#pragma unroll
      for (int dp = 0; dp < NDP; ++dp) {
        vop[2 * dp] = *reinterpret_cast<const vec8*>(vb + dp * 2048);
        vop[2 * dp + 1] = *reinterpret_cast<const vec8*>(vb + dp * 2048 + 512);
      }
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- online softmax in the exp2 domain; this lane holds 16 keys of query n.
    // The reference max m_run only moves when some score of the wave exceeds
    // it by more than kRescaleSlack (2^8 in probability): until then p is
    // taken against the stale max (p <= 256, harmless in fp32 / fp16 / bf16)
    // and neither the cross-lane max nor the rescale of the 128 accumulator
    // registers is needed. m_run is shared by the two lanes of a query.
    if (softcap > 0.f) {
      const float inv_cap = sc / softcap, cap2 = softcap * kLog2e;
#pragma unroll
      for (int e = 0; e < 16; ++e) s[e] = cap2 * fast_tanh(s[e] * inv_cap);
    } else {
      s *= sc * kLog2e;
    }
    const int key0 = (kb_lo + i) * kKeysPerBlock;
    const bool interior = (key0 + 31 <= my_pos0) && (window <= 0 || my_pos0 + 31 - key0 < window);
    if (!interior) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int key = key0 + key_of_row(8 * (e >> 2) + 4 * hh + (e & 3));
        const bool vis = key <= my_pos && (window <= 0 || my_pos - key < window);
        s[e] = vis ? s[e] : -INFINITY;
      }
    }
    float bm = s[0];
#pragma unroll
    for (int e = 1; e < 16; ++e) bm = fmaxf(bm, s[e]);
    if (__any(bm > m_run + kRescaleSlack)) {
      bm = wave_xor_max(bm, 32);
      const float m_new = fmaxf(m_run, bm);
      const float alpha = (m_new == -INFINITY) ? 1.f : fast_exp2(m_run - m_new);
      l_run *= alpha;
      // The accumulators live in AGPRs (the MFMAs read and write them there);
      // the two pins keep their detour through VGPRs inside this rare block.
#pragma unroll
      for (int dp = 0; dp < NDP; ++dp) asm volatile("" : "+a"(acc[dp]));
#pragma unroll
      for (int dp = 0; dp < NDP; ++dp) acc[dp] *= alpha;
#pragma unroll
      for (int dp = 0; dp < NDP; ++dp) asm volatile("" : "+a"(acc[dp]));
      m_run = m_new;
    }
    const float m_use = (m_run == -INFINITY) ? 0.f : m_run;
    float lsum = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      s[e] = fast_exp2(s[e] - m_use);
      lsum += s[e];
    }
    l_run += lsum;

    // K operands of the next block (resident since the previous barrier) and
    // the first half of the Q slices are requested now and arrive during P.V
    __builtin_amdgcn_sched_barrier(0);
    if (i + 1 < nblk) {
      const uint8_t* nx = sm_k + ((i + 1) % kStages) * kBlockBytes + k_off;
#pragma unroll
      for (int j = 0; j < NJ; ++j) kop[j] = *reinterpret_cast<const vec8*>(nx + j * 512);
#pragma unroll
      for (int j = 0; j < NJ / 2; ++j) qa[j] = sm_q[j * 64];
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- O^T += V^T . P^T
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
        acc[dp] = E::mfma(vop[2 * dp], p0, acc[dp]);
        acc[dp] = E::mfma(vop[2 * dp + 1], p1, acc[dp]);
        acc[dp] = E::mfma(vop[2 * dp], q0, acc[dp]);
        acc[dp] = E::mfma(vop[2 * dp + 1], q1, acc[dp]);
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
        acc[dp] = E::mfma(vop[2 * dp], p0, acc[dp]);
        acc[dp] = E::mfma(vop[2 * dp + 1], p1, acc[dp]);
      }
    }

    // this wave's shares of K(i+2) and V(i+1) have landed; what was requested
    // in this iteration may still be in flight
    if (fetch_k) __builtin_amdgcn_s_waitcnt(kWaitVm8);
    else if (fetch_v) __builtin_amdgcn_s_waitcnt(kWaitVm4);
    else __builtin_amdgcn_s_waitcnt(kWaitVm0);
    __syncthreads();
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

template <int DT, int D, int HPB>
hipError_t launch_hpb(const PrefillArgs& a, dim3 grid, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  constexpr int kLds = prefill_lds_bytes<D>();
  static bool configured = false;  // more than 64 KiB of LDS has to be requested once per kernel
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_attn_kernel<DT, D, HPB>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess) return e;
    configured = true;
  }
  // ev0/ev1 ride on the dispatch: the kernel's own begin / end timestamps
  hipExtLaunchKernelGGL((prefill_attn_kernel<DT, D, HPB>), grid, dim3(256), kLds, stream, ev0, ev1, 0, a);
  return hipGetLastError();
}

template <int DT, int D>
hipError_t launch_typed(const PrefillArgs& a, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  const int G = a.group;
  const int hpb = (G % 4 == 0) ? 4 : ((G % 2 == 0) ? 2 : 1);
  const int pt = 4 / hpb;
  const dim3 grid(a.n_layers * a.geom.hkv * (G / hpb), (a.n + 32 * pt - 1) / (32 * pt), 1);
  if (hpb == 4) return launch_hpb<DT, D, 4>(a, grid, stream, ev0, ev1);
  if (hpb == 2) return launch_hpb<DT, D, 2>(a, grid, stream, ev0, ev1);
  return launch_hpb<DT, D, 1>(a, grid, stream, ev0, ev1);
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
