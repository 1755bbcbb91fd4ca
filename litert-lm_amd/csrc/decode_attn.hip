// One-token decode attention over the KV cache (gfx950, wave64, MFMA).
//
// Grid: x = split-KV partition, y = KV head, z = (layer, sequence) item.
// A workgroup of NW waves streams the K and V rows of its partition exactly
// once. Each wave owns every NW-th block of VB tokens and, per block, issues
// 32 wave-wide 1 KiB streaming loads (16 of K, 16 of V at head_dim 256); the
// K loads of the next block are issued as soon as the current scores exist and
// the V loads right after P.V, so memory stays busy during the arithmetic. Scores are
// S^T = K . Q^T on the matrix cores with the (at most 16) query heads of the KV
// head in the column dimension, so each lane keeps the running max / sum of
// one query head; the probabilities leave the first MFMA already in the
// operand layout of the second (O^T = V^T . P^T). Waves are merged through
// LDS; partitions write (max, sum, accumulator) partials to a workspace that a
// small second kernel merges by log-sum-exp.
//
// Replaces the decode-time attention that the reference reaches through
// compiled_model_.Run("decode", ...)
// (runtime/executor/llm_litert_compiled_model_executor.cc:407,522).
#include <hip/hip_runtime.h>
#include <math.h>

#include "attn_params.h"
#include "kernels.h"
#include <hip/hip_ext.h>

#include "mfma_util.h"
#include "pre_attn_rows.h"

namespace mi355 {
namespace {

constexpr float kLog2e = 1.4426950408889634f;

template <int KV>
struct KvT;
template <>
struct KvT<kF16> { static constexpr int EPC = 8, VB = 32; };
template <>
struct KvT<kBF16> { static constexpr int EPC = 8, VB = 32; };
template <>
struct KvT<kF32> { static constexpr int EPC = 4, VB = 16; };
template <>
struct KvT<kI8> { static constexpr int EPC = 16, VB = 64; };

template <int IO>
struct IoT;
template <>
struct IoT<kF32> { using type = float; };
template <>
struct IoT<kF16> { using type = _Float16; };
template <>
struct IoT<kBF16> { using type = __bf16; };

// A block of VB tokens is 64*D bytes in both planes, laid out so that load i
// of a wave is bytes [i*1024, (i+1)*1024) of the block. Buffer loads keep the
// plane base and the block offset in scalar registers (one VGPR of address per
// lane for all 32 loads) and are bounds-checked against the plane size.
constexpr int kStreamingLoad = 2;  // "nt": the rows are read once per call

__device__ __forceinline__ __amdgpu_buffer_rsrc_t plane_resource(const uint8_t* plane, int64_t plane_bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(plane), 0, (int)plane_bytes, 0x00020000);
}

template <int D>
__device__ __forceinline__ void load_plane_block(u4 (&r)[D / 16], __amdgpu_buffer_rsrc_t rsrc, int block_off,
                                                 int lane_off) {
#pragma unroll
  for (int i = 0; i < D / 16; ++i)
    r[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_off + (i & 3) * 1024, block_off + (i >> 2) * 4096,
                                                 kStreamingLoad);
}

// Q^T as the B operand, kept by every wave in its own LDS slice as [step][lane]
// 16-byte entries: entry (jj, lane) with n = lane%16, g = lane/16 holds the
// elements of query head n that pair with K chunk 4*jj + g (for an int8 cache:
// with one half of that chunk, pre-multiplied by the K scales). Heads
// n >= group are zero columns. A lane only ever reads the entries it wrote
// itself, so no barrier is needed; keeping Q out of the register file leaves
// room for two waves per SIMD next to the 128 registers of K/V data in flight.
// q_rows: the `group` query rows of this KV head, [group][D] (in HBM, or in LDS when the kernel has
// produced them itself).
// Eight consecutive query elements of the io type as float32 (two vectors of four: plain values, no array
// that could end up in scratch memory).
struct Q8 { f4 lo, hi; };
template <int IO>
__device__ __forceinline__ Q8 load_q8(const typename IoT<IO>::type* p) {
  Q8 r;
  if constexpr (IO == kF32) {
    r.lo = *reinterpret_cast<const f4*>(p);
    r.hi = *reinterpret_cast<const f4*>(p + 4);
  } else if constexpr (IO == kF16) {
    const h8 v = *reinterpret_cast<const h8*>(p);
    r.lo = f4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
    r.hi = f4{(float)v[4], (float)v[5], (float)v[6], (float)v[7]};
  } else {
    const b8 v = *reinterpret_cast<const b8*>(p);
    r.lo = f4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
    r.hi = f4{(float)v[4], (float)v[5], (float)v[6], (float)v[7]};
  }
  return r;
}

// The activation type (IO: queries in, attention out) need not be the cache's: a 16-bit cache serves float32
// activations (the reference's ActivationDataType::FLOAT32 over its fp16 GPU cache,
// runtime/executor/executor_settings_base.h:54-66), an int8 cache any of the three. The matrix cores take
// the queries in the cache's operand type, so float32 queries are rounded to it here (to nearest even), once
// per call; the output is written in the io type from the float32 accumulators.
template <int KV, int IO, int D>
__device__ __forceinline__ void stage_q(u4* sm_q, const DecodeArgs& a, const typename IoT<IO>::type* q_rows, int kvh,
                                        int seq, int layer, int lane) {
  using io_t = typename IoT<IO>::type;
  constexpr int EPC = KvT<KV>::EPC;
  constexpr int NQ = KV == kF32 ? D / 16 : D / 32;
  const int n = lane & 15, g = lane >> 4;
  const bool live = n < a.group;
  const io_t* qrow = q_rows + (live ? n : 0) * D;
#pragma unroll
  for (int step = 0; step < NQ; ++step) {
    u4 w;
    if constexpr (KV == kI8) {
      const float* ks = a.scales + a.geom.scale_offset(layer, seq, 0, kvh);
      const int d0 = (4 * (step >> 1) + g) * EPC + 8 * (step & 1);
      const Q8 x = load_q8<IO>(qrow + d0);
      const f4 s0 = *reinterpret_cast<const f4*>(ks + d0), s1 = *reinterpret_cast<const f4*>(ks + d0 + 4);
      const f4 y0 = x.lo * s0, y1 = x.hi * s1;
      const h8 o = {(_Float16)y0[0], (_Float16)y0[1], (_Float16)y0[2], (_Float16)y0[3],
                    (_Float16)y1[0], (_Float16)y1[1], (_Float16)y1[2], (_Float16)y1[3]};
      w = bit_cast<u4>(o);
    } else if constexpr (KV == IO) {
      w = *reinterpret_cast<const u4*>(qrow + (4 * step + g) * EPC);
    } else {
      static_assert(IO == kF32 && (KV == kF16 || KV == kBF16), "float32 activations over a 16-bit cache");
      const Q8 x = load_q8<IO>(qrow + (4 * step + g) * EPC);
      if constexpr (KV == kF16) {
        const h8 o = {(_Float16)x.lo[0], (_Float16)x.lo[1], (_Float16)x.lo[2], (_Float16)x.lo[3],
                      (_Float16)x.hi[0], (_Float16)x.hi[1], (_Float16)x.hi[2], (_Float16)x.hi[3]};
        w = bit_cast<u4>(o);
      } else {
        const b8 o = {(__bf16)x.lo[0], (__bf16)x.lo[1], (__bf16)x.lo[2], (__bf16)x.lo[3],
                      (__bf16)x.hi[0], (__bf16)x.hi[1], (__bf16)x.hi[2], (__bf16)x.hi[3]};
        w = bit_cast<u4>(o);
      }
    }
    sm_q[step * 64 + lane] = live ? w : u4{0, 0, 0, 0};
  }
}

// S^T tiles of one block: s[T][i] is the raw score of token 16*T + 4*g + i
// against head n. sm_q[step * 64 + qi] is this lane's Q operand of a step; each
// is read once and used for every tile of the block.
template <int KV, int D>
__device__ __forceinline__ void qk_block(const u4 (&kreg)[D / 16], const u4* sm_q, int qi,
                                         f4 (&s)[KvT<KV>::VB / 16]) {
  constexpr int NT = KvT<KV>::VB / 16;
  constexpr int KPT = (D / 16) / NT;  // K loads per 16-token tile
#pragma unroll
  for (int T = 0; T < NT; ++T) s[T] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < KPT; ++j) {
    if constexpr (KV == kF16) {
      const h8 qv = bit_cast<h8>(sm_q[j * 64 + qi]);
#pragma unroll
      for (int T = 0; T < NT; ++T) s[T] = mfma16_f16(bit_cast<h8>(kreg[T * KPT + j]), qv, s[T]);
    } else if constexpr (KV == kBF16) {
      const b8 qv = bit_cast<b8>(sm_q[j * 64 + qi]);
#pragma unroll
      for (int T = 0; T < NT; ++T) s[T] = mfma16_bf16(bit_cast<b8>(kreg[T * KPT + j]), qv, s[T]);
    } else if constexpr (KV == kF32) {
      const f4 qf = bit_cast<f4>(sm_q[j * 64 + qi]);
#pragma unroll
      for (int T = 0; T < NT; ++T) {
        const f4 kf = bit_cast<f4>(kreg[T * KPT + j]);
#pragma unroll
        for (int e = 0; e < 4; ++e) s[T] = mfma16_f32(kf[e], qf[e], s[T]);
      }
    } else {
      const h8 q0 = bit_cast<h8>(sm_q[(2 * j) * 64 + qi]), q1 = bit_cast<h8>(sm_q[(2 * j + 1) * 64 + qi]);
#pragma unroll
      for (int T = 0; T < NT; ++T) {
        h8 lo, hi;
        cvt_i8x16_to_h8x2(kreg[T * KPT + j], lo, hi);
        s[T] = mfma16_f16(lo, q0, s[T]);
        s[T] = mfma16_f16(hi, q1, s[T]);
      }
    }
  }
}

// O^T += V^T . P^T for one block; p[T][i] pairs with token 16*T + 4*g + i.
template <int KV, int D>
__device__ __forceinline__ void pv_block(const u4 (&vreg)[D / 16], const f4 (&p)[KvT<KV>::VB / 16], f4 (&acc)[D / 16]) {
  if constexpr (KV == kF16 || KV == kBF16) {
    // (the V planes of a bfloat16 cache hold IEEE half values, attn_params.h: both run on the fp16 MFMA)
    h8 pp;
#pragma unroll
    for (int e = 0; e < 4; ++e) { pp[e] = (_Float16)p[0][e]; pp[4 + e] = (_Float16)p[1][e]; }
#pragma unroll
    for (int db = 0; db < D / 16; ++db) acc[db] = mfma16_f16(bit_cast<h8>(vreg[db]), pp, acc[db]);
  } else if constexpr (KV == kF32) {
#pragma unroll
    for (int db = 0; db < D / 16; ++db) {
      const f4 vf = bit_cast<f4>(vreg[db]);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[db] = mfma16_f32(vf[e], p[0][e], acc[db]);
    }
  } else {
    h8 p01, p23;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      p01[e] = (_Float16)p[0][e]; p01[4 + e] = (_Float16)p[1][e];
      p23[e] = (_Float16)p[2][e]; p23[4 + e] = (_Float16)p[3][e];
    }
#pragma unroll
    for (int db = 0; db < D / 16; ++db) {
      h8 lo, hi;
      cvt_i8x16_to_h8x2(vreg[db], lo, hi);
      acc[db] = mfma16_f16(lo, p01, acc[db]);
      acc[db] = mfma16_f16(hi, p23, acc[db]);
    }
  }
}

// One wave's share of a partition: blocks first, first + step, ... < blk_end of
// the K / V planes behind krsrc / vrsrc, through the online softmax. Leaves the
// reference max (exp2 domain), this lane's share of the sum (lane (n, g): head n,
// tokens 4 g .. 4 g + 3 of every 16) and the unnormalised accumulators (channels
// 16 * db + 4 * g .. + 3 of head n). Keys outside [vlo, p_hi) are masked.
// The caller has requested block `first` into kreg / vreg (request_first_block) and left the Q
// operands in sm_q while those loads were under way.
// patch_blk: a block one of whose rows is not in the cache yet (-1: none); patch(kreg, vreg) puts that
// row into the block's registers once they are loaded.
template <int D>
__device__ __forceinline__ void request_first_block(u4 (&kreg)[D / 16], u4 (&vreg)[D / 16], __amdgpu_buffer_rsrc_t krsrc,
                                                    __amdgpu_buffer_rsrc_t vrsrc, bool streams, int first, int lane) {
  // `first` is wave-uniform (the caller has taken it through readfirstlane) and is the very value the block
  // loop starts from. A wave that streams nothing gets zeros, so that the registers hold defined values on
  // every path.
  if (streams) {
    load_plane_block<D>(kreg, krsrc, first * (64 * D), lane * 16);
    load_plane_block<D>(vreg, vrsrc, first * (64 * D), lane * 16);
  } else {
    const u4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < D / 16; ++i) kreg[i] = zero;
#pragma unroll
    for (int i = 0; i < D / 16; ++i) vreg[i] = zero;
  }
}

template <int KV, int IO, int D, class Patch>
__device__ __forceinline__ void stream_blocks(const DecodeArgs& a, __amdgpu_buffer_rsrc_t krsrc,
                                              __amdgpu_buffer_rsrc_t vrsrc, u4 (&kreg)[D / 16], u4 (&vreg)[D / 16],
                                              int first, int blk_end, int step, int vlo, int p_hi, const u4* sm_q,
                                              int patch_blk, Patch&& patch, int lane, float& m_run, float& l_run,
                                              f4 (&acc)[D / 16]) {
  constexpr int VB = KvT<KV>::VB, NT = VB / 16, NL = D / 16;
  constexpr int kBlockBytes = 64 * D;
  const int g = lane >> 4;
  const int lane_off = lane * 16;
  // Rolling prefetch: the K registers are refilled with the next block as soon
  // as the QK^T product has consumed them, the V registers right after P.V, so
  // 16 to 32 KiB per wave are in flight while it computes.
  int blk = first;  // (wave-uniform: the caller's readfirstlane)

  m_run = -INFINITY;
  l_run = 0.f;
#pragma unroll
  for (int i = 0; i < NL; ++i) acc[i] = f4{0.f, 0.f, 0.f, 0.f};
  const float sc = a.scale, softcap = a.softcap;

  while (blk < blk_end) {
    // The index is made opaque so the Q reads stay inside the loop: hoisted
    // they would occupy 32 to 64 registers for the whole kernel.
    int qi = lane;
    asm volatile("" : "+v"(qi));
    if (blk == patch_blk) patch(kreg, vreg);
    f4 s[NT];
    qk_block<KV, D>(kreg, sm_q, qi, s);
    const int nxt = blk + step;
    if (nxt < blk_end) load_plane_block<D>(kreg, krsrc, nxt * kBlockBytes, lane_off);

    // scores in the exp2 domain; soft-capping and the range mask are uniform
    // branches taken only by the layers / boundary blocks that need them
    if (softcap > 0.f) {
      const float inv_cap = sc / softcap, cap2 = softcap * kLog2e;
#pragma unroll
      for (int T = 0; T < NT; ++T)
#pragma unroll
        for (int i = 0; i < 4; ++i) s[T][i] = cap2 * fast_tanh(s[T][i] * inv_cap);
    } else {
      const float sc2 = sc * kLog2e;
#pragma unroll
      for (int T = 0; T < NT; ++T) s[T] *= sc2;
    }
    if (blk * VB < vlo || (blk + 1) * VB > p_hi) {
      const int tok0 = blk * VB + 4 * g;
#pragma unroll
      for (int T = 0; T < NT; ++T)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int tok = tok0 + 16 * T + i;
          s[T][i] = (tok >= vlo && tok < p_hi) ? s[T][i] : -INFINITY;
        }
    }
    float bm = -INFINITY;
#pragma unroll
    for (int T = 0; T < NT; ++T)
#pragma unroll
      for (int i = 0; i < 4; ++i) bm = fmaxf(bm, s[T][i]);
    bm = wave_xor_max(bm, 16);
    bm = wave_xor_max(bm, 32);
    const float m_new = fmaxf(m_run, bm);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_use);
    float lsum = 0.f;
#pragma unroll
    for (int T = 0; T < NT; ++T) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pv = fast_exp2(s[T][i] - m_use);
        s[T][i] = pv;
        lsum += pv;
      }
    }
    l_run = l_run * alpha + lsum;
    m_run = m_new;
#pragma unroll
    for (int i = 0; i < NL; ++i) acc[i] *= alpha;
    pv_block<KV, D>(vreg, s, acc);
    if (nxt < blk_end) load_plane_block<D>(vreg, vrsrc, nxt * kBlockBytes, lane_off);
    blk = nxt;
  }

  // The four lanes (g = 0..3) of a head each summed their own tokens.
}

// Log-sum-exp merge of the split-KV partials: grid (query head, item), one
// thread per channel. A separate launch because partials written by workgroups
// on other XCDs are only guaranteed visible across a kernel boundary; an
// in-kernel "last arrival merges" needs an L2 write-back and invalidate per
// workgroup, which measured several times slower than this launch.
// Grid (query head, sequence, layer). INL and the argument loads in front of the
// first read of the partials: as in decode_attn_kernel.
template <int KV, int IO, int D, bool INL>
__global__ void __launch_bounds__(D) decode_merge_kernel(const DecodeArgs a) {
  using io_t = typename IoT<IO>::type;
  __shared__ float sm_m[kMaxDecodeSplits], sm_l[kMaxDecodeSplits];
  const int head = blockIdx.x, j = blockIdx.y, li = blockIdx.z, d = threadIdx.x;  // j: dispatch slot of the sequence
  int batch = a.batch, layer_begin = a.layer_begin, num_splits = a.num_splits, max_kv_len = a.max_kv_len, hq = a.hq;
  const float* ws_ml = a.ws_ml;
  const float* ws_acc = a.ws_acc;
  int kv_len = 0, window = 0, b = j;
  if constexpr (INL) {
    kv_len = a.inline_lens[j];
    b = a.inline_row[j];
    window = a.inline_window[li];
  }
  asm volatile("" : "+s"(batch), "+s"(layer_begin), "+s"(num_splits), "+s"(max_kv_len), "+s"(hq), "+s"(ws_ml),
               "+s"(ws_acc), "+s"(kv_len), "+s"(window), "+s"(b));
  if constexpr (!INL) {
    if (a.inline_items) b = a.inline_row[j];
    else if (a.rows) b = a.rows[j];
    b = __builtin_amdgcn_readfirstlane(b);
  }
  const int item = li * batch + b;
  const int layer = layer_begin + li;
  if constexpr (!INL) {
    kv_len = a.inline_items ? a.inline_lens[j] : a.kv_lens[j];
    window = a.n_layers <= kInlineLayers ? a.inline_window[li] : a.layer_window[layer];
    kv_len = __builtin_amdgcn_readfirstlane(kv_len);
    window = __builtin_amdgcn_readfirstlane(window);
  }
  int vlo, start;
  decode_visible_range(kv_len, window, &vlo, &start);
  const int per = decode_partition_tokens(max_kv_len, window, num_splits);
  int nparts = (kv_len - start + per - 1) / per;
  nparts = nparts < num_splits ? nparts : num_splits;
  const int64_t slot0 = ((int64_t)item * hq + head) * num_splits;
  // one round trip for all (max, sum) pairs, then the weights come from LDS
  for (int s = d; s < nparts; s += D) {
    const float2 ml = *reinterpret_cast<const float2*>(ws_ml + (slot0 + s) * 2);
    sm_m[s] = ml.x;
    sm_l[s] = ml.y;
  }
  __syncthreads();
  float M = -INFINITY;
  for (int s = 0; s < nparts; ++s) M = fmaxf(M, sm_m[s]);
  const float m_use = (M == -INFINITY) ? 0.f : M;
  float A = 0.f, L = 0.f;
  const float* accp = ws_acc + slot0 * D + d;
  int s = 0;
  for (; s + 8 <= nparts; s += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = accp[(int64_t)(s + u) * D];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const float wgt = fast_exp2(sm_m[s + u] - m_use);
      A += wgt * v[u];
      L += wgt * sm_l[s + u];
    }
  }
  for (; s < nparts; ++s) {
    const float wgt = fast_exp2(sm_m[s] - m_use);
    A += wgt * accp[(int64_t)s * D];
    L += wgt * sm_l[s];
  }
  float o = L > 0.f ? A / L : 0.f;
  if constexpr (KV == kI8) {
    const int seq = a.inline_items ? a.inline_seq[j] : (a.seq_ids ? a.seq_ids[j] : j);
    o *= a.scales[a.geom.scale_offset(layer, seq, 1, head / a.group) + d];
  }
  reinterpret_cast<io_t*>(a.out)[((int64_t)item * hq + head) * D + d] = (io_t)o;
}

// INL: lengths, sequence ids and windows travel in the argument block (the host
// knows: a.inline_items and n_layers <= kInlineLayers). Then everything in front
// of the first loads is one round of scalar loads at addresses that depend on
// the block index only. (With both sources behind one `cond ? a.inline_x[b] :
// a.x[b]` the compiler selects a pointer and issues vector loads, one after the
// other, and a wave spent 2 to 4 us before its first K/V load.)
//
// PRE (with INL, one layer): the kernel runs the step before attention for the one new token of its
// sequence itself (row t = kv_len - 1): every workgroup norms and rotates the query rows of its KV
// head into LDS; the workgroup whose partition ends at kv_len also norms / rotates the key and value
// rows, stores them into the cache planes for later calls, and keeps them in LDS in the planes' element
// format: the wave that streams the block of row t loads it like any other block (the row's bytes are
// stale, or change under the load) and overwrites the row's bytes in its registers from LDS before the
// block is used. The MFMAs see the operands that a load after pre_attention_kernel would have
// delivered, so the results are the same bit for bit, and nothing waits for a store. No other
// workgroup reads that block (partitions are whole blocks). Same arithmetic, lane for lane, as
// pre_attention_kernel.
// The rows are serial work for a wave (a norm with its cross-lane sums per row, two full-precision
// sincosf per lane), so a PRE workgroup always has four waves to share them; those beyond NW leave
// after the rows, and the attention itself runs on NW waves exactly as without PRE.
template <int NW, bool PRE>
constexpr int decode_wg_waves() { return PRE && NW < 4 ? 4 : NW; }

template <int KV, int IO, int D, int NW, bool INL, bool PRE>
__global__ void __launch_bounds__((decode_wg_waves<NW, PRE>()) * 64, 2) decode_attn_kernel(const DecodeArgs a) {
  static_assert(!PRE || INL, "the fused step needs the items in the argument block");
  constexpr int NWP = decode_wg_waves<NW, PRE>();  // waves of the workgroup; the first NW do the attention
  constexpr int VB = KvT<KV>::VB, NL = D / 16;
  constexpr int NQ = KV == kF32 ? D / 16 : D / 32;
  extern __shared__ float smem[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: block addresses stay scalar
  const int n = lane & 15, g = lane >> 4;
  // Grid (layer, sequence slot, partition x KV head): partitions vary slowest in
  // dispatch order, so with ragged lengths the empty ones (sequences shorter than
  // the longest) come last instead of between the full ones; inside a partition
  // index the host has put the longest sequences first (all their layers, then the
  // next sequence), so that the short ones fill the end of the launch.
  const int li = blockIdx.x, j = blockIdx.y;
  // What the code in front of the first K/V loads needs from the argument block is
  // read here in one go (left alone, the compiler sinks each scalar load behind the
  // branch that needs it: four dependent round trips instead of one).
  int hkv = a.geom.hkv, batch = a.batch, layer_begin = a.layer_begin, max_seqs = a.geom.max_seqs;
  int num_splits = a.num_splits, max_kv_len = a.max_kv_len;
  int64_t plane_bytes = a.geom.plane_bytes;
  const uint8_t* cache = a.cache;
  int seq = 0, kv_len = 0, window = 0, b = j;
  if constexpr (INL) {  // (addresses that depend on the block index only: the same round)
    seq = a.inline_seq[j];
    kv_len = a.inline_lens[j];
    b = a.inline_row[j];
    window = a.inline_window[li];
  }
  asm volatile("" : "+s"(hkv), "+s"(batch), "+s"(layer_begin), "+s"(max_seqs), "+s"(num_splits), "+s"(max_kv_len),
               "+s"(plane_bytes), "+s"(cache), "+s"(seq), "+s"(kv_len), "+s"(window), "+s"(b));
  const int split = blockIdx.z / hkv, kvh = blockIdx.z - split * hkv;
  const int layer = layer_begin + li;
  if constexpr (!INL) {
    seq = a.inline_items ? a.inline_seq[j] : (a.seq_ids ? a.seq_ids[j] : j);
    kv_len = a.inline_items ? a.inline_lens[j] : a.kv_lens[j];
    if (a.inline_items) b = a.inline_row[j];
    else if (a.rows) b = a.rows[j];
    window = a.n_layers <= kInlineLayers ? a.inline_window[li] : a.layer_window[layer];
  }
  b = __builtin_amdgcn_readfirstlane(b);
  const int item = li * batch + b;  // row of q, out and the partials
  seq = __builtin_amdgcn_readfirstlane(seq);
  kv_len = __builtin_amdgcn_readfirstlane(kv_len);
  window = __builtin_amdgcn_readfirstlane(window);
  int vlo, start;
  decode_visible_range(kv_len, window, &vlo, &start);
  const int per = decode_partition_tokens(max_kv_len, window, num_splits);
  const int p_lo = start + split * per;
  const int p_hi = min(kv_len, p_lo + per);
  if (p_lo >= p_hi) return;  // empty partition: uniform over the workgroup

  const uint8_t* kplane = cache + ((((int64_t)layer * max_seqs + seq) * hkv + kvh) * 2) * plane_bytes;  // geom.plane_offset
  const __amdgpu_buffer_rsrc_t krsrc = plane_resource(kplane, plane_bytes);
  const __amdgpu_buffer_rsrc_t vrsrc = plane_resource(kplane + plane_bytes, plane_bytes);
  const int blk_end = (p_hi + VB - 1) / VB;

  u4* sm_q = reinterpret_cast<u4*>(smem) + wave * (NQ * 64);
  float m_run, l_run;
  f4 acc[NL];
  using io_t = typename IoT<IO>::type;
  // The first block's loads go out before anything else (a helper wave of a PRE workgroup streams nothing).
  u4 kreg[NL], vreg[NL];
  const int first_blk = __builtin_amdgcn_readfirstlane(p_lo / VB + wave);
  request_first_block<D>(kreg, vreg, krsrc, vrsrc, wave < NW && first_blk < blk_end, first_blk, lane);
  if constexpr (PRE) {
    static_assert(D == kRowD, "row helpers are written for head_dim 256");
    constexpr int ESZ = KV == kF32 ? 4 : (KV == kI8 ? 1 : 2);
    constexpr int NT = VB / 16, KPT = NL / NT;
    const int G = a.group;
    // behind the merge area: [G][D] query rows (io type), then the new key and value row as the planes hold them
    io_t* sm_rows = reinterpret_cast<io_t*>(smem + NW * NQ * 64 * 4 + NW * G * (D + 2));
    uint8_t* sm_krow = reinterpret_cast<uint8_t*>(sm_rows + G * D);
    uint8_t* sm_vrow = sm_krow + D * ESZ;
    const int t = kv_len - 1;
    const bool owns_row = p_hi == kv_len;  // exactly one partition per sequence and KV head
    // The rows: one copy of the code, at kernel scope, run by every wave of the workgroup (attention waves
    // and helper waves alike) and closed by the workgroup's one barrier, which all NWP waves reach exactly
    // once.
    {
      const int nrows = G + (owns_row ? 2 : 0);  // G query rows, then the key and the value row
      constexpr int kMaxRows = (kMaxGroup + 2 + NWP - 1) / NWP;
      const int d0 = 2 * lane, d1 = D / 2 + 2 * lane;
      float xs[kMaxRows][4];
      // every row of this wave in flight before the first is waited for
#pragma unroll
      for (int r = 0; r < kMaxRows; ++r) {
        const int row = wave + r * NWP;
        if (row < nrows) {
          const void* src = row < G ? a.pre_q : (row == G ? a.pre_k : a.pre_v);
          const int64_t base = row < G ? ((int64_t)b * a.hq + kvh * G + row) * D : ((int64_t)b * hkv + kvh) * D;
          load_pair<IO>(src, base + d0, xs[r][0], xs[r][1]);
          load_pair<IO>(src, base + d1, xs[r][2], xs[r][3]);
        }
      }
      const RowAngles ang = row_angles(a.pre_rope ? a.pre_constants : nullptr, t, lane);
#pragma unroll
      for (int r = 0; r < kMaxRows; ++r) {
        const int row = wave + r * NWP;
        if (row < nrows) {
          const int kind = row < G ? 0 : (row == G ? 1 : 2);
          const bool norm = kind == 0 ? a.pre_norm_q != 0 : (kind == 1 ? a.pre_norm_k != 0 : a.pre_norm_v != 0);
          transform_row(xs[r], norm, row_weights(a.pre_constants, kind, a.pre_q_scaled != 0, a.pre_k_scaled != 0),
                        a.pre_weight_offset, a.pre_eps, a.pre_rope != 0 && kind != 2, ang, lane);
          if (kind == 0) {
            uint8_t* dst = reinterpret_cast<uint8_t*>(sm_rows + row * D);
            store_pair<IO>(dst + d0 * sizeof(io_t), xs[r][0], xs[r][1]);
            store_pair<IO>(dst + d1 * sizeof(io_t), xs[r][2], xs[r][3]);
          } else {
            const int is_v = kind - 1;
            uint8_t* plane = const_cast<uint8_t*>(kplane) + is_v * plane_bytes;
            const float* sc = KV == kI8 ? a.scales + a.geom.scale_offset(layer, seq, is_v, kvh) : nullptr;
            store_cache_row<KV, false>(plane, sc, is_v, t, xs[r], lane);
            store_cache_row<KV, true>(is_v ? sm_vrow : sm_krow, sc, is_v, t, xs[r], lane);
          }
        }
      }
    }
    __syncthreads();
    if (wave >= NW) return;  // a helper wave: its share of the rows, nothing else
    stage_q<KV, IO, D>(sm_q, a, sm_rows, kvh, seq, layer, lane);
    // Row t in the registers of its block. K: chunk c of the row is the 16 bytes of lane (t % 16, g) in load
    // (t % VB) / 16 * KPT + j with c = 4 j + g. V: element d of the row sits in lane (d % 16, (t % 16) / 4), load
    // d / 16, at element slot 4 * ((t % VB) / 16) + t % 4 of the lane's 16 bytes.
    auto patch = [&](u4 (&kr)[NL], u4 (&vr)[NL]) __attribute__((always_inline)) {
      const int tb = t % VB;
      const int tile = tb >> 4;
      const bool k_lane = (lane & 15) == (tb & 15);
#pragma unroll
      for (int T = 0; T < NT; ++T) {
        if (T == tile) {
#pragma unroll
          for (int j = 0; j < KPT; ++j) {
            const u4 fresh = *reinterpret_cast<const u4*>(sm_krow + (4 * j + g) * 16);
            kr[T * KPT + j] = k_lane ? fresh : kr[T * KPT + j];
          }
        }
      }
      const int byte0 = (4 * tile + (tb & 3)) * ESZ;  // of the lane's 16 bytes
      const unsigned in_word = ESZ == 4 ? 0xffffffffu : ((ESZ == 2 ? 0xffffu : 0xffu) << (8 * (byte0 & 3)));
      const bool v_lane = g == ((tb & 15) >> 2);
      // The row's element slot in the lane's 16 bytes, as whole-vector operations on purpose. Written element
      // by element (vr[db][w] = ... for one w) this compiler's register allocator gave registers of the patched
      // group to the softmax as temporaries before the matrix instruction that reads the group: a sixteenth of
      // the outputs came out wrong (first seen as "wrong unless a lambda is forced inline": any change of the
      // code's shape moved it). check_decode_kernels.py looks for that pattern in every build.
      u4 mask;
#pragma unroll
      for (int w = 0; w < 4; ++w) mask[w] = (v_lane && w == (byte0 >> 2)) ? in_word : 0u;
      const u4 keep = ~mask;
#pragma unroll
      for (int db = 0; db < NL; ++db) {
        const uint8_t* src = sm_vrow + (16 * db + n) * ESZ;
        unsigned e;
        if constexpr (ESZ == 4) e = *reinterpret_cast<const unsigned*>(src);
        else if constexpr (ESZ == 2) e = *reinterpret_cast<const uint16_t*>(src);
        else e = *src;
        e <<= 8 * (byte0 & 3);
        const u4 ev = {e, e, e, e};
        vr[db] = (vr[db] & keep) | (ev & mask);
      }
    };
    stream_blocks<KV, IO, D>(a, krsrc, vrsrc, kreg, vreg, first_blk, blk_end, NW, vlo, p_hi, sm_q, owns_row ? t / VB : -1,
                             patch, lane, m_run, l_run, acc);
  } else {
    const io_t* q_rows = reinterpret_cast<const io_t*>(a.q) + ((int64_t)item * a.hq + kvh * a.group) * D;
    stage_q<KV, IO, D>(sm_q, a, q_rows, kvh, seq, layer, lane);
    auto patch = [](u4 (&)[NL], u4 (&)[NL]) {};
    stream_blocks<KV, IO, D>(a, krsrc, vrsrc, kreg, vreg, first_blk, blk_end, NW, vlo, p_hi, sm_q, -1, patch, lane, m_run,
                             l_run, acc);
  }
  float l_tot = wave_xor_add(l_run, 16);
  l_tot = wave_xor_add(l_tot, 32);

  const int G = a.group;
  if constexpr (NW == 1) {
    // One wave: nothing to merge. Lane (n, g) holds channels 16 * db + 4 * g .. + 3 of head n.
    if (n < G) {
      const int head = kvh * G + n;
      if (a.num_splits == 1) {
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        io_t* orow = reinterpret_cast<io_t*>(a.out) + ((int64_t)item * a.hq + head) * D + 4 * g;
        const float* vs = nullptr;
        if constexpr (KV == kI8) vs = a.scales + a.geom.scale_offset(layer, seq, 1, kvh) + 4 * g;
#pragma unroll
        for (int db = 0; db < NL; ++db) {
          io_t o[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float x = acc[db][e] * inv;
            if constexpr (KV == kI8) x *= vs[16 * db + e];
            o[e] = (io_t)x;
          }
          if constexpr (sizeof(io_t) == 4) *reinterpret_cast<u4*>(orow + 16 * db) = *reinterpret_cast<const u4*>(o);
          else *reinterpret_cast<u2*>(orow + 16 * db) = *reinterpret_cast<const u2*>(o);
        }
      } else {
        const int64_t slot = ((int64_t)item * a.hq + head) * a.num_splits + split;
        float* prow = a.ws_acc + slot * D + 4 * g;
#pragma unroll
        for (int db = 0; db < NL; ++db) *reinterpret_cast<f4*>(prow + 16 * db) = acc[db];
        if (g == 0) *reinterpret_cast<float2*>(a.ws_ml + slot * 2) = float2{m_run, l_tot};
      }
    }
    return;
  }
  // Merge the waves through LDS: [NW][group][D] accumulators, then max, sum.
  float* sm_acc = smem + NW * NQ * 64 * 4;  // behind the waves' Q slices
  float* sm_m = sm_acc + NW * G * D;
  float* sm_l = sm_m + NW * G;
  if (n < G) {
    float* dst = sm_acc + (wave * G + n) * D + 4 * g;
#pragma unroll
    for (int db = 0; db < NL; ++db) *reinterpret_cast<f4*>(dst + 16 * db) = acc[db];
    if (g == 0) {
      sm_m[wave * G + n] = m_run;
      sm_l[wave * G + n] = l_tot;
    }
  }
  __syncthreads();

  for (int e = threadIdx.x; e < G * D; e += NW * 64) {
    const int hn = e / D, d = e - hn * D;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, sm_m[w * G + hn]);
    const float m_use = (M == -INFINITY) ? 0.f : M;
    float A = 0.f, L = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float wgt = fast_exp2(sm_m[w * G + hn] - m_use);
      A += wgt * sm_acc[(w * G + hn) * D + d];
      L += wgt * sm_l[w * G + hn];
    }
    const int head = kvh * G + hn;
    if (a.num_splits == 1) {
      float o = L > 0.f ? A / L : 0.f;
      if constexpr (KV == kI8) o *= a.scales[a.geom.scale_offset(layer, seq, 1, kvh) + d];
      reinterpret_cast<io_t*>(a.out)[((int64_t)item * a.hq + head) * D + d] = (io_t)o;
    } else {
      const int64_t slot = ((int64_t)item * a.hq + head) * a.num_splits + split;
      a.ws_acc[slot * D + d] = A;
      if (d == 0) {
        a.ws_ml[slot * 2] = M;
        a.ws_ml[slot * 2 + 1] = L;
      }
    }
  }
}

template <int KV, int IO, int D, int NW, bool INL, bool PRE = false>
hipError_t launch_inl(const DecodeArgs& a, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  const dim3 grid(a.n_layers, a.batch, a.num_splits * a.geom.hkv);
  constexpr int NQ = KV == kF32 ? D / 16 : D / 32;
  const size_t lds = (size_t)NW * NQ * 64 * 16 + (size_t)NW * a.group * (D + 2) * sizeof(float) +
                     (PRE ? (size_t)a.group * D * sizeof(typename IoT<IO>::type) + 2 * (size_t)D * a.geom.esize : 0);
  // ev0/ev1 are attached to the dispatch itself: they carry the kernel's own
  // begin and end timestamps, not the host-side launch latency around it.
  hipExtLaunchKernelGGL((decode_attn_kernel<KV, IO, D, NW, INL, PRE>), grid, dim3(decode_wg_waves<NW, PRE>() * 64), lds,
                        stream, ev0, ev1, 0, a);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess || a.num_splits == 1) return err;
  hipLaunchKernelGGL((decode_merge_kernel<KV, IO, D, INL>), dim3(a.hq, a.batch, a.n_layers), dim3(D), 0, stream, a);
  return hipGetLastError();
}

template <int KV, int IO, int D, int NW>
hipError_t launch_variant(const DecodeArgs& a, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  if (a.pre_q) {
    if (!a.inline_items || a.n_layers != 1) return hipErrorInvalidValue;
    return launch_inl<KV, IO, D, NW, true, true>(a, stream, ev0, ev1);
  }
  if (a.inline_items && a.n_layers <= kInlineLayers) return launch_inl<KV, IO, D, NW, true>(a, stream, ev0, ev1);
  return launch_inl<KV, IO, D, NW, false>(a, stream, ev0, ev1);
}

template <int KV, int IO, int D>
hipError_t launch_typed(const DecodeArgs& a, const DecodeTuning& t, hipStream_t s, hipEvent_t e0, hipEvent_t e1) {
  int waves = t.waves;
  if (waves == 0) {
    // Measured on MI355X (head_dim 256, 4096-token context): with several
    // workgroups per CU one wave each is as fast or faster (fewer LDS merges),
    // with less than one per CU more waves per workgroup hide the latency.
    const int wgs = a.n_layers * (a.rule_batch > 0 ? a.rule_batch : a.batch) * a.geom.hkv * a.num_splits;
    waves = wgs >= 768 ? 1 : wgs >= 256 ? 2 : 4;
    // ... and one wave when a partition is one or two key blocks: more waves
    // would only add to the merge (one layer of 1024 tokens in 64-token
    // partitions: 7.7 us instead of 8.7 us per call).
    constexpr int VB = KvT<KV>::VB;
    if (decode_partition_tokens(a.max_kv_len, 0, a.num_splits) <= 2 * VB) waves = 1;
    // ... and four waves for a big launch of whole sequences of unequal lengths: the wave slots of
    // the chip then hold a quarter of the workgroups at a time instead of all of them, and the short
    // sequences, dispatched last, fill in behind the long ones (16 layers x 64 sequences of 256 to
    // 4096 tokens: 6.5 instead of 6.1 TB/s; sequences of equal length lose 1 % and keep one wave).
    if (a.num_splits == 1 && wgs >= 1024 && a.min_kv_len * 4 < a.max_kv_len * 3) waves = 4;
  }
  if (waves == 1) return launch_variant<KV, IO, D, 1>(a, s, e0, e1);
  if (waves == 2) return launch_variant<KV, IO, D, 2>(a, s, e0, e1);
  return launch_variant<KV, IO, D, 4>(a, s, e0, e1);
}

}  // namespace

bool decode_supported(int kv_dtype, int io_dtype, int head_dim) {
  if (head_dim != 256) return false;
  if (io_dtype != kF32 && io_dtype != kF16 && io_dtype != kBF16) return false;
  if (kv_dtype == kI8) return true;                      // int8 cache: any activation type
  return kv_dtype == io_dtype || (io_dtype == kF32 && (kv_dtype == kF16 || kv_dtype == kBF16));
}

hipError_t launch_decode(const DecodeArgs& a, int kv_dtype, int io_dtype, const DecodeTuning& tuning,
                         hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  switch (kv_dtype * 4 + io_dtype) {
    case kF32 * 4 + kF32: return launch_typed<kF32, kF32, 256>(a, tuning, stream, ev0, ev1);
    case kF16 * 4 + kF16: return launch_typed<kF16, kF16, 256>(a, tuning, stream, ev0, ev1);
    case kF16 * 4 + kF32: return launch_typed<kF16, kF32, 256>(a, tuning, stream, ev0, ev1);
    case kBF16 * 4 + kBF16: return launch_typed<kBF16, kBF16, 256>(a, tuning, stream, ev0, ev1);
    case kBF16 * 4 + kF32: return launch_typed<kBF16, kF32, 256>(a, tuning, stream, ev0, ev1);
    case kI8 * 4 + kF16: return launch_typed<kI8, kF16, 256>(a, tuning, stream, ev0, ev1);
    case kI8 * 4 + kBF16: return launch_typed<kI8, kBF16, 256>(a, tuning, stream, ev0, ev1);
    case kI8 * 4 + kF32: return launch_typed<kI8, kF32, 256>(a, tuning, stream, ev0, ev1);
  }
  return hipErrorInvalidValue;
}

}  // namespace mi355
