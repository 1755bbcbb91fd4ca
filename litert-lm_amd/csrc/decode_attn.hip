// One-token decode attention over the KV cache (gfx950, wave64, MFMA).
//
// Grid: x = split-KV partition, y = KV head, z = (layer, sequence) item.
// A workgroup of NW waves streams the K and V rows of its partition exactly
// once. Each wave owns every NW-th block of VB tokens and, per block, issues
// 32 wave-wide 1 KiB streaming loads (16 of K, 16 of V at head_dim 256), the
// next block's loads before the current block's arithmetic. Scores are
// S^T = K . Q^T on the matrix cores with the (at most 16) query heads of the KV
// head in the column dimension, so each lane keeps the running max / sum of
// one query head; the probabilities leave the first MFMA already in the
// operand layout of the second (O^T = V^T . P^T). Waves are merged through
// LDS, partitions through a workspace and a small log-sum-exp merge kernel.
//
// Replaces the decode-time attention that the reference reaches through
// compiled_model_.Run("decode", ...)
// (runtime/executor/llm_litert_compiled_model_executor.cc:407,522).
#include <hip/hip_runtime.h>
#include <math.h>

#include "attn_params.h"
#include "kernels.h"
#include "mfma_util.h"

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

// K and V bytes of one block of VB tokens as they sit in a wave's registers.
template <int D>
struct BlockRegs {
  u4 k[D / 16];
  u4 v[D / 16];
};

template <int D>
__device__ __forceinline__ void load_block(BlockRegs<D>& r, const uint8_t* kblock, const uint8_t* vblock,
                                           int lane) {
  // A block is 64*D bytes in both planes, laid out so that load i of a wave is
  // bytes [i*1024, (i+1)*1024) of the block.
#pragma unroll
  for (int i = 0; i < D / 16; ++i) r.k[i] = load_stream16(kblock + i * 1024 + lane * 16);
#pragma unroll
  for (int i = 0; i < D / 16; ++i) r.v[i] = load_stream16(vblock + i * 1024 + lane * 16);
}

// Q^T as the B operand: lane (n = lane%16, g = lane/16) holds, for chunk step
// jj, the elements of head n that pair with K chunk 4*jj + g. Heads n >= group
// are zero columns.
template <int KV, int IO, int D>
__device__ __forceinline__ void load_q(u4 (&qreg)[KV == kF32 ? D / 16 : D / 32], const DecodeArgs& a,
                                       int item, int kvh, int seq, int layer, int lane) {
  using io_t = typename IoT<IO>::type;
  constexpr int EPC = KvT<KV>::EPC;
  const int n = lane & 15, g = lane >> 4;
  const bool live = n < a.group;
  const io_t* qrow = reinterpret_cast<const io_t*>(a.q) + ((int64_t)item * a.hq + kvh * a.group + (live ? n : 0)) * D;
  if constexpr (KV == kI8) {
    static_assert(IO == kF16, "int8 cache pairs with fp16 queries");
    const float* ks = a.scales + a.geom.scale_offset(layer, seq, 0, kvh);
#pragma unroll
    for (int jj = 0; jj < D / 64; ++jj) {
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int d0 = (4 * jj + g) * EPC + 8 * half;
        h8 qv = *reinterpret_cast<const h8*>(qrow + d0);
        h8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = live ? (_Float16)((float)qv[e] * ks[d0 + e]) : (_Float16)0;
        qreg[2 * jj + half] = bit_cast<u4>(o);
      }
    }
  } else {
    constexpr int NQ = KV == kF32 ? D / 16 : D / 32;
#pragma unroll
    for (int jj = 0; jj < NQ; ++jj) {
      u4 w = *reinterpret_cast<const u4*>(qrow + (4 * jj + g) * EPC);
      qreg[jj] = live ? w : u4{0, 0, 0, 0};
    }
  }
}

// S^T tiles of one block: s[T][i] is the raw score of token 16*T + 4*g + i
// against head n.
template <int KV, int D>
__device__ __forceinline__ void qk_block(const BlockRegs<D>& r, const u4 (&qreg)[KV == kF32 ? D / 16 : D / 32],
                                         f4 (&s)[KvT<KV>::VB / 16]) {
  constexpr int NT = KvT<KV>::VB / 16;
  constexpr int KPT = (D / 16) / NT;  // K loads per 16-token tile
#pragma unroll
  for (int T = 0; T < NT; ++T) {
    f4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < KPT; ++j) {
      const u4 kw = r.k[T * KPT + j];
      if constexpr (KV == kF16) {
        acc = mfma16_f16(bit_cast<h8>(kw), bit_cast<h8>(qreg[j]), acc);
      } else if constexpr (KV == kBF16) {
        acc = mfma16_bf16(bit_cast<b8>(kw), bit_cast<b8>(qreg[j]), acc);
      } else if constexpr (KV == kF32) {
        const f4 kf = bit_cast<f4>(kw), qf = bit_cast<f4>(qreg[j]);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = mfma16_f32(kf[e], qf[e], acc);
      } else {
        h8 lo, hi;
        cvt_i8x16_to_h8x2(kw, lo, hi);
        acc = mfma16_f16(lo, bit_cast<h8>(qreg[2 * j]), acc);
        acc = mfma16_f16(hi, bit_cast<h8>(qreg[2 * j + 1]), acc);
      }
    }
    s[T] = acc;
  }
}

// O^T += V^T . P^T for one block; p[T][i] pairs with token 16*T + 4*g + i.
template <int KV, int D>
__device__ __forceinline__ void pv_block(const BlockRegs<D>& r, const f4 (&p)[KvT<KV>::VB / 16], f4 (&acc)[D / 16]) {
  if constexpr (KV == kF16) {
    h8 pp;
#pragma unroll
    for (int e = 0; e < 4; ++e) { pp[e] = (_Float16)p[0][e]; pp[4 + e] = (_Float16)p[1][e]; }
#pragma unroll
    for (int db = 0; db < D / 16; ++db) acc[db] = mfma16_f16(bit_cast<h8>(r.v[db]), pp, acc[db]);
  } else if constexpr (KV == kBF16) {
    b8 pp;
#pragma unroll
    for (int e = 0; e < 4; ++e) { pp[e] = (__bf16)p[0][e]; pp[4 + e] = (__bf16)p[1][e]; }
#pragma unroll
    for (int db = 0; db < D / 16; ++db) acc[db] = mfma16_bf16(bit_cast<b8>(r.v[db]), pp, acc[db]);
  } else if constexpr (KV == kF32) {
#pragma unroll
    for (int db = 0; db < D / 16; ++db) {
      const f4 vf = bit_cast<f4>(r.v[db]);
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
      cvt_i8x16_to_h8x2(r.v[db], lo, hi);
      acc[db] = mfma16_f16(lo, p01, acc[db]);
      acc[db] = mfma16_f16(hi, p23, acc[db]);
    }
  }
}

template <int KV, int IO, int D, int NW, bool PIPE>
__global__ void __launch_bounds__(NW * 64) decode_attn_kernel(const DecodeArgs a) {
  constexpr int VB = KvT<KV>::VB, NT = VB / 16, NL = D / 16;
  constexpr int NQ = KV == kF32 ? D / 16 : D / 32;
  extern __shared__ float smem[];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int split = blockIdx.x, kvh = blockIdx.y, item = blockIdx.z;
  const int li = item / a.batch, b = item - li * a.batch;
  const int layer = a.layer_begin + li;
  const int seq = a.seq_ids ? a.seq_ids[b] : b;
  const int kv_len = a.kv_lens[b];
  const int window = a.layer_window[layer];
  int vlo, start;
  decode_visible_range(kv_len, window, &vlo, &start);
  const int per = decode_partition_tokens(a.max_kv_len, window, a.num_splits);
  const int p_lo = start + split * per;
  const int p_hi = min(kv_len, p_lo + per);
  if (p_lo >= p_hi) return;  // empty partition: uniform over the workgroup

  const uint8_t* kplane = a.cache + a.geom.plane_offset(layer, seq, kvh, 0);
  const uint8_t* vplane = kplane + a.geom.plane_bytes;
  constexpr int64_t kBlockBytes = 64 * D;

  u4 qreg[NQ];
  load_q<KV, IO, D>(qreg, a, item, kvh, seq, layer, lane);

  float m_run = -INFINITY, l_run = 0.f;
  f4 acc[NL];
#pragma unroll
  for (int i = 0; i < NL; ++i) acc[i] = f4{0.f, 0.f, 0.f, 0.f};

  const float sc = a.scale, softcap = a.softcap;
  const int blk_end = (p_hi + VB - 1) / VB;

  auto process = [&](const BlockRegs<D>& r, int blk) {
    f4 s[NT];
    qk_block<KV, D>(r, qreg, s);
    const int tok0 = blk * VB + 4 * g;
    float bm = -INFINITY;
#pragma unroll
    for (int T = 0; T < NT; ++T) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int tok = tok0 + 16 * T + i;
        float x = s[T][i] * sc;
        if (softcap > 0.f) x = softcap * tanhf(x / softcap);
        x *= kLog2e;
        x = (tok >= vlo && tok < p_hi) ? x : -INFINITY;
        s[T][i] = x;
        bm = fmaxf(bm, x);
      }
    }
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
#pragma unroll
    for (int i = 0; i < NL; ++i) acc[i] *= alpha;
    pv_block<KV, D>(r, s, acc);
    m_run = m_new;
  };

  int blk = p_lo / VB + wave;
  if constexpr (PIPE) {
    BlockRegs<D> ra, rb;
    if (blk < blk_end) load_block<D>(ra, kplane + blk * kBlockBytes, vplane + blk * kBlockBytes, lane);
    while (blk < blk_end) {
      if (blk + NW < blk_end)
        load_block<D>(rb, kplane + (blk + NW) * kBlockBytes, vplane + (blk + NW) * kBlockBytes, lane);
      process(ra, blk);
      blk += NW;
      if (blk >= blk_end) break;
      if (blk + NW < blk_end)
        load_block<D>(ra, kplane + (blk + NW) * kBlockBytes, vplane + (blk + NW) * kBlockBytes, lane);
      process(rb, blk);
      blk += NW;
    }
  } else {
    for (; blk < blk_end; blk += NW) {
      BlockRegs<D> r;
      load_block<D>(r, kplane + blk * kBlockBytes, vplane + blk * kBlockBytes, lane);
      process(r, blk);
    }
  }

  // The four lanes (g = 0..3) of a head each summed their own tokens.
  float l_tot = wave_xor_add(l_run, 16);
  l_tot = wave_xor_add(l_tot, 32);

  // Merge the waves through LDS: [NW][group][D] accumulators, then max, sum.
  const int G = a.group;
  float* sm_acc = smem;
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

  using io_t = typename IoT<IO>::type;
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

// Log-sum-exp merge of the split-KV partials: grid (query head, item), one
// thread per channel.
template <int KV, int IO, int D>
__global__ void __launch_bounds__(D) decode_merge_kernel(const DecodeArgs a) {
  using io_t = typename IoT<IO>::type;
  const int head = blockIdx.x, item = blockIdx.y, d = threadIdx.x;
  const int li = item / a.batch, b = item - li * a.batch;
  const int layer = a.layer_begin + li;
  const int kv_len = a.kv_lens[b];
  const int window = a.layer_window[layer];
  int vlo, start;
  decode_visible_range(kv_len, window, &vlo, &start);
  const int per = decode_partition_tokens(a.max_kv_len, window, a.num_splits);
  int nparts = (kv_len - start + per - 1) / per;
  nparts = nparts < a.num_splits ? nparts : a.num_splits;
  const int64_t slot0 = ((int64_t)item * a.hq + head) * a.num_splits;
  float M = -INFINITY;
  for (int s = 0; s < nparts; ++s) M = fmaxf(M, a.ws_ml[(slot0 + s) * 2]);
  const float m_use = (M == -INFINITY) ? 0.f : M;
  float A = 0.f, L = 0.f;
  for (int s = 0; s < nparts; ++s) {
    const float wgt = fast_exp2(a.ws_ml[(slot0 + s) * 2] - m_use);
    A += wgt * a.ws_acc[(slot0 + s) * D + d];
    L += wgt * a.ws_ml[(slot0 + s) * 2 + 1];
  }
  float o = L > 0.f ? A / L : 0.f;
  if constexpr (KV == kI8) {
    const int seq = a.seq_ids ? a.seq_ids[b] : b;
    o *= a.scales[a.geom.scale_offset(layer, seq, 1, head / a.group) + d];
  }
  reinterpret_cast<io_t*>(a.out)[((int64_t)item * a.hq + head) * D + d] = (io_t)o;
}

template <int KV, int IO, int D, int NW, bool PIPE>
hipError_t launch_variant(const DecodeArgs& a, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  const int items = a.n_layers * a.batch;
  const dim3 grid(a.num_splits, a.geom.hkv, items);
  const size_t lds = (size_t)NW * a.group * (D + 2) * sizeof(float);
  if (ev0) (void)hipEventRecord(ev0, stream);
  hipLaunchKernelGGL((decode_attn_kernel<KV, IO, D, NW, PIPE>), grid, dim3(NW * 64), lds, stream, a);
  if (ev1) (void)hipEventRecord(ev1, stream);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  if (a.num_splits > 1) {
    hipLaunchKernelGGL((decode_merge_kernel<KV, IO, D>), dim3(a.hq, items), dim3(D), 0, stream, a);
    err = hipGetLastError();
  }
  return err;
}

template <int KV, int IO, int D>
hipError_t launch_typed(const DecodeArgs& a, const DecodeTuning& t, hipStream_t s, hipEvent_t e0, hipEvent_t e1) {
  if (t.waves == 2) {
    return t.pipeline ? launch_variant<KV, IO, D, 2, true>(a, s, e0, e1)
                      : launch_variant<KV, IO, D, 2, false>(a, s, e0, e1);
  }
  return t.pipeline ? launch_variant<KV, IO, D, 4, true>(a, s, e0, e1)
                    : launch_variant<KV, IO, D, 4, false>(a, s, e0, e1);
}

}  // namespace

bool decode_supported(int kv_dtype, int io_dtype, int head_dim) {
  if (head_dim != 256) return false;
  if (kv_dtype == kI8) return io_dtype == kF16;
  return kv_dtype == io_dtype;
}

hipError_t launch_decode(const DecodeArgs& a, int kv_dtype, int io_dtype, const DecodeTuning& tuning,
                         hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  switch (kv_dtype) {
    case kF32: return launch_typed<kF32, kF32, 256>(a, tuning, stream, ev0, ev1);
    case kF16: return launch_typed<kF16, kF16, 256>(a, tuning, stream, ev0, ev1);
    case kBF16: return launch_typed<kBF16, kBF16, 256>(a, tuning, stream, ev0, ev1);
    case kI8: return launch_typed<kI8, kF16, 256>(a, tuning, stream, ev0, ev1);
  }
  return hipErrorInvalidValue;
}

}  // namespace mi355
