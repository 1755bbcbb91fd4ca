// Token sampling on the device (gfx950): top-k -> softmax with temperature ->
// top-p nucleus -> one draw.
//
// Replaces the reference's CPU arithmetic
//   TopKIndicies       runtime/components/sampling_cpu_util.cc:21-64
//   Softmax            runtime/components/sampling_cpu_util.cc:66-134
//   TopKTopPSampling   runtime/components/sampling_cpu_util.cc:136-233
// behind the C ABI shape of its GPU sampler plugin
// (runtime/components/sampler_factory.cc:34-46).
//
// One launch per call (sample_kernel). A row of ~262k logits is cut into up to
// 16 segments, one workgroup of 1024 threads each, so that one row already
// spreads over 16 CUs; a call of so many rows that this would make more than two
// workgroups per compute unit takes segments four times as long. A workgroup
// reads its segment once, 16 (or 64) logits per thread that stay in registers,
// all loads issued at once. Every thread takes the maximum of its logits; every
// wave reports the ceil(k/16)-th largest of its 64 maxima (DPP reductions); at
// least k logits of the segment reach the smallest of those 16 numbers, so only
// what reaches it - a few hundred candidates - is packed as (order-preserving
// key, index) words. Up to 256 of them go to a workspace as they are; more are
// ranked by counting in LDS (no sort) and the segment's k best go there.
// Segments for which that bound is too weak (more than 2048 candidates: long
// runs of equal values) or that hold fewer than k numbers fall back to a radix
// descent on the keys with LDS histograms (12 + 12 + 8 bits); exact ties at the
// k-th value are then taken in ascending index order.
// The workgroup that delivers the last segment of a row (a ticket per row) then
// thresholds and ranks the segments' candidates the same way and walks the k
// winners in the reference's op order (finish_row). Vocabularies beyond 16 x
// 16,384 entries in calls of few rows re-read their segments per pass and run
// as two launches (select_kernel, finish_kernel).
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <float.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>

#include "../../include/mi355_sampler.h"

namespace {

constexpr int kThreads = 1024;
constexpr int kWavesPerWg = kThreads / 64;
constexpr int kPerIter = kThreads * 4;  // logits per pass iteration: 4 consecutive ones per thread
constexpr int kUnroll = 4;              // iterations whose loads are in flight together
constexpr int kBins = 4096;
constexpr int kCap = 2048;              // candidates of one segment that fit in LDS for the sort
constexpr int kMaxK = MI355_SAMPLER_MAX_K;
constexpr int kMaxSegments = 16;
constexpr int kSlots = kMaxK;            // workspace words per segment; a zero word is an empty slot
constexpr int kMergeCap = kMaxSegments * kSlots;  // 4096 words of one row in finish_row
constexpr int kResident = 16;           // logits per thread of a short segment, which stay in registers between the passes
constexpr int kResidentWide = 64;       // ... and of a wide one (calls with many rows)
constexpr int kSegmentMin = kThreads * kResident;  // a segment is this long unless the row needs more than kMaxSegments

typedef unsigned long long u64;

struct SamplerArgs {
  const float* logits;    // [batch][vocab]
  const float* uniforms;  // [batch] or null: Philox draws
  int32_t* ids;           // [batch] or null
  float* scores;          // [batch] or null
  int32_t* topk_idx;      // [batch][k] or null
  float* topk_prob;       // [batch][k] or null
  u64* workspace;         // [batch][segments][kSlots] candidates, (key << 32) | ~index, 0 = empty
  uint32_t* tickets;      // [batch] segments of the row that are done; all zero between calls (sample_kernel)
#ifdef MI355_SAMPLER_TRACE
  unsigned long long* trace;  // [workgroups][16] (event << 56 | 100 MHz time)
#endif
  int32_t vocab, k, segments, seg_len;
  float p, temperature;
  uint32_t seed;
  uint64_t call_index;
};

// Larger float <=> larger key; -0 and +0 share a key; NaN sorts below everything.
__device__ __forceinline__ uint32_t key_of(float x) {
  if (x != x) return 0u;
  uint32_t u = __float_as_uint(x == 0.f ? 0.f : x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float logit_of(uint32_t key) {
  return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}
// Candidate word: descending order of the word = descending key, then ascending index.
__device__ __forceinline__ u64 pack(uint32_t key, int index) { return ((u64)key << 32) | (uint32_t)~(uint32_t)index; }
__device__ __forceinline__ int index_of(u64 c) { return (int)~(uint32_t)c; }

__device__ __forceinline__ void philox_round(uint32_t (&c)[4], uint32_t (&k)[2]) {
  const uint32_t lo0 = 0xD2511F53u * c[0], hi0 = __umulhi(0xD2511F53u, c[0]);
  const uint32_t lo1 = 0xCD9E8D57u * c[2], hi1 = __umulhi(0xCD9E8D57u, c[2]);
  const uint32_t n0 = hi1 ^ c[1] ^ k[0], n2 = hi0 ^ c[3] ^ k[1];
  c[0] = n0; c[1] = lo1; c[2] = n2; c[3] = lo0;
  k[0] += 0x9E3779B9u; k[1] += 0xBB67AE85u;
}
// Philox4x32-10 (Salmon et al., SC'11); the first output word.
__device__ __forceinline__ uint32_t philox_first_word(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                                      uint32_t k1) {
  uint32_t c[4] = {c0, c1, c2, c3}, k[2] = {k0, k1};
#pragma unroll
  for (int r = 0; r < 10; ++r) philox_round(c, k);
  return c[0];
}

// One pass over a segment: f(key, local index) for every logit, 4 consecutive
// ones per thread and iteration (so that waves, lanes and elements run in
// ascending index order), the loads of kUnroll iterations in flight together.
template <class F>
__device__ __forceinline__ void for_each_key(const float* seg, int len, bool vec_ok, int tid, F&& f) {
  int base = tid * 4;
  if (vec_ok) {
    for (; base + (kUnroll - 1) * kPerIter + 3 < len; base += kUnroll * kPerIter) {
      float4 x[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) x[u] = *reinterpret_cast<const float4*>(seg + base + u * kPerIter);
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int i = base + u * kPerIter;
        f(key_of(x[u].x), i); f(key_of(x[u].y), i + 1); f(key_of(x[u].z), i + 2); f(key_of(x[u].w), i + 3);
      }
    }
    for (; base + 3 < len; base += kPerIter) {
      const float4 x = *reinterpret_cast<const float4*>(seg + base);
      f(key_of(x.x), base); f(key_of(x.y), base + 1); f(key_of(x.z), base + 2); f(key_of(x.w), base + 3);
    }
  }
  for (; base < len; base += kPerIter)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (base + j < len) f(key_of(seg[base + j]), base + j);
}

// The bin, counted from the top, in which the cumulative count of hist[0..nbins)
// reaches `need` (1 <= need <= total): found = {bin, count above it, count in it}.
// Thread t owns bins 4t .. 4t+3; suffix sums over the threads above it. Ends
// with a barrier; found[] is valid for every thread afterwards.
__device__ __forceinline__ void find_bin(const uint32_t* hist, int nbins, uint32_t need, uint32_t* wave_sum,
                                         uint32_t* found, int tid) {
  const int lane = tid & 63, wave = tid >> 6;
  uint32_t h[4], s = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) { h[j] = 4 * tid + j < nbins ? hist[4 * tid + j] : 0u; s += h[j]; }
  uint32_t incl = s;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t v = __shfl_down(incl, off, 64);
    if (lane + off < 64) incl += v;
  }
  if (lane == 0) wave_sum[wave] = incl;
  __syncthreads();
  uint32_t cum = incl - s;
  for (int w = wave + 1; w < kWavesPerWg; ++w) cum += wave_sum[w];
#pragma unroll
  for (int j = 3; j >= 0; --j) {
    if (cum < need && cum + h[j] >= need) { found[0] = 4 * tid + j; found[1] = cum; found[2] = h[j]; }
    cum += h[j];
  }
  __syncthreads();
}

// Maximum over the wave, in every lane, by DPP row shifts and row broadcasts
// (no LDS round trips). 0 is the identity.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#define MI355_DPP_MAX(ctrl, row_mask) \
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, ctrl, row_mask, 0xf, false))
  MI355_DPP_MAX(0x111, 0xf);  // row_shr:1
  MI355_DPP_MAX(0x112, 0xf);  // row_shr:2
  MI355_DPP_MAX(0x114, 0xf);  // row_shr:4
  MI355_DPP_MAX(0x118, 0xf);  // row_shr:8   -> lane 15 of each row of 16 holds the row's maximum
  MI355_DPP_MAX(0x142, 0xa);  // row_bcast:15 into rows 1 and 3
  MI355_DPP_MAX(0x143, 0xc);  // row_bcast:31 into rows 2 and 3 -> lane 63 holds the wave's maximum
#undef MI355_DPP_MAX
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

// The same for floats; -inf is the identity, NaN never wins (v_max_f32 returns the other operand).
__device__ __forceinline__ float wave_max_f32(float v) {
  const int ninf = 0xff800000;
#define MI355_DPP_FMAX(ctrl, row_mask) \
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(ninf, __float_as_int(v), ctrl, row_mask, 0xf, false)))
  MI355_DPP_FMAX(0x111, 0xf);
  MI355_DPP_FMAX(0x112, 0xf);
  MI355_DPP_FMAX(0x114, 0xf);
  MI355_DPP_FMAX(0x118, 0xf);
  MI355_DPP_FMAX(0x142, 0xa);
  MI355_DPP_FMAX(0x143, 0xc);
#undef MI355_DPP_FMAX
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// A lower bound that at least k of the values v (one per thread, 0 = none) reach:
// each of the first `waves` waves reports the j-th largest of its 64 values,
// j = ceil(k / waves); at least waves * j >= k values reach the smallest of those
// numbers (0, a bound that everything reaches, if a wave holds fewer than j
// values). The values of the other waves are not looked at. One barrier.
__device__ __forceinline__ uint32_t lower_bound_of_kth(uint32_t v, int k, int waves, uint32_t* wave_val, int tid) {
  const int lane = tid & 63, wave = tid >> 6;
  const int j_th = (k + waves - 1) / waves;
  if (j_th > 16) {  // few waves: at most 64 * waves values anyway, and the rounds below cost more than they save
    __syncthreads();
    return 0;
  }
  if (wave < waves) {
    uint32_t m = 0;
    for (int r = 0; r < j_th && (r == 0 || m != 0); ++r) {
      m = wave_max_u32(v);
      const u64 holders = __ballot(v == m);
      if (lane == __ffsll((long long)holders) - 1) v = 0;  // drop one holder of the maximum
    }
    if (lane == 0) wave_val[wave] = m;
  }
  __syncthreads();
  uint32_t tau = wave_val[0];
  for (int w = 1; w < waves; ++w) tau = min(tau, wave_val[w]);
  return tau;
}

// Number of set bits of `mask` below this lane.
__device__ __forceinline__ uint32_t lanes_below(u64 mask) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// List slots for the values of a wave that pass a test: take[e] = ballot of value e
// passing. One atomic per wave on the list's length (an atomic per thread on one
// address is compiled to a loop over the lanes); returns the wave's first slot, value
// e of a passing lane goes to first + (set bits of take[0..e)) + lanes_below(take[e]).
template <int NV>
__device__ __forceinline__ uint32_t reserve_slots(const u64 (&take)[NV], uint32_t* length, int lane) {
  uint32_t total = 0;
#pragma unroll
  for (int e = 0; e < NV; ++e) total += (uint32_t)__popcll(take[e]);
  uint32_t first = 0;
  if (lane == 0 && total) first = atomicAdd(length, total);
  return (uint32_t)__builtin_amdgcn_readfirstlane((int)first);
}

// Workgroup barrier that orders LDS traffic only. __syncthreads() also waits for every outstanding global load
// of the wave, and the wide segments' loads are meant to stay in flight across the barrier below.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// The float version (-inf = none): used on the logits themselves.
__device__ __forceinline__ float lower_bound_of_kth_f32(float v, int k, float* wave_val, int tid) {
  const int lane = tid & 63, wave = tid >> 6;
  const int j_th = (k + kWavesPerWg - 1) / kWavesPerWg;
  float m = -INFINITY;
  for (int r = 0; r < j_th; ++r) {
    m = wave_max_f32(v);
    const u64 holders = __ballot(v == m);
    if (lane == __ffsll((long long)holders) - 1) v = -INFINITY;  // drop one holder of the maximum
  }
  if (lane == 0) wave_val[wave] = m;
  lds_barrier();
  float tau = wave_val[0];
  for (int w = 1; w < kWavesPerWg; ++w) tau = fminf(tau, wave_val[w]);
  return tau;
}

constexpr int kRankParts = 8;            // threads that share the comparisons of one candidate, at most
constexpr int kRankPad = 8 * kRankParts;  // zero words a candidate list needs behind its last entry

// top[r] = the candidate of rank r (number of larger candidates; the words are
// distinct and not zero) for r < k, by counting instead of sorting. Up to 1024
// candidates at a time, the comparisons of each split over min(8, 1024 / n)
// threads in runs of a multiple of 8 words. cand[n .. n + kRankPad) are zero
// words (a zero is larger than nothing, so the runs need no bounds), cand is
// 16-byte aligned, and rank_sm[] is all zero on entry (both written before the
// caller's last barrier). Ends with a barrier.
__device__ __forceinline__ void rank_select(const u64* cand, int n, u64* top, int k, uint32_t* rank_sm, int tid) {
  const int width = max(1, min(n, kThreads));
  const int parts = min(kRankParts, kThreads / width);
  const int slot = tid % width, part = tid / width;
  const int span = ((n + parts - 1) / parts + 7) & ~7, j0 = part * span;
  for (int blk = 0; blk < n; blk += width) {
    if (blk > 0) {
      if (tid < width) rank_sm[tid] = 0;
      __syncthreads();
    }
    if (part < parts && blk + slot < n) {
      const u64 c = cand[blk + slot];
      uint32_t cnt = 0;
      for (int j = j0; j < j0 + span; j += 8) {  // (the same words for every lane of a wave: broadcast reads)
        ulonglong2 x[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) x[u] = *reinterpret_cast<const ulonglong2*>(cand + j + 2 * u);
#pragma unroll
        for (int u = 0; u < 4; ++u) cnt += (x[u].x > c ? 1u : 0u) + (x[u].y > c ? 1u : 0u);
      }
      if (cnt) atomicAdd(&rank_sm[slot], cnt);
    }
    __syncthreads();
    if (tid < width && blk + tid < n && rank_sm[tid] < (uint32_t)k) top[rank_sm[tid]] = cand[blk + tid];
    __syncthreads();
  }
}

// The candidate workspace is written by one workgroup and read by another of the same launch (sample_kernel),
// which may sit on another XCD, whose L2 is a different one: stores and loads of device scope, which go
// through to memory, instead of a write-back and an invalidation of whole caches around ordinary ones (measured:
// those made the launch three times slower).
__device__ __forceinline__ void ws_store(u64* p, u64 v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ u64 ws_load(const u64* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

#ifdef MI355_SAMPLER_TRACE
__device__ unsigned long long* g_trace_dev;
__device__ __forceinline__ void trace_mark(int ev) {
  __shared__ int n_marks;  // (thread 0 only; set to zero by mark 1)
  if (threadIdx.x == 0) {
    if (ev == 1) n_marks = 0;
    unsigned long long* row = g_trace_dev + (blockIdx.y * gridDim.x + blockIdx.x) * 16;
    if (n_marks < 16) row[n_marks++] = ((unsigned long long)ev << 56) | (__builtin_amdgcn_s_memrealtime() & 0xffffffffffull);
  }
}
#define TRACE_MARK(ev) trace_mark(ev)
#else
#define TRACE_MARK(ev)
#endif

struct SelectLds {
  uint32_t hist[kBins];
  alignas(16) u64 cand[kCap + kRankPad];  // zero behind the last candidate (rank_select)
  u64 top[kMaxK];
  uint32_t rank_sm[kThreads];
  uint32_t wave_sum[kWavesPerWg];
  uint32_t found[3];  // bin, count above it, count in it
  uint32_t n_cand, n_ties;
};

// A segment of up to R logits per thread, read from memory once: it stays in registers for all passes (same
// index layout as for_each_key); slots past the segment's end hold NaN, which no comparison and no maximum
// ever picks.
template <int R>
__device__ __forceinline__ void load_segment(const SamplerArgs& a, int b, int sgm, float (&xreg)[R]) {
  const int tid = threadIdx.x;
  const int index0 = sgm * a.seg_len;
  const int len = min(a.seg_len, a.vocab - index0);
  const float* seg = a.logits + (size_t)b * a.vocab + index0;
  const bool vec_ok = (a.vocab % 4 == 0) && ((reinterpret_cast<uintptr_t>(a.logits) & 15) == 0);
  if (vec_ok && len == kThreads * R) {
    // a whole segment (the usual case): all loads at once and nothing between them (behind per-thread
    // conditions each load would wait for the one before it)
#pragma unroll
    for (int u = 0; u < R / 4; ++u) {
      const float4 x = *reinterpret_cast<const float4*>(seg + u * kPerIter + tid * 4);
      xreg[4 * u] = x.x; xreg[4 * u + 1] = x.y; xreg[4 * u + 2] = x.z; xreg[4 * u + 3] = x.w;
    }
    return;
  }
#pragma unroll
  for (int u = 0; u < R / 4; ++u) {
    const int base = u * kPerIter + tid * 4;
    if (vec_ok && base + 3 < len) {
      const float4 x = *reinterpret_cast<const float4*>(seg + base);
      xreg[4 * u] = x.x; xreg[4 * u + 1] = x.y; xreg[4 * u + 2] = x.z; xreg[4 * u + 3] = x.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) xreg[4 * u + j] = base + j < len ? seg[base + j] : __int_as_float(0x7fc00000);
    }
  }
}

// The candidates of segment `sgm` of row `b` into the workspace: everything that
// reaches the threshold when that is at most kSlots words (the usual case: the
// row's kernel ranks them anyway), else the segment's k largest.
// R > 0: the segment has at most kThreads * R logits (the host knows) and xreg holds them (load_segment);
// R == 0: they are re-read (from L2) per pass, xreg is unused. Every return is taken by the whole workgroup.
template <int R>
__device__ __forceinline__ void select_segment(const SamplerArgs& a, SelectLds& sm, int b, int sgm,
                                               const float (&xreg)[R > 0 ? R : 1]) {
  uint32_t* const hist = sm.hist;
  u64* const cand = sm.cand;
  u64* const top = sm.top;
  uint32_t* const rank_sm = sm.rank_sm;
  uint32_t* const wave_sum = sm.wave_sum;
  uint32_t* const found = sm.found;
  uint32_t& n_cand = sm.n_cand;
  uint32_t& n_ties = sm.n_ties;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int index0 = sgm * a.seg_len;                 // first vocabulary index of the segment
  const int len = min(a.seg_len, a.vocab - index0);   // > 0 by construction of the grid
  const int k = min(a.k, len);
  const float* seg = a.logits + (size_t)b * a.vocab + index0;
  const bool vec_ok = (a.vocab % 4 == 0) && ((reinterpret_cast<uintptr_t>(a.logits) & 15) == 0);
  u64* out = a.workspace + ((size_t)b * a.segments + sgm) * kSlots;

  constexpr bool resident = R > 0;
  // (the passes of the rare paths below go over the registers of a short segment, but re-read a wide one, from
  // L2: unrolled over 64 registers they would be most of the kernel's code and cost the common path registers)
  auto each = [&](auto&& f) {
    if constexpr (resident && R <= kResident) {
#pragma unroll
      for (int u = 0; u < R / 4; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int i = u * kPerIter + tid * 4 + j;
          if (i < len) f(key_of(xreg[4 * u + j]), i);
        }
    } else {
      for_each_key(seg, len, vec_ok, tid, f);
    }
  };

  if (k == 1) {
    // the first maximum (std::max_element), one pass
    u64 best = 0;
    each([&](uint32_t key, int i) { best = max(best, pack(key, index0 + i)); });
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) best = max(best, (u64)__shfl_xor((long long)best, off, 64));
    if (lane == 0) cand[wave] = best;
    __syncthreads();
    if (tid == 0) {
      for (int w = 1; w < kWavesPerWg; ++w) best = max(best, cand[w]);
      ws_store(out, best);
    }
    for (int i = 1 + tid; i < kSlots; i += kThreads) ws_store(out + i, 0);
    return;
  }

  // ---- a threshold from the per-thread maxima, then everything that reaches it
  rank_sm[tid] = 0;  // (for rank_select, as the zeros behind the candidates; barriers follow on every path)
  for (int i = tid; i < kCap + kRankPad; i += kThreads) cand[i] = 0;
  if constexpr (resident) {
    // on the logits themselves: three instructions per logit, keys only for the candidates
    float tmax = -INFINITY;
#pragma unroll
    for (int e = 0; e < R; ++e) tmax = fmaxf(tmax, xreg[e]);
    if (tid == 0) n_cand = 0;
    const float tau = lower_bound_of_kth_f32(tmax, k, reinterpret_cast<float*>(wave_sum), tid);  // (barrier inside)
    TRACE_MARK(6);
    // sixteen logits per thread at a time (their ballots live in scalar registers)
#pragma unroll
    for (int c0 = 0; c0 < R; c0 += 16) {
      u64 take[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) take[e] = __ballot(xreg[c0 + e] >= tau);
      uint32_t slot0 = reserve_slots(take, &n_cand, lane);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        if (take[e]) {  // (uniform over the wave; most are zero)
          const uint32_t pos = slot0 + lanes_below(take[e]);
          const int u = (c0 + e) >> 2, j = (c0 + e) & 3;
          if (xreg[c0 + e] >= tau && pos < (uint32_t)kCap) cand[pos] = pack(key_of(xreg[c0 + e]), index0 + u * kPerIter + tid * 4 + j);
          slot0 += (uint32_t)__popcll(take[e]);
        }
      }
    }
    __syncthreads();
  } else {
    uint32_t tmax = 0;
    each([&](uint32_t key, int) { tmax = max(tmax, key); });
    if (tid == 0) n_cand = 0;
    const uint32_t tau = lower_bound_of_kth(tmax, k, kWavesPerWg, wave_sum, tid);  // (barrier inside)
    uint32_t mine = 0;
    each([&](uint32_t key, int) { mine += key >= tau ? 1u : 0u; });
    uint32_t pos = mine ? atomicAdd(&n_cand, mine) : 0u;
    each([&](uint32_t key, int i) {
      if (key >= tau) {
        if (pos < (uint32_t)kCap) cand[pos] = pack(key, index0 + i);
        ++pos;
      }
    });
    __syncthreads();
  }
  TRACE_MARK(7);
  // (n_cand is only written again behind further barriers)
  const bool fast_ok = n_cand <= (uint32_t)kCap && n_cand >= (uint32_t)k;  // (fewer than k: NaNs among the logits)
  if (fast_ok && n_cand <= (uint32_t)kSlots) {
    const int n = (int)n_cand;
    if (tid < kSlots) ws_store(out + tid, tid < n ? cand[tid] : 0);
    return;
  }

  if (!fast_ok) {
    // ---- radix descent: (mask, val) = the key prefix of the k-th largest value so far
    uint32_t mask = 0, val = 0, need = (uint32_t)k;
    bool exact_ties = false;
    for (int level = 0; level < 3; ++level) {
      const int shift = level == 0 ? 20 : (level == 1 ? 8 : 0);
      const int nbins = level == 2 ? 256 : kBins;
      for (int i = tid; i < kBins; i += kThreads) hist[i] = 0;
      __syncthreads();
      each([&](uint32_t key, int) {
        if ((key & mask) == val) atomicAdd(&hist[(key >> shift) & (nbins - 1)], 1u);
      });
      __syncthreads();
      find_bin(hist, nbins, need, wave_sum, found, tid);
      val |= found[0] << shift;
      mask |= (uint32_t)(nbins - 1) << shift;
      need -= found[1];
      const uint32_t in_bin = found[2];
      if (in_bin + ((uint32_t)k - need) <= (uint32_t)kCap) break;
      exact_ties = level == 2;  // the whole key is fixed and still too many: equal values
      __syncthreads();          // found[] is rewritten by the next level
    }

    // ---- collection: everything above the prefix, and the prefix bin itself
    // (of exact ties only the `need` lowest indices)
    if (tid == 0) { n_cand = 0; n_ties = 0; }
    for (int i = tid; i < kCap + kRankPad; i += kThreads) cand[i] = 0;
    __syncthreads();
    if (!exact_ties) {
      each([&](uint32_t key, int i) {
        if ((key & mask) >= val) cand[atomicAdd(&n_cand, 1u)] = pack(key, index0 + i);
      });
    } else {
      // every iteration in step, so that ties are ranked in index order: waves,
      // lanes and a thread's four elements are laid out ascending
      for (int base0 = 0; base0 < len; base0 += kPerIter) {
        const int base = base0 + tid * 4;
        uint32_t key[4];
        int mine = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          key[j] = base + j < len ? key_of(seg[base + j]) : 0u;
          if (base + j < len && key[j] > val) cand[atomicAdd(&n_cand, 1u)] = pack(key[j], index0 + base + j);
          if (base + j < len && key[j] == val) ++mine;
        }
        uint32_t incl = (uint32_t)mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
          const uint32_t v = __shfl_up(incl, off, 64);
          if (lane >= off) incl += v;
        }
        if (lane == 63) wave_sum[wave] = incl;
        __syncthreads();
        uint32_t rank = n_ties + incl - (uint32_t)mine, total = 0;
        for (int w = 0; w < kWavesPerWg; ++w) { if (w < wave) rank += wave_sum[w]; total += wave_sum[w]; }
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (base + j < len && key[j] == val) {
            if (rank < need) cand[atomicAdd(&n_cand, 1u)] = pack(key[j], index0 + base + j);
            ++rank;
          }
        __syncthreads();
        if (tid == 0) n_ties += total;
        __syncthreads();
      }
    }
    __syncthreads();
  }
  const int n = (int)n_cand;  // k <= n <= kCap
  rank_select(cand, n, top, k, rank_sm, tid);
  if (tid < kSlots) ws_store(out + tid, tid < k ? top[tid] : 0);
}

// Grid (segments, rows): the first of two launches for rows whose segments do not fit in registers.
// 64 registers at most, so that two workgroups share a compute unit.
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(8, 8)))
select_kernel(const SamplerArgs a) {
  __shared__ SelectLds sm;
  const float none[1] = {0.f};
  select_segment<0>(a, sm, blockIdx.y, blockIdx.x, none);
}

struct FinishLds {
  alignas(16) u64 surv[kMergeCap + kRankPad];  // the segments' candidates that reach the threshold, then zeros
  u64 cand[kMaxK];      // the row's k winners, descending
  alignas(16) float e_sm[kMaxK + 16];  // (+16: the loops below read up to 15 entries past the last one they use)
  uint32_t rank_sm[kThreads];
  uint32_t wave_val[kWavesPerWg];
  uint32_t n_surv;
  float inv_sm;
  double cum_sm[kMaxK];
};

// Merges the segments' candidates of row `b` and draws (sampling_cpu_util.cc:98-131, 189-230). Returns early
// for the waves that hold none of the k winners: the caller has nothing left to do after it but for thread 0.
__device__ __forceinline__ void finish_row(const SamplerArgs& a, FinishLds& sm, int b) {
  u64* const surv = sm.surv;
  u64* const cand = sm.cand;
  float* const e_sm = sm.e_sm;
  uint32_t* const rank_sm = sm.rank_sm;
  uint32_t* const wave_val = sm.wave_val;
  uint32_t& n_surv = sm.n_surv;
  float& inv_sm = sm.inv_sm;
  double* const cum_sm = sm.cum_sm;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int k = min(a.k, a.vocab);
  // The row's n = segments x kSlots words (zero words are empty slots; a segment fills its slots from the front).
  // More than four segments: wave s holds the words of segment s, four consecutive ones per thread. Up to four:
  // one word per thread, every fourth slot of a segment per wave, so that each of the 4 x segments waves gets its
  // share of the filled slots at the front (the bound below takes a wave with few words for an empty one).
  const int n = a.segments * kSlots;  // <= kMergeCap
  const u64* in = a.workspace + (size_t)b * n;
  const bool one_each = n <= kThreads;
  const int waves = one_each ? n / 64 : n / 256;
  u64 w[4] = {0, 0, 0, 0};
  uint32_t wmax = 0;
  static_assert(kSlots == 4 * 64, "one wave of four-word threads per segment, or four waves of one-word threads");
  if (one_each) {
    if (tid < n) {
      const int r = tid % kSlots;
      w[0] = ws_load(in + (tid - r) + (r % 64) * 4 + r / 64);
    }
  } else if (4 * tid < n) {
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = ws_load(in + 4 * tid + j);
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) wmax = max(wmax, (uint32_t)(w[j] >> 32));
  if (tid == 0) n_surv = 0;
  rank_sm[tid] = 0;  // (for rank_select)
  for (int i = tid; i < kMergeCap + kRankPad; i += kThreads) surv[i] = 0;
  // same scheme as in select_segment: a lower bound of the k-th largest key, the
  // words that reach it, their ranks by counting
  TRACE_MARK(8);
  const uint32_t tau = lower_bound_of_kth(wmax, k, waves, wave_val, tid);  // (barrier inside)
  TRACE_MARK(9);
  u64 take[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) take[j] = __ballot(w[j] != 0 && (uint32_t)(w[j] >> 32) >= tau);
  uint32_t slot0 = reserve_slots(take, &n_surv, lane);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (w[j] != 0 && (uint32_t)(w[j] >> 32) >= tau) surv[slot0 + lanes_below(take[j])] = w[j];
    slot0 += (uint32_t)__popcll(take[j]);
  }
  __syncthreads();
  TRACE_MARK(10);
  rank_select(surv, (int)n_surv, cand, k, rank_sm, tid);
  TRACE_MARK(11);
  // The rest is the work of k threads: the other waves leave (a barrier waits only for the waves of the workgroup
  // that are still running; nothing comes after the merge for them in either kernel).
  if (tid >= ((k + 63) & ~63)) return;
  if (k == 1) {
    if (tid == 0) {
      const int idx = index_of(cand[0]);
      if (a.ids) a.ids[b] = idx;
      if (a.scores) a.scores[b] = 0.f;  // log(1)
      if (a.topk_idx) a.topk_idx[b] = idx;
      if (a.topk_prob) a.topk_prob[b] = 1.f;
    }
    return;
  }
  // ---- the k winners in the reference's op order (sampling_cpu_util.cc:98-131, 189-230)
  const float m = logit_of((uint32_t)(cand[0] >> 32));
  const float t_soft = fmaxf(a.temperature, FLT_EPSILON);
  if (tid < k) e_sm[tid] = expf((logit_of((uint32_t)(cand[tid] >> 32)) - m) / t_soft);
  if (tid < 16) e_sm[k + tid] = 0.f;
  __syncthreads();
  if (tid == 0) {
    // sequential float32 sum, as the reference; the LDS reads run ahead of the adds
    float sum = 0.f;
    for (int i = 0; i < k; i += 8) {
      float x[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) x[u] = e_sm[i + u];  // zeros behind entry k - 1
#pragma unroll
      for (int u = 0; u < 8; ++u) sum += x[u];
    }
    inv_sm = sum <= FLT_EPSILON ? -1.f : (isinf(sum) ? -2.f : 1.f / sum);
  }
  __syncthreads();
  if (tid < k) {
    const float inv = inv_sm;
    e_sm[tid] = inv == -1.f ? 1.f / (float)k : (inv == -2.f ? (tid == 0 ? 1.f : 0.f) : e_sm[tid] * inv);
  }
  __syncthreads();
  // Cumulative probabilities in float64, every thread summing its own prefix in
  // the reference's order; the nucleus ends at the first one that reaches p, the
  // draw picks the first one that covers it (sampling_cpu_util.cc:189-230).
  bool reaches = false;
  if (tid < k) {
    double c = 0.0;
    for (int i = 0; i <= tid; i += 16) {
      // 16 probabilities per round trip; conversion and selection are off the chain of additions
      float4 x[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) x[u] = *reinterpret_cast<const float4*>(&e_sm[i + 4 * u]);
      double d[16];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        d[4 * u] = i + 4 * u <= tid ? (double)x[u].x : 0.0;  // (+0.0 leaves c >= 0 as it is)
        d[4 * u + 1] = i + 4 * u + 1 <= tid ? (double)x[u].y : 0.0;
        d[4 * u + 2] = i + 4 * u + 2 <= tid ? (double)x[u].z : 0.0;
        d[4 * u + 3] = i + 4 * u + 3 <= tid ? (double)x[u].w : 0.0;
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) c += d[u];
    }
    cum_sm[tid] = c;
    reaches = c >= (double)a.p;
  }
  // the first thread of all that reaches p (k - 1 if none does: then the nucleus is all k candidates)
  const int k_waves = (k + 63) >> 6;  // the waves that hold winners
  static_assert(kMaxK <= 8 * 64, "wave_val holds two entries per wave of winners");
  {
    const u64 m = __ballot(reaches);
    if (lane == 0 && wave < k_waves) wave_val[wave] = m ? (uint32_t)(wave * 64 + __ffsll((long long)m) - 1) : (uint32_t)kMaxK;
  }
  __syncthreads();
  int first_reach = k - 1;
  for (int wv = 0; wv < k_waves; ++wv) first_reach = min(first_reach, (int)wave_val[wv]);
  const int nucleus = first_reach + 1;
  const double mass = cum_sm[first_reach];
  float u01;
  if (a.uniforms) u01 = a.uniforms[b];
  else u01 = (float)(philox_first_word((uint32_t)b, (uint32_t)a.call_index, (uint32_t)(a.call_index >> 32), 0u, a.seed,
                                       0x4D493335u) >> 8) * (1.f / 16777216.f);
  const double draw = (double)u01 * mass;
  {
    const u64 m = __ballot(tid < nucleus && draw <= cum_sm[tid]);
    if (lane == 0 && wave < k_waves) wave_val[8 + wave] = m ? (uint32_t)(wave * 64 + __ffsll((long long)m) - 1) : (uint32_t)kMaxK;
  }
  __syncthreads();
  if (tid == 0) {
    int first_hit = kMaxK;
    for (int wv = 0; wv < k_waves; ++wv) first_hit = min(first_hit, (int)wave_val[8 + wv]);
    const int chosen = mass > DBL_EPSILON ? min(first_hit, nucleus - 1) : 0;
    if (a.ids) a.ids[b] = index_of(cand[chosen]);
    if (a.scores) a.scores[b] = logf(expf((logit_of((uint32_t)(cand[chosen] >> 32)) - m) / a.temperature));
  }
  __syncthreads();
  if (tid < k) {
    if (a.topk_idx) a.topk_idx[(size_t)b * k + tid] = index_of(cand[tid]);
    if (a.topk_prob) a.topk_prob[(size_t)b * k + tid] = e_sm[tid];
  }
}

// Grid (rows): the second of the two launches.
__global__ void __launch_bounds__(kThreads) finish_kernel(const SamplerArgs a) {
  __shared__ FinishLds sm;
  finish_row(a, sm, blockIdx.x);
}

// Both steps in one launch, for rows whose segments stay in registers: grid (segments, rows), one workgroup per
// segment of R logits per thread. Every load of the segment is issued at once, so that the whole call is on its
// way from HBM from the first microsecond on; the per-thread maxima are taken as the loads land. The workgroup
// that delivers the last segment of a row (a ticket per row, drawn once the segment's candidates are written)
// finishes the row.
template <int R>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(R <= kResident ? 8 : 4, R <= kResident ? 8 : 4)))
sample_kernel(const SamplerArgs a) {
  __shared__ union Lds {
    SelectLds select;
    FinishLds finish;
    __device__ Lds() {}
  } sm;
  __shared__ uint32_t ticket_sm;
  const int tid = threadIdx.x;
  const int b = blockIdx.y, sgm = blockIdx.x;
#ifdef MI355_SAMPLER_TRACE
  int n_ev = 0;
  auto mark = [&](int ev) { (void)n_ev; trace_mark(ev); };
#else
  auto mark = [&](int) {};
#endif
  mark(1);
  float xreg[R];
  load_segment<R>(a, b, sgm, xreg);
#ifdef MI355_SAMPLER_TRACE
  __builtin_amdgcn_s_waitcnt(0x0F70);
  mark(2);
#endif
  select_segment<R>(a, sm.select, b, sgm, xreg);
  mark(3);
  // The candidates are written (ws_store): once every thread's stores have been acknowledged, draw the row's
  // ticket. Who draws the last one reads what the others wrote before they drew theirs (ws_load).
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  __syncthreads();
  if (tid == 0) ticket_sm = __hip_atomic_fetch_add(a.tickets + b, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  mark(4);
  if (ticket_sm != (uint32_t)a.segments - 1u) return;
  __syncthreads();  // (the arrays of the selection become those of the merge)
  finish_row(a, sm.finish, b);
  mark(5);
  if (tid == 0) a.tickets[b] = 0;  // for the next launch
}

int fail(char** error_msg, int code, const char* fmt, ...) {
  if (error_msg) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    *error_msg = strdup(buf);
  }
  return code;
}

#define HIP_OR_RETURN(expr)                                                                          \
  do {                                                                                               \
    hipError_t e_ = (expr);                                                                          \
    if (e_ != hipSuccess)                                                                            \
      return fail(error_msg, e_ == hipErrorOutOfMemory ? MI355_SAMPLER_RESOURCE_EXHAUSTED            \
                                                        : MI355_SAMPLER_INTERNAL,                    \
                  "%s: %s", #expr, hipGetErrorString(e_));                                           \
  } while (0)

}  // namespace

#ifdef MI355_SAMPLER_TRACE  // (development builds: a timeline per workgroup)
static unsigned long long* g_trace = nullptr;
extern "C" int mi355_sampler_trace_read(void* dst, size_t bytes) {
  return (int)hipMemcpy(dst, g_trace, bytes, hipMemcpyDeviceToHost);
}
#endif

struct mi355_sampler {
  mi355_sampler_config cfg{};
  int k = 1;
  float p = 1.f;
  hipStream_t stream = nullptr;
  bool owns_stream = false;
  uint64_t calls = 0;
  bool timing = false, timed = false;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  // host_io staging
  float* d_logits = nullptr;
  float* d_uniforms = nullptr;
  int32_t* d_ids = nullptr;
  float* d_scores = nullptr;
  int32_t* d_topk_idx = nullptr;
  float* d_topk_prob = nullptr;
  // candidates of the segments, [batch][segments][k]
  unsigned long long* d_workspace = nullptr;
  uint32_t* d_tickets = nullptr;  // [batch], all zero between calls
  int segments = 1, seg_len = 0;
  bool wide = false;  // segments of up to kThreads * kResidentWide logits (sample_kernel<kResidentWide>)
};

namespace {

int run(mi355_sampler* h, const float* logits, const float* uniforms, int32_t* ids, float* scores, int32_t* topk_idx,
        float* topk_prob, bool counts_as_draw, char** error_msg) {
  if (!h) return fail(error_msg, MI355_SAMPLER_INVALID_ARGUMENT, "null sampler");
  if (!logits) return fail(error_msg, MI355_SAMPLER_INVALID_ARGUMENT, "null logits");
  HIP_OR_RETURN(hipSetDevice(h->cfg.device));
  const size_t B = h->cfg.batch_size, V = h->cfg.vocab_size, K = std::min<size_t>(h->k, V);
  SamplerArgs a{};
  if (h->cfg.host_io) {
    HIP_OR_RETURN(hipMemcpyAsync(h->d_logits, logits, B * V * sizeof(float), hipMemcpyHostToDevice, h->stream));
    if (uniforms)
      HIP_OR_RETURN(hipMemcpyAsync(h->d_uniforms, uniforms, B * sizeof(float), hipMemcpyHostToDevice, h->stream));
    a.logits = h->d_logits;
    a.uniforms = uniforms ? h->d_uniforms : nullptr;
    a.ids = ids ? h->d_ids : nullptr;
    a.scores = scores ? h->d_scores : nullptr;
    a.topk_idx = topk_idx ? h->d_topk_idx : nullptr;
    a.topk_prob = topk_prob ? h->d_topk_prob : nullptr;
  } else {
    a.logits = logits; a.uniforms = uniforms; a.ids = ids; a.scores = scores;
    a.topk_idx = topk_idx; a.topk_prob = topk_prob;
  }
  a.vocab = (int32_t)V;
  a.k = h->k;
  a.p = h->p;
  a.temperature = h->cfg.temperature;
  a.seed = (uint32_t)h->cfg.seed;
  a.call_index = h->calls;
  if (counts_as_draw) ++h->calls;
  a.workspace = h->d_workspace;
  a.segments = h->segments;
  a.seg_len = h->seg_len;
  a.tickets = h->d_tickets;
#ifdef MI355_SAMPLER_TRACE
  if (!g_trace) HIP_OR_RETURN(hipMalloc(&g_trace, 8 * 16 * 4096));
  HIP_OR_RETURN(hipMemsetAsync(g_trace, 0, 8 * 16 * 4096, h->stream));
  a.trace = g_trace;
  HIP_OR_RETURN(hipMemcpyToSymbol(HIP_SYMBOL(g_trace_dev), &g_trace, sizeof(g_trace)));
#endif
  // ev0 / ev1 ride on the dispatches: begin of the first kernel, end of the last
  hipEvent_t e0 = h->timing ? h->ev0 : nullptr, e1 = h->timing ? h->ev1 : nullptr;
  const dim3 grid((unsigned)h->segments, (unsigned)B);
  if (h->seg_len <= kSegmentMin) {
    hipExtLaunchKernelGGL(sample_kernel<kResident>, grid, dim3(kThreads), 0, h->stream, e0, e1, 0, a);
    HIP_OR_RETURN(hipGetLastError());
  } else if (h->wide) {
    hipExtLaunchKernelGGL(sample_kernel<kResidentWide>, grid, dim3(kThreads), 0, h->stream, e0, e1, 0, a);
    HIP_OR_RETURN(hipGetLastError());
  } else {
    hipExtLaunchKernelGGL(select_kernel, grid, dim3(kThreads), 0, h->stream, e0, nullptr, 0, a);
    HIP_OR_RETURN(hipGetLastError());
    hipExtLaunchKernelGGL(finish_kernel, dim3((unsigned)B), dim3(kThreads), 0, h->stream, nullptr, e1, 0, a);
    HIP_OR_RETURN(hipGetLastError());
  }
  h->timed = h->timing;
  if (h->cfg.host_io) {
    if (ids) HIP_OR_RETURN(hipMemcpyAsync(ids, h->d_ids, B * sizeof(int32_t), hipMemcpyDeviceToHost, h->stream));
    if (scores) HIP_OR_RETURN(hipMemcpyAsync(scores, h->d_scores, B * sizeof(float), hipMemcpyDeviceToHost, h->stream));
    if (topk_idx)
      HIP_OR_RETURN(hipMemcpyAsync(topk_idx, h->d_topk_idx, B * K * sizeof(int32_t), hipMemcpyDeviceToHost, h->stream));
    if (topk_prob)
      HIP_OR_RETURN(hipMemcpyAsync(topk_prob, h->d_topk_prob, B * K * sizeof(float), hipMemcpyDeviceToHost, h->stream));
    HIP_OR_RETURN(hipStreamSynchronize(h->stream));
  }
  return MI355_SAMPLER_OK;
}

}  // namespace

extern "C" {

int mi355_sampler_create(const mi355_sampler_config* c, mi355_sampler** out, char** error_msg) {
  if (!c || !out) return fail(error_msg, MI355_SAMPLER_INVALID_ARGUMENT, "null config or output pointer");
  *out = nullptr;
  if (c->struct_size != sizeof(mi355_sampler_config))
    return fail(error_msg, MI355_SAMPLER_INVALID_ARGUMENT, "mi355_sampler_config.struct_size %u, expected %zu",
                c->struct_size, sizeof(mi355_sampler_config));
  int k = c->k;
  float p = c->p;
  switch (c->type) {
    case MI355_SAMPLER_GREEDY: k = 1; p = 1.f; break;
    case MI355_SAMPLER_TOP_K: p = 1.f; break;
    case MI355_SAMPLER_TOP_P:
    case MI355_SAMPLER_TYPE_UNSPECIFIED: break;
    default: return fail(error_msg, MI355_SAMPLER_INVALID_ARGUMENT, "unknown sampler type %d", c->type);
  }
  // messages of TopPSampler::Create (top_p_cpu_sampler.cc:42-55)
  if (k <= 0) return fail(error_msg, MI355_SAMPLER_INVALID_ARGUMENT, "k must be positive.");
  if (!(p >= 0.0f && p <= 1.0f)) return fail(error_msg, MI355_SAMPLER_INVALID_ARGUMENT, "p must be in [0, 1].");
  if (c->batch_size <= 0) return fail(error_msg, MI355_SAMPLER_INVALID_ARGUMENT, "batch_size must be positive.");
  if (!(c->temperature > 0.0f))
    return fail(error_msg, MI355_SAMPLER_INVALID_ARGUMENT, "Temperature must be positive, but got %g", c->temperature);
  if (c->vocab_size <= 0) return fail(error_msg, MI355_SAMPLER_INVALID_ARGUMENT, "vocab_size must be positive.");
  if (std::min(k, c->vocab_size) > kMaxK)
    return fail(error_msg, MI355_SAMPLER_UNIMPLEMENTED, "k = %d: at most %d candidates are supported", k, kMaxK);
  int ndev = 0;
  if (hipGetDeviceCount(&ndev) != hipSuccess || c->device < 0 || c->device >= ndev)
    return fail(error_msg, MI355_SAMPLER_UNAVAILABLE, "no usable HIP device %d", c->device);
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, c->device) != hipSuccess || strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(error_msg, MI355_SAMPLER_UNAVAILABLE, "device %d is not gfx950", c->device);
  HIP_OR_RETURN(hipSetDevice(c->device));
  mi355_sampler* h = new mi355_sampler();
  h->cfg = *c;
  h->k = k;
  h->p = p;
  auto bail = [&](int code, const char* what, hipError_t e) {
    mi355_sampler_destroy(h);
    return fail(error_msg, code, "%s: %s", what, hipGetErrorString(e));
  };
  hipError_t e;
  if (c->own_stream) {
    if ((e = hipStreamCreate(&h->stream)) != hipSuccess) return bail(MI355_SAMPLER_INTERNAL, "hipStreamCreate", e);
    h->owns_stream = true;
  } else {
    h->stream = static_cast<hipStream_t>(c->stream);
  }
  if ((e = hipEventCreate(&h->ev0)) != hipSuccess || (e = hipEventCreate(&h->ev1)) != hipSuccess)
    return bail(MI355_SAMPLER_INTERNAL, "hipEventCreate", e);
  // Segments of kSegmentMin logits or less (a multiple of 4), unless that would take more than kMaxSegments:
  // 1, 2, 4, 8 or 16 segments (with three, the row's kernel could not bound its candidates: lower_bound_of_kth).
  // A call of so many rows that the short segments would make more than two workgroups per compute unit takes
  // segments four times as long (64 logits per thread in registers): the threshold, the barriers and the ticket
  // are then paid once for four times the logits, and the row's merge has a quarter of the words to look at.
  h->segments = 1;
  while (h->segments < kMaxSegments && (size_t)h->segments * kSegmentMin < (size_t)c->vocab_size) h->segments *= 2;
  if (h->segments >= 4 && (size_t)c->batch_size * h->segments > 2 * (size_t)std::max(1, prop.multiProcessorCount) &&
      (size_t)(h->segments / 4) * kThreads * kResidentWide >= (size_t)c->vocab_size) {
    h->segments /= 4;
    h->wide = true;
  }
  h->seg_len = ((c->vocab_size + h->segments - 1) / h->segments + 3) / 4 * 4;
  h->segments = (c->vocab_size + h->seg_len - 1) / h->seg_len;
  if ((e = hipMalloc(&h->d_workspace, sizeof(unsigned long long) * c->batch_size * h->segments * kSlots)) != hipSuccess)
    return bail(MI355_SAMPLER_RESOURCE_EXHAUSTED, "candidate workspace", e);
  if ((e = hipMalloc(&h->d_tickets, sizeof(uint32_t) * c->batch_size)) != hipSuccess)
    return bail(MI355_SAMPLER_RESOURCE_EXHAUSTED, "row tickets", e);
  if ((e = hipMemsetAsync(h->d_tickets, 0, sizeof(uint32_t) * c->batch_size, h->stream)) != hipSuccess ||
      (e = hipStreamSynchronize(h->stream)) != hipSuccess)
    return bail(MI355_SAMPLER_INTERNAL, "row tickets clear", e);
  if (c->host_io) {
    const size_t B = c->batch_size, V = c->vocab_size, K = std::min<size_t>(k, V);
    if ((e = hipMalloc(&h->d_logits, B * V * sizeof(float))) != hipSuccess ||
        (e = hipMalloc(&h->d_uniforms, B * sizeof(float))) != hipSuccess ||
        (e = hipMalloc(&h->d_ids, B * sizeof(int32_t))) != hipSuccess ||
        (e = hipMalloc(&h->d_scores, B * sizeof(float))) != hipSuccess ||
        (e = hipMalloc(&h->d_topk_idx, B * K * sizeof(int32_t))) != hipSuccess ||
        (e = hipMalloc(&h->d_topk_prob, B * K * sizeof(float))) != hipSuccess)
      return bail(MI355_SAMPLER_RESOURCE_EXHAUSTED, "staging buffers", e);
  }
  *out = h;
  return MI355_SAMPLER_OK;
}

void mi355_sampler_destroy(mi355_sampler* h) {
  if (!h) return;
  (void)hipSetDevice(h->cfg.device);
  (void)hipStreamSynchronize(h->stream);
  for (void* p : {(void*)h->d_logits, (void*)h->d_uniforms, (void*)h->d_ids, (void*)h->d_scores, (void*)h->d_topk_idx,
                  (void*)h->d_topk_prob, (void*)h->d_workspace, (void*)h->d_tickets})
    if (p) (void)hipFree(p);
  if (h->ev0) (void)hipEventDestroy(h->ev0);
  if (h->ev1) (void)hipEventDestroy(h->ev1);
  if (h->owns_stream && h->stream) (void)hipStreamDestroy(h->stream);
  delete h;
}

int mi355_sampler_sample(mi355_sampler* h, const float* logits, int32_t* ids, float* scores, char** error_msg) {
  if (!ids) return fail(error_msg, MI355_SAMPLER_INVALID_ARGUMENT, "null ids");
  return run(h, logits, nullptr, ids, scores, nullptr, nullptr, true, error_msg);
}

int mi355_sampler_sample_with_uniforms(mi355_sampler* h, const float* logits, const float* uniforms, int32_t* ids,
                                       float* scores, char** error_msg) {
  if (!ids || !uniforms) return fail(error_msg, MI355_SAMPLER_INVALID_ARGUMENT, "null ids or uniforms");
  return run(h, logits, uniforms, ids, scores, nullptr, nullptr, false, error_msg);
}

int mi355_sampler_top_k(mi355_sampler* h, const float* logits, int32_t* indices, float* probabilities,
                        char** error_msg) {
  if (!indices || !probabilities)
    return fail(error_msg, MI355_SAMPLER_INVALID_ARGUMENT, "null indices or probabilities");
  return run(h, logits, nullptr, nullptr, nullptr, indices, probabilities, false, error_msg);
}

int mi355_sampler_sync(mi355_sampler* h, char** error_msg) {
  if (!h) return fail(error_msg, MI355_SAMPLER_INVALID_ARGUMENT, "null sampler");
  HIP_OR_RETURN(hipSetDevice(h->cfg.device));
  HIP_OR_RETURN(hipStreamSynchronize(h->stream));
  return MI355_SAMPLER_OK;
}

int mi355_sampler_set_timing(mi355_sampler* h, int32_t enabled) {
  if (!h) return MI355_SAMPLER_INVALID_ARGUMENT;
  h->timing = enabled != 0;
  if (!h->timing) h->timed = false;
  return MI355_SAMPLER_OK;
}

float mi355_sampler_last_kernel_ms(mi355_sampler* h) {
  if (!h || !h->timed) return -1.f;
  if (hipEventSynchronize(h->ev1) != hipSuccess) return -1.f;
  float ms = -1.f;
  if (hipEventElapsedTime(&ms, h->ev0, h->ev1) != hipSuccess) return -1.f;
  return ms;
}

}  // extern "C"
