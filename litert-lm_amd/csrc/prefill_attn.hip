// Causal / sliding-window prefill attention over the KV cache (gfx950, MFMA).
//
// A workgroup of 4 waves (one per SIMD) covers HPB query heads of one KV head
// times PT stretches of 64 consecutive positions (HPB * PT = 4); each wave owns
// one head and one stretch = two tiles of 32 queries. All waves walk the same
// 32-key blocks, so each K/V block is brought from HBM/L2 into an LDS ring once
// per workgroup (global_load ... lds, no registers in between, one iteration
// ahead), and every K or V operand a wave reads from LDS feeds two MFMAs, one
// per tile. The key loop starts at the first block the window still reaches and
// stops at the diagonal.
//
// Per wave, key block and tile (32x32x16 MFMA, transposed formulation so that
// one lane owns one query):
//   S^T[key][query] = K . Q^T        16 MFMAs (head_dim 256); Q^T of the first tile
//                                    in registers, of the second in a per-wave LDS slice
//   online softmax on the 16 scores a lane holds for its query
//   O^T[d][query]  += V^T . P^T      16 MFMAs, P^T taken from S^T's registers
// The row order in which K is fed to the first MFMA is chosen so that the
// probabilities already sit in the token order of the V plane. The two tiles'
// 256 accumulator registers fill the AGPR half of the register file.
//
// Work distribution: persistent workgroups, one per CU, draw (unit, stretch)
// items from per-XCD queues of atomic tickets, longest key loops first.
//
// Replaces the prefill-time attention the reference reaches through
// compiled_model_.Run(prefill_signature, ...)
// (runtime/executor/llm_litert_compiled_model_executor.cc:271) and the
// [1,1,S,ctx] mask built for it
// (runtime/executor/litert_compiled_model_executor_utils.cc:332-397).
#include <atomic>
#include <hip/hip_runtime.h>
#include <math.h>

#include <type_traits>
#include <utility>

#include <algorithm>
#include <set>
#include <vector>

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

// Output element type: the cache's own 16-bit type, or float32 for float32 activations (the queries of such a
// call are rounded to the cache's type by convert_queries_kernel before the attention kernel runs).
template <int OUT>
struct OutEl;
template <>
struct OutEl<kF32> { using type = float; };
template <>
struct OutEl<kF16> { using type = _Float16; };
template <>
struct OutEl<kBF16> { using type = __bf16; };

// Key (0..31, within a block) that MFMA row m of S^T stands for.
__device__ __forceinline__ int key_of_row(int m) { return 16 * ((m >> 3) & 1) + 8 * (m >> 4) + (m & 7); }

// LDS plan (dynamic): a ring of three K blocks and a ring of three V blocks
// (2 * 3 * 64*D bytes = 96 KiB at head_dim 256), then the query rows of the
// four waves (64 KiB): 160 KiB, all a CU has.
constexpr int kStages = 3;
constexpr int kWaves = 4;       // per workgroup
constexpr int kStretch = 32;    // query positions per wave: one tile

template <int D>
constexpr int prefill_lds_bytes() { return 2 * kStages * 64 * D + kWaves * kStretch * 2 * D; }  // rings + query rows

// s_waitcnt immediates (gfx9 encoding: vmcnt[3:0], expcnt[6:4], lgkmcnt[11:8],
// vmcnt[15:14]) that wait on vector-memory operations only.
// "all but the n most recent vector-memory operations of this wave have completed" (n <= 63)
constexpr int wait_vm(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }
constexpr int kWaitVm0 = 0x0F70;  // all of this wave's transfers have landed
constexpr int kWaitVm4 = 0x0F74;  // all but the 4 most recent ones
constexpr int kWaitVm8 = 0x0F78;  // all but the 8 most recent ones


// Workgroup barrier that orders LDS traffic only. __syncthreads() (and any fence
// the compiler knows of) also waits for every outstanding vector-memory
// operation, LDS transfers included: here those are the K / V blocks still on
// their way into other ring stages, exactly what is meant to stay in flight
// across a barrier. What must have landed before a barrier is waited for
// explicitly (s_waitcnt vmcnt) in front of it. The "memory" clobber keeps the
// compiler from moving memory operations across.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), in order.
template <int... Is, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F&& f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

template <int DT, int OUT, int D, int HPB, bool CAP>
__global__ void __launch_bounds__(kWaves * 64) prefill_attn_kernel(const PrefillArgs a) {
  using E = El<DT>;
  using out_t = typename OutEl<OUT>::type;
  using vec8 = typename E::vec8;
  constexpr int PT = 4 / HPB;            // stretches per workgroup
  constexpr int NJ = D / 16;             // K-slices of the QK^T product
  constexpr int NDP = D / 32;            // 32-channel tiles of O^T
  constexpr int kBlockBytes = 64 * D;    // one 32-key block of a 16-bit plane
  constexpr int kXfers = 16 / kWaves;    // 1 KiB transfers per wave, block and plane
  // P operands per block: keys 0-15 and 16-31. They are IEEE half values for both cache types (the V
  // planes of a bfloat16 cache hold half values, attn_params.h), so P.V always runs on the fp16 MFMA.
  constexpr int NP = 2;

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint8_t* const sm_k = smem;                              // [kStages][K block]
  uint8_t* const sm_v = smem + kStages * kBlockBytes;      // [kStages][V block]
  // The ticket of the next work item is passed through the last V stage, which
  // no transfer writes before the second barrier of an item.
  volatile int* const sm_ticket = reinterpret_cast<volatile int*>(sm_v + (kStages - 1) * kBlockBytes);
  uint8_t* const sm_q = smem + 2 * kStages * kBlockBytes;  // [kWaves][kStretch rows of 2 * D bytes]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, hh = lane >> 5;
  // Persistent workgroups, one per CU, draw work items = (unit, stretch) from
  // queues of atomic tickets. A unit = (layer, KV head, head block) shares one
  // K/V plane. The units are dealt to the queues in order of decreasing work
  // (the host sorts them: global layers before windowed ones), and a queue hands
  // out all stretches of its units, longest key loops first. Workgroup k starts
  // on queue k % 2, i.e. the workgroups of every other XCD share a queue and the
  // K/V blocks they ask for are mostly in their XCDs' L2 caches already; a
  // workgroup whose queue has run dry takes from the other one, which evens out
  // the tail. (Eight queues, one per XCD, kept the blocks closer but left the
  // tail 11 % long: with 26 layers a queue held three or four units.)
  const int hblocks = a.group / HPB;
  const int per_layer = a.geom.hkv * hblocks;
  const int units = a.n_layers * per_layer;
  const int tiles = (a.n + kStretch * PT - 1) / (kStretch * PT);
  const int home = blockIdx.x & (kPrefillQueues - 1);
  int tried = 0;  // queues this workgroup has found empty (kept by thread 0)
  bool first_draw = true;
  const int smax = a.kchunk > 0 ? a.smax : 1;  // work items per tile (key split), some of them empty
  const float softcap = a.softcap;  // CAP: > 0, scores go through softcap * tanh(score / softcap)
  const float c = CAP ? 1.f : a.scale * kLog2e;
  const int pos_end = a.q_pos0 + a.n;                // one past the last query position
  // LDS offsets of this lane's operands inside a block
  const int key_row = key_of_row(n);
  const int k_off = (key_row >> 4) * (16 * D * 2) + (key_row & 15) * 16 + hh * 256;
  const int v_off = (n >> 4) * 1024 + hh * 256 + (n & 15) * 16;
  constexpr int kAhead = 4;  // K operand reads in flight ahead of their MFMAs

  // A ticket of a queue with qcnt units is (tile, part, unit), tile-major: a
  // queue's longest key loops first. Key blocks of a tile: from the first one the
  // window of its first row reaches to the one holding the diagonal of its last
  // valid row; part p of a split tile covers blocks [p * kchunk, (p + 1) * kchunk)
  // of those.
  struct Item { int li, kvh, hb, tile, part, layer, window, wg_pos0, kb_lo, nblk_tile; };
  auto item_of = [&](int qx, int ticket) {
    Item it;
    const int qcnt = (units - qx + kPrefillQueues - 1) / kPrefillQueues;
    const int per_tile = qcnt * smax;
    const int ti = ticket / per_tile, r2 = ticket - ti * per_tile;
    it.part = r2 / qcnt;
    const int slot = qx + kPrefillQueues * (r2 - it.part * qcnt);
    const int u = a.use_order ? a.unit_order[slot] : slot;
    it.li = u / per_layer;
    const int rem = u - it.li * per_layer;
    it.kvh = rem / hblocks;
    it.hb = rem - it.kvh * hblocks;
    it.tile = tiles - 1 - ti;
    it.layer = a.layer_begin + it.li;
    it.window = a.layer_window[it.layer];
    it.wg_pos0 = a.q_pos0 + it.tile * (kStretch * PT);  // first position of the workgroup
    const int last_pos = min(it.wg_pos0 + kStretch * PT, pos_end) - 1;
    it.kb_lo = 0;
    if (it.window > 0 && it.wg_pos0 - it.window + 1 > 0) it.kb_lo = (it.wg_pos0 - it.window + 1) / kKeysPerBlock;
    it.nblk_tile = last_pos / kKeysPerBlock - it.kb_lo + 1;
    return it;
  };

  for (;;) {
  if (tid == 0) {
    int x = 0, t = -1;
    while (tried < kPrefillQueues) {
      x = (home + tried) & (kPrefillQueues - 1);
      const int cnt = (units - x + kPrefillQueues - 1) / kPrefillQueues;  // units x, x + 2, ...
      if (cnt > 0) {
        // The first ticket of a workgroup on its home queue is its index among that
        // queue's workgroups (hundreds of workgroups asking two counters at the
        // start of a launch wait microseconds for each other); the counters hand
        // out what follows.
        const int home_wgs = ((int)gridDim.x - x + kPrefillQueues - 1) / kPrefillQueues;
        if (first_draw && tried == 0) t = (int)blockIdx.x / kPrefillQueues;
        else t = atomicAdd(a.sched + x, 1) + home_wgs;
        first_draw = false;
        if (t < cnt * tiles * smax) {
          if (smax == 1) break;
          const Item it = item_of(x, t);
          if (it.part * a.kchunk < it.nblk_tile) break;
          t = -1;  // a part past the tile's last block: draw again from the same queue
          continue;
        }
        t = -1;
      }
      ++tried;
    }
    sm_ticket[0] = x;
    sm_ticket[1] = t;
  }
  lds_barrier();  // also: every wave is done with the LDS rings of the previous item
  // (uniform values, kept in scalar registers)
  const int qx = __builtin_amdgcn_readfirstlane(sm_ticket[0]);
  const int ticket = __builtin_amdgcn_readfirstlane(sm_ticket[1]);
  if (ticket < 0) break;  // every queue is empty: the only exit, reached by all workgroups
  const Item it = item_of(qx, ticket);
  const int li = it.li, kvh = it.kvh, hb = it.hb, layer = it.layer, window = it.window, wg_pos0 = it.wg_pos0;
  const int head = kvh * a.group + hb * HPB + (wave % HPB);
  const int my_pos0 = wg_pos0 + (wave / HPB) * kStretch;  // first position of this wave's stretch
  const int my_pos = my_pos0 + n;

  const uint8_t* kplane = a.cache + a.geom.plane_offset(layer, a.seq, kvh, 0);
  const uint8_t* vplane = kplane + a.geom.plane_bytes;

  // Key blocks the workgroup walks (every wave walks all of them; blocks outside
  // a row's range are masked): the tile's, or this part of them.
  const bool split_tile = smax > 1 && it.nblk_tile > a.kchunk;
  const int kb_lo = it.kb_lo + (smax > 1 ? it.part * a.kchunk : 0);
  const int nblk = smax > 1 ? min(a.kchunk, it.nblk_tile - it.part * a.kchunk) : it.nblk_tile;

  // A K or V block travels HBM/L2 -> LDS without touching registers: every
  // wave issues kXfers of the 16 wave-wide 1 KiB transfers of a block; the data
  // of lane l lands at the stage offset of the transfer + 16 * l.
  auto fetch_one = [&](const uint8_t* plane, uint8_t* ring, int i, int t) {
    const int off = (wave + kWaves * t) * 1024;
    const uint8_t* g = plane + (int64_t)(kb_lo + i) * kBlockBytes + lane * 16 + off;
    uint8_t* dst = ring + (i % kStages) * kBlockBytes + off;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                     (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
  };
  auto fetch = [&](const uint8_t* plane, uint8_t* ring, int i) {
#pragma unroll
    for (int t = 0; t < kXfers; ++t) fetch_one(plane, ring, i, t);
  };
  // Ring protocol. Iteration i computes the scores of block i+1 and multiplies
  // the probabilities of block i-1 into the accumulators, so K runs two blocks
  // ahead of V: iteration i requests K block i+3 and V block i+1. The stage of
  // K(i+3) held K(i), read during iteration i-1; the stage of V(i+1) held
  // V(i-2), also read during iteration i-1. At the bottom of iteration i every
  // wave waits for its share of K(i+2) and V(i) (requested one iteration
  // earlier), so after the barrier iteration i+1 finds them resident: every
  // transfer has a whole iteration to land.
  fetch(kplane, sm_k, 0);
  fetch(vplane, sm_v, 0);
  if (nblk > 1) fetch(kplane, sm_k, 1);
  if (nblk > 2) fetch(kplane, sm_k, 2);

  vec8 q0[NJ];  // Q^T operand, filled from LDS once the rows have landed
  // The wave's 32 query rows travel to LDS as whole rows, two per transfer
  // (lanes 0-31 one row, lanes 32-63 the next). Lane l of a transfer asks for the
  // 16-byte piece (l % 32) ^ (row % 16) of its row, so a row's pieces sit
  // permuted in LDS and the reads below, 16 lanes on 16 different rows at a
  // time, fall on 16 different bank groups.
  {
    uint8_t* const qpatch = sm_q + wave * (kStretch * 2 * D);
#pragma unroll
    for (int t = 0; t < kStretch / 2; ++t) {
      const int r = 2 * t + hh;
      const int row = min(my_pos0 - a.q_pos0 + r, a.n - 1);  // rows past the end repeat the last one; never stored
      const uint8_t* g = reinterpret_cast<const uint8_t*>(a.q) +
                         ((((int64_t)li * a.n + row) * a.hq + head) * D) * 2 + ((n ^ (r & 15)) * 16);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                       (__attribute__((address_space(3))) void*)(qpatch + t * 1024), 16, 0, 0);
    }
  }

  f16v acc0[NDP];
#pragma unroll
  for (int i = 0; i < NDP; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc0[i][e] = 0.f;
  float m_run0 = -INFINITY, l_run0 = 0.f;

  // Rare (see kRescaleSlack). The accumulators live in AGPRs (the MFMAs read
  // and write them there); the pins keep their detour through VGPRs inside
  // this block.
  auto rescale = [&](f16v (&acc)[NDP], float alpha) {
#pragma unroll
    for (int dp = 0; dp < NDP; ++dp) asm volatile("" : "+a"(acc[dp]));
#pragma unroll
    for (int dp = 0; dp < NDP; ++dp) acc[dp] *= alpha;
#pragma unroll
    for (int dp = 0; dp < NDP; ++dp) asm volatile("" : "+a"(acc[dp]));
  };

  // Window test in one unsigned comparison: key visible <=> 0 <= pos - key < wlim.
  const unsigned wlim = window > 0 ? (unsigned)window : 0x7fffffffu;
  constexpr int kVAhead = 2;  // channel tiles of V (two operands each) read ahead
  vec8 kk[kAhead];
  h8 vv[kVAhead][2];
  f16v sa, na;                 // scores of the block in the softmax / of the next block
  h8 p_prev[NP], p_cur[NP];  // probabilities of the previous block / of this one
  float bm, alpha, neg_m, lsum;

  // The visibility test rides on the accumulator the scores of a block are summed
  // into: 0 where the key is visible, -inf where not. Blocks in the middle of the
  // causal triangle (every key visible to every row of the wave) start from plain
  // zeros, so only the block on the diagonal and the one at the window's edge pay
  // for the 16 comparisons. With a soft cap the test follows the cap instead.
  const int wave_pos0 = __builtin_amdgcn_readfirstlane(my_pos0);
  auto koff_of = [](int e) { return 16 * ((e >> 2) & 1) + 8 * (e >> 3) + (e & 3); };  // key_of_row(8*(e>>2) + 4*hh + (e&3)) - 4*hh
  auto all_visible = [&](int blk) {
    const int key0 = (kb_lo + blk) * kKeysPerBlock;
    return CAP || (key0 + kKeysPerBlock - 1 <= wave_pos0 && (unsigned)(wave_pos0 + kStretch - 1 - key0) < wlim);
  };
  // the first MFMA of a block's scores, on zeros or on the 0 / -inf tile
  auto first_scores = [&](vec8 k_op, vec8 q_op, int blk) {
    f16v init;
    if (all_visible(blk)) {
#pragma unroll
      for (int e = 0; e < 16; ++e) init[e] = 0.f;
      return E::mfma(k_op, q_op, init);
    }
    const int d0 = my_pos - (kb_lo + blk) * kKeysPerBlock - 4 * hh;
#pragma unroll
    for (int e = 0; e < 16; ++e) init[e] = (unsigned)(d0 - koff_of(e)) < wlim ? 0.f : -INFINITY;
    return E::mfma(k_op, q_op, init);
  };

  // One pipeline step: the vector ALU turns the scores of block i (in sa) into
  // probabilities while the matrix core multiplies the probabilities of block
  // i-1 into the accumulators (PREV) and computes the scores of block i+1
  // (NEXT). The step is cut into one chunk per MFMA; a chunk holds the MFMA,
  // the LDS read of an operand a few MFMAs ahead and a slice of the softmax,
  // and the compiler may not move code across chunk borders, so the three
  // instruction streams stay dealt out evenly. The softmax is a list of 34
  // pieces: 16 x (soft cap and its visibility test if any, running max of one score), the
  // exchange of the max between the two lanes of a query (2 pieces, the LDS
  // crossbar has latency), 16 x (exp2, sum, conversion of one score).
  // A single variant of the loop body keeps the accumulators in place.
  auto step = [&](int i, bool fetch_k, bool fetch_v, auto has_prev, auto has_next) {
    constexpr bool PREV = decltype(has_prev)::value, NEXT = decltype(has_next)::value;
    constexpr int GP = PREV ? NDP * NP : 0;  // chunks with a P.V MFMA
    constexpr int GQ = NEXT ? NJ : 0;        // chunks with a Q.K MFMA
    constexpr int G = GP + GQ > 0 ? GP + GQ : 1;
    constexpr int kPieces = 34;
    const uint8_t* vb = sm_v + ((i + kStages - 1) % kStages) * kBlockBytes + v_off;  // V(i-1)
    const uint8_t* kb = sm_k + ((i + 1) % kStages) * kBlockBytes + k_off;            // K(i+1)
    // pos - key of score e is dist0 - (key offset of e inside the block)
    const int dist0 = my_pos - (kb_lo + i) * kKeysPerBlock - 4 * hh;

    auto piece = [&](auto pc) {
      constexpr int P = decltype(pc)::value;
      if constexpr (P < 16) {
        constexpr int e = P;
        float x = sa[e];
        if constexpr (CAP) {
          // (the cap maps -inf to -cap, so here the test cannot ride on the accumulator)
          x = (softcap * kLog2e) * fast_tanh(x * (a.scale / softcap));
          x = (unsigned)(dist0 - koff_of(e)) < wlim ? x : -INFINITY;
          sa[e] = x;
        }
        bm = e == 0 ? x : fmaxf(bm, x);
      } else if constexpr (P == 16) {
        lsum = __shfl_xor(bm, 32, 64);  // (lsum is free until the sums start)
      } else if constexpr (P == 17) {
        bm = fmaxf(bm, lsum) * c;
        const float m_new = bm > m_run0 + kRescaleSlack ? bm : m_run0;
        alpha = (m_run0 == -INFINITY) ? 1.f : fast_exp2(m_run0 - m_new);
        neg_m = (m_new == -INFINITY) ? 0.f : -m_new;
        m_run0 = m_new;
        lsum = 0.f;
      } else {
        constexpr int e = P - 18;
        sa[e] = fast_exp2(fmaf(sa[e], c, neg_m));
        lsum += sa[e];
        if constexpr (e & 1) {
          // probabilities as MFMA operands
#pragma unroll
          for (int ee = e - 1; ee <= e; ++ee) p_cur[ee >> 3][ee & 7] = (_Float16)sa[ee];
        }
        // Pins: without them the compiler sinks this arithmetic, whose results
        // are only needed in the next iteration, out of the chunk.
        asm volatile("" : "+v"(sa[e]), "+v"(lsum));
        if constexpr ((e & 7) == 7) {
          asm volatile("" : "+v"(p_cur[e >> 3]));
        }
      }
    };

    __builtin_amdgcn_sched_barrier(0);
    if constexpr (PREV) {
#pragma unroll
      for (int dp = 0; dp < kVAhead; ++dp) {
        vv[dp][0] = *reinterpret_cast<const h8*>(vb + dp * 2048);
        vv[dp][1] = *reinterpret_cast<const h8*>(vb + dp * 2048 + 512);
      }
    }
    if constexpr (NEXT && !PREV) {
#pragma unroll
      for (int j = 0; j < kAhead; ++j) kk[j] = *reinterpret_cast<const vec8*>(kb + j * 512);
    }
    // The transfers of K(i+3) and V(i+1) are requested one at a time, spread
    // over the step: issued back to back by all four waves they would queue
    // up in the CU's one vector-memory pipeline and stall the waves in front
    // of their MFMAs.
    constexpr int kXferEvery = G >= 2 * kXfers ? G / (2 * kXfers) : 1;
    static_for<G>([&](auto gc) {
      constexpr int g = decltype(gc)::value;
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (g % kXferEvery == 0 && g / kXferEvery < 2 * kXfers) {
        constexpr int t = g / kXferEvery;
        if (t < kXfers ? fetch_k : fetch_v) {
          if constexpr (t < kXfers) fetch_one(kplane, sm_k, i + 3, t);
          else fetch_one(vplane, sm_v, i + 1, t - kXfers);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (g < GP) {
        constexpr int dp = g / NP, t = g % NP;
        acc0[dp] = mfma32_f16(vv[dp % kVAhead][t & 1], p_prev[t], acc0[dp]);
        if constexpr (t == NP - 1 && dp + kVAhead < NDP) {
          vv[dp % kVAhead][0] = *reinterpret_cast<const h8*>(vb + (dp + kVAhead) * 2048);
          vv[dp % kVAhead][1] = *reinterpret_cast<const h8*>(vb + (dp + kVAhead) * 2048 + 512);
        }
        // the first K operands of the next block, under the last P.V MFMAs
        if constexpr (NEXT && g >= GP - kAhead)
          kk[g - (GP - kAhead)] = *reinterpret_cast<const vec8*>(kb + (g - (GP - kAhead)) * 512);
      } else if constexpr (g < GP + GQ) {
        constexpr int j = g - GP;
        if constexpr (j == 0) na = first_scores(kk[0], q0[0], i + 1);
        else na = E::mfma(kk[j % kAhead], q0[j], na);
        if constexpr (j + kAhead < NJ) kk[j % kAhead] = *reinterpret_cast<const vec8*>(kb + (j + kAhead) * 512);
      }
      static_for<kPieces>([&](auto pc) {
        constexpr int P = decltype(pc)::value;
        if constexpr (P * G / kPieces == g) piece(pc);
      });
    });
    __builtin_amdgcn_sched_barrier(0);
    l_run0 = l_run0 * alpha + lsum;
  };

  __builtin_amdgcn_s_waitcnt(0);
  lds_barrier();  // the first blocks are resident

  // Q^T operand in registers: slice j of lane (n, hh) holds channels
  // 16*j + 8*hh .. +7 of the lane's query = piece 2*j + hh of row n.
  {
    const uint8_t* const qrow = sm_q + wave * (kStretch * 2 * D) + n * (2 * D);
#pragma unroll
    for (int j = 0; j < NJ; ++j) q0[j] = *reinterpret_cast<const vec8*>(qrow + (((2 * j + hh) ^ (n & 15)) * 16));
  }

  constexpr std::true_type yes{};
  constexpr std::false_type no{};
  {  // scores of block 0
    const uint8_t* kb = sm_k + k_off;
#pragma unroll
    for (int j = 0; j < kAhead; ++j) kk[j] = *reinterpret_cast<const vec8*>(kb + j * 512);
    static_for<NJ>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (j == 0) sa = first_scores(kk[0], q0[0], 0);
      else sa = E::mfma(kk[j % kAhead], q0[j], sa);
      if constexpr (j + kAhead < NJ) kk[j % kAhead] = *reinterpret_cast<const vec8*>(kb + (j + kAhead) * 512);
    });
    __builtin_amdgcn_sched_barrier(0);
  }
  lds_barrier();  // every wave has read K block 0: iteration 0 sends a new block into its stage
  auto iteration = [&](int i, auto has_prev, auto has_next) {
    const bool fetch_k = i + 3 < nblk, fetch_v = i + 1 < nblk;
    // The accumulators stay in the AGPR half of the register file; scores,
    // operands and Q^T live in the VGPR half.
#pragma unroll
    for (int dp = 0; dp < NDP; ++dp) asm volatile("" : "+a"(acc0[dp]));
    step(i, fetch_k, fetch_v, has_prev, has_next);
    if (__any(alpha != 1.f)) rescale(acc0, alpha);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < NP; ++t) p_prev[t] = p_cur[t];
    if constexpr (decltype(has_next)::value) sa = na;

    // this wave's shares of K(i+2) and V(i) have landed; what was requested in
    // this iteration may still be in flight
    if (fetch_k && fetch_v) __builtin_amdgcn_s_waitcnt(kWaitVm8);
    else if (fetch_k || fetch_v) __builtin_amdgcn_s_waitcnt(kWaitVm4);
    else __builtin_amdgcn_s_waitcnt(kWaitVm0);
    lds_barrier();
  };
  if (nblk == 1) {
    iteration(0, no, no);
  } else {
    iteration(0, no, yes);
    for (int i = 1; i < nblk - 1; ++i) iteration(i, yes, yes);
    iteration(nblk - 1, yes, no);
  }
  {  // the last block's probabilities
    const uint8_t* vb = sm_v + ((nblk - 1) % kStages) * kBlockBytes + v_off;
#pragma unroll
    for (int dp = 0; dp < kVAhead; ++dp) {
      vv[dp][0] = *reinterpret_cast<const h8*>(vb + dp * 2048);
      vv[dp][1] = *reinterpret_cast<const h8*>(vb + dp * 2048 + 512);
    }
    static_for<NDP * NP>([&](auto gc) {
      constexpr int g = decltype(gc)::value;
      constexpr int dp = g / NP, t = g % NP;
      __builtin_amdgcn_sched_barrier(0);
      acc0[dp] = mfma32_f16(vv[dp % kVAhead][t & 1], p_prev[t], acc0[dp]);
      if constexpr (t == NP - 1 && dp + kVAhead < NDP) {
        vv[dp % kVAhead][0] = *reinterpret_cast<const h8*>(vb + (dp + kVAhead) * 2048);
        vv[dp % kVAhead][1] = *reinterpret_cast<const h8*>(vb + (dp + kVAhead) * 2048 + 512);
      }
    });
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- normalise and store. Lane (n, hh) holds channels 32*dp + 8*a + 4*hh + b of
  // query n: written from there, one store instruction would touch 32 rows with
  // 16 bytes each. The rows go through LDS instead (the rings are idle now; every
  // wave has its own patch, rows padded to 528 bytes against bank conflicts) and
  // leave as whole 512-byte rows, two per store instruction.
  lds_barrier();  // every wave is done with the last V block
  if (split_tile) {
    // A part of a split tile: the unnormalised accumulators (fp32) and the row's
    // (reference max, sum) go to the workspace, again as whole rows through LDS.
    // The patches of waves 2 and 3 start behind the ticket words, which thread 0
    // may rewrite for the next item while they are still being read.
    constexpr int kRowStrideF = 4 * D + 16;
    static_assert(2 * (kStretch * kRowStrideF) <= (kStages + kStages - 1) * kBlockBytes, "patches 0, 1 before the ticket");
    uint8_t* const patch = smem + wave * (kStretch * kRowStrideF) + (wave >= 2 ? 16384 : 0);
    const float l_tot = wave_xor_add(l_run0, 32);
#pragma unroll
    for (int dp = 0; dp < NDP; ++dp) {
#pragma unroll
      for (int aa = 0; aa < 4; ++aa) {
        f4 o;
#pragma unroll
        for (int b = 0; b < 4; ++b) o[b] = acc0[dp][4 * aa + b];
        *reinterpret_cast<f4*>(patch + n * kRowStrideF + (32 * dp + 8 * aa + 4 * hh) * 4) = o;
      }
    }
    const int row_base = my_pos0 - a.q_pos0;
    if (hh == 0 && row_base + n < a.n) {
      const int64_t slot = (((int64_t)li * a.n + row_base + n) * a.hq + head) * smax + it.part;
      *reinterpret_cast<float2*>(a.ws_ml + slot * 2) = float2{m_run0, l_tot};
    }
#pragma unroll 4
    for (int r = 0; r < kStretch; ++r) {
      const u4 w = *reinterpret_cast<const u4*>(patch + r * kRowStrideF + lane * 16);
      const int row = row_base + r;
      if (row < a.n) {
        const int64_t slot = (((int64_t)li * a.n + row) * a.hq + head) * smax + it.part;
        *reinterpret_cast<u4*>(a.ws_acc + slot * D + lane * 4) = w;
      }
    }
  } else if constexpr (OUT == kF32) {
    // float32 rows: the same route as the parts of a split tile, normalised, to the output
    constexpr int kRowStrideF = 4 * D + 16;
    uint8_t* const patch = smem + wave * (kStretch * kRowStrideF) + (wave >= 2 ? 16384 : 0);
    const float l_tot = wave_xor_add(l_run0, 32);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
#pragma unroll
    for (int dp = 0; dp < NDP; ++dp) {
#pragma unroll
      for (int aa = 0; aa < 4; ++aa) {
        f4 o;
#pragma unroll
        for (int b = 0; b < 4; ++b) o[b] = acc0[dp][4 * aa + b] * inv;
        *reinterpret_cast<f4*>(patch + n * kRowStrideF + (32 * dp + 8 * aa + 4 * hh) * 4) = o;
      }
    }
    const int row_base = my_pos0 - a.q_pos0;
#pragma unroll 4
    for (int r = 0; r < kStretch; ++r) {
      const u4 w = *reinterpret_cast<const u4*>(patch + r * kRowStrideF + lane * 16);
      const int row = row_base + r;
      if (row < a.n) {
        float* orow = reinterpret_cast<float*>(a.out) + (((int64_t)li * a.n + row) * a.hq + head) * D;
        *reinterpret_cast<u4*>(orow + lane * 4) = w;
      }
    }
  } else {
    constexpr int kRowStride = 2 * D + 16;
    uint8_t* const patch = smem + wave * (kStretch * kRowStride);
    const float l_tot = wave_xor_add(l_run0, 32);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
#pragma unroll
    for (int dp = 0; dp < NDP; ++dp) {
#pragma unroll
      for (int aa = 0; aa < 4; ++aa) {
        out_t o[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) o[b] = (out_t)(acc0[dp][4 * aa + b] * inv);
        *reinterpret_cast<u2*>(patch + n * kRowStride + (32 * dp + 8 * aa + 4 * hh) * 2) = *reinterpret_cast<const u2*>(o);
      }
    }
    // (the patch is private to the wave and LDS operations of a wave stay in order: no barrier)
    const int row_base = my_pos0 - a.q_pos0;
    const int chunk = lane & 31;
#pragma unroll
    for (int j = 0; j < kStretch / 2; ++j) {
      const int r = 2 * j + hh;
      const u4 w = *reinterpret_cast<const u4*>(patch + r * kRowStride + chunk * 16);
      const int row = row_base + r;
      if (row < a.n) {
        out_t* orow = reinterpret_cast<out_t*>(a.out) + (((int64_t)li * a.n + row) * a.hq + head) * D;
        *reinterpret_cast<u4*>(orow + chunk * 8) = w;
      }
    }
  }
  }  // next work item

  // The last workgroup to get here (all others have drawn their final, failed
  // tickets) puts the counters back to zero for the next launch.
  if (tid == 0) {
    const int done = atomicAdd(a.sched + kPrefillQueues, 1);
    if (done == (int)gridDim.x - 1)
      for (int i = 0; i < kPrefillSchedInts; ++i) atomicExch(a.sched + i, 0);
  }
}

// ---------------------------------------------------------------------------
// The same work on v_mfma_f32_16x16x32 with two workgroups per compute unit:
// four waves of 32 query positions (two sub-tiles of 16) each, S^T tiles of 16
// keys x 16 queries, O^T tiles of 16 channels x 16 queries, operands read
// straight in the cache planes' order (the layout the decode kernel uses), every
// operand read from LDS feeding two MFMAs (one per sub-tile). A workgroup needs
// 80 KiB of LDS (K ring of three blocks, V ring of two) and 256 registers per
// wave, so two workgroups share a CU, two waves a SIMD: they work on different
// items and fill each other's stalls. The probabilities enter P.V as IEEE half
// operands for both cache types (the V planes of a bfloat16 cache hold half values,
// attn_params.h), so P.V always runs on the fp16 MFMA.
// (Measured and not kept: the same loop software-pipelined inside the wave - scores of
// the next half-block and the exponentials of the current one dealt out in one
// instruction stream, operand reads with counted waits, one continuous read stream
// across the phases - is 3 to 10 % slower on the 26-layer launch: the exponentials
// were already hidden by the other wave of the SIMD, and what the hand-placed order
// adds in scheduling regions and waits costs more than the phases' ramps it removes.)
// A read of read-only, wave-uniform data through the scalar cache (constant address space).
__device__ __forceinline__ int32_t scalar_load(const int32_t* p) {
  return *reinterpret_cast<const __attribute__((address_space(4))) int32_t*>(reinterpret_cast<uintptr_t>(p));
}

constexpr int kWaves16 = 4;
constexpr int kRows16 = 16;
constexpr int kSub16 = 2;       // sub-tiles of 16 query positions per wave
constexpr int kKStages16 = 3, kVStages16 = 2;
constexpr float kNoKeyYet = -1e30f;  // running reference of a query that has not met a visible key yet
// LDS operand reads in flight ahead of their MFMAs, scores and P.V (four each would not fit in 256 registers)
constexpr int kOpAhead = 3;
constexpr int kOpAheadV = 4;

template <int D>
constexpr int prefill16_lds_bytes() { return (kKStages16 + kVStages16) * 64 * D; }  // 80 KiB: two workgroups fill a CU's LDS

template <int DT, int OUT, int D, int HPB, bool CAP>
__global__ void __launch_bounds__(kWaves16 * 64, 2) prefill_attn16_kernel(const PrefillArgs a) {
  using E = El<DT>;
  using elem_t = typename E::type;
  using out_t = typename OutEl<OUT>::type;
  using vec8 = typename E::vec8;
  constexpr int PT = 4 / HPB;
  constexpr int NJ = D / 32;  // 32-channel steps of the QK^T product
  constexpr int NL = D / 16;  // 16-channel tiles of O^T
  constexpr int kBlockBytes = 64 * D;
  constexpr int kXfers = 16 / kWaves16;
  auto mfma = [](vec8 x, vec8 y, f4 z) {
    if constexpr (DT == kF16) return mfma16_f16(x, y, z);
    else return mfma16_bf16(x, y, z);
  };

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint8_t* const sm_k = smem;
  uint8_t* const sm_v = smem + kKStages16 * kBlockBytes;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int hblocks = a.group / HPB;
  const int per_layer = a.geom.hkv * hblocks;
  const int smax = a.kchunk > 0 ? a.smax : 1;
  const float softcap = a.softcap;
  const float c = CAP ? 1.f : a.scale * kLog2e;
  const int pos_end = a.q_pos0 + a.n;

  // This workgroup's items, in the order the host planned them (no queue, no ticket: every wave reads the list).
  const int32_t* const plan_items = a.plan + gridDim.x + 1;
  const int item_end = scalar_load(a.plan + blockIdx.x + 1);

  struct Item { int li, kvh, layer, window, wg_pos0, part, head, my_pos0, kb0, nblk; bool split; };
  auto item_at = [&](int idx) {
    Item it;
    // (read through the scalar cache: a vector load here would make every item wait for all memory
    // operations under way, the previous item's stores included)
    const int u = scalar_load(plan_items + 2 * idx);
    const int w1 = scalar_load(plan_items + 2 * idx + 1);
    const int tile = w1 & 0xFFFFF;
    it.part = w1 >> 20;
    it.li = u / per_layer;
    const int rem = u - it.li * per_layer;
    it.kvh = rem / hblocks;
    const int hb = rem - it.kvh * hblocks;
    it.layer = a.layer_begin + it.li;
    it.window = scalar_load(a.layer_window + it.layer);
    it.wg_pos0 = a.q_pos0 + tile * (kStretch * PT);
    const int last_pos = min(it.wg_pos0 + kStretch * PT, pos_end) - 1;
    int kb_lo = 0;
    if (it.window > 0 && it.wg_pos0 - it.window + 1 > 0) kb_lo = (it.wg_pos0 - it.window + 1) / kKeysPerBlock;
    const int nblk_tile = last_pos / kKeysPerBlock - kb_lo + 1;
    it.split = smax > 1 && nblk_tile > a.kchunk;
    it.kb0 = kb_lo + (smax > 1 ? it.part * a.kchunk : 0);
    it.nblk = smax > 1 ? min(a.kchunk, nblk_tile - it.part * a.kchunk) : nblk_tile;
    it.head = it.kvh * a.group + hb * HPB + (wave % HPB);
    it.my_pos0 = it.wg_pos0 + (wave / HPB) * kStretch;  // first of the wave's 32 positions
    return it;
  };
  auto k_plane = [&](const Item& it) { return a.cache + a.geom.plane_offset(it.layer, a.seq, it.kvh, 0); };
  // One 16 KiB block from a cache plane into a ring stage: every wave moves four 1 KiB pieces. The source is
  // a wave-uniform address (scalar registers) plus the lane's 16-byte slot, so that the transfers need no
  // vector arithmetic and no address registers of their own.
  const uint32_t lane_slot = (uint32_t)lane * 16u;
  auto fetch = [&](const uint8_t* plane, int block, uint8_t* stage) {
    const uint8_t* const base = plane + (int64_t)block * kBlockBytes + wave * 1024;
#pragma unroll
    for (int t = 0; t < kXfers; ++t) {
      const uint8_t* src = base + t * (kWaves16 * 1024) + lane_slot;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(stage + (wave + kWaves16 * t) * 1024),
                                       16, 0, 0);
    }
  };
  // Q^T operands: lane (n, g) holds, for sub-tile u and step j, channels 32 j + 8 g .. + 7 of query my_pos0 + 16 u + n.
  // They are loaded behind the compiler's back (it would wait for ALL memory operations under way before the
  // first use of a register loaded across the item loop): q_wait() below is the matching wait.
  vec8 q[kSub16][NJ];
  static_assert(NJ == 8, "load_q spells out eight steps");
#define MI355_LOAD_Q(u, j) \
  asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "+v"(q[u][j]) : "v"(qrow), "n"(64 * (j)) : "memory")
  auto load_q = [&](const Item& it) {
#pragma unroll
    for (int u = 0; u < kSub16; ++u) {
      const int row = min(it.my_pos0 + kRows16 * u + n - a.q_pos0, a.n - 1);  // rows past the end repeat the last one; never stored
      const elem_t* qrow = reinterpret_cast<const elem_t*>(a.q) + (((int64_t)it.li * a.n + row) * a.hq + it.head) * D + 8 * g;
      MI355_LOAD_Q(u, 0); MI355_LOAD_Q(u, 1); MI355_LOAD_Q(u, 2); MI355_LOAD_Q(u, 3);
      MI355_LOAD_Q(u, 4); MI355_LOAD_Q(u, 5); MI355_LOAD_Q(u, 6); MI355_LOAD_Q(u, 7);
    }
  };
#undef MI355_LOAD_Q
  // After a wait that covers the query loads: from here on the compiler may read q.
  auto q_ready = [&]() {
#pragma unroll
    for (int u = 0; u < kSub16; ++u)
#pragma unroll
      for (int j = 0; j < NJ; ++j) asm volatile("" : "+v"(q[u][j]));
  };

  // The key blocks of all items of this workgroup form one stream through the rings: block s of the stream
  // sits in K stage s % 3 and V stage s % 2, whatever item it belongs to. While block s is worked on, K(s + 2)
  // is asked for after the scores (its stage held K(s - 1), last read before the barrier of block s - 1) and
  // V(s + 1) after the barrier of block s (its stage held V(s - 1), last read before that barrier) - also
  // when those blocks belong to the next item, whose first blocks, and whose queries (loaded into the
  // registers the last scores have just freed), are therefore under way while this item's last P.V and
  // its store run. Nothing waits and no barrier stands between two items.
  int idx = scalar_load(a.plan + blockIdx.x);
  if (idx >= item_end) return;
  Item it = item_at(idx);
  int ks = 0;        // K stage of the block being worked on
  int kfs = 0;       // K stage the next block asked for goes to
  int vs = 0;        // V stage of the block being worked on
  int kreq = 0;      // K blocks of the current item already asked for when it starts (0 .. 2)
  bool v_asked = false, q_loaded = false, k0_landed = false;
  int stores_after_q = 0;  // store instructions certainly issued after the latest query loads (never more than were)

  for (;;) {
    const bool has_next = idx + 1 < item_end;
    const Item nx = item_at(has_next ? idx + 1 : idx);
    const int nblk = it.nblk;
    const int lim = nblk + (has_next ? min(2, nx.nblk) : 0);  // stream blocks (counted from this item's first) that may be asked for
    const uint8_t* const kplane = k_plane(it);
    const uint8_t* const vplane = kplane + a.geom.plane_bytes;
    const uint8_t* const kplane_nx = k_plane(nx);
    auto ask_k = [&](int r) {  // r: stream block counted from this item's first
      if (r < nblk) fetch(kplane, it.kb0 + r, sm_k + kfs * kBlockBytes);
      else fetch(kplane_nx, nx.kb0 + (r - nblk), sm_k + kfs * kBlockBytes);
      kfs = kfs == kKStages16 - 1 ? 0 : kfs + 1;
    };
    // What the previous item has not asked for already: everything, for a workgroup's first item, whose queries
    // and first K block go first, so that its first scores need not wait for V(0) and K(1) as well (at the start
    // of a launch every workgroup asks at once and the loads are served at the rate of the memory).
    const bool first_item = !q_loaded;
    if (first_item) load_q(it);
    int req = kreq;
    if (req < 1) { ask_k(0); req = 1; }
    int after_k0 = 0;  // blocks asked for after K(0)
    if (!v_asked) { fetch(vplane, it.kb0, sm_v + vs * kBlockBytes); ++after_k0; }
    if (req < 2 && nblk > 1) { ask_k(1); req = 2; ++after_k0; }
    if (!k0_landed) {
      // K(0) has to be there for everybody: a workgroup's first item, or one after a one-block item, whose K(0)
      // was asked for only during that item's single block (then everything is waited for: rare).
      if (first_item && after_k0 == 2) __builtin_amdgcn_s_waitcnt(wait_vm(2 * kXfers));
      else if (first_item && after_k0 == 1) __builtin_amdgcn_s_waitcnt(wait_vm(kXfers));
      else __builtin_amdgcn_s_waitcnt(0x0F70);
      lds_barrier();
    } else {
      // The queries were loaded during the previous item's last P.V; since then: V(0) of this item (one
      // block's transfers) and that item's stores. Memory operations complete in the order issued.
      if (stores_after_q >= 2 * NL) __builtin_amdgcn_s_waitcnt(wait_vm(kXfers + 2 * NL));
      else if (stores_after_q >= NL) __builtin_amdgcn_s_waitcnt(wait_vm(kXfers + NL));
      else if (stores_after_q >= NL / 2) __builtin_amdgcn_s_waitcnt(wait_vm(kXfers + NL / 2));
      else __builtin_amdgcn_s_waitcnt(wait_vm(kXfers));
    }
    q_ready();

    f4 acc[kSub16][NL];
#pragma unroll
    for (int u = 0; u < kSub16; ++u)
#pragma unroll
      for (int i = 0; i < NL; ++i) acc[u][i] = f4{0.f, 0.f, 0.f, 0.f};
    float m_run[kSub16], l_run[kSub16];
#pragma unroll
    for (int u = 0; u < kSub16; ++u) { m_run[u] = kNoKeyYet; l_run[u] = 0.f; }
    const int window = it.window, my_pos0 = it.my_pos0;
    const unsigned wlim = window > 0 ? (unsigned)window : 0x7fffffffu;
    const int wave_pos0 = __builtin_amdgcn_readfirstlane(my_pos0);

    for (int i = 0; i < nblk; ++i) {
      const uint8_t* kb = sm_k + ks * kBlockBytes + lane * 16;
      const uint8_t* vb = sm_v + vs * kBlockBytes + lane * 16;
      f4 sc[kSub16][2];
#pragma unroll
      for (int u = 0; u < kSub16; ++u)
#pragma unroll
        for (int T = 0; T < 2; ++T) sc[u][T] = f4{0.f, 0.f, 0.f, 0.f};
      {
        // operand reads run kOpAhead steps ahead of the MFMAs that use them (an LDS read takes longer
        // than the two MFMAs of a step)
        auto k_at = [&](int step) { return *reinterpret_cast<const vec8*>(kb + (step & 1) * (16 * D * 2) + (step >> 1) * 1024); };
        vec8 kop[kOpAhead];
#pragma unroll
        for (int st = 0; st < kOpAhead; ++st) kop[st] = k_at(st);
#pragma unroll
        for (int st = 0; st < 2 * NJ; ++st) {
          const int j = st >> 1, T = st & 1;
#pragma unroll
          for (int u = 0; u < kSub16; ++u) sc[u][T] = mfma(kop[st % kOpAhead], q[u][j], sc[u][T]);
          if (st + kOpAhead < 2 * NJ) kop[st % kOpAhead] = k_at(st + kOpAhead);
        }
        // keep that order: kOpAhead reads, then two MFMAs and one read per step (left alone, the scheduler
        // saves registers by reading every operand right before its use, and each step waits for LDS)
        __builtin_amdgcn_sched_group_barrier(0x100, kOpAhead, 0);
#pragma unroll
        for (int st = 0; st < 2 * NJ; ++st) {
          __builtin_amdgcn_sched_group_barrier(0x008, kSub16, 0);
          if (st + kOpAhead < 2 * NJ) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
      }
      // K two blocks ahead in the stream (normally one block; two after a one-block item's only scores)
      int asked = 0;
      if (req <= i + 2 && req < lim) { ask_k(req); ++req; ++asked; }
      if (req <= i + 2 && req < lim) { ask_k(req); ++req; ++asked; }
      // score sc[u][T][e]: key key0 + 16 T + 4 g + e against query my_pos0 + 16 u + n
      const int key0 = (it.kb0 + i) * kKeysPerBlock;
      const bool all_vis = key0 + kKeysPerBlock - 1 <= wave_pos0 && (unsigned)(wave_pos0 + kStretch - 1 - key0) < wlim;
      if constexpr (CAP) {
#pragma unroll
        for (int u = 0; u < kSub16; ++u)
#pragma unroll
          for (int T = 0; T < 2; ++T)
#pragma unroll
            for (int e = 0; e < 4; ++e) sc[u][T][e] = (softcap * kLog2e) * fast_tanh(sc[u][T][e] * (a.scale / softcap));
      }
      if (!all_vis) {
        // Only the block on the diagonal and the one at the window's edge hold keys that some query of the wave
        // does not see. (A branch of its own: as part of the loop below the compiler turns the test into
        // selects that every block pays for, 35 of ~130 vector-ALU instructions.)
        asm volatile("; block with masked keys" ::: "memory");
#pragma unroll
        for (int u = 0; u < kSub16; ++u) {
          const int my_pos = my_pos0 + kRows16 * u + n;
#pragma unroll
          for (int T = 0; T < 2; ++T)
#pragma unroll
            for (int e = 0; e < 4; ++e)
              sc[u][T][e] = (unsigned)(my_pos - (key0 + 16 * T + 4 * g + e)) < wlim ? sc[u][T][e] : -INFINITY;
        }
      }
      h8 p_hi[kSub16];
#pragma unroll
      for (int u = 0; u < kSub16; ++u) {
        float bm = -INFINITY;
#pragma unroll
        for (int T = 0; T < 2; ++T)
#pragma unroll
          for (int e = 0; e < 4; ++e) bm = fmaxf(bm, sc[u][T][e]);
        bm *= c;
        // The four lanes of a query compare notes only when one of them has seen a score that
        // exceeds the reference by more than the slack: rare after the first blocks.
        if (__any(bm > m_run[u] + kRescaleSlack)) {
          bm = wave_xor_max(bm, 16);
          bm = wave_xor_max(bm, 32);
        }
        const float m_new = bm > m_run[u] + kRescaleSlack ? bm : m_run[u];
        // (the reference starts at a finite kNoKeyYet, not at -inf: exp2(m_run - m_new) is then 0 when the first
        // visible key arrives and 1 while none has, with no special cases; masked scores are -inf, so they weigh 0
        // against either)
        const float alpha = fast_exp2(m_run[u] - m_new);
        const float neg_m = -m_new;
        m_run[u] = m_new;
        float lsum = 0.f;
        {
#pragma unroll
          for (int T = 0; T < 2; ++T)
#pragma unroll
            for (int e = 0; e < 4; ++e) p_hi[u][4 * T + e] = (_Float16)fast_exp2(fmaf(sc[u][T][e], c, neg_m));
          // the row sum is taken over the probabilities as P.V will see them (rounded to half), two per
          // instruction, accumulated in float32
          using h2 = __attribute__((ext_vector_type(2))) _Float16;
          const h2 ones = {(_Float16)1.f, (_Float16)1.f};
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            const h2 pair = {p_hi[u][2 * w], p_hi[u][2 * w + 1]};
            lsum = __builtin_amdgcn_fdot2(pair, ones, lsum, false);
          }
        }
        l_run[u] = l_run[u] * alpha + lsum;
        if (__any(alpha != 1.f)) {
#pragma unroll
          for (int db = 0; db < NL; ++db) acc[u][db] *= alpha;
        }
      }
      // This wave's share of V(i) and of K(i + 1) has landed; what was asked for after these scores may be under way.
      if (asked == 0) __builtin_amdgcn_s_waitcnt(0x0F70);
      else if (asked == 1) __builtin_amdgcn_s_waitcnt(wait_vm(kXfers));
      else __builtin_amdgcn_s_waitcnt(wait_vm(2 * kXfers));
      lds_barrier();
      const bool last = i + 1 == nblk;
      if (!last) fetch(vplane, it.kb0 + i + 1, sm_v + (vs ^ 1) * kBlockBytes);
      else if (has_next) {
        load_q(nx);  // the scores of this item are done with the query registers
        fetch(kplane_nx + a.geom.plane_bytes, nx.kb0, sm_v + (vs ^ 1) * kBlockBytes);
      }
      {
        h8 vop[kOpAheadV];
#pragma unroll
        for (int st = 0; st < kOpAheadV; ++st) vop[st] = *reinterpret_cast<const h8*>(vb + st * 1024);
#pragma unroll
        for (int db = 0; db < NL; ++db) {
#pragma unroll
          for (int u = 0; u < kSub16; ++u) {
            acc[u][db] = mfma16_f16(vop[db % kOpAheadV], p_hi[u], acc[u][db]);
          }
          if (db + kOpAheadV < NL) vop[db % kOpAheadV] = *reinterpret_cast<const h8*>(vb + (db + kOpAheadV) * 1024);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, kOpAheadV, 0);
#pragma unroll
        for (int db = 0; db < NL; ++db) {
          __builtin_amdgcn_sched_group_barrier(0x008, kSub16, 0);
          if (db + kOpAheadV < NL) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
      }
      ks = ks == kKStages16 - 1 ? 0 : ks + 1;
      vs ^= 1;
      // (no barrier here: the next one, in the middle of the stream's next block, is passed only when every
      // wave is done with this P.V, and V(i)'s stage is written no earlier than that)
    }

    // ---- store, straight from the registers (the rings belong to the stream): lane (n, g) holds channels
    // 16 db + 4 g .. + 3 of query my_pos0 + 16 u + n
    stores_after_q = 0;
#pragma unroll
    for (int u = 0; u < kSub16; ++u) {
      float l_tot = wave_xor_add(l_run[u], 16);
      l_tot = wave_xor_add(l_tot, 32);
      const int row = my_pos0 + kRows16 * u + n - a.q_pos0;
      // (lane n = 0 has a row to store: the wave issues the sub-tile's store instructions, NL / 2 of 16 bytes, NL
      // for float32 output, or NL + 1 for a part of a split tile)
      if (wave_pos0 + kRows16 * u - a.q_pos0 < a.n) stores_after_q += (it.split || OUT == kF32) ? NL : NL / 2;
      if (row < a.n) {
        if (it.split) {
          const int64_t slot = (((int64_t)it.li * a.n + row) * a.hq + it.head) * smax + it.part;
          float* prow = a.ws_acc + slot * D + 4 * g;
#pragma unroll
          for (int db = 0; db < NL; ++db) *reinterpret_cast<f4*>(prow + 16 * db) = acc[u][db];
          if (g == 0) *reinterpret_cast<float2*>(a.ws_ml + slot * 2) = float2{m_run[u], l_tot};
        }
      }
      if (!it.split) {
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        if constexpr (OUT == kF32) {
          // float32 output: a lane's four channels of a tile are 16 bytes already, the four lanes of a query
          // 64 consecutive bytes per store instruction
          float* orow = reinterpret_cast<float*>(a.out) + (((int64_t)it.li * a.n + row) * a.hq + it.head) * D + 4 * g;
#pragma unroll
          for (int db = 0; db < NL; ++db) {
            const f4 o = acc[u][db] * inv;
            if (row < a.n) *reinterpret_cast<f4*>(orow + 16 * db) = o;
          }
        } else {
          // Pairs of channel tiles trade halves between the lanes g and g ^ 1 of a query (v_permlane16_swap), so
          // that a lane ends up with 8 consecutive channels, 16 bytes, and the four lanes of a query with 64
          // consecutive bytes per store instruction (8-byte pieces straight from the MFMA layout cost four
          // times the write requests). Every lane takes part in the trade; only rows that exist are stored.
          uint32_t packed[NL][2];
#pragma unroll
          for (int db = 0; db < NL; ++db) {
            out_t o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (out_t)(acc[u][db][e] * inv);
            const u2 w = *reinterpret_cast<const u2*>(o);
            packed[db][0] = w[0];
            packed[db][1] = w[1];
          }
          // lanes g = 0, 2 keep tile 2k (channels 32k + 4g .. + 7), lanes g = 1, 3 tile 2k + 1 (32k + 16 + 4(g - 1) .. + 7)
          const int first = (g & 1) * 16 + (g >> 1) * 8;
          out_t* orow = reinterpret_cast<out_t*>(a.out) + (((int64_t)it.li * a.n + row) * a.hq + it.head) * D + first;
#pragma unroll
          for (int k = 0; k < NL / 2; ++k) {
            const auto lo = __builtin_amdgcn_permlane16_swap(packed[2 * k][0], packed[2 * k + 1][0], false, false);
            const auto hi = __builtin_amdgcn_permlane16_swap(packed[2 * k][1], packed[2 * k + 1][1], false, false);
            const u4 w = {lo[0], hi[0], lo[1], hi[1]};
            if (row < a.n) *reinterpret_cast<u4*>(orow + 32 * k) = w;
          }
        }
      }
    }

    if (!has_next) break;
    kreq = req - nblk;
    v_asked = true;
    q_loaded = true;
    k0_landed = nblk >= 2;  // then K(0) of the next item was asked for a block before this item's last barrier
    it = nx;
    ++idx;
  }
}

// Combines the parts of split tiles: grid (query head, row, layer), one thread
// per channel. Rows of tiles that were not split have been written by the
// attention kernel itself.
template <int OUT, int D>
__global__ void __launch_bounds__(D) prefill_merge_kernel(const PrefillArgs a, int rows_per_tile) {
  using elem_t = typename OutEl<OUT>::type;
  const int head = blockIdx.x, row = blockIdx.y, li = blockIdx.z, d = threadIdx.x;
  const int window = a.layer_window[a.layer_begin + li];
  const int wg_pos0 = a.q_pos0 + (row / rows_per_tile) * rows_per_tile;
  const int last_pos = min(wg_pos0 + rows_per_tile, a.q_pos0 + a.n) - 1;
  int kb_lo = 0;
  if (window > 0 && wg_pos0 - window + 1 > 0) kb_lo = (wg_pos0 - window + 1) / kKeysPerBlock;
  const int nblk = last_pos / kKeysPerBlock - kb_lo + 1;
  if (nblk <= a.kchunk) return;
  const int parts = (nblk + a.kchunk - 1) / a.kchunk;
  const int64_t slot0 = (((int64_t)li * a.n + row) * a.hq + head) * a.smax;
  float M = -INFINITY;
  for (int p = 0; p < parts; ++p) M = fmaxf(M, a.ws_ml[(slot0 + p) * 2]);
  float A = 0.f, L = 0.f;
  for (int p = 0; p < parts; ++p) {
    const float m = a.ws_ml[(slot0 + p) * 2];
    const float wgt = m == -INFINITY ? 0.f : fast_exp2(m - M);  // (a part none of whose keys the row sees)
    A += wgt * a.ws_acc[(slot0 + p) * D + d];
    L += wgt * a.ws_ml[(slot0 + p) * 2 + 1];
  }
  reinterpret_cast<elem_t*>(a.out)[(((int64_t)li * a.n + row) * a.hq + head) * D + d] = (elem_t)(L > 0.f ? A / L : 0.f);
}

// float32 queries rounded (to nearest even) to the element type of the cache, 8 per thread: what the
// matrix cores take. One pass over the call's query rows in front of the attention kernel.
template <int DT>
__global__ void __launch_bounds__(256) convert_queries_kernel(const float* __restrict__ src, void* __restrict__ dst, int64_t n8) {
  using vec8 = typename El<DT>::vec8;
  using elem_t = typename El<DT>::type;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n8) return;
  const f4 x0 = *reinterpret_cast<const f4*>(src + 8 * i), x1 = *reinterpret_cast<const f4*>(src + 8 * i + 4);
  vec8 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) { o[e] = (elem_t)x0[e]; o[4 + e] = (elem_t)x1[e]; }
  reinterpret_cast<vec8*>(dst)[i] = o;
}

template <int DT, int OUT, int D, int HPB, bool CAP>
hipError_t launch_variant(const PrefillArgs& a, dim3 grid, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  constexpr int kLds = prefill_lds_bytes<D>();
  // more than 64 KiB of LDS has to be requested once per kernel (callers on several threads may both
  // make the request; it is idempotent)
  static std::atomic<bool> configured{false};
  if (!configured.load(std::memory_order_acquire)) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_attn_kernel<DT, OUT, D, HPB, CAP>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess) return e;
    configured.store(true, std::memory_order_release);
  }
  // ev0/ev1 ride on the dispatch: the kernel's own begin / end timestamps
  hipExtLaunchKernelGGL((prefill_attn_kernel<DT, OUT, D, HPB, CAP>), grid, dim3(kWaves * 64), kLds, stream, ev0, ev1, 0,
                        a);
  return hipGetLastError();
}

template <int DT, int OUT, int D, int HPB, bool CAP>
hipError_t launch_variant16(const PrefillArgs& a, dim3 grid, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  constexpr int kLds = prefill16_lds_bytes<D>();
  static std::atomic<bool> configured{false};
  if (!configured.load(std::memory_order_acquire)) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_attn16_kernel<DT, OUT, D, HPB, CAP>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess) return e;
    configured.store(true, std::memory_order_release);
  }
  hipExtLaunchKernelGGL((prefill_attn16_kernel<DT, OUT, D, HPB, CAP>), grid, dim3(kWaves16 * 64), kLds, stream, ev0,
                        ev1, 0, a);
  return hipGetLastError();
}

template <int DT, int OUT, int D, int HPB>
hipError_t launch_hpb(const PrefillArgs& a, dim3 grid, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  if (a.rows16)
    return a.softcap > 0.f ? launch_variant16<DT, OUT, D, HPB, true>(a, grid, stream, ev0, ev1)
                           : launch_variant16<DT, OUT, D, HPB, false>(a, grid, stream, ev0, ev1);
  return a.softcap > 0.f ? launch_variant<DT, OUT, D, HPB, true>(a, grid, stream, ev0, ev1)
                         : launch_variant<DT, OUT, D, HPB, false>(a, grid, stream, ev0, ev1);
}

// Key blocks of tile `t` of a layer with window `w` (0: global): the kernels' own arithmetic.
int tile_key_blocks(const PrefillArgs& a, int rows_per_tile, int w, int t) {
  const int p0 = a.q_pos0 + t * rows_per_tile;
  const int last = std::min(p0 + rows_per_tile, a.q_pos0 + a.n) - 1;
  const int lo = (w > 0 && p0 - w + 1 > 0) ? (p0 - w + 1) / kKeysPerBlock : 0;
  return last / kKeysPerBlock - lo + 1;
}

// The work plan of a launch on `wgs` workgroups: items are dealt out longest first, each to the workgroup that
// would be done with it earliest. The clock is a model of the measured launch (MI355X, 26 layers x 1024 tokens):
// with two workgroups per compute unit (wgs == 2 * cus) the one the dispatcher places first (index < cus) has
// its first loads served first and is at its first key block after about 5.7 us, the second after about 9.8 us;
// sharing the compute unit, the first gets through a key block in about 2.1 us, the second in 2.45 us; an item
// costs about 3 us besides its blocks (start, store). Both workgroups of a compute unit should finish together:
// a workgroup left alone runs faster (1.5 us per block) but the compute unit as a whole slower than the pair.
// With one workgroup per compute unit or fewer, all workgroups are alike.
//
// Launches over several layers, of two workgroups per compute unit and up to kPackMaxItems items, are packed instead
// (pack_by_deadline):
// longest first is a poor packer when most items are of one size (config 2: 356 of 832 items are 17 key blocks
// for 512 workgroups, and the items of 9 to 16 blocks end up on top of a 17 instead of on top of each other).
constexpr long kPlanMaxItems = 1L << 22;
constexpr size_t kPackMaxItems = 4096;

// Best fit, decreasing, under a deadline found by bisection: every item (longest first) goes to the workgroup
// that it fills up best without passing the deadline - of its layer's home XCD if one there can take it, else
// of any. The clock is a least-squares fit of the lifetimes of the 512 workgroups of the measured launch
// (times in units of 0.05 us): a first-placed workgroup 8.1 us + 1.4 us per key block, a second-placed one
// 7.05 us + 2.2 us per block (it is served second whenever both want the same pipe), 5 us per item.
// blocks[i], home_xcd[i]: key blocks and home XCD of item i (items sorted by blocks, longest first).
// Returns false when nothing was packed (never with the bounds of the bisection below).
bool pack_by_deadline(const std::vector<int32_t>& blocks, const std::vector<int>& home_xcd, int wgs, int cus, int xcds,
                      std::vector<int>* owner) {
  constexpr long kStart[2] = {162, 141}, kBlock[2] = {28, 44}, kItem = 100;  // [0] first-placed, [1] second-placed
  // The workgroups of an XCD and a kind, ordered by the time they are done: the best fit for an item is the
  // last one that still meets the deadline with it (a search in the ordered set, not a scan of all workgroups:
  // a plan is built whenever a launch shape is new, and a scan costs milliseconds).
  using Slot = std::pair<long, int>;  // (time done, workgroup)
  std::vector<std::set<Slot>> sets((size_t)xcds * 2);
  auto attempt = [&](long deadline, std::vector<int>* out) {
    for (auto& s : sets) s.clear();
    for (int g = 0; g < wgs; ++g) {
      const int kind = g < cus ? 0 : 1;
      sets[(size_t)(g % xcds) * 2 + kind].insert({kStart[kind], g});
    }
    for (size_t i = 0; i < blocks.size(); ++i) {
      std::set<Slot>* pick_set = nullptr;
      std::set<Slot>::iterator pick_it;
      long pick_done = -1;
      auto look = [&](int x) {
        for (int kind = 0; kind < 2; ++kind) {
          std::set<Slot>& s = sets[(size_t)x * 2 + kind];
          const long cost = kBlock[kind] * blocks[i] + kItem;
          auto it = s.upper_bound({deadline - cost, INT32_MAX});
          if (it == s.begin()) continue;
          --it;
          if (it->first + cost > pick_done) {
            pick_done = it->first + cost;
            pick_set = &s;
            pick_it = it;
          }
        }
      };
      look(xcds > 1 ? home_xcd[i] : 0);
      if (!pick_set)
        for (int x = 0; x < xcds; ++x) look(x);
      if (!pick_set) return false;
      const int g = pick_it->second;
      pick_set->erase(pick_it);
      pick_set->insert({pick_done, g});
      if (out) (*out)[i] = g;
    }
    return true;
  };
  long total = 0;
  for (int32_t b : blocks) total += b;
  long lo = 0, hi = kStart[0] + kStart[1] + kBlock[1] * total + kItem * (long)blocks.size();  // one workgroup takes all
  while (hi - lo > 4) {
    const long mid = (lo + hi) / 2;
    if (attempt(mid, nullptr)) hi = mid;
    else lo = mid;
  }
  return attempt(hi, owner);
}

void build_prefill_plan(const PrefillArgs& a, int hpb, int wgs, int cus, std::vector<int32_t>* words) {
  const int rows_per_tile = kStretch * (4 / hpb);
  const int tiles = (a.n + rows_per_tile - 1) / rows_per_tile;
  const int per_layer = a.geom.hkv * (a.group / hpb);
  struct It { int32_t unit, w1, blocks; };
  std::vector<It> items;
  for (int li = 0; li < a.n_layers; ++li) {
    const int w = a.host_window[a.layer_begin + li];
    for (int t = 0; t < tiles; ++t) {
      const int nblk = tile_key_blocks(a, rows_per_tile, w, t);
      const int parts = a.kchunk > 0 ? (nblk + a.kchunk - 1) / a.kchunk : 1;
      for (int part = 0; part < parts; ++part) {
        const int blocks = a.kchunk > 0 ? std::min(a.kchunk, nblk - part * a.kchunk) : nblk;
        for (int r = 0; r < per_layer; ++r) items.push_back(It{li * per_layer + r, t | (part << 20), blocks});
      }
    }
  }
  std::stable_sort(items.begin(), items.end(), [](const It& x, const It& y) { return x.blocks > y.blocks; });
  // times in units of 0.05 us
  constexpr long kFirstStart = 114, kSecondStart = 196, kFirstBlock = 42, kSecondBlock = 49, kItem = 60;
  const bool paired = cus > 0 && wgs > cus;
  // Workgroup g runs on XCD g % kXcds (the dispatcher deals workgroups out round robin), each XCD with an L2 of
  // its own: a layer's items go to the workgroups of one XCD, so that its K / V planes are pulled into one L2
  // instead of all eight - unless that XCD is behind the best workgroup anywhere by more than kStray, then the
  // item strays (layers differ in work, and 26 layers do not divide by 8). Layers are dealt to the XCDs heaviest
  // first, each to the XCD with the least work so far.
  constexpr int kXcds = 8;
  constexpr long kStray = 60;
  const int xcds = wgs >= 4 * kXcds ? kXcds : 1;
  std::vector<int> home(a.n_layers, 0);
  if (xcds > 1) {
    std::vector<long> layer_work(a.n_layers, 0), xcd_work(xcds, 0);
    for (const It& it : items) layer_work[it.unit / per_layer] += it.blocks;
    std::vector<int> by_work(a.n_layers);
    for (int li = 0; li < a.n_layers; ++li) by_work[li] = li;
    std::stable_sort(by_work.begin(), by_work.end(), [&](int x, int y) { return layer_work[x] > layer_work[y]; });
    for (int li : by_work) {
      const int x = (int)(std::min_element(xcd_work.begin(), xcd_work.end()) - xcd_work.begin());
      home[li] = x;
      xcd_work[x] += layer_work[li];
    }
  }
  std::vector<int> owner(items.size());
  std::vector<int> count(wgs, 0);
  bool packed = false;
  // (launches over several layers only: their shapes repeat, and the plan is kept; packing costs about a millisecond
  // of host time per new shape, longest-first a tenth of that)
  if (paired && a.n_layers > 1 && items.size() <= kPackMaxItems) {
    std::vector<int32_t> blocks(items.size());
    std::vector<int> home_xcd(items.size());
    for (size_t i = 0; i < items.size(); ++i) {
      blocks[i] = items[i].blocks;
      home_xcd[i] = home[items[i].unit / per_layer];
    }
    packed = pack_by_deadline(blocks, home_xcd, wgs, cus, xcds, &owner);
    if (packed)
      for (size_t i = 0; i < items.size(); ++i) ++count[owner[i]];
  }
  // (time done, workgroup) min-heaps per XCD: the first-placed workgroups and the second-placed ones
  using Entry = std::pair<long, int>;
  auto later = [](const Entry& x, const Entry& y) { return x > y; };
  std::vector<std::vector<Entry>> first(xcds), second(xcds);
  for (int g = 0; g < wgs; ++g) {
    if (paired && g >= cus) second[g % xcds].push_back({kSecondStart, g});
    else first[g % xcds].push_back({paired ? kFirstStart : 0L, g});
  }
  for (int x = 0; x < xcds; ++x) {
    std::make_heap(first[x].begin(), first[x].end(), later);
    std::make_heap(second[x].begin(), second[x].end(), later);
  }
  for (size_t i = 0; i < items.size() && !packed; ++i) {
    // the best workgroup of an XCD for this item: (time it would be done, which heap)
    auto best_of = [&](int x) {
      long t = -1;
      std::vector<Entry>* heap = nullptr;
      if (!first[x].empty()) {
        t = first[x].front().first + items[i].blocks * kFirstBlock + kItem;
        heap = &first[x];
      }
      if (!second[x].empty()) {
        const long t2 = second[x].front().first + items[i].blocks * kSecondBlock + kItem;
        if (t < 0 || t2 < t) {
          t = t2;
          heap = &second[x];
        }
      }
      return std::make_pair(t, heap);
    };
    auto pick = best_of(home[items[i].unit / per_layer]);
    auto best = pick;
    for (int x = 0; x < xcds; ++x) {
      const auto other = best_of(x);
      if (other.second && (!best.second || other.first < best.first)) best = other;
    }
    if (!pick.second || best.first + kStray < pick.first) pick = best;
    std::vector<Entry>& heap = *pick.second;
    std::pop_heap(heap.begin(), heap.end(), later);
    heap.back().first = pick.first;
    owner[i] = heap.back().second;
    ++count[owner[i]];
    std::push_heap(heap.begin(), heap.end(), later);
  }
  words->assign((size_t)wgs + 1 + 2 * items.size(), 0);
  int32_t* offs = words->data();
  for (int g = 0; g < wgs; ++g) offs[g + 1] = offs[g] + count[g];
  std::vector<int> fill(offs, offs + wgs);
  int32_t* list = words->data() + wgs + 1;
  for (size_t i = 0; i < items.size(); ++i) {
    const int at = fill[owner[i]]++;
    list[2 * at] = items[i].unit;
    list[2 * at + 1] = items[i].w1;
  }
}

void release_plan_slot(PrefillPlans* p, int s) {
  if (p->d_words[s]) (void)hipFree(p->d_words[s]);
  if (p->h_words[s]) (void)hipHostFree(p->h_words[s]);
  p->d_words[s] = p->h_words[s] = nullptr;
  p->cap[s] = 0;
  p->valid[s] = false;
}

// Device copy of the plan for this launch shape: a cached one, or a new one built into the least recently used
// slot that no captured graph holds and copied on `stream` ahead of the launch. *slot_out stays -1 when this
// launch cannot have a plan: the shape is new and the stream is being captured (building one needs a copy and a
// wait that a capture cannot hold), or every slot belongs to a captured graph. The caller then runs the kernel
// that needs no plan.
hipError_t plan_for(const PrefillArgs& a, int hpb, int wgs, int cus, PrefillPlans* p, hipStream_t stream, int* slot_out) {
  *slot_out = -1;
  // (layer_begin + plan_layer_offset: the first layer of the handle that the launch covers, whose windows the plan
  // depends on; a launch over staged planes addresses its layers from 0)
  const int64_t key[8] = {a.layer_begin + a.plan_layer_offset, a.n_layers, a.q_pos0, a.n, a.kchunk, wgs, hpb, a.seq};
  for (int s = 0; s < PrefillPlans::kSlots; ++s)
    if (p->valid[s] && std::equal(key, key + 8, p->key[s])) {
      p->last_use[s] = ++p->clock;
      *slot_out = s;
      return hipSuccess;
    }
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  hipError_t e = hipStreamIsCapturing(stream, &capturing);
  if (e != hipSuccess) return e;
  if (capturing != hipStreamCaptureStatusNone) return hipSuccess;
  int s = -1;
  for (int k = 0; k < PrefillPlans::kSlots; ++k)
    if (!p->pinned[k] && (s < 0 || p->last_use[k] < p->last_use[s])) s = k;
  if (s < 0) return hipSuccess;  // every slot belongs to a captured graph
  if (!p->used[s] && (e = hipEventCreateWithFlags(&p->used[s], hipEventDisableTiming)) != hipSuccess) return e;
  if ((e = hipEventSynchronize(p->used[s])) != hipSuccess) return e;  // the last launch that read this slot is over
  p->valid[s] = false;
  std::vector<int32_t> words;
  build_prefill_plan(a, hpb, wgs, cus, &words);
  if (p->cap[s] < words.size()) {
    release_plan_slot(p, s);
    const size_t cap = words.size() + words.size() / 2;
    if ((e = hipMalloc(&p->d_words[s], cap * sizeof(int32_t))) != hipSuccess) return e;
    if ((e = hipHostMalloc(&p->h_words[s], cap * sizeof(int32_t))) != hipSuccess) return e;
    p->cap[s] = cap;
  }
  std::copy(words.begin(), words.end(), p->h_words[s]);
  e = hipMemcpyAsync(p->d_words[s], p->h_words[s], words.size() * sizeof(int32_t), hipMemcpyHostToDevice, stream);
  if (e != hipSuccess) return e;
  std::copy(key, key + 8, p->key[s]);
  p->valid[s] = true;
  p->last_use[s] = ++p->clock;
  *slot_out = s;
  return hipSuccess;
}

template <int DT, int OUT, int D>
hipError_t launch_typed(const PrefillArgs& a, PrefillPlans* plans, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  const int G = a.group;
  const int hpb = (G % 4 == 0) ? 4 : ((G % 2 == 0) ? 2 : 1);
  const int pt = 4 / hpb;
  const int items = a.n_layers * a.geom.hkv * (G / hpb) * ((a.n + kStretch * pt - 1) / (kStretch * pt));
  static std::atomic<int> cus_cached{0};  // persistent workgroups are sized by the CU count
  int cus = cus_cached.load(std::memory_order_relaxed);
  if (cus == 0) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    cus_cached.store(cus, std::memory_order_relaxed);
  }
  PrefillArgs b = a;
  b.use_order = 0;
  if (OUT != DT && !a.q_staged) {
    // float32 activations: the queries go through the staging rows in the cache's type first
    if (!a.q_stage) return hipErrorInvalidValue;
    const int64_t n8 = (int64_t)a.n_layers * a.n * a.hq * D / 8;
    hipLaunchKernelGGL((convert_queries_kernel<DT>), dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const float*>(a.q), a.q_stage, n8);
    hipError_t ce = hipGetLastError();
    if (ce != hipSuccess) return ce;
    b.q = a.q_stage;
  }

  const int units = a.n_layers * a.geom.hkv * (G / hpb);
  if (units <= kPrefillOrderUnits && a.host_window) {
    // work of a unit = key blocks over all stretches of its layer; stable sort, heaviest first
    const int per_layer = a.geom.hkv * (G / hpb);
    const int tiles = (a.n + kStretch * pt - 1) / (kStretch * pt);
    std::vector<long> work(a.n_layers);
    for (int li = 0; li < a.n_layers; ++li) {
      const int w = a.host_window[a.layer_begin + li];
      long sum = 0;
      for (int t = 0; t < tiles; ++t) {
        const int p0 = a.q_pos0 + t * kStretch * pt;
        const int last = std::min(p0 + kStretch * pt, a.q_pos0 + a.n) - 1;
        const int lo = (w > 0 && p0 - w + 1 > 0) ? (p0 - w + 1) / kKeysPerBlock : 0;
        sum += last / kKeysPerBlock - lo + 1;
      }
      work[li] = sum;
    }
    std::vector<int> order(units);
    for (int u = 0; u < units; ++u) order[u] = u;
    std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return work[x / per_layer] > work[y / per_layer]; });
    for (int u = 0; u < units; ++u) b.unit_order[u] = (uint16_t)order[u];
    b.use_order = 1;
  }
  long all_items = items;
  if (a.kchunk > 0 && a.host_window) {
    // work items of a key split: the parts that hold at least one key block (the tickets also
    // number the empty ones, which the drawing thread skips)
    const int tiles = (a.n + kStretch * pt - 1) / (kStretch * pt);
    all_items = 0;
    for (int li = 0; li < a.n_layers; ++li) {
      const int w = a.host_window[a.layer_begin + li];
      for (int t = 0; t < tiles; ++t) {
        const int p0 = a.q_pos0 + t * kStretch * pt;
        const int last = std::min(p0 + kStretch * pt, a.q_pos0 + a.n) - 1;
        const int lo = (w > 0 && p0 - w + 1 > 0) ? (p0 - w + 1) / kKeysPerBlock : 0;
        const int nblk = last / kKeysPerBlock - lo + 1;
        all_items += (long)((nblk + a.kchunk - 1) / a.kchunk) * a.geom.hkv * (G / hpb);
      }
    }
  }
  // Which kernel: rows16 < 0 leaves it to this rule: the kernel on 16x16x32 MFMAs (two workgroups
  // per CU) when there are at least two work items per CU, else the one on 32x32x16 MFMAs, whose
  // single workgroup per CU gets through an item in half the time.
  b.rows16 = a.rows16 < 0 ? (all_items >= 2L * cus ? 1 : 0) : a.rows16;
  // (the planned kernel needs the host's copy of the windows, and a plan of bounded size)
  if (b.rows16 == 1 && (!a.host_window || all_items > kPlanMaxItems)) b.rows16 = 0;
  auto workgroups = [&]() {
    const int slots = b.rows16 == 1 ? 2 * cus : cus;
    int w = all_items < slots ? (int)all_items : slots;
    if (a.max_workgroups > 0 && a.max_workgroups < w) w = a.max_workgroups;
    return w;
  };
  int wgs = workgroups();
  int plan_slot = -1;
  if (b.rows16 == 1) {
    hipError_t pe = plan_for(a, hpb, wgs, cus, plans, stream, &plan_slot);
    if (pe != hipSuccess) return pe;
    if (plan_slot >= 0) {
      b.plan = plans->d_words[plan_slot];
    } else {  // no plan to be had for this launch (see plan_for): the kernel that draws its work from queues
      b.rows16 = 0;
      wgs = workgroups();
    }
  }
  const dim3 grid(wgs, 1, 1);
#ifdef MI355_PREFILL_ONE_SHAPE  // (development builds: one instantiation compiles in a tenth of the time)
  hipError_t err = hpb == 4 ? launch_hpb<DT, OUT, D, 4>(b, grid, stream, ev0, ev1) : hipErrorInvalidValue;
#else
  hipError_t err = hpb == 4   ? launch_hpb<DT, OUT, D, 4>(b, grid, stream, ev0, ev1)
                   : hpb == 2 ? launch_hpb<DT, OUT, D, 2>(b, grid, stream, ev0, ev1)
                              : launch_hpb<DT, OUT, D, 1>(b, grid, stream, ev0, ev1);
#endif
  if (err == hipSuccess && plan_slot >= 0) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    err = hipStreamIsCapturing(stream, &capturing);
    // (a captured launch keeps its plan for as long as the graph may be replayed: the slot is never reused)
    if (err == hipSuccess && capturing == hipStreamCaptureStatusNone) err = hipEventRecord(plans->used[plan_slot], stream);
    else if (err == hipSuccess) plans->pinned[plan_slot] = true;
  }
  if (err != hipSuccess || a.kchunk <= 0) return err;
  hipLaunchKernelGGL((prefill_merge_kernel<OUT, D>), dim3(a.hq, a.n, a.n_layers), dim3(D), 0, stream, b, kStretch * pt);
  return hipGetLastError();
}

}  // namespace

// Host only: the work plan of a launch shape without launching anything (tests of the planner).
int prefill_plan_probe(int n_layers, int n, int q_pos0, int hq, int hkv, const int32_t* layer_window, int wgs, int cus,
                       int32_t* items_per_wg, int32_t* blocks_per_wg, int32_t* items_off_home) {
  if (n_layers < 1 || n < 1 || q_pos0 < 0 || hq < 1 || hkv < 1 || hq % hkv != 0 || wgs < 1 || cus < 0 || !layer_window ||
      !items_per_wg || !blocks_per_wg)
    return -1;
  PrefillArgs a{};
  a.n_layers = n_layers;
  a.n = n;
  a.q_pos0 = q_pos0;
  a.hq = hq;
  a.group = hq / hkv;
  a.geom.hkv = hkv;
  a.host_window = layer_window;
  const int G = a.group;
  const int hpb = (G % 4 == 0) ? 4 : ((G % 2 == 0) ? 2 : 1);
  const int rows_per_tile = kStretch * (4 / hpb);
  const int per_layer = hkv * (G / hpb);
  std::vector<int32_t> words;
  build_prefill_plan(a, hpb, wgs, cus, &words);
  const int32_t* offs = words.data();
  const int32_t* list = words.data() + wgs + 1;
  const int total = offs[wgs];
  // every (unit, tile) exactly once
  std::set<std::pair<int32_t, int32_t>> seen;
  for (int i = 0; i < total; ++i)
    if (!seen.insert({list[2 * i], list[2 * i + 1]}).second) return -2;
  const int tiles = (n + rows_per_tile - 1) / rows_per_tile;
  if ((long)seen.size() != (long)n_layers * per_layer * tiles) return -3;
  // the home XCD of a layer as the planner computes it is not recomputed here: a layer's home is taken to be the XCD
  // that holds most of its items
  constexpr int kXcds = 8;
  std::vector<std::vector<int>> per_layer_xcd(n_layers, std::vector<int>(kXcds, 0));
  for (int g = 0; g < wgs; ++g) {
    items_per_wg[g] = offs[g + 1] - offs[g];
    long blocks = 0;
    for (int i = offs[g]; i < offs[g + 1]; ++i) {
      const int li = list[2 * i] / per_layer, tile = list[2 * i + 1] & 0xFFFFF;
      blocks += tile_key_blocks(a, rows_per_tile, layer_window[li], tile);
      ++per_layer_xcd[li][g % kXcds];
    }
    blocks_per_wg[g] = (int32_t)blocks;
  }
  if (items_off_home) {
    long off = 0;
    for (int li = 0; li < n_layers; ++li) {
      const auto& v = per_layer_xcd[li];
      const int most = *std::max_element(v.begin(), v.end());
      for (int x = 0; x < kXcds; ++x) off += v[x];
      off -= most;
    }
    *items_off_home = (int32_t)off;
  }
  return total;
}

PrefillSplit plan_prefill_split(const PrefillArgs& a, int option) {
  PrefillSplit out;
  if (option == 0 || !a.host_window) return out;
  const int G = a.group;
  const int hpb = (G % 4 == 0) ? 4 : ((G % 2 == 0) ? 2 : 1);
  const int rows_per_tile = kStretch * (4 / hpb);
  const int tiles = (a.n + rows_per_tile - 1) / rows_per_tile;
  const long items = (long)a.n_layers * a.geom.hkv * (G / hpb) * tiles;
  int max_nblk = 1;
  for (int li = 0; li < a.n_layers; ++li) {
    const int w = a.host_window[a.layer_begin + li];
    for (int t = 0; t < tiles; ++t) {
      const int p0 = a.q_pos0 + t * rows_per_tile;
      const int last = std::min(p0 + rows_per_tile, a.q_pos0 + a.n) - 1;
      const int lo = (w > 0 && p0 - w + 1 > 0) ? (p0 - w + 1) / kKeysPerBlock : 0;
      max_nblk = std::max(max_nblk, last / kKeysPerBlock - lo + 1);
    }
  }
  int kchunk;
  if (option > 0) {
    kchunk = option;
  } else {
    int cus = 0, dev = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
      return out;
    if (items * 4 >= (long)cus * 3) return out;
    int want = (int)std::min<long>(8, (cus + items - 1) / items);
    want = std::min(want, max_nblk / 4);  // at least 4 key blocks per item
    if (want <= 1) return out;
    kchunk = (max_nblk + want - 1) / want;
  }
  const int smax = (max_nblk + kchunk - 1) / kchunk;
  if (smax <= 1) return out;
  out.kchunk = kchunk;
  out.smax = smax;
  out.rows = (size_t)a.n_layers * a.n * a.hq * smax;
  return out;
}

bool prefill_supported(int kv_dtype, int io_dtype, int head_dim) {
  if (head_dim != 256) return false;
  if (kv_dtype == kI8) return io_dtype == kF32 || io_dtype == kF16 || io_dtype == kBF16;
  return (kv_dtype == kF16 || kv_dtype == kBF16) && (io_dtype == kv_dtype || io_dtype == kF32);
}

// ---------------------------------------------------------------------------
// An int8 cache on the matrix cores: the planes the call reads are turned into IEEE half planes once, in a staging
// area of the handle, and the kernels of a half cache run on those. The V planes take their scales with them
// (half(int8 value x float32 scale of its channel)). The K scales go where they cost nothing:
//   - float32 and bfloat16 activations pass through a conversion to half anyway, and take the scales there
//     (half(q x scale)); the K planes are then the int8 values themselves, exact in half;
//   - half activations are read by the attention kernel as they are (a pass over them just for the scales is 27 us
//     of an 83 us call at 26 layers x 1,024 rows), and the K planes take the scales (half(value x scale)).
// Either way a product of the scores has one operand rounded to half once, as in the decode kernel.
//   Why not in the attention kernel's registers, as the decode kernel does it: there every byte is converted once;
// here a K or V block is an operand of every query tile that sees it, so each of the workgroup's four waves would
// convert it again for each of its tiles, ten vector instructions for every two matrix instructions of 16 cycles,
// which bounds the kernel at half the matrix rate before the softmax is counted; and with 192 of a wave's 256
// registers holding accumulators and queries, the converted operands and their temporaries find no room (every
// arrangement tried spilled 30 to 150 registers, queries loaded behind the compiler's back among them).
// Converting once per call costs three bytes of HBM traffic per cache byte, against attention work that grows
// with the number of query rows.
// float32 or bfloat16 queries as the halves the kernels take, with the K scales of the head's plane folded in (the
// K planes of such a call are staged as the int8 values themselves): half(q x scale), one thread per 8 channels of
// a query row.
template <int IO, int D>
__global__ void __launch_bounds__(256) stage_queries_i8_kernel(const void* __restrict__ q, _Float16* __restrict__ dst,
                                                               const float* __restrict__ scales, CacheGeom geom, int layer_begin,
                                                               int seq, int n, int hq, int group, int64_t pieces) {
  static_assert(IO == kF32 || IO == kBF16, "half queries are taken as they are");
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= pieces) return;
  constexpr int kPieces = D / 8;
  const int d0 = 8 * (int)(i % kPieces);
  const int64_t row = i / kPieces;  // (layer, token, head)
  const int head = (int)(row % hq);
  const int li = (int)(row / ((int64_t)n * hq));
  const float* ks = scales + geom.scale_offset(layer_begin + li, seq, 0, head / group) + d0;
  f4 x0, x1;
  if constexpr (IO == kF32) {
    const float* src = reinterpret_cast<const float*>(q) + row * D + d0;
    x0 = *reinterpret_cast<const f4*>(src);
    x1 = *reinterpret_cast<const f4*>(src + 4);
  } else {
    const b8 v = *reinterpret_cast<const b8*>(reinterpret_cast<const __bf16*>(q) + row * D + d0);
#pragma unroll
    for (int e = 0; e < 4; ++e) { x0[e] = (float)v[e]; x1[e] = (float)v[4 + e]; }
  }
  const f4 s0 = *reinterpret_cast<const f4*>(ks), s1 = *reinterpret_cast<const f4*>(ks + 4);
  h8 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) { o[e] = (_Float16)(x0[e] * s0[e]); o[4 + e] = (_Float16)(x1[e] * s1[e]); }
  *reinterpret_cast<h8*>(dst + row * D + d0) = o;
}

// Grid (chunks of a plane's range / 256, planes of the call): one thread per 16-byte chunk of an int8 plane, which
// becomes two 16-byte chunks of the half plane (attn_params.h has both layouts):
//   K: chunk c of token t (channels 16 c .. + 15) -> chunks 2 c and 2 c + 1 of the same token, tile and row;
//   V: a chunk holds 16 tokens of one channel, slots 4 T + j of a 64-token block; slots 0..7 are the 8 slots of the
//      same chunk position in half block 2 B, slots 8..15 those in half block 2 B + 1.
// Blocks of 64 tokens that no query of the call sees (in front of a layer's window) are left alone.
__global__ void __launch_bounds__(256) dequant_planes_kernel(const uint8_t* __restrict__ cache, const float* __restrict__ scales,
                                                             CacheGeom src, uint8_t* __restrict__ staged, CacheGeom dst,
                                                             const int32_t* __restrict__ layer_window, int layer_begin,
                                                             int seq, int q_pos0, int64_t chunks, int scale_k) {
  const int64_t ci = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (ci >= chunks) return;
  const int D = src.head_dim;
  const int plane = blockIdx.y;  // (layer of the call, KV head, K / V)
  const int is_v = plane & 1;
  const int kvh = (plane >> 1) % src.hkv;
  const int li = (plane >> 1) / src.hkv;
  const int layer = layer_begin + li;
  const int window = layer_window[layer];
  const int chunks_per_block = 4 * D;  // 64 tokens x D bytes / 16
  const int64_t B = ci / chunks_per_block;
  const int x = (int)(ci % chunks_per_block);
  if (window > 0 && (B + 1) * 64 <= (int64_t)q_pos0 - window + 1) return;
  const u4 w = load_stream16(cache + src.plane_offset(layer, seq, kvh, is_v) + ci * 16);
  uint8_t* const out = staged + dst.plane_offset(li, 0, kvh, is_v);
  const float* const sc = scales + src.scale_offset(layer, seq, is_v, kvh);
  h8 lo, hi;
  cvt_i8x16_to_h8x2(w, lo, hi);
  if (!is_v) {
    const int tile = x / D, c = (x % D) >> 4, r = x & 15;  // (16-token tile of the block, chunk, row)
    if (scale_k) {
      const f4 s0 = *reinterpret_cast<const f4*>(sc + 16 * c), s1 = *reinterpret_cast<const f4*>(sc + 16 * c + 4);
      const f4 s2 = *reinterpret_cast<const f4*>(sc + 16 * c + 8), s3 = *reinterpret_cast<const f4*>(sc + 16 * c + 12);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo[e] = (_Float16)((float)lo[e] * s0[e]);
        lo[4 + e] = (_Float16)((float)lo[4 + e] * s1[e]);
        hi[e] = (_Float16)((float)hi[e] * s2[e]);
        hi[4 + e] = (_Float16)((float)hi[4 + e] * s3[e]);
      }
    }
    uint8_t* t0 = out + (B * 4 + tile) * (int64_t)(32 * D);
    *reinterpret_cast<h8*>(t0 + ((2 * c) * 16 + r) * 16) = lo;
    *reinterpret_cast<h8*>(t0 + ((2 * c + 1) * 16 + r) * 16) = hi;
  } else {
    const float vs = sc[16 * (x >> 6) + (x & 15)];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      lo[e] = (_Float16)((float)lo[e] * vs);
      hi[e] = (_Float16)((float)hi[e] * vs);
    }
    *reinterpret_cast<h8*>(out + (2 * B) * (int64_t)(64 * D) + x * 16) = lo;
    *reinterpret_cast<h8*>(out + (2 * B + 1) * (int64_t)(64 * D) + x * 16) = hi;
  }
}

// Bytes of the staging area for `n_layers` layers of a call that ends at position `end` (exclusive).
int64_t prefill_i8_stage_bytes(const CacheGeom& g, int n_layers, int end) {
  return (int64_t)n_layers * g.hkv * 2 * round_up64(end, kTokenAlign) * g.head_dim * 2;
}

template <int OUT>
hipError_t launch_i8(const PrefillArgs& a, PrefillPlans* plans, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  constexpr int D = 256;
  if (!a.kv_stage || !a.scales || (OUT != kF16 && !a.q_stage)) return hipErrorInvalidValue;
  const int end = a.q_pos0 + a.n;
  if (a.kv_stage_bytes < prefill_i8_stage_bytes(a.geom, a.n_layers, end)) return hipErrorInvalidValue;
  // the staged planes: a half cache of the call's layers and of one sequence, just long enough
  CacheGeom g = a.geom;
  g.num_layers = a.n_layers;
  g.max_seqs = 1;
  g.cap = (int32_t)round_up64(end, kTokenAlign);
  g.esize = 2;
  g.plane_bytes = (int64_t)g.cap * g.head_dim * 2;
  const int64_t chunks = (int64_t)(g.cap / 64) * 4 * D;
  // (the first launch of the call carries the start event of a timed call, the attention kernel the stop event)
  hipExtLaunchKernelGGL(dequant_planes_kernel, dim3((unsigned)((chunks + 255) / 256), a.n_layers * a.geom.hkv * 2), dim3(256),
                        0, stream, ev0, nullptr, 0, a.cache, a.scales, a.geom, reinterpret_cast<uint8_t*>(a.kv_stage), g,
                        a.layer_window, a.layer_begin, a.seq, a.q_pos0, chunks, OUT == kF16 ? 1 : 0);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  PrefillArgs b = a;
  if constexpr (OUT != kF16) {
    const int64_t pieces = (int64_t)a.n_layers * a.n * a.hq * (D / 8);
    hipLaunchKernelGGL((stage_queries_i8_kernel<OUT, D>), dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, stream, a.q,
                       reinterpret_cast<_Float16*>(a.q_stage), a.scales, a.geom, a.layer_begin, a.seq, a.n, a.hq, a.group,
                       pieces);
    if ((e = hipGetLastError()) != hipSuccess) return e;
    b.q = a.q_stage;
  }
  b.q_staged = 1;
  b.cache = reinterpret_cast<const uint8_t*>(a.kv_stage);
  b.geom = g;
  b.scales = nullptr;
  b.seq = 0;
  // (the kernels address layers from layer_begin on; the staged cache starts at the call's first layer)
  b.layer_begin = 0;
  b.plan_layer_offset = a.layer_begin;
  b.layer_window = a.layer_window + a.layer_begin;
  if (a.host_window) b.host_window = a.host_window + a.layer_begin;
  return launch_typed<kF16, OUT, D>(b, plans, stream, nullptr, ev1);
}

hipError_t launch_prefill(const PrefillArgs& a, int kv_dtype, int io_dtype, PrefillPlans* plans, hipStream_t stream,
                          hipEvent_t ev0, hipEvent_t ev1) {
#ifdef MI355_PREFILL_ONE_SHAPE
  if (kv_dtype == kBF16 && io_dtype == kBF16) return launch_typed<kBF16, kBF16, 256>(a, plans, stream, ev0, ev1);
#else
  if (kv_dtype == kF16 && io_dtype == kF16) return launch_typed<kF16, kF16, 256>(a, plans, stream, ev0, ev1);
  if (kv_dtype == kF16 && io_dtype == kF32) return launch_typed<kF16, kF32, 256>(a, plans, stream, ev0, ev1);
  if (kv_dtype == kBF16 && io_dtype == kBF16) return launch_typed<kBF16, kBF16, 256>(a, plans, stream, ev0, ev1);
  if (kv_dtype == kBF16 && io_dtype == kF32) return launch_typed<kBF16, kF32, 256>(a, plans, stream, ev0, ev1);
  if (kv_dtype == kI8 && io_dtype == kF16) return launch_i8<kF16>(a, plans, stream, ev0, ev1);
  if (kv_dtype == kI8 && io_dtype == kBF16) return launch_i8<kBF16>(a, plans, stream, ev0, ev1);
  if (kv_dtype == kI8 && io_dtype == kF32) return launch_i8<kF32>(a, plans, stream, ev0, ev1);
#endif
  return hipErrorInvalidValue;
}

void free_prefill_plans(PrefillPlans* p) {
  for (int s = 0; s < PrefillPlans::kSlots; ++s) {
    if (p->d_words[s]) (void)hipFree(p->d_words[s]);
    if (p->h_words[s]) (void)hipHostFree(p->h_words[s]);
    if (p->used[s]) (void)hipEventDestroy(p->used[s]);
    p->d_words[s] = p->h_words[s] = nullptr;
    p->used[s] = nullptr;
    p->valid[s] = false;
  }
}

}  // namespace mi355
