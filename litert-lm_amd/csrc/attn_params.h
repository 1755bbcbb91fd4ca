// Shared between the host side of the C ABI and the gfx950 kernels: element
// types, the KV-cache layout in HBM and the kernel argument blocks.
//
// KV-cache layout (one "plane" per layer x sequence x KV head x {K,V}).
// A plane holds `cap` token rows (cap = max_tokens rounded up to 64) of
// head_dim elements, stored so that every MFMA operand a wave needs is one
// 16-byte load per lane and every wave-wide load instruction covers 1 KiB of
// consecutive bytes:
//
//   EPC = 16 / sizeof(element)  elements per 16-byte chunk (4 f32, 8 f16/bf16, 16 i8)
//
//   K plane: tiles of 16 tokens. Inside a tile, chunk c = d / EPC of token
//   r = t % 16 sits at byte (c * 16 + r) * 16. A lane (r = lane % 16,
//   g = lane / 16) loading chunk 4*j + g of token r for j = 0,1,.. holds the
//   A operand (16 tokens x K-slice) of S^T = K . Q^T directly.
//
//   V plane: blocks of VB = 4 * EPC tokens. Token tb = t % VB of a block is
//   tile T = tb / 16, group g = (tb % 16) / 4, slot = 4 * T + tb % 4; element
//   (t, d) sits at byte ((d / 16 * 4 + g) * 16 + d % 16) * 16 + slot * sizeof.
//   The 16 bytes of lane (r = d % 16, g) are the A operand (16 channels x
//   token-slice) of O^T = V^T . P^T, and their token order matches the
//   accumulator layout in which S^T leaves the first MFMA, so P never moves
//   between lanes.
//
//   V planes of a bfloat16 cache hold IEEE half (binary16) values: the
//   probabilities that multiply V are numbers in [0, 1] that need mantissa, not
//   range, and as half operands they enter O^T = V^T . P^T with 11 significant bits
//   instead of 8 (one bfloat16 operand per probability costs ~1e-3 of relative
//   error, two operands half the matrix-core rate). A bfloat16 value v converts
//   without loss for 2^-17 <= |v| <= 65504; larger magnitudes saturate at +-65504
//   and smaller ones round to the nearest multiple of 2^-24. K planes stay bfloat16.
#ifndef LITERT_LM_AMD_CSRC_ATTN_PARAMS_H_
#define LITERT_LM_AMD_CSRC_ATTN_PARAMS_H_

#include <stdint.h>

#if defined(__HIPCC__)
#define MI355_HD __host__ __device__ inline
#else
#define MI355_HD inline
#endif

namespace mi355 {

enum DType : int32_t { kF32 = 0, kF16 = 1, kBF16 = 2, kI8 = 3 };

MI355_HD int dtype_size(int dt) { return dt == kF32 ? 4 : (dt == kI8 ? 1 : 2); }

constexpr int kTokenAlign = 64;  // planes hold a multiple of 64 rows
constexpr int kMaxGroup = 16;    // query heads per KV head handled by one MFMA column block
constexpr int kInlineItems = 64; // batches up to this size need no upload of their lengths
constexpr int kMaxDecodeSplits = 256;
constexpr int kInlineLayers = 64;  // calls over up to this many layers carry their windows in the argument block

MI355_HD int64_t round_up64(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

struct CacheGeom {
  int32_t num_layers, max_seqs, hkv, head_dim, cap, esize;
  int64_t plane_bytes;  // cap * head_dim * esize
  // plane index order: [layer][seq][kv_head][K=0 / V=1]
  MI355_HD int64_t plane_offset(int layer, int seq, int kvh, int is_v) const {
    return ((((int64_t)layer * max_seqs + seq) * hkv + kvh) * 2 + is_v) * plane_bytes;
  }
  // scales: float [layer][seq][K=0 / V=1][kv_head][head_dim]
  MI355_HD int64_t scale_offset(int layer, int seq, int is_v, int kvh) const {
    return ((((int64_t)layer * max_seqs + seq) * 2 + is_v) * hkv + kvh) * head_dim;
  }
};

// Byte offset of the 16-byte chunk holding elements [c*EPC, (c+1)*EPC) of token t in a K plane.
MI355_HD int64_t k_chunk_offset(int t, int c, int head_dim, int esize) {
  const int64_t tile_bytes = (int64_t)16 * head_dim * esize;
  return (int64_t)(t >> 4) * tile_bytes + ((int64_t)c * 16 + (t & 15)) * 16;
}

// Byte offset of element (t, d) in a V plane.
MI355_HD int64_t v_elem_offset(int t, int d, int head_dim, int esize) {
  const int epc = 16 / esize;
  const int vb = 4 * epc;
  const int64_t block_bytes = (int64_t)vb * head_dim * esize;
  const int tb = t % vb;
  const int T = tb >> 4, g = (tb & 15) >> 2, slot = 4 * T + (tb & 3);
  return (int64_t)(t / vb) * block_bytes + ((int64_t)((d >> 4) * 4 + g) * 16 + (d & 15)) * 16 +
         (int64_t)slot * esize;
}

// Arguments of the decode kernels (passed by value).
struct DecodeArgs {
  const void* q;             // [n_layers][batch][hq][D] io dtype
  void* out;                 // same shape
  const uint8_t* cache;      // base of all planes
  const float* scales;       // int8 cache only
  float* ws_acc;             // [items][hq][num_splits][D] partial accumulators
  float* ws_ml;              // [items][hq][num_splits][2] partial (max, sum)
  const int32_t* kv_lens;    // [batch] in dispatch order (unused when inline_items != 0)
  const int32_t* seq_ids;    // [batch] or nullptr
  const int32_t* rows;       // [batch] row in q / out of dispatch slot j (batches beyond kInlineItems), or nullptr
  int32_t inline_items;      // != 0: batch <= kInlineItems and lens / sequence ids travel in the argument block,
                             // in dispatch order (longest sequence first): entry j belongs to batch row inline_row[j]
  int32_t inline_lens[kInlineItems];
  int32_t inline_seq[kInlineItems];
  int32_t inline_row[kInlineItems];
  const int32_t* layer_window;  // [num_layers] (read only when n_layers > kInlineLayers)
  int32_t inline_window[kInlineLayers];  // windows of layers layer_begin .. layer_begin + n_layers - 1
  CacheGeom geom;
  int32_t hq, group;
  int32_t layer_begin, n_layers, batch;
  int32_t num_splits;
  int32_t max_kv_len;        // max over kv_lens (host computed), sizes the partitions
  int32_t min_kv_len;        // min over kv_lens (host computed; only the launch rules look at it)
  int32_t rule_batch;        // sequences the launch rules count: batch, or those of the larger batch this launch is a part of
  float scale;               // softmax scale
  float softcap;
  // The step before attention, run by the decode kernel itself for the one new token of every sequence
  // (one layer, inline_items != 0): raw projections [batch][hq][D] / [batch][hkv][D] in the io dtype; the
  // token's row is kv_len - 1. q is then unused. pre_q == nullptr: off. Flags and constants as in
  // PreAttentionArgs.
  const void* pre_q;
  const void* pre_k;
  const void* pre_v;
  const float* pre_constants;
  int32_t pre_rope, pre_norm_q, pre_norm_k, pre_norm_v, pre_q_scaled, pre_k_scaled;
  float pre_eps, pre_weight_offset;
};

// Tokens per split-KV partition for a layer with the given window: the same
// formula runs in the attention kernel and in the merge kernel.
MI355_HD int decode_partition_tokens(int max_kv_len, int window, int num_splits) {
  int span = max_kv_len;
  if (window > 0 && window + (kTokenAlign - 1) < span) span = window + (kTokenAlign - 1);
  int per = (span + num_splits - 1) / num_splits;
  per = (per + kTokenAlign - 1) / kTokenAlign * kTokenAlign;
  return per < kTokenAlign ? kTokenAlign : per;
}

// First visible key and the 64-aligned row at which partition 0 starts.
MI355_HD void decode_visible_range(int kv_len, int window, int* vlo, int* start) {
  int lo = 0;
  if (window > 0 && kv_len > window) lo = kv_len - window;
  *vlo = lo;
  *start = lo & ~(kTokenAlign - 1);
}

struct PrefillArgs {
  const void* q;   // [n_layers][n][hq][D], io type
  void* out;
  void* q_stage;   // room for the call's queries in the type the matrix cores take, 2 bytes per element, where that is
                   // not the activations' type: float32 activations, bfloat16 activations over an int8 cache
  int32_t q_staged;        // != 0: q is of the kernels' type already (set by the int8 path for the kernels it runs)
  int32_t plan_layer_offset;  // added to layer_begin in the key of the plan cache (launches over staged planes)
  void* kv_stage;          // int8 cache: room for the half planes the call reads (prefill_i8_stage_bytes)
  int64_t kv_stage_bytes;
  const uint8_t* cache;
  const float* scales;
  const int32_t* layer_window;
  int32_t* sched;  // kPrefillSchedInts work-queue counters, all zero between launches
  CacheGeom geom;
  int32_t hq, group;
  int32_t layer_begin, n_layers;
  int32_t seq, q_pos0, n;
  float scale, softcap;
  int32_t max_workgroups;  // 0 = one per CU; else an upper bound (tests: many work items per workgroup)
  // Units (layer, KV head, head block) in the order the queues deal them out: longest key loops first
  // (global layers before windowed ones). use_order == 0: identity (more units than the table holds).
  const int32_t* host_window;  // host copy of layer_window (for the ordering), may be null
  int32_t use_order;
  // Key split (launches with fewer work items than compute units): a work item covers at most kchunk
  // key blocks of its tile, tiles with more blocks are cut into up to smax items whose unnormalised
  // fp32 accumulators and (max, sum) pairs go to ws_acc / ws_ml, [layer][row][head][smax] x head_dim
  // and x 2 floats, and prefill_merge_kernel combines them. kchunk == 0: off.
  int32_t kchunk, smax;
  float* ws_acc;
  float* ws_ml;
  int32_t rows16;  // 1: the kernel on 16x16x32 MFMAs, two workgroups per compute unit; 0: the one on 32x32x16; < 0: by rule
  // Work plan of the kernel on 16x16x32 MFMAs (device memory): [workgroups + 1] offsets into the item list, then
  // two words per item, (unit, tile | part << 20), each workgroup's items in the order it runs them.
  const int32_t* plan;
  uint16_t unit_order[128];
};
constexpr int kPrefillQueues = 2;                     // ticket queues; workgroup k draws from queue k % 2 first
constexpr int kPrefillOrderUnits = 128;               // entries of PrefillArgs::unit_order
constexpr int kPrefillSchedInts = kPrefillQueues + 1;  // + count of workgroups that are done

struct KvCopyArgs {
  uint8_t* cache;
  CacheGeom geom;
  int32_t v_half;  // != 0: a bfloat16 cache, whose V planes hold IEEE half values (see the V plane note above)
  int32_t layer, seq, pos, n;
  void* k;  // [n][hkv][D] boundary layout (source for append, destination for read)
  void* v;
};

// Per-layer constants of the step before attention, float32 in HBM:
// [head_dim / 2] rotary frequencies, [head_dim] query norm weights, [head_dim] key norm weights.
MI355_HD int transform_floats(int head_dim) { return head_dim / 2 + 2 * head_dim; }

// Arguments of pre_attention_kernel (norm + rotary embedding + cache write).
struct PreAttentionArgs {
  const void* q;   // [n][hq][D] io dtype
  const void* k;   // [n][hkv][D] io dtype
  const void* v;   // [n][hkv][D] io dtype
  void* q_out;     // [n][hq][D] io dtype (may be q)
  uint8_t* cache;
  const float* scales;     // int8 cache: [layer][seq][K/V][hkv][D]
  const float* constants;  // this layer's transform_floats(D) floats
  CacheGeom geom;
  int32_t layer, seq, pos, n, hq;
  int32_t rope, norm_q, norm_k, norm_v, q_scaled, k_scaled;  // flags
  float eps, weight_offset;
};

}  // namespace mi355
#endif  // LITERT_LM_AMD_CSRC_ATTN_PARAMS_H_
