// C ABI of the MI355X attention library (see include/mi355_attn.h): handle
// lifetime, host-side validation of every shape before a kernel is launched,
// status/error-message conventions, staging for host-pointer callers.
#include "../../include/mi355_attn.h"

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <cmath>
#include <new>
#include <string>
#include <vector>

#include "attn_params.h"
#include "kernels.h"

using namespace mi355;

// Workspace of mi355_attn_decode_noalloc: the split-KV partials of one call, (head_dim + 2) floats per
// (layer, sequence, query head, partition), in device memory that exists from the moment the library
// is loaded. Each GPU holds its own copy; host code reaches it only through the address that
// hipGetSymbolAddress returns with that GPU current (resolved in mi355_attn_create), never through
// the array's name.
constexpr size_t kNoAllocSlots = 8192;  // partial slots: 8192 x 258 floats = 8.06 MiB per GPU
constexpr int kNoAllocHeadDim = 256;
static __device__ __align__(256) float scratch[kNoAllocSlots * (kNoAllocHeadDim + 2)];

namespace {

constexpr int kMaxDevices = 64;
float* g_scratch_ptr[kMaxDevices] = {};  // [device]: address of `scratch` on that GPU, set once by create
// Calls on different streams of one GPU share that GPU's `scratch`: each call waits (on its stream, not on the
// host) for the event that the previous call left behind when that call ran on another stream, so eager calls
// never overlap in the workspace. The events are made once per GPU by create. (Captured calls skip this: an
// event recorded inside a capture belongs to the graph.)
hipEvent_t g_scratch_done[kMaxDevices] = {};
hipStream_t g_scratch_stream[kMaxDevices] = {};
bool g_scratch_used[kMaxDevices] = {};

constexpr int kRingSlots = 64;
constexpr int kMaxSplits = kMaxDecodeSplits;

int fail(char** error_msg, int code, const char* fmt, ...) {
  if (error_msg) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    const size_t len = strlen(buf) + 1;
    char* msg = static_cast<char*>(malloc(len));
    if (msg) memcpy(msg, buf, len);
    *error_msg = msg;
  }
  return code;
}

#define HIP_OR_RETURN(expr)                                                                       \
  do {                                                                                            \
    hipError_t e_ = (expr);                                                                       \
    if (e_ != hipSuccess)                                                                         \
      return fail(error_msg, e_ == hipErrorOutOfMemory ? MI355_ATTN_RESOURCE_EXHAUSTED            \
                                                       : MI355_ATTN_INTERNAL,                     \
                  "%s failed: %s", #expr, hipGetErrorString(e_));                                 \
  } while (0)

__global__ void iota_items_kernel(int32_t* lens, int32_t* seq_ids, int n, int q_pos0, int seq) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    lens[i] = q_pos0 + i + 1;
    seq_ids[i] = seq;
  }
}

}  // namespace

struct mi355_attn {
  mi355_attn_config cfg{};
  CacheGeom geom{};
  int device = 0;
  hipStream_t stream = nullptr;
  bool own_stream = false;
  uint8_t* cache = nullptr;
  uint64_t cache_bytes = 0;
  float* scales = nullptr;
  int32_t* d_window = nullptr;
  int32_t* d_sched = nullptr;  // prefill work-queue counters
  PrefillPlans pf_plans;       // prefill work plans by launch shape
  float* d_pf_acc = nullptr;   // prefill key split: parts of split tiles, allocated on first use
  float* d_pf_ml = nullptr;
  size_t pf_rows = 0;          // rows (of head_dim / of 2 floats) the two hold
  void* d_q_stage = nullptr;   // prefill whose queries are staged (float32 activations; bfloat16 ones over an int8 cache)
  size_t q_stage_bytes = 0;
  void* d_kv_stage = nullptr;  // prefill over an int8 cache: the half planes of the layers of a pass
  size_t kv_stage_bytes = 0;
  int prefill_i8_min_rows = 16;  // int8 cache: calls of fewer rows take the row-wise path
  int prefill_i8_stage_mib = 2048;  // int8 cache: limit of the staging area (a pass covers as many layers as fit, at least one)
  int prefill_key_split = -1;  // < 0 by rule, 0 off, > 0 key blocks per work item
  int prefill_rows16 = -1;     // which prefill kernel: 1 the one on 16x16x32 MFMAs, 0 the one on 32x32x16, < 0 by rule
  // the step before attention: per-layer constants in HBM and what is switched on
  struct LayerTransform {
    bool set = false, rope = false, norm_q = false, norm_k = false, norm_v = false, q_scaled = false, k_scaled = false;
    float eps = 1e-6f, weight_offset = 1.f;
  };
  float* d_transform = nullptr;  // [num_layers][transform_floats(head_dim)]
  std::vector<LayerTransform> transform;
  std::vector<int32_t> window;
  std::vector<int32_t> filled;  // [layer][seq] rows written since the last reset
  // split-KV workspace
  float* ws_acc = nullptr;
  float* ws_ml = nullptr;
  size_t ws_slots = 0;

  // ring of (kv_lens, seq_ids) uploads
  int32_t* h_ring = nullptr;
  int32_t* d_ring = nullptr;
  hipEvent_t ring_ev[kRingSlots] = {};
  bool ring_used[kRingSlots] = {};
  int ring_next = 0;
  int ring_slot_ints = 0;
  // per-row items of the row-wise prefill path
  int32_t* d_items = nullptr;
  size_t d_items_cap = 0;
  // staging for host_io
  void* stage[4] = {nullptr, nullptr, nullptr, nullptr};
  size_t stage_cap[4] = {0, 0, 0, 0};
  // timing
  bool timing = false;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  bool timed = false;
  DecodeTuning tuning;
  bool rowwise_prefill = false;  // force the row-wise prefill path (cross-checks)
  int prefill_workgroups = 0;    // 0 = one per CU
};

namespace {

int io_size(const mi355_attn* h) { return dtype_size(h->cfg.io_dtype); }
int kv_size(const mi355_attn* h) { return dtype_size(h->cfg.kv_dtype); }

int ensure_stage(mi355_attn* h, int which, size_t bytes, char** error_msg) {
  if (h->stage_cap[which] >= bytes) return 0;
  HIP_OR_RETURN(hipStreamSynchronize(h->stream));
  if (h->stage[which]) HIP_OR_RETURN(hipFree(h->stage[which]));
  h->stage[which] = nullptr;
  h->stage_cap[which] = 0;
  const size_t cap = std::max(bytes, (size_t)1 << 20);
  HIP_OR_RETURN(hipMalloc(&h->stage[which], cap));
  h->stage_cap[which] = cap;
  return 0;
}

// Device view of a caller buffer that the kernels read.
int stage_in(mi355_attn* h, int which, const void* p, size_t bytes, const void** dev, char** error_msg) {
  if (!h->cfg.host_io) {
    *dev = p;
    return 0;
  }
  if (int rc = ensure_stage(h, which, bytes, error_msg)) return rc;
  HIP_OR_RETURN(hipMemcpyAsync(h->stage[which], p, bytes, hipMemcpyHostToDevice, h->stream));
  *dev = h->stage[which];
  return 0;
}

int stage_out_begin(mi355_attn* h, int which, void* p, size_t bytes, void** dev, char** error_msg) {
  if (!h->cfg.host_io) {
    *dev = p;
    return 0;
  }
  if (int rc = ensure_stage(h, which, bytes, error_msg)) return rc;
  *dev = h->stage[which];
  return 0;
}

int stage_out_end(mi355_attn* h, int which, void* p, size_t bytes, char** error_msg) {
  if (!h->cfg.host_io) return 0;
  HIP_OR_RETURN(hipMemcpyAsync(p, h->stage[which], bytes, hipMemcpyDeviceToHost, h->stream));
  HIP_OR_RETURN(hipStreamSynchronize(h->stream));
  return 0;
}

int ensure_workspace(mi355_attn* h, size_t slots, char** error_msg) {
  if (h->ws_slots >= slots) return 0;
  HIP_OR_RETURN(hipStreamSynchronize(h->stream));
  if (h->ws_acc) HIP_OR_RETURN(hipFree(h->ws_acc));
  if (h->ws_ml) HIP_OR_RETURN(hipFree(h->ws_ml));
  h->ws_acc = h->ws_ml = nullptr;
  h->ws_slots = 0;
  HIP_OR_RETURN(hipMalloc(&h->ws_acc, slots * h->cfg.head_dim * sizeof(float)));
  HIP_OR_RETURN(hipMalloc(&h->ws_ml, slots * 2 * sizeof(float)));
  h->ws_slots = slots;
  return 0;
}

// Uploads lengths, cache slots and rows in dispatch order (longest sequence
// first) through a ring of pinned slots so that calls can be queued back to
// back without waiting for earlier uploads.
int upload_items(mi355_attn* h, const int32_t* seq_ids, const int32_t* kv_lens, int batch,
                 const int32_t** d_lens, const int32_t** d_seq, const int32_t** d_rows, char** error_msg) {
  const int slot = h->ring_next;
  h->ring_next = (slot + 1) % kRingSlots;
  if (h->ring_used[slot]) HIP_OR_RETURN(hipEventSynchronize(h->ring_ev[slot]));
  int32_t* hs = h->h_ring + (size_t)slot * h->ring_slot_ints;
  int32_t* ds = h->d_ring + (size_t)slot * h->ring_slot_ints;
  int32_t* order = hs + 2 * (size_t)batch;
  for (int b = 0; b < batch; ++b) order[b] = b;
  std::stable_sort(order, order + batch, [&](int x, int y) { return kv_lens[x] > kv_lens[y]; });
  for (int j = 0; j < batch; ++j) {
    hs[j] = kv_lens[order[j]];
    hs[batch + j] = seq_ids ? seq_ids[order[j]] : order[j];
  }
  const size_t bytes = sizeof(int32_t) * batch * 3;
  HIP_OR_RETURN(hipMemcpyAsync(ds, hs, bytes, hipMemcpyHostToDevice, h->stream));
  HIP_OR_RETURN(hipEventRecord(h->ring_ev[slot], h->stream));
  h->ring_used[slot] = true;
  *d_lens = ds;
  *d_seq = ds + batch;
  *d_rows = ds + 2 * (size_t)batch;
  return 0;
}

// Rows count as appended only while they extend the unbroken prefix [0, filled) of their
// (layer, sequence): rows written behind a gap are stored, but attention never takes the unwritten
// (or, after a reset, stale) rows of the gap for appended ones.
void note_rows_written(mi355_attn* h, int layer, int seq, int pos, int n) {
  int32_t& f = h->filled[(size_t)layer * h->cfg.max_seqs + seq];
  if (pos <= f) f = std::max(f, pos + n);
}

int check_layers(const mi355_attn* h, int layer_begin, int n_layers, char** error_msg) {
  if (layer_begin < 0 || n_layers < 1 || layer_begin + n_layers > h->cfg.num_layers)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "layers [%d, %d) outside [0, %d)", layer_begin,
                layer_begin + n_layers, h->cfg.num_layers);
  return 0;
}

void fill_decode_common(const mi355_attn* h, DecodeArgs* a) {
  a->cache = h->cache;
  a->scales = h->scales;
  a->ws_acc = h->ws_acc;
  a->ws_ml = h->ws_ml;
  a->layer_window = h->d_window;
  a->geom = h->geom;
  a->hq = h->cfg.num_q_heads;
  a->group = h->cfg.num_q_heads / h->cfg.num_kv_heads;
  a->scale = h->cfg.scale;
  a->softcap = h->cfg.softcap;
}

void fill_inline_windows(const mi355_attn* h, DecodeArgs* a) {
  if (a->n_layers > kInlineLayers) return;
  for (int i = 0; i < a->n_layers; ++i) a->inline_window[i] = h->window[a->layer_begin + i];
}

// Raw projections of the one new token of every sequence (mi355_attn_decode_step): the decode kernel runs the
// step before attention itself.
struct NewRows {
  const void* k;
  const void* v;
};

// no_alloc: the call may not allocate (mi355_attn_decode_noalloc): device pointers only, and the
// partials go to this GPU's `scratch` instead of the handle's growable workspace.
// new_rows: q holds raw query projections and the new token's key / value rows come with the call
// (its row, kv_lens[b] - 1, need not have been appended).
// The batch a launch is a part of (mi355_attn_decode_step cuts large batches into several launches): the launch rules
// then look at the whole batch, so that every part runs as the same sequences would in one launch of all of them,
// partitions and waves included, and the results are the same bits.
struct WholeBatch { int batch, max_len, min_len; };

int decode_impl(mi355_attn* h, int layer_begin, int n_layers, const int32_t* seq_ids, const int32_t* kv_lens,
                int batch, const void* q, void* out, int num_splits, char** error_msg, bool no_alloc = false,
                const NewRows* new_rows = nullptr, const WholeBatch* whole = nullptr) {
  if (!h) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null handle");
  if (new_rows) {
    if (!new_rows->k || !new_rows->v) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null k or v");
    if (batch > kInlineItems)  // (mi355_attn_decode_step cuts larger batches into launches of this size)
      return fail(error_msg, MI355_ATTN_INTERNAL, "a fused decode step launch holds up to %d sequences (got %d)",
                  kInlineItems, batch);
  }
  if (no_alloc && h->cfg.host_io)
    return fail(error_msg, MI355_ATTN_FAILED_PRECONDITION,
                "mi355_attn_decode_noalloc needs device pointers (the handle was created with host_io = 1, "
                "whose staging buffers are allocated on demand)");
  if (int rc = check_layers(h, layer_begin, n_layers, error_msg)) return rc;
  if (!kv_lens || !q || !out) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null kv_lens, q or out");
  if (batch < 1 || batch > h->cfg.max_seqs)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "batch %d outside [1, max_seqs=%d]", batch,
                h->cfg.max_seqs);
  if (num_splits < 0 || num_splits > kMaxSplits)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "num_splits %d outside [0, %d]", num_splits, kMaxSplits);
  if (batch > 65535) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "batch %d exceeds the launch grid (65535)", batch);
  if (!decode_supported(h->cfg.kv_dtype, h->cfg.io_dtype, h->cfg.head_dim))
    return fail(error_msg, MI355_ATTN_UNIMPLEMENTED, "decode: unsupported kv/io dtype pair %d/%d",
                h->cfg.kv_dtype, h->cfg.io_dtype);
  int max_len = 0, min_len = INT32_MAX;
  for (int b = 0; b < batch; ++b) {
    const int seq = seq_ids ? seq_ids[b] : b;
    if (seq < 0 || seq >= h->cfg.max_seqs)
      return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "seq_ids[%d]=%d outside [0, %d)", b, seq,
                  h->cfg.max_seqs);
    const int len = kv_lens[b];
    if (len < 1 || len > h->cfg.max_tokens)
      return fail(error_msg, MI355_ATTN_OUT_OF_RANGE, "kv_lens[%d]=%d outside [1, max_tokens=%d]", b, len,
                  h->cfg.max_tokens);
    for (int l = layer_begin; l < layer_begin + n_layers; ++l)
      if (len - (new_rows ? 1 : 0) > h->filled[(size_t)l * h->cfg.max_seqs + seq])
        return fail(error_msg, MI355_ATTN_OUT_OF_RANGE,
                    "kv_lens[%d]=%d but only %d rows of layer %d, sequence %d were appended", b, len,
                    h->filled[(size_t)l * h->cfg.max_seqs + seq], l, seq);
    if (new_rows)  // every sequence gets one new row: the same sequence twice would write two
      for (int c = 0; c < b; ++c)
        if ((seq_ids ? seq_ids[c] : c) == seq)
          return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "seq_ids[%d] and seq_ids[%d] name the same sequence %d", c,
                      b, seq);
    max_len = std::max(max_len, len);
    min_len = std::min(min_len, len);
  }
  HIP_OR_RETURN(hipSetDevice(h->device));
  const int items = n_layers * batch;
  const bool splits_chosen = num_splits == 0;
  if (whole) {
    max_len = whole->max_len;
    min_len = whole->min_len;
  }
  if (num_splits == 0) {
    // About 1024 workgroups (four waves per CU saturate HBM; measured: 30 layers x 2 KV heads at 4096 tokens
    // run 8 % faster with 16-18 partitions than with 35, 16 layers x 64 sequences fastest without any split),
    // partitions of >= 64 tokens.
    const int rule_items = whole ? n_layers * whole->batch : items;
    const int want = (1024 + rule_items * h->cfg.num_kv_heads - 1) / (rule_items * h->cfg.num_kv_heads);
    num_splits = std::max(1, std::min({want, (max_len + 63) / 64, 64}));
    // Contexts of up to 512 tokens: one partition, and with it no merge launch. Measured (one layer, fp16, Hq8/Hkv2,
    // calls queued back to back): 1 sequence of 256 / 512 tokens 6.7 / 8.6 us against 9.9 / 9.8 us split and merged,
    // 64 sequences 9.7 / 15.4 against 11.0 / 16.1 us, 256 sequences 26.9 / 46.3 against 32.4 / 51.8 us; from 640
    // tokens on the split wins for small batches (1 sequence of 768 tokens: 10.9 against 9.8 us).
    if (max_len <= 512) num_splits = 1;
  }
  DecodeArgs a{};
  const size_t slots = (size_t)items * h->cfg.num_q_heads * num_splits;
  if (no_alloc) {
    // the library's own choice of partitions is trimmed to the workspace; an explicit count is an error
    if (num_splits > 1 && slots > kNoAllocSlots) {
      if (splits_chosen) {
        num_splits = (int)(kNoAllocSlots / ((size_t)items * h->cfg.num_q_heads));
      } else {
        return fail(error_msg, MI355_ATTN_RESOURCE_EXHAUSTED,
                    "mi355_attn_decode_noalloc: %d layers x %d sequences x %d query heads x %d partitions = %zu partial "
                    "results, the fixed workspace holds %zu (pass fewer partitions, or 0 to let the library choose)",
                    n_layers, batch, h->cfg.num_q_heads, num_splits, slots, kNoAllocSlots);
      }
      if (num_splits < 1) num_splits = 1;
    }
  } else if (num_splits > 1) {
    if (int rc = ensure_workspace(h, slots, error_msg)) return rc;
  }
  fill_decode_common(h, &a);
  if (no_alloc) {
    float* const base = g_scratch_ptr[h->device];  // this GPU's copy of `scratch`
    a.ws_acc = base;
    a.ws_ml = base + kNoAllocSlots * kNoAllocHeadDim;
  }
  const size_t io_bytes = (size_t)items * h->cfg.num_q_heads * h->cfg.head_dim * io_size(h);
  const void* dq = nullptr;
  void* dout = nullptr;
  if (int rc = stage_in(h, 0, q, io_bytes, &dq, error_msg)) return rc;
  if (new_rows) {
    const size_t kv_bytes = (size_t)batch * h->cfg.num_kv_heads * h->cfg.head_dim * io_size(h);
    if (int rc = stage_in(h, 2, new_rows->k, kv_bytes, &a.pre_k, error_msg)) return rc;
    if (int rc = stage_in(h, 3, new_rows->v, kv_bytes, &a.pre_v, error_msg)) return rc;
    a.pre_q = dq;
    const mi355_attn::LayerTransform& lt = h->transform[layer_begin];  // never set: a plain append
    a.pre_constants = h->d_transform + (size_t)layer_begin * transform_floats(h->cfg.head_dim);
    a.pre_rope = lt.rope;
    a.pre_norm_q = lt.norm_q;
    a.pre_norm_k = lt.norm_k;
    a.pre_norm_v = lt.norm_v;
    a.pre_q_scaled = lt.q_scaled;
    a.pre_k_scaled = lt.k_scaled;
    a.pre_eps = lt.eps;
    a.pre_weight_offset = lt.weight_offset;
  }
  if (int rc = stage_out_begin(h, 1, out, io_bytes, &dout, error_msg)) return rc;
  if (batch <= kInlineItems) {
    a.inline_items = 1;
    // dispatch order: longest sequence first (rows keep their places in q and out)
    int order[kInlineItems];
    for (int b = 0; b < batch; ++b) order[b] = b;
    std::stable_sort(order, order + batch, [&](int x, int y) { return kv_lens[x] > kv_lens[y]; });
    for (int j = 0; j < batch; ++j) {
      const int b = order[j];
      a.inline_lens[j] = kv_lens[b];
      a.inline_seq[j] = seq_ids ? seq_ids[b] : b;
      a.inline_row[j] = b;
    }
  } else {
    // lengths and slots of a larger batch go up through the pinned ring: a copy and, when the ring wraps, a wait
    // on the host - neither can be part of a stream capture
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    HIP_OR_RETURN(hipStreamIsCapturing(h->stream, &capturing));
    if (capturing != hipStreamCaptureStatusNone)
      return fail(error_msg, MI355_ATTN_FAILED_PRECONDITION,
                  "decode of %d sequences while the stream is being captured: more than %d sequences per call need "
                  "an upload that a capture cannot hold (capture calls of up to %d sequences)",
                  batch, kInlineItems, kInlineItems);
    if (int rc = upload_items(h, seq_ids, kv_lens, batch, &a.kv_lens, &a.seq_ids, &a.rows, error_msg)) return rc;
  }
  a.q = dq;
  a.out = dout;
  a.layer_begin = layer_begin;
  a.n_layers = n_layers;
  a.batch = batch;
  a.num_splits = num_splits;
  a.max_kv_len = max_len;
  a.min_kv_len = min_len;
  a.rule_batch = whole ? whole->batch : batch;
  fill_inline_windows(h, &a);
  bool scratch_fence = false;
  if (no_alloc && num_splits > 1) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    HIP_OR_RETURN(hipStreamIsCapturing(h->stream, &capturing));
    scratch_fence = capturing == hipStreamCaptureStatusNone;
    if (scratch_fence && g_scratch_used[h->device] && g_scratch_stream[h->device] != h->stream)
      HIP_OR_RETURN(hipStreamWaitEvent(h->stream, g_scratch_done[h->device], 0));
  }
  HIP_OR_RETURN(launch_decode(a, h->cfg.kv_dtype, h->cfg.io_dtype, h->tuning, h->stream,
                              h->timing ? h->ev0 : nullptr, h->timing ? h->ev1 : nullptr));
  if (scratch_fence) {
    HIP_OR_RETURN(hipEventRecord(g_scratch_done[h->device], h->stream));
    g_scratch_stream[h->device] = h->stream;
    g_scratch_used[h->device] = true;
  }
  h->timed = h->timing;
  if (new_rows)
    for (int b = 0; b < batch; ++b) note_rows_written(h, layer_begin, seq_ids ? seq_ids[b] : b, kv_lens[b] - 1, 1);
  return stage_out_end(h, 1, out, io_bytes, error_msg);
}

int prefill_impl(mi355_attn* h, int layer_begin, int n_layers, int seq, int q_pos0, int n, const void* q,
                 void* out, char** error_msg) {
  if (!h) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null handle");
  if (int rc = check_layers(h, layer_begin, n_layers, error_msg)) return rc;
  if (!q || !out) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null q or out");
  if (seq < 0 || seq >= h->cfg.max_seqs)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "seq %d outside [0, %d)", seq, h->cfg.max_seqs);
  if (n < 1 || q_pos0 < 0 || (int64_t)q_pos0 + n > h->cfg.max_tokens)
    return fail(error_msg, MI355_ATTN_OUT_OF_RANGE, "rows [%d, %lld) outside [0, max_tokens=%d]", q_pos0,
                (long long)q_pos0 + n, h->cfg.max_tokens);
  for (int l = layer_begin; l < layer_begin + n_layers; ++l)
    if (q_pos0 + n > h->filled[(size_t)l * h->cfg.max_seqs + seq])
      return fail(error_msg, MI355_ATTN_OUT_OF_RANGE,
                  "prefill over rows [0, %d) but only %d rows of layer %d, sequence %d were appended",
                  q_pos0 + n, h->filled[(size_t)l * h->cfg.max_seqs + seq], l, seq);
  HIP_OR_RETURN(hipSetDevice(h->device));
  const size_t io_bytes = (size_t)n_layers * n * h->cfg.num_q_heads * h->cfg.head_dim * io_size(h);
  const void* dq = nullptr;
  void* dout = nullptr;
  if (int rc = stage_in(h, 0, q, io_bytes, &dq, error_msg)) return rc;
  if (int rc = stage_out_begin(h, 1, out, io_bytes, &dout, error_msg)) return rc;
  hipEvent_t e0 = h->timing ? h->ev0 : nullptr, e1 = h->timing ? h->ev1 : nullptr;
  bool rowwise = !prefill_supported(h->cfg.kv_dtype, h->cfg.io_dtype, h->cfg.head_dim) || h->rowwise_prefill;
  // An int8 cache goes to the matrix cores through half planes staged per call (prefill_attn.hip): from a tile's
  // worth of rows on, in passes of as many layers as the staging area's limit holds.
  const bool i8 = h->cfg.kv_dtype == MI355_ATTN_I8;
  int layers_per_pass = n_layers;
  if (!rowwise && i8) {
    if (n < h->prefill_i8_min_rows) {
      rowwise = true;
    } else {
      const int64_t kStageMax = (int64_t)h->prefill_i8_stage_mib << 20;
      const int64_t per_layer = prefill_i8_stage_bytes(h->geom, 1, q_pos0 + n);
      layers_per_pass = (int)std::min<int64_t>(n_layers, std::max<int64_t>(1, kStageMax / per_layer));
      const size_t need = (size_t)per_layer * layers_per_pass;
      if (h->kv_stage_bytes < need) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        HIP_OR_RETURN(hipStreamIsCapturing(h->stream, &capturing));
        if (capturing != hipStreamCaptureStatusNone) {
          rowwise = true;  // (nothing can be allocated while a graph is recorded: the path that needs no room)
        } else {
          HIP_OR_RETURN(hipStreamSynchronize(h->stream));
          if (h->d_kv_stage) HIP_OR_RETURN(hipFree(h->d_kv_stage));
          h->d_kv_stage = nullptr;
          h->kv_stage_bytes = 0;
          HIP_OR_RETURN(hipMalloc(&h->d_kv_stage, need));
          h->kv_stage_bytes = need;
        }
      }
    }
  }
  const size_t layer_io_bytes = (size_t)n * h->cfg.num_q_heads * h->cfg.head_dim * io_size(h);
  for (int l0 = 0; !rowwise && l0 < n_layers; l0 += layers_per_pass) {
    const int nl = std::min(layers_per_pass, n_layers - l0);
    hipEvent_t pe0 = l0 == 0 ? e0 : nullptr, pe1 = l0 + nl == n_layers ? e1 : nullptr;
    PrefillArgs a{};
    a.q = static_cast<const uint8_t*>(dq) + l0 * layer_io_bytes;
    a.out = static_cast<uint8_t*>(dout) + l0 * layer_io_bytes;
    a.cache = h->cache;
    a.scales = h->scales;
    a.layer_window = h->d_window;
    a.sched = h->d_sched;
    a.geom = h->geom;
    a.hq = h->cfg.num_q_heads;
    a.group = h->cfg.num_q_heads / h->cfg.num_kv_heads;
    a.layer_begin = layer_begin + l0;
    a.n_layers = nl;
    a.seq = seq;
    a.q_pos0 = q_pos0;
    a.n = n;
    a.scale = h->cfg.scale;
    a.softcap = h->cfg.softcap;
    a.max_workgroups = h->prefill_workgroups;
    a.rows16 = h->prefill_rows16;
    a.host_window = h->window.data();
    if (h->cfg.io_dtype != h->cfg.kv_dtype && !(i8 && h->cfg.io_dtype == MI355_ATTN_F16)) {
      const size_t need = (size_t)nl * n * h->cfg.num_q_heads * h->cfg.head_dim * 2;
      if (h->q_stage_bytes < need) {
        HIP_OR_RETURN(hipStreamSynchronize(h->stream));
        if (h->d_q_stage) HIP_OR_RETURN(hipFree(h->d_q_stage));
        h->d_q_stage = nullptr;
        h->q_stage_bytes = 0;
        HIP_OR_RETURN(hipMalloc(&h->d_q_stage, need));
        h->q_stage_bytes = need;
      }
      a.q_stage = h->d_q_stage;
    }
    a.kv_stage = h->d_kv_stage;
    a.kv_stage_bytes = (int64_t)h->kv_stage_bytes;
    PrefillSplit split = plan_prefill_split(a, h->prefill_key_split);
    constexpr size_t kSplitRowsMax = (size_t)256 << 10;  // 256 Ki rows = 258 MiB at head_dim 256
    if (split.kchunk > 0 && split.rows > kSplitRowsMax && h->prefill_key_split < 0) split = PrefillSplit{};
    if (split.kchunk > 0) {
      if (split.rows > kSplitRowsMax)
        return fail(error_msg, MI355_ATTN_RESOURCE_EXHAUSTED, "prefill_key_split=%d needs %zu workspace rows (limit %zu)",
                    h->prefill_key_split, split.rows, kSplitRowsMax);
      if (h->pf_rows < split.rows) {
        HIP_OR_RETURN(hipStreamSynchronize(h->stream));
        if (h->d_pf_acc) HIP_OR_RETURN(hipFree(h->d_pf_acc));
        if (h->d_pf_ml) HIP_OR_RETURN(hipFree(h->d_pf_ml));
        h->d_pf_acc = h->d_pf_ml = nullptr;
        h->pf_rows = 0;
        HIP_OR_RETURN(hipMalloc(&h->d_pf_acc, split.rows * h->cfg.head_dim * sizeof(float)));
        HIP_OR_RETURN(hipMalloc(&h->d_pf_ml, split.rows * 2 * sizeof(float)));
        h->pf_rows = split.rows;
      }
      a.kchunk = split.kchunk;
      a.smax = split.smax;
      a.ws_acc = h->d_pf_acc;
      a.ws_ml = h->d_pf_ml;
    }
    HIP_OR_RETURN(launch_prefill(a, h->cfg.kv_dtype, h->cfg.io_dtype, &h->pf_plans, h->stream, pe0, pe1));
  }
  if (rowwise) {
    // Row-wise path (fp32 and int8 caches): every query row is one decode item
    // whose key range ends at its own position.
    if (!decode_supported(h->cfg.kv_dtype, h->cfg.io_dtype, h->cfg.head_dim))
      return fail(error_msg, MI355_ATTN_UNIMPLEMENTED, "prefill: unsupported kv/io dtype pair %d/%d",
                  h->cfg.kv_dtype, h->cfg.io_dtype);
    if (n > 65535)
      return fail(error_msg, MI355_ATTN_UNIMPLEMENTED,
                  "row-wise prefill (fp32 / int8 cache): %d rows exceed the launch grid (65535); call in chunks", n);
    if (h->d_items_cap < (size_t)n) {  // (never for an int8 or float32 cache: theirs is there from the start)
      hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
      HIP_OR_RETURN(hipStreamIsCapturing(h->stream, &capturing));
      if (capturing != hipStreamCaptureStatusNone)
        return fail(error_msg, MI355_ATTN_FAILED_PRECONDITION,
                    "row-wise prefill needs its item list allocated, which cannot happen while the stream is being "
                    "captured: run one row-wise prefill before the capture");
      HIP_OR_RETURN(hipStreamSynchronize(h->stream));
      if (h->d_items) HIP_OR_RETURN(hipFree(h->d_items));
      h->d_items = nullptr;
      h->d_items_cap = 0;
      HIP_OR_RETURN(hipMalloc(&h->d_items, sizeof(int32_t) * 2 * (size_t)h->cfg.max_tokens));
      h->d_items_cap = h->cfg.max_tokens;
    }
    int32_t* lens = h->d_items;
    int32_t* seqs = h->d_items + h->d_items_cap;
    hipLaunchKernelGGL(iota_items_kernel, dim3((n + 255) / 256), dim3(256), 0, h->stream, lens, seqs, n, q_pos0,
                       seq);
    HIP_OR_RETURN(hipGetLastError());
    DecodeArgs a{};
    fill_decode_common(h, &a);
    a.q = dq;
    a.out = dout;
    a.kv_lens = lens;
    a.seq_ids = seqs;
    a.layer_begin = layer_begin;
    a.n_layers = n_layers;
    a.batch = n;
    a.num_splits = 1;
    a.max_kv_len = q_pos0 + n;
    fill_inline_windows(h, &a);
    HIP_OR_RETURN(launch_decode(a, h->cfg.kv_dtype, h->cfg.io_dtype, h->tuning, h->stream, e0, e1));
  }
  h->timed = h->timing;
  return stage_out_end(h, 1, out, io_bytes, error_msg);
}

}  // namespace

extern "C" {

const char* mi355_attn_version(void) { return "mi355_attn 0.1 (gfx950)"; }

int mi355_attn_create(const mi355_attn_config* c, mi355_attn** out, char** error_msg) {
  if (out) *out = nullptr;
  if (!c || !out) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null config or out");
  if (c->struct_size != sizeof(mi355_attn_config))
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "config.struct_size %u != %zu", c->struct_size,
                sizeof(mi355_attn_config));
  if (c->num_layers < 1 || c->num_q_heads < 1 || c->num_kv_heads < 1 || c->max_tokens < 1 || c->max_seqs < 1)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "layers, heads, max_tokens and max_seqs must be >= 1");
  if (c->num_q_heads % c->num_kv_heads)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "num_q_heads %d is not a multiple of num_kv_heads %d",
                c->num_q_heads, c->num_kv_heads);
  if (c->num_q_heads / c->num_kv_heads > kMaxGroup)
    return fail(error_msg, MI355_ATTN_UNIMPLEMENTED, "more than %d query heads per KV head", kMaxGroup);
  if (c->head_dim != 256)
    return fail(error_msg, MI355_ATTN_UNIMPLEMENTED, "head_dim %d (only 256 is built)", c->head_dim);
  if (c->kv_dtype < MI355_ATTN_F32 || c->kv_dtype > MI355_ATTN_I8 || c->io_dtype < MI355_ATTN_F32 ||
      c->io_dtype > MI355_ATTN_BF16)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "bad kv_dtype %d or io_dtype %d", c->kv_dtype,
                c->io_dtype);
  if (!decode_supported(c->kv_dtype, c->io_dtype, c->head_dim))
    return fail(error_msg, MI355_ATTN_UNIMPLEMENTED,
                "kv_dtype %d with io_dtype %d (supported: equal f32 / f16 / bf16; f16 or bf16 cache with f32 io; int8 "
                "cache with f16, bf16 or f32 io)",
                c->kv_dtype, c->io_dtype);
  if (c->softcap < 0.f || c->scale < 0.f)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "scale and softcap must be >= 0");
  if (c->layer_window)
    for (int l = 0; l < c->num_layers; ++l)
      if (c->layer_window[l] < 0)
        return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "layer_window[%d] < 0", l);

  int ndev = 0;
  if (hipGetDeviceCount(&ndev) != hipSuccess || ndev < 1)
    return fail(error_msg, MI355_ATTN_UNAVAILABLE, "no HIP device");
  if (c->device < 0 || c->device >= ndev)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "device %d outside [0, %d)", c->device, ndev);
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, c->device) != hipSuccess)
    return fail(error_msg, MI355_ATTN_UNAVAILABLE, "cannot query device %d", c->device);
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(error_msg, MI355_ATTN_UNAVAILABLE, "device %d is %s; this library is built for gfx950 only",
                c->device, prop.gcnArchName);

  mi355_attn* h = new (std::nothrow) mi355_attn();
  if (!h) return fail(error_msg, MI355_ATTN_RESOURCE_EXHAUSTED, "out of host memory");
  h->cfg = *c;
  h->cfg.layer_window = nullptr;
  if (h->cfg.scale == 0.f) h->cfg.scale = 1.0f / sqrtf((float)c->head_dim);
  h->device = c->device;
  h->window.assign(c->num_layers, 0);
  if (c->layer_window) h->window.assign(c->layer_window, c->layer_window + c->num_layers);
  h->filled.assign((size_t)c->num_layers * c->max_seqs, 0);
  h->geom.num_layers = c->num_layers;
  h->geom.max_seqs = c->max_seqs;
  h->geom.hkv = c->num_kv_heads;
  h->geom.head_dim = c->head_dim;
  h->geom.cap = (int32_t)round_up64(c->max_tokens, kTokenAlign);
  h->geom.esize = dtype_size(c->kv_dtype);
  h->geom.plane_bytes = (int64_t)h->geom.cap * c->head_dim * h->geom.esize;
  // the kernels address a plane through a 32-bit buffer descriptor and 32-bit block offsets
  if (h->geom.plane_bytes > (int64_t)INT32_MAX) {
    const long long pb = (long long)h->geom.plane_bytes;
    delete h;
    return fail(error_msg, MI355_ATTN_UNIMPLEMENTED, "max_tokens %d: one plane would hold %lld bytes (limit 2 GiB - 1)",
                c->max_tokens, pb);
  }
  h->cache_bytes = (uint64_t)h->geom.plane_bytes * 2 * c->num_kv_heads * c->max_seqs * c->num_layers;

  auto bail = [&](int code, const char* what, hipError_t e) {
    int rc = fail(error_msg, code, "%s: %s", what, hipGetErrorString(e));
    mi355_attn_destroy(h);
    return rc;
  };
  hipError_t e;
  if ((e = hipSetDevice(h->device)) != hipSuccess) return bail(MI355_ATTN_UNAVAILABLE, "hipSetDevice", e);
  if (h->device >= kMaxDevices) {
    int rc = fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "device %d: at most %d devices", h->device, kMaxDevices);
    mi355_attn_destroy(h);
    return rc;
  }
  if (!g_scratch_ptr[h->device]) {  // once per GPU, with that GPU current
    float* p = nullptr;
    if ((e = hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch))) != hipSuccess || !p)
      return bail(MI355_ATTN_INTERNAL, "hipGetSymbolAddress(scratch)", e);
    g_scratch_ptr[h->device] = p;
  }
  if (!g_scratch_done[h->device] &&
      (e = hipEventCreateWithFlags(&g_scratch_done[h->device], hipEventDisableTiming)) != hipSuccess)
    return bail(MI355_ATTN_INTERNAL, "hipEventCreate", e);
  if (c->own_stream) {
    if ((e = hipStreamCreateWithFlags(&h->stream, hipStreamNonBlocking)) != hipSuccess)
      return bail(MI355_ATTN_INTERNAL, "hipStreamCreate", e);
    h->own_stream = true;
  } else {
    h->stream = static_cast<hipStream_t>(c->stream);  // nullptr is the HIP default stream
  }
  if ((e = hipMalloc(&h->cache, h->cache_bytes)) != hipSuccess)
    return bail(MI355_ATTN_RESOURCE_EXHAUSTED, "KV cache allocation", e);
  // Rows that were never written must read as finite numbers: a masked key
  // still enters P.V with probability 0, and 0 * NaN would poison the output.
  if ((e = hipMemsetAsync(h->cache, 0, h->cache_bytes, h->stream)) != hipSuccess)
    return bail(MI355_ATTN_INTERNAL, "KV cache clear", e);
  if (c->kv_dtype == MI355_ATTN_I8) {
    const size_t nsc = (size_t)c->num_layers * c->max_seqs * 2 * c->num_kv_heads * c->head_dim;
    if ((e = hipMalloc(&h->scales, nsc * sizeof(float))) != hipSuccess)
      return bail(MI355_ATTN_RESOURCE_EXHAUSTED, "scale allocation", e);
    if ((e = hipMemsetAsync(h->scales, 0, nsc * sizeof(float), h->stream)) != hipSuccess)
      return bail(MI355_ATTN_INTERNAL, "scale clear", e);
  }
  if ((e = hipMalloc(&h->d_window, sizeof(int32_t) * c->num_layers)) != hipSuccess)
    return bail(MI355_ATTN_RESOURCE_EXHAUSTED, "window table", e);
  if ((e = hipMemcpyAsync(h->d_window, h->window.data(), sizeof(int32_t) * c->num_layers, hipMemcpyHostToDevice,
                          h->stream)) != hipSuccess)
    return bail(MI355_ATTN_INTERNAL, "window upload", e);
  if ((e = hipMalloc(&h->d_sched, sizeof(int32_t) * (kPrefillSchedInts + 1))) != hipSuccess)  // (+ the stream probe's sink word)
    return bail(MI355_ATTN_RESOURCE_EXHAUSTED, "prefill queue counters", e);
  h->transform.assign(c->num_layers, mi355_attn::LayerTransform{});
  const size_t transform_bytes = sizeof(float) * (size_t)c->num_layers * transform_floats(c->head_dim);
  if ((e = hipMalloc(&h->d_transform, transform_bytes)) != hipSuccess)
    return bail(MI355_ATTN_RESOURCE_EXHAUSTED, "layer transform constants", e);
  if ((e = hipMemsetAsync(h->d_transform, 0, transform_bytes, h->stream)) != hipSuccess)
    return bail(MI355_ATTN_INTERNAL, "layer transform clear", e);
  if ((e = hipMemsetAsync(h->d_sched, 0, sizeof(int32_t) * kPrefillSchedInts, h->stream)) != hipSuccess)
    return bail(MI355_ATTN_INTERNAL, "prefill queue clear", e);
  if (c->kv_dtype == MI355_ATTN_I8 || c->kv_dtype == MI355_ATTN_F32) {
    // the row-wise prefill path's item list (these caches may take that path inside a captured graph, where nothing
    // can be allocated)
    if ((e = hipMalloc(&h->d_items, sizeof(int32_t) * 2 * (size_t)c->max_tokens)) != hipSuccess)
      return bail(MI355_ATTN_RESOURCE_EXHAUSTED, "row-wise prefill items", e);
    h->d_items_cap = c->max_tokens;
  }
  h->ring_slot_ints = 3 * c->max_seqs;
  if ((e = hipHostMalloc(&h->h_ring, sizeof(int32_t) * h->ring_slot_ints * kRingSlots)) != hipSuccess)
    return bail(MI355_ATTN_RESOURCE_EXHAUSTED, "pinned ring", e);
  if ((e = hipMalloc(&h->d_ring, sizeof(int32_t) * h->ring_slot_ints * kRingSlots)) != hipSuccess)
    return bail(MI355_ATTN_RESOURCE_EXHAUSTED, "device ring", e);
  for (int i = 0; i < kRingSlots; ++i)
    if ((e = hipEventCreateWithFlags(&h->ring_ev[i], hipEventDisableTiming)) != hipSuccess)
      return bail(MI355_ATTN_INTERNAL, "hipEventCreate", e);
  if ((e = hipEventCreate(&h->ev0)) != hipSuccess || (e = hipEventCreate(&h->ev1)) != hipSuccess)
    return bail(MI355_ATTN_INTERNAL, "hipEventCreate", e);
  if ((e = hipStreamSynchronize(h->stream)) != hipSuccess) return bail(MI355_ATTN_INTERNAL, "create sync", e);
  *out = h;
  return MI355_ATTN_OK;
}

void mi355_attn_destroy(mi355_attn* h) {
  if (!h) return;
  (void)hipSetDevice(h->device);
  (void)hipStreamSynchronize(h->stream);
  if (h->cache) (void)hipFree(h->cache);
  if (h->scales) (void)hipFree(h->scales);
  if (h->d_window) (void)hipFree(h->d_window);
  if (h->d_sched) (void)hipFree(h->d_sched);
  free_prefill_plans(&h->pf_plans);
  if (h->d_pf_acc) (void)hipFree(h->d_pf_acc);
  if (h->d_pf_ml) (void)hipFree(h->d_pf_ml);
  if (h->d_q_stage) (void)hipFree(h->d_q_stage);
  if (h->d_kv_stage) (void)hipFree(h->d_kv_stage);
  if (h->d_transform) (void)hipFree(h->d_transform);
  if (h->ws_acc) (void)hipFree(h->ws_acc);
  if (h->ws_ml) (void)hipFree(h->ws_ml);
  if (h->d_ring) (void)hipFree(h->d_ring);
  if (h->h_ring) (void)hipHostFree(h->h_ring);
  if (h->d_items) (void)hipFree(h->d_items);
  for (auto& s : h->stage)
    if (s) (void)hipFree(s);
  for (auto& ev : h->ring_ev)
    if (ev) (void)hipEventDestroy(ev);
  if (h->ev0) (void)hipEventDestroy(h->ev0);
  if (h->ev1) (void)hipEventDestroy(h->ev1);
  if (h->device < kMaxDevices && g_scratch_stream[h->device] == h->stream && g_scratch_used[h->device]) {
    // (the stream was synchronised above: its last use of the shared workspace is over, and a later stream
    // that happens to get the same address must not be taken for it)
    g_scratch_used[h->device] = false;
    g_scratch_stream[h->device] = nullptr;
  }
  if (h->own_stream && h->stream) (void)hipStreamDestroy(h->stream);
  delete h;
}

int mi355_attn_kv_append(mi355_attn* h, int32_t layer, int32_t seq, int32_t pos, int32_t n, const void* k,
                         const void* v, char** error_msg) {
  if (!h) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null handle");
  if (int rc = check_layers(h, layer, 1, error_msg)) return rc;
  if (seq < 0 || seq >= h->cfg.max_seqs)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "seq %d outside [0, %d)", seq, h->cfg.max_seqs);
  if (n < 0 || pos < 0 || (int64_t)pos + n > h->cfg.max_tokens)
    return fail(error_msg, MI355_ATTN_OUT_OF_RANGE, "rows [%d, %lld) outside [0, max_tokens=%d]", pos,
                (long long)pos + n, h->cfg.max_tokens);
  if (n == 0) return MI355_ATTN_OK;
  if (!k || !v) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null k or v");
  HIP_OR_RETURN(hipSetDevice(h->device));
  const size_t bytes = (size_t)n * h->cfg.num_kv_heads * h->cfg.head_dim * kv_size(h);
  const void *dk = nullptr, *dv = nullptr;
  if (int rc = stage_in(h, 2, k, bytes, &dk, error_msg)) return rc;
  if (int rc = stage_in(h, 3, v, bytes, &dv, error_msg)) return rc;
  KvCopyArgs a{};
  a.cache = h->cache;
  a.geom = h->geom;
  a.v_half = h->cfg.kv_dtype == MI355_ATTN_BF16;
  a.layer = layer;
  a.seq = seq;
  a.pos = pos;
  a.n = n;
  a.k = const_cast<void*>(dk);
  a.v = const_cast<void*>(dv);
  HIP_OR_RETURN(launch_kv_append(a, h->stream));
  if (h->cfg.host_io) HIP_OR_RETURN(hipStreamSynchronize(h->stream));
  note_rows_written(h, layer, seq, pos, n);
  return MI355_ATTN_OK;
}

int mi355_attn_kv_set_scales(mi355_attn* h, int32_t layer, int32_t seq, const float* k_scale,
                             const float* v_scale, char** error_msg) {
  if (!h) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null handle");
  if (h->cfg.kv_dtype != MI355_ATTN_I8)
    return fail(error_msg, MI355_ATTN_FAILED_PRECONDITION, "scales apply to an int8 cache only");
  if (int rc = check_layers(h, layer, 1, error_msg)) return rc;
  if (seq < 0 || seq >= h->cfg.max_seqs)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "seq %d outside [0, %d)", seq, h->cfg.max_seqs);
  if (!k_scale || !v_scale) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null scales");
  HIP_OR_RETURN(hipSetDevice(h->device));
  const size_t n = (size_t)h->cfg.num_kv_heads * h->cfg.head_dim;
  const hipMemcpyKind kind = h->cfg.host_io ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice;
  HIP_OR_RETURN(hipMemcpyAsync(h->scales + h->geom.scale_offset(layer, seq, 0, 0), k_scale, n * sizeof(float), kind,
                               h->stream));
  HIP_OR_RETURN(hipMemcpyAsync(h->scales + h->geom.scale_offset(layer, seq, 1, 0), v_scale, n * sizeof(float), kind,
                               h->stream));
  if (h->cfg.host_io) HIP_OR_RETURN(hipStreamSynchronize(h->stream));
  return MI355_ATTN_OK;
}

int mi355_attn_set_layer_transform(mi355_attn* h, int32_t layer, const mi355_attn_layer_transform* t,
                                   char** error_msg) {
  if (!h) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null handle");
  if (!t || t->struct_size != sizeof(mi355_attn_layer_transform))
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null transform or struct_size mismatch");
  if (int rc = check_layers(h, layer, 1, error_msg)) return rc;
  if (!(t->eps >= 0.f) || !std::isfinite(t->eps) || !std::isfinite(t->weight_offset))
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "eps %g must be finite and >= 0, weight_offset %g finite",
                (double)t->eps, (double)t->weight_offset);
  const int D = h->cfg.head_dim;
  if (t->rope_inv_freq)
    for (int d = 0; d < D / 2; ++d)
      if (!std::isfinite(t->rope_inv_freq[d]))
        return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "rope_inv_freq[%d] is not finite", d);
  HIP_OR_RETURN(hipSetDevice(h->device));
  // the constants are host arrays whatever host_io says; copied before this call returns
  std::vector<float> row((size_t)transform_floats(D), 0.f);
  if (t->rope_inv_freq) memcpy(row.data(), t->rope_inv_freq, sizeof(float) * (D / 2));
  if (t->q_weight) memcpy(row.data() + D / 2, t->q_weight, sizeof(float) * D);
  if (t->k_weight) memcpy(row.data() + D / 2 + D, t->k_weight, sizeof(float) * D);
  HIP_OR_RETURN(hipStreamSynchronize(h->stream));  // earlier launches may still read the old constants
  HIP_OR_RETURN(hipMemcpy(h->d_transform + (size_t)layer * transform_floats(D), row.data(), sizeof(float) * row.size(),
                          hipMemcpyHostToDevice));
  mi355_attn::LayerTransform& lt = h->transform[layer];
  lt.set = true;
  lt.rope = t->rope_inv_freq != nullptr;
  lt.norm_q = t->norm_q != 0;
  lt.norm_k = t->norm_k != 0;
  lt.norm_v = t->norm_v != 0;
  lt.q_scaled = lt.norm_q && t->q_weight != nullptr;
  lt.k_scaled = lt.norm_k && t->k_weight != nullptr;
  lt.eps = t->eps;
  lt.weight_offset = t->weight_offset;
  return MI355_ATTN_OK;
}

int mi355_attn_pre_attention(mi355_attn* h, int32_t layer, int32_t seq, int32_t pos, int32_t n, const void* q,
                             const void* k, const void* v, void* q_out, char** error_msg) {
  if (!h) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null handle");
  if (int rc = check_layers(h, layer, 1, error_msg)) return rc;
  if (seq < 0 || seq >= h->cfg.max_seqs)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "seq %d outside [0, %d)", seq, h->cfg.max_seqs);
  if (n < 0 || pos < 0 || (int64_t)pos + n > h->cfg.max_tokens)
    return fail(error_msg, MI355_ATTN_OUT_OF_RANGE, "rows [%d, %lld) outside [0, max_tokens=%d]", pos,
                (long long)pos + n, h->cfg.max_tokens);
  if (n == 0) return MI355_ATTN_OK;
  if (!q || !k || !v || !q_out) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null q, k, v or q_out");
  HIP_OR_RETURN(hipSetDevice(h->device));
  const size_t q_bytes = (size_t)n * h->cfg.num_q_heads * h->cfg.head_dim * io_size(h);
  const size_t kv_bytes = (size_t)n * h->cfg.num_kv_heads * h->cfg.head_dim * io_size(h);
  const void *dq = nullptr, *dk = nullptr, *dv = nullptr;
  void* dout = nullptr;
  if (int rc = stage_in(h, 0, q, q_bytes, &dq, error_msg)) return rc;
  if (int rc = stage_in(h, 2, k, kv_bytes, &dk, error_msg)) return rc;
  if (int rc = stage_in(h, 3, v, kv_bytes, &dv, error_msg)) return rc;
  if (int rc = stage_out_begin(h, 1, q_out, q_bytes, &dout, error_msg)) return rc;
  const mi355_attn::LayerTransform& lt = h->transform[layer];  // never set: a plain append
  PreAttentionArgs a{};
  a.q = dq;
  a.k = dk;
  a.v = dv;
  a.q_out = dout;
  a.cache = h->cache;
  a.scales = h->scales;
  a.constants = h->d_transform + (size_t)layer * transform_floats(h->cfg.head_dim);
  a.geom = h->geom;
  a.layer = layer;
  a.seq = seq;
  a.pos = pos;
  a.n = n;
  a.hq = h->cfg.num_q_heads;
  a.rope = lt.rope;
  a.norm_q = lt.norm_q;
  a.norm_k = lt.norm_k;
  a.norm_v = lt.norm_v;
  a.q_scaled = lt.q_scaled;
  a.k_scaled = lt.k_scaled;
  a.eps = lt.eps;
  a.weight_offset = lt.weight_offset;
  HIP_OR_RETURN(launch_pre_attention(a, h->cfg.kv_dtype, h->cfg.io_dtype, h->stream, h->timing ? h->ev0 : nullptr,
                                     h->timing ? h->ev1 : nullptr));
  h->timed = h->timing;
  note_rows_written(h, layer, seq, pos, n);
  return stage_out_end(h, 1, q_out, q_bytes, error_msg);
}

int mi355_attn_kv_read(mi355_attn* h, int32_t layer, int32_t seq, int32_t pos, int32_t n, void* k_out, void* v_out,
                       char** error_msg) {
  if (!h) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null handle");
  if (int rc = check_layers(h, layer, 1, error_msg)) return rc;
  if (seq < 0 || seq >= h->cfg.max_seqs)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "seq %d outside [0, %d)", seq, h->cfg.max_seqs);
  if (n < 0 || pos < 0 || (int64_t)pos + n > h->cfg.max_tokens)
    return fail(error_msg, MI355_ATTN_OUT_OF_RANGE, "rows [%d, %lld) outside [0, max_tokens=%d]", pos,
                (long long)pos + n, h->cfg.max_tokens);
  if (n == 0) return MI355_ATTN_OK;
  if (!k_out || !v_out) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null k_out or v_out");
  HIP_OR_RETURN(hipSetDevice(h->device));
  const size_t bytes = (size_t)n * h->cfg.num_kv_heads * h->cfg.head_dim * kv_size(h);
  void *dk = nullptr, *dv = nullptr;
  if (int rc = stage_out_begin(h, 2, k_out, bytes, &dk, error_msg)) return rc;
  if (int rc = stage_out_begin(h, 3, v_out, bytes, &dv, error_msg)) return rc;
  KvCopyArgs a{};
  a.cache = h->cache;
  a.geom = h->geom;
  a.v_half = h->cfg.kv_dtype == MI355_ATTN_BF16;
  a.layer = layer;
  a.seq = seq;
  a.pos = pos;
  a.n = n;
  a.k = dk;
  a.v = dv;
  HIP_OR_RETURN(launch_kv_read(a, h->stream));
  if (int rc = stage_out_end(h, 2, k_out, bytes, error_msg)) return rc;
  return stage_out_end(h, 3, v_out, bytes, error_msg);
}

int mi355_attn_prefill(mi355_attn* h, int32_t layer, int32_t seq, int32_t q_pos0, int32_t n, const void* q,
                       void* out, char** error_msg) {
  return prefill_impl(h, layer, 1, seq, q_pos0, n, q, out, error_msg);
}

int mi355_attn_prefill_layers(mi355_attn* h, int32_t layer_begin, int32_t n_layers, int32_t seq, int32_t q_pos0,
                              int32_t n, const void* q, void* out, char** error_msg) {
  return prefill_impl(h, layer_begin, n_layers, seq, q_pos0, n, q, out, error_msg);
}

int mi355_attn_decode(mi355_attn* h, int32_t layer, const int32_t* seq_ids, const int32_t* kv_lens, int32_t batch,
                      const void* q, void* out, int32_t num_splits, char** error_msg) {
  return decode_impl(h, layer, 1, seq_ids, kv_lens, batch, q, out, num_splits, error_msg);
}

int mi355_attn_decode_layers(mi355_attn* h, int32_t layer_begin, int32_t n_layers, const int32_t* seq_ids,
                             const int32_t* kv_lens, int32_t batch, const void* q, void* out, int32_t num_splits,
                             char** error_msg) {
  return decode_impl(h, layer_begin, n_layers, seq_ids, kv_lens, batch, q, out, num_splits, error_msg);
}

int mi355_attn_prefill_plan_probe(int32_t n_layers, int32_t n, int32_t q_pos0, int32_t num_q_heads, int32_t num_kv_heads,
                                  const int32_t* layer_window, int32_t workgroups, int32_t compute_units,
                                  int32_t* items_per_wg, int32_t* blocks_per_wg, int32_t* items_off_home) {
  return mi355::prefill_plan_probe(n_layers, n, q_pos0, num_q_heads, num_kv_heads, layer_window, workgroups, compute_units,
                                   items_per_wg, blocks_per_wg, items_off_home);
}

int mi355_attn_decode_step(mi355_attn* h, int32_t layer, const int32_t* seq_ids, const int32_t* kv_lens, int32_t batch,
                           const void* q, const void* k, const void* v, void* out, int32_t num_splits,
                           char** error_msg) {
  if (!h) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null handle");
  if (batch <= kInlineItems) {
    const NewRows rows{k, v};
    return decode_impl(h, layer, 1, seq_ids, kv_lens, batch, q, out, num_splits, error_msg, /*no_alloc=*/false, &rows);
  }
  // More sequences than one launch carries in its argument block: launches of kInlineItems sequences each, queued
  // back to back. Everything that can be refused is checked for the whole batch first, so that a call either
  // runs all of its launches or none.
  if (int rc = check_layers(h, layer, 1, error_msg)) return rc;
  if (!kv_lens || !q || !k || !v || !out) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null kv_lens, q, k, v or out");
  if (batch > h->cfg.max_seqs)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "batch %d outside [1, max_seqs=%d]", batch, h->cfg.max_seqs);
  if (num_splits < 0 || num_splits > kMaxSplits)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "num_splits %d outside [0, %d]", num_splits, kMaxSplits);
  std::vector<int32_t> ids(batch);
  std::vector<char> named(h->cfg.max_seqs, 0);
  for (int b = 0; b < batch; ++b) {
    const int seq = seq_ids ? seq_ids[b] : b;
    if (seq < 0 || seq >= h->cfg.max_seqs)
      return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "seq_ids[%d]=%d outside [0, %d)", b, seq, h->cfg.max_seqs);
    if (named[seq]) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "seq_ids names sequence %d twice (entry %d)", seq, b);
    named[seq] = 1;
    ids[b] = seq;
    const int len = kv_lens[b];
    if (len < 1 || len > h->cfg.max_tokens)
      return fail(error_msg, MI355_ATTN_OUT_OF_RANGE, "kv_lens[%d]=%d outside [1, max_tokens=%d]", b, len, h->cfg.max_tokens);
    if (len - 1 > h->filled[(size_t)layer * h->cfg.max_seqs + seq])
      return fail(error_msg, MI355_ATTN_OUT_OF_RANGE, "kv_lens[%d]=%d but only %d rows of layer %d, sequence %d were appended",
                  b, len, h->filled[(size_t)layer * h->cfg.max_seqs + seq], layer, seq);
  }
  const size_t q_row = (size_t)h->cfg.num_q_heads * h->cfg.head_dim * io_size(h);
  const size_t kv_row = (size_t)h->cfg.num_kv_heads * h->cfg.head_dim * io_size(h);
  WholeBatch whole{batch, 0, INT32_MAX};
  for (int b = 0; b < batch; ++b) {
    whole.max_len = std::max(whole.max_len, kv_lens[b]);
    whole.min_len = std::min(whole.min_len, kv_lens[b]);
  }
  for (int b0 = 0; b0 < batch; b0 += kInlineItems) {
    const int nb = std::min<int>(kInlineItems, batch - b0);
    const NewRows rows{static_cast<const uint8_t*>(k) + b0 * kv_row, static_cast<const uint8_t*>(v) + b0 * kv_row};
    if (int rc = decode_impl(h, layer, 1, ids.data() + b0, kv_lens + b0, nb, static_cast<const uint8_t*>(q) + b0 * q_row,
                             static_cast<uint8_t*>(out) + b0 * q_row, num_splits, error_msg, /*no_alloc=*/false, &rows,
                             &whole))
      return rc;
  }
  return MI355_ATTN_OK;
}

int mi355_attn_decode_noalloc(mi355_attn* h, int32_t layer, const int32_t* seq_ids, const int32_t* kv_lens,
                              int32_t batch, const void* q, void* out, int32_t num_splits, char** error_msg) {
  static_assert(kNoAllocHeadDim == 256, "the workspace is laid out for the one head_dim the library builds");
  return decode_impl(h, layer, 1, seq_ids, kv_lens, batch, q, out, num_splits, error_msg, /*no_alloc=*/true);
}

int mi355_attn_stream_probe(mi355_attn* h, uint64_t offset, uint64_t bytes, int32_t workgroups, int32_t waves,
                            char** error_msg) {
  if (!h) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null handle");
  if (workgroups < 1 || waves < 1 || waves > 16 || bytes < 1)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "workgroups >= 1, 1 <= waves <= 16 and bytes >= 1");
  HIP_OR_RETURN(hipSetDevice(h->device));
  hipError_t e = launch_stream_probe(h->cache, (int64_t)h->cache_bytes, (int64_t)offset, (int64_t)bytes, workgroups, waves,
                                     reinterpret_cast<uint32_t*>(h->d_sched) + kPrefillSchedInts, h->stream,
                                     h->timing ? h->ev0 : nullptr, h->timing ? h->ev1 : nullptr);
  if (e == hipErrorInvalidValue)
    return fail(error_msg, MI355_ATTN_OUT_OF_RANGE,
                "%llu bytes from offset %llu in %d x %d shares of whole 32 KiB pieces do not fit the cache (%llu bytes), or "
                "the offset is not a multiple of 16",
                (unsigned long long)bytes, (unsigned long long)offset, workgroups, waves, (unsigned long long)h->cache_bytes);
  HIP_OR_RETURN(e);
  h->timed = h->timing;
  return MI355_ATTN_OK;
}

int mi355_attn_reset(mi355_attn* h, int32_t seq, char** error_msg) {
  if (!h) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null handle");
  if (seq >= h->cfg.max_seqs)
    return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "seq %d outside [0, %d)", seq, h->cfg.max_seqs);
  for (int l = 0; l < h->cfg.num_layers; ++l)
    for (int s = 0; s < h->cfg.max_seqs; ++s)
      if (seq < 0 || s == seq) h->filled[(size_t)l * h->cfg.max_seqs + s] = 0;
  return MI355_ATTN_OK;
}

int mi355_attn_sync(mi355_attn* h, char** error_msg) {
  if (!h) return fail(error_msg, MI355_ATTN_INVALID_ARGUMENT, "null handle");
  HIP_OR_RETURN(hipSetDevice(h->device));
  HIP_OR_RETURN(hipStreamSynchronize(h->stream));
  return MI355_ATTN_OK;
}

void* mi355_attn_stream(mi355_attn* h) { return h ? h->stream : nullptr; }

int mi355_attn_set_timing(mi355_attn* h, int32_t enabled) {
  if (!h) return MI355_ATTN_INVALID_ARGUMENT;
  h->timing = enabled != 0;
  h->timed = false;
  return MI355_ATTN_OK;
}

float mi355_attn_last_kernel_ms(mi355_attn* h) {
  if (!h || !h->timed) return -1.f;
  if (hipEventSynchronize(h->ev1) != hipSuccess) return -1.f;
  float ms = -1.f;
  if (hipEventElapsedTime(&ms, h->ev0, h->ev1) != hipSuccess) return -1.f;
  return ms;
}

int mi355_attn_set_option(mi355_attn* h, const char* name, int32_t value) {
  if (!h || !name) return MI355_ATTN_INVALID_ARGUMENT;
  if (!strcmp(name, "decode_waves")) {
    if (value != 0 && value != 1 && value != 2 && value != 4) return MI355_ATTN_INVALID_ARGUMENT;
    h->tuning.waves = value;
  } else if (!strcmp(name, "rowwise_prefill")) {
    h->rowwise_prefill = value != 0;
  } else if (!strcmp(name, "prefill_workgroups")) {
    if (value < 0) return MI355_ATTN_INVALID_ARGUMENT;
    h->prefill_workgroups = value;
  } else if (!strcmp(name, "prefill_rows16")) {
    if (value < -1 || value > 1) return MI355_ATTN_INVALID_ARGUMENT;
    h->prefill_rows16 = value;
  } else if (!strcmp(name, "prefill_i8_stage_mib")) {
    if (value < 1) return MI355_ATTN_INVALID_ARGUMENT;
    h->prefill_i8_stage_mib = value;
  } else if (!strcmp(name, "prefill_i8_min_rows")) {
    if (value < 1) return MI355_ATTN_INVALID_ARGUMENT;
    h->prefill_i8_min_rows = value;
  } else if (!strcmp(name, "prefill_key_split")) {
    if (value < -1 || value > 4096) return MI355_ATTN_INVALID_ARGUMENT;
    h->prefill_key_split = value;
  } else {
    return MI355_ATTN_INVALID_ARGUMENT;
  }
  return MI355_ATTN_OK;
}

uint64_t mi355_attn_cache_bytes(const mi355_attn* h) { return h ? h->cache_bytes : 0; }

}  // extern "C"
