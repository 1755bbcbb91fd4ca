// Launchers of the gfx950 kernels; the C ABI in mi355_attn.hip validates
// shapes on the host and then calls these.
#ifndef LITERT_LM_AMD_CSRC_KERNELS_H_
#define LITERT_LM_AMD_CSRC_KERNELS_H_

#include <hip/hip_runtime.h>

#include "attn_params.h"

namespace mi355 {

struct DecodeTuning {
  int waves = 0;  // waves per workgroup: 1, 2 or 4; 0 picks by workgroup count
};

bool decode_supported(int kv_dtype, int io_dtype, int head_dim);

// Queues the decode attention kernel (bracketed by ev0/ev1 when non-null) and,
// for num_splits > 1, the log-sum-exp merge kernel.
hipError_t launch_decode(const DecodeArgs& args, int kv_dtype, int io_dtype, const DecodeTuning& tuning,
                         hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1);

bool prefill_supported(int kv_dtype, int io_dtype, int head_dim);
// Bytes of half planes that a prefill over an int8 cache stages for `n_layers` layers of a call ending at row `end`.
int64_t prefill_i8_stage_bytes(const CacheGeom& geom, int n_layers, int end);

// Key split of a prefill launch (PrefillArgs::kchunk / smax): none (kchunk 0) unless the launch has
// fewer work items than three quarters of the compute units; then at most 8 items per tile of at
// least 4 key blocks each. option > 0 forces that many key blocks per item (tests), option 0 is off,
// option < 0 the rule above. Reads n_layers, geom.hkv, group, n, q_pos0, layer_begin, host_window.
struct PrefillSplit {
  int kchunk = 0, smax = 1;
  size_t rows = 0;  // rows of the workspace: n_layers * n * hq * smax
};
PrefillSplit plan_prefill_split(const PrefillArgs& args, int option);

// Work plans of the prefill kernel on 16x16x32 MFMAs, kept by the handle: which workgroup runs which work items
// in which order, computed on the host (longest processing time first over the workgroups: an item's time is
// known from its number of key blocks) and cached by launch shape. A slot's device copy is rewritten only
// after the last launch that reads it has finished (`used`); a slot whose launch was captured into a HIP graph
// is kept for good (`pinned`: the graph may be replayed at any time). A new shape takes the least recently used
// slot that is not pinned. A launch that cannot get a plan - a shape seen for the first time while its stream is
// being captured, or all slots pinned - runs on the other prefill kernel, which needs none: same results to the
// tolerance, not bit for bit.
struct PrefillPlans {
  static constexpr int kSlots = 4;
  int32_t* d_words[kSlots] = {};
  int32_t* h_words[kSlots] = {};  // pinned staging
  size_t cap[kSlots] = {};        // words
  hipEvent_t used[kSlots] = {};
  int64_t key[kSlots][8] = {};
  bool valid[kSlots] = {};
  bool pinned[kSlots] = {};
  uint64_t last_use[kSlots] = {};
  uint64_t clock = 0;
};
void free_prefill_plans(PrefillPlans* plans);

// Host only (no device is touched): the plan of a launch of n query rows at q_pos0 over n_layers layers on `wgs`
// workgroups of a part with `cus` compute units. items_per_wg / blocks_per_wg: [wgs] out; items_off_home (may be
// null): items that run on another XCD than most of their layer. Returns the number of items, -1 for bad
// arguments, -2 when an item appears twice, -3 when one is missing.
int prefill_plan_probe(int n_layers, int n, int q_pos0, int hq, int hkv, const int32_t* layer_window, int wgs, int cus,
                       int32_t* items_per_wg, int32_t* blocks_per_wg, int32_t* items_off_home);

// With args.kchunk > 0 the merge kernel follows the attention kernel (ev1 then marks the end of the
// attention kernel alone).
hipError_t launch_prefill(const PrefillArgs& args, int kv_dtype, int io_dtype, PrefillPlans* plans,
                          hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1);

// Scatter n boundary-layout rows into the cache planes / gather them back.
hipError_t launch_kv_append(const KvCopyArgs& args, hipStream_t stream);
hipError_t launch_kv_read(const KvCopyArgs& args, hipStream_t stream);

// Streams `bytes` of the cache from `offset` on with the decode kernel's load pattern and nothing else (the floor a
// decode launch of that many bytes and that shape is priced against); `sink` is one device word that is never
// written in practice. hipErrorInvalidValue when the share of the last wave would pass the end of the cache.
hipError_t launch_stream_probe(const uint8_t* cache, int64_t cache_bytes, int64_t offset, int64_t bytes, int workgroups,
                               int waves, uint32_t* sink, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1);

// Norm + rotary embedding of n new rows, query written out, key / value rows
// written into the cache planes (quantised for an int8 cache).
hipError_t launch_pre_attention(const PreAttentionArgs& args, int kv_dtype, int io_dtype, hipStream_t stream,
                                hipEvent_t ev0, hipEvent_t ev1);

}  // namespace mi355
#endif  // LITERT_LM_AMD_CSRC_KERNELS_H_
