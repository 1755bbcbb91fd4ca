/*
 * mi355_attn.h - C ABI of the MI355X (gfx950) attention library.
 *
 * The library owns a KV cache in HBM and runs scaled-dot-product attention over
 * it: causal prefill (global and sliding-window layers) and one-token decode
 * (GQA/MQA, split-KV partitions merged by log-sum-exp). It is the thin layer a
 * C++ LlmExecutor implementation calls where the reference executor calls
 * litert::CompiledModel::Run.
 *
 * Conventions follow the reference's own dlopen'd plugin ABI
 * (runtime/components/sampler_factory.cc:34-57,119-133,156-188):
 *   - every call returns an absl::StatusCode integer (0 = OK);
 *   - `char** error_msg` (may be NULL) receives a malloc'd message that the
 *     caller releases with free();
 *   - plain C types only; nothing throws across the boundary.
 * A handle is not thread-safe: like the reference executor it is driven from
 * one worker thread (runtime/core/engine_impl.cc:185-186).
 *
 * Tensor layouts at the boundary (row-major, dense):
 *   q, out : [n][num_q_heads][head_dim]          io_dtype
 *   k, v   : [n][num_kv_heads][head_dim]         kv_dtype
 *   scales : [num_kv_heads][head_dim]            float32 (int8 cache only)
 * Query head h reads KV head h / (num_q_heads / num_kv_heads).
 * Cache type and activation type (io_dtype: queries in, attention out) are set
 * apart as the reference sets them apart (ActivationDataType,
 * runtime/executor/executor_settings_base.h:54-66; its GPU path keeps an fp16
 * cache under fp32 activations when asked,
 * llm_litert_compiled_model_executor.cc:609-617). Pairs: io_dtype equal to
 * kv_dtype (f32, f16, bf16); f32 activations over an f16 or bf16 cache; an
 * int8 cache under f16, bf16 or f32 activations. The matrix cores take the
 * queries in the cache's operand type: float32 queries over a 16-bit cache
 * are rounded to it (nearest even) on the way in (a prefill call does so in a
 * pass of its own over the query rows), products accumulate in float32 and
 * the output is written in io_dtype from those sums.
 * An int8 cache enters the matrix cores as IEEE half values. Decode converts in
 * registers (K scales folded into the queries, V scales applied to the sums). A
 * prefill call of 16 rows or more first turns the planes it reads into half
 * planes in a staging area of the handle (2 bytes per cache byte of the layers of
 * a pass, grown on demand up to "prefill_i8_stage_mib"; the call runs in passes
 * over as many layers as fit), V as half(value x scale), K as the values
 * themselves with the scales folded into float32 / bfloat16 queries on their way
 * to half, or as half(value x scale) under half queries, which are read as they
 * are; smaller calls, and calls that would have to allocate while the stream is
 * being captured, run row by row through the decode kernel.
 * A bfloat16 cache keeps its K planes in bfloat16 and its V planes as IEEE half
 * values, so that the probabilities multiply V with 11 significant bits on the
 * fp16 matrix-core path: a bfloat16 value v is stored without loss for
 * 2^-17 <= |v| <= 65504, larger magnitudes saturate at +-65504 and smaller ones
 * round to the nearest multiple of 2^-24 (mi355_attn_kv_read returns what is stored).
 * Key j is visible to the query at absolute position p iff j <= p and, on a
 * layer with window W > 0, p - j < W.
 */
#ifndef MI355_ATTN_H_
#define MI355_ATTN_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mi355_attn mi355_attn;

/* Element types. */
enum {
  MI355_ATTN_F32 = 0,
  MI355_ATTN_F16 = 1,
  MI355_ATTN_BF16 = 2,
  MI355_ATTN_I8 = 3 /* kv_dtype only: symmetric int8, per-(kv head, channel) scale */
};

/* absl::StatusCode values used by this library. */
enum {
  MI355_ATTN_OK = 0,
  MI355_ATTN_INVALID_ARGUMENT = 3,
  MI355_ATTN_RESOURCE_EXHAUSTED = 8,
  MI355_ATTN_FAILED_PRECONDITION = 9,
  MI355_ATTN_OUT_OF_RANGE = 11,
  MI355_ATTN_UNIMPLEMENTED = 12,
  MI355_ATTN_INTERNAL = 13,
  MI355_ATTN_UNAVAILABLE = 14
};

/*
 * Static description of one executor's attention stack. Plays the part that the
 * .tflite signature shapes plus LlmExecutorSettings play in the reference
 * (runtime/executor/llm_executor_settings.h:95-154: max_num_tokens is the KV
 * capacity; runtime/executor/llm_litert_compiled_model_executor.cc:716-761:
 * one K and one V tensor per layer).
 */
typedef struct mi355_attn_config {
  uint32_t struct_size;        /* sizeof(mi355_attn_config) */
  int32_t num_layers;
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t head_dim;            /* 256 */
  int32_t max_tokens;          /* KV rows per sequence */
  int32_t max_seqs;            /* sequences (cache slots) held at once */
  int32_t kv_dtype;            /* MI355_ATTN_* */
  int32_t io_dtype;            /* MI355_ATTN_F32 / F16 / BF16 */
  float scale;                 /* 0 => head_dim^-0.5 */
  float softcap;               /* 0 => off; else cap * tanh(s / cap) */
  const int32_t* layer_window; /* [num_layers], 0 = global layer; NULL = all global */
  int32_t device;              /* HIP device ordinal */
  int32_t host_io;             /* 0: q/k/v/out/scales are device pointers;
                                  1: host pointers, staged by the library and
                                     every call returns with results in place */
  int32_t own_stream;          /* 1: run on a new non-blocking stream owned by the handle
                                  (`stream` is ignored); 0: run on `stream` */
  void* stream;                /* hipStream_t; NULL = the HIP default stream */
} mi355_attn_config;

/*
 * Builds the handle and its zero-initialised KV cache.
 * Replaces: LlmLiteRtCompiledModelExecutor::Create's KV-buffer allocation
 * (runtime/executor/llm_litert_compiled_model_executor.cc:705-761).
 * kUnavailable when no gfx950 device can be used.
 */
int mi355_attn_create(const mi355_attn_config* config, mi355_attn** out, char** error_msg);

void mi355_attn_destroy(mi355_attn* handle);

/*
 * Writes n new K/V rows of one layer of sequence `seq` at rows pos .. pos+n-1.
 * Replaces: the in-graph KV update behind compiled_model_.Run, visible in tree
 * as the cache tensors being both inputs and outputs of every signature
 * (llm_litert_compiled_model_executor.cc:733-757) and as the explicit
 * cache-update signature of the NPU flow
 * (llm_litert_npu_compiled_model_executor.cc:105-110,1294-1333).
 * For an int8 cache k and v hold int8 values; set the scales with
 * mi355_attn_kv_set_scales.
 * Rows count as appended (for the checks of prefill and decode) while they extend
 * the unbroken prefix [0, rows appended so far) of their layer and sequence: rows
 * written behind a gap are stored but not counted, so the unwritten rows of the
 * gap (or, after mi355_attn_reset, a previous sequence's) are never attended to.
 */
int mi355_attn_kv_append(mi355_attn* handle, int32_t layer, int32_t seq, int32_t pos, int32_t n,
                         const void* k, const void* v, char** error_msg);

/* int8 cache: per-(kv head, channel) dequantisation scales of (layer, seq). */
int mi355_attn_kv_set_scales(mi355_attn* handle, int32_t layer, int32_t seq, const float* k_scale,
                             const float* v_scale, char** error_msg);

/*
 * Per-layer constants of the step before attention (mi355_attn_pre_attention).
 * All pointers are HOST arrays (whatever host_io says), copied before the call
 * returns. In the reference these are weights and tables of the model graph:
 * the NPU flow computes the rotary cos / sin tables for local and global layers
 * from `input_pos` in a signature of its own
 * (llm_litert_npu_compiled_model_executor.cc:82-94,1209-1219), the norms sit in
 * the transformer stack behind compiled_model_.Run.
 *   RMS norm over head_dim:  y = x / sqrt(mean(x^2) + eps) * (weight_offset + weight[d])
 *                            (weight NULL: no learned scale; Gemma 3: weight_offset 1)
 *   rotary embedding:        angle = float32(position) * rope_inv_freq[d], d < head_dim/2;
 *                            (x[d], x[d + head_dim/2]) is rotated by angle
 *                            (the "rotate half" pairing; rope_inv_freq NULL: no rotation).
 *                            A global layer passes theta^(-2d/head_dim) / factor of its
 *                            own theta, a local layer that of the local theta.
 */
typedef struct mi355_attn_layer_transform {
  uint32_t struct_size;       /* sizeof(mi355_attn_layer_transform) */
  int32_t norm_q;             /* != 0: RMS-normalise every query head */
  int32_t norm_k;             /* != 0: RMS-normalise every key head */
  int32_t norm_v;             /* != 0: RMS-normalise every value head, no learned scale */
  const float* q_weight;      /* [head_dim] or NULL */
  const float* k_weight;      /* [head_dim] or NULL */
  float eps;                  /* >= 0 */
  float weight_offset;
  const float* rope_inv_freq; /* [head_dim / 2] or NULL */
} mi355_attn_layer_transform;

/* Sets the constants of one layer; waits for the work queued on the handle first. */
int mi355_attn_set_layer_transform(mi355_attn* handle, int32_t layer, const mi355_attn_layer_transform* transform,
                                   char** error_msg);

/*
 * The step before attention for n new tokens of one layer of sequence `seq` at
 * positions pos .. pos+n-1, in one launch: RMS norm of q / k (/ v), rotary
 * embedding of q and k (as set by mi355_attn_set_layer_transform; a layer
 * without constants gets neither), q_out = the query rows attention reads
 * (io_dtype, may be q itself), and the key / value rows written into the cache
 * exactly as mi355_attn_kv_append would write them.
 * q [n][num_q_heads][head_dim], k, v [n][num_kv_heads][head_dim], all io_dtype.
 * int8 cache: the rows are quantised with the scales set by
 * mi355_attn_kv_set_scales, value = clamp(round(x * (1 / scale)), -127, 127)
 * (round half away from zero; a zero scale stores 0).
 * Replaces: the RoPE and cache-update signatures of the NPU flow
 * (llm_litert_npu_compiled_model_executor.cc:82-110,1209-1219,1294-1333) and
 * its float -> integer quantise step (:116-148); in the CPU/GPU executor the
 * same work is inside compiled_model_.Run
 * (llm_litert_compiled_model_executor.cc:271,407,522).
 */
int mi355_attn_pre_attention(mi355_attn* handle, int32_t layer, int32_t seq, int32_t pos, int32_t n,
                             const void* q, const void* k, const void* v, void* q_out, char** error_msg);

/* Reads cache rows pos .. pos+n-1 back in boundary layout (tests, debugging). */
int mi355_attn_kv_read(mi355_attn* handle, int32_t layer, int32_t seq, int32_t pos, int32_t n, void* k_out,
                       void* v_out, char** error_msg);

/*
 * Prefill attention of one layer: n query rows at absolute positions
 * q_pos0 .. q_pos0+n-1 of sequence `seq` over cache rows [0, q_pos0+n), causal,
 * windowed on local layers. The rows' own K/V must already be appended.
 * Replaces: the attention inside compiled_model_.Run(prefill_signature, ...)
 * (llm_litert_compiled_model_executor.cc:271) together with the causal mask
 * the executor builds for it
 * (runtime/executor/litert_compiled_model_executor_utils.cc:332-397).
 */
int mi355_attn_prefill(mi355_attn* handle, int32_t layer, int32_t seq, int32_t q_pos0, int32_t n,
                       const void* q, void* out, char** error_msg);

/*
 * Same for n_layers consecutive layers in one launch; q and out are
 * [n_layers][n][num_q_heads][head_dim]. The layers' problems are independent
 * (throughput sweeps; a real forward pass calls mi355_attn_prefill per layer).
 */
int mi355_attn_prefill_layers(mi355_attn* handle, int32_t layer_begin, int32_t n_layers, int32_t seq,
                              int32_t q_pos0, int32_t n, const void* q, void* out, char** error_msg);

/*
 * One-token decode attention of one layer for `batch` sequences.
 * seq_ids[b] (host array, NULL = 0..batch-1) names the cache slot and
 * kv_lens[b] (host array) the number of valid rows, the new token's row
 * included: the query of item b sits at position kv_lens[b]-1.
 * num_splits >= 1 cuts each key range into that many partitions whose partial
 * (max, sum, accumulator) are merged by log-sum-exp; 0 lets the library choose.
 * Replaces: the attention inside compiled_model_.Run("decode", ...)
 * (llm_litert_compiled_model_executor.cc:407,522) and its one-row mask
 * (:485-492).
 */
int mi355_attn_decode(mi355_attn* handle, int32_t layer, const int32_t* seq_ids, const int32_t* kv_lens,
                      int32_t batch, const void* q, void* out, int32_t num_splits, char** error_msg);

/* n_layers consecutive layers in one launch; q, out [n_layers][batch][Hq][D]. */
int mi355_attn_decode_layers(mi355_attn* handle, int32_t layer_begin, int32_t n_layers,
                             const int32_t* seq_ids, const int32_t* kv_lens, int32_t batch, const void* q,
                             void* out, int32_t num_splits, char** error_msg);

/*
 * One decode step of one layer in one launch: mi355_attn_pre_attention for the
 * one new token of each of `batch` sequences (its row is kv_lens[b] - 1) and
 * mi355_attn_decode over rows [0, kv_lens[b]). q [batch][num_q_heads][head_dim],
 * k, v [batch][num_kv_heads][head_dim] are the raw projections (io_dtype); the
 * normed / rotated key and value rows end up in the cache as
 * mi355_attn_pre_attention leaves them, and `out` holds, bit for bit, what the
 * two calls produce. Rows [0, kv_lens[b] - 1) must have been appended; the
 * sequences of one call must differ. A launch carries up to 64 sequences; a
 * larger batch runs as several launches queued back to back (everything that
 * can be refused is checked for the whole batch before the first).
 * Replaces: one layer's share of compiled_model_.Run("decode", ...)
 * (llm_litert_compiled_model_executor.cc:407,522: cache update and attention
 * are one graph invocation there) and, in the NPU flow, its RoPE, cache-update
 * and attention signatures in turn
 * (llm_litert_npu_compiled_model_executor.cc:1337-1530).
 */
int mi355_attn_decode_step(mi355_attn* handle, int32_t layer, const int32_t* seq_ids, const int32_t* kv_lens,
                           int32_t batch, const void* q, const void* k, const void* v, void* out,
                           int32_t num_splits, char** error_msg);

/*
 * mi355_attn_decode for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc. It has no
 * counterpart in the reference. Same arguments, same kernels and bit-identical
 * results, but the split-KV partials go to a fixed workspace that is part of the
 * library image (8 MiB per GPU, held until the process ends) instead of the
 * handle's growable one, and the call makes no hipMalloc / hipFree.
 * Limits: the handle must use device pointers (host_io = 0, else
 * kFailedPrecondition); batch x num_q_heads x num_splits <= 8192 partial results
 * (an explicit num_splits beyond that is kResourceExhausted; with num_splits = 0
 * the library chooses within the limit). All calls on one GPU share the
 * workspace. Calls queued on one stream never overlap. Eager calls on different
 * streams are ordered by the library (each waits, on its stream, for the event
 * the previous one left), so they do not overlap either. Calls recorded into HIP
 * graphs are not ordered against anything outside their graph: replays of two
 * graphs (or a replay and an eager call) that run at the same time on one GPU
 * race in the workspace - keep them on one stream.
 * Under capture (this entry point, mi355_attn_decode and mi355_attn_decode_step
 * alike): up to 64 sequences per call (more need an upload that a capture cannot
 * hold: kFailedPrecondition); kv_lens and seq_ids are baked into the recorded
 * launch, so a replay attends exactly the rows of the captured call - one graph
 * per position - and does not advance the handle's count of appended rows.
 */
int mi355_attn_decode_noalloc(mi355_attn* handle, int32_t layer, const int32_t* seq_ids, const int32_t* kv_lens,
                              int32_t batch, const void* q, void* out, int32_t num_splits, char** error_msg);

/*
 * Host only, no device needed (tests of the planner; no counterpart in the reference): the work plan that a
 * prefill launch of n rows at q_pos0 over n_layers layers gets on `workgroups` workgroups of a part with
 * `compute_units` compute units (the kernel on 16x16x32 MFMAs: which workgroup runs which (layer, head block,
 * 32-position tile) items). items_per_wg / blocks_per_wg: [workgroups] out, the items and the key blocks of each
 * workgroup; items_off_home (may be NULL): items placed on another XCD than most of their layer's.
 * Returns the number of items (every item of the launch exactly once), < 0 on bad arguments or a broken plan.
 */
int mi355_attn_prefill_plan_probe(int32_t n_layers, int32_t n, int32_t q_pos0, int32_t num_q_heads,
                                  int32_t num_kv_heads, const int32_t* layer_window, int32_t workgroups,
                                  int32_t compute_units, int32_t* items_per_wg, int32_t* blocks_per_wg,
                                  int32_t* items_off_home);

/*
 * Measurement aid, no counterpart in the reference: streams `bytes` of the KV
 * cache, starting `offset` bytes into it, through `workgroups` workgroups of
 * `waves` waves with the decode kernel's load pattern (non-temporal 16-byte
 * loads, 32 KiB per wave in flight) and does nothing with the data. With
 * mi355_attn_set_timing on, mi355_attn_last_kernel_ms then returns the floor
 * for a decode launch of that many bytes and that launch shape: dispatch,
 * first-load latency and the memory's rate, no arithmetic. The cache is not
 * changed. kOutOfRange when the shares (rounded up to whole 32 KiB pieces per
 * wave) would pass the end of the cache.
 */
int mi355_attn_stream_probe(mi355_attn* handle, uint64_t offset, uint64_t bytes, int32_t workgroups, int32_t waves,
                            char** error_msg);

/*
 * Forgets the rows of sequence `seq` (seq < 0: all). Like
 * LlmLiteRtCompiledModelExecutor::Reset
 * (llm_litert_compiled_model_executor.cc:568-574) the cache memory itself is
 * not cleared; stale rows are never visible because visibility is bounded by
 * the positions the caller passes.
 */
int mi355_attn_reset(mi355_attn* handle, int32_t seq, char** error_msg);

/* Blocks until all work queued on the handle's stream has finished. */
int mi355_attn_sync(mi355_attn* handle, char** error_msg);

/* The stream work is queued on (hipStream_t). */
void* mi355_attn_stream(mi355_attn* handle);

/*
 * Duration in milliseconds of the kernel of the most recent
 * prefill / decode / pre_attention call, measured with HIP events on the handle's stream
 * (the split-merge pass is excluded). Blocks until that call has finished.
 * Timing is recorded only after mi355_attn_set_timing(handle, 1).
 */
int mi355_attn_set_timing(mi355_attn* handle, int32_t enabled);
float mi355_attn_last_kernel_ms(mi355_attn* handle);

/*
 * Tuning and cross-check switches (return kInvalidArgument for unknown names):
 *   "decode_waves"     1, 2 or 4 waves per decode workgroup, 0 (default) = chosen
 *                      from the number of workgroups of the launch
 *   "rowwise_prefill"  0/1 run prefill row by row through the decode kernel
 *                      (the only path for an fp32 cache)
 *   "prefill_i8_min_rows" int8 cache: prefill calls of fewer rows run row by row
 *                      (default 16)
 *   "prefill_i8_stage_mib" int8 cache: limit of the staging area for half planes,
 *                      MiB (default 2048; one layer's planes are staged even when
 *                      they exceed it)
 *   "prefill_workgroups" upper bound of the persistent workgroups of the prefill
 *                      kernel, 0 (default) = one per compute unit
 *   "prefill_rows16"   which of the two prefill kernels runs: 1 the one on 16x16x32 MFMAs
 *                      (four waves of 32 query positions, 80 KiB of LDS, two workgroups
 *                      per compute unit), 0 the one on 32x32x16 MFMAs (one workgroup per
 *                      compute unit), -1 (default): the first when the launch has at least
 *                      two work items per compute unit, else the second
 *   "prefill_key_split" -1 (default): a prefill launch with fewer work items than
 *                      three quarters of the compute units (a single layer, say) cuts
 *                      the key range of its tiles into up to 8 work items each and
 *                      merges their results in a second kernel; the fp32 parts go to a
 *                      workspace allocated on first use, [layers][rows][heads][parts]
 *                      x (head_dim + 2) floats, at most 258 MiB (else no split).
 *                      0: never; n > 0: n key blocks (of 32 keys) per work item
 */
int mi355_attn_set_option(mi355_attn* handle, const char* name, int32_t value);

/* Bytes of HBM held by the KV cache of this handle. */
uint64_t mi355_attn_cache_bytes(const mi355_attn* handle);

/* Library version string, e.g. "mi355_attn 0.1 (gfx950)". */
const char* mi355_attn_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MI355_ATTN_H_ */
