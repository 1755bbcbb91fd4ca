/*
 * mi355_sampler.h - C ABI of the MI355X (gfx950) token sampler.
 *
 * One kernel launch per call turns a [batch, vocab] tensor of float32 logits
 * that is already in HBM (the step right after the attention path) into one
 * token id per row: top-k selection, softmax with temperature over the k
 * candidates, top-p nucleus, one draw. Nothing but the ids (and optionally
 * their scores) has to leave the device.
 *
 * It stands where the reference loads its GPU sampler plugin:
 *   runtime/components/sampler.h:10-25          Sampler::SampleToIdAndScoreBuffer
 *   runtime/components/sampler_factory.cc:34-46 LiteRtTopKOpenClSampler_{Create,Destroy,
 *                                               SampleToIdAndScoreBuffer} (dlopen'd C ABI)
 *   runtime/components/top_p_cpu_sampler.cc:40-112, sampling_cpu_util.cc:21-233
 *                                               the arithmetic (CPU sampler)
 * and keeps that plugin's conventions: every call returns an absl::StatusCode
 * integer (0 = OK), `char** error_msg` (may be NULL) receives a malloc'd message
 * the caller frees, plain C types only, a handle is driven from one thread.
 * The reference passes LiteRtTensorBuffer handles; here they are plain pointers.
 *
 * Arithmetic per row (candidates ordered by descending logit, equal logits by
 * ascending index):
 *   k' = min(k, vocab) candidates; m = largest logit;
 *   e_i = exp((logit_i - m) / max(temperature, FLT_EPSILON)), summed in float32 in
 *   candidate order; sum <= FLT_EPSILON -> all probabilities 1/k'; sum infinite ->
 *   probability 1 for the first candidate; else e_i / sum;
 *   nucleus = shortest prefix whose probabilities (accumulated in float64) reach p;
 *   draw = u * (mass of the nucleus), u in [0, 1); the sampled candidate is the
 *   first whose cumulative probability is >= draw;
 *   score = log(exp((logit - m) / temperature)) (k' == 1: log(1) = 0), which is
 *   what the reference's sampler writes (top_p_cpu_sampler.cc:96-107).
 * This is what the reference's comments describe; as written, its CPU code walks
 * the candidates in the order std::nth_element leaves them (the sort at
 * sampling_cpu_util.cc:186-187 covers an empty range) and always takes the last
 * candidate of the nucleus (no break at :222-229). The two agree wherever the
 * reference's tests hold values.
 */
#ifndef MI355_SAMPLER_H_
#define MI355_SAMPLER_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mi355_sampler mi355_sampler;

/* absl::StatusCode values used by this library. */
enum {
  MI355_SAMPLER_OK = 0,
  MI355_SAMPLER_INVALID_ARGUMENT = 3,
  MI355_SAMPLER_RESOURCE_EXHAUSTED = 8,
  MI355_SAMPLER_UNIMPLEMENTED = 12,
  MI355_SAMPLER_INTERNAL = 13,
  MI355_SAMPLER_UNAVAILABLE = 14
};

/* proto::SamplerParameters::Type (runtime/proto/sampler_params.proto:24-33). */
enum {
  MI355_SAMPLER_TYPE_UNSPECIFIED = 0, /* treated as TOP_P, like the reference's GPU path */
  MI355_SAMPLER_TOP_K = 1,            /* p is ignored (1.0) */
  MI355_SAMPLER_TOP_P = 2,
  MI355_SAMPLER_GREEDY = 3            /* k is ignored (1) */
};

enum { MI355_SAMPLER_MAX_K = 256 };

/*
 * What LiteRtTopKOpenClSampler_Create receives as (batch_size, vocab_size,
 * sampler_params) (sampler_factory.cc:34-38) plus where the tensors live.
 */
typedef struct mi355_sampler_config {
  uint32_t struct_size; /* sizeof(mi355_sampler_config), checked */
  int32_t batch_size;   /* rows per call, > 0 */
  int32_t vocab_size;   /* logits per row, > 0 */
  int32_t type;         /* MI355_SAMPLER_* */
  int32_t k;            /* 1 .. MI355_SAMPLER_MAX_K (values above vocab_size mean vocab_size) */
  float p;              /* in [0, 1] */
  float temperature;    /* > 0 */
  int32_t seed;         /* of the counter-based generator (Philox4x32-10) behind mi355_sampler_sample */
  int32_t device;       /* HIP device ordinal */
  int32_t host_io;      /* != 0: logits / uniforms / ids / scores are host pointers, every call stages and syncs */
  int32_t own_stream;   /* != 0: create a private stream; else use `stream` (NULL = the default stream) */
  void* stream;         /* hipStream_t */
} mi355_sampler_config;

/*
 * Replaces LiteRtTopKOpenClSampler_Create (sampler_factory.cc:34-38) and the
 * argument checks of TopPSampler::Create (top_p_cpu_sampler.cc:40-57):
 * kInvalidArgument for k <= 0, p outside [0,1], batch_size <= 0, temperature <= 0;
 * kUnavailable when no gfx950 device is usable (the reference falls back to its
 * CPU sampler on that code, sampler_factory.cc:248-265).
 */
int mi355_sampler_create(const mi355_sampler_config* config, mi355_sampler** out, char** error_msg);

/* Replaces LiteRtTopKOpenClSampler_Destroy (sampler_factory.cc:40-41). */
void mi355_sampler_destroy(mi355_sampler* sampler);

/*
 * Replaces LiteRtTopKOpenClSampler_SampleToIdAndScoreBuffer
 * (sampler_factory.cc:43-46) / TopPSampler::SampleToIdAndScoreBuffer
 * (top_p_cpu_sampler.cc:59-110).
 * logits [batch_size][vocab_size] float32; ids [batch_size] int32;
 * scores [batch_size] float32 or NULL. The draw of row r in the n-th call on
 * this handle is the 24 high bits of the first word of
 * Philox4x32-10(counter = {r, n, 0, 0}, key = {seed, 0x4D493335}) / 2^24.
 */
int mi355_sampler_sample(mi355_sampler* sampler, const float* logits, int32_t* ids, float* scores,
                         char** error_msg);

/*
 * The same with the draws supplied by the caller (uniforms [batch_size] float32
 * in [0, 1)): no counterpart in the reference, whose generator (absl::BitGen,
 * top_p_cpu_sampler.h:44-48) cannot be reproduced; used for parity tests and by
 * callers that own their random stream.
 */
int mi355_sampler_sample_with_uniforms(mi355_sampler* sampler, const float* logits, const float* uniforms,
                                       int32_t* ids, float* scores, char** error_msg);

/*
 * The intermediate the reference computes in TopKIndicies + Softmax
 * (sampling_cpu_util.cc:21-134): indices [batch_size][k'] and probabilities
 * [batch_size][k'] of the candidates in descending order, k' = min(k, vocab_size).
 */
int mi355_sampler_top_k(mi355_sampler* sampler, const float* logits, int32_t* indices, float* probabilities,
                        char** error_msg);

/* Waits for everything queued on the handle's stream. */
int mi355_sampler_sync(mi355_sampler* sampler, char** error_msg);

/* Duration of the last sampling kernel in milliseconds (after mi355_sampler_set_timing(h, 1)), < 0 if none. */
int mi355_sampler_set_timing(mi355_sampler* sampler, int32_t enabled);
float mi355_sampler_last_kernel_ms(mi355_sampler* sampler);

#ifdef __cplusplus
}
#endif
#endif /* MI355_SAMPLER_H_ */
