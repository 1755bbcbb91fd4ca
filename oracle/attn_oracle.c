/*
 * CPU oracle for the attention hot path, plain C (TEST INFRASTRUCTURE).
 *
 * Only tests, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may
 * load this library, and only as the checker / reported CPU baseline. The
 * product library (include/mi355_attn.h) never links or calls it.
 *
 * The attention arithmetic of the reference runs inside
 * litert::CompiledModel::Run
 * (runtime/executor/llm_litert_compiled_model_executor.cc:271,407,522), i.e.
 * in LiteRT @c8f55dfb / TFLite+XNNPACK @734f7085 (WORKSPACE:6-9,73-78,261-270),
 * which are not vendored. What the reference tree fixes and this file follows:
 *   - the causal float mask and its constants
 *     (runtime/executor/litert_compiled_model_executor_utils.cc:332-397);
 *   - max-subtracted softmax in the style of
 *     runtime/components/sampling_cpu_util.cc:94-131.
 * The rest restates the published scaled-dot-product-attention definition in
 * the op order the call sites imply: scale -> QK^T -> + mask -> softmax -> PV,
 * GQA by KV-head broadcast (kv_head = q_head / (Hq / Hkv)).
 *
 * PARITY UNPINNED: fp32 bit patterns of XNNPACK; the sliding-window boundary
 * (here 0 <= p - j < window); the soft-cap form (cap * tanh(s / cap)).
 *
 * Tensor layouts: q, out [n_q][Hq][D]; k, v [L][Hkv][D], all row-major.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <float.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_MASK_NEG_F16 (-45824.0f)

/* utils.cc:332-359 then :361-397 for a float mask of `rows` x `ctx`. */
void oracle_fill_mask_f32(float* mask, int rows, int ctx, int start_timestep, int steps, int is_f16) {
  const float neg = is_f16 ? ORACLE_MASK_NEG_F16 : -0.7f * FLT_MAX;
  for (long i = 0; i < (long)rows * ctx; ++i) mask[i] = neg;
  for (int i = 0; i < steps; ++i) {
    float* row = mask + (long)i * ctx;
    for (int j = 0; j <= start_timestep + i && j < ctx; ++j) row[j] = 0.0f;
  }
}

static int key_visible(int p, int j, int window) {
  if (j > p) return 0;
  if (window > 0 && p - j >= window) return 0;
  return 1;
}

/*
 * fp64-accumulating attention by predicate. Query row i sits at absolute
 * position q_pos0 + i and sees keys j < kv_len with j <= p and, if window > 0,
 * p - j < window. Returns 0 on success.
 */
int oracle_sdpa_f64(const float* q, const float* k, const float* v, int n_q, int hq, int hkv, int d,
                    int kv_len, float scale, float softcap, int q_pos0, int window, double* out) {
  if (hkv <= 0 || hq % hkv) return 3;
  const int group = hq / hkv;
  double* s = (double*)malloc(sizeof(double) * (size_t)(kv_len > 0 ? kv_len : 1));
  if (!s) return 8;
  for (int i = 0; i < n_q; ++i) {
    const int p = q_pos0 + i;
    for (int h = 0; h < hq; ++h) {
      const int kvh = h / group;
      const float* qr = q + ((size_t)i * hq + h) * d;
      double m = -INFINITY;
      for (int j = 0; j < kv_len; ++j) {
        if (!key_visible(p, j, window)) { s[j] = -INFINITY; continue; }
        const float* kr = k + ((size_t)j * hkv + kvh) * d;
        double acc = 0.0;
        for (int c = 0; c < d; ++c) acc += ((double)qr[c] * (double)scale) * (double)kr[c];
        if (softcap > 0.0f) acc = (double)softcap * tanh(acc / (double)softcap);
        s[j] = acc;
        if (acc > m) m = acc;
      }
      double* o = out + ((size_t)i * hq + h) * d;
      for (int c = 0; c < d; ++c) o[c] = 0.0;
      if (!(m > -INFINITY)) continue;
      double den = 0.0;
      for (int j = 0; j < kv_len; ++j) {
        if (s[j] == -INFINITY) { s[j] = 0.0; continue; }
        s[j] = exp(s[j] - m);
        den += s[j];
      }
      for (int j = 0; j < kv_len; ++j) {
        if (s[j] == 0.0) continue;
        const float* vr = v + ((size_t)j * hkv + kvh) * d;
        const double pj = s[j] / den;
        for (int c = 0; c < d; ++c) o[c] += pj * (double)vr[c];
      }
    }
  }
  free(s);
  return 0;
}

/*
 * fp32 restatement of the reference CPU op order with an additive mask, used
 * as the timed CPU stand-in. One (query row, head) problem:
 *   qs = q * scale;  s = qs . K^T;  s += mask_row;  softmax;  o = p . V
 * mask_row may be NULL, in which case keys j >= n_keys_visible are skipped
 * (equivalent to the -45824 mask: exp underflows to exactly 0).
 */
static void head_attention_f32(const float* qr, const float* k, const float* v, int hkv, int kvh, int d,
                               int ctx, const float* mask_row, float scale, float* scratch, float* o) {
  float qs[1024];
  for (int c = 0; c < d; ++c) qs[c] = qr[c] * scale;
  float m = -INFINITY;
  for (int j = 0; j < ctx; ++j) {
    const float* kr = k + ((size_t)j * hkv + kvh) * d;
    float acc = 0.0f;
    for (int c = 0; c < d; ++c) acc += qs[c] * kr[c];
    if (mask_row) acc += mask_row[j];
    scratch[j] = acc;
    if (acc > m) m = acc;
  }
  float den = 0.0f;
  for (int j = 0; j < ctx; ++j) {
    scratch[j] = expf(scratch[j] - m);
    den += scratch[j];
  }
  const float inv = 1.0f / den;
  for (int c = 0; c < d; ++c) o[c] = 0.0f;
  for (int j = 0; j < ctx; ++j) {
    const float pj = scratch[j] * inv;
    if (pj == 0.0f) continue;
    const float* vr = v + ((size_t)j * hkv + kvh) * d;
    for (int c = 0; c < d; ++c) o[c] += pj * vr[c];
  }
}

/*
 * Prefill/decode of one sequence with an additive [n_q][ctx] float mask (as the
 * reference executor would hand to the graph). d <= 1024. threads <= 0 means the
 * OpenMP default. Returns 0 on success.
 */
int oracle_sdpa_ref_f32(const float* q, const float* k, const float* v, int n_q, int hq, int hkv, int d,
                        int ctx, const float* mask, float scale, int threads, float* out) {
  if (hkv <= 0 || hq % hkv || d > 1024) return 3;
  const int group = hq / hkv;
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#endif
  const long total = (long)n_q * hq;
#pragma omp parallel
  {
    float* scratch = (float*)malloc(sizeof(float) * (size_t)(ctx > 0 ? ctx : 1));
#pragma omp for schedule(dynamic, 1)
    for (long t = 0; t < total; ++t) {
      const int i = (int)(t / hq), h = (int)(t % hq);
      head_attention_f32(q + ((size_t)i * hq + h) * d, k, v, hkv, h / group, d, ctx,
                         mask ? mask + (size_t)i * ctx : NULL, scale, scratch,
                         out + ((size_t)i * hq + h) * d);
    }
    free(scratch);
  }
  return 0;
}

/*
 * Batched one-token decode in the same fp32 op order: sequence b has its own
 * contiguous cache k_ptrs[b], v_ptrs[b] of lens[b] rows; q, out [B][Hq][D].
 * The mask of the reference (one row, keys 0..len-1 open) is applied by
 * bounding the key loop, which is bit-identical to adding 0 / -45824.
 */
int oracle_decode_batch_ref_f32(const float* q, const float* const* k_ptrs, const float* const* v_ptrs,
                                const int32_t* lens, int batch, int hq, int hkv, int d, float scale,
                                int threads, float* out) {
  if (hkv <= 0 || hq % hkv || d > 1024) return 3;
  const int group = hq / hkv;
  int max_len = 1;
  for (int b = 0; b < batch; ++b) if (lens[b] > max_len) max_len = lens[b];
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#endif
  const long total = (long)batch * hq;
#pragma omp parallel
  {
    float* scratch = (float*)malloc(sizeof(float) * (size_t)max_len);
#pragma omp for schedule(dynamic, 1)
    for (long t = 0; t < total; ++t) {
      const int b = (int)(t / hq), h = (int)(t % hq);
      head_attention_f32(q + ((size_t)b * hq + h) * d, k_ptrs[b], v_ptrs[b], hkv, h / group, d, lens[b],
                         NULL, scale, scratch, out + ((size_t)b * hq + h) * d);
    }
    free(scratch);
  }
  return 0;
}

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
