// The step right before attention, in one pass over the new rows: per-head RMS
// norm of the query / key (/ value) projections, rotary position embedding of
// query and key, the query written out for the attention kernels and the key /
// value rows written straight into the cache planes in MFMA operand order
// (quantised with the plane's fixed scales for an int8 cache).
//
// Replaces, in the reference's NPU flow, the RoPE signature that turns
// `input_pos` into cos / sin tables and the cache-update signature that merges
// the new `kv_slice_{k,v}_i` rows at `input_pos`
// (runtime/executor/llm_litert_npu_compiled_model_executor.cc:82-110,1209-1219,
// 1294-1333); in the CPU/GPU executor the same work sits inside the graph behind
// compiled_model_.Run (llm_litert_compiled_model_executor.cc:271,407,522). The
// int8 write follows the quantise idiom of
// llm_litert_npu_compiled_model_executor.cc:116-148 (reciprocal scale,
// std::round, clamp).
//
// Bound: HBM. Each row of 256 channels is read once and written once; one wave
// owns one (token, head) row, a lane the channel pairs (2l, 2l+1) and
// (128+2l, 128+2l+1), so both members of every rotated pair (d, d+128) are in
// the same lane and the only cross-lane step is the sum of squares of the norm.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include "attn_params.h"
#include "kernels.h"
#include "mfma_util.h"
#include "pre_attn_rows.h"

namespace mi355 {
namespace {

constexpr int kD = kRowD;
constexpr int kRowsPerWg = 4;  // waves per workgroup

template <int IO, int KV>
__global__ void __launch_bounds__(64 * kRowsPerWg) pre_attention_kernel(const PreAttentionArgs a) {
  const int lane = threadIdx.x & 63;
  const int rows_per_token = a.hq + 2 * a.geom.hkv;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerWg + (threadIdx.x >> 6);
  if (row >= (int64_t)a.n * rows_per_token) return;  // whole waves leave; no barrier below
  const int i = (int)(row / rows_per_token);
  const int j = (int)(row % rows_per_token);
  const int kind = j < a.hq ? 0 : (j < a.hq + a.geom.hkv ? 1 : 2);  // 0 = query, 1 = key, 2 = value
  const int head = kind == 0 ? j : (kind == 1 ? j - a.hq : j - a.hq - a.geom.hkv);
  const void* src = kind == 0 ? a.q : (kind == 1 ? a.k : a.v);
  const int heads = kind == 0 ? a.hq : a.geom.hkv;
  const int64_t base = ((int64_t)i * heads + head) * kD;
  const int d0 = 2 * lane, d1 = kD / 2 + 2 * lane;  // the lane's channels: d0, d0+1, d1, d1+1

  float x[4];
  load_pair<IO>(src, base + d0, x[0], x[1]);
  load_pair<IO>(src, base + d1, x[2], x[3]);

  // sine / cosine of the lane's two angles first: they depend on the position
  // only, so their ~200 instructions run while the row's loads are in flight
  const int t = a.pos + i;
  const bool rotate = a.rope && kind != 2;
  const RowAngles ang = row_angles(rotate ? a.constants : nullptr, t, lane);
  const bool norm = kind == 0 ? a.norm_q != 0 : (kind == 1 ? a.norm_k != 0 : a.norm_v != 0);
  transform_row(x, norm, row_weights(a.constants, kind, a.q_scaled != 0, a.k_scaled != 0), a.weight_offset, a.eps, rotate,
                ang, lane);

  if (kind == 0) {
    uint8_t* out = reinterpret_cast<uint8_t*>(a.q_out);
    constexpr int IOSZ = IO == kF32 ? 4 : 2;
    store_pair<IO>(out + (base + d0) * IOSZ, x[0], x[1]);
    store_pair<IO>(out + (base + d1) * IOSZ, x[2], x[3]);
    return;
  }
  const int is_v = kind == 2 ? 1 : 0;
  uint8_t* plane = a.cache + a.geom.plane_offset(a.layer, a.seq, head, is_v);
  const float* sc = KV == kI8 ? a.scales + a.geom.scale_offset(a.layer, a.seq, is_v, head) : nullptr;
  store_cache_row<KV>(plane, sc, is_v, t, x, lane);
}

template <int IO, int KV>
hipError_t launch_typed(const PreAttentionArgs& a, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  const int64_t rows = (int64_t)a.n * (a.hq + 2 * a.geom.hkv);
  const dim3 grid((unsigned)((rows + kRowsPerWg - 1) / kRowsPerWg));
  hipExtLaunchKernelGGL((pre_attention_kernel<IO, KV>), grid, dim3(64 * kRowsPerWg), 0, stream, ev0, ev1, 0, a);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_pre_attention(const PreAttentionArgs& a, int kv_dtype, int io_dtype, hipStream_t stream,
                                hipEvent_t ev0, hipEvent_t ev1) {
  if (a.n <= 0) return hipSuccess;
  if (a.geom.head_dim != kD) return hipErrorInvalidValue;
  switch (kv_dtype * 4 + io_dtype) {
    case kF32 * 4 + kF32: return launch_typed<kF32, kF32>(a, stream, ev0, ev1);
    case kF16 * 4 + kF16: return launch_typed<kF16, kF16>(a, stream, ev0, ev1);
    case kF16 * 4 + kF32: return launch_typed<kF32, kF16>(a, stream, ev0, ev1);
    case kBF16 * 4 + kBF16: return launch_typed<kBF16, kBF16>(a, stream, ev0, ev1);
    case kBF16 * 4 + kF32: return launch_typed<kF32, kBF16>(a, stream, ev0, ev1);
    case kI8 * 4 + kF16: return launch_typed<kF16, kI8>(a, stream, ev0, ev1);
    case kI8 * 4 + kBF16: return launch_typed<kBF16, kI8>(a, stream, ev0, ev1);
    case kI8 * 4 + kF32: return launch_typed<kF32, kI8>(a, stream, ev0, ev1);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace mi355
