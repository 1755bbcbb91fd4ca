// KV-cache update and read-back kernels: move token rows between the boundary
// layout [n][kv_heads][head_dim] and the MFMA-operand layout of the planes.
//
// Replaces the in-graph cache update that the reference reaches through
// compiled_model_.Run (cache tensors are inputs and outputs of every
// signature, runtime/executor/llm_litert_compiled_model_executor.cc:733-757).
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include "attn_params.h"
#include "kernels.h"
#include "mfma_util.h"

namespace mi355 {
namespace {

// One thread per 16-byte chunk of a source row. ESZ = element bytes. VHALF: a bfloat16 cache,
// whose V planes hold IEEE half values (attn_params.h): converted on the way in and out.
template <int ESZ, bool APPEND, bool VHALF>
__global__ void __launch_bounds__(256) kv_copy_kernel(const KvCopyArgs a) {
  constexpr int EPC = 16 / ESZ;
  const int D = a.geom.head_dim;
  const int chunks = D / EPC;
  const int64_t total = (int64_t)a.n * a.geom.hkv * chunks;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  // token index fastest: consecutive threads touch consecutive 16-byte chunks of a K tile
  const int i = (int)(idx % a.n);
  const int c = (int)((idx / a.n) % chunks);
  const int h = (int)(idx / ((int64_t)a.n * chunks));
  const int t = a.pos + i;
  uint8_t* kplane = a.cache + a.geom.plane_offset(a.layer, a.seq, h, 0);
  uint8_t* vplane = kplane + a.geom.plane_bytes;
  const int64_t row = ((int64_t)i * a.geom.hkv + h) * D + (int64_t)c * EPC;  // element index in k / v
  uint8_t* kb = reinterpret_cast<uint8_t*>(a.k) + row * ESZ;
  uint8_t* vb = reinterpret_cast<uint8_t*>(a.v) + row * ESZ;
  u4* kc = reinterpret_cast<u4*>(kplane + k_chunk_offset(t, c, D, ESZ));
  if constexpr (APPEND) {
    *kc = *reinterpret_cast<const u4*>(kb);
    const u4 vw = *reinterpret_cast<const u4*>(vb);
    const uint8_t* src = reinterpret_cast<const uint8_t*>(&vw);
#pragma unroll
    for (int e = 0; e < EPC; ++e) {
      uint8_t* dst = vplane + v_elem_offset(t, c * EPC + e, D, ESZ);
      if constexpr (ESZ == 4) *reinterpret_cast<uint32_t*>(dst) = *reinterpret_cast<const uint32_t*>(src + 4 * e);
      else if constexpr (ESZ == 2) {
        const uint16_t w = *reinterpret_cast<const uint16_t*>(src + 2 * e);
        *reinterpret_cast<uint16_t*>(dst) = VHALF ? bf16_bits_to_half_bits(w) : w;
      } else *dst = src[e];
    }
  } else {
    *reinterpret_cast<u4*>(kb) = *kc;
    u4 vw;
    uint8_t* dstb = reinterpret_cast<uint8_t*>(&vw);
#pragma unroll
    for (int e = 0; e < EPC; ++e) {
      const uint8_t* s = vplane + v_elem_offset(t, c * EPC + e, D, ESZ);
      if constexpr (ESZ == 4) *reinterpret_cast<uint32_t*>(dstb + 4 * e) = *reinterpret_cast<const uint32_t*>(s);
      else if constexpr (ESZ == 2) {
        const uint16_t w = *reinterpret_cast<const uint16_t*>(s);
        *reinterpret_cast<uint16_t*>(dstb + 2 * e) = VHALF ? half_bits_to_bf16_bits(w) : w;
      } else dstb[e] = *s;
    }
    *reinterpret_cast<u4*>(vb) = vw;
  }
}

template <bool APPEND>
hipError_t launch_copy(const KvCopyArgs& a, hipStream_t stream) {
  if (a.n <= 0) return hipSuccess;
  const int esz = a.geom.esize;
  const int64_t total = (int64_t)a.n * a.geom.hkv * (a.geom.head_dim / (16 / esz));
  const dim3 grid((unsigned)((total + 255) / 256));
  if (esz == 4) hipLaunchKernelGGL((kv_copy_kernel<4, APPEND, false>), grid, dim3(256), 0, stream, a);
  else if (esz == 2 && a.v_half) hipLaunchKernelGGL((kv_copy_kernel<2, APPEND, true>), grid, dim3(256), 0, stream, a);
  else if (esz == 2) hipLaunchKernelGGL((kv_copy_kernel<2, APPEND, false>), grid, dim3(256), 0, stream, a);
  else hipLaunchKernelGGL((kv_copy_kernel<1, APPEND, false>), grid, dim3(256), 0, stream, a);
  return hipGetLastError();
}

// Reads `bytes` of the cache and does nothing with them: `workgroups` x `waves` waves, each streaming a contiguous
// share with the decode kernel's load pattern (non-temporal 16-byte loads, 32 KiB per wave in flight). The time of
// this launch is the floor for a decode launch of the same bytes and shape: dispatch, first-load latency and the
// memory's own rate, no arithmetic, no partial results.
__global__ void stream_probe_kernel(const uint8_t* src, int64_t per_wave, uint32_t* sink) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const uint8_t* p = src + wave * per_wave + lane * 16;
  u4 acc = {0, 0, 0, 0};
  for (int64_t off = 0; off < per_wave; off += 32768) {
    u4 r[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) r[i] = load_stream16(p + off + i * 1024);
#pragma unroll
    for (int i = 0; i < 32; ++i) acc ^= r[i];
  }
  // (the zero-initialised cache and random rows never xor to this word in every lane; the store keeps the loads alive)
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9E3779B9u && lane == 63) sink[0] = 1;
}

}  // namespace

hipError_t launch_stream_probe(const uint8_t* cache, int64_t cache_bytes, int64_t offset, int64_t bytes, int workgroups,
                               int waves, uint32_t* sink, hipStream_t stream, hipEvent_t ev0, hipEvent_t ev1) {
  if (workgroups < 1 || waves < 1 || waves > 16 || bytes < 1 || offset < 0) return hipErrorInvalidValue;
  const int64_t nwaves = (int64_t)workgroups * waves;
  const int64_t per_wave = (bytes / nwaves + 32767) / 32768 * 32768;
  if (offset % 16 || offset + per_wave * nwaves > cache_bytes) return hipErrorInvalidValue;  // every load inside the cache
  hipExtLaunchKernelGGL(stream_probe_kernel, dim3(workgroups), dim3(waves * 64), 0, stream, ev0, ev1, 0, cache + offset,
                        per_wave, sink);
  return hipGetLastError();
}

hipError_t launch_kv_append(const KvCopyArgs& a, hipStream_t stream) { return launch_copy<true>(a, stream); }
hipError_t launch_kv_read(const KvCopyArgs& a, hipStream_t stream) { return launch_copy<false>(a, stream); }

}  // namespace mi355
