// Plain streaming kernels - copy, read-only, write-only - whose rate is the ceiling the
// HBM-bound kernels of this library are measured against on the machine they run on
// (ptx_hbm_stream).  16 bytes per lane and access, four accesses in flight per lane, one
// workgroup per 16 KB; optionally with non-temporal accesses.
#include "common.h"
#include "kernels.h"

namespace ptx {

static __device__ u32x4_t g_stream_sink[256];   // target of the read-only kernel's never-taken store

template <bool NT>
__global__ __launch_bounds__(256) void hbm_stream_kernel(const u32x4_t* __restrict__ src,
                                                         u32x4_t* __restrict__ dst, int64_t n16) {
  constexpr int U = 4;
  const int64_t base = (int64_t)blockIdx.x * 256 * U + threadIdx.x;
  u32x4_t v[U];
  u32x4_t acc = {1u, 2u, 3u, 4u};
  if (src) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + u * 256;
      v[u] = acc;
      if (i < n16) v[u] = NT ? __builtin_nontemporal_load(src + i) : src[i];
    }
  } else {
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = acc;
  }
  if (dst) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + u * 256;
      if (i < n16) {
        if (NT) __builtin_nontemporal_store(v[u], dst + i); else dst[i] = v[u];
      }
    }
  } else {
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u];
    // (keeps the loads alive; the condition holds for one value in 2^32 of unrelated data)
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) g_stream_sink[threadIdx.x] = acc;
  }
}

int hbm_stream(const void* src, void* dst, int64_t bytes, int nontemporal, hipStream_t stream) {
  const int64_t n16 = bytes / 16;
  if (n16 == 0) return 0;
  const int64_t blocks = (n16 + 1023) / 1024;
  if (nontemporal)
    hbm_stream_kernel<true><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
        (const u32x4_t*)src, (u32x4_t*)dst, n16);
  else
    hbm_stream_kernel<false><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
        (const u32x4_t*)src, (u32x4_t*)dst, n16);
  return 0;
}

}  // namespace ptx
