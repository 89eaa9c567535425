// Repack of standard-layout attention operands into the layouts of the triangle-attention
// core (common.h): K and V [rows][n][heads][32] -> fragment-ordered K and V^T key tiles, the
// pair bias [heads][n][n] -> fragment-ordered bias tiles in log2 units, q -> q * log2(e).
// One thread per 16-byte destination vector; plain gathers, bandwidth-bound.
#include "common.h"
#include "kernels.h"

namespace ptx {

constexpr float kPackLog2e = 1.4426950408889634f;

template <typename T>
__global__ __launch_bounds__(256) void attn_pack_qk_kernel(const T* __restrict__ q,
                                                           const T* __restrict__ k,
                                                           T* __restrict__ qs, T* __restrict__ kf,
                                                           int n_rows, int n, int heads,
                                                           int key_tiles) {
  // vector v = ((i * n + j) * heads + h) * 4 + c8: 8 channels of one (row, position, head)
  const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t total = (int64_t)n_rows * n * heads * 4;
  if (v >= total) return;
  const int c8 = (int)(v & 3);
  const int64_t p = v >> 2;
  const int h = (int)(p % heads);
  const int64_t ij = p / heads;
  const int j = (int)(ij % n), i = (int)(ij / n);
  const typename Vec8<T>::type kv = load8<T>(k + v * 8);
  store8<T>(kf + attn_k_offset(h, i, j, 8 * c8, n_rows, key_tiles), kv);
  f32x8 qv = to_f32(load8<T>(q + v * 8));
#pragma unroll
  for (int t = 0; t < 8; ++t) qv[t] *= kPackLog2e;
  store8<T>(qs + v * 8, from_f32<T>(qv));
}

template <typename T>
__global__ __launch_bounds__(256) void attn_pack_v_kernel(const T* __restrict__ vsrc,
                                                          T* __restrict__ vtf, int n_rows, int n,
                                                          int heads, int key_tiles) {
  // vector = ((i * key_blocks + jb) * heads + h) * 32 + d: keys 8*jb .. +7 of channel d
  const int key_blocks = key_tiles * 8;
  const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t total = (int64_t)n_rows * key_blocks * heads * 32;
  if (v >= total) return;
  const int d = (int)(v & 31);
  const int64_t p = v >> 5;
  const int h = (int)(p % heads);
  const int64_t ib = p / heads;
  const int jb = (int)(ib % key_blocks), i = (int)(ib / key_blocks);
  typename Vec8<T>::type out;
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const int j = 8 * jb + t;
    out[t] = j < n ? vsrc[(((int64_t)i * n + j) * heads + h) * 32 + d] : (T)0.0f;
  }
  store8<T>(vtf + attn_v_offset(h, i, 8 * jb, d, n_rows, key_tiles), out);
}

template <typename T>
__global__ __launch_bounds__(256) void attn_pack_bias_kernel(const T* __restrict__ bias2,
                                                             T* __restrict__ bf, int n, int heads,
                                                             int key_tiles) {
  // vector = (h * n + q) * key_blocks + jb: keys 8*jb .. +7 of query q
  const int key_blocks = key_tiles * 8;
  const int q_blocks = (n + 31) >> 5;
  const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t total = (int64_t)heads * n * key_blocks;
  if (v >= total) return;
  const int jb = (int)(v % key_blocks);
  const int64_t hq = v / key_blocks;
  const int qq = (int)(hq % n), h = (int)(hq / n);
  typename Vec8<T>::type out;
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const int j = 8 * jb + t;
    out[t] = j < n ? from_f32<T>(to_f32(bias2[((int64_t)h * n + qq) * n + j]) * kPackLog2e) : (T)0.0f;
  }
  store8<T>(bf + attn_b_offset(h, qq, 8 * jb, q_blocks, key_tiles), out);
}

template <typename T>
int triattn_pack(const T* q, const T* k, const T* v, const T* bias2, T* qs, T* kf, T* vtf, T* bf,
                 int n_rows, int n, int heads, int key_pitch, hipStream_t stream) {
  if (n_rows == 0 || n == 0 || heads == 0) return 0;
  const int key_tiles = key_pitch >> 6;
  const int64_t nqk = (int64_t)n_rows * n * heads * 4;
  attn_pack_qk_kernel<T><<<dim3((unsigned)((nqk + 255) / 256)), dim3(256), 0, stream>>>(
      q, k, qs, kf, n_rows, n, heads, key_tiles);
  const int64_t nv = (int64_t)n_rows * key_tiles * 8 * heads * 32;
  attn_pack_v_kernel<T><<<dim3((unsigned)((nv + 255) / 256)), dim3(256), 0, stream>>>(
      v, vtf, n_rows, n, heads, key_tiles);
  const int64_t nb = (int64_t)heads * n * key_tiles * 8;
  attn_pack_bias_kernel<T><<<dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, stream>>>(
      bias2, bf, n, heads, key_tiles);
  return 0;
}

template int triattn_pack<float>(const float*, const float*, const float*, const float*, float*,
                                 float*, float*, float*, int, int, int, int, hipStream_t);
template int triattn_pack<bf16_t>(const bf16_t*, const bf16_t*, const bf16_t*, const bf16_t*,
                                  bf16_t*, bf16_t*, bf16_t*, bf16_t*, int, int, int, int,
                                  hipStream_t);

}  // namespace ptx
