// LayerNorm forward over the last dimension, HBM-bound.
//
// A group of G lanes (G a power of two, 1..64) owns one row: each lane keeps
// NCHUNK vectors of VEC elements in registers (16-byte loads where alignment
// allows), so the row is read from HBM exactly once.  Statistics are fp32,
// two-pass in registers (mean, then centred second moment), reduced across the
// group with xor-shuffles.  A wave issues the loads of UNROLL independent rows
// per group before touching any of them, to keep enough bytes in flight.
// Algorithmic traffic: 2 * rows * cols * sizeof(T) bytes.
#include "common.h"

namespace ptx {

template <typename T, int VEC> struct VecN;
template <> struct VecN<bf16_t, 8> { typedef bf16x8 type; typedef f32x8 ftype; };
template <> struct VecN<bf16_t, 4> { typedef bf16x4 type; typedef f32x4 ftype; };
template <> struct VecN<bf16_t, 2> { typedef bf16x2 type; typedef f32x2 ftype; };
template <> struct VecN<float, 4> { typedef f32x4 type; typedef f32x4 ftype; };
template <> struct VecN<float, 2> { typedef f32x2 type; typedef f32x2 ftype; };
typedef __attribute__((ext_vector_type(1))) float f32x1;
typedef __attribute__((ext_vector_type(1))) __bf16 bf16x1;
template <> struct VecN<bf16_t, 1> { typedef bf16x1 type; typedef f32x1 ftype; };
template <> struct VecN<float, 1> { typedef f32x1 type; typedef f32x1 ftype; };

template <int G>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int m = G / 2; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}

template <typename T, int VEC, int G, int NCHUNK, int UNROLL>
__global__ __launch_bounds__(256) void layernorm_fwd_kernel(
    const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ beta,
    T* __restrict__ y, float* __restrict__ mean_out, float* __restrict__ rstd_out, int64_t rows,
    int cols, float eps) {
  typedef typename VecN<T, VEC>::type V;
  typedef typename VecN<T, VEC>::ftype F;
  constexpr int ROWS_PER_WAVE = (kWave / G) * UNROLL;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int sub = lane % G;   // lane within the row group
  const int grp = lane / G;   // which row of the wave's batch
  const int64_t row0 = ((int64_t)blockIdx.x * (blockDim.x >> 6) + wave) * ROWS_PER_WAVE;
  const float inv_n = 1.0f / (float)cols;

  F v[UNROLL][NCHUNK];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int64_t row = row0 + (int64_t)u * (kWave / G) + grp;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      const int col = (c * G + sub) * VEC;
      if (row < rows && col < cols) {
        v[u][c] = __builtin_convertvector(*reinterpret_cast<const V*>(x + row * cols + col), F);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[u][c][e] = 0.0f;
      }
    }
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int64_t row = row0 + (int64_t)u * (kWave / G) + grp;
    float s = 0.0f;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
      for (int e = 0; e < VEC; ++e) s += v[u][c][e];
    const float mean = group_sum<G>(s) * inv_n;
    float q = 0.0f;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      const int col = (c * G + sub) * VEC;
      if (col < cols) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float d = v[u][c][e] - mean;
          q += d * d;
        }
      }
    }
    const float var = group_sum<G>(q) * inv_n;
    const float rstd = rsqrtf(fmaxf(var, 0.0f) + eps);
    if (row < rows) {
      if (sub == 0) {
        if (mean_out) mean_out[row] = mean;
        if (rstd_out) rstd_out[row] = rstd;
      }
#pragma unroll
      for (int c = 0; c < NCHUNK; ++c) {
        const int col = (c * G + sub) * VEC;
        if (col < cols) {
          F o;
#pragma unroll
          for (int e = 0; e < VEC; ++e) o[e] = (v[u][c][e] - mean) * rstd;
          if (gamma) {
            F gm = __builtin_convertvector(*reinterpret_cast<const V*>(gamma + col), F);
#pragma unroll
            for (int e = 0; e < VEC; ++e) o[e] *= gm[e];
          }
          if (beta) {
            F bt = __builtin_convertvector(*reinterpret_cast<const V*>(beta + col), F);
#pragma unroll
            for (int e = 0; e < VEC; ++e) o[e] += bt[e];
          }
          *reinterpret_cast<V*>(y + row * cols + col) = __builtin_convertvector(o, V);
        }
      }
    }
  }
}

// Rows too long to keep in registers: one wave per row, three passes over a row
// that stays in cache after the first.
template <typename T>
__global__ __launch_bounds__(256) void layernorm_fwd_long_kernel(
    const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ beta,
    T* __restrict__ y, float* __restrict__ mean_out, float* __restrict__ rstd_out, int64_t rows,
    int cols, float eps) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* xr = x + row * cols;
  float s = 0.0f;
  for (int c = lane; c < cols; c += kWave) s += to_f32(xr[c]);
  const float mean = group_sum<64>(s) / (float)cols;
  float q = 0.0f;
  for (int c = lane; c < cols; c += kWave) {
    const float d = to_f32(xr[c]) - mean;
    q += d * d;
  }
  const float rstd = rsqrtf(fmaxf(group_sum<64>(q) / (float)cols, 0.0f) + eps);
  if (lane == 0) {
    if (mean_out) mean_out[row] = mean;
    if (rstd_out) rstd_out[row] = rstd;
  }
  for (int c = lane; c < cols; c += kWave) {
    float o = (to_f32(xr[c]) - mean) * rstd;
    if (gamma) o *= to_f32(gamma[c]);
    if (beta) o += to_f32(beta[c]);
    y[row * cols + c] = from_f32<T>(o);
  }
}

template <typename T, int VEC, int G, int NCHUNK>
static void launch_ln(const T* x, const T* gamma, const T* beta, T* y, float* mean, float* rstd,
                      int64_t rows, int cols, float eps, hipStream_t stream) {
  constexpr int UNROLL = (NCHUNK * VEC * (int)sizeof(T) <= 16) ? 4 : (NCHUNK <= 2 ? 2 : 1);
  constexpr int ROWS_PER_BLOCK = 4 * (kWave / G) * UNROLL;
  const int64_t blocks = (rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
  layernorm_fwd_kernel<T, VEC, G, NCHUNK, UNROLL>
      <<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(x, gamma, beta, y, mean, rstd, rows, cols, eps);
}

template <typename T, int VEC>
static bool dispatch_ln_vec(const T* x, const T* gamma, const T* beta, T* y, float* mean,
                            float* rstd, int64_t rows, int cols, float eps, hipStream_t stream) {
  const int nvec = cols / VEC;
#define PTX_LN_CASE(G, NC)                                                                  \
  if (nvec <= (G) * (NC)) {                                                                 \
    launch_ln<T, VEC, G, NC>(x, gamma, beta, y, mean, rstd, rows, cols, eps, stream);       \
    return true;                                                                            \
  }
  PTX_LN_CASE(1, 1) PTX_LN_CASE(2, 1) PTX_LN_CASE(4, 1) PTX_LN_CASE(8, 1) PTX_LN_CASE(16, 1)
  PTX_LN_CASE(16, 2) PTX_LN_CASE(16, 3) PTX_LN_CASE(64, 1) PTX_LN_CASE(64, 2) PTX_LN_CASE(64, 4)
  PTX_LN_CASE(64, 8)
#undef PTX_LN_CASE
  return false;
}

// Returns 0 on success, 1 if the launch geometry cannot be formed.
template <typename T>
int layernorm_fwd(const T* x, const T* gamma, const T* beta, T* y, float* mean, float* rstd,
                  int64_t rows, int cols, float eps, hipStream_t stream) {
  if (rows == 0) return 0;
  constexpr int MAXVEC = 16 / (int)sizeof(T);
  auto aligned = [&](int vec) {
    const uintptr_t bytes = (uintptr_t)vec * sizeof(T);
    return cols % vec == 0 && ((uintptr_t)x % bytes) == 0 && ((uintptr_t)y % bytes) == 0 &&
           (!gamma || ((uintptr_t)gamma % bytes) == 0) && (!beta || ((uintptr_t)beta % bytes) == 0);
  };
  bool done = false;
  if (MAXVEC >= 8 && aligned(8)) {
    if constexpr (sizeof(T) == 2) done = dispatch_ln_vec<T, 8>(x, gamma, beta, y, mean, rstd, rows, cols, eps, stream);
  }
  if (!done && aligned(4)) done = dispatch_ln_vec<T, 4>(x, gamma, beta, y, mean, rstd, rows, cols, eps, stream);
  if (!done && aligned(2)) done = dispatch_ln_vec<T, 2>(x, gamma, beta, y, mean, rstd, rows, cols, eps, stream);
  if (!done) done = dispatch_ln_vec<T, 1>(x, gamma, beta, y, mean, rstd, rows, cols, eps, stream);
  if (!done) {
    const int64_t blocks = (rows + 3) / 4;
    layernorm_fwd_long_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
        x, gamma, beta, y, mean, rstd, rows, cols, eps);
  }
  return 0;
}

template int layernorm_fwd<float>(const float*, const float*, const float*, float*, float*, float*,
                                  int64_t, int, float, hipStream_t);
template int layernorm_fwd<bf16_t>(const bf16_t*, const bf16_t*, const bf16_t*, bf16_t*, float*,
                                   float*, int64_t, int, float, hipStream_t);

}  // namespace ptx
