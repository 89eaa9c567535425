// LayerNorm over the last dimension, forward and backward, HBM-bound.
//
// Forward:
//
// A group of G lanes (G a power of two, 1..64) owns one row: each lane keeps
// NCHUNK vectors of VEC elements in registers (16-byte loads where alignment
// allows), so the row is read from HBM exactly once.  Statistics are fp32,
// two-pass in registers (mean, then centred second moment), reduced across the
// group with xor-shuffles.  A wave issues the loads of UNROLL independent rows
// per group before touching any of them, to keep enough bytes in flight.
// Algorithmic traffic: 2 * rows * cols * sizeof(T) bytes.
#include <algorithm>

#include "common.h"
#include "kernels.h"

namespace ptx {

template <typename T, int VEC> struct VecN;
template <> struct VecN<bf16_t, 8> { typedef bf16x8 type; typedef f32x8 ftype; };
template <> struct VecN<bf16_t, 4> { typedef bf16x4 type; typedef f32x4 ftype; };
template <> struct VecN<bf16_t, 2> { typedef bf16x2 type; typedef f32x2 ftype; };
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(1))) _Float16 f16x1;
template <> struct VecN<f16_t, 8> { typedef f16x8 type; typedef f32x8 ftype; };
template <> struct VecN<f16_t, 4> { typedef f16x4 type; typedef f32x4 ftype; };
template <> struct VecN<f16_t, 2> { typedef f16x2 type; typedef f32x2 ftype; };
template <> struct VecN<float, 4> { typedef f32x4 type; typedef f32x4 ftype; };
template <> struct VecN<float, 2> { typedef f32x2 type; typedef f32x2 ftype; };
typedef __attribute__((ext_vector_type(1))) float f32x1;
typedef __attribute__((ext_vector_type(1))) __bf16 bf16x1;
template <> struct VecN<bf16_t, 1> { typedef bf16x1 type; typedef f32x1 ftype; };
template <> struct VecN<float, 1> { typedef f32x1 type; typedef f32x1 ftype; };
template <> struct VecN<f16_t, 1> { typedef f16x1 type; typedef f32x1 ftype; };

template <int G>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int m = G / 2; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}

// HOIST: gamma and beta of the lane's columns are read once, before the rows (short rows: a
// load per row and vector otherwise, more load instructions than the rows themselves need).
// NT: rows are read and written with non-temporal accesses (tensors that do not fit the
// memory-side cache anyway).  Waves walk over row batches with a grid stride and request the
// next batch before they work on the current one; with one batch per wave that is a plain
// one-shot kernel.
template <typename T, int VEC, int G, int NCHUNK, int UNROLL, bool HOIST, bool NT>
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
  const float inv_n = 1.0f / (float)cols;
  const int64_t n_batches = (rows + ROWS_PER_WAVE - 1) / ROWS_PER_WAVE;
  const int64_t stride = (int64_t)gridDim.x * (blockDim.x >> 6);
  int64_t batch = (int64_t)blockIdx.x * (blockDim.x >> 6) + wave;
  if (batch >= n_batches) return;

  F gm[HOIST ? NCHUNK : 1], bt[HOIST ? NCHUNK : 1];
  if (HOIST) {
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      const int col = (c * G + sub) * VEC;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        gm[c][e] = 1.0f;
        bt[c][e] = 0.0f;
      }
      if (col < cols) {
        if (gamma) gm[c] = __builtin_convertvector(*reinterpret_cast<const V*>(gamma + col), F);
        if (beta) bt[c] = __builtin_convertvector(*reinterpret_cast<const V*>(beta + col), F);
      }
    }
  }

  // raw rows of one batch: rows and columns beyond the end repeat the last valid ones (their
  // values are masked where they are used), so the loads themselves are unconditional
  auto load = [&](V (&r)[UNROLL][NCHUNK], int64_t b) {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      int64_t row = b * ROWS_PER_WAVE + (int64_t)u * (kWave / G) + grp;
      row = row < rows ? row : rows - 1;
#pragma unroll
      for (int c = 0; c < NCHUNK; ++c) {
        int col = (c * G + sub) * VEC;
        col = col < cols ? col : 0;
        const V* p = reinterpret_cast<const V*>(x + row * cols + col);
        r[u][c] = NT ? __builtin_nontemporal_load(p) : *p;
      }
    }
  };
  auto work = [&](const V (&r)[UNROLL][NCHUNK], int64_t b) {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t row = b * ROWS_PER_WAVE + (int64_t)u * (kWave / G) + grp;
      F v[NCHUNK];
      float s = 0.0f;
#pragma unroll
      for (int c = 0; c < NCHUNK; ++c) {
        v[c] = __builtin_convertvector(r[u][c], F);
        if ((c * G + sub) * VEC < cols) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) s += v[c][e];
        }
      }
      const float mean = group_sum<G>(s) * inv_n;
      float q = 0.0f;
#pragma unroll
      for (int c = 0; c < NCHUNK; ++c) {
        if ((c * G + sub) * VEC < cols) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const float d = v[c][e] - mean;
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
            for (int e = 0; e < VEC; ++e) o[e] = (v[c][e] - mean) * rstd;
            if (HOIST) {
#pragma unroll
              for (int e = 0; e < VEC; ++e) o[e] = o[e] * gm[c][e] + bt[c][e];
            } else {
              if (gamma) {
                F g1 = __builtin_convertvector(*reinterpret_cast<const V*>(gamma + col), F);
#pragma unroll
                for (int e = 0; e < VEC; ++e) o[e] *= g1[e];
              }
              if (beta) {
                F b1 = __builtin_convertvector(*reinterpret_cast<const V*>(beta + col), F);
#pragma unroll
                for (int e = 0; e < VEC; ++e) o[e] += b1[e];
              }
            }
            V* p = reinterpret_cast<V*>(y + row * cols + col);
            const V ov = __builtin_convertvector(o, V);
            if (NT) __builtin_nontemporal_store(ov, p); else *p = ov;
          }
        }
      }
    }
  };

  V cur[UNROLL][NCHUNK];
  load(cur, batch);
  for (; batch < n_batches; batch += stride) {
    const bool more = batch + stride < n_batches;
    V nxt[UNROLL][NCHUNK];
    if (more) load(nxt, batch + stride);
    work(cur, batch);
    if (more) {
#pragma unroll
      for (int u = 0; u < UNROLL; ++u)
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) cur[u][c] = nxt[u][c];
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

// Tensors whose read + write traffic exceeds this are streamed with non-temporal accesses:
// measured on [768^2, 128], fp32 rows (604 MB of traffic, more than the 256 MB memory-side
// cache holds) 0.101 -> 0.095 ms, bf16 rows (302 MB) no gain.
constexpr int64_t kLnNonTemporalBytes = (int64_t)384 << 20;

template <typename T, int VEC, int G, int NCHUNK>
static void launch_ln(const T* x, const T* gamma, const T* beta, T* y, float* mean, float* rstd,
                      int64_t rows, int cols, float eps, hipStream_t stream) {
  // Row groups in flight per lane group, and how the grid is formed.  Measured on [768^2, 128]:
  // 16-bit rows of one vector per lane are fastest as 16 workgroups per compute unit whose waves
  // walk over batches of 2 row groups with the next batch requested ahead (0.047 ms against
  // 0.050 one-shot with 4 row groups, 0.051 with 2); 32-bit rows as a one-shot grid with 4 row
  // groups per wave (persistent: 0.101 against 0.095 ms).
  constexpr bool SHORT = NCHUNK * VEC * (int)sizeof(T) <= 16;
  constexpr int UNROLL = SHORT ? (sizeof(T) == 2 ? 2 : 4) : (NCHUNK <= 2 ? 2 : 1);
  constexpr bool HOIST = NCHUNK * VEC <= 16;
  constexpr int ROWS_PER_BLOCK = 4 * (kWave / G) * UNROLL;
  int64_t blocks = (rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
  if (sizeof(T) == 2 && SHORT) blocks = std::min<int64_t>(blocks, 16 * 256);
  blocks = std::min<int64_t>(blocks, 0x7fffffff);
  const bool nt = 2 * rows * (int64_t)cols * (int64_t)sizeof(T) > kLnNonTemporalBytes;
  if (nt)
    layernorm_fwd_kernel<T, VEC, G, NCHUNK, UNROLL, HOIST, true>
        <<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(x, gamma, beta, y, mean, rstd, rows, cols, eps);
  else
    layernorm_fwd_kernel<T, VEC, G, NCHUNK, UNROLL, HOIST, false>
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
  PTX_LN_CASE(32, 1) PTX_LN_CASE(16, 2) PTX_LN_CASE(16, 3) PTX_LN_CASE(64, 1) PTX_LN_CASE(64, 2) PTX_LN_CASE(64, 4)
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
template int layernorm_fwd<f16_t>(const f16_t*, const f16_t*, const f16_t*, f16_t*, float*, float*,
                                  int64_t, int, float, hipStream_t);

// ---------------------------------------------------------------------------
// Backward.  With xc = x - mean, gd = gamma * dout (gamma = 1 when absent), all in fp32:
//   dx     = gd * rstd - sum_c(gd) * rstd / cols - xc * sum_c(gd * xc) * rstd^3 / cols
//   dgamma = sum_rows dout * xc * rstd,   dbeta = sum_rows dout
// One pass over x and dout serves all three: the rows are laid out over the lanes as in the
// forward kernel, a wave walks over row batches with a grid stride and keeps its column sums
// of dgamma / dbeta in registers; at the end every workgroup writes one row of partial sums
// ([2][parts][cols] fp32, parts = gridDim.x) and a second small kernel adds them up in a
// fixed order (no atomics: the result does not depend on scheduling).
// Algorithmic traffic: 3 * rows * cols * sizeof(T) bytes.
// ---------------------------------------------------------------------------
constexpr int kLnBwdMaxBlocks = 1024;   // = most rows of partial sums

template <typename T, int VEC, int G, int NCHUNK>
__global__ __launch_bounds__(256) void layernorm_bwd_kernel(
    const T* __restrict__ dout, const T* __restrict__ x, const float* __restrict__ mean,
    const float* __restrict__ rstd, const T* __restrict__ gamma, T* __restrict__ dx,
    float* __restrict__ part, int64_t rows, int cols) {
  typedef typename VecN<T, VEC>::type V;
  typedef typename VecN<T, VEC>::ftype F;
  constexpr int RPW = kWave / G;   // rows per wave and batch
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int sub = lane % G, grp = lane / G;
  const float inv_n = 1.0f / (float)cols;
  const int64_t n_batches = (rows + RPW - 1) / RPW;

  F gm[NCHUNK], dg[NCHUNK], db[NCHUNK];
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const int col = (c * G + sub) * VEC;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      gm[c][e] = 1.0f;
      dg[c][e] = 0.0f;
      db[c][e] = 0.0f;
    }
    if (gamma && col < cols) gm[c] = __builtin_convertvector(*reinterpret_cast<const V*>(gamma + col), F);
  }

  for (int64_t batch = (int64_t)blockIdx.x * 4 + wave; batch < n_batches; batch += (int64_t)gridDim.x * 4) {
    const int64_t row = batch * RPW + grp;
    const bool ok = row < rows;
    const float mu = ok ? mean[row] : 0.0f;
    const float rs = ok ? rstd[row] : 0.0f;
    F xc[NCHUNK], dv[NCHUNK];
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      const int col = (c * G + sub) * VEC;
      if (ok && col < cols) {
        xc[c] = __builtin_convertvector(*reinterpret_cast<const V*>(x + row * cols + col), F);
        dv[c] = __builtin_convertvector(*reinterpret_cast<const V*>(dout + row * cols + col), F);
      } else {
        // dout = 0 keeps the padding out of every sum below
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          xc[c][e] = 0.0f;
          dv[c][e] = 0.0f;
        }
      }
    }
    float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        xc[c][e] -= mu;
        const float gd = gm[c][e] * dv[c][e];
        s1 += gd;
        s2 += gd * xc[c][e];
      }
    const float p2 = group_sum<G>(s1) * rs * inv_n;
    const float p3 = group_sum<G>(s2) * rs * rs * rs * inv_n;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      const int col = (c * G + sub) * VEC;
      F o;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        o[e] = gm[c][e] * dv[c][e] * rs - p2 - xc[c][e] * p3;
        dg[c][e] += dv[c][e] * xc[c][e] * rs;
        db[c][e] += dv[c][e];
      }
      if (ok && col < cols) *reinterpret_cast<V*>(dx + row * cols + col) = __builtin_convertvector(o, V);
    }
  }

  if (part) {
    // wave: lanes that share `sub` hold the same columns of different rows; workgroup: the
    // four waves through LDS, added in wave order
    constexpr int WIDTH = G * NCHUNK * VEC;
    __shared__ float red[2][4][WIDTH];
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      const int col = (c * G + sub) * VEC;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float a = dg[c][e], b = db[c][e];
#pragma unroll
        for (int m = G; m < kWave; m <<= 1) {
          a += __shfl_xor(a, m, 64);
          b += __shfl_xor(b, m, 64);
        }
        if (grp == 0) {
          red[0][wave][col + e] = a;
          red[1][wave][col + e] = b;
        }
      }
    }
    __syncthreads();
    const int64_t parts = gridDim.x;
    for (int col = threadIdx.x; col < cols; col += 256) {
      part[(int64_t)blockIdx.x * cols + col] =
          (red[0][0][col] + red[0][1][col]) + (red[0][2][col] + red[0][3][col]);
      part[(parts + blockIdx.x) * cols + col] =
          (red[1][0][col] + red[1][1][col]) + (red[1][2][col] + red[1][3][col]);
    }
  }
}

// Rows too long for the register layout: dx with one wave per row (the row is re-read from
// cache), dgamma / dbeta partial sums with one thread per column over a slice of the rows.
template <typename T>
__global__ __launch_bounds__(256) void layernorm_bwd_long_kernel(
    const T* __restrict__ dout, const T* __restrict__ x, const float* __restrict__ mean,
    const float* __restrict__ rstd, const T* __restrict__ gamma, T* __restrict__ dx, int64_t rows,
    int cols) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* xr = x + row * cols;
  const T* dr = dout + row * cols;
  const float mu = mean[row], rs = rstd[row];
  float s1 = 0.0f, s2 = 0.0f;
  for (int c = lane; c < cols; c += kWave) {
    const float gd = (gamma ? to_f32(gamma[c]) : 1.0f) * to_f32(dr[c]);
    s1 += gd;
    s2 += gd * (to_f32(xr[c]) - mu);
  }
  const float p2 = group_sum<64>(s1) * rs / (float)cols;
  const float p3 = group_sum<64>(s2) * rs * rs * rs / (float)cols;
  for (int c = lane; c < cols; c += kWave) {
    const float gd = (gamma ? to_f32(gamma[c]) : 1.0f) * to_f32(dr[c]);
    dx[row * cols + c] = from_f32<T>(gd * rs - p2 - (to_f32(xr[c]) - mu) * p3);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void layernorm_bwd_params_kernel(
    const T* __restrict__ dout, const T* __restrict__ x, const float* __restrict__ mean,
    const float* __restrict__ rstd, float* __restrict__ part, int64_t rows, int cols) {
  // grid: (column blocks of 256, parts); part p owns rows p, p + parts, ...
  const int col = blockIdx.x * 256 + threadIdx.x;
  const int64_t parts = gridDim.y, p = blockIdx.y;
  if (col >= cols) return;
  float a = 0.0f, b = 0.0f;
  for (int64_t row = p; row < rows; row += parts) {
    const float d = to_f32(dout[row * cols + col]);
    a += d * (to_f32(x[row * cols + col]) - mean[row]) * rstd[row];
    b += d;
  }
  part[p * cols + col] = a;
  part[(parts + p) * cols + col] = b;
}

// Column sums of the partial rows: 64 columns per workgroup, the parts dealt to 16 waves.
template <typename T>
__global__ __launch_bounds__(1024) void layernorm_bwd_reduce_kernel(
    const float* __restrict__ part, int parts, int cols, T* __restrict__ dgamma,
    T* __restrict__ dbeta) {
  constexpr int SL = 16;
  __shared__ float red[2][SL][kWave];
  const int cl = threadIdx.x & (kWave - 1), sl = threadIdx.x >> 6;
  const int col = blockIdx.x * kWave + cl;
  float a[2] = {0.0f, 0.0f}, b[2] = {0.0f, 0.0f};
  if (col < cols) {
    int p = sl;
    for (; p + SL < parts; p += 2 * SL) {   // two independent chains per sum
      a[0] += part[(int64_t)p * cols + col];
      a[1] += part[(int64_t)(p + SL) * cols + col];
      b[0] += part[((int64_t)parts + p) * cols + col];
      b[1] += part[((int64_t)parts + p + SL) * cols + col];
    }
    if (p < parts) {
      a[0] += part[(int64_t)p * cols + col];
      b[0] += part[((int64_t)parts + p) * cols + col];
    }
  }
  red[0][sl][cl] = a[0] + a[1];
  red[1][sl][cl] = b[0] + b[1];
  __syncthreads();
  if (sl == 0 && col < cols) {
    float sa = 0.0f, sb = 0.0f;
#pragma unroll
    for (int w = 0; w < SL; ++w) {
      sa += red[0][w][cl];
      sb += red[1][w][cl];
    }
    if (dgamma) dgamma[col] = from_f32<T>(sa);
    if (dbeta) dbeta[col] = from_f32<T>(sb);
  }
}

template <typename T, int VEC>
static int dispatch_ln_bwd_vec(const T* dout, const T* x, const float* mean, const float* rstd,
                               const T* gamma, T* dx, float* part, int64_t rows, int cols,
                               hipStream_t stream) {
  const int nvec = cols / VEC;
  // returns the number of partial-sum rows written (0: no kernel fits)
#define PTX_LNB_CASE(G, NC)                                                                    \
  if (nvec <= (G) * (NC)) {                                                                    \
    const int64_t batches = (rows + (kWave / (G)) - 1) / (kWave / (G));                        \
    const int blocks = (int)std::min<int64_t>((batches + 3) / 4, kLnBwdMaxBlocks);             \
    layernorm_bwd_kernel<T, VEC, G, NC><<<dim3(blocks), dim3(256), 0, stream>>>(               \
        dout, x, mean, rstd, gamma, dx, part, rows, cols);                                     \
    return blocks;                                                                             \
  }
  PTX_LNB_CASE(1, 1) PTX_LNB_CASE(2, 1) PTX_LNB_CASE(4, 1) PTX_LNB_CASE(8, 1) PTX_LNB_CASE(16, 1)
  PTX_LNB_CASE(16, 2) PTX_LNB_CASE(16, 3) PTX_LNB_CASE(64, 1) PTX_LNB_CASE(64, 2) PTX_LNB_CASE(64, 4)
  if constexpr (VEC <= 4) {
    PTX_LNB_CASE(64, 8)
  }
#undef PTX_LNB_CASE
  return 0;
}

int64_t layernorm_bwd_workspace_elems(int64_t rows, int cols) {
  if (rows <= 0 || cols <= 0) return 0;
  return 2 * (int64_t)kLnBwdMaxBlocks * cols;
}

template <typename T>
int layernorm_bwd(const T* dout, const T* x, const float* mean, const float* rstd, const T* gamma,
                  T* dx, T* dgamma, T* dbeta, float* workspace, int64_t rows, int cols,
                  hipStream_t stream) {
  const bool params = dgamma || dbeta;
  if (rows == 0) {
    // empty input: the parameter gradients are sums over no rows (written by a kernel, so
    // that the call can be captured into a HIP graph like every other one)
    if (params)
      layernorm_bwd_reduce_kernel<T><<<dim3((cols + kWave - 1) / kWave), dim3(1024), 0, stream>>>(
          nullptr, 0, cols, dgamma, dbeta);
    return 0;
  }
  float* part = params ? workspace : nullptr;
  auto aligned = [&](int vec) {
    const uintptr_t bytes = (uintptr_t)vec * sizeof(T);
    return cols % vec == 0 && ((uintptr_t)x % bytes) == 0 && ((uintptr_t)dout % bytes) == 0 &&
           ((uintptr_t)dx % bytes) == 0 && (!gamma || ((uintptr_t)gamma % bytes) == 0);
  };
  int parts = 0;
  if constexpr (sizeof(T) == 2) {
    if (aligned(8)) parts = dispatch_ln_bwd_vec<T, 8>(dout, x, mean, rstd, gamma, dx, part, rows, cols, stream);
  }
  if (!parts && aligned(4)) parts = dispatch_ln_bwd_vec<T, 4>(dout, x, mean, rstd, gamma, dx, part, rows, cols, stream);
  if (!parts && aligned(2)) parts = dispatch_ln_bwd_vec<T, 2>(dout, x, mean, rstd, gamma, dx, part, rows, cols, stream);
  if (!parts) parts = dispatch_ln_bwd_vec<T, 1>(dout, x, mean, rstd, gamma, dx, part, rows, cols, stream);
  if (!parts) {
    const int64_t blocks = (rows + 3) / 4;
    layernorm_bwd_long_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
        dout, x, mean, rstd, gamma, dx, rows, cols);
    if (params) {
      parts = (int)std::min<int64_t>(rows, 256);
      layernorm_bwd_params_kernel<T><<<dim3((cols + 255) / 256, parts), dim3(256), 0, stream>>>(
          dout, x, mean, rstd, part, rows, cols);
    }
  }
  if (params)
    layernorm_bwd_reduce_kernel<T><<<dim3((cols + kWave - 1) / kWave), dim3(1024), 0, stream>>>(
        part, parts, cols, dgamma, dbeta);
  return 0;
}

template int layernorm_bwd<float>(const float*, const float*, const float*, const float*,
                                  const float*, float*, float*, float*, float*, int64_t, int,
                                  hipStream_t);
template int layernorm_bwd<bf16_t>(const bf16_t*, const bf16_t*, const float*, const float*,
                                   const bf16_t*, bf16_t*, bf16_t*, bf16_t*, float*, int64_t, int,
                                   hipStream_t);
template int layernorm_bwd<f16_t>(const f16_t*, const f16_t*, const float*, const float*,
                                  const f16_t*, f16_t*, f16_t*, f16_t*, float*, int64_t, int,
                                  hipStream_t);

}  // namespace ptx
