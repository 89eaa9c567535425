// Triangle-multiplication contraction: for every channel c an independent
//   x[c][i][j] = sum_k a[c][i][k] * b[c][j][k]          (A * B^T, both K-contiguous)
// on MFMA with fp32 accumulation.
//
// Workgroup tile 256 (i) x 128 (j), 4 waves stacked along i: a wave owns 64 rows
// of A and all 128 columns, i.e. 2 x 4 accumulator tiles of 32 x 32.  Its A
// operand fragments are private, so they go global -> registers directly
// (prefetched one K stage ahead); only the B tile, which all 4 waves share, is
// staged through LDS in fragment order ([fragment][lane], conflict-free 16-byte
// reads), double-buffered with one barrier per K stage.  That halves LDS
// traffic per MFMA against a both-operands-in-LDS tiling.
//
// Workgroups are numbered so that all tiles of one channel land on one XCD
// (round-robin dispatch: id % 8), keeping that channel's a/b panels in its L2.
#include "common.h"
#include "kernels.h"

namespace ptx {

template <typename T>
__global__ __launch_bounds__(256, 2) void nt_gemm_batched_kernel(const T* __restrict__ a,
                                                              const T* __restrict__ b,
                                                              T* __restrict__ x, int n, int k_pitch,
                                                              int batch, int tiles_i, int tiles_j) {
  typedef typename Vec8<T>::type V8;
  constexpr int KK = sizeof(T) == 2 ? 4 : 2;   // 16-deep K steps per stage
  constexpr int BK = 16 * KK;
  __shared__ V8 lds_b[2][4 * KK][kWave];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ln = lane & 31, g = lane >> 5;

  const int tiles = tiles_i * tiles_j;
  const int slot = blockIdx.x >> 3;
  const int c = (slot / tiles) * 8 + (blockIdx.x & 7);
  if (c >= batch) return;
  const int tile = slot % tiles;
  const int i0 = (tile / tiles_j) * 256 + wave * 64;
  const int j0 = (tile % tiles_j) * 128;

  const T* a_c = a + (int64_t)c * n * k_pitch;
  const T* b_c = b + (int64_t)c * n * k_pitch;

  // per-lane row pointers (rows beyond n read row 0; those outputs are never stored)
  const T* a_ptr[2];
  bool a_ok[2];
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
    const int i = i0 + rb * 32 + ln;
    a_ok[rb] = i < n;
    a_ptr[rb] = a_c + (int64_t)(a_ok[rb] ? i : 0) * k_pitch + 8 * g;
  }
  const int jb_row = j0 + wave * 32 + ln;   // B row this lane stages
  const bool b_ok = jb_row < n;
  const T* b_ptr = b_c + (int64_t)(b_ok ? jb_row : 0) * k_pitch + 8 * g;

  const int n_stages = (n + BK - 1) / BK;

  V8 a_nxt[2][KK], b_pre[KK];
  auto fetch = [&](int stage) {
    const int k0 = stage * BK;
    const bool tail = k0 + BK > n;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        V8 v = load8<T>(a_ptr[rb] + k0 + 16 * kk);   // rows beyond n: clamped, never stored
        if (tail) {
#pragma unroll
          for (int t = 0; t < 8; ++t)
            if (k0 + 16 * kk + 8 * g + t >= n) v[t] = (T)0.0f;
        }
        a_nxt[rb][kk] = v;
      }
      V8 v = load8<T>(b_ptr + k0 + 16 * kk);
      if (tail) {
#pragma unroll
        for (int t = 0; t < 8; ++t)
          if (k0 + 16 * kk + 8 * g + t >= n) v[t] = (T)0.0f;
      }
      b_pre[kk] = v;
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) lds_b[buf][wave * KK + kk][lane] = b_pre[kk];
  };

  f32x16 acc[2][4];
#pragma unroll
  for (int rb = 0; rb < 2; ++rb)
#pragma unroll
    for (int jb = 0; jb < 4; ++jb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rb][jb][r] = 0.0f;

  fetch(0);
  stash(0);
  __syncthreads();

  for (int stage = 0; stage < n_stages; ++stage) {
    const int buf = stage & 1;
    V8 a_cur[2][KK];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) a_cur[rb][kk] = a_nxt[rb][kk];
    fetch(min(stage + 1, n_stages - 1));   // unconditional: static outstanding-load count

#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) {
        const V8 bf = lds_b[buf][jb * KK + kk][lane];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) mma32(acc[rb][jb], a_cur[rb][kk], bf);
      }
    }
    stash(buf ^ 1);
    __syncthreads();
  }

  // lane <-> column j, register <-> row i: 64-byte contiguous stores per register
  T* x_c = x + (int64_t)c * n * n;
#pragma unroll
  for (int rb = 0; rb < 2; ++rb)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = i0 + rb * 32 + acc_row(r, g);
      if (i < n) {
#pragma unroll
        for (int jb = 0; jb < 4; ++jb) {
          const int j = j0 + jb * 32 + ln;
          if (j < n) x_c[(int64_t)i * n + j] = from_f32<T>(acc[rb][jb][r]);
        }
      }
    }
}

template <typename T>
int nt_gemm_batched(const T* a, const T* b, T* x, int n, int k_pitch, int batch,
                    hipStream_t stream) {
  if (n == 0 || batch == 0) return 0;
  const int tiles_i = (n + 255) / 256, tiles_j = (n + 127) / 128;
  const int64_t groups = (batch + 7) / 8;
  const int64_t blocks = groups * tiles_i * tiles_j * 8;
  nt_gemm_batched_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
      a, b, x, n, k_pitch, batch, tiles_i, tiles_j);
  return 0;
}

template int nt_gemm_batched<float>(const float*, const float*, float*, int, int, int, hipStream_t);
template int nt_gemm_batched<bf16_t>(const bf16_t*, const bf16_t*, bf16_t*, int, int, int,
                                     hipStream_t);

}  // namespace ptx
