// Triangle-multiplication contraction: for every channel c an independent
//   x[c][i][j] = sum_k a[c][i][k] * b[c][j][k]
// on MFMA with fp32 accumulation.
//
// Operands arrive in MFMA fragment order (trimul_frag_offset in common.h): one
// fragment = 32 rows x 16 K values = 64 lanes x 16 bytes (bf16), contiguous, so
// every global load instruction of this kernel is one 1 KB run and the LDS image
// of a fragment is the global image ([fragment][lane], conflict-free 16-byte
// reads).
//
// Workgroup = 4 waves (2 x 2), tile 256 (i) x 256 (j); a wave owns 128 x 128:
// 4 x 4 accumulator tiles of 32 x 32 (256 accumulator registers, one wave per
// SIMD), so each fragment read from LDS feeds 4 MFMAs.  A K stage (KK steps of
// 16) of both operand panels is staged through LDS, double-buffered.  The wave
// is software-pipelined by hand, because with one wave per SIMD nothing else
// hides latency: the fragments of K step t+1 are read from LDS between the two
// halves of step t's MFMAs, the next stage's global loads are issued a whole
// stage before they are written to LDS, and the LDS write + workgroup barrier
// sit in the middle of a step's MFMAs as well.
//
// MFMA operands are ordered so that a lane ends up holding 4 consecutive j per
// register quad of one row i: results leave through a per-wave LDS tile as
// 16-byte stores along j.  No load sits under a branch (indices are clamped, K
// beyond n is zeroed on the way into LDS).  Workgroups are numbered so that all
// tiles of one channel land on one XCD (round-robin dispatch: id % 8), keeping
// that channel's panels in its L2.
#include "common.h"
#include "kernels.h"

namespace ptx {

template <typename T> struct GemmCfg {
  static constexpr int KK = sizeof(T) == 2 ? 4 : 1;   // 16-deep K steps per stage
  static constexpr int BK = 16 * KK;
  static constexpr int U = KK == 1 ? 2 : KK;          // K steps per loop trip (even: register sets alternate)
  static constexpr int NF = 16 * KK;                  // fragments per stage (a: 8 row blocks, b: 8)
  static constexpr int FPW = NF / 4;                  // fragments each wave moves per stage
  static constexpr int VE = 16 / (int)sizeof(T);      // elements per 16-byte vector
  static constexpr int LPM = 32 / VE;                 // lanes per 32-long row of the staging tile
  static constexpr int MPP = kWave / LPM;             // rows per read-back pass
  static constexpr int NPASS = 32 / MPP;
  static constexpr int PITCH = 32 + 8 / (int)sizeof(T);   // staging row pitch, 8-byte aligned rows
};

template <typename T>
__global__ __launch_bounds__(256) void nt_gemm_batched_kernel(const T* __restrict__ a,
                                                              const T* __restrict__ b,
                                                              T* __restrict__ x, int n, int k_pitch,
                                                              int batch, int tiles_i, int tiles_j) {
  typedef typename Vec8<T>::type V8;
  typedef typename Vec4<T>::type V4;
  typedef GemmCfg<T> G;
  constexpr int KK = G::KK, BK = G::BK, U = G::U, FPW = G::FPW;
  __shared__ V8 lds_f[2][G::NF][kWave];   // [buffer][operand*8*KK + row block*KK + kk][lane]
  __shared__ __attribute__((aligned(16))) T lds_stage[4][32 * G::PITCH];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ln = lane & 31, g = lane >> 5;
  const int wi = wave >> 1, wj = wave & 1;

  const int tiles = tiles_i * tiles_j;
  const int slot = blockIdx.x >> 3;
  const int c = (slot / tiles) * 8 + (blockIdx.x & 7);
  if (c >= batch) return;
  const int tile = slot % tiles;
  const int ti = tile / tiles_j, tj = tile % tiles_j;

  const int n_rb = (n + 31) >> 5;          // row blocks per channel
  const int n_ks = k_pitch >> 4;           // K steps per row block
  const int n_stages = (n + BK - 1) / BK;

  // The fragments this wave moves global -> LDS each stage: ids wave*FPW .. +FPW-1, in
  // runs of KK consecutive K steps of one row block (consecutive in memory).
  const T* src[FPW / KK];
#pragma unroll
  for (int q = 0; q < FPW / KK; ++q) {
    const int run = wave * (FPW / KK) + q;        // 0..15: operand = run / 8, row block = run % 8
    const int op = run >> 3;
    const int rb = min((op ? tj : ti) * 8 + (run & 7), n_rb - 1);   // blocks past the end re-read the last
    src[q] = (op ? b : a) + trimul_frag_offset(c, rb, 0, n_rb, n_ks) + lane * 8;
  }

  V8 pre[FPW];
  auto fetch = [&](int stage) {   // issues loads only; the stage index is clamped for the address
    const int ks0 = min(stage, n_stages - 1) * KK;
#pragma unroll
    for (int q = 0; q < FPW / KK; ++q)
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) pre[q * KK + kk] = load8<T>(src[q] + (int64_t)(ks0 + kk) * 512);
  };
  auto stash = [&](int stage) {   // K slots beyond n (row padding, phantom stages) become zero
    const int buf = stage & 1;
    if (stage * BK + BK > n) {    // uniform
#pragma unroll
      for (int f = 0; f < FPW; ++f) {
        const int kbase = stage * BK + 16 * (f % KK) + 8 * g;
#pragma unroll
        for (int t = 0; t < 8; ++t) pre[f][t] = kbase + t < n ? pre[f][t] : (T)0.0f;
      }
    }
#pragma unroll
    for (int f = 0; f < FPW; ++f) lds_f[buf][wave * FPW + f][lane] = pre[f];
  };
  // fragments of one K step: this wave's 4 row blocks of a and 4 of b
  auto read_frags = [&](int buf, int kk, V8 (&af)[4], V8 (&bf)[4]) {
#pragma unroll
    for (int r = 0; r < 4; ++r) af[r] = lds_f[buf][(wi * 4 + r) * KK + kk][lane];
#pragma unroll
    for (int r = 0; r < 4; ++r) bf[r] = lds_f[buf][(8 + wj * 4 + r) * KK + kk][lane];
  };

  f32x16 acc[4][4];   // [row block of a][row block of b]
#pragma unroll
  for (int rb = 0; rb < 4; ++rb)
#pragma unroll
    for (int jb = 0; jb < 4; ++jb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rb][jb][r] = 0.0f;

  // A operand = b rows (register <-> j), B operand = a rows (lane <-> i)
  auto mma_half = [&](int half, V8 (&af)[4], V8 (&bf)[4]) {
#pragma unroll
    for (int rb = 2 * half; rb < 2 * half + 2; ++rb)
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) mma32(acc[rb][jb], bf[jb], af[rb]);
  };

  // One K step.  `cur` holds its fragments; `nxt` receives the following step's.
  auto k_step = [&](int stage, int kk, V8 (&a_cur)[4], V8 (&b_cur)[4], V8 (&a_nxt)[4],
                    V8 (&b_nxt)[4]) {
    if (kk == 0) fetch(stage + 1);
    mma_half(0, a_cur, b_cur);
    __builtin_amdgcn_sched_barrier(0);
    if (kk == KK - 1) {
      // every wave finished reading buffer (stage+1)&1 before the previous barrier
      stash(stage + 1);
      __syncthreads();
      read_frags((stage + 1) & 1, 0, a_nxt, b_nxt);
    } else {
      read_frags(stage & 1, kk + 1, a_nxt, b_nxt);
    }
    __builtin_amdgcn_sched_barrier(0);
    mma_half(1, a_cur, b_cur);
  };

  V8 a0[4], b0[4], a1[4], b1[4];
  fetch(0);
  stash(0);
  __syncthreads();
  read_frags(0, 0, a0, b0);
  // U K steps per trip; stages past the end (when KK == 1 and n_stages is odd) add zeros
  const int n_steps = n_stages * KK;
  for (int t0 = 0; t0 < n_steps; t0 += U) {
#pragma unroll
    for (int u = 0; u < U; u += 2) {
      k_step(t0 / KK + u / KK, u % KK, a0, b0, a1, b1);
      k_step(t0 / KK + (u + 1) / KK, (u + 1) % KK, a1, b1, a0, b0);
    }
  }

  // ---- epilogue: lane <-> row i, register quads <-> 4 consecutive j ----
  T* x_c = x + (int64_t)c * n * n;
  T* st = lds_stage[wave];
  const int i0 = ti * 256 + wi * 128, j0 = tj * 256 + wj * 128;
  const bool vec_ok = (n % G::VE) == 0;
#pragma unroll
  for (int rb = 0; rb < 4; ++rb)
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      // put: lane ln = row i (major), acc register r = column j (minor) acc_row(r, g)
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        f32x4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[rb][jb][4 * qd + e];
        const V4 pk = from_f32<T>(v);
        T* dst = st + ln * G::PITCH + 8 * qd + 4 * g;
        if constexpr (sizeof(T) == 2) {
          *reinterpret_cast<V4*>(dst) = pk;
        } else {
          reinterpret_cast<f32x2*>(dst)[0] = f32x2{pk[0], pk[1]};
          reinterpret_cast<f32x2*>(dst)[1] = f32x2{pk[2], pk[3]};
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int ps = 0; ps < G::NPASS; ++ps) {
        const int row = ps * G::MPP + lane / G::LPM;
        const int col = (lane % G::LPM) * G::VE;
        const int i = i0 + rb * 32 + row, j = j0 + jb * 32 + col;
        const T* s = st + row * G::PITCH + col;
        if (i < n) {
          T* dst = x_c + (int64_t)i * n + j;
          if (vec_ok) {
            if (j < n) {   // n % VE == 0: the whole vector is in range
              typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
              typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
              const u32x2 lo = reinterpret_cast<const u32x2*>(s)[0];
              const u32x2 hi = reinterpret_cast<const u32x2*>(s)[1];
              *reinterpret_cast<u32x4*>(dst) = u32x4{lo[0], lo[1], hi[0], hi[1]};
            }
          } else {
#pragma unroll
            for (int e = 0; e < G::VE; ++e)
              if (j + e < n) dst[e] = s[e];
          }
        }
      }
    }
}

template <typename T>
int nt_gemm_batched(const T* a, const T* b, T* x, int n, int k_pitch, int batch,
                    hipStream_t stream) {
  if (n == 0 || batch == 0) return 0;
  const int tiles_i = (n + 255) / 256, tiles_j = (n + 255) / 256;
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
