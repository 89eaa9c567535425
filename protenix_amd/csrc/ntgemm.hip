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
// hides latency: the fragments of K step t+1 are read from LDS under step t's
// MFMAs, global loads are issued two stages before they are written to LDS, and
// loads, LDS writes and LDS reads are spread evenly between the MFMAs.
//
// MFMA operands are ordered so that a lane ends up holding 4 consecutive j per
// register quad of one row i: results leave through a per-wave LDS tile as
// 16-byte stores along j.  No load sits under a branch (indices are clamped;
// K between n and k_pitch must hold zeros, which the projection kernel writes).  Workgroups are numbered so that all
// tiles of one channel land on one XCD (round-robin dispatch: id % 8), keeping
// that channel's panels in its L2.
#include "common.h"
#include "kernels.h"

namespace ptx {

template <typename T> struct GemmCfg {
  static constexpr int KK = sizeof(T) == 2 ? 4 : 1;   // 16-deep K steps per stage
  static constexpr int BK = 16 * KK;
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
  constexpr int KK = G::KK, BK = G::BK, FPW = G::FPW;
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
  const int n_stages = k_pitch / BK;        // K padding up to k_pitch holds zeros

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

  // Loads are issued two stages ahead of their LDS write (HBM latency under load exceeds one
  // stage of MFMA work) into two register sets that alternate by stage parity.  Everything
  // is spread evenly over the K steps of a stage so that no queue sees a burst: step kk
  // issues the loads of K step kk of stage + 2, and steps 0 .. KK-2 each write a share of
  // stage + 1 into the LDS buffer that the barrier of the previous stage's last step freed.
  V8 pre0[FPW], pre1[FPW];
  auto fetch_part = [&](int stage, int kk, V8 (&pre)[FPW]) {   // stage clamped for the address
    const int ks = min(stage, n_stages - 1) * KK + kk;
#pragma unroll
    for (int q = 0; q < FPW / KK; ++q) pre[q * KK + kk] = load8<T>(src[q] + (int64_t)ks * 512);
  };
  // share `part` of `parts`: fragments in the order their loads were issued (K step major),
  // so every fragment has been in flight for at least KK - 1 steps when it is written
  auto stash_part = [&](int stage, int part, int parts, V8 (&pre)[FPW]) {
#pragma unroll
    for (int f = 0; f < FPW; ++f) {
      const int order = (f % KK) * (FPW / KK) + f / KK;
      if (order * parts / FPW == part) lds_f[stage & 1][wave * FPW + f][lane] = pre[f];
    }
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

  // One K step.  `cur` holds its fragments; `nxt` receives the following step's.  `p_in` takes
  // the loads of stage + 2, `p_out` holds stage + 1.
  auto k_step = [&](int stage, int kk, V8 (&a_cur)[4], V8 (&b_cur)[4], V8 (&a_nxt)[4],
                    V8 (&b_nxt)[4], V8 (&p_in)[FPW], V8 (&p_out)[FPW]) {
    if (KK == 1) stash_part(stage + 1, 0, 1, p_out);
    // all shares of stage + 1 are in LDS once every wave passes here; nobody still reads
    // the other buffer's previous contents after the barrier one stage earlier
    if (kk == KK - 1) __syncthreads();
    if (kk == KK - 1) read_frags((stage + 1) & 1, 0, a_nxt, b_nxt);
    else read_frags(stage & 1, kk + 1, a_nxt, b_nxt);
    fetch_part(stage + 2, kk, p_in);
    if (KK > 1 && kk < KK - 1) stash_part(stage + 1, kk, KK - 1, p_out);
    // A operand = b rows (register <-> j), B operand = a rows (lane <-> i)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) mma32(acc[rb][jb], b_cur[jb], a_cur[rb]);
    if constexpr (sizeof(T) == 2) {
      // issue order: 2 MFMAs, then one LDS read, one global load (first 4 groups) and one
      // LDS write (first 6 groups)
#pragma unroll
      for (int grp = 0; grp < 8; ++grp) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        if (grp < 4) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        if (grp < 6) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
      }
    }
  };
  auto stage_steps = [&](int stage, V8 (&p_in)[FPW], V8 (&p_out)[FPW], V8 (&a_c)[4], V8 (&b_c)[4],
                         V8 (&a_n)[4], V8 (&b_n)[4]) {
    // KK is 1 or even: with KK even a stage starts and ends on the same fragment set
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      if ((kk & 1) == 0) k_step(stage, kk, a_c, b_c, a_n, b_n, p_in, p_out);
      else k_step(stage, kk, a_n, b_n, a_c, b_c, p_in, p_out);
    }
  };

  V8 a0[4], b0[4], a1[4], b1[4];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) fetch_part(0, kk, pre0);
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) fetch_part(1, kk, pre1);
  stash_part(0, 0, 1, pre0);
  __syncthreads();
  read_frags(0, 0, a0, b0);
  // Two stages per trip (prefetch sets alternate by parity), then a last single stage.  The
  // last stage's writes and reads for "stage + 1" move valid but unused data.
  int s0 = 0;
  for (; s0 + 1 < n_stages; s0 += 2) {
    if (KK == 1) {
      stage_steps(s0, pre0, pre1, a0, b0, a1, b1);
      stage_steps(s0 + 1, pre1, pre0, a1, b1, a0, b0);
    } else {
      stage_steps(s0, pre0, pre1, a0, b0, a1, b1);
      stage_steps(s0 + 1, pre1, pre0, a0, b0, a1, b1);
    }
  }
  if (s0 < n_stages) stage_steps(s0, pre0, pre1, a0, b0, a1, b1);

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
