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
// SIMD), so each fragment read from LDS feeds 4 MFMAs.  K stages (KK steps of
// 16) of both operand panels travel global -> LDS with direct-to-LDS loads
// (global_load_lds_dwordx4: no registers, no LDS write instructions) into a
// ring of 4 stage buffers, issued three stages ahead of their use: concurrent
// tiles of one channel walk K in lockstep, so every load sees HBM latency.
// With one wave per SIMD nothing else hides latency, so the wave is pipelined by
// hand: the fragments of K step t+1 are read from LDS under step t's MFMAs, and
// loads and LDS reads are spread evenly between the MFMAs.
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
  static constexpr int KK = sizeof(T) == 2 ? 2 : 1;   // 16-deep K steps per stage
  static constexpr int BK = 16 * KK;
  static constexpr int NBUF = 4;                      // LDS stage buffers (loads run 3 stages ahead)
  static constexpr int PIECES = (int)sizeof(T) / 2;   // 16-byte pieces per lane and fragment
  static constexpr int NF = 16 * KK;                  // fragments per stage (a: 8 row blocks, b: 8)
  static constexpr int RUNS = 4;                      // (operand, row block) runs each wave moves
  static constexpr int DMA_PER_STEP = RUNS * PIECES;  // direct-to-LDS loads a wave issues per K step
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
  constexpr int KK = G::KK, BK = G::BK, NBUF = G::NBUF, PIECES = G::PIECES, RUNS = G::RUNS;
  // [buffer][operand*8*KK + row block*KK + kk][16-byte piece][lane]
  __shared__ u32x4_t lds_f[NBUF][G::NF][PIECES][kWave];
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
  const int n_stages = k_pitch / BK;       // K padding up to k_pitch holds zeros

  // The fragments this wave moves global -> LDS each stage: RUNS runs of KK consecutive K
  // steps of one (operand, row block), consecutive in memory.  Lane address of piece 0.
  const T* src[RUNS];
#pragma unroll
  for (int q = 0; q < RUNS; ++q) {
    const int run = wave * RUNS + q;              // 0..15: operand = run / 8, row block = run % 8
    const int op = run >> 3;
    const int rb = min((op ? tj : ti) * 8 + (run & 7), n_rb - 1);   // blocks past the end re-read the last
    src[q] = (op ? b : a) + trimul_frag_offset(c, rb, 0, n_rb, n_ks) + lane * 8;
  }

  // Direct-to-LDS loads of K step kk of `stage` (clamped for the address): each moves 16
  // bytes per lane to consecutive LDS slots, which is the fragment image itself.
  auto dma_part = [&](int stage, int kk) {
    const int ks = min(stage, n_stages - 1) * KK + kk;
    const int buf = stage & (NBUF - 1);
#pragma unroll
    for (int q = 0; q < RUNS; ++q)
#pragma unroll
      for (int pc = 0; pc < PIECES; ++pc)
        load_to_lds16(src[q] + (int64_t)ks * 512 + pc * G::VE,
                      lds_address(&lds_f[buf][(wave * RUNS + q) * KK + kk][pc][0]));
  };
  auto read_one = [&](int buf, int frag) {
    V8 v;
    u32x4_t* d = reinterpret_cast<u32x4_t*>(&v);
#pragma unroll
    for (int pc = 0; pc < PIECES; ++pc) d[pc] = lds_f[buf][frag][pc][lane];
    return v;
  };
  // fragments of one K step: this wave's 4 row blocks of a and 4 of b
  auto read_frags = [&](int stage, int kk, V8 (&af)[4], V8 (&bf)[4]) {
    const int buf = stage & (NBUF - 1);
#pragma unroll
    for (int r = 0; r < 4; ++r) af[r] = read_one(buf, (wi * 4 + r) * KK + kk);
#pragma unroll
    for (int r = 0; r < 4; ++r) bf[r] = read_one(buf, (8 + wj * 4 + r) * KK + kk);
  };

  f32x16 acc[4][4];   // [row block of a][row block of b]
#pragma unroll
  for (int rb = 0; rb < 4; ++rb)
#pragma unroll
    for (int jb = 0; jb < 4; ++jb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rb][jb][r] = 0.0f;

  // One K step.  `cur` holds its fragments; `nxt` receives the following step's.
  //   Buffer use: stage s is computed from buffer s % 4 while the loads of stage s + 3 land
  // in buffer (s + 3) % 4, whose last readers (stage s - 1) finished before the barrier in
  // stage s - 1's last step.  Before that barrier each wave waits until its own loads of the
  // next stage have landed: loads complete in issue order, and the only younger ones are
  // those of stage s + 2 and the part of stage s + 3 issued so far.
  auto k_step = [&](int stage, int kk, V8 (&a_cur)[4], V8 (&b_cur)[4], V8 (&a_nxt)[4],
                    V8 (&b_nxt)[4]) {
    if (kk == KK - 1) {
      ring_barrier<G::DMA_PER_STEP * (KK + KK - 1)>();
      read_frags(stage + 1, 0, a_nxt, b_nxt);
    } else {
      read_frags(stage, kk + 1, a_nxt, b_nxt);
    }
    dma_part(stage + 3, kk);
    // A operand = b rows (register <-> j), B operand = a rows (lane <-> i)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) mma32(acc[rb][jb], b_cur[jb], a_cur[rb]);
    if constexpr (sizeof(T) == 2) {
      // issue order: 2 MFMAs, then one LDS read
#pragma unroll
      for (int grp = 0; grp < 8; ++grp) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    }
  };

  V8 a0[4], b0[4], a1[4], b1[4];
#pragma unroll
  for (int st0 = 0; st0 < 3; ++st0)
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) dma_part(st0, kk);
  ring_barrier<G::DMA_PER_STEP * KK * 2>();
  read_frags(0, 0, a0, b0);
  // Two K steps per trip (the fragment sets alternate); the number of K steps is even.
  const int n_steps = n_stages * KK;
  for (int t0 = 0; t0 < n_steps; t0 += 2) {
    k_step(t0 / KK, 0, a0, b0, a1, b1);
    k_step((t0 + 1) / KK, (t0 + 1) % KK, a1, b1, a0, b0);
  }

  // the loads issued for stages past the end are still in flight: let them land
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

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
