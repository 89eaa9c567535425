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
// (global_load_lds_dwordx4: no registers, no LDS write instructions; scalar base
// address + lane offset + immediate, so no vector ALU work either) into a ring of
// 4 stage buffers, issued three stages ahead of their use.
// With one wave per SIMD nothing else hides latency, so the wave is pipelined by
// hand: the fragments of K step t+1 are read from LDS under step t's MFMAs, and
// loads and LDS reads are spread evenly between the MFMAs.
//
// Workgroups are persistent, one per CU: each walks over its share of the
// (channel, tile) list and the stage ring runs on from one tile into the next, so
// the first stages of the next tile are in flight while the results of the
// current one are stored.  All tiles of one channel are handled by one XCD
// (workgroup id % 8), keeping that channel's panels in its L2.
//
// MFMA operands are ordered so that a lane ends up holding 4 consecutive j per
// register quad of one row i; the two half-waves exchange quads
// (v_permlane32_swap) and every lane stores 16-byte runs of its row straight from
// registers.  No load sits under a branch (indices are clamped; K between n and
// k_pitch must hold zeros, which the projection kernel writes).
#include <algorithm>
#include <type_traits>

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
};

// JB = 32-wide blocks of j per wave: the workgroup tile is 256 (i) x 64*JB (j).  Only JB = 4 is
// launched: a narrower tile (JB = 3 would give N = 768 twelve tiles per channel, exactly six
// rounds of the machine instead of 4.5) was measured to take as long per K stage as the full
// one - the stage time is set by the operand delivery, not by the MFMAs - so it only loses.
//
// A workgroup is persistent: it walks over its share of the (channel, tile) list, and the
// stage ring simply runs on from one tile into the next, so the loads of the next tile's first
// stages are in flight while the current tile's results are stored.
template <typename T, int JB>
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
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int ln = lane & 31, g = lane >> 5;
  const int wi = wave >> 1, wj = wave & 1;

  // Work list of this XCD (workgroups are dealt round-robin to the 8 XCDs): its channels
  // c = 8*q + xcd, all tiles of one channel in a row, so that a channel's panels stay in one
  // L2.  Workgroup `local` of the XCD takes entries local, local + per_xcd, ...
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3, per_xcd = gridDim.x >> 3;
  const int tiles = tiles_i * tiles_j;
  const int n_entries = batch > xcd ? ((batch - xcd + 7) >> 3) * tiles : 0;
  const int my_count = n_entries > local ? (n_entries - local + per_xcd - 1) / per_xcd : 0;
  if (my_count == 0) return;

  const int n_rb = (n + 31) >> 5;          // row blocks per channel
  const int n_ks = k_pitch >> 4;           // K steps per row block
  const int n_stages = k_pitch / BK;       // K padding up to k_pitch holds zeros

  auto entry_coords = [&](int m, int& c, int& ti, int& tj) {
    const int e = local + m * per_xcd;
    const int q = e / tiles, tile = e - q * tiles;
    c = q * 8 + xcd;
    ti = tile / tiles_j;
    tj = tile - ti * tiles_j;
  };

  // ---- load cursor: runs three stages ahead of the compute cursor, across tiles ----
  // The fragments this wave moves global -> LDS each stage: RUNS runs of KK consecutive K
  // steps of one (operand, row block), consecutive in memory; src = lane address of piece 0.
  // (With JB = 3 two of the sixteen runs have no row block: they re-load another one into a
  // slot nobody reads, which keeps the number of loads per wave and step fixed.)
  // The load address is a wave-uniform base per run (scalar registers), this lane's offset
  // inside a fragment, and an immediate for the K step and piece.
  constexpr int kFragBytes = kFragElems * (int)sizeof(T);
  const uint32_t lane_off = lane * 8 * (uint32_t)sizeof(T);
  auto run_bases = [&](int m, uint64_t (&base)[RUNS]) {
    int c, ti, tj;
    entry_coords(min(m, my_count - 1), c, ti, tj);
#pragma unroll
    for (int q = 0; q < RUNS; ++q) {
      const int run = wave * RUNS + q;              // 0..15: operand = run / 8, row block = run % 8
      const int op = run >> 3, rbi = run & 7;
      int rb = op ? tj * (2 * JB) + (rbi < 2 * JB ? rbi : 0) : ti * 8 + rbi;
      rb = min(rb, n_rb - 1);                       // blocks past the end re-read the last
      base[q] = uniform64((uint64_t)((op ? b : a) + trimul_frag_offset(c, rb, 0, n_rb, n_ks)));
    }
  };
  // cur_base: the cursor's stage (entry base + stage offset); next_base: the following entry.
  // Past the last entry the cursor wraps onto the last entry again: those loads land in
  // buffers nobody reads any more (no load sits under a branch).
  uint64_t cur_base[RUNS], next_base[RUNS];
  run_bases(0, cur_base);
  run_bases(1, next_base);   // (refreshed at the top of every tile)
  int dma_s = 0, dma_buf = 0;   // stage within the cursor's entry, ring buffer
  // Direct-to-LDS loads of K step KK_ of the load cursor's stage: each moves 16 bytes per
  // lane to consecutive LDS slots, which is the fragment image itself.
  // (The instruction's immediate offset applies to the global AND the LDS address.  For
  // bf16 the K steps of a run are 1 KB apart in both, so step kk is the immediate kk KB on
  // step 0's addresses; the second 16-byte piece of an fp32 fragment is 16 bytes on in
  // memory but a whole lane row on in LDS, so it gets a lane offset of its own.)
  auto dma_part = [&](auto kk_tag) {
    constexpr int kk = decltype(kk_tag)::value;
#pragma unroll
    for (int q = 0; q < RUNS; ++q) {
      const int frag0 = (wave * RUNS + q) * KK;
      if constexpr (PIECES == 1) {
        static_assert(PIECES != 1 || sizeof(u32x4_t) * kWave == kFragBytes, "LDS slot = fragment");
        load_to_lds16_s<kk * kFragBytes>(cur_base[q], lane_off,
                                         lds_address(&lds_f[dma_buf][frag0][0][0]));
      } else {
        static_assert(PIECES == 1 || KK == 1, "one K step per stage");
        load_to_lds16_s<0>(cur_base[q], lane_off, lds_address(&lds_f[dma_buf][frag0][0][0]));
        load_to_lds16_s<0>(cur_base[q], lane_off + 16, lds_address(&lds_f[dma_buf][frag0][1][0]));
      }
    }
  };
  // Next stage; at the end of an entry the cursor moves to the next one (branch-free: the
  // K loop must stay one basic block for its hand-placed issue order).
  auto dma_advance = [&]() {
    dma_buf = (dma_buf + 1) & (NBUF - 1);
    const bool wrap = dma_s + 1 == n_stages;
    dma_s = wrap ? 0 : dma_s + 1;
#pragma unroll
    for (int q = 0; q < RUNS; ++q)
      cur_base[q] = wrap ? next_base[q] : cur_base[q] + (uint64_t)(KK * kFragBytes);
  };

  auto read_one = [&](int buf, int frag) {
    V8 v;
    u32x4_t* d = reinterpret_cast<u32x4_t*>(&v);
#pragma unroll
    for (int pc = 0; pc < PIECES; ++pc) d[pc] = lds_f[buf][frag][pc][lane];
    return v;
  };
  // fragments of one K step: this wave's 4 row blocks of a and JB of b
  auto read_frags = [&](int buf, int kk, V8 (&af)[4], V8 (&bf)[JB]) {
#pragma unroll
    for (int r = 0; r < 4; ++r) af[r] = read_one(buf, (wi * 4 + r) * KK + kk);
#pragma unroll
    for (int r = 0; r < JB; ++r) bf[r] = read_one(buf, (8 + wj * JB + r) * KK + kk);
  };

  f32x16 acc[4][JB];   // [row block of a][row block of b]
  int cbuf = 0;        // ring buffer of the compute cursor's stage

  // One K step.  `cur` holds its fragments; `nxt` receives the following step's.
  //   Buffer use: stage S is computed from buffer S % 4 while the loads of stage S + 3 land
  // in buffer (S + 3) % 4, whose last readers (stage S - 1) finished before the barrier in
  // stage S - 1's last step.  Before that barrier each wave waits until its own loads of the
  // next stage have landed: loads complete in issue order, and the only younger ones are
  // those of stage S + 2 and the part of stage S + 3 issued so far (the stores of a tile's
  // results, issued between two stages, only make that wait stricter).
  auto k_step = [&](auto first_tag, auto kk_tag, V8 (&a_cur)[4], V8 (&b_cur)[JB], V8 (&a_nxt)[4],
                    V8 (&b_nxt)[JB]) {
    constexpr bool FIRST = decltype(first_tag)::value;   // first K step of a tile: acc = product
    constexpr int kk = decltype(kk_tag)::value;
    if (kk == KK - 1) {
      ring_barrier<G::DMA_PER_STEP * (KK + KK - 1)>();
      cbuf = (cbuf + 1) & (NBUF - 1);
      read_frags(cbuf, 0, a_nxt, b_nxt);
    } else {
      read_frags(cbuf, kk + 1, a_nxt, b_nxt);
    }
    dma_part(kk_tag);
    if (kk == KK - 1) dma_advance();
    // A operand = b rows (register <-> j), B operand = a rows (lane <-> i)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int jb = 0; jb < JB; ++jb) {
        if (FIRST) {
          const f32x16 z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
          acc[rb][jb] = z;
        }
        mma32(acc[rb][jb], b_cur[jb], a_cur[rb]);
      }
    if constexpr (sizeof(T) == 2) {
      // issue order: 2 MFMAs, then one LDS read
#pragma unroll
      for (int grp = 0; grp < 2 * JB; ++grp) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    }
  };

  // ---- results of one tile, straight from the accumulators ----
  // A lane holds row i = its lane % 32 and, per 32-wide block of j, the register quads
  // j = 8*qd + 4*g .. +3 (g = lane / 32).  fp32: a quad is 16 bytes, stored as it is.  bf16:
  // the two half-waves first exchange quads (v_permlane32_swap: the upper half of one
  // register with the lower half of another), after which the lower half-wave holds
  // j = 0..7 and 16..23 of its row and the upper one 8..15 and 24..31: 16-byte stores again,
  // and no trip through LDS.  (Measured against whole 128-byte lines through a per-wave LDS tile,
  // 8 rows per store instruction instead of 32-byte pieces of 32 lines: 150 against 145 us per
  // launch at N = 768, 1780 against 1745 at 2048 - with one wave per SIMD the extra LDS round
  // trips cost more than the lines save.)
  const bool vec_ok = (n % G::VE) == 0;
  auto store_tile = [&](int m) {
    int c, ti, tj;
    entry_coords(m, c, ti, tj);
    T* x_c = x + (int64_t)c * n * n;
    const int i0 = ti * 256 + wi * 128, j0 = tj * (64 * JB) + wj * (32 * JB);
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      const int i = i0 + rb * 32 + ln;
      T* x_row = x_c + (int64_t)i * n;
#pragma unroll
      for (int jb = 0; jb < JB; ++jb) {
        const int jt = j0 + jb * 32;
        if constexpr (sizeof(T) == 2) {
          typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
          uint32_t pk[4][2];   // [quad][pair]: two bf16 each
#pragma unroll
          for (int qd = 0; qd < 4; ++qd) {
            f32x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc[rb][jb][4 * qd + e];
            const V4 h = from_f32<T>(v);
            const uint32_t* hw = reinterpret_cast<const uint32_t*>(&h);
            pk[qd][0] = hw[0];
            pk[qd][1] = hw[1];
          }
#pragma unroll
          for (int p = 0; p < 2; ++p) {   // quads (0,1) and (2,3)
            u32x4 out;
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
              // upper lanes' quad 2p  <->  lower lanes' quad 2p+1
              const auto r = __builtin_amdgcn_permlane32_swap(pk[2 * p][hh], pk[2 * p + 1][hh],
                                                              false, false);
              out[hh] = r[0];       // lower: own quad 2p      | upper: partner's quad 2p+1
              out[2 + hh] = r[1];   // lower: partner's quad 2p | upper: own quad 2p+1
            }
            const int j = jt + 16 * p + 8 * g;
            if (i < n) {
              if (vec_ok) {
                if (j < n) *reinterpret_cast<u32x4*>(x_row + j) = out;   // n % 8 == 0: all in range
              } else {
                const T* e8 = reinterpret_cast<const T*>(&out);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                  if (j + e < n) x_row[j + e] = e8[e];
              }
            }
          }
        } else {
#pragma unroll
          for (int qd = 0; qd < 4; ++qd) {
            const int j = jt + 8 * qd + 4 * g;
            if (i < n) {
              if (vec_ok) {
                if (j < n)
                  *reinterpret_cast<f32x4*>(x_row + j) =
                      f32x4{acc[rb][jb][4 * qd], acc[rb][jb][4 * qd + 1], acc[rb][jb][4 * qd + 2],
                            acc[rb][jb][4 * qd + 3]};
              } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  if (j + e < n) x_row[j + e] = acc[rb][jb][4 * qd + e];
              }
            }
          }
        }
      }
    }
  };

  V8 a0[4], b0[JB], a1[4], b1[JB];
#pragma unroll
  for (int st0 = 0; st0 < 3; ++st0) {
    dma_part(std::integral_constant<int, 0>{});
    if constexpr (KK == 2) dma_part(std::integral_constant<int, 1>{});
    dma_advance();
  }
  ring_barrier<G::DMA_PER_STEP * KK * 2>();
  read_frags(0, 0, a0, b0);
  // Two K steps per trip (the fragment sets alternate); the number of K steps is even.
  const int n_steps = n_stages * KK;
  typedef std::integral_constant<int, 0> K0;
  typedef std::integral_constant<int, 1 % KK> K1;   // the second step of a pair
  for (int m = 0; m < my_count; ++m) {
    // (the load cursor enters entry m + 1 during this tile: its bases must be ready)
    run_bases(m + 1, next_base);
    k_step(std::true_type{}, K0{}, a0, b0, a1, b1);
    k_step(std::false_type{}, K1{}, a1, b1, a0, b0);
    for (int t0 = 2; t0 < n_steps; t0 += 2) {
      k_step(std::false_type{}, K0{}, a0, b0, a1, b1);
      k_step(std::false_type{}, K1{}, a1, b1, a0, b0);
    }
    store_tile(m);
  }

  // the loads issued past the end are still in flight: let them land
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Compute units of the current device, rounded down to whole groups of 8 (one per XCD).
static int contraction_grid() {
  static int cache[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cache[dev] == 0) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v < 8)
      v = 256;
    cache[dev] = v & ~7;
  }
  return cache[dev];
}

template <typename T>
int nt_gemm_batched(const T* a, const T* b, T* x, int n, int k_pitch, int batch,
                    hipStream_t stream) {
  if (n == 0 || batch == 0) return 0;
  const int grid = contraction_grid();
  const int tiles_i = (n + 255) / 256;
  const int64_t groups = (batch + 7) / 8;
  const int tiles_j = (n + 255) / 256;
  const int64_t blocks = std::min<int64_t>(grid, groups * tiles_i * tiles_j * 8);
  nt_gemm_batched_kernel<T, 4><<<dim3((unsigned)((blocks + 7) & ~7)), dim3(256), 0, stream>>>(
      a, b, x, n, k_pitch, batch, tiles_i, tiles_j);
  return 0;
}

template int nt_gemm_batched<float>(const float*, const float*, float*, int, int, int, hipStream_t);
template int nt_gemm_batched<bf16_t>(const bf16_t*, const bf16_t*, bf16_t*, int, int, int,
                                     hipStream_t);

}  // namespace ptx
