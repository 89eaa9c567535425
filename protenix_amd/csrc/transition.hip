// Transition (SwiGLU feed-forward) on rows of c = 128 (or 64; 256 in 16-bit arithmetic) channels, one kernel:
//   out = [x +] W_o ( silu(W_a LN(x)) * (W_b LN(x)) ),   W_a, W_b [c*n_factor][c]
// (the comments below give the sizes for c = 128).
// The hidden activations (n_factor * c per row) never leave the chip: a wave
// keeps its rows as MFMA operand fragments, walks the hidden dimension in chunks
// of 32 and accumulates the output projection as it goes.
//
//   GEMM1 (per chunk): h^T[32 hidden x 32 rows] = W[32 x 128] * LN(x)^T, so a lane ends up
//     with one row and 16 hidden values in its accumulator registers;
//   activation in registers, rounded to T;
//   GEMM2: out^T[128 x 32 rows] += W_o[:, chunk] * h^T.  Registers 8u .. 8u+7 of a lane are
//     used directly as the K slots of K step u: which hidden index a slot stands for is
//     free as long as both operands agree, and the packed W_o fragments follow the
//     accumulator's register order (no shuffles, no LDS round trip).
//
// Weights are packed once (transition_pack) into MFMA fragment order, chunk by
// chunk, and stream global -> LDS with direct-to-LDS loads into a ring of
// chunk buffers shared by the workgroup's waves.  One or two waves per SIMD (with two row
// blocks the accumulators and the row fragments take ~370 registers), so the wave is
// pipelined by hand: while the MFMAs of chunk j's GEMM1 run, the VALU computes
// the activation of chunk j-1, whose GEMM2 follows; LDS fragment reads are issued
// one step ahead of their use.
#include "common.h"
#include "kernels.h"
#include "rowtile.h"
#include <type_traits>

namespace ptx {

// KS = K steps of a row (c / 16: 8 for c = 128, 4 for c = 64, 16 for c = 256);
// NOB = c / 32 output blocks.
template <typename T, int KS> struct TrCfg {
  // (rows of 256 channels, bf16 only: one row block, and three 48 KB chunk buffers)
  // Four waves per workgroup.  bf16 rows of 128 channels: one row block per wave and a ring of
  // three chunk buffers (72 KB), so that two workgroups share a compute unit, two waves per
  // SIMD.  A single wave issues a vector instruction only every ~9 cycles (two waves: one every
  // ~5 per SIMD), and the SwiGLU is vector work, so two thin waves beat one fat one by 6 %
  // although every weight fragment read from LDS then feeds one MFMA instead of two; and two
  // workgroups of four beat one of eight by another 7 % although the weights then stream into
  // LDS twice per 256 rows: a workgroup's row loads, LayerNorm and stores leave the matrix pipe
  // idle unless another workgroup, at another point of its life, has the unit's other waves.
  static constexpr int NW = 4;
  static constexpr int RB = (sizeof(T) == 2 && KS == 4) ? 2 : 1;     // row blocks of 32 per wave
  static constexpr int NBUF = (sizeof(T) == 2 && KS == 4) ? 4 : 3;   // chunk buffers in LDS
  static constexpr int D = NBUF - 2;                    // chunks the loads run ahead (two are in use)
  static constexpr int PIECES = (int)sizeof(T) / 2;     // 16-byte pieces per lane and fragment
  static constexpr int NOB = KS / 2;
  // fragments per chunk of 32 hidden: W_a KS K steps, W_b KS, W_o NOB x 2
  static constexpr int FRAGS = 3 * KS;
  static constexpr int FPW = FRAGS / NW;                // fragments each wave moves per chunk
  static_assert(FRAGS % NW == 0, "every wave moves the same number of fragments");
  static constexpr int DMA_PER_CHUNK = FPW * PIECES;
};

// packed[chunk j][fragment f][lane][8]:
//   f <  KS:  W_a, K step f:      lane (m, g) = W_a[32j + m][16f + 8g .. +7]
//   f < 2KS:  W_b, K step f - KS
//   else:     W_o, output block ob = (f-2KS)/2, K step u = (f-2KS)%2:
//           lane (m, g), slot t = W_o[32 ob + m][32j + 8(2u + t/4) + 4g + t%4]
//           (slot t of K step u <-> accumulator register 8u + t of GEMM1)
template <typename T, int KS>
__global__ void transition_pack_kernel(const T* __restrict__ w_a, const T* __restrict__ w_b,
                                       const T* __restrict__ w_o, T* __restrict__ packed,
                                       int n_hidden) {
  constexpr int kFrags = 3 * KS;
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  const int n_chunks = n_hidden / 32;
  if (idx >= n_chunks * kFrags * kWave) return;
  const int lane = idx & 63, f = (idx >> 6) % kFrags, j = idx / (kWave * kFrags);
  const int m = lane & 31, g = lane >> 5;
  typename Vec8<T>::type v;
  if (f < 2 * KS) {
    const T* w = f < KS ? w_a : w_b;
    const int kk = f % KS;
#pragma unroll
    for (int t = 0; t < 8; ++t) v[t] = w[(int64_t)(32 * j + m) * (16 * KS) + 16 * kk + 8 * g + t];
  } else {
    const int ob = (f - 2 * KS) >> 1, u = (f - 2 * KS) & 1;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const int hidden = 32 * j + 8 * (2 * u + (t >> 2)) + 4 * g + (t & 3);
      v[t] = w_o[(int64_t)(32 * ob + m) * n_hidden + hidden];
    }
  }
  store8<T>(packed + (int64_t)idx * 8, v);
}

// TZ: storage type of x and out (float with T = bf16: rows of an fp32 residual stream are
// normalised in fp32 and rounded to T; the T-rounded update is added to the fp32 row).
// PB: the pair bias of the single-representation attention that follows the transition in
// a Pairformer block, bias[h][row] = (W LN_pb(out[row]))[h], formed from the finished rows
// while they pass through the epilogue (a kernel of its own would read the pair tensor once
// more for it).
// Sum over groups of LPM (4 or 8) neighbouring lanes on the vector ALU's lane-permute path
// (quad swaps, then the mirror of each half row): every lane of a group ends up with the sum.
template <int LPM> __device__ __forceinline__ float group_sum(float v) {
  static_assert(LPM == 4 || LPM == 8, "groups of 4 or 8 lanes");
  v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));   // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true));   // quad_perm [2,3,0,1]
  if (LPM == 8)
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true));  // row_half_mirror
  return v;
}

struct PairBiasArgs {
  const void *gamma, *beta, *w;   // LayerNorm of the bias (either may be null), W [heads][c]
  void* out;                      // [heads][n_rows], fp32 or T
  int heads, out_f32;
  float eps;
};

// AO: the last stage of a triangle attention in front of the transition,
//   x' = x + W_o (sigmoid(W_g LN_att(x)) * o)                      (layers.py:380-396)
//   out = x' + transition(x'),
// on rows of 128 channels, 4 heads of 32, 16-bit arithmetic: the attention's update never
// travels through memory as a pair tensor of its own (one write and one read of the residual
// stream less than the two kernels one after the other).  The kernel walks the rows of x in
// memory order, like the transition alone, and finds a row's attention output through a RowMap
// (the ending node's output for z[a][b] is row (b, a) of o: 64-byte pieces per head, where
// walking o's order instead would scatter the rows of x and, four bytes at a time, the pair
// bias: measured as 1.6 times the bytes written); x' exists in registers only, for the
// LayerNorm of the transition, and is formed again in the epilogue from x and the attention's
// update (kept in registers, rounded to T as the module's output is), with the roundings of
// the two separate kernels.  The two weight matrices of the attention stage travel through
// the chunk ring ahead of the transition's chunks, as three chunks of 24 fragments:
//   fragments 0 .. 31: W_g, (head c, K step kk) at 8 c + kk; 32 .. 63: W_o, (block ob, kk);
//   rows of a 32-row block permuted as in triattn_gate_out_kernel, so that accumulator
//   registers 8 u .. 8 u + 7 of half-wave g are the channels 16 u + 8 g .. + 7 of the block:
//   a lane's own fragment of K step 2 c + u.
struct AttnOutArgs {
  const void* o;             // attention output, head-major [4][n_rows][32], T, rows in the attention's order
  const void *gamma, *beta;  // the attention's LayerNorm (either may be null)
  RowMap omap;               // row of x -> element offset of its 32 channels inside a head's plane of o
  float eps;
};
constexpr int kAoChunks = 3;   // chunks of 24 fragments that hold the 64 fragments of W_g and W_o

template <typename T, int KS, typename TZ = T, bool PB = false, bool AO = false>
__global__ __launch_bounds__((TrCfg<T, KS>::NW * 64), 2) void transition_fused_kernel(
    const TZ* x, const T* __restrict__ gamma, const T* __restrict__ beta,
    const T* __restrict__ packed, TZ* out, int64_t n_rows, int n_chunks, int add_residual,
    float eps, PairBiasArgs pb, AttnOutArgs ao) {
  typedef typename Vec8<T>::type V8;
  typedef typename VecE<TZ>::type VE_t;
  typedef TrCfg<T, KS> G;
  typedef Cfg<TZ> C;   // staging tile and stores
  constexpr bool MIXED = !std::is_same<T, TZ>::value;
  constexpr int RB = G::RB, NBUF = G::NBUF, D = G::D, PIECES = G::PIECES, FPW = G::FPW, NW = G::NW;
  constexpr int NOB = G::NOB, kTrFrags = G::FRAGS, kCx = 16 * KS;
  static_assert(!AO || (KS == 8 && sizeof(T) == 2 && RB == 1 && D == 1),
                "attention-output prologue: rows of 128 channels, 16-bit arithmetic");
  constexpr int PRO = AO ? kAoChunks : 0;   // ring positions ahead of the transition's chunk 0
  const int n_ring = n_chunks + PRO;
  __shared__ u32x4_t lds_w[NBUF][kTrFrags][PIECES][kWave];
  static_assert(sizeof(TZ) * NW * 32 * C::PITCH <= sizeof(u32x4_t) * (NBUF - 1) * kTrFrags * PIECES * kWave,
                "the staging tiles reuse the chunk buffers");

  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // Workgroups take the rows back to front: the kernel before this one wrote the pair tensor
  // front to back, and its tail is what the memory-side cache still holds.
  const int64_t row0 = ((int64_t)(gridDim.x - 1 - blockIdx.x) * NW + wave) * (RB * 32);
  // Row m (0 .. 32 RB - 1) of this wave's tile in x / out, or -1.
  // (AO: tiles of two neighbouring rows a of the pair tensor times 16 positions b, so that the
  // 64-byte pieces of o for (a, b) and (a + 1, b) - rows (b, a) and (b, a + 1) of an ending
  // node's output, one 128-byte line - are read by the same wave, halved the kernel's fetches
  // of o and took 408 instead of 403 us: not used.)
  auto row_at = [&](int m) -> int64_t {
    const int64_t pr = row0 + m;
    return pr < n_rows ? pr : -1;
  };

  // PB: the bias' LayerNorm parameters as fp32, parked in LDS for the epilogue: fetched there
  // from global memory they would cost every tile a round trip that nothing hides.  (Visible
  // to all waves after the first ring barrier below.)  The bias' weight follows into the
  // freed chunk buffers when the epilogue starts.
  __shared__ __attribute__((aligned(16))) float lds_pba[2][PB ? 16 * KS : 4];
  if constexpr (PB) {
    for (int c = threadIdx.x; c < kCx; c += NW * kWave) {
      lds_pba[0][c] = pb.gamma ? to_f32(((const T*)pb.gamma)[c]) : 1.0f;
      lds_pba[1][c] = pb.beta ? to_f32(((const T*)pb.beta)[c]) : 0.0f;
    }
  }

  // chunk j (clamped for the address) -> buffer j % NBUF; every wave moves FPW fragments
  // (address = wave-uniform base in scalar registers + this lane's offset inside a fragment:
  // no vector ALU work per load)
  const uint32_t lane_off = lane * 8 * (uint32_t)sizeof(T);
  auto dma_chunk = [&](int j) {   // j: position in the ring (AO: the attention stage's chunks first)
    const int jc = min(j, n_ring - 1);
    const int buf = j % NBUF;
    const uint64_t base = uniform64(
        (uint64_t)(packed + ((int64_t)jc * kTrFrags + wave * FPW) * kFragElems));
#pragma unroll
    for (int q = 0; q < FPW; ++q) {
      const int frag = wave * FPW + q;
      const uint64_t fb = base + (uint64_t)q * (kFragElems * sizeof(T));
#pragma unroll
      for (int pc = 0; pc < PIECES; ++pc)
        load_to_lds16_s<0>(fb, lane_off + 16 * pc, lds_address(&lds_w[buf][frag][pc][0]));
    }
  };
  // A chunk buffer is read through this lane's LDS address of its first fragment, formed once
  // per chunk and made opaque: the fragment number is then the immediate offset of the LDS read.
  // (Left to itself the compiler keeps one address register per fragment and forms every
  // address with two vector adds from a buffer offset it tracks in scalar registers: 44 adds
  // per chunk next to the 104 instructions of the activation, and 25 registers.)
  typedef __attribute__((address_space(3))) const u32x4_t* BufPtr;
  auto buf_ptr = [&](int buf) -> BufPtr {
    uint32_t a = (uint32_t)(uintptr_t)(BufPtr)&lds_w[buf][0][0][lane];
    asm volatile("" : "+v"(a));
    return (BufPtr)(uintptr_t)a;
  };
  auto read_frag = [&](BufPtr base, int frag) {
    V8 v;
    u32x4_t* d = reinterpret_cast<u32x4_t*>(&v);
#pragma unroll
    for (int pc = 0; pc < PIECES; ++pc) d[pc] = base[(frag * PIECES + pc) * kWave];
    return v;
  };

  // start the weight ring, then fetch and normalise this wave's rows
  // (AO: the three chunks of the attention stage at once, into the three empty buffers - the
  // prologue's steps are far shorter than a chunk's way from the L2, one chunk ahead would not do)
#pragma unroll
  for (int j = 0; j < (AO ? PRO : D); ++j) dma_chunk(j);
  RowFrags<T, RB, KS> xf;
  V8 upd[AO ? KS : 1];   // AO: the attention's update of this lane's row, rounded to T
  if constexpr (!AO) {
    load_rows<T, RB, true>(xf, x, RowMap{kCx, 0, 1}, row0, n_rows, gamma, beta, eps, lane);
  } else {
    typedef typename Vec8<TZ>::type VZ;
    const int n = lane & 31, g = lane >> 5;
    const int64_t pr = row_at(n);
    const int64_t prc = pr >= 0 ? pr : n_rows - 1;
    const TZ* zp = x + prc * kCx + 8 * g;
    const T* op = (const T*)ao.o + ao.omap(prc) + 8 * g;
    f32x8 zr[KS];   // the raw row, then x'
    V8 of[KS];      // the attention output of the row, then gated
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) zr[kk] = to_f32(load8<TZ>(zp + 16 * kk));
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
      of[kk] = load8<T>(op + (int64_t)(kk >> 1) * n_rows * 32 + 16 * (kk & 1));
    V8 xg[KS];
    {
      f32x8 v[KS];
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) v[kk] = zr[kk];
      normalize_row<T, KS>(v, (const T*)ao.gamma, (const T*)ao.beta, ao.eps, g, xg);
    }
    // gate of head c from the fragments at `f0` of a chunk buffer, applied to the attention
    // output in place (both rounded to T like the reference's sigmoid(linear_g(x)) and o * g)
    auto gate_head = [&](BufPtr b, int f0, int c) {
      f32x16 accg;
#pragma unroll
      for (int r = 0; r < 16; ++r) accg[r] = 0.0f;
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) mma32(accg, read_frag(b, f0 + kk), xg[kk]);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const f32x8 ov = to_f32(of[2 * c + u]);
        f32x8 gated;
#pragma unroll
        for (int t = 0; t < 8; ++t)
          gated[t] = ov[t] * to_f32(from_f32<T>(sigmoidf_fast(accg[8 * u + t])));
        of[2 * c + u] = from_f32<T>(gated);
      }
    };
    // output block ob of the attention: the update rounded to T, then x' = x + update as stored
    auto out_block = [&](BufPtr b, int f0, int ob) {
      f32x16 acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) mma32(acc, read_frag(b, f0 + kk), of[kk]);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        f32x8 a8;
#pragma unroll
        for (int t = 0; t < 8; ++t) a8[t] = acc[8 * u + t];
        upd[2 * ob + u] = from_f32<T>(a8);
        const f32x8 uf = to_f32(upd[2 * ob + u]);
        f32x8 v;
#pragma unroll
        for (int t = 0; t < 8; ++t) v[t] = zr[2 * ob + u][t] + uf[t];
        zr[2 * ob + u] = to_f32(from_f32<TZ>(v));
      }
    };
    // ring positions 0 .. 2 sit in buffers 0 .. 2; the transition's first chunk follows into
    // buffer 0 once every wave is done with position 0, its second one (into buffer 1) is
    // requested by the main loop's first step, behind a barrier that every wave reaches after
    // its last read of positions 1 and 2
    static_assert(!AO || (NBUF == 3 && PRO == 3), "one buffer per prologue chunk");
    ring_barrier<0>();
    {
      const BufPtr b = buf_ptr(0);
#pragma unroll
      for (int c = 0; c < 3; ++c) gate_head(b, 8 * c, c);
    }
    ring_barrier<0>();
    dma_chunk(PRO);
    {
      const BufPtr b = buf_ptr(1);
      gate_head(b, 0, 3);
      out_block(b, 8, 0);
      out_block(b, 16, 1);
    }
    {
      const BufPtr b = buf_ptr(2);
      out_block(b, 0, 2);
      out_block(b, 8, 3);
    }
    normalize_row<T, KS>(zr, gamma, beta, eps, g, xf.f[0]);
  }

  f32x16 acc_o[RB][NOB];   // [row block][output column block]: lane <-> row, register <-> column
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int ob = 0; ob < NOB; ++ob)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc_o[rb][ob][r] = 0.0f;
  f32x16 ab0[RB][2], ab1[RB][2];   // GEMM1 accumulators (a, b) of even / odd chunks
  V8 hf[RB][2];                    // activated hidden values as GEMM2 operand fragments

  // One KS-th of a chunk's activation: accumulator registers (16/KS)*part .. +16/KS-1.
  // a and b stay in fp32 through the activation; the product is rounded to T once.
  auto act_part = [&](int part, f32x16 (&ab)[RB][2]) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int e = 0; e < 16 / KS; ++e) {
        const int r = (16 / KS) * part + e;
        const float a = ab[rb][0][r], b = ab[rb][1][r];
        hf[rb][r >> 3][r & 7] = from_f32<T>(a * b * sigmoidf_fast(a));
      }
  };
  // GEMM1 of the chunk in buffer `buf` into `cur` (lane <-> row, register <-> hidden), with
  // the activation of the previous chunk (`prev`) between its MFMAs when ACT.  Fragments
  // are read from LDS one K step before they are used; the last step fetches the first
  // W_o fragment of the GEMM2 that follows (buffer `tail_buf`) and returns it.
  auto gemm1 = [&](auto act_tag, BufPtr buf, f32x16 (&cur)[RB][2], f32x16 (&prev)[RB][2],
                   BufPtr tail_buf) {
    constexpr bool ACT = decltype(act_tag)::value;
    V8 wa = read_frag(buf, 0), wb = read_frag(buf, KS);
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
      V8 na, nb = wb;
      if (kk + 1 < KS) {
        na = read_frag(buf, kk + 1);
        nb = read_frag(buf, KS + kk + 1);
      } else {
        na = read_frag(tail_buf, 2 * KS);
      }
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        if (kk == 0) {   // first K step: accumulate onto a constant zero (no register clears)
          const f32x16 z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
          cur[rb][0] = z;
          cur[rb][1] = z;
        }
        mma32(cur[rb][0], wa, xf.f[rb][kk]);
        mma32(cur[rb][1], wb, xf.f[rb][kk]);
      }
      if (ACT) act_part(kk, prev);
      wa = na;
      wb = nb;
    }
    return wa;
  };
  // GEMM2 of the chunk whose W_o fragments sit in buffer `buf`; `wo` is its first fragment.
  auto gemm2 = [&](BufPtr buf, V8 wo) {
#pragma unroll
    for (int s2 = 0; s2 < 2 * NOB; ++s2) {
      const int u = s2 / NOB, ob = s2 % NOB;
      V8 nw = wo;
      if (s2 + 1 < 2 * NOB) nw = read_frag(buf, 2 * KS + ((s2 + 1) % NOB) * 2 + ((s2 + 1) / NOB));
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) mma32(acc_o[rb][ob], wo, hf[rb][u]);
      wo = nw;
    }
  };
  // Iteration j: chunk j has landed in every wave's share of buffer j % NBUF once all waves
  // pass the barrier (loads complete in issue order; the only younger ones are chunks
  // j+1 .. j+D-1), and every wave has finished reading buffer (j-2) % NBUF, which the loads
  // of chunk j + D now refill.
  auto iteration = [&](int j, f32x16 (&cur)[RB][2], f32x16 (&prev)[RB][2]) {   // j: ring position
    ring_barrier<(D - 1) * G::DMA_PER_CHUNK>();
    dma_chunk(j + D);
    const BufPtr cbuf = buf_ptr(j % NBUF), pbuf = buf_ptr((j + NBUF - 1) % NBUF);
    const V8 wo = gemm1(std::true_type{}, cbuf, cur, prev, pbuf);
    gemm2(pbuf, wo);
  };

  // chunk 0: GEMM1 only
  ring_barrier<(D - 1) * G::DMA_PER_CHUNK>();
  dma_chunk(PRO + D);
  {
    const BufPtr b0 = buf_ptr(PRO % NBUF);
    gemm1(std::false_type{}, b0, ab0, ab1, b0);
  }
  // chunks 1 .. n_chunks-1 (n_chunks is even): GEMM1(j), activation and GEMM2 of j-1
  int j = 1;
  for (; j + 1 < n_chunks; j += 2) {
    iteration(PRO + j, ab1, ab0);
    iteration(PRO + j + 1, ab0, ab1);
  }
  iteration(PRO + j, ab1, ab0);
  // The residual vectors this lane will add in the epilogue, requested now so that their
  // latency passes under the drain (loading each one next to its store would serialise a
  // full memory round trip per tile: out may alias x, so no load could move above the
  // previous store).  Each lane reads exactly the vectors it later overwrites.
  // (fp32 rows of 256 channels: 32 residual vectors per lane do not fit beside the output
  // accumulators; the second half of the column blocks is requested after the first half's
  // stores, one serialised round trip per wave)
  // (the lane index again, opaque to the compiler: the values derived from it up here would
  // otherwise be carried through the chunk loop, in registers the AO instantiations do not
  // have - they were spilled ahead of the prologue and read back here)
  int lane_e = (int)(threadIdx.x & 63);
  asm volatile("" : "+v"(lane_e));
  constexpr int GOB = (MIXED && NOB > 4) ? 4 : NOB;
  int64_t obase[RB][C::NPASS];
  VE_t resv[RB][GOB][C::NPASS];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int ps = 0; ps < C::NPASS; ++ps) {
      int mj, m0;
      stage_coord<TZ>(ps, lane_e, mj, m0);
      const int64_t pr = row_at(rb * 32 + mj);
      obase[rb][ps] = pr >= 0 ? pr * kCx + m0 : -1;
    }
  auto load_residual = [&](int ob0) {
    if (add_residual) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int ob = 0; ob < GOB; ++ob)
#pragma unroll
          for (int ps = 0; ps < C::NPASS; ++ps)
            if (obase[rb][ps] >= 0)
              resv[rb][ob][ps] = *reinterpret_cast<const VE_t*>(x + obase[rb][ps] + (ob0 + ob) * 32);
    }
  };
  load_residual(0);
  // drain: activation and GEMM2 of the last chunk
#pragma unroll
  for (int kk = 0; kk < KS; ++kk) act_part(kk, ab1);
  {
    const BufPtr lbuf = buf_ptr((PRO + n_chunks - 1) % NBUF);
    gemm2(lbuf, read_frag(lbuf, 2 * KS));
  }

  // ---- epilogue: out rows through the per-wave staging tile (reuses the chunk buffers once
  // every wave is past its last fragment read and all loads have landed) ----
  ring_barrier<0>();
  TZ* st = reinterpret_cast<TZ*>(&lds_w[0][0][0][0]) + wave * (32 * C::PITCH);
  // PB: the bias' weight as A fragments (rows beyond `heads` repeat the last head: those
  // accumulator rows are not stored), behind the staging and normalised tiles; it arrives
  // by direct-to-LDS loads while the rows are stored (waited for before its first use).
  constexpr int kPitchN = 64 + 4;      // normalised tile, elements: 34 dwords, rows 8-byte aligned
  constexpr size_t kPbwOffset = PB ? (NW * 32 * (C::PITCH * sizeof(TZ) + kPitchN * sizeof(T)) + 1023) / 1024 * 1024 : 0;
  static_assert(!PB || kPbwOffset + KS * kWave * sizeof(V8) <= sizeof(u32x4_t) * NBUF * kTrFrags * PIECES * kWave,
                "staging tiles, normalised tiles and the bias weight fit the chunk buffers");
  V8 (*lds_pbw)[kWave] = reinterpret_cast<V8 (*)[kWave]>(reinterpret_cast<char*>(&lds_w[0][0][0][0]) + kPbwOffset);
  if constexpr (PB) {
    static_assert(!PB || sizeof(V8) == 16, "one 16-byte piece per lane_e and fragment");
    const uint32_t voff = (uint32_t)((min(lane_e & 31, pb.heads - 1) * kCx + 8 * (lane_e >> 5)) * sizeof(T));
    for (int f = wave; f < KS; f += NW)
      load_to_lds16_s<0>(uniform64((uint64_t)((const T*)pb.w + 16 * f)), voff, lds_address(&lds_pbw[f][0]));
  }
  VE_t done[PB ? RB : 1][PB ? NOB : 1][PB ? C::NPASS : 1];   // PB: the finished rows, as stored
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
    for (int ob = 0; ob < NOB; ++ob) {
      if (GOB < NOB && ob > 0 && ob % GOB == 0) {
        static_assert(GOB == NOB || RB == 1, "column groups: one row block");
        load_residual(ob);
      }
      float vals[16];
#pragma unroll
      for (int r = 0; r < 16; ++r)   // (mixed: the update is rounded to T before it is added)
        vals[r] = MIXED ? to_f32(from_f32<T>(acc_o[rb][ob][r])) : acc_o[rb][ob][r];
      if constexpr (AO) {
        // x' of the block's columns, as the attention stage would have stored it: its update
        // goes from the fragment layout (lane_e <-> row, channels 16 u + 8 g .. + 7) through the
        // staging tile to the layout of the stores and meets the raw row there
        typedef typename Vec8<TZ>::type VZ;
        const int n = lane_e & 31, g = lane_e >> 5;
        wave_lds_sync();
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const VZ pk = from_f32<TZ>(to_f32(upd[2 * ob + u]));
          u32x2* d2 = reinterpret_cast<u32x2*>(st + n * C::PITCH + 16 * u + 8 * g);
          const u32x2* s2 = reinterpret_cast<const u32x2*>(&pk);
#pragma unroll
          for (int w8 = 0; w8 < (int)sizeof(VZ) / 8; ++w8) d2[w8] = s2[w8];
        }
        wave_lds_sync();
#pragma unroll
        for (int ps = 0; ps < C::NPASS; ++ps) {
          int mj, m0;
          stage_coord<TZ>(ps, lane_e, mj, m0);
          resv[rb][ob % GOB][ps] = add_vec<TZ>(stage_get_vec<TZ>(st, mj, m0), resv[rb][ob % GOB][ps]);
        }
      }
      wave_lds_sync();
      stage_put<TZ>(st, vals, lane_e);
      wave_lds_sync();
#pragma unroll
      for (int ps = 0; ps < C::NPASS; ++ps) {
        int mj, m0;
        stage_coord<TZ>(ps, lane_e, mj, m0);
        VE_t v = stage_get_vec<TZ>(st, mj, m0);
        if (obase[rb][ps] >= 0) {
          if (add_residual) v = add_vec<TZ>(v, resv[rb][ob % GOB][ps]);
          *reinterpret_cast<VE_t*>(out + obase[rb][ps] + ob * 32) = v;
        }
        if constexpr (PB) done[rb][ob][ps] = v;
      }
    }
  }

  if constexpr (PB) {
    static_assert(!PB || (RB == 1 && sizeof(T) == 2), "pair-bias epilogue: one row block, 16-bit arithmetic");
    const int n = lane_e & 31, g = lane_e >> 5;
    const int m0c = (lane_e % C::LPM) * C::VE;   // as stage_coord: the same columns in every pass
    // LayerNorm statistics of the finished rows (as stored: TZ), two passes in fp32.  In the
    // read-back layout a row's 32 columns of one block sit in LPM neighbouring lanes.
    float mean[C::NPASS], rstd[C::NPASS];
#pragma unroll
    for (int ps = 0; ps < C::NPASS; ++ps) {
      float sum = 0.0f;
#pragma unroll
      for (int ob = 0; ob < NOB; ++ob)
#pragma unroll
        for (int e = 0; e < C::VE; ++e) sum += to_f32(done[0][ob][ps][e]);
      sum = group_sum<C::LPM>(sum);
      mean[ps] = sum * (1.0f / kCx);
      float q = 0.0f;
#pragma unroll
      for (int ob = 0; ob < NOB; ++ob)
#pragma unroll
        for (int e = 0; e < C::VE; ++e) {
          const float d = to_f32(done[0][ob][ps][e]) - mean[ps];
          q += d * d;
        }
      q = group_sum<C::LPM>(q);
      rstd[ps] = rsqrtf(q * (1.0f / kCx) + pb.eps);
    }
    // per wave: 32 rows x 64 normalised columns in T, behind all waves' staging tiles (other
    // waves may still be storing their rows)
    static_assert(NW * 32 * (C::PITCH * sizeof(TZ) + kPitchN * sizeof(T)) <=
                      sizeof(u32x4_t) * (NBUF - 1) * kTrFrags * PIECES * kWave,
                  "staging tiles and normalised tiles fit the chunk buffers");
    T* stn = reinterpret_cast<T*>(reinterpret_cast<TZ*>(&lds_w[0][0][0][0]) + NW * (32 * C::PITCH)) +
             wave * (32 * kPitchN);
    f32x16 accb;
#pragma unroll
    for (int r = 0; r < 16; ++r) accb[r] = 0.0f;
    // every wave's share of the bias weight has landed (and this wave's row stores are out)
    ring_barrier<0>();
#pragma unroll
    for (int hb = 0; hb < NOB / 2; ++hb) {   // 64 columns at a time
      wave_lds_sync();
#pragma unroll
      for (int o2 = 0; o2 < 2; ++o2)
#pragma unroll
        for (int ps = 0; ps < C::NPASS; ++ps) {
          int mj, m0;
          stage_coord<TZ>(ps, lane_e, mj, m0);
          const int ob = 2 * hb + o2;
#pragma unroll
          for (int e4 = 0; e4 < C::VE; e4 += 4) {
            const f32x4 gm = *reinterpret_cast<const f32x4*>(&lds_pba[0][ob * 32 + m0c + e4]);
            const f32x4 bt = *reinterpret_cast<const f32x4*>(&lds_pba[1][ob * 32 + m0c + e4]);
            f32x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e)
              o[e] = (to_f32(done[0][ob][ps][e4 + e]) - mean[ps]) * rstd[ps] * gm[e] + bt[e];
            *reinterpret_cast<bf16x4*>(stn + mj * kPitchN + 32 * o2 + m0 + e4) = from_f32<T>(o);   // 8 bytes
          }
        }
      wave_lds_sync();
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const u32x2* src = reinterpret_cast<const u32x2*>(stn + n * kPitchN + 16 * u + 8 * g);
        u32x2 h2[2] = {src[0], src[1]};
        mma32(accb, lds_pbw[4 * hb + u][lane_e], *reinterpret_cast<const V8*>(h2));   // lane_e <-> row, register <-> head
      }
    }
    const int64_t pr = row_at(n);
    if (pr >= 0) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int head = acc_row(r, g);
        if (head < pb.heads) {
          if (pb.out_f32) ((float*)pb.out)[(int64_t)head * n_rows + pr] = accb[r];
          else ((T*)pb.out)[(int64_t)head * n_rows + pr] = from_f32<T>(accb[r]);
        }
      }
    }
  }
}

template <typename T, int KS>
static int transition_pack_ks(const void* w_a, const void* w_b, const void* w_o, void* packed,
                              int n_factor, hipStream_t stream) {
  const int n_hidden = 16 * KS * n_factor;
  const int total = (n_hidden / 32) * TrCfg<T, KS>::FRAGS * kWave;
  if (total == 0) return 0;
  transition_pack_kernel<T, KS><<<dim3((total + 255) / 256), dim3(256), 0, stream>>>(
      (const T*)w_a, (const T*)w_b, (const T*)w_o, (T*)packed, n_hidden);
  return 0;
}

template <typename T>
int transition_pack(const void* w_a, const void* w_b, const void* w_o, void* packed, int c,
                    int n_factor, hipStream_t stream) {
  if (c == 64) return transition_pack_ks<T, 4>(w_a, w_b, w_o, packed, n_factor, stream);
  if (c == 256) return transition_pack_ks<T, 16>(w_a, w_b, w_o, packed, n_factor, stream);
  return transition_pack_ks<T, 8>(w_a, w_b, w_o, packed, n_factor, stream);
}

template <typename T, int KS, typename TZ>
static int transition_fwd_ks(const void* x, const void* ln_w, const void* ln_b, const void* packed,
                             void* out, int64_t rows, int n_factor, int add_residual, float eps,
                             hipStream_t stream) {
  const int64_t rows_per_block = TrCfg<T, KS>::NW * TrCfg<T, KS>::RB * 32;
  const int64_t blocks = (rows + rows_per_block - 1) / rows_per_block;
  transition_fused_kernel<T, KS, TZ, false><<<dim3((unsigned)blocks), dim3(TrCfg<T, KS>::NW * 64), 0, stream>>>(
      (const TZ*)x, (const T*)ln_w, (const T*)ln_b, (const T*)packed, (TZ*)out, rows,
      16 * KS * n_factor / 32, add_residual, eps, PairBiasArgs{}, AttnOutArgs{});
  return 0;
}

template <typename T, typename TZ>
int transition_pair_bias_fwd(const void* x, const void* ln_w, const void* ln_b, const void* packed,
                             void* out, int64_t rows, int n_factor, int add_residual, float eps,
                             const void* pb_ln_w, const void* pb_ln_b, const void* pb_w,
                             void* bias, int heads, int bias_f32, float pb_eps,
                             hipStream_t stream) {
  if (rows == 0) return 0;
  if constexpr (sizeof(T) == 2) {
    constexpr int KS = 8;
    static_assert(TrCfg<T, KS>::RB == 1, "the pair-bias epilogue handles one row block per wave");
    const int64_t rows_per_block = TrCfg<T, KS>::NW * 32;
    const int64_t blocks = (rows + rows_per_block - 1) / rows_per_block;
    const PairBiasArgs pb = {pb_ln_w, pb_ln_b, pb_w, bias, heads, bias_f32, pb_eps};
    transition_fused_kernel<T, KS, TZ, true><<<dim3((unsigned)blocks), dim3(TrCfg<T, KS>::NW * 64), 0, stream>>>(
        (const TZ*)x, (const T*)ln_w, (const T*)ln_b, (const T*)packed, (TZ*)out, rows,
        16 * KS * n_factor / 32, add_residual, eps, pb, AttnOutArgs{});
    return 0;
  } else {
    return 1;   // 16-bit arithmetic only (the caller checks)
  }
}

// The 64 fragments of the attention stage's W_g and W_o, in the order the prologue reads them
// (see AttnOutArgs), padded to kAoChunks whole chunks.
template <typename T>
__global__ void attn_out_pack_kernel(const T* __restrict__ w_g, const T* __restrict__ w_o,
                                     T* __restrict__ packed) {
  constexpr int kFrags = kAoChunks * TrCfg<T, 8>::FRAGS;
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= kFrags * kWave) return;
  const int lane = idx & 63, f = idx >> 6;
  const int m = lane & 31, g = lane >> 5;
  typename Vec8<T>::type v;
#pragma unroll
  for (int t = 0; t < 8; ++t) v[t] = (T)0.0f;
  if (f < 64) {
    const T* w = f < 32 ? w_g : w_o;
    const int cb = (f & 31) >> 3, kk = f & 7;
    const int row = 32 * cb + 16 * (m >> 4) + 8 * ((m >> 2) & 1) + 4 * ((m >> 3) & 1) + (m & 3);
    v = load8<T>(w + (int64_t)row * 128 + 16 * kk + 8 * g);
  }
  store8<T>(packed + (int64_t)idx * 8, v);
}

int64_t triattn_output_transition_packed_elems(int n_factor) {
  return (int64_t)kAoChunks * 24 * kFragElems + (int64_t)3 * n_factor * 128 * 128;
}

template <typename T>
int triattn_output_transition_pack(const void* w_g, const void* w_o, const void* w_a,
                                   const void* w_b, const void* w_to, void* packed, int n_factor,
                                   hipStream_t stream) {
  if constexpr (sizeof(T) == 2) {
    constexpr int total = kAoChunks * TrCfg<T, 8>::FRAGS * kWave;
    attn_out_pack_kernel<T><<<dim3((total + 255) / 256), dim3(256), 0, stream>>>(
        (const T*)w_g, (const T*)w_o, (T*)packed);
    return transition_pack_ks<T, 8>(w_a, w_b, w_to, (T*)packed + (int64_t)kAoChunks * 24 * kFragElems,
                                    n_factor, stream);
  } else {
    return 1;
  }
}

template <typename T, typename TZ>
int triattn_output_transition_fwd(const void* o, const void* z, const void* att_ln_w,
                                  const void* att_ln_b, const void* packed, const void* ln_w,
                                  const void* ln_b, void* out, int n, int transposed, int n_factor,
                                  float att_eps, float eps, const void* pb_ln_w, const void* pb_ln_b,
                                  const void* pb_w, void* bias, int heads, int bias_f32, float pb_eps,
                                  hipStream_t stream) {
  if (n == 0) return 0;
  if constexpr (sizeof(T) == 2) {
    constexpr int KS = 8;
    const int64_t rows = (int64_t)n * n;
    const int64_t rows_per_block = TrCfg<T, KS>::NW * 32;
    const int64_t blocks = (rows + rows_per_block - 1) / rows_per_block;
    AttnOutArgs ao = {};
    ao.o = o;
    ao.gamma = att_ln_w;
    ao.beta = att_ln_b;
    ao.omap.n_inner = n;
    ao.omap.stride_outer = transposed ? 32 : (int64_t)n * 32;
    ao.omap.stride_inner = transposed ? (int64_t)n * 32 : 32;
    ao.eps = att_eps;
    const int n_chunks = 16 * KS * n_factor / 32;
    if (pb_w) {
      const PairBiasArgs pb = {pb_ln_w, pb_ln_b, pb_w, bias, heads, bias_f32, pb_eps};
      transition_fused_kernel<T, KS, TZ, true, true><<<dim3((unsigned)blocks), dim3(TrCfg<T, KS>::NW * 64), 0, stream>>>(
          (const TZ*)z, (const T*)ln_w, (const T*)ln_b, (const T*)packed, (TZ*)out, rows, n_chunks, 1, eps,
          pb, ao);
    } else {
      transition_fused_kernel<T, KS, TZ, false, true><<<dim3((unsigned)blocks), dim3(TrCfg<T, KS>::NW * 64), 0, stream>>>(
          (const TZ*)z, (const T*)ln_w, (const T*)ln_b, (const T*)packed, (TZ*)out, rows, n_chunks, 1, eps,
          PairBiasArgs{}, ao);
    }
    return 0;
  } else {
    return 1;
  }
}

template <typename T, typename TZ>
int transition_fwd(const void* x, const void* ln_w, const void* ln_b, const void* packed,
                   void* out, int64_t rows, int c, int n_factor, int add_residual, float eps,
                   hipStream_t stream) {
  if (rows == 0) return 0;
  if (c == 64)
    return transition_fwd_ks<T, 4, TZ>(x, ln_w, ln_b, packed, out, rows, n_factor, add_residual, eps,
                                   stream);
  if (c == 256) {
    // 16-bit arithmetic only: an fp32 chunk of weights (96 KB) leaves no room for a ring in LDS
    if constexpr (sizeof(T) == 2)
      return transition_fwd_ks<T, 16, TZ>(x, ln_w, ln_b, packed, out, rows, n_factor, add_residual,
                                      eps, stream);
    else
      return -1;
  }
  return transition_fwd_ks<T, 8, TZ>(x, ln_w, ln_b, packed, out, rows, n_factor, add_residual, eps,
                                 stream);
}

template int triattn_output_transition_pack<bf16_t>(const void*, const void*, const void*,
                                                    const void*, const void*, void*, int,
                                                    hipStream_t);
#define PTX_INSTANTIATE_AOT(TZ)                                                                    \
  template int triattn_output_transition_fwd<bf16_t, TZ>(                                          \
      const void*, const void*, const void*, const void*, const void*, const void*, const void*,   \
      void*, int, int, int, float, float, const void*, const void*, const void*, void*, int, int,  \
      float, hipStream_t);
PTX_INSTANTIATE_AOT(bf16_t)
PTX_INSTANTIATE_AOT(float)
#undef PTX_INSTANTIATE_AOT
template int transition_pack<float>(const void*, const void*, const void*, void*, int, int,
                                    hipStream_t);
template int transition_pack<bf16_t>(const void*, const void*, const void*, void*, int, int,
                                     hipStream_t);
template int transition_fwd<float, float>(const void*, const void*, const void*, const void*,
                                          void*, int64_t, int, int, int, float, hipStream_t);
template int transition_fwd<bf16_t, bf16_t>(const void*, const void*, const void*, const void*,
                                            void*, int64_t, int, int, int, float, hipStream_t);
template int transition_fwd<bf16_t, float>(const void*, const void*, const void*, const void*,
                                           void*, int64_t, int, int, int, float, hipStream_t);
template int transition_pair_bias_fwd<bf16_t, bf16_t>(const void*, const void*, const void*,
                                                      const void*, void*, int64_t, int, int, float,
                                                      const void*, const void*, const void*, void*,
                                                      int, int, float, hipStream_t);
template int transition_pair_bias_fwd<bf16_t, float>(const void*, const void*, const void*,
                                                     const void*, void*, int64_t, int, int, float,
                                                     const void*, const void*, const void*, void*,
                                                     int, int, float, hipStream_t);

}  // namespace ptx
