// Row-tile projections with K = c_z (64, 128 or 256): every pair-tensor row (one (i,j)
// position) is normalised in registers and multiplied by small weight matrices on MFMA;
// gates, masks and residual adds are applied to the accumulators, and results leave through
// an LDS transpose as 16-byte, fully coalesced stores.
//
// A wave owns RB blocks of 32 rows.  A row block lives in registers as KS = c_z / 16
// operand fragments (16-deep K steps, see common.h): lane l holds row l%32,
// channels 16*kk + 8*(l/32) .. +7.  The same registers serve as the B operand
// (result: lane <-> row, register <-> output column; used for row-major
// outputs) or as the A operand (lane <-> output channel, register <-> row; used
// for channel-major outputs).  Either way a 32 x 32 result tile sits in the
// wave as "lane = major index, 4 consecutive minors per register quad", is
// written to a per-wave LDS tile [major][minor] with 8-byte stores and read
// back as vectors of consecutive minors, which is exactly the global layout.
//
// Weights sit in LDS already permuted into fragment order ([fragment][lane] ->
// conflict-free 16-byte reads), in chunks of two 32-column tiles.  Three ways to get them
// there (InCfg below): bf16 with c_z <= 128 loads every chunk of the launch once per
// workgroup (one 8-wave workgroup per CU, whose waves then walk over row tiles with no
// workgroup barrier); bf16 with c_z = 256 and the pair-bias projection stream the chunks
// through a two-slot ring of direct-to-LDS loads; fp32 stages one chunk at a time through
// registers.  All loads and stores in the hot loops are unconditional (indices are clamped,
// lanes without a valid row store to a sink) so the MFMA loops carry no branches and the
// number of memory operations per chunk is a constant the hand-placed waits can count on.
#include "common.h"
#include "kernels.h"
#include "rowtile.h"
#include <algorithm>
#include <type_traits>

namespace ptx {

// ---------------------------------------------------------------------------
// rowgemm_in: LayerNorm -> chunks of two 32-column weight tiles -> epilogue.
// ---------------------------------------------------------------------------
struct RowGemmInParams {
  const void* x;        // pair tensor, rows addressed through xmap
  RowMap xmap;
  int64_t n_rows;
  const void* gamma;
  const void* beta;
  float eps;
  const void* w[5];     // mode-specific weight matrices, row-major [*][128]
  void* out[5];         // mode-specific outputs
  const void* mask;     // TRIMUL_IN: per-row mask through mmap, or null
  RowMap mmap;
  int n;                // tokens (n_rows = n*n for pair tensors)
  int pitch;            // row pitch of a, b (TRIMUL_IN) / v^T, triangle bias (TRIATTN_IN)
  int aux;              // TRIATTN_IN: heads; PAIRBIAS: heads | out_f32 << 8; TRIMUL_IN: walk back to front
  float q_scale;        // TRIATTN_IN: log2(e)/sqrt(d)
  // TRIMUL_OUT only
  const void* x2;       // channel-major triangle product [128][n_rows]
  const void* gamma2;
  const void* beta2;
  int add_residual;
};

enum RowGemmInMode { kTriMulIn = 0, kTriAttnIn = 1, kPairBias = 3, kTriMulOut = 4 };

// Where the 16-byte stores of lanes without a valid destination row go (lane l writes bytes
// 16*l .. +15).  Keeping every store unconditional makes the number of stores a wave issues
// per chunk a constant, which the weight ring below counts on.
static __device__ __attribute__((aligned(16))) uint32_t g_store_sink[kWave * 4];

// Widths.  KS = K steps of a pair-tensor row (c_z / 16: 4, 8 or 16).  The hidden widths
// (c_hidden_mul, heads * 32) are 128 for c_z <= 128 and c_z beyond ("hidden_scale_up" of the
// reference, pairformer.py:76-78): SL = hidden / 16 K steps, which is also the number of
// fragment slots a weight tile takes in LDS.
template <int KS> struct Widths {
  static constexpr int SL = KS > 8 ? KS : 8;
  static constexpr int HIDDEN = 16 * SL;
  static constexpr int HEADS = HIDDEN / 32;
};

// Weight matrix, its row count, first row, row length and K steps for tile `t` (0/1) of
// chunk `ch`.
template <typename T, int MODE, int KS>
__device__ __forceinline__ void chunk_tile(const RowGemmInParams& p, int ch, int t, const T*& w,
                                           int& n_out, int& col0, int& ldw, int& ksteps) {
  typedef Widths<KS> W;
  ldw = 16 * KS;
  ksteps = KS;
  if (MODE == kTriMulIn) {            // w: ap, ag, bp, bg ; tile0 = projection, tile1 = gate
    constexpr int CPM = W::HIDDEN / 32;   // chunks per operand
    w = (const T*)p.w[(ch / CPM) * 2 + t];
    n_out = W::HIDDEN;
    col0 = (ch % CPM) * 32;
  } else if (MODE == kTriAttnIn) {    // w: q, k, g, v, bias
    constexpr int CPM = W::HIDDEN / 64;   // chunks (of two heads) per matrix
    const int which = ch / CPM;
    w = (const T*)p.w[which];
    n_out = which == 4 ? p.aux : W::HIDDEN;
    col0 = which == 4 ? 0 : ((ch % CPM) * 2 + t) * 32;
  } else if (MODE == kPairBias) {
    w = (const T*)p.w[0];
    n_out = p.aux & 0xff;
    col0 = 0;
  } else {                            // kTriMulOut: w: z [c_z][hidden], g [c_z][c_z]
    w = (const T*)p.w[t];
    n_out = 16 * KS;
    col0 = ch * 32;
    if (t == 0) {
      ldw = W::HIDDEN;
      ksteps = W::SL;
    }
  }
}

// Geometry of one instantiation.  bf16 (all but the single-chunk pair bias) runs "resident":
// one workgroup of 8 waves per CU loads ALL weight fragments of the launch into LDS once, and
// its waves then walk over row tiles on their own, with no workgroup barrier and no weight
// traffic in the loop.  (With the weights re-read per workgroup, a 256-row workgroup pulls as
// many bytes of weights through the L2 as it moves pair-tensor data, and every wave's wait
// for its share of them also waits for the stores it issued before.)  fp32 weights are twice
// the size and do not fit: that path stages one chunk at a time through registers.
template <typename T, int MODE, int KS> struct InCfg {
  static constexpr int SL = Widths<KS>::SL;
  // (256-channel rows: the weights do not fit either; bf16 then takes the staged path too)
  static constexpr bool RES = sizeof(T) == 2 && MODE != kPairBias && KS <= 8;
  // waves per workgroup: 8 where the weights are resident, and in the attention projection on
  // 16-bit rows of 256 channels, whose ring of two 32 KB chunk buffers leaves room for one
  // workgroup per compute unit only: with four waves that was one wave per SIMD and a pass of
  // all weights through the L2 per 128 rows (875 -> 588 us per launch at N = 768).  The
  // triangle multiplication's projection of that width needs more than the 256 registers two
  // waves per SIMD leave it (with eight waves 536 bytes of spills, 597 -> 696 us): four waves.
  static constexpr int NW = (RES || (sizeof(T) == 2 && KS > 8 && MODE == kTriAttnIn)) ? 8 : 4;
  // chunks of two 32-column weight tiles: {a,b} x hidden/32 channel blocks | q,k,g,v: one per
  // two heads, bias: 1 | the pair bias | c_z / 32 output column blocks
  static constexpr int NCH = MODE == kTriMulIn    ? 2 * (SL / 2)
                             : MODE == kTriAttnIn ? 4 * (SL / 4) + 1
                             : MODE == kPairBias  ? 1
                                                  : KS / 2;
  // weight fragments held in LDS (2*SL per chunk; the resident triangle bias is one tile)
  static constexpr int NFRAG = RES ? (MODE == kTriAttnIn ? (NCH - 1) * 2 * SL + SL : NCH * 2 * SL)
                                   : Cfg<T>::NBUF * 2 * SL;
  static constexpr int FPW = 2 * SL / NW;  // staged path: fragments per wave and chunk
  static constexpr int MIN_WG = (RES || KS > 8) ? 1 : 2;
};

// VEC: n is a multiple of the 16-byte vector length, so channel-major vectors stay inside one
// plane row (the element-wise fallback for other n is a kernel of its own: compiled into the
// same one, its code and its registers weigh on the path every production shape takes).
// TZ: storage type of the pair tensor (p.x and, for kTriMulOut, the output).  TZ = float with
// T = bf16 is the fp32 residual stream of the reference's autocast inference: rows are read
// as fp32, normalised in fp32 and rounded to T for the matrix products; kTriMulOut adds its
// T-rounded update to the fp32 row.
template <typename T, int RB, int MODE, int KS, bool VEC, typename TZ = T>
__global__ __launch_bounds__((InCfg<T, MODE, KS>::NW * 64), (InCfg<T, MODE, KS>::MIN_WG)) void
rowgemm_in_kernel(RowGemmInParams p) {
  typedef typename Vec8<T>::type V8;
  typedef typename VecE<T>::type VE_t;
  typedef Cfg<T> C;
  typedef Cfg<TZ> CZ;
  typedef InCfg<T, MODE, KS> IC;
  constexpr bool MIXED = !std::is_same<T, TZ>::value;
  static_assert(!MIXED || (sizeof(T) == 2 && sizeof(TZ) == 4),
                "mixed storage: bf16 arithmetic on fp32 rows");
  // kTriMulOut with bf16 arithmetic on rows of at most 128 channels keeps the raw rows (as
  // fp32) in registers for the residual add instead of a copy in LDS (see below)
  constexpr bool kRegRes = MODE == kTriMulOut && sizeof(T) == 2 && KS <= 8;
  constexpr bool RES = IC::RES;
  constexpr int NW = IC::NW, SL = IC::SL, FPW = IC::FPW;
  // K steps by which the weight fragments' LDS reads run ahead of their products (see the chunk
  // body): one in the attention projection on rows of 128 channels, which has the registers
  // (168 -> 164 us per launch; in the triangle-multiplication kernels, at the register limit,
  // the ring's eight registers turn into spills: 161 -> 164 us)
  constexpr int kWeightPrefetch = (RES && MODE == kTriAttnIn && RB == 1) ? 1 : 0;
  __shared__ V8 lds_w[IC::NFRAG][kWave];
  // Staging tiles per wave.  Resident: one (LDS is full of weights).  Otherwise one per
  // 32 x 32 result tile of a chunk: all tiles of a chunk are written, then all are read back
  // and stored, so that a chunk pays one LDS round trip, not one per tile.
  constexpr int NST = (RES || MODE == kTriMulOut) ? 1 : 2 * RB;
  // kTriMulOut: the raw z rows of this wave, kept for the residual add (re-reading them from
  // HBM at the end costs a full extra pass: by then they have left the L2)
  constexpr int kCz = 16 * KS;   // channels of a pair-tensor row
  constexpr int kResPitch = kCz + 16 / (int)sizeof(T);
  // kGlobRes (fp32 rows of 256 channels): no copy of the raw rows is kept - an fp32 copy in LDS
  // would take 133 KB next to the weight ring, in registers 128 of them; each chunk reads the
  // residual of its own 32 columns from memory again before it stores them
  constexpr bool kGlobRes = MODE == kTriMulOut && !kRegRes && MIXED;
  constexpr bool kLdsRes = MODE == kTriMulOut && !kRegRes && !MIXED;
  __shared__ __attribute__((aligned(16))) T lds_res[kLdsRes ? NW : 1][kLdsRes ? RB * 32 : 1][kLdsRes ? kResPitch : 8];
  // kRegRes: staging tile of the fp32 output rows (one 32 x 32 tile per wave)
  __shared__ __attribute__((aligned(16))) TZ lds_stage_z[kRegRes ? NW : 1][kRegRes ? 32 * CZ::PITCH : 4];
  __shared__ __attribute__((aligned(16))) T lds_stage[NW][NST][32 * C::PITCH];
  __shared__ __attribute__((aligned(16))) float lds_mask[MODE == kTriMulIn ? NW : 1][RB * 32];
  // LayerNorm weight and bias (absent: 1 and 0) as fp32, converted once per workgroup: read
  // from global memory they cost every row tile as many load instructions as the tile's own
  // rows and, in 16 bits, a conversion per value and tile.  Only where the fp32 copies fit the
  // register budget: in the triangle-multiplication kernels the wider operands spill more
  // than the conversions cost, and those keep reading the parameters from global memory.
  constexpr bool kLdsAffine = MODE == kTriAttnIn || MODE == kPairBias;
  __shared__ __attribute__((aligned(16))) float lds_affine[2][kLdsAffine ? kCz : 1];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, g = lane >> 5;
  T* st = lds_stage[wave][0];
  auto stile = [&](int k) { return lds_stage[wave][k]; };
  constexpr bool vec_ok = VEC;
  T* const sink = reinterpret_cast<T*>(g_store_sink) + lane * C::VE;
  constexpr int nch = IC::NCH;

  // kRegRes: both LayerNorms' parameters as fp32 in LDS.  Read from global memory, all 32
  // parameter loads of a tile are issued (and converted) ahead of the rows, 128 registers
  // that this instantiation does not have.
  __shared__ __attribute__((aligned(16))) float lds_affine2[4][kRegRes ? 16 * SL : 1];
  if constexpr (kRegRes) {
    for (int c = threadIdx.x; c < 16 * SL; c += NW * kWave) {
      if (c < kCz) {
        lds_affine2[0][c] = p.gamma ? to_f32(((const T*)p.gamma)[c]) : 1.0f;
        lds_affine2[1][c] = p.beta ? to_f32(((const T*)p.beta)[c]) : 0.0f;
      }
      lds_affine2[2][c] = p.gamma2 ? to_f32(((const T*)p.gamma2)[c]) : 1.0f;
      lds_affine2[3][c] = p.beta2 ? to_f32(((const T*)p.beta2)[c]) : 0.0f;
    }
    __syncthreads();
  }
  if constexpr (kLdsAffine) {
    for (int c = threadIdx.x; c < kCz; c += NW * kWave) {
      lds_affine[0][c] = p.gamma ? to_f32(((const T*)p.gamma)[c]) : 1.0f;
      lds_affine[1][c] = p.beta ? to_f32(((const T*)p.beta)[c]) : 0.0f;
    }
    __syncthreads();
  }

  // Work units ("wave tiles").  kTriMulIn works on 2-D patches of the pair tensor instead of
  // runs of logical rows: four waves cover 16*RB outer indices x 8 inner indices, a row block
  // 4 x 8 (MFMA row r <-> outer pi0 + 4*rb + r/8, inner pk0 + r%8), which makes a row block's
  // 32 values of one channel 64 contiguous bytes of the contraction's fragment-ordered
  // operands.  The other modes take RB*32 consecutive logical rows.
  const uint32_t n_kb = (uint32_t)p.pitch >> 3;   // kTriMulIn: the K padding is written too (as zeros)
  int64_t n_tiles;
  if (MODE == kTriMulIn) n_tiles = (int64_t)((p.n + 16 * RB - 1) / (16 * RB)) * n_kb * 4;
  else n_tiles = (p.n_rows + RB * 32 - 1) / (RB * 32);
  // Resident: waves 0-3 of all workgroups come first in the walk, then waves 4-7, so that a
  // last round that covers half the machine's waves still gives every CU (and SIMD) its share.
  int64_t tile = RES ? (int64_t)(wave >> 2) * (gridDim.x * 4) + blockIdx.x * 4 + (wave & 3)
                     : (int64_t)blockIdx.x * NW + wave;
  const int64_t tile_step = (int64_t)gridDim.x * NW;

  // Weight fragment f = 2*SL * chunk + SL * tile + K step, from global memory straight into its
  // LDS slot (bf16).  These loads are invisible to the compiler's wait-count bookkeeping and
  // are waited for by hand.
  auto dma_frag = [&](int f_src, int f_dst) {
    const T* w;
    int n_out, col0, ldw, ksteps;
    const int kk = f_src % SL;
    chunk_tile<T, MODE, KS>(p, f_src / (2 * SL), (f_src / SL) & 1, w, n_out, col0, ldw, ksteps);
    if (kk >= ksteps) return;   // narrow rows: the slot stays unused
    // kRegRes: output column of MFMA row m is permuted so that the accumulator registers of
    // a lane cover the same 8-channel runs as its fragments of the z row: register r of
    // half-wave g <-> column 16*(r>>3) + 8*g + (r&7) of the chunk's 32
    int m = lane & 31;
    if constexpr (kRegRes) m = 16 * (m >> 4) + 8 * ((m >> 2) & 1) + 4 * ((m >> 3) & 1) + (m & 3);
    const int col = min(col0 + m, n_out - 1);   // as load_wfrag
    load_to_lds16(w + (int64_t)col * ldw + kk * 16 + 8 * (lane >> 5),
                  lds_address(&lds_w[f_dst][0]));
  };
  // bf16 without resident weights (the pair bias' single chunk; rows of 256 channels): a ring
  // of two chunk buffers filled by the same direct-to-LDS loads, one chunk ahead.  The wait
  // for a chunk counts the stores issued after its loads (see the end of the chunk loop): a
  // register-staged prefetch would make the compiler drain every store before each chunk.
  constexpr bool kDma = sizeof(T) == 2 && !RES;
  // kPrefetch: the raw rows of a tile are requested one tile ahead, so that their way from
  // memory lies under the previous tile's chunk loop.
  constexpr bool kPrefetch = RES && MODE == kTriAttnIn && RB == 1;
  typename Vec8<TZ>::type raw[kPrefetch ? KS : 1];
  auto issue_rows = [&](int64_t t) {
    if constexpr (kPrefetch) {
      const int64_t wt = n_tiles - 1 - t;          // back to front, as below
      int64_t pr = wt * 32 + (lane & 31);
      pr = pr < p.n_rows ? pr : p.n_rows - 1;
      const TZ* rp = (const TZ*)p.x + p.xmap(pr) + 8 * (lane >> 5);
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) raw[kk] = load8<TZ>(rp + 16 * kk);
    }
  };
  // (the first tile's rows go first: their LayerNorm then runs while the weights arrive)
  if (kPrefetch) issue_rows(tile < n_tiles ? tile : n_tiles - 1);
  RowFrags<T, RB, KS> xf;   // the tile's normalised rows (kPrefetch: carried from tile to tile)
  // (A wait for the resident weights deferred to the first tile's first chunk, so that they
  // would travel under that tile's row loads, was tried: the conditional barrier inside the
  // tile loop cost the triangle-multiplication output 848 bytes of spills per lane.)
  if constexpr (RES) {
    for (int f = wave; f < IC::NFRAG; f += NW) dma_frag(f, f);
    ring_barrier<0>();
  } else if constexpr (kDma) {
#pragma unroll
    for (int j = 0; j < FPW; ++j) dma_frag(wave * FPW + j, wave * FPW + j);
    ring_barrier<0>();
  }

  // kPrefetch: a tile's rows are normalised at the END of the tile before it, in the iteration
  // that requested them.  The wait for them then stands in straight-line code (the chunk loop
  // of this instantiation is unrolled) behind a number of stores the compiler can count, and
  // leaves those in flight: memory operations of a wave complete in order, and for a wait at the
  // head of the next iteration the compiler has to assume that nothing was issued behind the
  // loads, which drained every store of the tile there (181 -> 170 us per launch at N = 768).
  auto normalize_prefetched = [&]() {
    if constexpr (kPrefetch) {
      f32x8 v[KS];
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) v[kk] = to_f32(raw[kk]);
      normalize_row<T, KS, float, false>(v, lds_affine[0], lds_affine[1], p.eps, lane >> 5, xf.f[0]);
    }
  };
  normalize_prefetched();

  // Staged path (fp32; bf16 rows of 256 channels): the next chunk's fragments are prefetched
  // into registers and stored to LDS
  V8 pre[FPW];
  auto fetch = [&](int ch) {
#pragma unroll
    for (int j = 0; j < FPW; ++j) {
      const int fid = wave * FPW + j;   // 2*SL fragments per chunk: tile = fid/SL, kk = fid%SL
      const T* w;
      int n_out, col0, ldw, ksteps;
      chunk_tile<T, MODE, KS>(p, ch, fid / SL, w, n_out, col0, ldw, ksteps);
      // (K steps beyond a narrow row re-read the last one: their slots are never used)
      pre[j] = load_wfrag<T>(w, ldw, n_out, col0, min(fid % SL, ksteps - 1) * 16, lane);
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int j = 0; j < FPW; ++j) lds_w[buf * 2 * SL + wave * FPW + j][lane] = pre[j];
  };

  while (true) {
    if (RES && tile >= n_tiles) break;
    // kTriMulIn (at the register limit): the lane index and what is derived from it are formed
    // again in every tile, from a copy the compiler cannot see through - carried across the
    // loop they were spilled (88 bytes per lane instead of 44, six registers instead of four
    // written back in every tile: the kernel's 1.08 times its algorithmic bytes written).
    int lane_s = threadIdx.x & 63;
    if constexpr (MODE == kTriMulIn) asm volatile("" : "+v"(lane_s));
    const int lane = lane_s;
    const int n = lane & 31, g = lane >> 5;
    T* const sink = reinterpret_cast<T*>(g_store_sink) + lane * C::VE;
    // The projections at the head of an update walk the pair tensor back to front.  The kernel
    // before them has just written it front to back, so its tail is what the 256 MB memory-side
    // cache still holds; read front to back, a tensor larger than that cache evicts its own
    // tail before reaching it.
    // (The outgoing triangle multiplication opens a block, behind the transition of the block
    // before, which itself walks back to front: that projection walks forward.)
    const bool backward = MODE == kTriAttnIn || (MODE == kTriMulIn && p.aux != 0);
    const int64_t wtile = (backward && tile < n_tiles) ? n_tiles - 1 - tile : tile;
    const int64_t row0 = wtile * (RB * 32);
    int pi0 = 0, pk0 = 0;
    if constexpr (MODE == kTriMulIn) {
      // Patches in the order of the memory rows they read: the outer index is the slow one for
      // the outgoing product (z[i][k]), the inner one for the incoming product (z[k][i]), whose
      // walk then runs through the pair tensor's rows back to front like the other projections'
      // instead of sweeping all rows once per strip of columns.
      const uint32_t vb = (uint32_t)(wtile >> 2);
      uint32_t ip, kb;
      if (p.aux != 0) {
        const uint32_t n_ip = (uint32_t)(p.n + 16 * RB - 1) / (16 * RB);
        kb = vb / n_ip;
        ip = vb - kb * n_ip;
      } else {
        ip = vb / n_kb;
        kb = vb - ip * n_kb;
      }
      pk0 = (int)kb * 8;
      pi0 = (int)ip * (16 * RB) + (int)(wtile & 3) * (4 * RB);
    }
    // (resident: made opaque per tile, or the affine parameters' loads and conversions are
    // hoisted out of the tile loop and held in registers)
    const T* gamma = (const T*)p.gamma;
    const T* beta = (const T*)p.beta;
    const T* gamma2 = (const T*)p.gamma2;
    const T* beta2 = (const T*)p.beta2;
    if constexpr (RES) asm volatile("" : "+s"(gamma), "+s"(beta), "+s"(gamma2), "+s"(beta2));

  // (the raw rows in their storage type: fp32 rows as fp32, bf16 rows as bf16 - half the registers)
  typename Vec8<TZ>::type zres[kRegRes ? RB : 1][kRegRes ? KS : 1];
  if constexpr (MODE == kTriMulIn) {
    int64_t off[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int i = min(pi0 + 4 * rb + (n >> 3), p.n - 1), k = min(pk0 + (n & 7), p.n - 1);
      off[rb] = (int64_t)i * p.xmap.stride_outer + (int64_t)k * p.xmap.stride_inner;
    }
    load_rows_at<T, RB, true>(xf, (const TZ*)p.x, off, gamma, beta, p.eps, lane);
  } else if constexpr (kRegRes) {
    // (the fp32 rows are requested further down, once the triangle product's rows are on
    // their way through the staging tile: both sets of raw rows at once do not fit the
    // registers)
  } else if constexpr (kGlobRes) {
    load_rows<T, RB, true>(xf, (const TZ*)p.x, p.xmap, row0, p.n_rows, gamma, beta, p.eps, lane);
  } else if constexpr (MODE == kTriMulOut) {
    RowFrags<T, RB, KS> zraw;
    load_rows<T, RB, false>(zraw, (const T*)p.x, p.xmap, row0, p.n_rows, (const T*)nullptr,
                            (const T*)nullptr, 0.0f, lane);
    wave_lds_sync();   // the previous tile's residual reads are done
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
      for (int kk = 0; kk < KS; ++kk)
        store8<T>(&lds_res[wave][rb * 32 + n][16 * kk + 8 * g], zraw.f[rb][kk]);
      normalize_raw<T>(zraw.f[rb], gamma, beta, p.eps, g, xf.f[rb]);
    }
  } else {
    if constexpr (kPrefetch) {
      // the next tile's rows, normalised at the end of this iteration
      // (no branch around the loads: with one, this instantiation spills.  A wave past its
      // last tile reads the rows every such wave reads, out of the L2.)
      const int64_t nt = tile + tile_step;
      issue_rows(nt < n_tiles ? nt : n_tiles - 1);
    } else if constexpr (kLdsAffine)
      load_rows<T, RB, true, KS, float, false>(xf, (const TZ*)p.x, p.xmap, row0, p.n_rows, lds_affine[0],
                                               lds_affine[1], p.eps, lane);
    else
      load_rows<T, RB, true>(xf, (const TZ*)p.x, p.xmap, row0, p.n_rows, gamma, beta, p.eps, lane);
  }

  // kTriMulOut: second fragment set = LayerNorm_out of the channel-major triangle product,
  // transposed through the staging tile 32 channels at a time.
  RowFrags<T, RB, SL> xf2;   // dead (and removed by the compiler) in the other modes
  if constexpr (MODE == kTriMulOut) {
    const T* x2 = (const T*)p.x2;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      f32x8 v[SL];
      // all channel groups (of 32) are requested at once: one memory round trip
      VE_t vec[SL / 2][C::NPASS];
#pragma unroll
      for (int cg = 0; cg < SL / 2; ++cg)
#pragma unroll
        for (int ps = 0; ps < C::NPASS; ++ps) {
          int chn, r0;
          stage_coord<T>(ps, lane, chn, r0);
          // (fp32 residual rows in registers: opaque per tile, or the eight plane offsets are
          // kept in registers across the tile loop, which has none to spare)
          if constexpr (kRegRes) asm volatile("" : "+v"(chn));
          const int64_t pr = row0 + rb * 32 + r0;
          const T* src = x2 + (int64_t)(32 * cg + chn) * p.n_rows;
          if constexpr (vec_ok) {
            const int64_t pc = pr + C::VE <= p.n_rows ? pr : 0;
            vec[cg][ps] = *reinterpret_cast<const VE_t*>(src + pc);
          } else {
#pragma unroll
            for (int e = 0; e < C::VE; ++e) {
              const int64_t pe = pr + e < p.n_rows ? pr + e : p.n_rows - 1;
              vec[cg][ps][e] = src[pe];
            }
          }
        }
#pragma unroll
      for (int cg = 0; cg < SL / 2; ++cg) {      // channels 32*cg .. +31
        wave_lds_sync();
#pragma unroll
        for (int ps = 0; ps < C::NPASS; ++ps) {
          int chn, r0;
          stage_coord<T>(ps, lane, chn, r0);
          stage_put_vec<T>(st, chn, r0, vec[cg][ps]);
        }
        wave_lds_sync();
        // lane (row n, half g) picks channels 16*kk + 8*g + t of this group
#pragma unroll
        for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
          for (int t = 0; t < 8; ++t)
            v[2 * cg + k2][t] = to_f32(st[(16 * k2 + 8 * g + t) * C::PITCH + n]);
      }
      if constexpr (kRegRes)
        normalize_row<T, SL, float, false>(v, lds_affine2[2], lds_affine2[3], p.eps, g, xf2.f[rb]);
      else
        normalize_row<T>(v, gamma2, beta2, p.eps, g, xf2.f[rb]);
      if constexpr (kRegRes) {
        // The raw fp32 rows stay in registers for the residual add: lane (row n, half g)
        // holds channels 16*kk + 8*g .. +7, which the permuted weight columns make the very
        // channels its accumulator registers stand for.  Requested only now (the row index
        // is made to depend on the last normalised fragment, which keeps the loads from
        // moving up): together with the fp32 copy of the triangle product's rows they do
        // not fit the registers.
        static_assert(RB == 1, "one row block per wave");
        int64_t pr = row0 + n;
        asm volatile("" : "+v"(pr) : "v"(xf2.f[rb][SL - 1]));
        pr = pr < p.n_rows ? pr : p.n_rows - 1;
        const TZ* rp = (const TZ*)p.x + p.xmap(pr) + 8 * g;
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) zres[rb][kk] = load8<TZ>(rp + 16 * kk);
        if constexpr (MIXED)
          normalize_row<T, KS, float, false>(zres[rb], lds_affine2[0], lds_affine2[1], p.eps, g, xf.f[rb]);
        else
          normalize_raw<T, KS, float, false>(zres[rb], lds_affine2[0], lds_affine2[1], p.eps, g, xf.f[rb]);
      }
    }
  }

  // TriMulIn: the 32 mask values of each row block, shared through LDS
  // (inner indices between n and the pitch get factor 0: the contraction relies on zeros there)
  if constexpr (MODE == kTriMulIn) {
    wave_lds_sync();   // the previous tile's mask reads are done
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int i = min(pi0 + 4 * rb + (n >> 3), p.n - 1), k = min(pk0 + (n & 7), p.n - 1);
      float mv = 1.0f;
      if (p.mask)
        mv = to_f32(((const T*)p.mask)[(int64_t)i * p.mmap.stride_outer +
                                       (int64_t)k * p.mmap.stride_inner]);
      if (pk0 + (n & 7) >= p.n) mv = 0.0f;
      if (g == 0) lds_mask[wave][rb * 32 + n] = mv;
    }
    wave_lds_sync();
  }

  // Row-major destinations (kTriAttnIn q/k/g, kTriMulOut out): the logical row this lane
  // stores in each read-back pass, or -1.
  int64_t rrow[RB][C::NPASS];
  int rm_i[RB][C::NPASS], rm_j[RB][C::NPASS];   // the same rows as (outer, inner) of the pair tensor
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int ps = 0; ps < C::NPASS; ++ps) {
      int mj, m0;
      stage_coord<T>(ps, lane, mj, m0);
      const int64_t pr = row0 + rb * 32 + mj;
      rrow[rb][ps] = pr < p.n_rows ? pr : -1;
      const uint32_t pc = (uint32_t)(pr < p.n_rows ? pr : 0);
      rm_i[rb][ps] = pc / (uint32_t)p.n;
      rm_j[rb][ps] = pc - rm_i[rb][ps] * (uint32_t)p.n;
    }
  // kRegRes: the rows this lane stores in the read-back passes of the fp32 staging tile
  int64_t rrow_z[kRegRes ? RB : 1][kRegRes ? CZ::NPASS : 1];
  if constexpr (kRegRes) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int ps = 0; ps < CZ::NPASS; ++ps) {
        int mj, m0;
        stage_coord<TZ>(ps, lane, mj, m0);
        const int64_t pr = row0 + rb * 32 + mj;
        rrow_z[rb][ps] = pr < p.n_rows ? pr : -1;
      }
  }
  // Channel-major destinations: the VE consecutive logical rows this lane stores (the same
  // in every read-back pass), as (outer, inner) of the pair tensor; all address divisions
  // happen here, once, outside the chunk loop.
  int cm_i[RB], cm_j[RB];
  bool cm_ok[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int64_t pr = row0 + rb * 32 + (lane % C::LPM) * C::VE;
    cm_ok[rb] = pr < p.n_rows;
    const uint32_t pc = (uint32_t)(cm_ok[rb] ? pr : 0);
    cm_i[rb] = pc / (uint32_t)p.n;
    cm_j[rb] = pc - cm_i[rb] * (uint32_t)p.n;
  }

  // Element offsets of this lane's vectors inside the fragment-ordered destinations, relative
  // to the head (K, V^T) or channel block (a, b) the chunk writes: the index arithmetic of
  // the layouts (common.h) runs once per tile here instead of once per store.  32 bits
  // suffice: a plane has n * pitch * 32 elements and the entry points bound n by 8192.
  uint32_t rel_k[RB][C::NPASS], rel_v[RB][C::NPASS], rel_b[RB][C::NPASS], rel_a[RB][C::NPASS];
  if constexpr (MODE == kTriAttnIn) {
    const int key_tiles = p.pitch >> 6, q_blocks = (p.n + 31) >> 5;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int ps = 0; ps < C::NPASS; ++ps) {
        int mj, m0;
        stage_coord<T>(ps, lane, mj, m0);   // K: major = key row, minor = d; V^T, bias: major = channel
        rel_k[rb][ps] = (uint32_t)attn_k_offset(0, rm_i[rb][ps], rm_j[rb][ps], m0, p.n, key_tiles);
        rel_v[rb][ps] = (uint32_t)attn_v_offset(0, cm_i[rb], cm_j[rb], mj, p.n, key_tiles);
        rel_b[rb][ps] = (uint32_t)attn_b_offset(mj, cm_i[rb], cm_j[rb], q_blocks, key_tiles);
      }
  }
  if constexpr (MODE == kTriMulIn) {
    const int n_rb = (p.n + 31) >> 5, n_ks = p.pitch >> 4;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int ps = 0; ps < C::NPASS; ++ps) {
        int chn, r0;
        stage_coord<T>(ps, lane, chn, r0);
        const int i = pi0 + 4 * rb + (r0 >> 3);
        rel_a[rb][ps] = (uint32_t)(trimul_frag_offset(chn, i >> 5, pk0 >> 4, n_rb, n_ks) +
                                   ((pk0 >> 3) & 1) * 256 + (i & 31) * 8 + (r0 & 7));
      }
  }

  if constexpr (!RES && !kDma) {
    fetch(0);
    stash(0);
    __syncthreads();
  }

  // Row-major store of the staged tile (major = row, minor = 32 output columns at col0).
  // Lanes without a valid row store to the sink: the store count stays fixed.
  auto store_row_major = [&](const T* stg, T* outp, int64_t ld, int col0, int rb, const VE_t* resv) {
#pragma unroll
    for (int ps = 0; ps < C::NPASS; ++ps) {
      int mj, m0;
      stage_coord<T>(ps, lane, mj, m0);
      const int64_t off = rrow[rb][ps] * ld + col0 + m0;
      VE_t v = stage_get_vec<T>(stg, mj, m0);
      if (resv) v = add_vec<T>(v, resv[ps]);
      *reinterpret_cast<VE_t*>(rrow[rb][ps] >= 0 ? outp + off : sink) = v;
    }
  };
  // (not unrolled: unrolled, the compiler hoists every chunk's loads to the top and spills them)
  // `part`: 0 = the whole chunk; 1 = its matrix products only (into acc); 2 = its epilogue only
  // (from acc).  (Issuing the products of chunk ch + 1 ahead of the epilogue of chunk ch, over
  // two accumulator sets, was measured in the attention projection: 171 against 170 us - the
  // other wave of the SIMD already fills those gaps.)
  auto chunk_body = [&](int ch, f32x16 (&acc)[RB][2], int part) {
    // kTriAttnIn without a gate output (the gate is then formed by the output kernel): the
    // gate's chunks are passed over (resident weights only: the rings count their loads)
    if constexpr (MODE == kTriAttnIn && RES) {
      if (!p.out[2] && ch / (Widths<KS>::HIDDEN / 64) == 2) return;
    }
    const int buf = (!RES && C::NBUF == 2) ? (ch & 1) : 0;
    if constexpr (kDma) {
      // the other buffer was last read in the previous chunk, which every wave has left
      if (ch + 1 < nch) {
#pragma unroll
        for (int j = 0; j < FPW; ++j)
          dma_frag((ch + 1) * 2 * SL + wave * FPW + j, (buf ^ 1) * 2 * SL + wave * FPW + j);
      }
    } else if constexpr (!RES) {
      fetch(min(ch + 1, nch - 1));   // unconditional: static load count
    }
    // first fragment of this chunk's two weight tiles (the resident triangle bias is one tile)
    const int wf0 = RES ? ch * 2 * SL : buf * 2 * SL;
    const int wf1 = wf0 + ((RES && MODE == kTriAttnIn && ch == nch - 1) ? 0 : SL);
    // kTriMulOut: the residual vectors of this chunk's columns, from the wave's LDS copy of z
    VE_t resv[RB][C::NPASS];
    if constexpr (kLdsRes) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int ps = 0; ps < C::NPASS; ++ps) {
          int mj, m0;
          stage_coord<T>(ps, lane, mj, m0);
          resv[rb][ps] = *reinterpret_cast<const VE_t*>(&lds_res[wave][rb * 32 + mj][ch * 32 + m0]);
        }
    }
    // kGlobRes: the fp32 residual of this chunk's columns, read back from the pair tensor (the
    // same addresses this lane stores to below; other chunks touch other columns, so the values
    // are the kernel's input also where out aliases z)
    f32x4 resz[kGlobRes ? RB : 1][kGlobRes ? C::NPASS : 1][2];
    if constexpr (kGlobRes) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int ps = 0; ps < C::NPASS; ++ps) {
          int mj, m0;
          stage_coord<T>(ps, lane, mj, m0);
          const int64_t pr = rrow[rb][ps] >= 0 ? rrow[rb][ps] : 0;
          const TZ* src = (const TZ*)p.x + p.xmap(pr) + ch * 32 + m0;
          resz[rb][ps][0] = *reinterpret_cast<const f32x4*>(src);
          resz[rb][ps][1] = *reinterpret_cast<const f32x4*>(src + 4);
        }
    }
    // Orientation: channel-major outputs want lane <-> channel (x as A operand).
    bool chan_on_lanes;
    if (MODE == kTriMulIn || MODE == kPairBias) chan_on_lanes = true;
    else if (MODE == kTriAttnIn) chan_on_lanes = (ch >= 3 * (SL / 4));   // v^T and the triangle bias
    else chan_on_lanes = false;

    if (part != 2) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[rb][t][r] = 0.0f;

    // Weight fragments are read from LDS PF K steps ahead of the products that use them (a
    // ring of PF + 1 fragment pairs; PF = 0: each K step reads its own).  Left to the compiler,
    // every K step is "read two fragments, wait for them, two products" on one pair of
    // fragment registers.
    constexpr int PF = kWeightPrefetch;
    constexpr int NK0 = MODE == kTriMulOut ? SL : KS;   // K steps of tile 0; tile 1 has KS
    V8 wr0[PF + 1], wr1[PF + 1];
#pragma unroll
    for (int d = 0; d < PF; ++d) {
      wr0[d] = lds_w[wf0 + d][lane];
      if (d < KS) wr1[d] = lds_w[wf1 + d][lane];
    }
#pragma unroll
    for (int kk = 0; kk < NK0; ++kk) {
      if (kk + PF < NK0) wr0[(kk + PF) % (PF + 1)] = lds_w[wf0 + kk + PF][lane];
      if (kk + PF < KS) wr1[(kk + PF) % (PF + 1)] = lds_w[wf1 + kk + PF][lane];
      if constexpr (PF > 0) __builtin_amdgcn_sched_barrier(0);
      const V8 w0 = wr0[kk % (PF + 1)], w1 = wr1[kk % (PF + 1)];
      if (chan_on_lanes) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          mma32(acc[rb][0], xf.f[rb][kk], w0);
          mma32(acc[rb][1], xf.f[rb][kk], w1);
        }
      } else if constexpr (MODE == kTriMulOut) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) mma32(acc[rb][0], w0, xf2.f[rb][kk]);   // W_z LN_out(x)
        if (kk < KS) {
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) mma32(acc[rb][1], w1, xf.f[rb][kk]);  // W_g LN_in(z)
        }
      } else {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          mma32(acc[rb][0], w0, xf.f[rb][kk]);
          mma32(acc[rb][1], w1, xf.f[rb][kk]);
        }
      }
      if constexpr (PF > 0) __builtin_amdgcn_sched_barrier(0);
    }

    // fp32: the next chunk's weights go to LDS now, before this chunk's stores are issued:
    // waiting for those loads later would also wait for every store issued in between
    // (memory operations retire in order).
    if (!RES && !kDma && C::NBUF == 2) stash(buf ^ 1);
    }   // part != 2
    if (part == 1) return;

    // ------------------------------ epilogues ------------------------------
    if constexpr (MODE == kTriMulIn) {
      // a/b[c][i][k] = mask * sigmoid(gate) * proj ; lane <-> channel, register <-> row
      const int c0 = (ch % (SL / 2)) * 32;
      const int n_rb = (p.n + 31) >> 5, n_ks = p.pitch >> 4;
      T* outp_c0 = (T*)p.out[ch / (SL / 2)] + trimul_frag_offset(c0, 0, 0, n_rb, n_ks);
      constexpr int GT = NST < RB ? NST : RB;   // result tiles per LDS round trip
#pragma unroll
      for (int rb0 = 0; rb0 < RB; rb0 += GT) {
        wave_lds_sync();
#pragma unroll
        for (int q = 0; q < GT; ++q) {
          const int rb = rb0 + q;
          float vals[16];
#pragma unroll
          for (int qd = 0; qd < 4; ++qd) {
            const f32x4 m4 = *reinterpret_cast<const f32x4*>(&lds_mask[wave][rb * 32 + 8 * qd + 4 * g]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int r = 4 * qd + e;
              vals[r] = m4[e] * sigmoidf_fast(acc[rb][1][r]) * acc[rb][0][r];
            }
          }
          stage_put<T>(stile(q), vals, lane);
        }
        wave_lds_sync();
        // fragment-ordered store: 8 consecutive inner indices of one outer index = the 16
        // bytes of one operand lane (half-wave (pk0/8)%2, row outer%32)
#pragma unroll
        for (int q = 0; q < GT; ++q) {
          const int rb = rb0 + q;
#pragma unroll
          for (int ps = 0; ps < C::NPASS; ++ps) {
            int chn, r0;
            stage_coord<T>(ps, lane, chn, r0);
            *reinterpret_cast<VE_t*>(outp_c0 + rel_a[rb][ps]) = stage_get_vec<T>(stile(q), chn, r0);
          }
        }
      }
    } else if constexpr (MODE == kTriAttnIn) {
      // Outputs in the attention core's layouts (common.h): q and the gate head-major
      // [h][p][32], K / V^T / bias in fragment-ordered key tiles.
      const int which = ch / (SL / 4);
      const int key_tiles = p.pitch >> 6;
      const int q_blocks = (p.n + 31) >> 5;
      const int64_t head_plane = (int64_t)p.n * key_tiles * kAttnTileElems;   // K, V^T elements per head
      constexpr int GT = NST < 2 * RB ? NST : 2 * RB;   // result tiles per LDS round trip
#pragma unroll
      for (int k0 = 0; k0 < 2 * RB; k0 += GT) {
        // the group's result tiles go to the staging tiles first ...
        wave_lds_sync();
        auto put_group = [&](auto kind) {   // kind: 0 = q (rounded, then scaled), 2 = gate, 3 = bias, 1 = as is
          constexpr int KIND = decltype(kind)::value;
#pragma unroll
          for (int q = 0; q < GT; ++q) {
            const int rb = (k0 + q) >> 1, t = (k0 + q) & 1;
            float vals[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              float v = acc[rb][t][r];
              if (KIND == 0) v = to_f32(from_f32<T>(v)) * p.q_scale;
              if (KIND == 2) v = sigmoidf_fast(v);
              if (KIND == 3) v *= 1.4426950408889634f;   // log2(e): the attention core works in log2 units
              vals[r] = v;
            }
            stage_put<T>(stile(q), vals, lane);
          }
        };
        if (which == 0) put_group(std::integral_constant<int, 0>{});
        else if (which == 2) put_group(std::integral_constant<int, 2>{});
        else if (which == 4) put_group(std::integral_constant<int, 3>{});
        else put_group(std::integral_constant<int, 1>{});
        wave_lds_sync();
        // ... and are then read back as 16-byte vectors and stored
#pragma unroll
        for (int q = 0; q < GT; ++q) {
          const int rb = (k0 + q) >> 1, t = (k0 + q) & 1;
          const int h = (ch % (SL / 4)) * 2 + t;
          const T* stg = stile(q);
          if (which == 0 || which == 2) {
            // q and sigmoid(g): one 32 x 32 tile = one head, head-major rows
            store_row_major(stg, (T*)p.out[which] + (int64_t)h * p.n_rows * 32, 32, 0, rb, nullptr);
          } else if (which == 1) {
            // K: staged row-major (major = key row, minor = d); each 16-byte d-chunk goes to
            // its fragment slot
            T* outp = (T*)p.out[1] + h * head_plane;
#pragma unroll
            for (int ps = 0; ps < C::NPASS; ++ps) {
              int mj, m0;
              stage_coord<T>(ps, lane, mj, m0);
              *reinterpret_cast<VE_t*>(rrow[rb][ps] >= 0 ? outp + rel_k[rb][ps] : sink) =
                  stage_get_vec<T>(stg, mj, m0);
            }
          } else {
            // V^T (which == 3, major = channel d of head h) and the triangle bias (which == 4,
            // major = head, logical row = (query i, key j)): vectors of VE consecutive keys
            if (which == 4 && t == 1) continue;
#pragma unroll
            for (int ps = 0; ps < C::NPASS; ++ps) {
              int chn, r0;
              stage_coord<T>(ps, lane, chn, r0);
              const int64_t pr = row0 + rb * 32 + r0;
              if (which == 4 && chn >= p.aux) continue;
              const VE_t v = stage_get_vec<T>(stg, chn, r0);
              T* outp = (T*)p.out[which];
              if constexpr (vec_ok) {
                const int64_t off = which == 3 ? h * head_plane + rel_v[rb][ps] : (int64_t)rel_b[rb][ps];
                *reinterpret_cast<VE_t*>(cm_ok[rb] ? outp + off : sink) = v;
              } else {
                // (the row is made opaque here: the divisions below do not depend on the
                // chunk, so they would otherwise be hoisted out of the chunk loop for every
                // element and occupy some 240 registers in launches that never take this path)
                int64_t pr_here = pr;
                asm volatile("" : "+v"(pr_here));
#pragma unroll
                for (int e = 0; e < C::VE; ++e) {
                  if (pr_here + e < p.n_rows) {
                    const uint32_t pe = (uint32_t)(pr_here + e);
                    const uint32_t i = pe / (uint32_t)p.n, j = pe - i * (uint32_t)p.n;
                    const int64_t off = which == 3 ? attn_v_offset(h, i, j, chn, p.n, key_tiles)
                                                   : attn_b_offset(chn, i, j, q_blocks, key_tiles);
                    outp[off] = v[e];
                  }
                }
              }
            }
          }
        }
      }
    } else if constexpr (MODE == kPairBias) {
      // bias[h][p], dense planes of n*n elements, fp32 or T; lane <-> head, register <-> row
      const int heads = p.aux & 0xff;
      const bool f32_out = (p.aux >> 8) & 1;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int64_t pr0 = row0 + rb * 32;
        if (n < heads) {
#pragma unroll
          for (int qd = 0; qd < 4; ++qd) {
            const int64_t pr = pr0 + 8 * qd + 4 * g;
            if (f32_out) {
              float* dst = (float*)p.out[0] + (int64_t)n * p.n_rows + pr;
              if (pr + 4 <= p.n_rows && (p.n_rows & 3) == 0) {
                *reinterpret_cast<f32x4*>(dst) =
                    f32x4{acc[rb][0][4 * qd], acc[rb][0][4 * qd + 1], acc[rb][0][4 * qd + 2],
                          acc[rb][0][4 * qd + 3]};
              } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  if (pr + e < p.n_rows) dst[e] = acc[rb][0][4 * qd + e];
              }
            } else {
              T* dst = (T*)p.out[0] + (int64_t)n * p.n_rows + pr;
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (pr + e < p.n_rows) dst[e] = from_f32<T>(acc[rb][0][4 * qd + e]);
            }
          }
        }
      }
    } else {
      // kTriMulOut: out[p][col] = [z +] (W_z LN_out(x)) * sigmoid(W_g LN_in(z)), row-major.
      // out may alias z: the residual comes from the copy of z made before any store.
      if constexpr (kRegRes) {
        TZ* stz = lds_stage_z[wave];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          // this chunk's two fragments of the raw row (a uniform select: the chunk loop is
          // not unrolled, and registers cannot be indexed by a loop counter)
          f32x8 zr[2];
#pragma unroll
          for (int c = 0; c < KS / 2; ++c)
            if (ch == c) {
              zr[0] = to_f32(zres[rb][2 * c]);
              zr[1] = to_f32(zres[rb][2 * c + 1]);
            }
          wave_lds_sync();
#pragma unroll
          for (int k2 = 0; k2 < 2; ++k2) {
            f32x8 o;
#pragma unroll
            for (int t = 0; t < 8; ++t) {
              const int r = 8 * k2 + t;
              // linear_z output rounded to T, times the gate, rounded to T: the update
              const float u = to_f32(from_f32<T>(to_f32(from_f32<T>(acc[rb][0][r])) *
                                                 sigmoidf_fast(acc[rb][1][r])));
              // (bf16 rows: the sum is rounded once more on its way to the tile, like z + update)
              o[t] = p.add_residual ? zr[k2][t] + u : u;
            }
            // row n of the tile, columns 16*k2 + 8*g .. +7 (8-byte LDS stores)
            const typename Vec8<TZ>::type ov = from_f32<TZ>(o);
            u32x2* dst = reinterpret_cast<u32x2*>(stz + n * CZ::PITCH + 16 * k2 + 8 * g);
            const u32x2* src = reinterpret_cast<const u32x2*>(&ov);
#pragma unroll
            for (int h2 = 0; h2 < (int)sizeof(ov) / 8; ++h2) dst[h2] = src[h2];
          }
          wave_lds_sync();
#pragma unroll
          for (int ps = 0; ps < CZ::NPASS; ++ps) {
            int mj, m0;
            stage_coord<TZ>(ps, lane, mj, m0);
            const typename VecE<TZ>::type v = stage_get_vec<TZ>(stz, mj, m0);
            TZ* dstp = (TZ*)p.out[0] + rrow_z[rb][ps] * kCz + ch * 32 + m0;
            *reinterpret_cast<typename VecE<TZ>::type*>(
                rrow_z[rb][ps] >= 0 ? dstp : reinterpret_cast<TZ*>(g_store_sink) + lane * CZ::VE) = v;
          }
        }
      } else if constexpr (kGlobRes) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          float vals[16];
#pragma unroll
          for (int r = 0; r < 16; ++r)
            vals[r] = to_f32(from_f32<T>(acc[rb][0][r])) * sigmoidf_fast(acc[rb][1][r]);
          wave_lds_sync();
          stage_put<T>(st, vals, lane);   // (rounds the update to T)
          wave_lds_sync();
#pragma unroll
          for (int ps = 0; ps < C::NPASS; ++ps) {
            int mj, m0;
            stage_coord<T>(ps, lane, mj, m0);
            const f32x8 u = to_f32(stage_get_vec<T>(st, mj, m0));
            f32x4 o0 = {u[0], u[1], u[2], u[3]}, o1 = {u[4], u[5], u[6], u[7]};
            if (p.add_residual) {
              o0 += resz[rb][ps][0];
              o1 += resz[rb][ps][1];
            }
            TZ* dst = rrow[rb][ps] >= 0 ? (TZ*)p.out[0] + rrow[rb][ps] * kCz + ch * 32 + m0
                                        : reinterpret_cast<TZ*>(g_store_sink) + lane * 4;
            *reinterpret_cast<f32x4*>(dst) = o0;
            *reinterpret_cast<f32x4*>(rrow[rb][ps] >= 0 ? dst + 4 : dst) = o1;
          }
        }
      } else {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        float vals[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          // linear_z output is rounded to T before the gate multiply
          vals[r] = to_f32(from_f32<T>(acc[rb][0][r])) * sigmoidf_fast(acc[rb][1][r]);
        }
        wave_lds_sync();
        stage_put<T>(st, vals, lane);
        wave_lds_sync();
        store_row_major(st, (T*)p.out[0], kCz, ch * 32, rb, p.add_residual ? resv[rb] : nullptr);
      }
      }
    }

    if constexpr (kDma) {
      // The next chunk's weights must have landed: all but the stores this wave issued after
      // requesting them (a lower bound on that count is what is safe; the triangle bias,
      // whose store count varies, is the last chunk and has no successor).
      constexpr int kStores = MODE == kTriMulIn    ? RB * C::NPASS
                              : MODE == kTriAttnIn ? RB * 2 * C::NPASS
                              : MODE == kTriMulOut ? RB * C::NPASS
                                                   : 0;
      if (MODE != kTriAttnIn || vec_ok) ring_barrier<kStores>();
      else ring_barrier<0>();   // element-wise V^T stores: no fixed count
    } else if constexpr (!RES) {
      if (C::NBUF == 1) {
        __syncthreads();      // everyone is done reading the single buffer
        stash(0);
      }
      __syncthreads();
    }
  };
  if constexpr (kPrefetch) {
    // (unrolled: the stores between the request for the next rows and the wait for them are
    // then a count the compiler knows)
    f32x16 acc[RB][2];
#pragma unroll
    for (int ch = 0; ch < nch; ++ch) chunk_body(ch, acc, 0);
  } else {
    f32x16 acc[RB][2];
#pragma clang loop unroll(disable)
    for (int ch = 0; ch < nch; ++ch) chunk_body(ch, acc, 0);
  }
    if (!RES) break;
    normalize_prefetched();
    tile += tile_step;
  }
}

// Compute units of the current device (the resident kernels launch one workgroup per CU).
static int device_cu_count() {
  static int cache[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cache[dev] == 0) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
      v = 256;
    cache[dev] = v;
  }
  return cache[dev];
}

template <typename T, int MODE, int KS, typename TZ = T>
int launch_rowgemm_in(const RowGemmInParams& p, hipStream_t stream) {
  typedef InCfg<T, MODE, KS> IC;
  // (the attention projection on rows of 128 channels: one row block, and the registers the
  // second would take hold the next tile's raw rows instead - see kPrefetch in the kernel)
  constexpr int RB = (sizeof(T) == 2 && MODE != kTriMulOut && KS <= 8 && !(KS == 8 && MODE == kTriAttnIn)) ? 2 : 1;
  int64_t tiles = (p.n_rows + RB * 32 - 1) / (RB * 32);   // wave tiles, as in the kernel
  if (MODE == kTriMulIn) tiles = (int64_t)((p.n + 16 * RB - 1) / (16 * RB)) * (p.pitch / 8) * 4;
  if (tiles == 0) return 0;
  int64_t blocks = (tiles + IC::NW - 1) / IC::NW;
  if (IC::RES) blocks = std::min<int64_t>((tiles + IC::NW - 1) / IC::NW, device_cu_count());
  // (only the modes with channel-major vector stores have an element-wise variant)
  constexpr bool kHasScalarPath = MODE == kTriAttnIn || MODE == kTriMulOut;
  if (!kHasScalarPath || p.n % Cfg<T>::VE == 0)
    rowgemm_in_kernel<T, RB, MODE, KS, true, TZ><<<dim3((unsigned)blocks), dim3(IC::NW * 64), 0, stream>>>(p);
  else
    rowgemm_in_kernel<T, RB, MODE, KS, (kHasScalarPath ? false : true), TZ>
        <<<dim3((unsigned)blocks), dim3(IC::NW * 64), 0, stream>>>(p);
  return 0;
}

// ---------------------------------------------------------------------------
// rowgemm_out: out(p) = [res(p) +] A[p][0:K] W^T, K = 128 * n_slab, 128 output
// columns.  A is row-major with leading dimension K; out/res rows go through a
// RowMap (the ending-node attention writes z[j][i]).
// ---------------------------------------------------------------------------
struct RowGemmOutParams {
  const void* a;
  int a_head_major;     // A is [4][n_rows][32] (attention output) instead of [n_rows][K]
  int n_slab;
  const void* w;        // [128][128*n_slab]
  const void* res;      // residual source (same addressing as out) or null
  void* out;
  RowMap omap;
  int64_t n_rows;
};

// NOB = output column blocks of 32 (c_z / 32).  TZ: storage type of res and out (float with
// T = bf16: the T-rounded product is added to an fp32 residual stream).
template <typename T, int RB, int NOB, typename TZ = T>
__global__ __launch_bounds__(256, 2) void rowgemm_out_kernel(RowGemmOutParams p) {
  typedef typename Vec8<T>::type V8;
  typedef typename VecE<TZ>::type VE_t;
  typedef Cfg<T> CW;    // weight ring
  typedef Cfg<TZ> C;    // staging tile and stores
  constexpr bool MIXED = !std::is_same<T, TZ>::value;
  __shared__ V8 lds_w[CW::NBUF][2 * kKSteps][kWave];
  __shared__ __attribute__((aligned(16))) TZ lds_stage[4][32 * C::PITCH];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * (RB * 32);
  const int K = kC * p.n_slab;
  const T* w = (const T*)p.w;
  TZ* st = lds_stage[wave];

  f32x16 acc[RB][NOB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int t = 0; t < NOB; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rb][t][r] = 0.0f;

  // chunk c -> (slab = c / NH, column pair = c % NH), NH = NOB/2 chunks per slab; one slab
  // per outer iteration
  constexpr int NH = NOB / 2;
  V8 pre[4];
  auto fetch = [&](int ch) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int fid = wave * 4 + j;
      const int col0 = ((ch % NH) * 2 + (fid >> 3)) * 32;
      pre[j] = load_wfrag<T>(w, K, 32 * NOB, col0, (ch / NH) * kC + (fid & 7) * 16, lane);
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int j = 0; j < 4; ++j) lds_w[buf][wave * 4 + j][lane] = pre[j];
  };
  fetch(0);
  stash(0);
  __syncthreads();

  const RowMap amap{(int64_t)K, 0, 1};   // row p -> p*K (n_inner = 1, so outer = p)
  const int nch = NH * p.n_slab;
  for (int slab = 0; slab < p.n_slab; ++slab) {
    RowFrags<T, RB> af;
    if (p.a_head_major) {
      // channel 128*slab + 16*kk + 8*g + t = head 4*slab + kk/2, d = 16*(kk%2) + 8*g + t
      const int ln_ = lane & 31, g_ = lane >> 5;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        int64_t pr = row0 + rb * 32 + ln_;
        pr = pr < p.n_rows ? pr : p.n_rows - 1;
#pragma unroll
        for (int kk = 0; kk < kKSteps; ++kk)
          af.f[rb][kk] = load8<T>((const T*)p.a + ((int64_t)(slab * 4 + (kk >> 1)) * p.n_rows + pr) * 32 +
                                  16 * (kk & 1) + 8 * g_);
      }
    } else {
      load_rows<T, RB, false>(af, (const T*)p.a + slab * kC, amap, row0, p.n_rows,
                              (const T*)nullptr, (const T*)nullptr, 0.0f, lane);
    }
#pragma unroll
    for (int half = 0; half < NH; ++half) {
      const int ch = NH * slab + half;
      const int buf = CW::NBUF == 2 ? (ch & 1) : 0;
      fetch(min(ch + 1, nch - 1));
#pragma unroll
      for (int kk = 0; kk < kKSteps; ++kk) {
        const V8 w0 = lds_w[buf][kk][lane];
        const V8 w1 = lds_w[buf][kKSteps + kk][lane];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          // lane <-> row, register <-> output column
          mma32(acc[rb][2 * half], w0, af.f[rb][kk]);
          mma32(acc[rb][2 * half + 1], w1, af.f[rb][kk]);
        }
      }
      if (CW::NBUF == 1) __syncthreads();
      stash(CW::NBUF == 2 ? (buf ^ 1) : 0);
      __syncthreads();
    }
  }

  // out may alias res: a lane reads the residual vectors it is about to overwrite.  They
  // are requested up front, a group of output column blocks at a time: next to their stores
  // each would cost a serialised memory round trip, since no load can move above the previous
  // (possibly aliasing) store.  One group, except for fp32 rows of 256 channels, whose 32
  // residual vectors per lane do not fit beside the accumulators: two groups of four blocks.
  constexpr int GOB = (MIXED && NOB > 4) ? 4 : NOB;
  TZ* outp = (TZ*)p.out;
  const TZ* resp = (const TZ*)p.res;
  int64_t obase[RB][C::NPASS];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int ps = 0; ps < C::NPASS; ++ps) {
      int mj, m0;
      stage_coord<TZ>(ps, lane, mj, m0);
      const int64_t pr = row0 + rb * 32 + mj;
      obase[rb][ps] = pr < p.n_rows ? p.omap(pr) + m0 : -1;
    }
#pragma unroll
  for (int t0 = 0; t0 < NOB; t0 += GOB) {
    VE_t resv[RB][GOB][C::NPASS];
    if (resp) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int t = 0; t < GOB; ++t)
#pragma unroll
          for (int ps = 0; ps < C::NPASS; ++ps)
            if (obase[rb][ps] >= 0)
              resv[rb][t][ps] = *reinterpret_cast<const VE_t*>(resp + obase[rb][ps] + (t0 + t) * 32);
    }
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
      for (int t = 0; t < GOB; ++t) {
        float vals[16];
#pragma unroll
        for (int r = 0; r < 16; ++r)   // (mixed: the product is rounded to T before it is added)
          vals[r] = MIXED ? to_f32(from_f32<T>(acc[rb][t0 + t][r])) : acc[rb][t0 + t][r];
        wave_lds_sync();
        stage_put<TZ>(st, vals, lane);
        wave_lds_sync();
#pragma unroll
        for (int ps = 0; ps < C::NPASS; ++ps) {
          int mj, m0;
          stage_coord<TZ>(ps, lane, mj, m0);
          if (obase[rb][ps] >= 0) {
            VE_t v = stage_get_vec<TZ>(st, mj, m0);
            if (resp) v = add_vec<TZ>(v, resv[rb][t][ps]);
            *reinterpret_cast<VE_t*>(outp + obase[rb][ps] + (t0 + t) * 32) = v;
          }
        }
      }
    }
  }
}

template <typename T, int NOB, typename TZ = T>
int launch_rowgemm_out(const RowGemmOutParams& p, hipStream_t stream) {
  // (an fp32 residual stream doubles the residual vectors a lane holds: one row block then)
  constexpr int RB = (sizeof(T) == 2 && sizeof(TZ) == 2 && NOB <= 4) ? 2 : 1;
  const int64_t rows_per_block = 4 * RB * 32;
  const int64_t blocks = (p.n_rows + rows_per_block - 1) / rows_per_block;
  if (blocks == 0) return 0;
  rowgemm_out_kernel<T, RB, NOB, TZ><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(p);
  return 0;
}

// ---------------------------------------------------------------------------
// host entry points used by api.hip
// ---------------------------------------------------------------------------
static RowMap pair_map(int n, int c, bool transposed) {
  RowMap m;
  m.n_inner = n;
  m.stride_outer = transposed ? c : (int64_t)n * c;
  m.stride_inner = transposed ? (int64_t)n * c : c;
  return m;
}

template <typename T, typename TZ>
int trimul_project(const void* z, const void* mask, const void* ln_w, const void* ln_b,
                   const void* w_ap, const void* w_ag, const void* w_bp, const void* w_bg, void* a,
                   void* b, int n, int c_z, int k_pitch, int incoming, float eps,
                   hipStream_t stream) {
  RowGemmInParams p = {};
  p.x = z;
  p.xmap = pair_map(n, c_z, incoming != 0);
  p.n_rows = (int64_t)n * n;
  p.gamma = ln_w;
  p.beta = ln_b;
  p.eps = eps;
  p.w[0] = w_ap; p.w[1] = w_ag; p.w[2] = w_bp; p.w[3] = w_bg;
  p.out[0] = a; p.out[1] = b;
  p.mask = mask;
  p.mmap = pair_map(n, 1, incoming != 0);
  p.n = n;
  p.pitch = k_pitch;
  p.aux = incoming != 0;   // walk direction (see the kernel)
  if (c_z == 64) return launch_rowgemm_in<T, kTriMulIn, 4, TZ>(p, stream);
  if (c_z == 256) {
    if constexpr (sizeof(T) == 2) return launch_rowgemm_in<T, kTriMulIn, 16, TZ>(p, stream);
    else return -1;   // 256-channel rows are built for 16-bit arithmetic only (refused by the caller)
  }
  return launch_rowgemm_in<T, kTriMulIn, 8, TZ>(p, stream);
}

template <typename T, typename TZ>
int trimul_output(const void* x, const void* z, const void* ln_in_w, const void* ln_in_b,
                  const void* ln_out_w, const void* ln_out_b, const void* w_z, const void* w_g,
                  void* out, int n, int c_z, int add_residual, float eps, hipStream_t stream) {
  RowGemmInParams p = {};
  p.x = z;
  p.xmap = pair_map(n, c_z, false);
  p.n_rows = (int64_t)n * n;
  p.gamma = ln_in_w;
  p.beta = ln_in_b;
  p.eps = eps;
  p.w[0] = w_z; p.w[1] = w_g;
  p.out[0] = out;
  p.n = n;
  p.x2 = x;
  p.gamma2 = ln_out_w;
  p.beta2 = ln_out_b;
  p.add_residual = add_residual;
  if (c_z == 64) return launch_rowgemm_in<T, kTriMulOut, 4, TZ>(p, stream);
  if (c_z == 256) {
    if constexpr (sizeof(T) == 2) return launch_rowgemm_in<T, kTriMulOut, 16, TZ>(p, stream);
    else return -1;   // 256-channel rows are built for 16-bit arithmetic only (refused by the caller)
  }
  return launch_rowgemm_in<T, kTriMulOut, 8, TZ>(p, stream);
}

template <typename T, typename TZ>
int triattn_project(const void* z, const void* ln_w, const void* ln_b, const void* w_q,
                    const void* w_k, const void* w_v, const void* w_g, const void* w_b, void* q,
                    void* k, void* vt, void* g, void* tri_bias, int n, int c_z, int heads, int d,
                    int key_pitch, int transposed, float eps, hipStream_t stream) {
  RowGemmInParams p = {};
  p.x = z;
  p.xmap = pair_map(n, c_z, transposed != 0);
  p.n_rows = (int64_t)n * n;
  p.gamma = ln_w;
  p.beta = ln_b;
  p.eps = eps;
  p.w[0] = w_q; p.w[1] = w_k; p.w[2] = w_g; p.w[3] = w_v; p.w[4] = w_b;
  p.out[0] = q; p.out[1] = k; p.out[2] = g; p.out[3] = vt; p.out[4] = tri_bias;
  p.n = n;
  p.aux = heads;
  p.pitch = key_pitch;
  p.q_scale = 1.4426950408889634f / sqrtf((float)d);   // log2(e) / sqrt(d), see triattn.hip
  if (c_z == 64) return launch_rowgemm_in<T, kTriAttnIn, 4, TZ>(p, stream);
  if (c_z == 256) {
    if constexpr (sizeof(T) == 2) return launch_rowgemm_in<T, kTriAttnIn, 16, TZ>(p, stream);
    else return -1;   // 256-channel rows are built for 16-bit arithmetic only (refused by the caller)
  }
  return launch_rowgemm_in<T, kTriAttnIn, 8, TZ>(p, stream);
}

template <typename T, typename TZ>
int triattn_output(const void* o, const void* w_o, const void* z, void* out, int n, int c_z,
                   int transposed, int add_residual, hipStream_t stream) {
  RowGemmOutParams p = {};
  p.a = o;
  p.a_head_major = 1;
  p.n_slab = c_z == 256 ? 2 : 1;   // K = heads * 32 = 128, or 256 with the scaled-up hidden width
  p.w = w_o;
  p.res = add_residual ? z : nullptr;
  p.out = out;
  p.omap = pair_map(n, c_z, transposed != 0);
  p.n_rows = (int64_t)n * n;
  if (c_z == 64) return launch_rowgemm_out<T, 2, TZ>(p, stream);
  if (c_z == 256) {
    if constexpr (sizeof(T) == 2) return launch_rowgemm_out<T, 8, TZ>(p, stream);
    else return -1;
  }
  return launch_rowgemm_out<T, 4, TZ>(p, stream);
}

template <typename T, typename TZ>
int pair_bias_fwd(const void* z, const void* ln_w, const void* ln_b, const void* w, void* bias,
                  int n, int c_z, int heads, int out_f32, float eps, hipStream_t stream) {
  RowGemmInParams p = {};
  p.x = z;
  p.xmap = pair_map(n, c_z, false);
  p.n_rows = (int64_t)n * n;
  p.gamma = ln_w;
  p.beta = ln_b;
  p.eps = eps;
  p.w[0] = w;
  p.out[0] = bias;
  p.n = n;
  p.aux = heads | (out_f32 ? 0x100 : 0);
  if (c_z == 256) {
    if constexpr (sizeof(T) == 2) return launch_rowgemm_in<T, kPairBias, 16, TZ>(p, stream);
    else return -1;
  }
  return launch_rowgemm_in<T, kPairBias, 8, TZ>(p, stream);
}

#define PTX_INSTANTIATE(T, TZ)                                                                      \
  template int trimul_project<T, TZ>(const void*, const void*, const void*, const void*,           \
                                     const void*, const void*, const void*, const void*, void*,    \
                                     void*, int, int, int, int, float, hipStream_t);               \
  template int trimul_output<T, TZ>(const void*, const void*, const void*, const void*,            \
                                    const void*, const void*, const void*, const void*, void*,     \
                                    int, int, int, float, hipStream_t);                            \
  template int triattn_project<T, TZ>(const void*, const void*, const void*, const void*,          \
                                      const void*, const void*, const void*, const void*, void*,   \
                                      void*, void*, void*, void*, int, int, int, int, int, int,    \
                                      float, hipStream_t);                                         \
  template int triattn_output<T, TZ>(const void*, const void*, const void*, void*, int, int, int,  \
                                     int, hipStream_t);                                            \
  template int pair_bias_fwd<T, TZ>(const void*, const void*, const void*, const void*, void*,     \
                                    int, int, int, int, float, hipStream_t);
PTX_INSTANTIATE(float, float)
PTX_INSTANTIATE(bf16_t, bf16_t)
PTX_INSTANTIATE(bf16_t, float)
#undef PTX_INSTANTIATE

}  // namespace ptx
