// Triangle attention core: flash-style online softmax on MFMA, the N^3 logits
// are never written anywhere.
//
// One workgroup (4 waves) owns one (row i, head h) pair and 128 queries; each
// wave owns 32 queries and walks over the keys in staged tiles of 64, which it
// processes as two halves of 32 keys (16 logit registers at a time: four waves
// fit a SIMD).  Per half:
//   S^T[key][query]  = K Q^T + bias     2 + 2 MFMA
//   online softmax along keys = along the registers of a lane (+ one exchange
//   with the other half-wave), because MFMA puts the query on the lane
//   O^T[d][query]   += V^T P^T          2 MFMA, P^T taken straight from the S^T
//   accumulators with no shuffle
// MFMA row m of half u is mapped to key 32*((m>>2)&1) + 16*u + 4*(m>>3) + (m&3),
// which makes register r of half-wave g hold key 32*g + 16*u + r: 16 consecutive
// keys -> 16-byte bias loads, and 8 consecutive keys per P.V operand slot group.
// The triangle bias is the initial value of the S^T accumulators (converted to fp32 if it
// is stored in 16 bits).  q and the bias are stored multiplied by log2(e) (by the projection
// kernel), so on the common path the vector ALU executes per logit one conversion, one exp2,
// half a packed bf16 convert and half a dot2 (the row sum).
// K and V^T tiles are shared by the 4 waves through LDS in fragment order
// (a ring of three tiles, one barrier per tile); the bias tile is private to a wave
// and read straight from global (L2-resident: workgroups are numbered so that
// one XCD works on one head at a time).
//
// Mask semantics follow the reference's fp32 arithmetic exactly: on tiles that
// contain a masked (or out-of-range) key the logit is (q.k + inf*(mask-1)) +
// bias in that order on the vector ALU, so -1e9 absorbs small logits and a fully
// masked row averages v over all keys; tiles whose keys are all unmasked take
// the matrix-pipe path above.
#include <type_traits>

#include "common.h"
#include "kernels.h"

namespace ptx {

constexpr int kD = 32;          // head dim
constexpr int kKeyTile = 64;
constexpr float kLog2e = 1.4426950408889634f;
// half_row: code paths, and the largest per-lane probability sum of a half tile (16 values) the
// optimistic path accepts
enum { kOptimistic = 0, kClassic = 1, kMasked = 2, kOptimisticZero = 3 };
constexpr float kOptimisticLimit = 1.0e12f;
constexpr float kLn2 = 0.6931471805599453f;
// kClassic: a running maximum no larger than this (natural units, all lanes of the wave) is
// replaced by the reference 0, which makes exp2() of the raw logit the probability
constexpr float kZeroReferenceLimit = 14.0f;

// Addressing of q / gate / o and the optional outputs (see the kernel's header comment).
struct AttnAux {
  int64_t sh, si, sj;     // element strides of q, gate, o: head, row, query
  int n_rows;
  int mask_is_bias;
  float* lse;             // or null
  int64_t lh, li, lj;     // element strides of lse: head, row, query
  int row0, row_end;      // rows row0 .. row_end-1 are this launch's (a launch may cover a range)
  int n_keys;             // keys 0 .. n_keys-1 take part (n_keys <= n; the rest count as masked)
  int q_begin, q_end;     // queries q_begin .. q_end-1 of every row are this launch's (q_begin % 32 == 0)
};

// Rows of the pair tensor handled by one wave: R = 1 or 2, chosen per launch (triattn_fwd_ex).

// NWQ waves per workgroup (4 or 8), each with 32 queries: the workgroup's waves share the staged
// K / V^T tiles, so with 8 every wave moves one fragment per tile instead of two.
// n: queries = keys per row; ax.n_rows: rows (= n for a whole pair tensor, fewer for a chunk of
// rows).  q, gate and o are addressed through the element strides in `ax` (head, row, query; 32
// contiguous channels at each position); gate may be null (no gating).  mask: per (row, key),
// 0/1 values turned into inf*(mask-1), or with ax.mask_is_bias an additive bias used as it is.
// ax.lse: optional log2-sum-exp2 of the logits per (head, row, query).
// MK: kMaskGiven, or no mask (its own instantiations: a mask of all ones is passed as none by
// the host side).  Without a mask nothing of the masked path is left in the kernel; a last,
// partial key tile takes the same paths as the others with the logits of the keys beyond
// n_keys set to -inf (kMaskTail; kMaskNone where the keys fill whole tiles).
enum { kMaskNone = 0, kMaskTail = 1, kMaskGiven = 2 };
template <typename T, int R, int NWQ, int MK>
__global__ __launch_bounds__((NWQ * 64), (sizeof(T) == 2 ? (R == 1 ? 16 / NWQ : (NWQ == 8 ? (MK == kMaskTail ? 4 : 2) : 3)) : 2)) void triattn_fwd_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ vt,
    const T* gate, const T* __restrict__ bias, const T* __restrict__ mask,
    T* o, int n, int heads, int key_pitch, int mask_transposed, float inf,
    int n_qtiles, int n_rowgroups, int64_t total_items, AttnAux ax) {
  typedef typename Vec8<T>::type V8;
  typedef typename Vec4<T>::type V4;
  // ring of 3 key tiles x R rows: iteration t reads tile t while tile t+2 is written
  __shared__ V8 lds_kv[3][R][8][kWave];     // fragments 0-3: K (u,kk); 4-7: V^T (u,s)
  __shared__ __attribute__((aligned(16))) float lds_mb[3][R][kKeyTile];  // mask bias per key

  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int ln = lane & 31, g = lane >> 5;

  // Work item -> (h, row group, query tile), h-major, one contiguous span per XCD
  // (workgroups are dealt round-robin to the 8 XCDs).
  const int64_t per_xcd = (total_items + 7) / 8;
  const int64_t item = (int64_t)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (item >= total_items) return;
  const int qt = (int)(item % n_qtiles);
  const int i0 = ax.row0 + (int)((item / n_qtiles) % n_rowgroups) * R;   // first of this workgroup's R rows
  const int h = (int)(item / ((int64_t)n_qtiles * n_rowgroups));

  const int q0 = ax.q_begin + (qt * NWQ + wave) * 32;   // first query of this wave
  const int key_tiles = key_pitch >> 6;
  const int q_blocks = (n + 31) >> 5;
  const int nk = ax.n_keys;
  const int n_tiles = (nk + kKeyTile - 1) / kKeyTile;
  constexpr bool has_mask = MK == kMaskGiven;
  // Operand tiles in fragment order (common.h): 2048 elements per key tile, this lane's
  // 8 elements of fragment f at f*512 + lane*8.  Rows beyond n re-read row n-1, a wave whose
  // queries all lie beyond n re-reads the last query block; nothing of either is stored.
  const T* b_tiles = bias + ((int64_t)h * q_blocks + min(q0 >> 5, q_blocks - 1)) * key_tiles * kAttnTileElems + lane * 8;
  const int qi = min(q0 + ln, n - 1);
  const int n_rows = ax.n_rows;
  // Lanes whose query lies beyond n compute on whatever the bias workspace holds there; they
  // store nothing, and they are kept out of the wave-wide decisions below so that the path a
  // wave takes (and with it the rounding of its valid queries) never depends on that content.
  const bool q_ok = q0 + ln < ax.q_end;
  // (as a lane mask: wave-wide decisions are ballots of the condition alone, combined with this
  // mask on the scalar unit)
  const uint64_t q_ok_mask = __builtin_amdgcn_ballot_w64(q_ok);

  // Q fragments (B operand): lane <-> query, slots <-> d = 16*kk + 8*g + t
  V8 qf[R][2];
  int64_t qrow[R];                       // head-major q / gate / o row of this lane's query
#pragma unroll
  for (int r = 0; r < R; ++r) {
    qrow[r] = h * ax.sh + min(i0 + r, n_rows - 1) * ax.si + qi * ax.sj;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) qf[r][kk] = load8<T>(q + qrow[r] + 16 * kk + 8 * g);
  }

  // ---- cooperative tile loader: 8*R fragments per key tile, 2*R per wave ----
  // `tile` may run past the last tile: the pipeline below never branches around a load, so
  // that the compiler can count the outstanding loads exactly.  Addresses use the clamped
  // tile; the mask bias and the V^T zeroing use the real key index, which makes a phantom
  // tile contribute exactly nothing.  Keys beyond n_keys hold garbage (or, below n, keys that
  // are left out) in K, removed by the -inf mask bias, and are zeroed in V^T (0 * garbage must
  // stay 0).
  // fetch() only issues loads; everything that consumes a loaded value (mask -> additive
  // bias, zeroing of V^T beyond n) happens in stash(), one tile of work later, so no wait
  // for memory sits in the issue path.
  constexpr int FPW = 8 * R / NWQ;   // fragments each wave moves per tile
  V8 pre[FPW];
  T pre_mv;
  // mask value of key kc for this wave's row: m_base[kc * m_stride]
  const int m_row = min(i0 + min(wave, R - 1), n_rows - 1);
  const unsigned m_stride = mask_transposed ? n : 1;
  const T* m_base = has_mask ? mask + (mask_transposed ? (int64_t)m_row : (int64_t)m_row * n) : nullptr;
  auto fetch = [&](int tile) {
    const int64_t atile = min(tile, n_tiles - 1);
#pragma unroll
    for (int j = 0; j < FPW; ++j) {
      const int fid = wave * FPW + j;              // row = fid / 8, fragment = fid % 8
      const int r = fid >> 3, f = fid & 7;
      const int64_t rowtiles = ((int64_t)h * n_rows + min(i0 + r, n_rows - 1)) * key_tiles + atile;
      pre[j] = load8<T>((f < 4 ? k : vt) + rowtiles * kAttnTileElems + (f & 3) * 512 + lane * 8);
    }
    // wave w < R publishes the mask bias of row i0 + w; all waves load (uniform load count)
    if constexpr (has_mask) {
      const int kc = min(tile * kKeyTile + lane, n - 1);
      pre_mv = m_base[__umul24(kc, m_stride)];   // both below 2^15
    }
  };
  auto stash = [&](int tile) {
    const int buf = tile % 3;
    const int key0 = tile * kKeyTile;
    const bool tail = MK != kMaskNone && key0 + kKeyTile > nk;   // uniform (kMaskNone: whole tiles only)
#pragma unroll
    for (int j = 0; j < FPW; ++j) {
      const int fid = wave * FPW + j;
      const int f = fid & 7;
      V8 v = pre[j];
      if (tail && f >= 4) {
        // V^T fragment (u, s): slots <-> keys 32g + 16u + 8s + t
        const int koff = key0 + 32 * g + 16 * ((f >> 1) & 1) + 8 * (f & 1);
#pragma unroll
        for (int t = 0; t < 8; ++t) v[t] = koff + t < nk ? v[t] : (T)0.0f;
      }
      lds_kv[buf][fid >> 3][f][lane] = v;
    }
    if constexpr (has_mask) {
      if (wave < R) {
        const float mb = ax.mask_is_bias ? to_f32(pre_mv) : inf * (to_f32(pre_mv) - 1.0f);
        lds_mb[buf][wave][lane] = key0 + lane < nk ? mb : 0.0f;   // (beyond n_keys: see TAIL)
      }
    }
  };

  // ---- per-wave bias tile: lane <-> query, [u][c] = keys key0 + 32g + 16u + 8c .. +7 ----
  auto fetch_bias = [&](int tile, V8 (&dst)[2][2]) {
    const T* bp = b_tiles + (int64_t)min(tile, n_tiles - 1) * kAttnTileElems;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int c = 0; c < 2; ++c) dst[u][c] = load8<T>(bp + (u * 2 + c) * 512);
  };

  f32x16 acc_o[R];                // O^T per row
  float m_run[R], l_run[R];       // running max (natural units) and denominator (this lane's keys)
#pragma unroll
  for (int r = 0; r < R; ++r) {
#pragma unroll
    for (int e = 0; e < 16; ++e) acc_o[r][e] = 0.0f;
    m_run[r] = -INFINITY;
    l_run[r] = 0.0f;
  }

  // One half of a key tile: logits, online softmax, P^T.  `tb` was fetched one tile ago.
  // Complete instantiations, so that the rarer paths share no code with - and cannot be
  // speculated into - the common one:
  //   kOptimistic  The softmax reference m_run only has to keep exp() in
  //                range, so it is NOT updated: probabilities are taken against the reference
  //                left by earlier tiles, no tile maximum is formed and O, l are not rescaled.
  //                If a probability sum leaves the safe range (a logit ~28 above the
  //                reference, or no reference yet), nothing has been committed and the half
  //                is redone by kClassic.  Returns false in that case (same in all lanes).
  //   kOptimisticZero  the common path: the same with the reference 0 in all lanes.  q and
  //                the triangle bias arrive multiplied by log2(e), so the matrix pipe's
  //                result IS the exponent: one v_exp_f32 per logit and no other arithmetic.
  //   kClassic     running maximum, rescale of O and l (first tile, or redo).  A maximum of
  //                modest size is replaced by the reference 0 (any reference is exact as long
  //                as exp() stays in range), which puts the row on the kOptimisticZero path.
  //   kMasked      tiles with a masked or out-of-range key: the reference's exact fp32
  //                order (q.k + mask_bias) + triangle_bias.
  // A path works on one 32-key half u of the staged tile (keys 32g + 16u + 0..15 of half-wave
  // g): 16 logit registers instead of 32, which lets four waves share a SIMD (a wave issues a
  // vector instruction only every ~9 cycles; it takes several to keep the vector unit busy).
  // What a path hands to the commit point of its half: P^T as the B operand of P.V, this
  // lane's probability sum, and the factor by which O and l shrink first (1 unless the
  // reference moved).
  struct HalfOut {
    V8 pf[2];
    float psum, alpha;
  };
  // TAIL: the tile holds keys beyond n_keys; their logits, whatever was made of the K rows and
  // mask values found there, are replaced by -inf before the softmax (weight zero).  The other
  // keys of such a tile take the same path as in any other tile, so a mask of all ones gives
  // the bits that no mask gives.
  // `r`: which of the wave's R rows; `tbf`: the half's bias tile in fp32 (converted once per
  // half, for all R rows: they share the query block and with it the bias).
  auto half_row = [&](auto mode_tag, auto tail_tag, int r, int buf, int u, int key0, V8 (&tbh)[2],
                      const f32x16& tbf, HalfOut& out) -> bool {
    constexpr int MODE = decltype(mode_tag)::value;
    constexpr bool MASKED = MODE == kMasked;
    constexpr bool TAIL = decltype(tail_tag)::value;
    V8 kf[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) kf[kk] = lds_kv[buf][r][u * 2 + kk][lane];
    f32x16 s;
    if constexpr (!MASKED) {
      // S^T starts from the bias, the C operand of the first product: register e of this lane
      // <-> element e of its 16 stored values (16-bit: one conversion per logit, which with
      // four waves per SIMD costs less than adding the bias on the matrix pipe)
      s = tbf;
    } else {
#pragma unroll
      for (int e = 0; e < 16; ++e) s[e] = 0.0f;
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) mma32(s, kf[kk], qf[r][kk]);
    if constexpr (MASKED) {
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const f32x8 b = to_f32(tbh[c]);
        const f32x4 m0 = *reinterpret_cast<const f32x4*>(&lds_mb[buf][r][32 * g + 16 * u + 8 * c]);
        const f32x4 m1 = *reinterpret_cast<const f32x4*>(&lds_mb[buf][r][32 * g + 16 * u + 8 * c + 4]);
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          const float mbv = t < 4 ? m0[t & 3] : m1[t & 3];
          s[8 * c + t] = (s[8 * c + t] * kLn2 + mbv) + b[t] * kLn2;
        }
      }
    }
    if constexpr (TAIL) {
      const int kfirst = key0 + 32 * g + 16 * u;   // register e <-> key kfirst + e
#pragma unroll
      for (int e = 0; e < 16; ++e) s[e] = kfirst + e < nk ? s[e] : -INFINITY;
    }
    float alpha = 1.0f;
    if constexpr (MODE == kClassic || MODE == kMasked) {
      float mx[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) mx[j] = fmaxf(s[2 * j], s[2 * j + 1]);
      float mt = fmaxf(fmaxf(fmaxf(mx[0], mx[1]), fmaxf(mx[2], mx[3])),
                       fmaxf(fmaxf(mx[4], mx[5]), fmaxf(mx[6], mx[7])));
      mt = fmaxf(mt, swap32(mt));
      if (!MASKED) mt *= kLn2;
      // (a half whose keys all lie beyond n has mt = -inf: the reference stays where it is)
      float m_new = fmaxf(m_run[r], mt);
      if (!MASKED && (__builtin_amdgcn_ballot_w64(!(fabsf(m_new) < kZeroReferenceLimit)) & q_ok_mask) == 0ull) m_new = 0.0f;
      alpha = m_new == -INFINITY ? 1.0f : fast_exp2((m_run[r] - m_new) * kLog2e);
      m_run[r] = m_new;
    }
    if constexpr (MODE == kOptimisticZero) {
#pragma unroll
      for (int e = 0; e < 16; ++e) s[e] = fast_exp2(s[e]);
    } else if constexpr (!MASKED) {
      const float nml = -m_run[r] * kLog2e;
#pragma unroll
      for (int e = 0; e < 16; ++e) s[e] = fast_exp2(s[e] + nml);
    } else {
      // (no key with a finite logit yet: -inf minus a finite stand-in is -inf, weight 0, where
      // -inf minus -inf would not be a number)
      const float mref = fmaxf(m_run[r], -3.0e38f);
#pragma unroll
      for (int e = 0; e < 16; ++e) s[e] = fast_exp2((s[e] - mref) * kLog2e);
    }
    float psum = 0.0f;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      f32x8 p8;
#pragma unroll
      for (int t = 0; t < 8; ++t) p8[t] = s[8 * c + t];
      out.pf[c] = from_f32<T>(p8);
      if constexpr (sizeof(T) == 2) {
        typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
        bf16x2_t ones;
        ones[0] = (__bf16)1.0f;
        ones[1] = (__bf16)1.0f;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          bf16x2_t pr;
          pr[0] = out.pf[c][2 * t];
          pr[1] = out.pf[c][2 * t + 1];
          psum = __builtin_amdgcn_fdot2_f32_bf16(pr, ones, psum, false);
        }
      } else {
#pragma unroll
        for (int t = 0; t < 8; ++t) psum += p8[t];
      }
    }
    if constexpr (MODE == kOptimistic || MODE == kOptimisticZero) {
      if ((__builtin_amdgcn_ballot_w64(!(psum < kOptimisticLimit)) & q_ok_mask) != 0ull) return false;
    }
    out.psum = psum;
    out.alpha = alpha;
    return true;
  };
  auto process_tile = [&](auto tail_tag, int tile, V8 (&tb)[2][2]) {
    constexpr bool LAST_PARTIAL = decltype(tail_tag)::value;   // the one tile with keys beyond n_keys
    const int buf = tile % 3;
    const int key0 = tile * kKeyTile;
    // keys of the tile with a non-zero mask bias, per row, as a lane mask (key <-> lane); half
    // u's keys are the lanes with bit 4 == u
    uint64_t mb_mask[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      mb_mask[r] = 0ull;
      if constexpr (has_mask) mb_mask[r] = __builtin_amdgcn_ballot_w64(lds_mb[buf][r][lane] != 0.0f);
    }
    // keys of this tile that take part (uniform; 64 or more: all).  Half u holds the keys
    // 16u .. 16u+15 and 32+16u .. 32+16u+15 of the tile: complete from 48 + 16u keys on, empty
    // (and left out altogether) up to 16u.
    const int tile_keys = LAST_PARTIAL ? nk - key0 : kKeyTile;
    // A wave whose queries all lie beyond the launch's range only helps to stage the tiles (the
    // bias loads below stay unconditional: both paths then leave the same loads in flight).
    if (q_ok_mask != 0ull) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const bool tail_tile = LAST_PARTIAL && tile_keys < 48 + 16 * u;
      if (LAST_PARTIAL && tile_keys <= 16 * u) continue;
      const f32x8 b0 = to_f32(tb[u][0]), b1 = to_f32(tb[u][1]);
      const f32x16 tbf = __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        // the unmasked paths of one half: optimistic against the reference the earlier tiles
        // left, classic if there is none yet or the optimistic one had to give up
        auto unmasked_half = [&](auto ttag, HalfOut& out) -> bool {
          bool done = false;
          if (tile != 0 || u != 0) {
            if ((__builtin_amdgcn_ballot_w64(m_run[r] != 0.0f) & q_ok_mask) == 0ull)
              done = half_row(std::integral_constant<int, kOptimisticZero>{}, ttag, r, buf, u, key0, tb[u], tbf, out);
            else
              done = half_row(std::integral_constant<int, kOptimistic>{}, ttag, r, buf, u, key0, tb[u], tbf, out);
          }
          if (!done) half_row(std::integral_constant<int, kClassic>{}, ttag, r, buf, u, key0, tb[u], tbf, out);
          return !done;   // classic: O and l are rescaled first
        };
        HalfOut out;
        bool rescale = true;
        // this half's keys are those of lanes with bit 4 == u
        if (has_mask && (mb_mask[r] & (u ? 0xffff0000ffff0000ull : 0x0000ffff0000ffffull)) != 0ull) {
          if (tail_tile) half_row(std::integral_constant<int, kMasked>{}, std::true_type{}, r, buf, u, key0, tb[u], tbf, out);
          else half_row(std::integral_constant<int, kMasked>{}, std::false_type{}, r, buf, u, key0, tb[u], tbf, out);
        } else if (tail_tile) {
          rescale = unmasked_half(std::true_type{}, out);
        } else {
          rescale = unmasked_half(std::false_type{}, out);
        }
        if (rescale) {
#pragma unroll
          for (int e = 0; e < 16; ++e) acc_o[r][e] *= out.alpha;
          l_run[r] *= out.alpha;
        }
        l_run[r] += out.psum;
#pragma unroll
        for (int c = 0; c < 2; ++c) mma32(acc_o[r], lds_kv[buf][r][4 + u * 2 + c][lane], out.pf[c]);
      }
    }
    }
    fetch_bias(tile + 1, tb);
  };
  // Tile t+2 travels global -> registers -> LDS while tile t is processed; the bias tile of
  // t+1 is requested into the bias registers once tile t has consumed them.
  V8 tbias[2][2];
  auto step = [&](auto tail_tag, int tile) {
    fetch(tile + 2);
    process_tile(tail_tag, tile, tbias);
    stash(tile + 2);
    __syncthreads();
  };

  fetch(0);
  fetch_bias(0, tbias);
  stash(0);
  fetch(1);
  stash(1);
  __syncthreads();
  // the tiles whose keys all take part, in a loop that knows nothing of a partial tile (with
  // its tests in the loop every tile was 7 % slower), then the partial one if there is one
  const int n_full = MK == kMaskNone ? n_tiles : nk / kKeyTile;
  for (int tile = 0; tile < n_full; ++tile) step(std::false_type{}, tile);
  if constexpr (MK != kMaskNone) {
    if (n_full < n_tiles) step(std::true_type{}, n_full);
  }

  // ---- normalise, gate, store: lane <-> query, register e <-> d = acc_row(e, g) ----
  // o may alias gate: every gate load is issued before the first store.
  // (the row offsets are formed again from a laundered query index: kept across the key loop
  // they cost two registers of a budget that has none to spare)
  int qi_again = qi;
  asm volatile("" : "+v"(qi_again));
#pragma unroll
  for (int r = 0; r < R; ++r) qrow[r] = h * ax.sh + min(i0 + r, n_rows - 1) * ax.si + qi_again * ax.sj;
  f32x4 gv[R][4];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      gv[r][c] = f32x4{1.0f, 1.0f, 1.0f, 1.0f};
      if (gate) gv[r][c] = to_f32(*reinterpret_cast<const V4*>(gate + qrow[r] + 4 * g + 8 * c));
    }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const float l_tot = l_run[r] + swap32(l_run[r]);
    const float inv = fast_rcp(l_tot);
    if (ax.lse && g == 0 && q0 + ln < ax.q_end && i0 + r < ax.row_end)
      ax.lse[h * ax.lh + (int64_t)(i0 + r) * ax.li + (int64_t)qi_again * ax.lj] =
          m_run[r] * kLog2e + __builtin_amdgcn_logf(l_tot);   // v_log_f32 is log2
    if (q0 + ln < ax.q_end && i0 + r < ax.row_end) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        f32x4 ov;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          // attention output rounded to T before the gate multiply, as the reference does
          ov[t] = to_f32(from_f32<T>(acc_o[r][4 * c + t] * inv)) * gv[r][c][t];
        }
        *reinterpret_cast<V4*>(o + qrow[r] + 4 * g + 8 * c) = from_f32<T>(ov);
      }
    }
  }
}

template <typename T>
int triattn_fwd(const T* q, const T* k, const T* vt, const T* g, const T* tri_bias, const T* mask,
                T* o, int n, int heads, int key_pitch, int mask_transposed, float inf,
                int row_begin, int row_count, int n_keys, hipStream_t stream) {
  // head-major q, gate, o of a whole pair tensor: [heads][n][n][32]
  AttnAux ax = {};
  ax.sh = (int64_t)n * n * kD;
  ax.si = (int64_t)n * kD;
  ax.sj = kD;
  ax.n_rows = n;
  return triattn_fwd_ex<T>(q, k, vt, g, tri_bias, mask, o, n, n, heads, key_pitch, mask_transposed, inf,
                           0, ax.sh, ax.si, ax.sj, nullptr, 0, 0, 0, row_begin, row_count, n_keys, stream);
}

template <typename T>
int triattn_fwd_ex(const T* q, const T* k, const T* vt, const T* g, const T* tri_bias,
                   const T* mask, T* o, int n_rows, int n, int heads, int key_pitch,
                   int mask_transposed, float inf, int mask_is_bias, int64_t sh, int64_t si,
                   int64_t sj, float* lse, int64_t lh, int64_t li, int64_t lj, int row_begin,
                   int row_count, int n_keys, hipStream_t stream) {
  if (n == 0 || n_rows == 0 || row_count == 0) return 0;
  AttnAux ax = {sh, si, sj, n_rows, mask_is_bias, lse, lh, li, lj, row_begin, row_begin + row_count, n_keys, 0, n};
  // 8-wave workgroups for long rows (measured: +2 % at n = 768, even at 1024, -2.6 % at 1536,
  // -2.2 % at 2048), where their 256 queries divide n or n is large enough for the idle waves
  // of the last one not to matter
  const bool wide = sizeof(T) == 2 && ((n % 256 == 0 && n >= 1536) || n >= 2048);
  // Two rows per wave, in 8-wave workgroups (16-bit, no mask): the two rows
  // share the query block and with it the bias tile - one load and one conversion per logit for
  // both, half the bias stream from the L2 - at 123 registers, so that four waves still share a
  // SIMD (with a partial last key tile the register allocator is held to 128 by the kernel's
  // launch bounds and gets there without spills; with a mask the kernel needs 160 and loses a
  // wave; with four waves per workgroup the K / V tiles of two rows leave room for three
  // workgroups only: no gain).  Per launch: 395 -> 356 us at n = 768 in the trunk; in a loop of attention updates
  // -7 % at n = 512, -3 % at 768, -11 % at 1536, -13 % at 2048.  Where 256 queries do not divide
  // n, the waves of a row's last workgroup that have no queries skip the arithmetic and only
  // help to stage the K / V tiles; such a workgroup still holds its place for as long as the
  // staging takes (n = 776 against 768, same keys: +11 %), but a second launch for the
  // remaining queries - one row per wave, two or four waves per workgroup - was no better
  // (per update, against the split launches with every wave computing: 520 214 -> 208 us,
  // 640 270 -> 255, 704 369 -> 332, 800 592 -> 550, 1032 1127 -> 1055, 1100 1239 -> 1214).
  const bool r2 = sizeof(T) == 2 && !mask && n >= 512 && row_count >= 2;
  const int mk = mask ? kMaskGiven : n_keys % kKeyTile ? kMaskTail : kMaskNone;
  // one launch over the queries q_begin .. q_end-1 of the launch's rows
  auto launch = [&](int q_begin, int q_end, bool two_rows, bool wide8) {
    ax.q_begin = q_begin;
    ax.q_end = q_end;
    const int nq = q_end - q_begin;
    const int n_qtiles = (two_rows || wide8) ? (nq + 255) / 256 : (nq + 127) / 128;
    const int R = two_rows ? 2 : 1;
    const int n_rowgroups = (row_count + R - 1) / R;
    const int64_t total = (int64_t)heads * n_rowgroups * n_qtiles;
    const int64_t per_xcd = (total + 7) / 8;
#define PTX_ATTN_LAUNCH_R(RR, NWQ, MK)                                                            \
  triattn_fwd_kernel<T, RR, NWQ, MK><<<dim3((unsigned)(per_xcd * 8)), dim3(NWQ * 64), 0, stream>>>( \
      q, k, vt, g, tri_bias, mask, o, n, heads, key_pitch, mask_transposed, inf, n_qtiles,        \
      n_rowgroups, total, ax)
#define PTX_ATTN_LAUNCH(NWQ, MK) PTX_ATTN_LAUNCH_R(1, NWQ, MK)
    if (two_rows) {
      if constexpr (sizeof(T) == 2) {
        if (mk == kMaskTail) PTX_ATTN_LAUNCH_R(2, 8, kMaskTail);
        else PTX_ATTN_LAUNCH_R(2, 8, kMaskNone);
      }
    } else if (wide8) {
      if (mk == kMaskGiven) PTX_ATTN_LAUNCH(8, kMaskGiven);
      else if (mk == kMaskTail) PTX_ATTN_LAUNCH(8, kMaskTail);
      else PTX_ATTN_LAUNCH(8, kMaskNone);
    } else {
      if (mk == kMaskGiven) PTX_ATTN_LAUNCH(4, kMaskGiven);
      else if (mk == kMaskTail) PTX_ATTN_LAUNCH(4, kMaskTail);
      else PTX_ATTN_LAUNCH(4, kMaskNone);
    }
#undef PTX_ATTN_LAUNCH
#undef PTX_ATTN_LAUNCH_R
  };
  if (r2) {
    launch(0, n, true, false);
  } else {
    launch(0, n, false, wide);
  }
  return 0;
}

#define PTX_INSTANTIATE_EX(T)                                                                     \
  template int triattn_fwd_ex<T>(const T*, const T*, const T*, const T*, const T*, const T*, T*,  \
                                 int, int, int, int, int, float, int, int64_t, int64_t, int64_t,  \
                                 float*, int64_t, int64_t, int64_t, int, int, int, hipStream_t);
PTX_INSTANTIATE_EX(float)
PTX_INSTANTIATE_EX(bf16_t)
#undef PTX_INSTANTIATE_EX
template int triattn_fwd<float>(const float*, const float*, const float*, const float*,
                                const float*, const float*, float*, int, int, int, int, float,
                                int, int, int, hipStream_t);
template int triattn_fwd<bf16_t>(const bf16_t*, const bf16_t*, const bf16_t*, const bf16_t*,
                                 const bf16_t*, const bf16_t*, bf16_t*, int, int, int, int, float,
                                 int, int, int, hipStream_t);

}  // namespace ptx
