// Triangle attention core: flash-style online softmax on MFMA, the N^3 logits
// are never written anywhere.
//
// One workgroup (4 waves) owns one (row i, head h) pair and 128 queries; each
// wave owns 32 queries and walks over the keys in tiles of 64.  Per tile:
//   S^T[key][query]  = K Q^T + bias     2 x (2 + 2) MFMA (two 32-key halves)
//   online softmax along keys = along the registers of a lane (+ one exchange
//   with the other half-wave), because MFMA puts the query on the lane
//   O^T[d][query]   += V^T P^T          4 MFMA, P^T taken straight from the S^T
//   accumulators with no shuffle
// MFMA row m of half u is mapped to key 32*((m>>2)&1) + 16*u + 4*(m>>3) + (m&3),
// which makes register r of half-wave g hold key 32*g + 16*u + r: 16 consecutive
// keys -> 16-byte bias loads, and 8 consecutive keys per P.V operand slot group.
// The triangle bias never touches the vector ALU: its raw bf16 registers are the
// B operand of an MFMA whose A operand is the constant 0/1 matrix that undoes the
// key permutation, accumulating straight into S^T.  Per logit the vector ALU
// executes one fma, one exp2, half a max3 and half a packed bf16 convert.
// K and V^T tiles are shared by the 4 waves through LDS in fragment order
// (double-buffered, one barrier per tile); the bias tile is private to a wave
// and read straight from global (L2-resident: workgroups are numbered so that
// one XCD works on one head at a time).
//
// Mask semantics follow the reference's fp32 arithmetic exactly: on tiles that
// contain a masked (or out-of-range) key the logit is (q.k + inf*(mask-1)) +
// bias in that order on the vector ALU, so -1e9 absorbs small logits and a fully
// masked row averages v over all keys; tiles whose keys are all unmasked take
// the matrix-pipe path above.
#include "common.h"
#include "kernels.h"

namespace ptx {

constexpr int kD = 32;          // head dim
constexpr int kKeyTile = 64;
constexpr float kLog2e = 1.4426950408889634f;

template <typename T>
__global__ __launch_bounds__(256, 2) void triattn_fwd_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ vt,
    const T* gate, const T* __restrict__ bias, const T* __restrict__ mask,
    T* o, int n, int heads, int key_pitch, int mask_transposed, float inf,
    int n_qtiles, int64_t total_items) {
  typedef typename Vec8<T>::type V8;
  typedef typename Vec4<T>::type V4;
  // ring of 3 key tiles: iteration t reads V^T(t) and K(t+1) while tile t+2 is written
  __shared__ V8 lds_kv[3][8][kWave];     // fragments 0-3: K (u,kk); 4-7: V^T (u,s)
  __shared__ __attribute__((aligned(16))) float lds_mb[3][kKeyTile];  // mask bias of the tile's keys

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ln = lane & 31, g = lane >> 5;

  // Work item -> (h, i, query tile), h-major, one contiguous span per XCD
  // (workgroups are dealt round-robin to the 8 XCDs).
  const int64_t per_xcd = (total_items + 7) / 8;
  const int64_t item = (int64_t)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (item >= total_items) return;
  const int qt = (int)(item % n_qtiles);
  const int i = (int)((item / n_qtiles) % n);
  const int h = (int)(item / ((int64_t)n_qtiles * n));

  const int q0 = (qt * 4 + wave) * 32;   // first query of this wave
  const int key_tiles = key_pitch >> 6;
  const int q_blocks = (n + 31) >> 5;
  // operand tiles in fragment order (common.h): 2048 elements per key tile, this lane's
  // 8 elements of fragment f at f*512 + lane*8
  const T* k_tiles = k + ((int64_t)h * n + i) * key_tiles * kAttnTileElems + lane * 8;
  const T* v_tiles = vt + ((int64_t)h * n + i) * key_tiles * kAttnTileElems + lane * 8;
  // (a wave whose queries all lie beyond n re-reads the last block; nothing of it is stored)
  const T* b_tiles = bias + ((int64_t)h * q_blocks + min(q0 >> 5, q_blocks - 1)) * key_tiles * kAttnTileElems + lane * 8;
  // queries beyond n re-read the last one; their results are never stored
  const int qi = min(q0 + ln, n - 1);
  const int64_t qrow = (((int64_t)h * n + i) * n + qi) * kD;   // head-major q / gate / o row

  // Q fragments (B operand): lane <-> query, slots <-> d = 16*kk + 8*g + t
  V8 qf[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk)
    qf[kk] = load8<T>(q + qrow + 16 * kk + 8 * g);

  // Constant operands.  sel[s]: A operand with sel[m][slot (g,t)] = 1 iff key(m) is the key
  // behind slot (g,t) of step s, i.e. g == (m>>2)&1 and 8s+t == 4*(m>>3) + (m&3).
  V8 sel[2];
  {
    const int g_m = (ln >> 2) & 1, r_m = 4 * (ln >> 3) + (ln & 3);
#pragma unroll
    for (int sgrp = 0; sgrp < 2; ++sgrp)
#pragma unroll
      for (int t = 0; t < 8; ++t) sel[sgrp][t] = (T)((g == g_m && 8 * sgrp + t == r_m) ? 1.0f : 0.0f);
  }

  const int n_tiles = (n + kKeyTile - 1) / kKeyTile;
  const bool has_mask = mask != nullptr;
  const T* mask_or_dummy = has_mask ? mask : q;   // any valid address: the value is discarded

  // ---- cooperative tile loader: wave w fetches fragments 2w and 2w+1 ----
  // All loads are unconditional (indices clamped): keys beyond n get a -inf mask
  // bias below, which removes them from the softmax whatever K holds; V^T is zeroed
  // for them because 0 * garbage must stay 0.
  V8 pre[2];
  float pre_mb = 0.0f;
  auto fetch = [&](int tile) {
    // `tile` may run past the last tile (the pipeline below never branches around a load, so
    // that the compiler can count outstanding loads exactly): addresses use the clamped tile,
    // the mask bias and the V^T zeroing use the real key index, which makes a phantom tile
    // contribute exactly nothing.
    const int key0 = tile * kKeyTile;
    const int akey0 = min(tile, n_tiles - 1) * kKeyTile;
    const bool tail = key0 + kKeyTile > n;   // uniform
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int fid = wave * 2 + j;
      const int u = (fid >> 1) & 1, sub = fid & 1;
      if (fid < 4) {
        // K (A operand): MFMA row m <-> key 32*((m>>2)&1) + 16u + 4*(m>>3) + (m&3); slots <-> d.
        // Keys beyond n hold garbage; the -inf mask bias removes them.
        pre[j] = load8<T>(k_tiles + (int64_t)(akey0 >> 6) * kAttnTileElems + fid * 512);
      } else {
        // V^T (A operand): MFMA row <-> d = ln; slots <-> keys 32g + 16u + 8s + t
        const int koff = 32 * g + 16 * u + 8 * sub;
        V8 v = load8<T>(v_tiles + (int64_t)(akey0 >> 6) * kAttnTileElems + (fid - 4) * 512);
        if (tail) {
#pragma unroll
          for (int t = 0; t < 8; ++t) v[t] = key0 + koff + t < n ? v[t] : (T)0.0f;
        }
        pre[j] = v;
      }
    }
    {
      // every wave loads (keeps the load count uniform); wave 0 publishes it
      const int key = key0 + lane;
      const int kc = min(key, n - 1);
      const int64_t mi = mask_transposed ? (int64_t)kc * n + i : (int64_t)i * n + kc;
      const float mv = to_f32(mask_or_dummy[has_mask ? mi : 0]);
      const float mb = has_mask ? inf * (mv - 1.0f) : 0.0f;
      pre_mb = key < n ? mb : -INFINITY;
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int j = 0; j < 2; ++j) lds_kv[buf][wave * 2 + j][lane] = pre[j];
    if (wave == 0) lds_mb[buf][lane] = pre_mb;
  };

  // ---- per-wave bias tile: lane <-> query, [u][c] = keys key0 + 32g + 16u + 8c .. +7 ----
  auto fetch_bias = [&](int tile, V8 (&dst)[2][2]) {
    const T* bp = b_tiles + (int64_t)min(tile, n_tiles - 1) * kAttnTileElems;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int c = 0; c < 2; ++c) dst[u][c] = load8<T>(bp + (u * 2 + c) * 512);
  };

  f32x16 acc_o;                   // O^T
#pragma unroll
  for (int r = 0; r < 16; ++r) acc_o[r] = 0.0f;
  float m_run = -INFINITY;        // running max, natural units
  float l_run = 0.0f;             // running denominator over this lane's keys (halves add up at the end)

  // One key tile: logits, online softmax, P.V.  `tb` was fetched one tile ago.
  auto process_tile = [&](int tile, V8 (&tb)[2][2]) {
    const int buf = tile % 3;
    const float mb_lane = lds_mb[buf][lane];
    // Does this tile hold a masked or out-of-range key?  Same answer in all waves.
    const bool masked_tile = __ballot(mb_lane != 0.0f) != 0ull;
    f32x16 s[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[u][r] = 0.0f;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) mma32(s[u], lds_kv[buf][u * 2 + kk][lane], qf[kk]);
    }
    if (!masked_tile) {
      // bias on the matrix pipe: S^T += Sel * Bias
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int c = 0; c < 2; ++c) mma32(s[u], sel[c], tb[u][c]);
    } else {
      // exact reference order in fp32: (q.k + mask_bias) + triangle_bias
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          const f32x8 b = to_f32(tb[u][c]);
          const f32x4 m0 = *reinterpret_cast<const f32x4*>(&lds_mb[buf][32 * g + 16 * u + 8 * c]);
          const f32x4 m1 = *reinterpret_cast<const f32x4*>(&lds_mb[buf][32 * g + 16 * u + 8 * c + 4]);
#pragma unroll
          for (int t = 0; t < 8; ++t) {
            const float mbv = t < 4 ? m0[t & 3] : m1[t & 3];
            const float v = (s[u][8 * c + t] + mbv) + b[t];
            s[u][8 * c + t] = mbv == -INFINITY ? -INFINITY : v;   // key beyond n
          }
        }
    }

    float mx[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      mx[j] = fmaxf(fmaxf(s[0][2 * j], s[0][2 * j + 1]), fmaxf(s[1][2 * j], s[1][2 * j + 1]));
    float mt = fmaxf(fmaxf(fmaxf(mx[0], mx[1]), fmaxf(mx[2], mx[3])),
                     fmaxf(fmaxf(mx[4], mx[5]), fmaxf(mx[6], mx[7])));
    mt = fmaxf(mt, swap32(mt));
    const float m_new = fmaxf(m_run, mt);          // finite: key0 < n is never excluded
    const float alpha = fast_exp2((m_run - m_new) * kLog2e);   // 1 when the max did not move
    m_run = m_new;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc_o[r] *= alpha;

    if (!masked_tile) {
      const float nml = -m_new * kLog2e;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[u][r] = fmaf(s[u][r], kLog2e, nml);
    } else {
      // (s - m) first: exact when both sit near -1e9
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[u][r] = (s[u][r] - m_new) * kLog2e;
    }
    float psum = 0.0f;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        s[u][r] = fast_exp2(s[u][r]);
        psum += s[u][r];
      }
    l_run = l_run * alpha + psum;

    // O^T += V^T P^T
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        f32x8 p8;
#pragma unroll
        for (int t = 0; t < 8; ++t) p8[t] = s[u][8 * c + t];
        mma32(acc_o, lds_kv[buf][4 + u * 2 + c][lane], from_f32<T>(p8));
      }
  };

  // Tile t+2 travels global -> registers -> LDS while tile t is processed; the bias tile of
  // t+1 is in flight to registers.  No load sits under a branch, so the compiler counts the
  // outstanding loads exactly.
  V8 bias_a[2][2], bias_b[2][2];
  auto step = [&](int tile, V8 (&tb_cur)[2][2], V8 (&tb_nxt)[2][2]) {
    fetch(tile + 2);
    fetch_bias(tile + 1, tb_nxt);
    process_tile(tile, tb_cur);
    stash((tile + 2) % 3);
    __syncthreads();
  };

  fetch(0);
  fetch_bias(0, bias_a);
  stash(0);
  fetch(1);
  stash(1);
  __syncthreads();
  // tiles are processed in pairs; a phantom last tile (odd tile count) is all -inf logits
  for (int tile = 0; tile < n_tiles; tile += 2) {
    step(tile, bias_a, bias_b);
    step(tile + 1, bias_b, bias_a);
  }

  // ---- normalise, gate, store: lane <-> query, register r <-> d = acc_row(r, g) ----
  // o may alias gate: every gate load is issued before the first store.
  const int64_t base = qrow + 4 * g;
  f32x4 gv[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) gv[c] = to_f32(*reinterpret_cast<const V4*>(gate + base + 8 * c));
  const float inv = fast_rcp(l_run + swap32(l_run));
  if (q0 + ln < n) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      f32x4 ov;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        // attention output rounded to T before the gate multiply, as the reference does
        ov[t] = to_f32(from_f32<T>(acc_o[4 * c + t] * inv)) * gv[c][t];
      }
      *reinterpret_cast<V4*>(o + base + 8 * c) = from_f32<T>(ov);
    }
  }
}

template <typename T>
int triattn_fwd(const T* q, const T* k, const T* vt, const T* g, const T* tri_bias, const T* mask,
                T* o, int n, int heads, int key_pitch, int mask_transposed, float inf,
                hipStream_t stream) {
  if (n == 0) return 0;
  const int n_qtiles = (n + 127) / 128;
  const int64_t total = (int64_t)heads * n * n_qtiles;
  const int64_t per_xcd = (total + 7) / 8;
  triattn_fwd_kernel<T><<<dim3((unsigned)(per_xcd * 8)), dim3(256), 0, stream>>>(
      q, k, vt, g, tri_bias, mask, o, n, heads, key_pitch, mask_transposed, inf, n_qtiles, total);
  return 0;
}

template int triattn_fwd<float>(const float*, const float*, const float*, const float*,
                                const float*, const float*, float*, int, int, int, int, float,
                                hipStream_t);
template int triattn_fwd<bf16_t>(const bf16_t*, const bf16_t*, const bf16_t*, const bf16_t*,
                                 const bf16_t*, const bf16_t*, bf16_t*, int, int, int, int, float,
                                 hipStream_t);

}  // namespace ptx
