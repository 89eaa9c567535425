// Triangle attention core: flash-style online softmax on MFMA, the N^3 logits
// are never written anywhere.
//
// One workgroup (4 waves) owns one (row i, head h) pair and 4*NQ*32 queries;
// each wave owns NQ blocks of 32 queries and walks over the keys in tiles of 64.
// Per tile and query block:
//   S^T[key][query]  = K Q^T            2 x 2 MFMA (two 32-key halves, d = 32)
//   online softmax along keys = along the registers of a lane (+ one exchange
//   with the other half-wave), because MFMA puts the query on the lane
//   O^T[d][query]   += V^T P^T          4 MFMA, P^T taken straight from the S^T
//   accumulators with no shuffle: MFMA row m of half u is mapped to key
//   32*((m>>2)&1) + 16*u + 4*(m>>3) + (m&3), which makes register r of half-wave
//   g hold key 32*g + 16*u + r, i.e. 16 consecutive keys -> 16-byte bias loads
//   and 8 consecutive keys per PV operand slot group.
// K and V^T tiles are shared by the 4 waves through LDS in fragment order
// (double-buffered, one barrier per tile); the triangle-bias tile is private to
// a wave and read straight from global (L2-resident: workgroups are numbered so
// that one XCD works on one head at a time).
//
// Mask semantics follow the reference's fp32 arithmetic exactly: on tiles that
// contain a masked (or out-of-range) key the logit is (q.k + inf*(mask-1)) +
// bias in that order, so -1e9 absorbs small logits and a fully masked row
// averages v over all keys; tiles whose keys are all unmasked take a shorter
// path with the bias preloaded into the MFMA accumulator.
#include "common.h"
#include "kernels.h"

namespace ptx {

constexpr int kD = 32;          // head dim
constexpr int kKeyTile = 64;
constexpr float kLog2e = 1.4426950408889634f;

template <typename T, int NQ>
__global__ __launch_bounds__(256) void triattn_fwd_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ vt,
    const T* gate, const T* __restrict__ bias, const T* __restrict__ mask,
    T* o, int n, int heads, int key_pitch, int mask_transposed, float inf,
    int n_qtiles, int64_t total_items) {
  typedef typename Vec8<T>::type V8;
  typedef typename Vec4<T>::type V4;
  __shared__ V8 lds_kv[2][8][kWave];     // fragments 0-3: K (u,kk); 4-7: V^T (u,s)
  __shared__ __attribute__((aligned(16))) float lds_mb[2][kKeyTile];  // additive mask bias of the tile's keys

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ln = lane & 31, g = lane >> 5;
  const int C = heads * kD;

  // Work item -> (h, i, query tile), h-major, one contiguous span per XCD
  // (workgroups are dealt round-robin to the 8 XCDs).
  const int64_t per_xcd = (total_items + 7) / 8;
  const int64_t item = (int64_t)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if ((int64_t)(blockIdx.x >> 3) >= per_xcd || item >= total_items) return;
  const int qt = (int)(item % n_qtiles);
  const int i = (int)((item / n_qtiles) % n);
  const int h = (int)(item / ((int64_t)n_qtiles * n));

  const int q0 = (qt * 4 + wave) * (NQ * 32);   // first query of this wave
  const T* q_row = q + (int64_t)i * n * C + h * kD;
  const T* k_row = k + (int64_t)i * n * C + h * kD;
  const T* vt_row = vt + ((int64_t)i * C + h * kD) * key_pitch;
  const T* bias_h = bias + (int64_t)h * n * key_pitch;

  // Q fragments (B operand): lane <-> query, slots <-> d = 16*kk + 8*g + t
  V8 qf[NQ][2];
#pragma unroll
  for (int qb = 0; qb < NQ; ++qb) {
    // queries beyond n re-read the last one; their results are never stored
    const int qi = min(q0 + qb * 32 + ln, n - 1);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) qf[qb][kk] = load8<T>(q_row + (int64_t)qi * C + 16 * kk + 8 * g);
  }

  const int n_tiles = (n + kKeyTile - 1) / kKeyTile;

  // ---- cooperative tile loader: wave w fetches fragments 2w and 2w+1 ----
  V8 pre[2];
  float pre_mb = 0.0f;
  // All loads are unconditional (indices clamped): keys beyond n get a -inf mask
  // bias below, which removes them from the softmax whatever K holds; V^T is zeroed
  // for them because 0 * garbage must stay 0.
  auto fetch = [&](int tile) {
    const int key0 = tile * kKeyTile;
    const bool tail = key0 + kKeyTile > n;   // uniform
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int fid = wave * 2 + j;
      const int u = (fid >> 1) & 1, sub = fid & 1;
      if (fid < 4) {
        // K (A operand): MFMA row m <-> key 32*((m>>2)&1) + 16u + 4*(m>>3) + (m&3); slots <-> d
        const int key = key0 + 32 * ((ln >> 2) & 1) + 16 * u + 4 * (ln >> 3) + (ln & 3);
        pre[j] = load8<T>(k_row + (int64_t)min(key, n - 1) * C + 16 * sub + 8 * g);
      } else {
        // V^T (A operand): MFMA row <-> d = ln; slots <-> keys 32g + 16u + 8s + t
        const int key = key0 + 32 * g + 16 * u + 8 * sub;
        V8 v = load8<T>(vt_row + (int64_t)ln * key_pitch + key);
        if (tail) {
#pragma unroll
          for (int t = 0; t < 8; ++t) v[t] = key + t < n ? v[t] : (T)0.0f;
        }
        pre[j] = v;
      }
    }
    if (wave == 0) {
      const int key = key0 + lane;
      const int kc = min(key, n - 1);
      float mb = 0.0f;
      if (mask) {
        const int64_t mi = mask_transposed ? (int64_t)kc * n + i : (int64_t)i * n + kc;
        mb = inf * (to_f32(mask[mi]) - 1.0f);
      }
      pre_mb = key < n ? mb : -INFINITY;
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int j = 0; j < 2; ++j) lds_kv[buf][wave * 2 + j][lane] = pre[j];
    if (wave == 0) lds_mb[buf][lane] = pre_mb;
  };

  // ---- per-wave bias tile loader: lane <-> query, 16 consecutive keys per (qb,u) ----
  V8 bias_nxt[NQ][2][16 / 8];
  auto fetch_bias = [&](int tile) {
    const int key0 = tile * kKeyTile;
#pragma unroll
    for (int qb = 0; qb < NQ; ++qb) {
      const int qi = q0 + qb * 32 + ln;
      const T* bp = bias_h + (int64_t)(qi < n ? qi : 0) * key_pitch + key0 + 32 * g;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int c = 0; c < 2; ++c) bias_nxt[qb][u][c] = load8<T>(bp + 16 * u + 8 * c);
    }
  };

  f32x16 acc_o[NQ];
  float m_run[NQ], l_run[NQ];
#pragma unroll
  for (int qb = 0; qb < NQ; ++qb) {
#pragma unroll
    for (int r = 0; r < 16; ++r) acc_o[qb][r] = 0.0f;
    m_run[qb] = -INFINITY;
    l_run[qb] = 0.0f;
  }

  fetch(0);
  fetch_bias(0);
  stash(0);
  __syncthreads();

  for (int tile = 0; tile < n_tiles; ++tile) {
    const int buf = tile & 1;
    V8 bias_cur[NQ][2][2];
#pragma unroll
    for (int qb = 0; qb < NQ; ++qb)
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int c = 0; c < 2; ++c) bias_cur[qb][u][c] = bias_nxt[qb][u][c];
    if (tile + 1 < n_tiles) {
      fetch(tile + 1);
      fetch_bias(tile + 1);
    }

    // Does this tile hold a masked or out-of-range key?  Same answer in all waves.
    const float mb_lane = lds_mb[buf][lane];
    const bool masked_tile = __ballot(mb_lane != 0.0f) != 0ull;

    V8 kf[2][2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) kf[u][kk] = lds_kv[buf][u * 2 + kk][lane];

    f32x16 s[NQ][2];
    if (!masked_tile) {
#pragma unroll
      for (int qb = 0; qb < NQ; ++qb)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
          for (int c = 0; c < 2; ++c) {
            const f32x8 b = to_f32(bias_cur[qb][u][c]);
#pragma unroll
            for (int t = 0; t < 8; ++t) s[qb][u][8 * c + t] = b[t];
          }
#pragma unroll
          for (int kk = 0; kk < 2; ++kk) mma32(s[qb][u], kf[u][kk], qf[qb][kk]);
        }
    } else {
      // exact reference order in fp32: (q.k + mask_bias) + triangle_bias
      float mb[2][16];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const f32x4 m4 = *reinterpret_cast<const f32x4*>(&lds_mb[buf][32 * g + 16 * u + 4 * c]);
#pragma unroll
          for (int t = 0; t < 4; ++t) mb[u][4 * c + t] = m4[t];
        }
#pragma unroll
      for (int qb = 0; qb < NQ; ++qb)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
          for (int r = 0; r < 16; ++r) s[qb][u][r] = 0.0f;
#pragma unroll
          for (int kk = 0; kk < 2; ++kk) mma32(s[qb][u], kf[u][kk], qf[qb][kk]);
#pragma unroll
          for (int c = 0; c < 2; ++c) {
            const f32x8 b = to_f32(bias_cur[qb][u][c]);
#pragma unroll
            for (int t = 0; t < 8; ++t) {
              const int r = 8 * c + t;
              const float v = (s[qb][u][r] + mb[u][r]) + b[t];
              s[qb][u][r] = mb[u][r] == -INFINITY ? -INFINITY : v;   // key beyond n
            }
          }
        }
    }

    // ---- online softmax over this tile's 64 keys, per query (= per lane pair) ----
    V8 pf[NQ][2][2];
#pragma unroll
    for (int qb = 0; qb < NQ; ++qb) {
      float mx = s[qb][0][0];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[qb][u][r]);
      mx = fmaxf(mx, swap32(mx));
      const float m_new = fmaxf(m_run[qb], mx);          // finite: key0 < n is never excluded
      const float alpha = fast_exp2((m_run[qb] - m_new) * kLog2e);
      m_run[qb] = m_new;
      float psum = 0.0f;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        f32x16 p;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          p[r] = fast_exp2((s[qb][u][r] - m_new) * kLog2e);
          psum += p[r];
        }
#pragma unroll
        for (int sgrp = 0; sgrp < 2; ++sgrp) {
          f32x8 p8;
#pragma unroll
          for (int t = 0; t < 8; ++t) p8[t] = p[8 * sgrp + t];
          pf[qb][u][sgrp] = from_f32<T>(p8);
        }
      }
      l_run[qb] = l_run[qb] * alpha + psum;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc_o[qb][r] *= alpha;
    }

    // ---- O^T += V^T P^T ----
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int sgrp = 0; sgrp < 2; ++sgrp) {
        const V8 vf = lds_kv[buf][4 + u * 2 + sgrp][lane];
#pragma unroll
        for (int qb = 0; qb < NQ; ++qb) mma32(acc_o[qb], vf, pf[qb][u][sgrp]);
      }

    if (tile + 1 < n_tiles) stash(buf ^ 1);
    __syncthreads();
  }

  // ---- normalise, gate, store: lane <-> query, register r <-> d = acc_row(r, g) ----
  // o may alias gate: every gate load is issued before the first store.
  f32x4 gv[NQ][4];
#pragma unroll
  for (int qb = 0; qb < NQ; ++qb) {
    const int qi = q0 + qb * 32 + ln;
    const int64_t base = ((int64_t)i * n + (qi < n ? qi : 0)) * C + h * kD + 4 * g;
#pragma unroll
    for (int c = 0; c < 4; ++c) gv[qb][c] = to_f32(*reinterpret_cast<const V4*>(gate + base + 8 * c));
  }
#pragma unroll
  for (int qb = 0; qb < NQ; ++qb) {
    const int qi = q0 + qb * 32 + ln;
    const float l_tot = l_run[qb] + swap32(l_run[qb]);
    const float inv = 1.0f / l_tot;
    if (qi < n) {
      const int64_t base = ((int64_t)i * n + qi) * C + h * kD + 4 * g;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        f32x4 ov;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          // attention output rounded to T before the gate multiply, as the reference does
          ov[t] = to_f32(from_f32<T>(acc_o[qb][4 * c + t] * inv)) * gv[qb][c][t];
        }
        *reinterpret_cast<V4*>(o + base + 8 * c) = from_f32<T>(ov);
      }
    }
  }
}

template <typename T>
int triattn_fwd(const T* q, const T* k, const T* vt, const T* g, const T* tri_bias, const T* mask,
                T* o, int n, int heads, int key_pitch, int mask_transposed, float inf,
                hipStream_t stream) {
  if (n == 0) return 0;
  // fp32 fragments are twice as wide: one query block per wave keeps registers in check;
  // bf16 uses two when the query count fills them.
  const bool two = sizeof(T) == 2 && n >= 256;
  const int q_per_wg = 4 * 32 * (two ? 2 : 1);
  const int n_qtiles = (n + q_per_wg - 1) / q_per_wg;
  const int64_t total = (int64_t)heads * n * n_qtiles;
  const int64_t per_xcd = (total + 7) / 8;
  const dim3 grid((unsigned)(per_xcd * 8)), block(256);
  if constexpr (sizeof(T) == 2) {
    if (two) {
      triattn_fwd_kernel<T, 2><<<grid, block, 0, stream>>>(q, k, vt, g, tri_bias, mask, o, n, heads,
                                                           key_pitch, mask_transposed, inf,
                                                           n_qtiles, total);
      return 0;
    }
  }
  triattn_fwd_kernel<T, 1><<<grid, block, 0, stream>>>(q, k, vt, g, tri_bias, mask, o, n, heads,
                                                       key_pitch, mask_transposed, inf, n_qtiles,
                                                       total);
  return 0;
}

template int triattn_fwd<float>(const float*, const float*, const float*, const float*,
                                const float*, const float*, float*, int, int, int, int, float,
                                hipStream_t);
template int triattn_fwd<bf16_t>(const bf16_t*, const bf16_t*, const bf16_t*, const bf16_t*,
                                 const bf16_t*, const bf16_t*, bf16_t*, int, int, int, int, float,
                                 hipStream_t);

}  // namespace ptx
