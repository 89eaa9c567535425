// Backward of the fused attention operator on standard-layout tensors
// (the contract of tri_attention/op.py:79-163 and tri_attention/backward.py:27-609 of the
// reference): given Q (already scaled), K, V, O, dO [rows][S][H][32], Bias1 [rows][S],
// Bias2 [H][S][S] and the forward's M = log2 sum_k 2^(logit * log2 e) [rows][S][H], with
//   P = 2^(S log2 e - M),  S = Q K^T + Bias1 + Bias2,  Delta = rowsum(O * dO),
//   dS = P * (dO V^T - Delta)
// it produces  dV = P^T dO,  dK = dS^T Q,  dQ = dS K,  dBias2[h] = sum over rows of dS.
// Four kernels, as in the reference (preprocess, dK/dV, dQ, dBias2); P is recomputed, the
// logits are never stored.  One wave owns a 32 x 32 block of (query, key) pairs and walks over
// the other index; every product runs on MFMA with fp32 accumulation (conventions of
// common.h).  The register <-> index permutation of single.hip makes the recomputed P and dS
// usable as MFMA operands as they sit in the accumulators.
// What bounds these kernels is the operand stream out of L2 (6 to 8 KB per block pair when
// every wave fetches its own), so the four waves of a workgroup take neighbouring blocks and
// share the tiles that walk: the workgroup loads each tile once, one step ahead, into
// registers, parks it in LDS row-major and (for the operands a product needs with the walking
// index in the K slots: K^T for dQ, Q^T and dO^T for dK / dV) transposed, and every wave reads
// its MFMA fragments from there.
#include "common.h"
#include "kernels.h"

namespace ptx {

namespace {

constexpr float kBwdLog2e = 1.4426950408889634f;
constexpr int kTP = 40;   // pitch of the LDS tiles (elements): 16-byte aligned rows, spread over banks

struct BwdParams {
  const void *q, *k, *v, *o, *dout, *b1, *b2;
  const float* lse;
  float* delta;
  void *dq, *dk, *dv, *db2;
  int n_rows, s, heads;
};

__device__ __forceinline__ int perm_row(int m) {   // MFMA row m of a 32-block <-> index in the block
  return 16 * (m >> 4) + 8 * ((m >> 2) & 1) + 4 * ((m >> 3) & 1) + (m & 3);
}
__device__ __forceinline__ int64_t elem(const BwdParams& p, int i, int pos, int h) {
  return (((int64_t)i * p.s + pos) * p.heads + h) * 32;
}
// index (within a 32-block) that accumulator register r of half-wave g stands for
__device__ __forceinline__ int reg_index(int r, int g) { return 16 * (r >> 3) + 8 * g + (r & 7); }

template <typename T> __device__ __forceinline__ typename Vec8<T>::type zero_frag() {
  typename Vec8<T>::type z;
#pragma unroll
  for (int t = 0; t < 8; ++t) z[t] = (T)0.0f;
  return z;
}

// 8 consecutive bias values starting at key block `kb` (a multiple of 8) of a row of `s` keys,
// one vector load where rows are 8-aligned (s % 8 == 0: a block of 8 keys is then
// inside the row or outside as a whole, and an outside block is read from the row's last one;
// the caller masks it), scalar loads with clamped keys otherwise.
template <typename T>
__device__ __forceinline__ typename Vec8<T>::type load_bias8_raw(const T* row, int kb, int s,
                                                                bool vec) {
  if (vec) return load8<T>(row + min(kb, s - 8));
  typename Vec8<T>::type v;
#pragma unroll
  for (int t = 0; t < 8; ++t) v[t] = row[min(kb + t, s - 1)];
  return v;
}
template <typename T>
__device__ __forceinline__ f32x8 load_bias8(const T* row, int kb, int s, bool vec) {
  return to_f32(load_bias8_raw<T>(row, kb, s, vec));
}

}  // namespace

// Delta[i][j][h] = sum_d O * dO
template <typename T>
__global__ __launch_bounds__(256) void attn_bwd_delta_kernel(BwdParams p) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t total = (int64_t)p.n_rows * p.s * p.heads;
  if (idx >= total) return;
  const T* o = (const T*)p.o + idx * 32;
  const T* d = (const T*)p.dout + idx * 32;
  float acc = 0.0f;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const f32x8 a = to_f32(load8<T>(o + 8 * c)), b = to_f32(load8<T>(d + 8 * c));
#pragma unroll
    for (int t = 0; t < 8; ++t) acc += a[t] * b[t];
  }
  p.delta[idx] = acc;
}

// The workgroup's 256 threads load two [32 rows][32 channels] tiles (rows `pos0 ..` of tensors
// a and b at (row i, head h)): thread t takes 8 channels of one row of one tile.
template <typename T> struct TilePiece {
  typename Vec8<T>::type v;
  __device__ __forceinline__ void fetch(const BwdParams& p, const void* a, const void* b, int i,
                                        int pos0, int h, int tid) {
    const int row = min(pos0 + ((tid & 127) >> 2), p.s - 1);
    v = load8<T>((const T*)(tid >> 7 ? b : a) + elem(p, i, row, h) + 8 * (tid & 3));
  }
  // row-major into rm[tid >> 7]; with `tr`, transposed ([channel][row]) into tr[tid >> 7] as well
  __device__ __forceinline__ void park(T (*rm)[32 * kTP], T (*tr)[32 * kTP], int n_tr, int tid) const {
    const int which = tid >> 7, row = (tid & 127) >> 2, c0 = 8 * (tid & 3);
    store8<T>(&rm[which][row * kTP + c0], v);
    if (which < n_tr) {
#pragma unroll
      for (int t = 0; t < 8; ++t) tr[which][(c0 + t) * kTP + row] = v[t];
    }
  }
};

// dQ: a workgroup takes 128 queries of one (row, head), a wave 32 of them, and walks over the
// key blocks; K, V and K^T are shared.  Works on S^T: lane <-> query, register <-> key, so the
// biases arrive as 8 consecutive keys per load and the row statistics are per-lane scalars.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void attn_bwd_dq_kernel(BwdParams p) {
  typedef typename Vec8<T>::type V8;
  typedef typename Vec4<T>::type V4;
  __shared__ __attribute__((aligned(32))) T rm[2][32 * kTP];   // K, V
  __shared__ __attribute__((aligned(32))) T tr[1][32 * kTP];   // K^T
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, ln = lane & 31, g = lane >> 5;
  const int s = p.s, H = p.heads;
  constexpr bool vec = VEC;   // rows of s keys are 8-aligned
  const int h = blockIdx.y, i = blockIdx.z;
  const int q0 = (blockIdx.x * 4 + wave) * 32;
  const int qi = min(q0 + ln, s - 1);
  const bool q_ok = q0 + ln < s;
  const T* b2row = (const T*)p.b2 + ((int64_t)h * s + qi) * s;
  const T* b1row = p.b1 ? (const T*)p.b1 + (int64_t)i * s : nullptr;

  V8 qf[2], dof[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    qf[kk] = load8<T>((const T*)p.q + elem(p, i, qi, h) + 16 * kk + 8 * g);
    dof[kk] = load8<T>((const T*)p.dout + elem(p, i, qi, h) + 16 * kk + 8 * g);
  }
  const float mq = p.lse[((int64_t)i * s + qi) * H + h];
  const float dq_ = p.delta[((int64_t)i * s + qi) * H + h];
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

  TilePiece<T> piece;
  V8 b1n[2], b2n[2];
  auto fetch = [&](int key0) {
    piece.fetch(p, p.k, p.v, i, key0, h, tid);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      b2n[ks] = load_bias8_raw<T>(b2row, key0 + 16 * ks + 8 * g, s, vec);
      b1n[ks] = b1row ? load_bias8_raw<T>(b1row, key0 + 16 * ks + 8 * g, s, vec) : zero_frag<T>();
    }
  };
  fetch(0);
  for (int key0 = 0; key0 < s; key0 += 32) {
    piece.park(rm, tr, 1, tid);
    f32x8 b1f[2], b2f[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      b1f[ks] = to_f32(b1n[ks]);
      b2f[ks] = to_f32(b2n[ks]);
    }
    __syncthreads();
    if (key0 + 32 < s) fetch(key0 + 32);   // in flight while this step computes

    V8 kf[2], vf[2], ktf[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      kf[kk] = load8<T>(&rm[0][perm_row(ln) * kTP + 16 * kk + 8 * g]);
      vf[kk] = load8<T>(&rm[1][perm_row(ln) * kTP + 16 * kk + 8 * g]);
      ktf[kk] = load8<T>(&tr[0][ln * kTP + 16 * kk + 8 * g]);
    }
    f32x16 st, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) st[r] = dp[r] = 0.0f;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      mma32(st, kf[kk], qf[kk]);    // S^T[key][query]
      mma32(dp, vf[kk], dof[kk]);   // dP^T[key][query]
    }
    V8 dsf[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      f32x8 ds;
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const int r = 8 * ks + t;
        // (q.k + Bias1) + Bias2, the order of the forward
        const float x = (st[r] + b1f[ks][t]) + b2f[ks][t];
        const float pr = (key0 + reg_index(r, g) < s && q_ok) ? fast_exp2(x * kBwdLog2e - mq) : 0.0f;
        ds[t] = pr * (dp[r] - dq_);
      }
      dsf[ks] = from_f32<T>(ds);
    }
    // dQ^T[d][query] += K^T[d][key] dS^T[key][query]: lane <-> query, register <-> d
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) mma32(acc, ktf[ks], dsf[ks]);
    __syncthreads();   // every wave is done with the tiles before the next step's are parked
  }
  if (q_ok) {
    T* dst = (T*)p.dq + elem(p, i, qi, h);
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      f32x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = acc[4 * a + e];
      *reinterpret_cast<V4*>(dst + 8 * a + 4 * g) = from_f32<T>(v);
    }
  }
}

// dK and dV: a workgroup takes 128 keys of one (row, head), a wave 32 of them, and walks over
// the query blocks; Q, dO, their transposes and the queries' statistics are shared.  Works on
// S (not S^T): lane <-> key, register <-> query.  Each wave's Bias2 tile is loaded with the
// lane on the query (8 keys per load) and turned through its own LDS tile.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void attn_bwd_kv_kernel(BwdParams p) {
  typedef typename Vec8<T>::type V8;
  typedef typename Vec4<T>::type V4;
  __shared__ __attribute__((aligned(32))) T rm[2][32 * kTP];    // Q, dO
  __shared__ __attribute__((aligned(32))) T tr[2][32 * kTP];    // Q^T, dO^T
  __shared__ __attribute__((aligned(32))) T b2t[4][32 * kTP];   // per wave: Bias2 as [key][query]
  __shared__ __attribute__((aligned(32))) float stats[2][32];   // log-sum-exp, Delta of the 32 queries
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, ln = lane & 31, g = lane >> 5;
  const int s = p.s, H = p.heads;
  constexpr bool vec = VEC;
  const int h = blockIdx.y, i = blockIdx.z;
  const int key0 = (blockIdx.x * 4 + wave) * 32;
  const int kc = min(key0 + ln, s - 1);
  const bool k_ok = key0 + ln < s;
  V8 kf[2], vf[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    kf[kk] = load8<T>((const T*)p.k + elem(p, i, kc, h) + 16 * kk + 8 * g);
    vf[kk] = load8<T>((const T*)p.v + elem(p, i, kc, h) + 16 * kk + 8 * g);
  }
  const float b1v = p.b1 ? to_f32(((const T*)p.b1)[(int64_t)i * s + kc]) : 0.0f;
  const float* stat_src = g == 0 ? p.lse : p.delta;   // wave 0 fetches the statistics
  f32x16 acc_dk, acc_dv;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc_dk[r] = acc_dv[r] = 0.0f;

  TilePiece<T> piece;
  float stat = 0.0f;
  V8 b2a, b2b;   // lane (ln, g): Bias2 of query q0 + ln for keys key0 + 16 g .. + 15
  auto fetch = [&](int q0) {
    piece.fetch(p, p.q, p.dout, i, q0, h, tid);
    const int ql = min(q0 + ln, s - 1);
    if (wave == 0) stat = stat_src[((int64_t)i * s + ql) * H + h];
    const T* b2row = (const T*)p.b2 + ((int64_t)h * s + ql) * s;
    b2a = load_bias8_raw<T>(b2row, key0 + 16 * g, s, vec);
    b2b = load_bias8_raw<T>(b2row, key0 + 16 * g + 8, s, vec);
  };
  fetch(0);
  for (int q0 = 0; q0 < s; q0 += 32) {
    piece.park(rm, tr, 2, tid);
    if (wave == 0) stats[g][ln] = stat;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      b2t[wave][(16 * g + t) * kTP + ln] = b2a[t];
      b2t[wave][(16 * g + 8 + t) * kTP + ln] = b2b[t];
    }
    __syncthreads();
    if (q0 + 32 < s) fetch(q0 + 32);   // in flight while this step computes

    V8 qf[2], dof[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      qf[kk] = load8<T>(&rm[0][perm_row(ln) * kTP + 16 * kk + 8 * g]);
      dof[kk] = load8<T>(&rm[1][perm_row(ln) * kTP + 16 * kk + 8 * g]);
    }
    f32x16 sm, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) sm[r] = dp[r] = 0.0f;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      mma32(sm, qf[kk], kf[kk]);    // S[query][key]: lane <-> key, register <-> query
      mma32(dp, dof[kk], vf[kk]);   // dP[query][key]
    }
    V8 pf[2], dsf[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int qb = 16 * ks + 8 * g;   // queries q0 + qb .. + 7 sit in registers 8 ks .. 8 ks + 7
      const f32x8 lse8 = *reinterpret_cast<const f32x8*>(&stats[0][qb]);
      const f32x8 del8 = *reinterpret_cast<const f32x8*>(&stats[1][qb]);
      const f32x8 b28 = to_f32(load8<T>(&b2t[wave][ln * kTP + qb]));
      f32x8 pv, dv;
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const int r = 8 * ks + t;
        const float x = (sm[r] + b1v) + b28[t];   // (q.k + Bias1) + Bias2, the order of the forward
        const float pr = (q0 + qb + t < s && k_ok) ? fast_exp2(x * kBwdLog2e - lse8[t]) : 0.0f;
        pv[t] = pr;
        dv[t] = pr * (dp[r] - del8[t]);
      }
      pf[ks] = from_f32<T>(pv);
      dsf[ks] = from_f32<T>(dv);
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const V8 qtf = load8<T>(&tr[0][ln * kTP + 16 * ks + 8 * g]);
      const V8 dotf = load8<T>(&tr[1][ln * kTP + 16 * ks + 8 * g]);
      mma32(acc_dv, dotf, pf[ks]);    // dV^T[d][key] += dO^T[d][query] P[query][key]
      mma32(acc_dk, qtf, dsf[ks]);    // dK^T[d][key] += Q^T[d][query] dS[query][key]
    }
    __syncthreads();   // every wave is done with the tiles before the next step's are parked
  }
  if (k_ok) {
    T* dk = (T*)p.dk + elem(p, i, kc, h);
    T* dv = (T*)p.dv + elem(p, i, kc, h);
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      f32x4 x, y;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        x[e] = acc_dk[4 * a + e];
        y[e] = acc_dv[4 * a + e];
      }
      *reinterpret_cast<V4*>(dk + 8 * a + 4 * g) = from_f32<T>(x);
      *reinterpret_cast<V4*>(dv + 8 * a + 4 * g) = from_f32<T>(y);
    }
  }
}

// dBias2: a workgroup takes 64 queries x 64 keys of one head, a wave one 32 x 32 quadrant, and
// walks over the rows; the two Q / dO tiles and the two K / V tiles of a row are shared.
// Works on S^T like dQ.  Bias2 itself does not change along the walk and stays in registers.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void attn_bwd_db2_kernel(BwdParams p) {
  typedef typename Vec8<T>::type V8;
  __shared__ __attribute__((aligned(32))) T tiles[4][64 * kTP];   // Q, dO (64 queries), K, V (64 keys)
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, ln = lane & 31, g = lane >> 5;
  const int s = p.s, H = p.heads;
  constexpr bool vec = VEC;
  const int h = blockIdx.y;
  const int qs0 = blockIdx.x * 64, ks0 = blockIdx.z * 64;
  const int wq = wave >> 1, wk = wave & 1;
  const int q0 = qs0 + 32 * wq, key0 = ks0 + 32 * wk;
  const int qi = min(q0 + ln, s - 1);
  const bool q_ok = q0 + ln < s;
  const T* b2row = (const T*)p.b2 + ((int64_t)h * s + qi) * s;
  f32x8 b2f[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) b2f[ks] = load_bias8<T>(b2row, key0 + 16 * ks + 8 * g, s, vec);
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

  // thread t: 8 channels (t & 3) of row t >> 2 of each of the four 64-row tiles
  const int crow = tid >> 2, cc = 8 * (tid & 3);
  const int cq = min(qs0 + crow, s - 1), ck = min(ks0 + crow, s - 1);
  V8 piece[4], b1n[2];
  float mq_n = 0.0f, dq_n = 0.0f;
  auto fetch = [&](int i) {
    piece[0] = load8<T>((const T*)p.q + elem(p, i, cq, h) + cc);
    piece[1] = load8<T>((const T*)p.dout + elem(p, i, cq, h) + cc);
    piece[2] = load8<T>((const T*)p.k + elem(p, i, ck, h) + cc);
    piece[3] = load8<T>((const T*)p.v + elem(p, i, ck, h) + cc);
    mq_n = p.lse[((int64_t)i * s + qi) * H + h];
    dq_n = p.delta[((int64_t)i * s + qi) * H + h];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
      b1n[ks] = p.b1 ? load_bias8_raw<T>((const T*)p.b1 + (int64_t)i * s, key0 + 16 * ks + 8 * g, s, vec)
                     : zero_frag<T>();
  };
  fetch(0);
  for (int i = 0; i < p.n_rows; ++i) {
#pragma unroll
    for (int w = 0; w < 4; ++w) store8<T>(&tiles[w][crow * kTP + cc], piece[w]);
    const float mq = mq_n, dq_ = dq_n;
    f32x8 b1f[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) b1f[ks] = to_f32(b1n[ks]);
    __syncthreads();
    if (i + 1 < p.n_rows) fetch(i + 1);   // in flight while this step computes

    f32x16 st, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) st[r] = dp[r] = 0.0f;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const V8 qf = load8<T>(&tiles[0][(32 * wq + ln) * kTP + 16 * kk + 8 * g]);
      const V8 dof = load8<T>(&tiles[1][(32 * wq + ln) * kTP + 16 * kk + 8 * g]);
      const V8 kf = load8<T>(&tiles[2][(32 * wk + perm_row(ln)) * kTP + 16 * kk + 8 * g]);
      const V8 vf = load8<T>(&tiles[3][(32 * wk + perm_row(ln)) * kTP + 16 * kk + 8 * g]);
      mma32(st, kf, qf);    // S^T[key][query]
      mma32(dp, vf, dof);   // dP^T[key][query]
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float x = (st[r] + b1f[r >> 3][r & 7]) + b2f[r >> 3][r & 7];
      const float pr = (key0 + reg_index(r, g) < s && q_ok) ? fast_exp2(x * kBwdLog2e - mq) : 0.0f;
      acc[r] += pr * (dp[r] - dq_);
    }
    __syncthreads();   // every wave is done with the tiles before the next row's are parked
  }
  if (q_ok) {
    T* dst = (T*)p.db2 + ((int64_t)h * s + qi) * s;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int kb = key0 + 16 * ks + 8 * g;
      f32x8 v;
#pragma unroll
      for (int t = 0; t < 8; ++t) v[t] = acc[8 * ks + t];
      if (vec) {
        if (kb < s) store8<T>(dst + kb, from_f32<T>(v));
      } else {
#pragma unroll
        for (int t = 0; t < 8; ++t)
          if (kb + t < s) dst[kb + t] = from_f32<T>(v[t]);
      }
    }
  }
}

template <typename T>
int triattn_bwd(const void* q, const void* k, const void* v, const void* b1, const void* b2,
                const void* o, const float* lse, const void* dout, void* dq, void* dk, void* dv,
                void* db2, float* delta, int n_rows, int s, int heads, hipStream_t stream) {
  if (n_rows == 0 || s == 0 || heads == 0) return 0;
  BwdParams p = {q, k, v, o, dout, b1, b2, lse, delta, dq, dk, dv, db2, n_rows, s, heads};
  const int64_t total = (int64_t)n_rows * s * heads;
  const unsigned blocks = (unsigned)((s + 31) / 32);
  attn_bwd_delta_kernel<T><<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream>>>(p);
  const dim3 walk((blocks + 3) / 4, heads, n_rows), pairs((blocks + 1) / 2, heads, (blocks + 1) / 2);
  if ((s & 7) == 0) {
    attn_bwd_kv_kernel<T, true><<<walk, dim3(256), 0, stream>>>(p);
    attn_bwd_dq_kernel<T, true><<<walk, dim3(256), 0, stream>>>(p);
    if (db2) attn_bwd_db2_kernel<T, true><<<pairs, dim3(256), 0, stream>>>(p);
  } else {
    attn_bwd_kv_kernel<T, false><<<walk, dim3(256), 0, stream>>>(p);
    attn_bwd_dq_kernel<T, false><<<walk, dim3(256), 0, stream>>>(p);
    if (db2) attn_bwd_db2_kernel<T, false><<<pairs, dim3(256), 0, stream>>>(p);
  }
  return 0;
}

template int triattn_bwd<float>(const void*, const void*, const void*, const void*, const void*,
                                const void*, const float*, const void*, void*, void*, void*, void*,
                                float*, int, int, int, hipStream_t);
template int triattn_bwd<bf16_t>(const void*, const void*, const void*, const void*, const void*,
                                 const void*, const float*, const void*, void*, void*, void*, void*,
                                 float*, int, int, int, hipStream_t);

}  // namespace ptx
