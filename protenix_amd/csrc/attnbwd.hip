// Backward of the fused attention operator on standard-layout tensors
// (the contract of tri_attention/op.py:79-163 and tri_attention/backward.py:27-609 of the
// reference): given Q (already scaled), K, V, O, dO [rows][S][H][32], Bias1 [rows][S],
// Bias2 [H][S][S] and the forward's M = log2 sum_k 2^(logit * log2 e) [rows][S][H], with
//   P = 2^(S log2 e - M),  S = Q K^T + Bias1 + Bias2,  Delta = rowsum(O * dO),
//   dS = P * (dO V^T - Delta)
// it produces  dV = P^T dO,  dK = dS^T Q,  dQ = dS K,  dBias2[h] = sum over rows of dS.
// Four kernels, as in the reference (preprocess, dK/dV, dQ, dBias2); P is recomputed, the
// logits are never stored.  One wave per 32 x 32 block of (query, key) pairs walks over the
// other index; every product runs on MFMA with fp32 accumulation (conventions of common.h).
// The register <-> index permutation of single.hip makes the recomputed P and dS usable as
// MFMA operands as they sit in the accumulators; the transposed operands (K^T for dQ, Q^T and
// dO^T for dK / dV) go through a per-wave LDS tile.  Written for correctness and a sane
// memory pattern, not tuned: the inference path never runs it.
#include "common.h"
#include "kernels.h"

namespace ptx {

namespace {

constexpr float kBwdLog2e = 1.4426950408889634f;
constexpr int kTP = 40;   // pitch of the LDS transpose tiles (elements): 16-byte aligned rows

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

// A 32 x 32 block held as row fragments (lane (m, g): row perm_row(m), channels 16*kk + 8*g + t)
// written to an LDS tile as its transpose [channel][row], then read back as fragments of the
// transpose: lane <-> channel, slots <-> rows 16*ks + 8*g + t.
template <typename T>
__device__ __forceinline__ void transpose_frags(T* tile, const typename Vec8<T>::type (&in)[2],
                                                typename Vec8<T>::type (&out)[2], int lane) {
  const int m = lane & 31, g = lane >> 5, row = perm_row(m);
  __syncthreads();
#pragma unroll
  for (int kk = 0; kk < 2; ++kk)
#pragma unroll
    for (int t = 0; t < 8; ++t) tile[(16 * kk + 8 * g + t) * kTP + row] = in[kk][t];
  __syncthreads();
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) out[ks] = load8<T>(tile + m * kTP + 16 * ks + 8 * g);
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

// MODE 0: dQ (block = 32 queries of one (row, head), loop over key blocks)
// MODE 1: dBias2 (block = 32 queries x 32 keys of one head, loop over rows)
// Both work on S^T: lane <-> query, accumulator register <-> key.  Global-memory instructions
// are what this kernel pays for, so everything a lane needs of the biases arrives as 8
// consecutive keys per load, and whatever does not change along the loop is loaded once.
template <typename T, int MODE, bool VEC>
__global__ __launch_bounds__(64) void attn_bwd_q_kernel(BwdParams p) {
  typedef typename Vec8<T>::type V8;
  typedef typename Vec4<T>::type V4;
  __shared__ __attribute__((aligned(32))) T tile[32 * kTP];
  const int lane = threadIdx.x & 63, ln = lane & 31, g = lane >> 5;
  const int s = p.s, H = p.heads;
  constexpr bool vec = VEC;   // rows of s keys are 8-aligned
  const int h = blockIdx.y;
  const int q0 = blockIdx.x * 32;
  const int qi = min(q0 + ln, s - 1);
  const bool q_ok = q0 + ln < s;
  const T* b2row = (const T*)p.b2 + ((int64_t)h * s + qi) * s;

  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

  // What one step reads from global memory, fetched one step ahead.  MODE 0 walks over key
  // blocks (K, V, both biases change; the query side is loaded once), MODE 1 over rows (K, V,
  // Bias1 and the query side change; Bias2 is loaded once).
  struct Step {
    V8 kf[2], vf[2], b1v[2], b2v[2], qf[2], dof[2];
    float mq, dq_;
  };
  Step cur, nxt;
  auto load_query_side = [&](Step& o, int i) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      o.qf[kk] = load8<T>((const T*)p.q + elem(p, i, qi, h) + 16 * kk + 8 * g);
      o.dof[kk] = load8<T>((const T*)p.dout + elem(p, i, qi, h) + 16 * kk + 8 * g);
    }
    o.mq = p.lse[((int64_t)i * s + qi) * H + h];
    o.dq_ = p.delta[((int64_t)i * s + qi) * H + h];
  };
  auto load_bias2 = [&](Step& o, int key0) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) o.b2v[ks] = load_bias8_raw<T>(b2row, key0 + 16 * ks + 8 * g, s, vec);
  };
  auto fetch = [&](Step& o, int it) {
    const int i = MODE == 0 ? (int)blockIdx.z : it;
    const int key0 = MODE == 0 ? it * 32 : (int)blockIdx.z * 32;
    const int krow = min(key0 + perm_row(ln), s - 1);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      o.kf[kk] = load8<T>((const T*)p.k + elem(p, i, krow, h) + 16 * kk + 8 * g);
      o.vf[kk] = load8<T>((const T*)p.v + elem(p, i, krow, h) + 16 * kk + 8 * g);
    }
    if (MODE == 0) load_bias2(o, key0);
    else load_query_side(o, i);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
      o.b1v[ks] = p.b1 ? load_bias8_raw<T>((const T*)p.b1 + (int64_t)i * s, key0 + 16 * ks + 8 * g, s, vec)
                       : zero_frag<T>();
  };
  if (MODE == 0) load_query_side(nxt, blockIdx.z);
  else load_bias2(nxt, blockIdx.z * 32);
  fetch(nxt, 0);

  const int n_outer = MODE == 0 ? (s + 31) / 32 : p.n_rows;
  for (int it = 0; it < n_outer; ++it) {
    const int key0 = MODE == 0 ? it * 32 : (int)blockIdx.z * 32;
    cur = nxt;
    if (it + 1 < n_outer) fetch(nxt, it + 1);
    const V8 (&kf)[2] = cur.kf, (&vf)[2] = cur.vf, (&qf)[2] = cur.qf, (&dof)[2] = cur.dof;
    const float mq = cur.mq, dq_ = cur.dq_;
    f32x8 b1f[2], b2f[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      b1f[ks] = to_f32(cur.b1v[ks]);
      b2f[ks] = to_f32(cur.b2v[ks]);
    }
    f32x16 st, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) st[r] = dp[r] = 0.0f;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      mma32(st, kf[kk], qf[kk]);    // S^T[key][query]
      mma32(dp, vf[kk], dof[kk]);   // dP^T[key][query]
    }
    float ds[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = key0 + reg_index(r, g);
      // (q.k + Bias1) + Bias2, the order of the forward
      const float x = (st[r] + b1f[r >> 3][r & 7]) + b2f[r >> 3][r & 7];
      const float pr = (key < s && q_ok) ? fast_exp2(x * kBwdLog2e - mq) : 0.0f;
      ds[r] = pr * (dp[r] - dq_);
    }
    if (MODE == 1) {
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] += ds[r];
    } else {
      // dQ^T[d][query] += K^T[d][key] dS^T[key][query]
      V8 dsf[2], ktf[2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        f32x8 v;
#pragma unroll
        for (int t = 0; t < 8; ++t) v[t] = ds[8 * ks + t];
        dsf[ks] = from_f32<T>(v);
      }
      transpose_frags<T>(tile, kf, ktf, lane);
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) mma32(acc, ktf[ks], dsf[ks]);   // lane <-> query, register <-> d
    }
  }

  if (MODE == 0) {
    if (q_ok) {
      T* dst = (T*)p.dq + elem(p, blockIdx.z, qi, h);
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        f32x4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[4 * a + e];
        *reinterpret_cast<V4*>(dst + 8 * a + 4 * g) = from_f32<T>(v);
      }
    }
  } else {
    if (q_ok) {
      T* dst = (T*)p.db2 + ((int64_t)h * s + qi) * s;
      const int key0 = blockIdx.z * 32;
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
}

// dK and dV: block = 32 keys of one (row, head), loop over query blocks.  Works on S (not S^T):
// lane <-> key, accumulator register <-> query.  The per-query statistics (log-sum-exp, Delta)
// and the Bias2 tile are loaded with the lane on the query and turned through LDS, which costs
// a handful of global-memory instructions per step instead of three per accumulator register.
template <typename T, bool VEC>
__global__ __launch_bounds__(64) void attn_bwd_kv_kernel(BwdParams p) {
  typedef typename Vec8<T>::type V8;
  typedef typename Vec4<T>::type V4;
  __shared__ __attribute__((aligned(32))) T tile[3][32 * kTP];
  __shared__ __attribute__((aligned(32))) float stats[2][32];
  const int lane = threadIdx.x & 63, ln = lane & 31, g = lane >> 5;
  const int s = p.s, H = p.heads;
  constexpr bool vec = VEC;   // rows of s keys are 8-aligned
  const int h = blockIdx.y, i = blockIdx.z;
  const int key0 = blockIdx.x * 32;
  const int kc = min(key0 + ln, s - 1);
  const bool k_ok = key0 + ln < s;
  V8 kf[2], vf[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    kf[kk] = load8<T>((const T*)p.k + elem(p, i, kc, h) + 16 * kk + 8 * g);
    vf[kk] = load8<T>((const T*)p.v + elem(p, i, kc, h) + 16 * kk + 8 * g);
  }
  const float b1v = p.b1 ? to_f32(((const T*)p.b1)[(int64_t)i * s + kc]) : 0.0f;
  const float* stat_src = g == 0 ? p.lse : p.delta;
  f32x16 acc_dk, acc_dv;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc_dk[r] = acc_dv[r] = 0.0f;

  // operands of one step, loaded one step ahead: lane (ln, g) takes its A fragments of Q and dO,
  // statistic g of query q0 + ln, and Bias2 of that query for keys 16 g .. 16 g + 15
  V8 qf[2], dof[2], qf_n[2], dof_n[2];
  float stat = 0.0f, stat_n = 0.0f;
  V8 b2a, b2b, b2a_n, b2b_n;
  auto fetch = [&](int q0, V8 (&qx)[2], V8 (&dx)[2], float& st, V8& ba, V8& bb) {
    const int qrow = min(q0 + perm_row(ln), s - 1);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      qx[kk] = load8<T>((const T*)p.q + elem(p, i, qrow, h) + 16 * kk + 8 * g);
      dx[kk] = load8<T>((const T*)p.dout + elem(p, i, qrow, h) + 16 * kk + 8 * g);
    }
    const int ql = min(q0 + ln, s - 1);
    st = stat_src[((int64_t)i * s + ql) * H + h];
    const T* b2row = (const T*)p.b2 + ((int64_t)h * s + ql) * s;
    ba = load_bias8_raw<T>(b2row, key0 + 16 * g, s, vec);
    bb = load_bias8_raw<T>(b2row, key0 + 16 * g + 8, s, vec);
  };
  fetch(0, qf_n, dof_n, stat_n, b2a_n, b2b_n);

  for (int q0 = 0; q0 < s; q0 += 32) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      qf[kk] = qf_n[kk];
      dof[kk] = dof_n[kk];
    }
    stat = stat_n;
    b2a = b2a_n;
    b2b = b2b_n;
    if (q0 + 32 < s) fetch(q0 + 32, qf_n, dof_n, stat_n, b2a_n, b2b_n);

    __syncthreads();   // the previous step's reads of the tiles are done
    stats[g][ln] = stat;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      tile[2][(16 * g + t) * kTP + ln] = b2a[t];
      tile[2][(16 * g + 8 + t) * kTP + ln] = b2b[t];
    }
    {
      const int row = perm_row(ln);
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          tile[0][(16 * kk + 8 * g + t) * kTP + row] = qf[kk][t];
          tile[1][(16 * kk + 8 * g + t) * kTP + row] = dof[kk][t];
        }
    }
    __syncthreads();

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
      const f32x8 b28 = to_f32(load8<T>(&tile[2][ln * kTP + qb]));
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
    V8 qtf[2], dotf[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      qtf[ks] = load8<T>(&tile[0][ln * kTP + 16 * ks + 8 * g]);
      dotf[ks] = load8<T>(&tile[1][ln * kTP + 16 * ks + 8 * g]);
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      mma32(acc_dv, dotf[ks], pf[ks]);    // dV^T[d][key] += dO^T[d][query] P[query][key]
      mma32(acc_dk, qtf[ks], dsf[ks]);    // dK^T[d][key] += Q^T[d][query] dS[query][key]
    }
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

template <typename T>
int triattn_bwd(const void* q, const void* k, const void* v, const void* b1, const void* b2,
                const void* o, const float* lse, const void* dout, void* dq, void* dk, void* dv,
                void* db2, float* delta, int n_rows, int s, int heads, hipStream_t stream) {
  if (n_rows == 0 || s == 0 || heads == 0) return 0;
  BwdParams p = {q, k, v, o, dout, b1, b2, lse, delta, dq, dk, dv, db2, n_rows, s, heads};
  const int64_t total = (int64_t)n_rows * s * heads;
  const unsigned blocks = (unsigned)((s + 31) / 32);
  attn_bwd_delta_kernel<T><<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream>>>(p);
  if ((s & 7) == 0) {
    attn_bwd_kv_kernel<T, true><<<dim3(blocks, heads, n_rows), dim3(64), 0, stream>>>(p);
    attn_bwd_q_kernel<T, 0, true><<<dim3(blocks, heads, n_rows), dim3(64), 0, stream>>>(p);
    if (db2) attn_bwd_q_kernel<T, 1, true><<<dim3(blocks, heads, blocks), dim3(64), 0, stream>>>(p);
  } else {
    attn_bwd_kv_kernel<T, false><<<dim3(blocks, heads, n_rows), dim3(64), 0, stream>>>(p);
    attn_bwd_q_kernel<T, 0, false><<<dim3(blocks, heads, n_rows), dim3(64), 0, stream>>>(p);
    if (db2) attn_bwd_q_kernel<T, 1, false><<<dim3(blocks, heads, blocks), dim3(64), 0, stream>>>(p);
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
