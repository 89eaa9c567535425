// Backward of the fused attention operator on standard-layout tensors
// (the contract of tri_attention/op.py:79-163 and tri_attention/backward.py:27-609 of the
// reference): given Q (already scaled), K, V, O, dO [rows][S][H][32], Bias1 [rows][S],
// Bias2 [H][S][S] and the forward's M = log2 sum_k 2^(logit * log2 e) [rows][S][H], with
//   P = 2^(S log2 e - M),  S = Q K^T + Bias1 + Bias2,  Delta = rowsum(O * dO),
//   dS = P * (dO V^T - Delta)
// it produces  dV = P^T dO,  dK = dS^T Q,  dQ = dS K,  dBias2[h] = sum over rows of dS.
// Three kernels - dQ, which also forms Delta (the reference's preprocess kernel) and leaves it
// for the others, dK/dV, dBias2 - where the reference has four; P is recomputed, the
// logits are never stored.  One wave owns a 32 x 32 block of (query, key) pairs and walks over
// the other index; every product runs on MFMA with fp32 accumulation (conventions of
// common.h).  The register <-> index permutation of single.hip makes the recomputed P and dS
// usable as MFMA operands as they sit in the accumulators.
// What bounds these kernels is the operand stream out of L2 (6 to 8 KB per block pair when
// every wave fetches its own) and the cache lines each load touches, so the four waves of a
// workgroup take neighbouring blocks and share the tiles that walk: the workgroup loads each
// tile once, one step ahead, into registers, parks it in LDS row-major, and every wave reads
// its MFMA fragments from there - also those a product needs with the walking index in the K
// slots (K^T for dQ, Q^T and dO^T for dK / dV), which 16-bit tiles give through the
// transposing LDS load and fp32 tiles through a transposed copy.
#include <type_traits>
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

// 16-bit kernels double-buffer their shared tiles (one barrier a step) and are held to the
// registers of three waves per SIMD where rows are 8-aligned; fp32 tiles are twice as
// large and stay single-buffered (two barriers a step).
template <typename T, bool VEC> struct BwdCfg {
  static constexpr int kBuffers = sizeof(T) == 2 ? 2 : 1;
  // (the second argument of __launch_bounds__: waves per SIMD the register budget allows for)
  static constexpr int kMinWaves = sizeof(T) == 2 ? (VEC ? 3 : 2) : 1;
};

// 16-bit tiles are parked in LDS row-major only; an operand that a product needs with the
// tile's rows in the K slots is read with the transposing LDS load of gfx950
// (ds_read_b64_tr_b16: the 16 lanes of a block hand in the addresses of 4 x 16 elements, 4
// lanes per row, and lane j of the block gets column j of the 4 rows).  Two of them: the lane
// gets column col0 + lane % 16 of rows row0 .. row0 + 7.  fp32 has no such load and keeps
// transposed copies of its tiles.
template <typename T> struct Turned {
  static constexpr bool value = sizeof(T) == 2;
};
__device__ __forceinline__ bf16x8 load8_turned(const bf16_t* tile, int pitch, int row0, int col0, int lane) {
  typedef short v4s __attribute__((ext_vector_type(4)));
  typedef short v8s __attribute__((ext_vector_type(8)));
  typedef __attribute__((address_space(3))) v4s* LdsV4;
  const int i = lane & 15;
  const bf16_t* a = tile + (row0 + (i >> 2)) * pitch + col0 + 4 * (i & 3);
  const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsV4)a);
  const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsV4)(a + 4 * pitch));
  return __builtin_bit_cast(bf16x8, (v8s)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}
__device__ __forceinline__ f32x8 load8_turned(const float*, int, int, int, int) { return f32x8{}; }   // (never called)

// The workgroup's 256 threads load two [32 rows][32 channels] tiles (rows `pos0 ..` of tensors
// a and b at (row i, head h)): thread t takes 8 channels of one row of one tile.
template <typename T> struct TilePiece {
  typename Vec8<T>::type v;
  __device__ __forceinline__ void fetch(const BwdParams& p, const void* a, const void* b, int i,
                                        int pos0, int h, int tid) {
    const int row = min(pos0 + ((tid & 127) >> 2), p.s - 1);
    v = load8<T>((const T*)(tid >> 7 ? b : a) + elem(p, i, row, h) + 8 * (tid & 3));
  }
  // row-major into rm[tid >> 7]; the first n_tr tiles also transposed ([channel][row]) into
  // tr + (tid >> 7) * 32 * kTP
  __device__ __forceinline__ void park(T (*rm)[32 * kTP], T* tr, int n_tr, int tid) const {
    const int which = tid >> 7, row = (tid & 127) >> 2, c0 = 8 * (tid & 3);
    store8<T>(&rm[which][row * kTP + c0], v);
    if (which < n_tr) {
#pragma unroll
      for (int t = 0; t < 8; ++t) tr[which * 32 * kTP + (c0 + t) * kTP + row] = v[t];
    }
  }
};

// dQ: a workgroup takes 128 queries of one (row, head), a wave 32 of them, and walks over the
// key blocks; K, V and K^T are shared.  Works on S^T: lane <-> query, register <-> key, so the
// biases arrive as 8 consecutive keys per load and the row statistics are per-lane scalars.
// The biases are the initial value of the S^T accumulator and -Delta that of dP^T, so that a
// logit costs one multiply-add, one exponential and one multiply.  Lanes whose query lies
// beyond s repeat query s - 1 and store nothing; keys beyond s exist in the last block only,
// which has its own copy of the step.  The shared tiles are double-buffered: one barrier a step.
template <typename T, bool VEC>
__global__ __launch_bounds__(256, (BwdCfg<T, VEC>::kMinWaves)) void attn_bwd_dq_kernel(BwdParams p) {
  typedef typename Vec8<T>::type V8;
  typedef typename Vec4<T>::type V4;
  constexpr int NB = BwdCfg<T, VEC>::kBuffers;
  __shared__ __attribute__((aligned(32))) T rm[NB][2][32 * kTP];   // K, V
  constexpr bool TURN = Turned<T>::value;
  __shared__ __attribute__((aligned(32))) T tr[TURN ? 8 : NB * 32 * kTP];   // K^T (fp32 only)
  __shared__ __attribute__((aligned(32))) T b2s[NB][128 * kTP];    // Bias2 of the 128 queries x 32 keys
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, ln = lane & 31, g = lane >> 5;
  const int s = p.s, H = p.heads;
  constexpr bool vec = VEC;   // rows of s keys are 8-aligned
  const int h = blockIdx.y, i = blockIdx.z;
  const int q0 = (blockIdx.x * 4 + wave) * 32;
  const int qi = min(q0 + ln, s - 1);
  const bool q_ok = q0 + ln < s;
  // (without a Bias1 the loads go to a row of Bias2 and count for nothing: a load under a
  // branch would make every wait for memory a wait for all of it)
  const T* b1row = p.b1 ? (const T*)p.b1 + (int64_t)i * s : (const T*)p.b2 + (int64_t)h * s * s;
  const float b1on = p.b1 ? 1.0f : 0.0f;
  // 16-bit: the biases reach the S^T accumulator on the matrix pipe, which these kernels leave
  // idle four fifths of the time, instead of being converted and added on the vector ALU:
  //   Bias2  S^T += E * B2, B2 the block's [key][query] values as they lie in LDS for this
  //          lane's query (B operand: slots <-> keys), E the 0/1 matrix that sends key j to
  //          the accumulator row that stands for it (row m <-> key perm_row(m));
  //   Bias1  S^T += b * 1^T: Bias1 of the row's key in K slot 0 of one more product, against
  //          a B operand with 1 in that slot (0 without a Bias1).  Products with 1 are exact.
  constexpr bool MMB = sizeof(T) == 2;
  V8 e_frag[2], one_frag;
#pragma unroll
  for (int kk = 0; kk < 2; ++kk)
#pragma unroll
    for (int t = 0; t < 8; ++t) e_frag[kk][t] = (T)(perm_row(ln) == 16 * kk + 8 * g + t ? 1.0f : 0.0f);
#pragma unroll
  for (int t = 0; t < 8; ++t) one_frag[t] = (T)(t == 0 && g == 0 ? b1on : 0.0f);

  V8 qf[2], dof[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    qf[kk] = load8<T>((const T*)p.q + elem(p, i, qi, h) + 16 * kk + 8 * g);
    dof[kk] = load8<T>((const T*)p.dout + elem(p, i, qi, h) + 16 * kk + 8 * g);
  }
  const float neg_mq = -p.lse[((int64_t)i * s + qi) * H + h];
  // Delta = sum_d O * dO of this lane's query, formed here (the lane holds half of the query's
  // channels, the other half-wave the rest) and left in p.delta for the two kernels that follow
  float delta = 0.0f;
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    const f32x8 of = to_f32(load8<T>((const T*)p.o + elem(p, i, qi, h) + 16 * kk + 8 * g));
    const f32x8 df = to_f32(dof[kk]);
#pragma unroll
    for (int t = 0; t < 8; ++t) delta += of[t] * df[t];
  }
  delta += swap32(delta);
  if (g == 0 && q_ok) p.delta[((int64_t)i * s + qi) * H + h] = delta;
  const float neg_dq = -delta;
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

  // Bias2 comes in through LDS like the tiles: four neighbouring lanes read the 64 bytes a
  // query's row has for the block (a lane reading 16 bytes of its own query's row touches as
  // many cache lines per load as it has lanes, and the texture path was busy 96 % of the time).
  TilePiece<T> piece;
  V8 b1n[2], b2n[2];
  T b1m = (T)0.0f;   // (16-bit) Bias1 of key perm_row(ln) of the block
  const int b2col = 8 * (tid & 3);
  const T* b2rows[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
    b2rows[j] = (const T*)p.b2 + ((int64_t)h * s + min((int)blockIdx.x * 128 + 64 * j + (tid >> 2), s - 1)) * s;
  // (the compiler barriers keep the loads where they are written, a step ahead of their use:
  // left alone, the compiler moves them down to the use and waits there)
  auto fetch = [&](int key0) {
    piece.fetch(p, p.k, p.v, i, key0, h, tid);
#pragma unroll
    for (int j = 0; j < 2; ++j) b2n[j] = load_bias8_raw<T>(b2rows[j], key0 + b2col, s, vec);
    asm volatile("" ::: "memory");
  };
  auto park = [&](int buf) {
    piece.park(rm[buf], tr + (TURN ? 0 : buf * 32 * kTP), TURN ? 0 : 1, tid);
#pragma unroll
    for (int j = 0; j < 2; ++j) store8<T>(&b2s[buf][(64 * j + (tid >> 2)) * kTP + b2col], b2n[j]);
  };
  auto fetch_bias = [&](int key0) {
    if (MMB) {
      b1m = b1row[min(key0 + perm_row(ln), s - 1)];
    } else {
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) b1n[ks] = load_bias8_raw<T>(b1row, key0 + 16 * ks + 8 * g, s, vec);
    }
    asm volatile("" ::: "memory");
  };
  // one block of 32 keys out of buffer `buf`; TAIL: the block holds keys beyond s.  The biases
  // of the next block are requested as soon as this block's sit in the accumulator.
  auto step = [&](auto tail_tag, int buf, int key0, int next_key0) {
    constexpr bool TAIL = decltype(tail_tag)::value;
    V8 kf[2], vf[2], ktf[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      kf[kk] = load8<T>(&rm[buf][0][perm_row(ln) * kTP + 16 * kk + 8 * g]);
      vf[kk] = load8<T>(&rm[buf][1][perm_row(ln) * kTP + 16 * kk + 8 * g]);
      ktf[kk] = TURN ? load8_turned(rm[buf][0], kTP, 16 * kk + 8 * g, 16 * ((lane >> 4) & 1), lane)
                     : load8<T>(&tr[TURN ? 0 : buf * 32 * kTP + ln * kTP + 16 * kk + 8 * g]);
    }
    f32x16 st, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) dp[r] = neg_dq;
    if constexpr (MMB) {
      V8 b1a;
#pragma unroll
      for (int t = 0; t < 8; ++t) b1a[t] = (T)0.0f;
      b1a[0] = (g == 0 && b1on != 0.0f) ? b1m : (T)0.0f;
      V8 b2v[2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) b2v[ks] = load8<T>(&b2s[buf][(32 * wave + ln) * kTP + 16 * ks + 8 * g]);
      fetch_bias(next_key0);
#pragma unroll
      for (int r = 0; r < 16; ++r) st[r] = 0.0f;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) mma32(st, kf[kk], qf[kk]);      // S^T[key][query]
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) mma32(st, e_frag[kk], b2v[kk]);  // + Bias2
      mma32(st, b1a, one_frag);                                        // + Bias1
    } else {
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const f32x8 b1f = to_f32(b1n[ks]);
        const f32x8 b2f = to_f32(load8<T>(&b2s[buf][(32 * wave + ln) * kTP + 16 * ks + 8 * g]));
#pragma unroll
        for (int t = 0; t < 8; ++t) st[8 * ks + t] = b1f[t] * b1on + b2f[t];
      }
      fetch_bias(next_key0);
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) mma32(st, kf[kk], qf[kk]);    // S^T[key][query] (+ biases)
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) mma32(dp, vf[kk], dof[kk]);   // dP^T[key][query] - Delta
    V8 dsf[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      f32x8 ds;
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const int r = 8 * ks + t;
        float pr = fast_exp2(st[r] * kBwdLog2e + neg_mq);
        if (TAIL) pr = key0 + reg_index(r, g) < s ? pr : 0.0f;
        ds[t] = pr * dp[r];
      }
      dsf[ks] = from_f32<T>(ds);
    }
    // dQ^T[d][query] += K^T[d][key] dS^T[key][query]: lane <-> query, register <-> d
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) mma32(acc, ktf[ks], dsf[ks]);
  };

  // Block t is computed out of buffer t & 1 while block t + 1 waits in registers (fetched a
  // step earlier) and is parked into the other buffer, which every wave has left at the
  // barrier that ended step t - 1.
  const int n_steps = (s + 31) >> 5;
  const int n_full = s >> 5;
  fetch(0);
  fetch_bias(0);
  park(0);
  __syncthreads();
  fetch(min(1, n_steps - 1) * 32);
  for (int t = 0; t < n_full; ++t) {
    step(std::false_type{}, t % NB, t * 32, min(t + 1, n_steps - 1) * 32);
    if (NB == 1) __syncthreads();
    park((t + 1) % NB);
    __syncthreads();
    fetch(min(t + 2, n_steps - 1) * 32);
  }
  if (n_full < n_steps) step(std::true_type{}, n_full % NB, n_full * 32, n_full * 32);
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
// S (not S^T): lane <-> key, register <-> query.  Bias2 is loaded along the queries' rows (8
// keys per load) and turned on its way through LDS; with Bias1 added it is the initial value
// of the S accumulator, -Delta that of dP.  Lanes whose key lies beyond s
// repeat key s - 1 and store nothing; queries beyond s exist in the last block only, which has
// its own copy of the step.  Everything shared is double-buffered: one barrier a step.
template <typename T, bool VEC>
__global__ __launch_bounds__(256, (BwdCfg<T, VEC>::kMinWaves)) void attn_bwd_kv_kernel(BwdParams p) {
  typedef typename Vec8<T>::type V8;
  typedef typename Vec4<T>::type V4;
  constexpr int NB = BwdCfg<T, VEC>::kBuffers;
  __shared__ __attribute__((aligned(32))) T rm[NB][2][32 * kTP];    // Q, dO
  constexpr bool TURN = Turned<T>::value;
  __shared__ __attribute__((aligned(32))) T tr[TURN ? 8 : NB * 2 * 32 * kTP];   // Q^T, dO^T (fp32 only)
  // Bias2 of the step: fp32 per wave as [key][query]; 16-bit one tile [query][128 keys] for
  // the workgroup, as it was loaded
  constexpr int kB2P = 136;   // pitch of the 16-bit tile (elements)
  __shared__ __attribute__((aligned(32))) T b2t[NB][TURN ? 32 * kB2P : 4 * 32 * kTP];
  __shared__ __attribute__((aligned(32))) float stats[NB][2][32];   // -log-sum-exp, -Delta of the 32 queries
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
  const float* stat_src = g == 0 ? p.lse : p.delta;   // every wave fetches, wave 0 publishes
  f32x16 acc_dk, acc_dv;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc_dk[r] = acc_dv[r] = 0.0f;

  TilePiece<T> piece;
  float stat = 0.0f;
  // fp32: lane (ln, g) loads Bias2 of query q0 + ln for this wave's keys key0 + 16 g .. + 15.
  // 16-bit: thread t loads keys 8 (t & 7) .. + 7 of both halves of the workgroup's 128 keys for
  // query q0 + (t >> 3): eight neighbouring lanes read one 128-byte line (a lane per query
  // touches as many lines per load as it has lanes).
  V8 b2a, b2b;
  const int b2q = TURN ? tid >> 3 : ln;
  const int b2k = TURN ? (int)blockIdx.x * 128 + 8 * (tid & 7) : key0 + 16 * g;
  auto fetch = [&](int q0) {
    piece.fetch(p, p.q, p.dout, i, q0, h, tid);
    stat = stat_src[((int64_t)i * s + min(q0 + ln, s - 1)) * H + h];
    const T* b2row = (const T*)p.b2 + ((int64_t)h * s + min(q0 + b2q, s - 1)) * s;
    b2a = load_bias8_raw<T>(b2row, b2k, s, vec);
    b2b = load_bias8_raw<T>(b2row, b2k + (TURN ? 64 : 8), s, vec);
    asm volatile("" ::: "memory");   // the loads are issued here, a step ahead of their use
  };
  auto park = [&](int buf) {
    piece.park(rm[buf], tr + (TURN ? 0 : buf * 2 * 32 * kTP), TURN ? 0 : 2, tid);
    if (wave == 0) stats[buf][g][ln] = -stat;
    if (TURN) {
      store8<T>(&b2t[buf][b2q * kB2P + 8 * (tid & 7)], b2a);
      store8<T>(&b2t[buf][b2q * kB2P + 8 * (tid & 7) + 64], b2b);
    } else {
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        b2t[buf][wave * 32 * kTP + (16 * g + t) * kTP + ln] = b2a[t];
        b2t[buf][wave * 32 * kTP + (16 * g + 8 + t) * kTP + ln] = b2b[t];
      }
    }
  };
  // one block of 32 queries out of buffer `buf`; TAIL: the block holds queries beyond s
  auto step = [&](auto tail_tag, int buf, int q0) {
    constexpr bool TAIL = decltype(tail_tag)::value;
    V8 qf[2], dof[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      qf[kk] = load8<T>(&rm[buf][0][perm_row(ln) * kTP + 16 * kk + 8 * g]);
      dof[kk] = load8<T>(&rm[buf][1][perm_row(ln) * kTP + 16 * kk + 8 * g]);
    }
    f32x16 sm, dp;
    f32x8 nlse[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int qb = 16 * ks + 8 * g;   // queries q0 + qb .. + 7 sit in registers 8 ks .. 8 ks + 7
      nlse[ks] = *reinterpret_cast<const f32x8*>(&stats[buf][0][qb]);
      const f32x8 ndel = *reinterpret_cast<const f32x8*>(&stats[buf][1][qb]);
      const f32x8 b28 = to_f32(TURN ? load8_turned(b2t[buf], kB2P, qb, 32 * wave + 16 * ((lane >> 4) & 1), lane)
                                    : load8<T>(&b2t[buf][wave * 32 * kTP + ln * kTP + qb]));
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        sm[8 * ks + t] = b1v + b28[t];
        dp[8 * ks + t] = ndel[t];
      }
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      mma32(sm, qf[kk], kf[kk]);    // S[query][key] (+ biases): lane <-> key, register <-> query
      mma32(dp, dof[kk], vf[kk]);   // dP[query][key] - Delta
    }
    V8 pf[2], dsf[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int qb = 16 * ks + 8 * g;
      f32x8 pv, dv;
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const int r = 8 * ks + t;
        float pr = fast_exp2(sm[r] * kBwdLog2e + nlse[ks][t]);
        if (TAIL) pr = q0 + qb + t < s ? pr : 0.0f;
        pv[t] = pr;
        dv[t] = pr * dp[r];
      }
      pf[ks] = from_f32<T>(pv);
      dsf[ks] = from_f32<T>(dv);
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const V8 qtf = TURN ? load8_turned(rm[buf][0], kTP, 16 * ks + 8 * g, 16 * ((lane >> 4) & 1), lane)
                          : load8<T>(&tr[TURN ? 0 : (buf * 2 + 0) * 32 * kTP + ln * kTP + 16 * ks + 8 * g]);
      const V8 dotf = TURN ? load8_turned(rm[buf][1], kTP, 16 * ks + 8 * g, 16 * ((lane >> 4) & 1), lane)
                           : load8<T>(&tr[TURN ? 0 : (buf * 2 + 1) * 32 * kTP + ln * kTP + 16 * ks + 8 * g]);
      mma32(acc_dv, dotf, pf[ks]);    // dV^T[d][key] += dO^T[d][query] P[query][key]
      mma32(acc_dk, qtf, dsf[ks]);    // dK^T[d][key] += Q^T[d][query] dS[query][key]
    }
  };

  // Block t is computed out of buffer t & 1 while block t + 1 waits in registers (fetched a
  // step earlier) and is parked into the other buffer, which every wave has left at the
  // barrier that ended step t - 1.
  const int n_steps = (s + 31) >> 5;
  const int n_full = s >> 5;
  fetch(0);
  park(0);
  __syncthreads();
  fetch(min(1, n_steps - 1) * 32);
  for (int t = 0; t < n_full; ++t) {
    step(std::false_type{}, t % NB, t * 32);
    if (NB == 1) __syncthreads();
    park((t + 1) % NB);
    __syncthreads();
    fetch(min(t + 2, n_steps - 1) * 32);
  }
  if (n_full < n_steps) step(std::true_type{}, n_full % NB, n_full * 32);
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
// Works on S^T like dQ.  Bias2 itself does not change along the walk and stays in registers;
// a row's Bias1 is added to it for the initial value of the S^T accumulator, -Delta is that of
// dP^T.  Nothing in the walk looks at s: queries and keys beyond it repeat the last one, and
// what accumulates for them is not stored.
template <typename T, bool VEC>
__global__ __launch_bounds__(256, (BwdCfg<T, VEC>::kMinWaves)) void attn_bwd_db2_kernel(BwdParams p) {
  typedef typename Vec8<T>::type V8;
  constexpr int NB = BwdCfg<T, VEC>::kBuffers;
  __shared__ __attribute__((aligned(32))) T tiles[NB][4][64 * kTP];   // Q, dO (64 queries), K, V (64 keys)
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
  // (without a Bias1 the loads go to Bias2's row and count for nothing: no load under a branch)
  const T* b1base = p.b1 ? (const T*)p.b1 : b2row;
  const int64_t b1pitch = p.b1 ? s : 0;
  const float b1on = p.b1 ? 1.0f : 0.0f;
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

  // thread t: 8 channels (t & 3) of row t >> 2 of each of the four 64-row tiles.  Along the
  // walk only the row's base address changes, the same for all lanes: what a lane adds to it
  // is formed once.
  const int crow = tid >> 2, cc = 8 * (tid & 3);
  const unsigned off_q = ((unsigned)min(qs0 + crow, s - 1) * H + h) * 32 + cc;
  const unsigned off_k = ((unsigned)min(ks0 + crow, s - 1) * H + h) * 32 + cc;
  const unsigned off_stat = (unsigned)qi * H + h;
  unsigned off_b1[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) off_b1[ks] = vec ? min(key0 + 16 * ks + 8 * g, s - 8) : 0;
  const int64_t row_elems = (int64_t)s * H * 32, row_stats = (int64_t)s * H;
  V8 piece[4], b1n[2];
  float mq_n = 0.0f, dq_n = 0.0f;
  // 16-bit: Bias1 reaches the accumulator on the matrix pipe (see the dQ kernel): one value
  // per lane, that of the key its accumulator row stands for, in K slot 0 of one more product
  constexpr bool MMB = sizeof(T) == 2;
  const unsigned off_b1m = min(key0 + perm_row(ln), s - 1);
  T b1m_n = (T)0.0f;
  V8 one_frag;
#pragma unroll
  for (int t = 0; t < 8; ++t) one_frag[t] = (T)(t == 0 && g == 0 ? b1on : 0.0f);
  f32x16 b2acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) b2acc[r] = b2f[r >> 3][r & 7];
  auto fetch = [&](int i) {
    piece[0] = load8<T>((const T*)p.q + i * row_elems + off_q);
    piece[1] = load8<T>((const T*)p.dout + i * row_elems + off_q);
    piece[2] = load8<T>((const T*)p.k + i * row_elems + off_k);
    piece[3] = load8<T>((const T*)p.v + i * row_elems + off_k);
    mq_n = (p.lse + i * row_stats)[off_stat];
    dq_n = (p.delta + i * row_stats)[off_stat];
    const T* b1row = b1base + i * b1pitch;
    if (MMB) {
      b1m_n = b1row[off_b1m];
    } else {
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
        b1n[ks] = vec ? load8<T>(b1row + off_b1[ks]) : load_bias8_raw<T>(b1row, key0 + 16 * ks + 8 * g, s, false);
    }
  };
  // Row i is computed out of buffer i % NB while row i + 1, fetched a step earlier, is parked
  // (two buffers: into the other one, which every wave left at the last barrier).
  const int last = p.n_rows - 1;
  fetch(0);
#pragma unroll
  for (int w = 0; w < 4; ++w) store8<T>(&tiles[0][w][crow * kTP + cc], piece[w]);
  float neg_mq = -mq_n, neg_dq = -dq_n;
  V8 b1c[2] = {b1n[0], b1n[1]};
  T b1m = b1m_n;
  __syncthreads();
  for (int i = 0; i < p.n_rows; ++i) {
    const int buf = i % NB;
    fetch(min(i + 1, last));
    asm volatile("" ::: "memory");   // the loads are issued here, a step ahead of their use
    f32x16 st, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) dp[r] = neg_dq;
    if constexpr (MMB) {
      V8 b1a;
#pragma unroll
      for (int t = 0; t < 8; ++t) b1a[t] = (T)0.0f;
      b1a[0] = (g == 0 && b1on != 0.0f) ? b1m : (T)0.0f;
      st = b2acc;
      mma32(st, b1a, one_frag);   // Bias2 + Bias1
    } else {
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const f32x8 b1f = to_f32(b1c[ks]);
#pragma unroll
        for (int t = 0; t < 8; ++t) st[8 * ks + t] = b1f[t] * b1on + b2f[ks][t];
      }
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const V8 qf = load8<T>(&tiles[buf][0][(32 * wq + ln) * kTP + 16 * kk + 8 * g]);
      const V8 dof = load8<T>(&tiles[buf][1][(32 * wq + ln) * kTP + 16 * kk + 8 * g]);
      const V8 kf = load8<T>(&tiles[buf][2][(32 * wk + perm_row(ln)) * kTP + 16 * kk + 8 * g]);
      const V8 vf = load8<T>(&tiles[buf][3][(32 * wk + perm_row(ln)) * kTP + 16 * kk + 8 * g]);
      mma32(st, kf, qf);    // S^T[key][query] (+ biases)
      mma32(dp, vf, dof);   // dP^T[key][query] - Delta
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] += fast_exp2(st[r] * kBwdLog2e + neg_mq) * dp[r];
    if (NB == 1) __syncthreads();
    // the next row: tiles into LDS, its statistics and Bias1 into this step's places
#pragma unroll
    for (int w = 0; w < 4; ++w) store8<T>(&tiles[(i + 1) % NB][w][crow * kTP + cc], piece[w]);
    neg_mq = -mq_n;
    neg_dq = -dq_n;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) b1c[ks] = b1n[ks];
    b1m = b1m_n;
    __syncthreads();
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
  const unsigned blocks = (unsigned)((s + 31) / 32);
  const dim3 walk((blocks + 3) / 4, heads, n_rows), pairs((blocks + 1) / 2, heads, (blocks + 1) / 2);
  if ((s & 7) == 0) {
    attn_bwd_dq_kernel<T, true><<<walk, dim3(256), 0, stream>>>(p);   // (writes Delta: first)
    attn_bwd_kv_kernel<T, true><<<walk, dim3(256), 0, stream>>>(p);
    if (db2) attn_bwd_db2_kernel<T, true><<<pairs, dim3(256), 0, stream>>>(p);
  } else {
    attn_bwd_dq_kernel<T, false><<<walk, dim3(256), 0, stream>>>(p);
    attn_bwd_kv_kernel<T, false><<<walk, dim3(256), 0, stream>>>(p);
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
