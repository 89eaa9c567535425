// Helpers shared by the kernels that work on tiles of 32 pair-tensor rows
// (128 channels each): row fragments in MFMA operand order, in-register
// LayerNorm, and the per-wave 32 x 32 LDS staging tile that turns accumulator
// tiles into 16-byte coalesced global accesses.
#pragma once
#include "common.h"

namespace ptx {

constexpr int kC = 128;       // hidden channels (c_hidden_mul, heads * d) and the default row width
constexpr int kKSteps = 8;    // kC / 16
// Rows of the pair tensor itself may be narrower: KS = c_z / 16 K steps (template
// parameter of the helpers below, 8 by default; 4 serves c_z = 64).

template <typename T> struct Cfg {
  static constexpr int VE = 16 / (int)sizeof(T);     // elements per 16-byte vector
  static constexpr int LPM = 32 / VE;                // lanes that cover one 32-long major row
  static constexpr int MPP = kWave / LPM;            // major rows per read-back pass
  static constexpr int NPASS = 32 / MPP;             // passes per 32 x 32 tile
  // Row pitch of the staging tile: bf16 36 elements = 18 dwords, fp32 34 elements = 34
  // dwords; both spread the 16 lanes of an 8-byte store phase over all 32 banks.  Rows are
  // 8-byte aligned, so the tile is accessed with 8-byte LDS operations only.
  static constexpr int PITCH = 32 + 8 / (int)sizeof(T);
  static constexpr int NBUF = sizeof(T) == 2 ? 2 : 1;    // weight buffers in LDS
};

template <typename T, int RB, int KS = kKSteps>
struct RowFrags {
  typename Vec8<T>::type f[RB][KS];
};

// gamma = 1 / beta = 0 stand-ins for a LayerNorm without weight / bias: the affine loads
// below are unconditional (a load under a branch costs a full wait of its own), a missing
// parameter just points here.
#define PTX_REP8(x) x, x, x, x, x, x, x, x
#define PTX_REP128(x)                                                                           \
  PTX_REP8(x), PTX_REP8(x), PTX_REP8(x), PTX_REP8(x), PTX_REP8(x), PTX_REP8(x), PTX_REP8(x),   \
      PTX_REP8(x), PTX_REP8(x), PTX_REP8(x), PTX_REP8(x), PTX_REP8(x), PTX_REP8(x), PTX_REP8(x), \
      PTX_REP8(x), PTX_REP8(x)
// (256 entries: the widest row)
static __device__ const float kOnesF32[2 * kC] = {PTX_REP128(1.0f), PTX_REP128(1.0f)};
static __device__ const uint16_t kOnesBf16[2 * kC] = {PTX_REP128(0x3F80), PTX_REP128(0x3F80)};
static __device__ const float kZerosAny[2 * kC] = {PTX_REP128(0.0f), PTX_REP128(0.0f)};
#undef PTX_REP128
#undef PTX_REP8
template <typename T> __device__ __forceinline__ const T* default_gamma();
template <> __device__ __forceinline__ const float* default_gamma<float>() { return kOnesF32; }
template <> __device__ __forceinline__ const bf16_t* default_gamma<bf16_t>() {
  return reinterpret_cast<const bf16_t*>(kOnesBf16);
}
template <typename T> __device__ __forceinline__ const T* default_beta() {
  return reinterpret_cast<const T*>(kZerosAny);
}

// Mean / rstd of a row of 16*KS channels spread over the two half-wave lanes that hold it,
// then gamma/beta (either may be null); result rounded to T like the reference's
// LayerNorm output.
// gamma / beta are read as type P: T from global memory (null: the stand-ins above), or float
// from a copy the caller keeps in LDS (P = float, DEFAULTS = false: never null).
template <typename T, int KS, typename P = T, bool DEFAULTS = true>
__device__ __forceinline__ void normalize_row(f32x8 (&v)[KS], const P* __restrict__ gamma,
                                              const P* __restrict__ beta, float eps, int g,
                                              typename Vec8<T>::type (&out)[KS]) {
  const P* gp = (DEFAULTS && !gamma ? default_gamma<P>() : gamma) + 8 * g;
  const P* bp = (DEFAULTS && !beta ? default_beta<P>() : beta) + 8 * g;
  float s = 0.0f;
#pragma unroll
  for (int kk = 0; kk < KS; ++kk)
#pragma unroll
    for (int t = 0; t < 8; ++t) s += v[kk][t];
  s += swap32(s);
  const float mean = s * (1.0f / (16 * KS));
  float q = 0.0f;
#pragma unroll
  for (int kk = 0; kk < KS; ++kk)
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const float d = v[kk][t] - mean;
      q += d * d;
    }
  q += swap32(q);
  const float rstd = rsqrtf(q * (1.0f / (16 * KS)) + eps);
#pragma unroll
  for (int kk = 0; kk < KS; ++kk) {
    // (no branch around these loads, so the compiler may issue them as early as registers allow)
    const f32x8 gmf = to_f32(load8<P>(gp + 16 * kk)), btf = to_f32(load8<P>(bp + 16 * kk));
    f32x8 o;
#pragma unroll
    for (int t = 0; t < 8; ++t) o[t] = (v[kk][t] - mean) * rstd * gmf[t] + btf[t];
    out[kk] = from_f32<T>(o);
  }
}

// The same LayerNorm straight from the stored fragments, converting on the fly in each of
// its three passes: no fp32 copy of the row is kept, for callers short of registers.
template <typename T, int KS, typename P = T, bool DEFAULTS = true>
__device__ __forceinline__ void normalize_raw(const typename Vec8<T>::type (&raw)[KS],
                                              const P* __restrict__ gamma,
                                              const P* __restrict__ beta, float eps, int g,
                                              typename Vec8<T>::type (&out)[KS]) {
  const P* gp = (DEFAULTS && !gamma ? default_gamma<P>() : gamma) + 8 * g;
  const P* bp = (DEFAULTS && !beta ? default_beta<P>() : beta) + 8 * g;
  float s = 0.0f;
#pragma unroll
  for (int kk = 0; kk < KS; ++kk) {
    const f32x8 v = to_f32(raw[kk]);
#pragma unroll
    for (int t = 0; t < 8; ++t) s += v[t];
  }
  s += swap32(s);
  const float mean = s * (1.0f / (16 * KS));
  float q = 0.0f;
#pragma unroll
  for (int kk = 0; kk < KS; ++kk) {
    const f32x8 v = to_f32(raw[kk]);
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const float d = v[t] - mean;
      q += d * d;
    }
  }
  q += swap32(q);
  const float rstd = rsqrtf(q * (1.0f / (16 * KS)) + eps);
#pragma unroll
  for (int kk = 0; kk < KS; ++kk) {
    const f32x8 v = to_f32(raw[kk]);
    const f32x8 gmf = to_f32(load8<P>(gp + 16 * kk)), btf = to_f32(load8<P>(bp + 16 * kk));
    f32x8 o;
#pragma unroll
    for (int t = 0; t < 8; ++t) o[t] = (v[t] - mean) * rstd * gmf[t] + btf[t];
    out[kk] = from_f32<T>(o);
  }
}

// Load RB row blocks whose lane rows start at element offsets off[rb] (+ 8*g added here)
// and, if LN, normalise them.
// TZ: storage type of the rows (T, or float for an fp32 residual stream normalised and
// rounded to T here; LN only).
template <typename T, int RB, bool LN, int KS, typename P = T, bool DEFAULTS = true, typename TZ = T>
__device__ __forceinline__ void load_rows_at(RowFrags<T, RB, KS>& out, const TZ* __restrict__ x,
                                             const int64_t (&off)[RB], const P* __restrict__ gamma,
                                             const P* __restrict__ beta, float eps, int lane) {
  static_assert(LN || sizeof(TZ) == sizeof(T), "rows of another type are converted by the LayerNorm");
  const int g = lane >> 5;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const TZ* rp = x + off[rb] + 8 * g;
    if constexpr (!LN) {
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) out.f[rb][kk] = load8<T>((const T*)rp + 16 * kk);
    } else {
      f32x8 v[KS];
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) v[kk] = to_f32(load8<TZ>(rp + 16 * kk));
      normalize_row<T, KS, P, DEFAULTS>(v, gamma, beta, eps, g, out.f[rb]);
    }
  }
}

// Load RB*32 consecutive logical rows starting at row0 (rows >= n_rows re-read the last
// valid row; their results are never stored).
template <typename T, int RB, bool LN, int KS, typename P = T, bool DEFAULTS = true, typename TZ = T>
__device__ __forceinline__ void load_rows(RowFrags<T, RB, KS>& out, const TZ* __restrict__ x,
                                          const RowMap& map, int64_t row0, int64_t n_rows,
                                          const P* __restrict__ gamma, const P* __restrict__ beta,
                                          float eps, int lane) {
  int64_t off[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    int64_t p = row0 + rb * 32 + (lane & 31);
    p = p < n_rows ? p : n_rows - 1;
    off[rb] = map(p);
  }
  load_rows_at<T, RB, LN, KS, P, DEFAULTS, TZ>(out, x, off, gamma, beta, eps, lane);
}

// One weight fragment: 32 output columns x 16 K values, lane -> (column l%32,
// K = k0 + 8*(l/32) ..+7) of a row-major weight w[n_out][ldw].  Columns beyond
// n_out re-read the last row: their outputs are never stored.
template <typename T>
__device__ __forceinline__ typename Vec8<T>::type load_wfrag(const T* __restrict__ w, int ldw,
                                                             int n_out, int col0, int k0,
                                                             int lane) {
  int col = col0 + (lane & 31);
  col = col < n_out ? col : n_out - 1;
  return load8<T>(w + (int64_t)col * ldw + k0 + 8 * (lane >> 5));
}

// ---- per-wave 32 x 32 staging tile -----------------------------------------
template <typename T> struct VecE;
template <> struct VecE<bf16_t> { typedef bf16x8 type; };
template <> struct VecE<float> { typedef f32x4 type; };
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// put: lane n = major index, vals[r] = value at minor acc_row(r, g).
template <typename T>
__device__ __forceinline__ void stage_put(T* st, const float (&vals)[16], int lane) {
  typedef typename Vec4<T>::type V4;
  const int n = lane & 31, g = lane >> 5;
#pragma unroll
  for (int qd = 0; qd < 4; ++qd) {
    f32x4 v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = vals[4 * qd + e];
    const V4 pk = from_f32<T>(v);
    T* dst = st + n * Cfg<T>::PITCH + 8 * qd + 4 * g;
    if constexpr (sizeof(T) == 2) {
      *reinterpret_cast<V4*>(dst) = pk;                        // 8 bytes
    } else {
      reinterpret_cast<f32x2*>(dst)[0] = f32x2{pk[0], pk[1]};  // 2 x 8 bytes
      reinterpret_cast<f32x2*>(dst)[1] = f32x2{pk[2], pk[3]};
    }
  }
}
// Coordinates this lane serves in read-back pass `ps`: major row and first minor.
template <typename T>
__device__ __forceinline__ void stage_coord(int ps, int lane, int& major, int& minor0) {
  major = ps * Cfg<T>::MPP + lane / Cfg<T>::LPM;
  minor0 = (lane % Cfg<T>::LPM) * Cfg<T>::VE;
}
// get / put one 16-byte vector (VE consecutive minors of one major row), raw.
template <typename T>
__device__ __forceinline__ typename VecE<T>::type stage_get_vec(const T* st, int major,
                                                                int minor0) {
  const u32x2* src = reinterpret_cast<const u32x2*>(st + major * Cfg<T>::PITCH + minor0);
  u32x2 h[2] = {src[0], src[1]};
  return *reinterpret_cast<typename VecE<T>::type*>(h);
}
template <typename T>
__device__ __forceinline__ void stage_put_vec(T* st, int major, int minor0,
                                              typename VecE<T>::type v) {
  u32x2* dst = reinterpret_cast<u32x2*>(st + major * Cfg<T>::PITCH + minor0);
  const u32x2* s = reinterpret_cast<const u32x2*>(&v);
  dst[0] = s[0];
  dst[1] = s[1];
}
// v += residual (both in T, sum in fp32, rounded once more like the reference's `z + update`)
template <typename T>
__device__ __forceinline__ typename VecE<T>::type add_vec(typename VecE<T>::type v,
                                                          typename VecE<T>::type r) {
  typename VecE<T>::type o;
#pragma unroll
  for (int e = 0; e < Cfg<T>::VE; ++e) o[e] = from_f32<T>(to_f32(v[e]) + to_f32(r[e]));
  return o;
}

// LDS traffic inside one wave: make the stores visible before the loads.
// (LDS operations of one wave execute in order, so no hardware wait is needed; the fences
// only keep the compiler from reordering the accesses.)
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

}  // namespace ptx
