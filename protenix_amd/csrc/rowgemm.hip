// Row-tile projections with K = 128: every pair-tensor row (one (i,j) position,
// 128 channels) is normalised in registers and multiplied by small weight
// matrices on MFMA; gates, masks, SwiGLU and residual adds are applied to the
// accumulators before anything is written.
//
// A wave owns RB blocks of 32 rows.  A row block lives in registers as 8
// operand fragments (16-deep K steps, see common.h): lane (l%32) holds row
// l%32, channels 16*kk + 8*(l/32) .. +7.  The same registers serve as the A
// operand (result: lane <-> output column, used for row-major outputs) or as
// the B operand (result: lane <-> row, used for channel-major outputs), so one
// kernel writes both layouts with 64-byte-contiguous stores.
//
// Weights are staged through LDS already permuted into fragment order
// ([fragment][lane] -> conflict-free 16-byte reads), two 32-column tiles per
// chunk, double-buffered, one barrier per chunk.
#include "common.h"
#include "kernels.h"

namespace ptx {

constexpr int kC = 128;       // channels per pair-tensor row == K of every product here
constexpr int kKSteps = 8;    // kC / 16

template <typename T, int RB>
struct RowFrags {
  typename Vec8<T>::type f[RB][kKSteps];
};

// Load RB*32 rows starting at row0 (rows >= n_rows read as zero) and, if LN,
// normalise them: fp32 statistics, gamma/beta (either may be null) applied in
// fp32, result rounded to T like the reference's LayerNorm output.
template <typename T, int RB, bool LN>
__device__ __forceinline__ void load_rows(RowFrags<T, RB>& out, const T* __restrict__ x,
                                          const RowMap& map, int64_t row0, int64_t n_rows,
                                          const T* __restrict__ gamma, const T* __restrict__ beta,
                                          float eps, int lane) {
  const int n = lane & 31, g = lane >> 5;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int64_t p = row0 + rb * 32 + n;
    const bool valid = p < n_rows;
    const T* rp = x + map(valid ? p : 0) + 8 * g;
    if (!LN) {
#pragma unroll
      for (int kk = 0; kk < kKSteps; ++kk)
        out.f[rb][kk] = valid ? load8<T>(rp + 16 * kk) : zero8<T>();
    } else {
      f32x8 v[kKSteps];
#pragma unroll
      for (int kk = 0; kk < kKSteps; ++kk) v[kk] = to_f32(valid ? load8<T>(rp + 16 * kk) : zero8<T>());
      float s = 0.0f;
#pragma unroll
      for (int kk = 0; kk < kKSteps; ++kk)
#pragma unroll
        for (int t = 0; t < 8; ++t) s += v[kk][t];
      s += swap32(s);
      const float mean = s * (1.0f / kC);
      float q = 0.0f;
#pragma unroll
      for (int kk = 0; kk < kKSteps; ++kk)
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          const float d = v[kk][t] - mean;
          q += d * d;
        }
      q += swap32(q);
      const float rstd = rsqrtf(q * (1.0f / kC) + eps);
#pragma unroll
      for (int kk = 0; kk < kKSteps; ++kk) {
        f32x8 o;
#pragma unroll
        for (int t = 0; t < 8; ++t) o[t] = (v[kk][t] - mean) * rstd;
        if (gamma) {
          const f32x8 gm = to_f32(load8<T>(gamma + 16 * kk + 8 * g));
#pragma unroll
          for (int t = 0; t < 8; ++t) o[t] *= gm[t];
        }
        if (beta) {
          const f32x8 bt = to_f32(load8<T>(beta + 16 * kk + 8 * g));
#pragma unroll
          for (int t = 0; t < 8; ++t) o[t] += bt[t];
        }
        out.f[rb][kk] = from_f32<T>(o);
      }
    }
  }
}

// Same, for a channel-major source x[c][p] (the triangle product): lane gathers
// its 8 channels per fragment with element loads that are contiguous across
// lanes (32 consecutive rows per channel).
template <typename T, int RB>
__device__ __forceinline__ void load_rows_channel_major_ln(RowFrags<T, RB>& out,
                                                           const T* __restrict__ x,
                                                           int64_t chan_stride, int64_t row0,
                                                           int64_t n_rows,
                                                           const T* __restrict__ gamma,
                                                           const T* __restrict__ beta, float eps,
                                                           int lane) {
  const int n = lane & 31, g = lane >> 5;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int64_t p = row0 + rb * 32 + n;
    const bool valid = p < n_rows;
    const T* rp = x + (valid ? p : 0) + (int64_t)(8 * g) * chan_stride;
    f32x8 v[kKSteps];
#pragma unroll
    for (int kk = 0; kk < kKSteps; ++kk)
#pragma unroll
      for (int t = 0; t < 8; ++t)
        v[kk][t] = valid ? to_f32(rp[(int64_t)(16 * kk + t) * chan_stride]) : 0.0f;
    float s = 0.0f;
#pragma unroll
    for (int kk = 0; kk < kKSteps; ++kk)
#pragma unroll
      for (int t = 0; t < 8; ++t) s += v[kk][t];
    s += swap32(s);
    const float mean = s * (1.0f / kC);
    float q = 0.0f;
#pragma unroll
    for (int kk = 0; kk < kKSteps; ++kk)
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const float d = v[kk][t] - mean;
        q += d * d;
      }
    q += swap32(q);
    const float rstd = rsqrtf(q * (1.0f / kC) + eps);
#pragma unroll
    for (int kk = 0; kk < kKSteps; ++kk) {
      f32x8 o;
      const f32x8 gm = to_f32(load8<T>(gamma + 16 * kk + 8 * g));
      const f32x8 bt = to_f32(load8<T>(beta + 16 * kk + 8 * g));
#pragma unroll
      for (int t = 0; t < 8; ++t) o[t] = (v[kk][t] - mean) * rstd * gm[t] + bt[t];
      out.f[rb][kk] = from_f32<T>(o);
    }
  }
}

// One weight fragment: 32 output columns x 16 K values, lane -> (column l%32,
// K = k0 + 8*(l/32) ..+7) of a row-major weight w[n_out][ldw].  Rows >= n_out
// read as zero.
template <typename T>
__device__ __forceinline__ typename Vec8<T>::type load_wfrag(const T* __restrict__ w, int ldw,
                                                             int n_out, int col0, int k0,
                                                             int lane) {
  const int col = col0 + (lane & 31);
  if (col >= n_out) return zero8<T>();
  return load8<T>(w + (int64_t)col * ldw + k0 + 8 * (lane >> 5));
}

// ---------------------------------------------------------------------------
// rowgemm_in: [LayerNorm] -> chunks of two 32-column weight tiles -> epilogue.
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
  int aux;              // TRIATTN_IN: heads; PAIRBIAS: heads | out_f32 << 8; TRANSITION_IN: n_factor
  float q_scale;        // TRIATTN_IN: 1/sqrt(d)
  // TRIMUL_OUT only
  const void* x2;       // channel-major triangle product [128][n_rows]
  const void* gamma2;
  const void* beta2;
  int add_residual;
};

enum RowGemmInMode { kTriMulIn = 0, kTriAttnIn = 1, kTransitionIn = 2, kPairBias = 3, kTriMulOut = 4 };

template <int MODE>
__device__ __forceinline__ int n_chunks(const RowGemmInParams& p) {
  if (MODE == kTriMulIn) return 8;                 // {a,b} x 4 channel blocks
  if (MODE == kTriAttnIn) return 9;                // q,k,g,v: 2 chunks each; bias: 1
  if (MODE == kTransitionIn) return 4 * p.aux;     // n_factor*128/32 column blocks
  if (MODE == kPairBias) return 1;
  return 4;                                        // kTriMulOut: 4 column blocks
}

// Weight matrix, its row count, first row and whether the tile exists, for
// tile `t` (0/1) of chunk `ch`.
template <typename T, int MODE>
__device__ __forceinline__ void chunk_tile(const RowGemmInParams& p, int ch, int t, const T*& w,
                                           int& n_out, int& col0) {
  if (MODE == kTriMulIn) {            // w: ap, ag, bp, bg ; tile0 = projection, tile1 = gate
    w = (const T*)p.w[(ch >> 2) * 2 + t];
    n_out = kC;
    col0 = (ch & 3) * 32;
  } else if (MODE == kTriAttnIn) {    // w: q, k, g, v, bias
    const int which = ch >> 1;
    w = (const T*)p.w[which];
    n_out = which == 4 ? (t == 0 ? p.aux : 0) : kC;
    col0 = which == 4 ? 0 : ((ch & 1) * 2 + t) * 32;
  } else if (MODE == kTransitionIn) { // w: a, b ; tile0 = a, tile1 = b
    w = (const T*)p.w[t];
    n_out = kC * p.aux;
    col0 = ch * 32;
  } else if (MODE == kPairBias) {
    w = (const T*)p.w[0];
    n_out = t == 0 ? (p.aux & 0xff) : 0;
    col0 = 0;
  } else {                            // kTriMulOut: w: z, g
    w = (const T*)p.w[t];
    n_out = kC;
    col0 = ch * 32;
  }
}

template <typename T, int RB, int MODE>
__global__ __launch_bounds__(256) void rowgemm_in_kernel(RowGemmInParams p) {
  typedef typename Vec8<T>::type V8;
  __shared__ V8 lds_w[2][2 * kKSteps][kWave];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 31, g = lane >> 5;
  const int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * (RB * 32);

  RowFrags<T, RB> xf;
  load_rows<T, RB, true>(xf, (const T*)p.x, p.xmap, row0, p.n_rows, (const T*)p.gamma,
                         (const T*)p.beta, p.eps, lane);
  // second fragment set only exists for the triangle-product epilogue
  RowFrags<T, RB> xf2;   // dead (and removed by the compiler) in the other modes
  if constexpr (MODE == kTriMulOut) {
    load_rows_channel_major_ln<T, RB>(xf2, (const T*)p.x2, p.n_rows, row0, p.n_rows,
                                      (const T*)p.gamma2, (const T*)p.beta2, p.eps, lane);
  }

  const int nch = n_chunks<MODE>(p);
  V8 pre[4];
  auto fetch = [&](int ch) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int fid = wave * 4 + j;   // 16 fragments per chunk: tile = fid/8, kk = fid%8
      const T* w;
      int n_out, col0;
      chunk_tile<T, MODE>(p, ch, fid >> 3, w, n_out, col0);
      pre[j] = load_wfrag<T>(w, kC, n_out, col0, (fid & 7) * 16, lane);
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int j = 0; j < 4; ++j) lds_w[buf][wave * 4 + j][lane] = pre[j];
  };
  fetch(0);
  stash(0);
  __syncthreads();

  for (int ch = 0; ch < nch; ++ch) {
    const int buf = ch & 1;
    if (ch + 1 < nch) fetch(ch + 1);

    // Orientation: channel-major outputs want lane <-> row (weights as A).
    bool rows_on_lanes;
    if (MODE == kTriMulIn || MODE == kPairBias) rows_on_lanes = true;
    else if (MODE == kTriAttnIn) rows_on_lanes = (ch >= 6);   // v^T and the triangle bias
    else rows_on_lanes = false;

    f32x16 acc[RB][2];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[rb][t][r] = 0.0f;

#pragma unroll
    for (int kk = 0; kk < kKSteps; ++kk) {
      const V8 w0 = lds_w[buf][kk][lane];
      const V8 w1 = lds_w[buf][kKSteps + kk][lane];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        if constexpr (MODE == kTriMulOut) {
          mma32(acc[rb][0], xf2.f[rb][kk], w0);   // W_z LN_out(x)
          mma32(acc[rb][1], xf.f[rb][kk], w1);    // W_g LN_in(z)
        } else {
          if (rows_on_lanes) {
            mma32(acc[rb][0], w0, xf.f[rb][kk]);
            mma32(acc[rb][1], w1, xf.f[rb][kk]);
          } else {
            mma32(acc[rb][0], xf.f[rb][kk], w0);
            mma32(acc[rb][1], xf.f[rb][kk], w1);
          }
        }
      }
    }

    // ------------------------------ epilogues ------------------------------
    if constexpr (MODE == kTriMulIn) {
      // a/b[c][p] = mask(p) * sigmoid(gate) * proj ; lane <-> row p, register <-> channel
      T* outp = (T*)p.out[ch >> 2];
      const int c0 = (ch & 3) * 32;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int64_t row = row0 + rb * 32 + n;
        if (row < p.n_rows) {
          const float m = p.mask ? to_f32(((const T*)p.mask)[p.mmap(row)]) : 1.0f;
          const int64_t i = row / p.n, kq = row - i * p.n;
          T* base = outp + i * p.pitch + kq;
          const int64_t cstride = (int64_t)p.n * p.pitch;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float v = m * sigmoidf_fast(acc[rb][1][r]) * acc[rb][0][r];
            base[(c0 + acc_row(r, g)) * cstride] = from_f32<T>(v);
          }
        }
      }
    } else if constexpr (MODE == kTriAttnIn) {
      const int which = ch >> 1;
      if (which < 3) {
        // q (scaled), k, sigmoid(g): row-major [p][128]; lane <-> column, register <-> row
        T* outp = (T*)p.out[which];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            const int col = ((ch & 1) * 2 + t) * 32 + n;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int64_t row = row0 + rb * 32 + acc_row(r, g);
              if (row < p.n_rows) {
                float v = acc[rb][t][r];
                if (which == 0) v = to_f32(from_f32<T>(v)) * p.q_scale;   // q rounded, then scaled
                if (which == 2) v = sigmoidf_fast(v);
                outp[row * kC + col] = from_f32<T>(v);
              }
            }
          }
      } else if (which == 3) {
        // v^T[i][c][j]: lane <-> row p = i*n + j, register <-> channel
        T* outp = (T*)p.out[3];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          const int64_t row = row0 + rb * 32 + n;
          if (row < p.n_rows) {
            const int64_t i = row / p.n, j = row - i * p.n;
            T* base = outp + i * (int64_t)kC * p.pitch + j;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                const int c = ((ch & 1) * 2 + t) * 32 + acc_row(r, g);
                base[(int64_t)c * p.pitch] = from_f32<T>(acc[rb][t][r]);
              }
          }
        }
      } else {
        // triangle bias [h][i][pitch]
        T* outp = (T*)p.out[4];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          const int64_t row = row0 + rb * 32 + n;
          if (row < p.n_rows) {
            const int64_t i = row / p.n, j = row - i * p.n;
            T* base = outp + i * p.pitch + j;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int h = acc_row(r, g);
              if (h < p.aux) base[(int64_t)h * p.n * p.pitch] = from_f32<T>(acc[rb][0][r]);
            }
          }
        }
      }
    } else if constexpr (MODE == kTransitionIn) {
      // hidden[p][col] = silu(a) * b ; lane <-> column, register <-> row
      T* outp = (T*)p.out[0];
      const int64_t ldh = (int64_t)kC * p.aux;
      const int col = ch * 32 + n;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t row = row0 + rb * 32 + acc_row(r, g);
          if (row < p.n_rows) {
            // the reference rounds a and b to T before the activation
            const float a = to_f32(from_f32<T>(acc[rb][0][r]));
            const float b = to_f32(from_f32<T>(acc[rb][1][r]));
            outp[row * ldh + col] = from_f32<T>(a * sigmoidf_fast(a) * b);
          }
        }
    } else if constexpr (MODE == kPairBias) {
      const int heads = p.aux & 0xff;
      const bool f32_out = (p.aux >> 8) & 1;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int64_t row = row0 + rb * 32 + n;
        if (row < p.n_rows) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int h = acc_row(r, g);
            if (h < heads) {
              if (f32_out) ((float*)p.out[0])[(int64_t)h * p.n_rows + row] = acc[rb][0][r];
              else ((T*)p.out[0])[(int64_t)h * p.n_rows + row] = from_f32<T>(acc[rb][0][r]);
            }
          }
        }
      }
    } else {
      // kTriMulOut: out[p][col] = [z +] (W_z LN_out(x)) * sigmoid(W_g LN_in(z))
      T* outp = (T*)p.out[0];
      const T* zres = (const T*)p.x;
      const int col = ch * 32 + n;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t row = row0 + rb * 32 + acc_row(r, g);
          if (row < p.n_rows) {
            // linear_z output is rounded to T before the gate multiply
            float v = to_f32(from_f32<T>(acc[rb][0][r])) * sigmoidf_fast(acc[rb][1][r]);
            if (p.add_residual) v = to_f32(from_f32<T>(v)) + to_f32(zres[row * kC + col]);
            outp[row * kC + col] = from_f32<T>(v);
          }
        }
    }

    if (ch + 1 < nch) stash(buf ^ 1);
    __syncthreads();
  }
}

template <typename T, int MODE>
int launch_rowgemm_in(const RowGemmInParams& p, hipStream_t stream) {
  constexpr int RB = (sizeof(T) == 2 && MODE != kTriMulOut) ? 2 : 1;
  const int64_t rows_per_block = 4 * RB * 32;
  const int64_t blocks = (p.n_rows + rows_per_block - 1) / rows_per_block;
  if (blocks == 0) return 0;
  rowgemm_in_kernel<T, RB, MODE><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(p);
  return 0;
}

// ---------------------------------------------------------------------------
// rowgemm_out: out(p) = [res(p) +] A[p][0:K] W^T, K = 128 * n_slab, 128 output
// columns.  A is row-major with leading dimension K; out/res rows go through a
// RowMap (the ending-node attention writes z[j][i]).
// ---------------------------------------------------------------------------
struct RowGemmOutParams {
  const void* a;
  int n_slab;
  const void* w;        // [128][128*n_slab]
  const void* res;      // residual source (same addressing as out) or null
  void* out;
  RowMap omap;
  int64_t n_rows;
};

template <typename T, int RB>
__global__ __launch_bounds__(256) void rowgemm_out_kernel(RowGemmOutParams p) {
  typedef typename Vec8<T>::type V8;
  __shared__ V8 lds_w[2][2 * kKSteps][kWave];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 31, g = lane >> 5;
  const int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * (RB * 32);
  const int K = kC * p.n_slab;
  const T* w = (const T*)p.w;

  f32x16 acc[RB][4];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rb][t][r] = 0.0f;

  // chunk index c -> (slab = c/2, column pair = c%2)
  const int nch = 2 * p.n_slab;
  V8 pre[4];
  auto fetch = [&](int ch) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int fid = wave * 4 + j;
      const int col0 = ((ch & 1) * 2 + (fid >> 3)) * 32;
      pre[j] = load_wfrag<T>(w, K, kC, col0, (ch >> 1) * kC + (fid & 7) * 16, lane);
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int j = 0; j < 4; ++j) lds_w[buf][wave * 4 + j][lane] = pre[j];
  };
  fetch(0);
  stash(0);
  __syncthreads();

  RowFrags<T, RB> af;
  const RowMap amap{(int64_t)K, 0, 1};   // row p -> p*K (n_inner = 1, so outer = p)
  for (int ch = 0; ch < nch; ++ch) {
    const int buf = ch & 1;
    if (ch + 1 < nch) fetch(ch + 1);
    if ((ch & 1) == 0) {
      load_rows<T, RB, false>(af, (const T*)p.a + (ch >> 1) * kC, amap, row0, p.n_rows, nullptr,
                              nullptr, 0.0f, lane);
    }
#pragma unroll
    for (int kk = 0; kk < kKSteps; ++kk) {
      const V8 w0 = lds_w[buf][kk][lane];
      const V8 w1 = lds_w[buf][kKSteps + kk][lane];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        if (ch & 1) {
          mma32(acc[rb][2], af.f[rb][kk], w0);
          mma32(acc[rb][3], af.f[rb][kk], w1);
        } else {
          mma32(acc[rb][0], af.f[rb][kk], w0);
          mma32(acc[rb][1], af.f[rb][kk], w1);
        }
      }
    }
    if (ch + 1 < nch) stash(buf ^ 1);
    __syncthreads();
  }

  T* outp = (T*)p.out;
  const T* resp = (const T*)p.res;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int64_t row = row0 + rb * 32 + acc_row(r, g);
      if (row < p.n_rows) {
        const int64_t off = p.omap(row) + n;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          float v = acc[rb][t][r];
          if (resp) v = to_f32(from_f32<T>(v)) + to_f32(resp[off + t * 32]);
          outp[off + t * 32] = from_f32<T>(v);
        }
      }
    }
}

template <typename T>
int launch_rowgemm_out(const RowGemmOutParams& p, hipStream_t stream) {
  constexpr int RB = sizeof(T) == 2 ? 2 : 1;
  const int64_t rows_per_block = 4 * RB * 32;
  const int64_t blocks = (p.n_rows + rows_per_block - 1) / rows_per_block;
  if (blocks == 0) return 0;
  rowgemm_out_kernel<T, RB><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(p);
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

template <typename T>
int trimul_project(const void* z, const void* mask, const void* ln_w, const void* ln_b,
                   const void* w_ap, const void* w_ag, const void* w_bp, const void* w_bg, void* a,
                   void* b, int n, int k_pitch, int incoming, float eps, hipStream_t stream) {
  RowGemmInParams p = {};
  p.x = z;
  p.xmap = pair_map(n, kC, incoming != 0);
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
  return launch_rowgemm_in<T, kTriMulIn>(p, stream);
}

template <typename T>
int trimul_output(const void* x, const void* z, const void* ln_in_w, const void* ln_in_b,
                  const void* ln_out_w, const void* ln_out_b, const void* w_z, const void* w_g,
                  void* out, int n, int add_residual, float eps, hipStream_t stream) {
  RowGemmInParams p = {};
  p.x = z;
  p.xmap = pair_map(n, kC, false);
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
  return launch_rowgemm_in<T, kTriMulOut>(p, stream);
}

template <typename T>
int triattn_project(const void* z, const void* ln_w, const void* ln_b, const void* w_q,
                    const void* w_k, const void* w_v, const void* w_g, const void* w_b, void* q,
                    void* k, void* vt, void* g, void* tri_bias, int n, int heads, int d,
                    int key_pitch, int transposed, float eps, hipStream_t stream) {
  RowGemmInParams p = {};
  p.x = z;
  p.xmap = pair_map(n, kC, transposed != 0);
  p.n_rows = (int64_t)n * n;
  p.gamma = ln_w;
  p.beta = ln_b;
  p.eps = eps;
  p.w[0] = w_q; p.w[1] = w_k; p.w[2] = w_g; p.w[3] = w_v; p.w[4] = w_b;
  p.out[0] = q; p.out[1] = k; p.out[2] = g; p.out[3] = vt; p.out[4] = tri_bias;
  p.n = n;
  p.aux = heads;
  p.pitch = key_pitch;
  p.q_scale = 1.0f / sqrtf((float)d);
  return launch_rowgemm_in<T, kTriAttnIn>(p, stream);
}

template <typename T>
int triattn_output(const void* o, const void* w_o, const void* z, void* out, int n, int transposed,
                   int add_residual, hipStream_t stream) {
  RowGemmOutParams p = {};
  p.a = o;
  p.n_slab = 1;
  p.w = w_o;
  p.res = add_residual ? z : nullptr;
  p.out = out;
  p.omap = pair_map(n, kC, transposed != 0);
  p.n_rows = (int64_t)n * n;
  return launch_rowgemm_out<T>(p, stream);
}

template <typename T>
int transition_fwd(const void* x, const void* ln_w, const void* ln_b, const void* w_a,
                   const void* w_b, const void* w_o, void* hidden, void* out, int64_t rows,
                   int n_factor, int add_residual, float eps, hipStream_t stream) {
  RowGemmInParams p = {};
  p.x = x;
  p.xmap = RowMap{kC, 0, 1};
  p.n_rows = rows;
  p.gamma = ln_w;
  p.beta = ln_b;
  p.eps = eps;
  p.w[0] = w_a; p.w[1] = w_b;
  p.out[0] = hidden;
  p.n = 1;
  p.aux = n_factor;
  launch_rowgemm_in<T, kTransitionIn>(p, stream);
  RowGemmOutParams q = {};
  q.a = hidden;
  q.n_slab = n_factor;
  q.w = w_o;
  q.res = add_residual ? x : nullptr;
  q.out = out;
  q.omap = RowMap{kC, 0, 1};
  q.n_rows = rows;
  return launch_rowgemm_out<T>(q, stream);
}

template <typename T>
int pair_bias_fwd(const void* z, const void* ln_w, const void* ln_b, const void* w, void* bias,
                  int n, int heads, int out_f32, float eps, hipStream_t stream) {
  RowGemmInParams p = {};
  p.x = z;
  p.xmap = pair_map(n, kC, false);
  p.n_rows = (int64_t)n * n;
  p.gamma = ln_w;
  p.beta = ln_b;
  p.eps = eps;
  p.w[0] = w;
  p.out[0] = bias;
  p.n = n;
  p.aux = heads | (out_f32 ? 0x100 : 0);
  return launch_rowgemm_in<T, kPairBias>(p, stream);
}

#define PTX_INSTANTIATE(T)                                                                          \
  template int trimul_project<T>(const void*, const void*, const void*, const void*, const void*,  \
                                 const void*, const void*, const void*, void*, void*, int, int,    \
                                 int, float, hipStream_t);                                            \
  template int trimul_output<T>(const void*, const void*, const void*, const void*, const void*,   \
                                const void*, const void*, const void*, void*, int, int, float,     \
                                hipStream_t);                                                      \
  template int triattn_project<T>(const void*, const void*, const void*, const void*, const void*, \
                                  const void*, const void*, const void*, void*, void*, void*,      \
                                  void*, void*, int, int, int, int, int, float, hipStream_t);         \
  template int triattn_output<T>(const void*, const void*, const void*, void*, int, int, int,      \
                                 hipStream_t);                                                     \
  template int transition_fwd<T>(const void*, const void*, const void*, const void*, const void*,  \
                                 const void*, void*, void*, int64_t, int, int, float,              \
                                 hipStream_t);                                                     \
  template int pair_bias_fwd<T>(const void*, const void*, const void*, const void*, void*, int,    \
                                int, int, float, hipStream_t);
PTX_INSTANTIATE(float)
PTX_INSTANTIATE(bf16_t)
#undef PTX_INSTANTIATE

}  // namespace ptx
