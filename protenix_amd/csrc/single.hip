// The single-representation track of a Pairformer block: small linear layers on [N, c_s]
// activations and the 16-head attention with pair bias.  A thousandth of the block's work,
// so these kernels aim at few launches and no intermediate round trips rather than at a
// roofline: operands go from global memory (L2-resident at these sizes) straight into MFMA
// fragments; a 32 x 32 output tile belongs to one workgroup.
//
//   linear_kernel           out = [res +] x W^T [+ bias], optionally with a tail of the output
//                           columns stored transposed (the attention's V^T); or, SwiGLU,
//                           out = silu(x W_a^T) * (x W_b^T)
//   single_attention_kernel flash-style softmax(q k^T * scale + bias) v per head, gated by
//                           sigmoid(g), logits never materialised
//
// MFMA conventions as in common.h.  In the attention kernel MFMA row m of a 32-key block stands
// for key 16*(m>>4) + 8*((m>>2)&1) + 4*((m>>3)&1) + (m&3), which makes accumulator registers
// 8*ks .. 8*ks+7 of half-wave g hold keys 16*ks + 8*g .. +7: the probabilities feed P.V as its
// B operand without a shuffle, and bias and V^T loads are runs of 8 consecutive keys.
#include "common.h"
#include "kernels.h"

namespace ptx {

enum { kEpiStore = 0, kEpiSwiGLU = 1 };

struct LinearParams {
  const void* x;      // [rows][k], row pitch ldx
  int64_t ldx;
  const void* w;      // [n_out][k]
  const void* w2;     // SwiGLU: the second matrix
  const void* bias;   // [bias_cols] or null: added to output columns < bias_cols
  int bias_cols;
  const void* res;    // [rows][n_out] (pitch ldr) or null
  int64_t ldr;
  void* out;          // [rows][*] (pitch ldo): output columns < split_col
  int64_t ldo;
  void* out_t;        // [n_out - split_col][ldt]: output columns >= split_col, transposed;
  int64_t ldt;        //   entries of rows in [rows, ldt) are written as zeros
  int split_col;      // multiple of 32 (n_out: nothing is transposed)
  int rows, k, n_out;
};

template <typename T> __device__ __forceinline__ typename Vec8<T>::type zero8() {
  typename Vec8<T>::type z;
#pragma unroll
  for (int t = 0; t < 8; ++t) z[t] = (T)0.0f;
  return z;
}

// One workgroup per 32 x 32 output tile; its kLinWaves waves each take a quarter of K and the
// partial tiles are summed through LDS in wave order.  The layers have 288 to 1152 tiles, a few
// per compute unit: with four small workgroups resident per unit, all of a unit's tiles are in
// flight together, their waves cover one another's load latency, and the fp32 MFMAs of a tile
// are spread over the unit's four SIMDs.
constexpr int kLinWaves = 4;

template <typename T, int EPI>
__global__ __launch_bounds__(kLinWaves * 64, 4) void linear_kernel(LinearParams p) {
  typedef typename Vec8<T>::type V8;
  typedef typename Vec4<T>::type V4;
  constexpr int NACC = EPI == kEpiSwiGLU ? 32 : 16;
  __shared__ float part[kLinWaves][NACC][kWave];
  const int lane = threadIdx.x & 63, ln = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col_blocks = (p.n_out + 31) >> 5;
  const int rb = blockIdx.x / col_blocks, cb = blockIdx.x - rb * col_blocks;
  const int row0 = rb * 32, col0 = cb * 32;
  const bool transposed = col0 >= p.split_col;   // the same for the whole workgroup
  const int xr = min(row0 + ln, p.rows - 1);
  const int wc = min(col0 + ln, p.n_out - 1);
  const T* xp = (const T*)p.x + (int64_t)xr * p.ldx + 8 * g;
  const T* wp = (const T*)p.w + (int64_t)wc * p.k + 8 * g;
  const T* wp2 = EPI == kEpiSwiGLU ? (const T*)p.w2 + (int64_t)wc * p.k + 8 * g : wp;

  // K steps of 16 (k is a multiple of 16), an equal share per wave
  const int steps = p.k >> 4;
  const int per_wave = (steps + kLinWaves - 1) / kLinWaves;
  const int s_begin = wave * per_wave, s_end = min(steps, s_begin + per_wave);

  f32x16 acc, acc2;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = acc2[r] = 0.0f;
  constexpr int KC = 3;   // K steps requested together
  for (int s0 = s_begin; s0 < s_end; s0 += KC) {
    V8 xa[KC], wa[KC], wb[KC];
#pragma unroll
    for (int s = 0; s < KC; ++s) {
      const int kk = 16 * min(s0 + s, steps - 1);   // steps beyond the slice re-read a valid one
      xa[s] = load8<T>(xp + kk);
      wa[s] = load8<T>(wp + kk);
      if (EPI == kEpiSwiGLU) wb[s] = load8<T>(wp2 + kk);
    }
#pragma unroll
    for (int s = 0; s < KC; ++s) {
      if (s0 + s < s_end) {
        if (transposed) {
          mma32(acc, xa[s], wa[s]);    // lane <-> column, register <-> row
        } else {
          mma32(acc, wa[s], xa[s]);    // lane <-> row, register <-> column
          if (EPI == kEpiSwiGLU) mma32(acc2, wb[s], xa[s]);
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    part[wave][r][lane] = acc[r];
    if (EPI == kEpiSwiGLU) part[wave][16 + r][lane] = acc2[r];
  }
  __syncthreads();

  // wave w finishes accumulator registers 4w .. 4w + 3 of every lane: four neighbouring output
  // columns (rows, for the transposed tail) 8*w + 4*g + {0 .. 3}
  f32x4 y = {0.0f, 0.0f, 0.0f, 0.0f}, y2 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int w = 0; w < kLinWaves; ++w) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      y[e] += part[w][4 * wave + e][lane];
      if (EPI == kEpiSwiGLU) y2[e] += part[w][16 + 4 * wave + e][lane];
    }
  }
  const int sub = 8 * wave + 4 * g;
  if (!transposed) {
    const int row = row0 + ln, col = col0 + sub;
    if (row < p.rows && col < p.n_out) {   // (n_out is a multiple of 4)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (EPI == kEpiSwiGLU) {
          // a and b rounded to T first, as the two linear layers of the reference do
          const float av = to_f32(from_f32<T>(y[e])), bv = to_f32(from_f32<T>(y2[e]));
          y[e] = to_f32(from_f32<T>(av * sigmoidf_fast(av))) * bv;
        } else if (p.bias && col + e < p.bias_cols) {
          y[e] += to_f32(((const T*)p.bias)[col + e]);
        }
      }
      if (p.res) {
        const f32x4 rv = to_f32(*reinterpret_cast<const V4*>((const T*)p.res + (int64_t)row * p.ldr + col));
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = to_f32(from_f32<T>(y[e])) + rv[e];
      }
      *reinterpret_cast<V4*>((T*)p.out + (int64_t)row * p.ldo + col) = from_f32<T>(y);
    }
  } else {
    const int col = col0 + ln, row = row0 + sub;
    if (col < p.n_out && row < p.ldt) {   // (ldt is a multiple of 4)
#pragma unroll
      for (int e = 0; e < 4; ++e) y[e] = row + e < p.rows ? y[e] : 0.0f;
      *reinterpret_cast<V4*>((T*)p.out_t + (int64_t)(col - p.split_col) * p.ldt + row) = from_f32<T>(y);
    }
  }
}

template <typename T>
int linear_fwd(const void* x, const void* w, const void* bias, int bias_cols, const void* res,
               void* out, void* out_t, int split_col, int64_t ldt, int rows, int k, int n_out,
               hipStream_t stream) {
  if (rows == 0 || n_out == 0) return 0;
  LinearParams p = {};
  p.x = x;
  p.ldx = k;
  p.w = w;
  p.bias = bias;
  p.bias_cols = bias_cols;
  p.res = res;
  p.ldr = n_out;
  p.out = out;
  p.ldo = split_col < n_out ? split_col : n_out;
  p.out_t = out_t;
  p.ldt = ldt;
  p.split_col = split_col < n_out ? split_col : n_out;
  p.rows = rows;
  p.k = k;
  p.n_out = n_out;
  const int64_t row_span = (p.split_col < n_out && ldt > rows) ? ldt : rows;
  const int64_t tiles = ((row_span + 31) / 32) * ((n_out + 31) / 32);
  linear_kernel<T, kEpiStore><<<dim3((unsigned)tiles), dim3(kLinWaves * 64), 0, stream>>>(p);
  return 0;
}

template <typename T>
int swiglu_fwd(const void* x, const void* w_a, const void* w_b, void* out, int rows, int k,
               int hidden, hipStream_t stream) {
  if (rows == 0 || hidden == 0) return 0;
  LinearParams p = {};
  p.x = x;
  p.ldx = k;
  p.w = w_a;
  p.w2 = w_b;
  p.out = out;
  p.ldo = hidden;
  p.split_col = hidden;
  p.rows = rows;
  p.k = k;
  p.n_out = hidden;
  const int64_t tiles = (((int64_t)rows + 31) / 32) * ((hidden + 31) / 32);
  linear_kernel<T, kEpiSwiGLU><<<dim3((unsigned)tiles), dim3(kLinWaves * 64), 0, stream>>>(p);
  return 0;
}

// ---------------------------------------------------------------------------------------
struct SingleAttnParams {
  const void* q;      // [n][ld]: heads * d channels per row, head-major
  const void* k;
  const void* g;      // gate logits, or null
  int64_t ld;
  const void* vt;     // [heads * d][ldt], keys in [n, ldt) hold zeros
  int64_t ldt;
  const void* bias;   // [heads][n][n], fp32 (bias_f32) or T, or null
  int bias_f32;
  int bias_vec;       // n is a multiple of 8: bias rows can be read as 16-byte vectors
  void* out;          // [n][ldo]
  int64_t ldo;
  int n, heads, d;
  float scale;
};

__device__ __forceinline__ int key_of_mfma_row(int m) {
  return 16 * (m >> 4) + 8 * ((m >> 2) & 1) + 4 * ((m >> 3) & 1) + (m & 3);
}

// One workgroup per (32 queries, head); its kAttnWaves waves take every kAttnWaves-th block of
// 32 keys each and merge their partial results through LDS in a fixed order: the chain of
// dependent loads a wave walks through is a quarter as long.
constexpr int kAttnWaves = 4;

template <typename T>
__global__ __launch_bounds__(kAttnWaves * 64) void single_attention_kernel(SingleAttnParams p) {
  typedef typename Vec8<T>::type V8;
  typedef typename Vec4<T>::type V4;
  constexpr float kL2e = 1.4426950408889634f;
  __shared__ float part_o[kAttnWaves][16][kWave];
  __shared__ float part_ml[kAttnWaves][2][kWave];
  const int lane = threadIdx.x & 63, ln = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int h = blockIdx.y, q0 = blockIdx.x * 32;
  const int n = p.n, d = p.d;
  const int qi = min(q0 + ln, n - 1);
  const T* qp = (const T*)p.q + (int64_t)qi * p.ld + h * d;
  // q fragments (B operand: lane <-> query, slots <-> channels 16*kk + 8*g .. +7), in log2 units
  V8 qf[2];
  const float qs = p.scale * kL2e;
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    qf[kk] = zero8<T>();
    if (16 * kk + 8 * g < d) {
      f32x8 v = to_f32(load8<T>(qp + 16 * kk + 8 * g));
#pragma unroll
      for (int t = 0; t < 8; ++t) v[t] *= qs;
      qf[kk] = from_f32<T>(v);
    }
  }
  const int krow = key_of_mfma_row(ln);
  const T* kbase = (const T*)p.k + h * d;
  const T* vrow = (const T*)p.vt + (int64_t)(h * d + min(ln, d - 1)) * p.ldt;
  const float* bf = (const float*)p.bias + ((int64_t)h * n + qi) * n;
  const T* bt = (const T*)p.bias + ((int64_t)h * n + qi) * n;

  f32x16 acc_o;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc_o[r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  for (int key0 = 32 * wave; key0 < n; key0 += 32 * kAttnWaves) {
    const bool tail = key0 + 32 > n;   // the same for the whole wave
    // K fragments (A operand: lane <-> key, slots <-> channels)
    const T* kp = kbase + (int64_t)min(key0 + krow, n - 1) * p.ld;
    V8 kf[2], vf[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      kf[kk] = zero8<T>();
      if (16 * kk + 8 * g < d) kf[kk] = load8<T>(kp + 16 * kk + 8 * g);
    }
    // V^T fragments (A operand: lane <-> channel, slots <-> keys key0 + 16*ks + 8*g .. +7)
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      vf[ks] = zero8<T>();
      if (ln < d) vf[ks] = load8<T>(vrow + key0 + 16 * ks + 8 * g);
    }
    // logits start from the bias: registers 8*ks + t <-> keys key0 + 16*ks + 8*g + t
    f32x16 s;
    if (p.bias && !tail && p.bias_vec) {
      // (n is a multiple of 8: the 8-key runs are 16-byte aligned vectors)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const int key = key0 + 16 * ks + 8 * g;
        f32x8 b;
        if (p.bias_f32) {
          const f32x4 b0 = *reinterpret_cast<const f32x4*>(bf + key);
          const f32x4 b1 = *reinterpret_cast<const f32x4*>(bf + key + 4);
          b = __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
          b = to_f32(load8<T>(bt + key));
        }
#pragma unroll
        for (int t = 0; t < 8; ++t) s[8 * ks + t] = b[t] * kL2e;
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          const int key = key0 + 16 * ks + 8 * g + t;
          float b = 0.0f;
          if (p.bias) {
            const int kc = min(key, n - 1);
            b = p.bias_f32 ? bf[kc] : to_f32(bt[kc]);
          }
          s[8 * ks + t] = b * kL2e;
        }
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) mma32(s, kf[kk], qf[kk]);
    if (tail) {
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int t = 0; t < 8; ++t)
          if (key0 + 16 * ks + 8 * g + t >= n) s[8 * ks + t] = -INFINITY;
    }
    float mx = s[0];
#pragma unroll
    for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s[r]);
    mx = fmaxf(mx, swap32(mx));
    const float m_new = fmaxf(m_run, mx);     // finite: every block holds at least one key
    const float alpha = fast_exp2(m_run - m_new);
    m_run = m_new;
    float psum = 0.0f;
    V8 pf[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      f32x8 p8;
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        p8[t] = fast_exp2(s[8 * ks + t] - m_new);
        psum += p8[t];
      }
      pf[ks] = from_f32<T>(p8);
    }
    l_run = l_run * alpha + psum;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc_o[r] *= alpha;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) mma32(acc_o, vf[ks], pf[ks]);   // lane <-> query, register <-> channel
  }

  // merge the waves' partial results (a wave without key blocks contributes m = -inf, l = 0)
  l_run += swap32(l_run);
#pragma unroll
  for (int r = 0; r < 16; ++r) part_o[wave][r][lane] = acc_o[r];
  part_ml[wave][0][lane] = m_run;
  part_ml[wave][1][lane] = l_run;
  __syncthreads();
  if (wave != 0) return;
  float m_all = part_ml[0][0][lane];
#pragma unroll
  for (int w = 1; w < kAttnWaves; ++w) m_all = fmaxf(m_all, part_ml[w][0][lane]);
  l_run = 0.0f;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc_o[r] = 0.0f;
#pragma unroll
  for (int w = 0; w < kAttnWaves; ++w) {
    const float f = fast_exp2(part_ml[w][0][lane] - m_all);   // wave 0 always has a block: m_all is finite
    l_run += part_ml[w][1][lane] * f;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc_o[r] += part_o[w][r][lane] * f;
  }
  const float inv = fast_rcp(l_run);
  if (q0 + ln < n) {
    const T* gp = p.g ? (const T*)p.g + (int64_t)qi * p.ld + h * d : nullptr;
    T* op = (T*)p.out + (int64_t)qi * p.ldo + h * d;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int c0 = 8 * a + 4 * g;
      if (c0 < d) {   // (d is a multiple of 4)
        f32x4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = to_f32(from_f32<T>(acc_o[4 * a + e] * inv));
        if (gp) {
          const f32x4 gv = to_f32(*reinterpret_cast<const V4*>(gp + c0));
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] *= to_f32(from_f32<T>(sigmoidf_fast(gv[e])));
        }
        *reinterpret_cast<V4*>(op + c0) = from_f32<T>(v);
      }
    }
  }
}

template <typename T>
int single_attention_fwd(const void* q, const void* k, const void* vt, const void* g,
                         const void* bias, int bias_f32, void* out, int n, int heads, int d,
                         int64_t ld, int64_t ldt, int64_t ldo, float scale, hipStream_t stream) {
  if (n == 0 || heads == 0) return 0;
  SingleAttnParams p = {};
  p.q = q;
  p.k = k;
  p.g = g;
  p.ld = ld;
  p.vt = vt;
  p.ldt = ldt;
  p.bias = bias;
  p.bias_f32 = bias_f32;
  p.bias_vec = (n % 8 == 0) && (((uintptr_t)bias & 15) == 0);
  p.out = out;
  p.ldo = ldo;
  p.n = n;
  p.heads = heads;
  p.d = d;
  p.scale = scale;
  single_attention_kernel<T><<<dim3((n + 31) / 32, heads), dim3(kAttnWaves * 64), 0, stream>>>(p);
  return 0;
}

#define PTX_INSTANTIATE_SINGLE(T)                                                                 \
  template int linear_fwd<T>(const void*, const void*, const void*, int, const void*, void*,     \
                             void*, int, int64_t, int, int, int, hipStream_t);                   \
  template int swiglu_fwd<T>(const void*, const void*, const void*, void*, int, int, int,        \
                             hipStream_t);                                                       \
  template int single_attention_fwd<T>(const void*, const void*, const void*, const void*,       \
                                       const void*, int, void*, int, int, int, int64_t, int64_t, \
                                       int64_t, float, hipStream_t);
PTX_INSTANTIATE_SINGLE(float)
PTX_INSTANTIATE_SINGLE(bf16_t)
#undef PTX_INSTANTIATE_SINGLE

}  // namespace ptx
