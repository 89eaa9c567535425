// Triangle attention, last stage, with the gate formed here instead of in the projection kernel:
//   out(p) = [z(p) +] W_o ( sigmoid(W_g LN(z(p))) * o(p) )            (layers.py:380-396)
// for rows of 128 channels, 4 heads of 32, 16-bit arithmetic; z rows as T or fp32 (TZ).  The
// projection then writes no gate tensor and the attention core reads none: one write and one
// read of N^2 x 128 elements less per update, paid for with a LayerNorm of rows this kernel
// loads anyway (for the residual) and 32 more MFMAs per 32 rows.
//
// One wave takes 32 logical rows.  Everything stays in the MFMA fragment layout of a row
// (lane (n, g): row n, channels 16 kk + 8 g .. + 7 in K step kk): the weight rows are read
// permuted (MFMA row m <-> channel 16 (m >> 4) + 8 ((m >> 2) & 1) + 4 ((m >> 3) & 1) + (m & 3)
// of a 32-channel block), which makes accumulator registers 8 u .. 8 u + 7 of half-wave g the
// channels 16 u + 8 g .. + 7 - the same 8 channels as the lane's fragment of K step 2 c + u.
// So the gate multiplies the attention output in registers, the gated product is the next
// GEMM's operand as it stands, and the result meets the raw z row, still in registers, for
// the residual add and a 32-byte (16-byte) store per fragment.
// Both weight matrices sit in LDS as fragments (64 KB) for the life of a workgroup, whose
// waves walk over the row tiles.
#include "common.h"
#include "kernels.h"
#include "rowtile.h"
#include <type_traits>

namespace ptx {

namespace {

struct GateOutParams {
  const void* o;      // attention output, head-major [4][n_rows][32], T
  const void* z;      // pair tensor rows through zmap (LayerNorm input and residual)
  const void *ln_w, *ln_b, *w_g, *w_o;   // T; w_g [128 (h, d)][128], w_o [128][128 (h, d)]
  void* out;          // rows through zmap (may be z)
  RowMap zmap;
  int64_t n_rows;
  float eps;
  int add_residual;
};

constexpr int kGoWaves = 8;

__device__ __forceinline__ int perm32(int m) {
  return 16 * (m >> 4) + 8 * ((m >> 2) & 1) + 4 * ((m >> 3) & 1) + (m & 3);
}

}  // namespace

template <typename TZ>
__global__ __launch_bounds__((kGoWaves * 64), 1) void triattn_gate_out_kernel(GateOutParams p) {
  typedef bf16_t T;
  typedef Vec8<T>::type V8;
  typedef typename Vec8<TZ>::type VZ;
  __shared__ V8 lds_wg[4 * kKSteps][kWave];   // fragment (c, kk): gate channels 32 c .. + 31, K step kk
  __shared__ V8 lds_wo[4 * kKSteps][kWave];   // fragment (ob, kk): output channels 32 ob .. + 31
  __shared__ __attribute__((aligned(16))) float lds_affine[2][kC];
  typedef Cfg<TZ> C;
  typedef typename VecE<TZ>::type VE_t;
  __shared__ __attribute__((aligned(16))) TZ lds_stage[kGoWaves][32 * C::PITCH];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, g = lane >> 5;

  for (int f = wave; f < 4 * kKSteps; f += kGoWaves) {
    const int cb = f >> 3, kk = f & 7;
    const int64_t off = (int64_t)(32 * cb + perm32(n)) * kC + 16 * kk + 8 * g;
    lds_wg[f][lane] = load8<T>((const T*)p.w_g + off);
    lds_wo[f][lane] = load8<T>((const T*)p.w_o + off);
  }
  for (int c = threadIdx.x; c < kC; c += kGoWaves * 64) {
    lds_affine[0][c] = p.ln_w ? to_f32(((const T*)p.ln_w)[c]) : 1.0f;
    lds_affine[1][c] = p.ln_b ? to_f32(((const T*)p.ln_b)[c]) : 0.0f;
  }
  __syncthreads();

  const int64_t n_tiles = (p.n_rows + 31) >> 5;
  const int64_t tile_step = (int64_t)gridDim.x * kGoWaves;
  for (int64_t tile = (int64_t)blockIdx.x * kGoWaves + wave; tile < n_tiles; tile += tile_step) {
    // (opaque per tile: the weight fragments in LDS never change, and read through a
    // loop-invariant index all 64 of them would be hoisted into registers)
    int wl = lane;
    asm volatile("" : "+v"(wl));
    const int64_t pr = tile * 32 + n;
    const int64_t prc = pr < p.n_rows ? pr : p.n_rows - 1;
    const int64_t zoff = p.zmap(prc) + 8 * g;
    VZ zraw[kKSteps];
    V8 of[kKSteps];
#pragma unroll
    for (int kk = 0; kk < kKSteps; ++kk) zraw[kk] = load8<TZ>((const TZ*)p.z + zoff + 16 * kk);
#pragma unroll
    for (int kk = 0; kk < kKSteps; ++kk)
      of[kk] = load8<T>((const T*)p.o + ((int64_t)(kk >> 1) * p.n_rows + prc) * 32 + 16 * (kk & 1) + 8 * g);

    // LayerNorm of the row (fp32, both half-waves of a row exchange their sums), rounded to T
    V8 xf[kKSteps];
    {
      f32x8 v[kKSteps];
#pragma unroll
      for (int kk = 0; kk < kKSteps; ++kk) v[kk] = to_f32(zraw[kk]);
      normalize_row<T, kKSteps, float, false>(v, lds_affine[0], lds_affine[1], p.eps, g, xf);
    }
    // gate per head, applied to the attention output in place (both rounded to T like the
    // reference's sigmoid(linear_g(x)) and o * g)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      f32x16 accg;
#pragma unroll
      for (int r = 0; r < 16; ++r) accg[r] = 0.0f;
#pragma unroll
      for (int kk = 0; kk < kKSteps; ++kk) mma32(accg, lds_wg[c * kKSteps + kk][wl], xf[kk]);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const f32x8 ov = to_f32(of[2 * c + u]);
        f32x8 gated;
#pragma unroll
        for (int t = 0; t < 8; ++t)
          gated[t] = ov[t] * to_f32(from_f32<T>(sigmoidf_fast(accg[8 * u + t])));
        of[2 * c + u] = from_f32<T>(gated);
      }
    }
    // output projection, 32 channels at a time (lane <-> row, register 8 u + t <-> channel
    // 32 ob + 16 u + 8 g + t).  Each block is added to its part of the raw row and leaves
    // through the wave's LDS tile, so that a row's 32 channels are written as one run (a whole
    // 128-byte line of an fp32 row) by neighbouring lanes instead of in 32-byte pieces.
    TZ* st = lds_stage[wave];
#pragma unroll
    for (int ob = 0; ob < 4; ++ob) {
      f32x16 acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
      for (int kk = 0; kk < kKSteps; ++kk) mma32(acc, lds_wo[ob * kKSteps + kk][wl], of[kk]);
      wave_lds_sync();   // the previous block's read-back is done
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const f32x8 zr = to_f32(zraw[2 * ob + u]);
        f32x8 v;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          // the update is rounded to T first, as the module's output is; then z + update
          const float upd = to_f32(from_f32<T>(acc[8 * u + t]));
          v[t] = p.add_residual ? zr[t] + upd : upd;
        }
        const VZ pk = from_f32<TZ>(v);
        // 8-byte LDS stores (rows of the tile are 8-byte aligned)
        u32x2* d2 = reinterpret_cast<u32x2*>(st + n * C::PITCH + 16 * u + 8 * g);
        const u32x2* s2 = reinterpret_cast<const u32x2*>(&pk);
#pragma unroll
        for (int w8 = 0; w8 < (int)sizeof(VZ) / 8; ++w8) d2[w8] = s2[w8];
      }
      wave_lds_sync();
#pragma unroll
      for (int ps = 0; ps < C::NPASS; ++ps) {
        int mj, m0;
        stage_coord<TZ>(ps, lane, mj, m0);
        const int64_t prow = tile * 32 + mj;
        if (prow < p.n_rows)
          *reinterpret_cast<VE_t*>((TZ*)p.out + p.zmap(prow) + 32 * ob + m0) = stage_get_vec<TZ>(st, mj, m0);
      }
    }
  }
}

template <typename TZ>
int triattn_gate_output(const void* o, const void* z, const void* ln_w, const void* ln_b,
                        const void* w_g, const void* w_o, void* out, int n, int transposed,
                        int add_residual, float eps, hipStream_t stream) {
  if (n == 0) return 0;
  GateOutParams p = {};
  p.o = o;
  p.z = z;
  p.ln_w = ln_w;
  p.ln_b = ln_b;
  p.w_g = w_g;
  p.w_o = w_o;
  p.out = out;
  p.zmap.n_inner = n;
  p.zmap.stride_outer = transposed ? kC : (int64_t)n * kC;
  p.zmap.stride_inner = transposed ? (int64_t)n * kC : kC;
  p.n_rows = (int64_t)n * n;
  p.eps = eps;
  p.add_residual = add_residual;
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
  }
  const int64_t n_tiles = (p.n_rows + 31) >> 5;
  const int64_t blocks = std::min<int64_t>(cus, (n_tiles + kGoWaves - 1) / kGoWaves);
  triattn_gate_out_kernel<TZ><<<dim3((unsigned)blocks), dim3(kGoWaves * 64), 0, stream>>>(p);
  return 0;
}

template int triattn_gate_output<bf16_t>(const void*, const void*, const void*, const void*,
                                         const void*, const void*, void*, int, int, int, float,
                                         hipStream_t);
template int triattn_gate_output<float>(const void*, const void*, const void*, const void*,
                                        const void*, const void*, void*, int, int, int, float,
                                        hipStream_t);

}  // namespace ptx
