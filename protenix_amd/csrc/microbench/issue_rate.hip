// Issue-rate micro-benchmark for gfx950: how fast one SIMD retires the vector and matrix
// instructions the attention core is made of, alone and mixed, with 1, 2 and 4 waves per SIMD.
// Stand-alone program (not part of libprotenix_amd.so):
//   hipcc --offload-arch=gfx950 -O3 -Xclang -target-feature -Xclang -packed-fp32-ops \
//         protenix_amd/csrc/microbench/issue_rate.hip -o /tmp/issue_rate && /tmp/issue_rate
// Every kernel runs one workgroup per compute unit (256 x W threads: W waves on each of the 4
// SIMDs) and a loop of independent instructions (8 dependency chains per lane, so latency does
// not bound a single wave); the figure printed is nanoseconds per instruction and SIMD,
// total_time / (instructions a SIMD retires), and the same in units of the v_mul_f32 figure
// at four waves (one full-rate issue slot).
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

enum { kMul, kFma, kExp, kRcp, kCvtPk, kDot2, kShift, kMfma, kMfmaMul, kMfmaExp };

// VALU: per iteration, 8 independent instructions of one kind.
// kMfma: per iteration, 4 independent 32x32x16 bf16 MFMAs.
// kMfmaMul / kMfmaExp: per iteration, 2 independent MFMAs followed by NV independent v_mul /
// v_exp on other registers - the mix of one half tile of the attention core.
template <int KIND, int NV>
__global__ __launch_bounds__(1024) void loop_kernel(float* out, int iters) {
  float a[8];
  for (int i = 0; i < 8; ++i) a[i] = -0.001f * (threadIdx.x + i + 1);
  f32x16 acc[4];
  bf16x8 fa, fb;
  for (int i = 0; i < 8; ++i) {
    fa[i] = (__bf16)(0.001f * (threadIdx.x & 15));
    fb[i] = (__bf16)(0.002f * i);
  }
  for (int j = 0; j < 4; ++j)
    for (int i = 0; i < 16; ++i) acc[j][i] = 0.0f;
  for (int it = 0; it < iters; ++it) {
    if (KIND == kMfma) {
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc[j], 0, 0, 0);
    } else if (KIND == kMfmaMul || KIND == kMfmaExp) {
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc[j], 0, 0, 0);
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        if (KIND == kMfmaMul) asm volatile("v_mul_f32_e32 %0, %0, %0" : "+v"(a[i & 7]));
        else asm volatile("v_exp_f32_e32 %0, %0" : "+v"(a[i & 7]));
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (KIND == kMul) asm volatile("v_mul_f32_e32 %0, %0, %0" : "+v"(a[i]));
        if (KIND == kFma) asm volatile("v_fma_f32 %0, %0, %0, %0" : "+v"(a[i]));
        if (KIND == kExp) asm volatile("v_exp_f32_e32 %0, %0" : "+v"(a[i]));
        if (KIND == kRcp) asm volatile("v_rcp_f32_e32 %0, %0" : "+v"(a[i]));
        if (KIND == kCvtPk) asm volatile("v_cvt_pk_bf16_f32 %0, %0, %0" : "+v"(a[i]));
        if (KIND == kDot2) asm volatile("v_dot2c_f32_bf16_e32 %0, %0, %0" : "+v"(a[i]));
        if (KIND == kShift) asm volatile("v_lshlrev_b32_e32 %0, 16, %0" : "+v"(a[i]));
      }
    }
  }
  float s = 0;
  for (int i = 0; i < 8; ++i) s += a[i];
  for (int j = 0; j < 4; ++j) s += acc[j][0] + acc[j][7];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

static float g_unit = 0.0f;   // ns of one v_mul_f32 per SIMD at four waves

template <int KIND, int NV>
static double run(const char* name, float* d, int waves, int cus, double per_iter) {
  const int iters = 20000;
  hipEvent_t e0, e1;
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  loop_kernel<KIND, NV><<<cus, 256 * waves>>>(d, 200);
  (void)hipEventRecord(e0);
  loop_kernel<KIND, NV><<<cus, 256 * waves>>>(d, iters);
  (void)hipEventRecord(e1);
  (void)hipEventSynchronize(e1);
  float ms = 0;
  (void)hipEventElapsedTime(&ms, e0, e1);
  const double ns_iter = ms * 1e6 / ((double)iters * waves);   // per SIMD and loop iteration of one wave
  const double ns = ns_iter / per_iter;
  if (g_unit == 0.0f && KIND == kMul && waves == 4) g_unit = (float)ns;
  printf("%-34s waves/SIMD=%d  %8.3f ms  %7.2f ns per SIMD-iteration  %6.2f ns per instruction", name, waves,
         ms, ns_iter, ns);
  if (g_unit > 0) printf("  = %5.2f slots", ns / g_unit);
  printf("\n");
  return ns;
}

int main() {
  int cus = 256;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, 0) == hipSuccess) cus = prop.multiProcessorCount;
  printf("device: %s, %d compute units, clock %d MHz\n", prop.name, cus, prop.clockRate / 1000);
  float* d = nullptr;
  if (hipMalloc(&d, (size_t)cus * 1024 * 4) != hipSuccess) return 1;
  run<kMul, 0>("v_mul_f32", d, 4, cus, 8);
  for (int w : {1, 2, 4}) {
    run<kMul, 0>("v_mul_f32", d, w, cus, 8);
    run<kFma, 0>("v_fma_f32", d, w, cus, 8);
    run<kShift, 0>("v_lshlrev_b32 (bf16 -> f32)", d, w, cus, 8);
    run<kCvtPk, 0>("v_cvt_pk_bf16_f32", d, w, cus, 8);
    run<kDot2, 0>("v_dot2c_f32_bf16", d, w, cus, 8);
    run<kExp, 0>("v_exp_f32", d, w, cus, 8);
    run<kRcp, 0>("v_rcp_f32", d, w, cus, 8);
    run<kMfma, 0>("v_mfma_f32_32x32x16_bf16", d, w, cus, 4);
  }
  printf("-- mixes: per iteration 2 MFMA + n vector instructions, all independent; ns per iteration;\n"
         "   'sum' and 'max' are what no overlap and perfect overlap of the two pipes would give\n");
  for (int w : {1, 2, 4}) {
    const double mf = run<kMfma, 0>("  (2 MFMA alone: half of 4)", d, w, cus, 2);
    const double mu = run<kMul, 0>("  (v_mul_f32 alone)", d, w, cus, 8);
    const double ex = run<kExp, 0>("  (v_exp_f32 alone)", d, w, cus, 8);
    const double a8 = run<kMfmaMul, 8>("2 MFMA + 8 v_mul_f32", d, w, cus, 1);
    printf("      sum %.1f  max %.1f\n", mf + 8 * mu, mf > 8 * mu ? mf : 8 * mu);
    const double a32 = run<kMfmaMul, 32>("2 MFMA + 32 v_mul_f32", d, w, cus, 1);
    printf("      sum %.1f  max %.1f\n", mf + 32 * mu, mf > 32 * mu ? mf : 32 * mu);
    const double e16 = run<kMfmaExp, 16>("2 MFMA + 16 v_exp_f32", d, w, cus, 1);
    printf("      sum %.1f  max %.1f\n", mf + 16 * ex, mf > 16 * ex ? mf : 16 * ex);
    (void)a8; (void)a32; (void)e16;
  }
  (void)hipFree(d);
  return 0;
}
