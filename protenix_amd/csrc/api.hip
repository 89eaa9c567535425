// extern "C" boundary of libprotenix_amd.so: argument validation, dtype
// dispatch, launch-error capture.  See include/protenix_amd.h for the contract.
#include <stdarg.h>
#include <stdio.h>

#include <mutex>

#include "../../include/protenix_amd.h"
#include "common.h"
#include "kernels.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int after_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(PTX_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  g_err[0] = 0;
  return PTX_OK;
}

bool dtype_ok(int dtype) { return dtype == PTX_F32 || dtype == PTX_BF16; }
// the stand-alone LayerNorm also takes IEEE half, like the reference's kernel
bool dtype_ok_ln(int dtype) { return dtype_ok(dtype) || dtype == PTX_F16; }
// entry points that read or write the residual stream also take PTX_MIXED
bool dtype_ok_z(int dtype) { return dtype_ok(dtype) || dtype == PTX_MIXED; }

size_t esize(int dtype) { return dtype == PTX_BF16 ? 2 : 4; }

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

#define PTX_REQUIRE(cond, code, ...) \
  do {                               \
    if (!(cond)) return fail(code, __VA_ARGS__); \
  } while (0)

#define PTX_DISPATCH_LN(dtype, CALL)     \
  do {                                   \
    if ((dtype) == PTX_F16) {            \
      typedef ptx::f16_t T;              \
      CALL;                              \
    } else if ((dtype) == PTX_BF16) {    \
      typedef ptx::bf16_t T;             \
      CALL;                              \
    } else {                             \
      typedef float T;                   \
      CALL;                              \
    }                                    \
  } while (0)

#define PTX_DISPATCH(dtype, CALL)        \
  do {                                   \
    if ((dtype) == PTX_BF16) {           \
      typedef ptx::bf16_t T;             \
      CALL;                              \
    } else {                             \
      typedef float T;                   \
      CALL;                              \
    }                                    \
  } while (0)

// Partial sums of ptx_layernorm_bwd_static: 2 x 1024 rows of fp32 partial column sums for rows
// of at most kStaticLnCols columns (8 MiB per GPU, held until the process ends).  In host
// code the array's name is only a handle; the device address comes from hipGetSymbolAddress,
// once per device, and is what the kernels receive.
constexpr int kStaticLnCols = 1024;
constexpr int kStaticLnParts = 1024;   // = the most partial rows layernorm_bwd ever writes
constexpr int kMaxDevices = 64;
static __device__ __align__(256) float scratch[2 * kStaticLnParts * kStaticLnCols];
float* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_lock;

// Device address of `scratch` on the current device (nullptr + error text on failure).
float* scratch_on_current_device() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    fail(PTX_ERR_LAUNCH, "layernorm_bwd_static: hipGetDevice: %s (device %d)",
         hipGetErrorString(e), dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      fail(PTX_ERR_LAUNCH, "layernorm_bwd_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = (float*)p;
  }
  return g_scratch_ptr[dev];
}

// T = arithmetic type, TZ = storage type of the residual stream (see PTX_MIXED)
#define PTX_DISPATCH_Z(dtype, CALL)      \
  do {                                   \
    if ((dtype) == PTX_BF16) {           \
      typedef ptx::bf16_t T;             \
      typedef ptx::bf16_t TZ;            \
      CALL;                              \
    } else if ((dtype) == PTX_MIXED) {   \
      typedef ptx::bf16_t T;             \
      typedef float TZ;                  \
      CALL;                              \
    } else {                             \
      typedef float T;                   \
      typedef float TZ;                  \
      CALL;                              \
    }                                    \
  } while (0)

}  // namespace

extern "C" {

PTX_API int ptx_version(void) { return PTX_ABI_VERSION; }

PTX_API const char* ptx_last_error_string(void) { return g_err; }

PTX_API int ptx_key_pitch(int n) { return n <= 0 ? 0 : ((n + 63) / 64) * 64; }
PTX_API int64_t ptx_trimul_operand_elems(int n, int c_hidden) {
  if (n <= 0 || c_hidden <= 0) return 0;
  return (int64_t)c_hidden * (((n + 31) / 32) * 32) * ptx_key_pitch(n);
}
PTX_API int64_t ptx_triattn_kv_elems(int n, int heads) {
  if (n <= 0 || heads <= 0) return 0;
  return (int64_t)heads * n * ptx_key_pitch(n) * 32;
}
PTX_API int64_t ptx_triattn_bias_elems(int n, int heads) {
  if (n <= 0 || heads <= 0) return 0;
  return (int64_t)heads * (((n + 31) / 32) * 32) * ptx_key_pitch(n);
}

PTX_API int ptx_layernorm_fwd(const void* x, const void* gamma, const void* beta, void* y, float* mean,
                      float* rstd, int64_t rows, int cols, float eps, int dtype, void* stream) {
  PTX_REQUIRE(dtype_ok_ln(dtype), PTX_ERR_BAD_ARG, "layernorm: unknown dtype %d", dtype);
  PTX_REQUIRE(rows >= 0 && cols > 0, PTX_ERR_BAD_ARG, "layernorm: rows=%lld cols=%d",
              (long long)rows, cols);
  if (rows == 0) return PTX_OK;
  PTX_REQUIRE(x && y, PTX_ERR_BAD_ARG, "layernorm: null x or y");
  PTX_REQUIRE(rows < ((int64_t)1 << 31), PTX_ERR_UNSUPPORTED, "layernorm: rows=%lld too large",
              (long long)rows);
  PTX_DISPATCH_LN(dtype, ptx::layernorm_fwd<T>((const T*)x, (const T*)gamma, (const T*)beta, (T*)y,
                                               mean, rstd, rows, cols, eps, (hipStream_t)stream));
  return after_launch("layernorm");
}

PTX_API int64_t ptx_layernorm_bwd_workspace_elems(int64_t rows, int cols) {
  return ptx::layernorm_bwd_workspace_elems(rows, cols);
}

PTX_API int ptx_layernorm_bwd(const void* dout, const void* x, const float* mean, const float* rstd,
                      const void* gamma, void* dx, void* dgamma, void* dbeta, float* workspace,
                      int64_t rows, int cols, int dtype, void* stream) {
  PTX_REQUIRE(dtype_ok_ln(dtype), PTX_ERR_BAD_ARG, "layernorm_bwd: unknown dtype %d", dtype);
  PTX_REQUIRE(rows >= 0 && cols > 0, PTX_ERR_BAD_ARG, "layernorm_bwd: rows=%lld cols=%d",
              (long long)rows, cols);
  PTX_REQUIRE(rows < ((int64_t)1 << 31), PTX_ERR_UNSUPPORTED,
              "layernorm_bwd: rows=%lld too large", (long long)rows);
  PTX_REQUIRE(!(dgamma || dbeta) || workspace, PTX_ERR_BAD_ARG,
              "layernorm_bwd: dgamma / dbeta need the workspace");
  if (rows == 0 && !dgamma && !dbeta) return PTX_OK;
  if (rows > 0)
    PTX_REQUIRE(dout && x && mean && rstd && dx, PTX_ERR_BAD_ARG, "layernorm_bwd: null pointer");
  PTX_DISPATCH_LN(dtype, ptx::layernorm_bwd<T>((const T*)dout, (const T*)x, mean, rstd,
                                               (const T*)gamma, (T*)dx, (T*)dgamma, (T*)dbeta,
                                               workspace, rows, cols, (hipStream_t)stream));
  return after_launch("layernorm_bwd");
}

PTX_API int ptx_layernorm_bwd_static(const void* dout, const void* x, const float* mean,
                                     const float* rstd, const void* gamma, void* dx, void* dgamma,
                                     void* dbeta, int64_t rows, int cols, int dtype, void* stream) {
  PTX_REQUIRE(cols <= kStaticLnCols, PTX_ERR_UNSUPPORTED,
              "layernorm_bwd_static: cols=%d exceeds the built-in scratch (%d columns at most); "
              "use ptx_layernorm_bwd with a workspace",
              cols, kStaticLnCols);
  PTX_REQUIRE(cols > 0 && ptx::layernorm_bwd_workspace_elems(1, cols) <=
                              (int64_t)2 * kStaticLnParts * kStaticLnCols,
              PTX_ERR_BAD_ARG, "layernorm_bwd_static: cols=%d", cols);
  float* ws = nullptr;
  if (dgamma || dbeta) {
    ws = scratch_on_current_device();
    if (!ws) return PTX_ERR_LAUNCH;
  }
  return ptx_layernorm_bwd(dout, x, mean, rstd, gamma, dx, dgamma, dbeta, ws, rows, cols, dtype,
                           stream);
}

// Pair-row widths the kernels are built for: c_z = 64 or 128 with hidden widths (c_hidden,
// heads * 32) of 128, or c_z = 256 in bf16 arithmetic with hidden widths of 256.
static bool pair_width_ok(int c_z, int hidden, int dtype) {
  if (c_z == 64 || c_z == 128) return hidden == 128;
  return c_z == 256 && hidden == 256 && dtype != PTX_F32;   // (bf16 arithmetic: PTX_BF16, PTX_MIXED)
}
static const char* const kWidthMsg =
    "only c_z = 64 / 128 with hidden width 128, or c_z = 256 with hidden width 256 in bf16 arithmetic, is built";

PTX_API int ptx_trimul_project(const void* z, const void* mask, const void* ln_w, const void* ln_b,
                       const void* w_ap, const void* w_ag, const void* w_bp, const void* w_bg,
                       void* a, void* b, int n, int c_z, int c_hidden, int k_pitch, int incoming,
                       float eps, int dtype, void* stream) {
  PTX_REQUIRE(dtype_ok_z(dtype), PTX_ERR_BAD_ARG, "trimul_project: unknown dtype %d", dtype);
  PTX_REQUIRE(n >= 0, PTX_ERR_BAD_ARG, "trimul_project: n=%d", n);
  PTX_REQUIRE(pair_width_ok(c_z, c_hidden, dtype), PTX_ERR_UNSUPPORTED,
              "trimul_project: %s (got c_z=%d c_hidden=%d)", kWidthMsg, c_z, c_hidden);
  PTX_REQUIRE(k_pitch == ptx_key_pitch(n), PTX_ERR_BAD_ARG,
              "trimul_project: k_pitch=%d, expected ptx_key_pitch(%d)=%d", k_pitch, n,
              ptx_key_pitch(n));
  PTX_REQUIRE(n <= 8192, PTX_ERR_UNSUPPORTED, "trimul_project: n=%d too large (8192 at most)", n);
  if (n == 0) return PTX_OK;
  PTX_REQUIRE(z && w_ap && w_ag && w_bp && w_bg && a && b, PTX_ERR_BAD_ARG,
              "trimul_project: null pointer");
  PTX_REQUIRE(aligned16(z) && aligned16(w_ap) && aligned16(w_ag) && aligned16(w_bp) &&
                  aligned16(w_bg) && aligned16(a) && aligned16(b) && (!ln_w || aligned16(ln_w)) &&
                  (!ln_b || aligned16(ln_b)),
              PTX_ERR_BAD_ARG, "trimul_project: pointers must be 16-byte aligned");
  PTX_DISPATCH_Z(dtype, (ptx::trimul_project<T, TZ>)(z, mask, ln_w, ln_b, w_ap, w_ag, w_bp, w_bg, a, b, n,
                                             c_z, k_pitch, incoming, eps, (hipStream_t)stream));
  return after_launch("trimul_project");
}

PTX_API int ptx_trimul_contract(const void* a, const void* b, void* x, int n, int c, int k_pitch, int dtype,
                        void* stream) {
  if (dtype == PTX_MIXED) dtype = PTX_BF16;   // no residual-stream tensor here
  PTX_REQUIRE(dtype_ok(dtype), PTX_ERR_BAD_ARG, "trimul_contract: unknown dtype %d", dtype);
  PTX_REQUIRE(n >= 0 && c >= 0, PTX_ERR_BAD_ARG, "trimul_contract: n=%d c=%d", n, c);
  PTX_REQUIRE(k_pitch == ptx_key_pitch(n), PTX_ERR_BAD_ARG,
              "trimul_contract: k_pitch=%d, expected %d", k_pitch, ptx_key_pitch(n));
  PTX_REQUIRE(n < 32768, PTX_ERR_UNSUPPORTED, "trimul_contract: n=%d too large", n);
  if (n == 0 || c == 0) return PTX_OK;
  PTX_REQUIRE(a && b && x, PTX_ERR_BAD_ARG, "trimul_contract: null pointer");
  PTX_REQUIRE(aligned16(a) && aligned16(b), PTX_ERR_BAD_ARG,
              "trimul_contract: a and b must be 16-byte aligned");
  PTX_DISPATCH(dtype, ptx::nt_gemm_batched<T>((const T*)a, (const T*)b, (T*)x, n, k_pitch, c,
                                              (hipStream_t)stream));
  return after_launch("trimul_contract");
}

PTX_API int ptx_trimul_output(const void* x, const void* z, const void* ln_in_w, const void* ln_in_b,
                      const void* ln_out_w, const void* ln_out_b, const void* w_z,
                      const void* w_g, void* out, int n, int c_z, int c_hidden, int add_residual,
                      float eps, int dtype, void* stream) {
  PTX_REQUIRE(dtype_ok_z(dtype), PTX_ERR_BAD_ARG, "trimul_output: unknown dtype %d", dtype);
  PTX_REQUIRE(n >= 0, PTX_ERR_BAD_ARG, "trimul_output: n=%d", n);
  PTX_REQUIRE(pair_width_ok(c_z, c_hidden, dtype), PTX_ERR_UNSUPPORTED,
              "trimul_output: %s (got c_z=%d c_hidden=%d)", kWidthMsg, c_z, c_hidden);
  PTX_REQUIRE(n < 32768, PTX_ERR_UNSUPPORTED, "trimul_output: n=%d too large", n);
  if (n == 0) return PTX_OK;
  PTX_REQUIRE(x && z && ln_out_w && ln_out_b && w_z && w_g && out, PTX_ERR_BAD_ARG,
              "trimul_output: null pointer");
  PTX_REQUIRE(aligned16(x) && aligned16(out) && aligned16(z) && aligned16(w_z) &&
                  aligned16(w_g) && aligned16(ln_out_w) && aligned16(ln_out_b) &&
                  (!ln_in_w || aligned16(ln_in_w)) &&
                  (!ln_in_b || aligned16(ln_in_b)),
              PTX_ERR_BAD_ARG, "trimul_output: pointers must be 16-byte aligned");
  PTX_DISPATCH_Z(dtype, (ptx::trimul_output<T, TZ>)(x, z, ln_in_w, ln_in_b, ln_out_w, ln_out_b, w_z, w_g,
                                            out, n, c_z, add_residual, eps, (hipStream_t)stream));
  return after_launch("trimul_output");
}

PTX_API int64_t ptx_triangle_multiplicative_update_workspace_elems(int n, int c_hidden) {
  if (n <= 0 || c_hidden <= 0) return 0;
  // a, b (fragment order) and the channel-major product x
  return 2 * ptx_trimul_operand_elems(n, c_hidden) + (int64_t)c_hidden * n * n;
}

PTX_API int ptx_triangle_multiplicative_update(
    const void* x, int incoming, const void* mask, const void* norm_in_weight,
    const void* norm_in_bias, const void* p_in_weight, const void* g_in_weight,
    const void* norm_out_weight, const void* norm_out_bias, const void* p_out_weight,
    const void* g_out_weight, void* out, void* workspace, int n, int c_z, int c_hidden,
    int add_residual, float eps, int dtype, void* stream) {
  PTX_REQUIRE(dtype_ok_z(dtype), PTX_ERR_BAD_ARG, "triangle_multiplicative_update: unknown dtype %d", dtype);
  PTX_REQUIRE(n >= 0, PTX_ERR_BAD_ARG, "triangle_multiplicative_update: n=%d", n);
  PTX_REQUIRE(pair_width_ok(c_z, c_hidden, dtype), PTX_ERR_UNSUPPORTED,
              "triangle_multiplicative_update: %s (got c_z=%d c_hidden=%d)", kWidthMsg, c_z, c_hidden);
  if (n == 0) return PTX_OK;
  PTX_REQUIRE(x && p_in_weight && g_in_weight && p_out_weight && g_out_weight && out && workspace,
              PTX_ERR_BAD_ARG, "triangle_multiplicative_update: null pointer");
  PTX_REQUIRE(aligned16(workspace), PTX_ERR_BAD_ARG,
              "triangle_multiplicative_update: workspace must be 16-byte aligned");
  // p_in_weight = [W_a_p ; W_b_p], g_in_weight = [W_a_g ; W_b_g], each [2 * c_hidden][c_z]
  const size_t es = esize(dtype == PTX_MIXED ? PTX_BF16 : dtype);
  const size_t half = (size_t)c_hidden * c_z * es;
  const char* w_p = (const char*)p_in_weight;
  const char* w_g = (const char*)g_in_weight;
  const int64_t n_op = ptx_trimul_operand_elems(n, c_hidden);
  char* a = (char*)workspace;
  char* b = a + n_op * es;
  char* xc = b + n_op * es;
  const int pitch = ptx_key_pitch(n);
  int rc = ptx_trimul_project(x, mask, norm_in_weight, norm_in_bias, w_p, w_g, w_p + half, w_g + half, a,
                              b, n, c_z, c_hidden, pitch, incoming, eps, dtype, stream);
  if (rc != PTX_OK) return rc;
  rc = ptx_trimul_contract(a, b, xc, n, c_hidden, pitch, dtype, stream);
  if (rc != PTX_OK) return rc;
  return ptx_trimul_output(xc, x, norm_in_weight, norm_in_bias, norm_out_weight, norm_out_bias,
                           p_out_weight, g_out_weight, out, n, c_z, c_hidden, add_residual, eps, dtype,
                           stream);
}

PTX_API int ptx_triattn_project(const void* z, const void* ln_w, const void* ln_b, const void* w_q,
                        const void* w_k, const void* w_v, const void* w_g, const void* w_b,
                        void* q, void* k, void* vt, void* g, void* tri_bias, int n, int c_in,
                        int heads, int d, int key_pitch, int transposed, float eps, int dtype,
                        void* stream) {
  PTX_REQUIRE(dtype_ok_z(dtype), PTX_ERR_BAD_ARG, "triattn_project: unknown dtype %d", dtype);
  PTX_REQUIRE(n >= 0, PTX_ERR_BAD_ARG, "triattn_project: n=%d", n);
  PTX_REQUIRE(d == 32 && heads > 0 && heads <= 8 && pair_width_ok(c_in, heads * 32, dtype),
              PTX_ERR_UNSUPPORTED, "triattn_project: %s, head dim 32 (got c_in=%d heads=%d d=%d)",
              kWidthMsg, c_in, heads, d);
  PTX_REQUIRE(key_pitch == ptx_key_pitch(n), PTX_ERR_BAD_ARG,
              "triattn_project: key_pitch=%d, expected %d", key_pitch, ptx_key_pitch(n));
  PTX_REQUIRE(n <= 8192, PTX_ERR_UNSUPPORTED, "triattn_project: n=%d too large (8192 at most)", n);
  if (n == 0) return PTX_OK;
  PTX_REQUIRE(z && w_q && w_k && w_v && w_g && w_b && q && k && vt && tri_bias,
              PTX_ERR_BAD_ARG, "triattn_project: null pointer");
  // without a gate output: where ptx_triattn_gate_output exists to form the gate instead
  PTX_REQUIRE(g || (c_in == 128 && heads == 4 && dtype != PTX_F32), PTX_ERR_UNSUPPORTED,
              "triattn_project: g = NULL needs c_in = 128, 4 heads and 16-bit arithmetic");
  PTX_REQUIRE(aligned16(z) && aligned16(w_q) && aligned16(w_k) && aligned16(w_v) &&
                  aligned16(w_g) && aligned16(w_b) && aligned16(q) && aligned16(k) &&
                  aligned16(vt) && (!g || aligned16(g)) && aligned16(tri_bias) &&
                  (!ln_w || aligned16(ln_w)) &&
                  (!ln_b || aligned16(ln_b)),
              PTX_ERR_BAD_ARG, "triattn_project: pointers must be 16-byte aligned");
  PTX_DISPATCH_Z(dtype, (ptx::triattn_project<T, TZ>)(z, ln_w, ln_b, w_q, w_k, w_v, w_g, w_b, q, k, vt, g,
                                              tri_bias, n, c_in, heads, d, key_pitch, transposed, eps,
                                              (hipStream_t)stream));
  return after_launch("triattn_project");
}

static int triattn_fwd_checked(const char* what, const void* q, const void* k, const void* vt,
                               const void* g, const void* tri_bias, const void* mask, void* o, int n,
                               int heads, int d, int key_pitch, int mask_transposed, float inf,
                               int row_begin, int row_count, int n_keys, int dtype, void* stream) {
  if (dtype == PTX_MIXED) dtype = PTX_BF16;   // no residual-stream tensor here
  PTX_REQUIRE(dtype_ok(dtype), PTX_ERR_BAD_ARG, "%s: unknown dtype %d", what, dtype);
  PTX_REQUIRE(n >= 0 && heads >= 0, PTX_ERR_BAD_ARG, "%s: n=%d heads=%d", what, n, heads);
  PTX_REQUIRE(d == 32, PTX_ERR_UNSUPPORTED, "%s: only head dim 32 is built (got %d)", what, d);
  PTX_REQUIRE(key_pitch == ptx_key_pitch(n), PTX_ERR_BAD_ARG, "%s: key_pitch=%d, expected %d", what,
              key_pitch, ptx_key_pitch(n));
  PTX_REQUIRE(n < 32768, PTX_ERR_UNSUPPORTED, "%s: n=%d too large", what, n);
  PTX_REQUIRE(row_begin >= 0 && row_count >= 0 && row_begin <= n - row_count, PTX_ERR_BAD_ARG,
              "%s: rows %d .. +%d of %d", what, row_begin, row_count, n);
  PTX_REQUIRE(n_keys >= (n > 0) && n_keys <= n, PTX_ERR_BAD_ARG, "%s: n_keys=%d of %d", what, n_keys, n);
  if (n == 0 || heads == 0 || row_count == 0) return PTX_OK;
  PTX_REQUIRE(q && k && vt && tri_bias && o, PTX_ERR_BAD_ARG, "%s: null pointer", what);
  PTX_REQUIRE(aligned16(q) && aligned16(k) && aligned16(vt) && (!g || aligned16(g)) &&
                  aligned16(tri_bias) && aligned16(o),
              PTX_ERR_BAD_ARG, "%s: pointers must be 16-byte aligned", what);
  PTX_DISPATCH(dtype, ptx::triattn_fwd<T>((const T*)q, (const T*)k, (const T*)vt, (const T*)g,
                                          (const T*)tri_bias, (const T*)mask, (T*)o, n, heads,
                                          key_pitch, mask_transposed, inf, row_begin, row_count,
                                          n_keys, (hipStream_t)stream));
  return after_launch(what);
}

PTX_API int ptx_triattn_fwd(const void* q, const void* k, const void* vt, const void* g,
                    const void* tri_bias, const void* mask, void* o, int n, int heads, int d,
                    int key_pitch, int mask_transposed, float inf, int dtype, void* stream) {
  return triattn_fwd_checked("triattn_fwd", q, k, vt, g, tri_bias, mask, o, n, heads, d, key_pitch,
                             mask_transposed, inf, 0, n, n, dtype, stream);
}

PTX_API int ptx_triattn_fwd_rows(const void* q, const void* k, const void* vt, const void* g,
                                 const void* tri_bias, const void* mask, void* o, int n, int heads,
                                 int d, int key_pitch, int mask_transposed, float inf, int row_begin,
                                 int row_count, int n_keys, int dtype, void* stream) {
  return triattn_fwd_checked("triattn_fwd_rows", q, k, vt, g, tri_bias, mask, o, n, heads, d,
                             key_pitch, mask_transposed, inf, row_begin, row_count, n_keys, dtype,
                             stream);
}

PTX_API int64_t ptx_triattn_core_workspace_elems(int n_rows, int s, int heads) {
  if (n_rows <= 0 || s <= 0 || heads <= 0) return 0;
  const int64_t pitch = ptx_key_pitch(s);
  return (int64_t)n_rows * s * heads * 32             // q in log2 units
         + 2 * (int64_t)heads * n_rows * pitch * 32   // K, V^T key tiles
         + ptx_triattn_bias_elems(s, heads);          // bias tiles
}

PTX_API int ptx_triattn_core_fwd(const void* q, const void* k, const void* v, const void* bias1,
                                 const void* bias2, void* o, float* lse, void* workspace, int batch,
                                 int n_rows, int s, int heads, int d, int dtype, void* stream) {
  PTX_REQUIRE(dtype_ok(dtype), PTX_ERR_BAD_ARG, "triattn_core_fwd: unknown dtype %d", dtype);
  PTX_REQUIRE(batch >= 0 && n_rows >= 0 && s >= 0 && heads >= 0, PTX_ERR_BAD_ARG,
              "triattn_core_fwd: batch=%d n_rows=%d s=%d heads=%d", batch, n_rows, s, heads);
  PTX_REQUIRE(d == 32, PTX_ERR_UNSUPPORTED, "triattn_core_fwd: only head dim 32 is built (got %d)", d);
  PTX_REQUIRE(s <= 8192 && n_rows < 32768 && heads <= 64, PTX_ERR_UNSUPPORTED,
              "triattn_core_fwd: n_rows=%d s=%d heads=%d too large", n_rows, s, heads);
  if (batch == 0 || n_rows == 0 || s == 0 || heads == 0) return PTX_OK;
  PTX_REQUIRE(q && k && v && bias2 && o && workspace, PTX_ERR_BAD_ARG,
              "triattn_core_fwd: null pointer");
  PTX_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(bias2) && aligned16(o) &&
                  aligned16(workspace),
              PTX_ERR_BAD_ARG, "triattn_core_fwd: pointers must be 16-byte aligned");
  const int pitch = ptx_key_pitch(s);
  const int64_t n_q = (int64_t)n_rows * s * heads * 32;
  const int64_t n_kv = (int64_t)heads * n_rows * pitch * 32;
  const int64_t n_b2 = (int64_t)heads * s * s, n_b1 = (int64_t)n_rows * s;
  const size_t es = esize(dtype);
  char* ws = (char*)workspace;
  void* qs = ws;
  void* kf = ws + n_q * es;
  void* vtf = ws + (n_q + n_kv) * es;
  void* bf = ws + (n_q + 2 * n_kv) * es;
  for (int b = 0; b < batch; ++b) {
    const char* qb = (const char*)q + b * n_q * es;
    const char* kb = (const char*)k + b * n_q * es;
    const char* vb = (const char*)v + b * n_q * es;
    const char* b2 = (const char*)bias2 + b * n_b2 * es;
    const char* b1 = bias1 ? (const char*)bias1 + b * n_b1 * es : nullptr;
    char* ob = (char*)o + b * n_q * es;
    float* lb = lse ? lse + (int64_t)b * n_rows * s * heads : nullptr;
    PTX_DISPATCH(dtype, {
      ptx::triattn_pack<T>((const T*)qb, (const T*)kb, (const T*)vb, (const T*)b2, (T*)qs, (T*)kf,
                           (T*)vtf, (T*)bf, n_rows, s, heads, pitch, (hipStream_t)stream);
      // standard layout [row][position][head][32]; no gate; bias1 is an additive bias per key
      ptx::triattn_fwd_ex<T>((const T*)qs, (const T*)kf, (const T*)vtf, (const T*)nullptr,
                             (const T*)bf, (const T*)b1, (T*)ob, n_rows, s, heads, pitch, 0, 0.0f, 1,
                             32, (int64_t)s * heads * 32, (int64_t)heads * 32, lb, 1,
                             (int64_t)s * heads, heads, 0, n_rows, s, (hipStream_t)stream);
    });
  }
  return after_launch("triattn_core_fwd");
}

PTX_API int ptx_triattn_core_bwd(const void* q, const void* k, const void* v, const void* bias1,
                                 const void* bias2, const void* o, const float* lse,
                                 const void* dout, void* dq, void* dk, void* dv, void* dbias2,
                                 float* delta, int batch, int n_rows, int s, int heads, int d,
                                 int dtype, void* stream) {
  PTX_REQUIRE(dtype_ok(dtype), PTX_ERR_BAD_ARG, "triattn_core_bwd: unknown dtype %d", dtype);
  PTX_REQUIRE(batch >= 0 && n_rows >= 0 && s >= 0 && heads >= 0, PTX_ERR_BAD_ARG,
              "triattn_core_bwd: batch=%d n_rows=%d s=%d heads=%d", batch, n_rows, s, heads);
  PTX_REQUIRE(d == 32, PTX_ERR_UNSUPPORTED, "triattn_core_bwd: only head dim 32 is built (got %d)", d);
  PTX_REQUIRE(s <= 8192 && n_rows < 32768 && heads <= 64, PTX_ERR_UNSUPPORTED,
              "triattn_core_bwd: n_rows=%d s=%d heads=%d too large", n_rows, s, heads);
  if (batch == 0 || n_rows == 0 || s == 0 || heads == 0) return PTX_OK;
  PTX_REQUIRE(q && k && v && bias2 && o && lse && dout && dq && dk && dv && delta, PTX_ERR_BAD_ARG,
              "triattn_core_bwd: null pointer");
  PTX_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(o) && aligned16(dout) &&
                  aligned16(dq) && aligned16(dk) && aligned16(dv),
              PTX_ERR_BAD_ARG, "triattn_core_bwd: pointers must be 16-byte aligned");
  const int64_t n_q = (int64_t)n_rows * s * heads * 32, n_l = (int64_t)n_rows * s * heads;
  const int64_t n_b2 = (int64_t)heads * s * s, n_b1 = (int64_t)n_rows * s;
  const size_t es = esize(dtype);
  for (int b = 0; b < batch; ++b) {
    const int64_t oq = b * n_q * (int64_t)es;
    const char* b1 = bias1 ? (const char*)bias1 + b * n_b1 * es : nullptr;
    char* db2 = dbias2 ? (char*)dbias2 + b * n_b2 * es : nullptr;
    PTX_DISPATCH(dtype, ptx::triattn_bwd<T>(
                            (const char*)q + oq, (const char*)k + oq, (const char*)v + oq, b1,
                            (const char*)bias2 + b * n_b2 * es, (const char*)o + oq, lse + b * n_l,
                            (const char*)dout + oq, (char*)dq + oq, (char*)dk + oq, (char*)dv + oq,
                            db2, delta, n_rows, s, heads, (hipStream_t)stream));
  }
  return after_launch("triattn_core_bwd");
}

PTX_API int ptx_triattn_output(const void* o, const void* w_o, const void* z, void* out, int n, int c_in,
                       int transposed, int add_residual, int dtype, void* stream) {
  PTX_REQUIRE(dtype_ok_z(dtype), PTX_ERR_BAD_ARG, "triattn_output: unknown dtype %d", dtype);
  PTX_REQUIRE(n >= 0, PTX_ERR_BAD_ARG, "triattn_output: n=%d", n);
  PTX_REQUIRE(pair_width_ok(c_in, c_in == 256 ? 256 : 128, dtype), PTX_ERR_UNSUPPORTED,
              "triattn_output: %s (got c_in=%d)", kWidthMsg, c_in);
  PTX_REQUIRE(n < 32768, PTX_ERR_UNSUPPORTED, "triattn_output: n=%d too large", n);
  if (n == 0) return PTX_OK;
  PTX_REQUIRE(o && w_o && out && (!add_residual || z), PTX_ERR_BAD_ARG,
              "triattn_output: null pointer");
  PTX_REQUIRE(aligned16(o) && aligned16(w_o) && aligned16(out) && (!z || aligned16(z)),
              PTX_ERR_BAD_ARG,
              "triattn_output: pointers must be 16-byte aligned");
  PTX_DISPATCH_Z(dtype, (ptx::triattn_output<T, TZ>)(o, w_o, z, out, n, c_in, transposed, add_residual,
                                             (hipStream_t)stream));
  return after_launch("triattn_output");
}

PTX_API int ptx_triattn_gate_output(const void* o, const void* z, const void* ln_w, const void* ln_b,
                                    const void* w_g, const void* w_o, void* out, int n, int c_in,
                                    int heads, int transposed, int add_residual, float eps, int dtype,
                                    void* stream) {
  PTX_REQUIRE(dtype == PTX_BF16 || dtype == PTX_MIXED, PTX_ERR_UNSUPPORTED,
              "triattn_gate_output: built for PTX_BF16 and PTX_MIXED only (got dtype %d)", dtype);
  PTX_REQUIRE(n >= 0, PTX_ERR_BAD_ARG, "triattn_gate_output: n=%d", n);
  PTX_REQUIRE(c_in == 128 && heads == 4, PTX_ERR_UNSUPPORTED,
              "triattn_gate_output: only c_in = 128 with 4 heads of 32 is built (got c_in=%d heads=%d)",
              c_in, heads);
  PTX_REQUIRE(n < 32768, PTX_ERR_UNSUPPORTED, "triattn_gate_output: n=%d too large", n);
  if (n == 0) return PTX_OK;
  PTX_REQUIRE(o && z && w_g && w_o && out, PTX_ERR_BAD_ARG, "triattn_gate_output: null pointer");
  PTX_REQUIRE(aligned16(o) && aligned16(z) && aligned16(w_g) && aligned16(w_o) && aligned16(out) &&
                  (!ln_w || aligned16(ln_w)) && (!ln_b || aligned16(ln_b)),
              PTX_ERR_BAD_ARG, "triattn_gate_output: pointers must be 16-byte aligned");
  if (dtype == PTX_MIXED)
    ptx::triattn_gate_output<float>(o, z, ln_w, ln_b, w_g, w_o, out, n, transposed, add_residual, eps,
                                    (hipStream_t)stream);
  else
    ptx::triattn_gate_output<ptx::bf16_t>(o, z, ln_w, ln_b, w_g, w_o, out, n, transposed, add_residual,
                                          eps, (hipStream_t)stream);
  return after_launch("triattn_gate_output");
}

PTX_API int64_t ptx_transition_packed_elems(int c, int n_factor) {
  if (c <= 0 || n_factor <= 0) return 0;
  return (int64_t)3 * n_factor * c * c;
}

PTX_API int ptx_transition_pack(const void* w_a, const void* w_b, const void* w_o, void* packed, int c,
                        int n_factor, int dtype, void* stream) {
  if (dtype == PTX_MIXED) dtype = PTX_BF16;   // no residual-stream tensor here
  PTX_REQUIRE(dtype_ok(dtype), PTX_ERR_BAD_ARG, "transition_pack: unknown dtype %d", dtype);
  PTX_REQUIRE(n_factor > 0, PTX_ERR_BAD_ARG, "transition_pack: n_factor=%d", n_factor);
  PTX_REQUIRE(c == 128 || c == 64 || (c == 256 && dtype == PTX_BF16), PTX_ERR_UNSUPPORTED,
              "transition_pack: only c = 64, 128, or 256 in bf16, is built (got %d)", c);
  PTX_REQUIRE((n_factor * c) % 64 == 0, PTX_ERR_UNSUPPORTED,
              "transition_pack: the hidden width %d is not a multiple of 64", n_factor * c);
  PTX_REQUIRE(n_factor <= 64, PTX_ERR_UNSUPPORTED, "transition_pack: n_factor=%d too large",
              n_factor);
  PTX_REQUIRE(w_a && w_b && w_o && packed, PTX_ERR_BAD_ARG, "transition_pack: null pointer");
  PTX_REQUIRE(aligned16(packed), PTX_ERR_BAD_ARG, "transition_pack: packed must be 16-byte aligned");
  PTX_DISPATCH(dtype, ptx::transition_pack<T>(w_a, w_b, w_o, packed, c, n_factor,
                                              (hipStream_t)stream));
  return after_launch("transition_pack");
}

PTX_API int ptx_transition_fwd(const void* x, const void* ln_w, const void* ln_b, const void* packed,
                       void* out, int64_t rows, int c, int n_factor, int add_residual, float eps,
                       int dtype, void* stream) {
  PTX_REQUIRE(dtype_ok_z(dtype), PTX_ERR_BAD_ARG, "transition: unknown dtype %d", dtype);
  PTX_REQUIRE(rows >= 0 && n_factor > 0, PTX_ERR_BAD_ARG, "transition: rows=%lld n_factor=%d",
              (long long)rows, n_factor);
  PTX_REQUIRE(c == 128 || c == 64 || (c == 256 && dtype != PTX_F32), PTX_ERR_UNSUPPORTED,
              "transition: only c = 64, 128, or 256 in bf16 arithmetic, is built (got %d)", c);
  PTX_REQUIRE((n_factor * c) % 64 == 0, PTX_ERR_UNSUPPORTED,
              "transition: the hidden width %d is not a multiple of 64", n_factor * c);
  PTX_REQUIRE(n_factor <= 64, PTX_ERR_UNSUPPORTED, "transition: n_factor=%d too large", n_factor);
  PTX_REQUIRE(rows < ((int64_t)1 << 30), PTX_ERR_UNSUPPORTED, "transition: rows=%lld too large",
              (long long)rows);
  if (rows == 0) return PTX_OK;
  PTX_REQUIRE(x && packed && out, PTX_ERR_BAD_ARG, "transition: null pointer");
  PTX_REQUIRE(aligned16(x) && aligned16(packed) && aligned16(out) && (!ln_w || aligned16(ln_w)) &&
                  (!ln_b || aligned16(ln_b)),
              PTX_ERR_BAD_ARG, "transition: pointers must be 16-byte aligned");
  PTX_DISPATCH_Z(dtype, (ptx::transition_fwd<T, TZ>)(x, ln_w, ln_b, packed, out, rows, c, n_factor,
                                             add_residual, eps, (hipStream_t)stream));
  return after_launch("transition");
}

PTX_API int ptx_transition_pair_bias_fwd(const void* x, const void* ln_w, const void* ln_b,
                                         const void* packed, void* out, int64_t rows, int c,
                                         int n_factor, int add_residual, float eps,
                                         const void* pb_ln_w, const void* pb_ln_b, const void* pb_w,
                                         void* bias, int heads, int bias_f32, float pb_eps,
                                         int dtype, void* stream) {
  PTX_REQUIRE(dtype == PTX_BF16 || dtype == PTX_MIXED, PTX_ERR_UNSUPPORTED,
              "transition_pair_bias: built for PTX_BF16 and PTX_MIXED only (got dtype %d)", dtype);
  PTX_REQUIRE(rows >= 0 && n_factor > 0, PTX_ERR_BAD_ARG, "transition_pair_bias: rows=%lld n_factor=%d",
              (long long)rows, n_factor);
  PTX_REQUIRE(c == 128, PTX_ERR_UNSUPPORTED, "transition_pair_bias: only c = 128 is built (got %d)", c);
  PTX_REQUIRE((n_factor * c) % 64 == 0 && n_factor <= 64, PTX_ERR_UNSUPPORTED,
              "transition_pair_bias: n_factor=%d", n_factor);
  PTX_REQUIRE(heads >= 1 && heads <= 32, PTX_ERR_UNSUPPORTED, "transition_pair_bias: heads=%d (1..32)",
              heads);
  PTX_REQUIRE(rows < ((int64_t)1 << 30), PTX_ERR_UNSUPPORTED, "transition_pair_bias: rows=%lld too large",
              (long long)rows);
  if (rows == 0) return PTX_OK;
  PTX_REQUIRE(x && packed && out && pb_w && bias, PTX_ERR_BAD_ARG, "transition_pair_bias: null pointer");
  PTX_REQUIRE(aligned16(x) && aligned16(packed) && aligned16(out) && aligned16(pb_w) && aligned16(bias) &&
                  (!ln_w || aligned16(ln_w)) && (!ln_b || aligned16(ln_b)) &&
                  (!pb_ln_w || aligned16(pb_ln_w)) && (!pb_ln_b || aligned16(pb_ln_b)),
              PTX_ERR_BAD_ARG, "transition_pair_bias: pointers must be 16-byte aligned");
  int rc;
  if (dtype == PTX_MIXED)
    rc = ptx::transition_pair_bias_fwd<ptx::bf16_t, float>(x, ln_w, ln_b, packed, out, rows, n_factor,
                                                         add_residual, eps, pb_ln_w, pb_ln_b, pb_w, bias,
                                                         heads, bias_f32, pb_eps, (hipStream_t)stream);
  else
    rc = ptx::transition_pair_bias_fwd<ptx::bf16_t, ptx::bf16_t>(x, ln_w, ln_b, packed, out, rows, n_factor,
                                                               add_residual, eps, pb_ln_w, pb_ln_b, pb_w,
                                                               bias, heads, bias_f32, pb_eps,
                                                               (hipStream_t)stream);
  PTX_REQUIRE(rc == 0, PTX_ERR_UNSUPPORTED, "transition_pair_bias: not built for this type");
  return after_launch("transition_pair_bias");
}

PTX_API int64_t ptx_triattn_output_transition_packed_elems(int n_factor) {
  return n_factor > 0 ? ptx::triattn_output_transition_packed_elems(n_factor) : 0;
}

PTX_API int ptx_triattn_output_transition_pack(const void* w_g, const void* w_o, const void* w_a,
                                               const void* w_b, const void* w_to, void* packed,
                                               int n_factor, int dtype, void* stream) {
  PTX_REQUIRE(dtype == PTX_BF16 || dtype == PTX_MIXED, PTX_ERR_UNSUPPORTED,
              "triattn_output_transition_pack: built for PTX_BF16 and PTX_MIXED only (got dtype %d)", dtype);
  PTX_REQUIRE(n_factor > 0 && n_factor <= 64 && (n_factor * 128) % 64 == 0, PTX_ERR_UNSUPPORTED,
              "triattn_output_transition_pack: n_factor=%d", n_factor);
  PTX_REQUIRE(w_g && w_o && w_a && w_b && w_to && packed, PTX_ERR_BAD_ARG,
              "triattn_output_transition_pack: null pointer");
  PTX_REQUIRE(aligned16(w_g) && aligned16(w_o) && aligned16(packed), PTX_ERR_BAD_ARG,
              "triattn_output_transition_pack: w_g, w_o and packed must be 16-byte aligned");
  const int rc = ptx::triattn_output_transition_pack<ptx::bf16_t>(w_g, w_o, w_a, w_b, w_to, packed, n_factor,
                                                                (hipStream_t)stream);
  PTX_REQUIRE(rc == 0, PTX_ERR_UNSUPPORTED, "triattn_output_transition_pack: not built for this type");
  return after_launch("triattn_output_transition_pack");
}

PTX_API int ptx_triattn_output_transition_fwd(const void* o, const void* z, const void* att_ln_w,
                                              const void* att_ln_b, const void* packed,
                                              const void* ln_w, const void* ln_b, void* out, int n,
                                              int c_in, int heads, int transposed, int n_factor,
                                              float att_eps, float eps, const void* pb_ln_w,
                                              const void* pb_ln_b, const void* pb_w, void* bias,
                                              int pb_heads, int bias_f32, float pb_eps, int dtype,
                                              void* stream) {
  PTX_REQUIRE(dtype == PTX_BF16 || dtype == PTX_MIXED, PTX_ERR_UNSUPPORTED,
              "triattn_output_transition: built for PTX_BF16 and PTX_MIXED only (got dtype %d)", dtype);
  PTX_REQUIRE(n >= 0, PTX_ERR_BAD_ARG, "triattn_output_transition: n=%d", n);
  PTX_REQUIRE(c_in == 128 && heads == 4, PTX_ERR_UNSUPPORTED,
              "triattn_output_transition: only c_in = 128 with 4 heads of 32 is built (got c_in=%d heads=%d)",
              c_in, heads);
  PTX_REQUIRE(n_factor > 0 && n_factor <= 64 && (n_factor * 128) % 64 == 0, PTX_ERR_UNSUPPORTED,
              "triattn_output_transition: n_factor=%d", n_factor);
  PTX_REQUIRE(n < 32768, PTX_ERR_UNSUPPORTED, "triattn_output_transition: n=%d too large", n);
  PTX_REQUIRE(!pb_w || (pb_heads >= 1 && pb_heads <= 32), PTX_ERR_UNSUPPORTED,
              "triattn_output_transition: pair-bias heads=%d (1..32)", pb_heads);
  if (n == 0) return PTX_OK;
  PTX_REQUIRE(o && z && packed && out && (!pb_w || bias), PTX_ERR_BAD_ARG,
              "triattn_output_transition: null pointer");
  PTX_REQUIRE(aligned16(o) && aligned16(z) && aligned16(packed) && aligned16(out) &&
                  (!att_ln_w || aligned16(att_ln_w)) && (!att_ln_b || aligned16(att_ln_b)) &&
                  (!ln_w || aligned16(ln_w)) && (!ln_b || aligned16(ln_b)) &&
                  (!pb_w || (aligned16(pb_w) && aligned16(bias))) &&
                  (!pb_ln_w || aligned16(pb_ln_w)) && (!pb_ln_b || aligned16(pb_ln_b)),
              PTX_ERR_BAD_ARG, "triattn_output_transition: pointers must be 16-byte aligned");
  int rc;
  if (dtype == PTX_MIXED)
    rc = ptx::triattn_output_transition_fwd<ptx::bf16_t, float>(
        o, z, att_ln_w, att_ln_b, packed, ln_w, ln_b, out, n, transposed, n_factor, att_eps, eps, pb_ln_w,
        pb_ln_b, pb_w, bias, pb_heads, bias_f32, pb_eps, (hipStream_t)stream);
  else
    rc = ptx::triattn_output_transition_fwd<ptx::bf16_t, ptx::bf16_t>(
        o, z, att_ln_w, att_ln_b, packed, ln_w, ln_b, out, n, transposed, n_factor, att_eps, eps, pb_ln_w,
        pb_ln_b, pb_w, bias, pb_heads, bias_f32, pb_eps, (hipStream_t)stream);
  PTX_REQUIRE(rc == 0, PTX_ERR_UNSUPPORTED, "triattn_output_transition: not built for this type");
  return after_launch("triattn_output_transition");
}

PTX_API int ptx_linear_fwd(const void* x, const void* w, const void* bias, int bias_cols,
                           const void* res, void* out, void* out_t, int split_col, int64_t ldt,
                           int rows, int k, int n_out, int dtype, void* stream) {
  PTX_REQUIRE(dtype_ok(dtype), PTX_ERR_BAD_ARG, "linear: unknown dtype %d", dtype);
  PTX_REQUIRE(rows >= 0 && k > 0 && n_out >= 0, PTX_ERR_BAD_ARG, "linear: rows=%d k=%d n_out=%d",
              rows, k, n_out);
  PTX_REQUIRE(k % 16 == 0 && n_out % 8 == 0, PTX_ERR_UNSUPPORTED,
              "linear: k must be a multiple of 16 and n_out of 8 (got k=%d n_out=%d)", k, n_out);
  if (split_col < 0 || split_col > n_out) split_col = n_out;
  if (rows == 0 || n_out == 0) return PTX_OK;
  PTX_REQUIRE(x && w && (out || split_col == 0), PTX_ERR_BAD_ARG, "linear: null pointer");
  if (split_col < n_out) {
    PTX_REQUIRE(out_t, PTX_ERR_BAD_ARG, "linear: out_t is null");
    PTX_REQUIRE(split_col % 32 == 0 && ldt % 8 == 0 && ldt >= rows && !res, PTX_ERR_BAD_ARG,
                "linear: transposed tail needs split_col %% 32 == 0, ldt %% 8 == 0, ldt >= rows and "
                "no residual (split_col=%d ldt=%lld)", split_col, (long long)ldt);
    PTX_REQUIRE(aligned16(out_t), PTX_ERR_BAD_ARG, "linear: out_t must be 16-byte aligned");
  }
  PTX_REQUIRE(aligned16(x) && aligned16(w) && (!out || aligned16(out)) && (!res || aligned16(res)),
              PTX_ERR_BAD_ARG, "linear: pointers must be 16-byte aligned");
  PTX_DISPATCH(dtype, ptx::linear_fwd<T>(x, w, bias, bias ? bias_cols : 0, res, out, out_t,
                                         split_col, ldt, rows, k, n_out, (hipStream_t)stream));
  return after_launch("linear");
}

PTX_API int ptx_swiglu_fwd(const void* x, const void* w_a, const void* w_b, void* out, int rows,
                           int k, int hidden, int dtype, void* stream) {
  PTX_REQUIRE(dtype_ok(dtype), PTX_ERR_BAD_ARG, "swiglu: unknown dtype %d", dtype);
  PTX_REQUIRE(rows >= 0 && k > 0 && hidden >= 0, PTX_ERR_BAD_ARG, "swiglu: rows=%d k=%d hidden=%d",
              rows, k, hidden);
  PTX_REQUIRE(k % 16 == 0 && hidden % 8 == 0, PTX_ERR_UNSUPPORTED,
              "swiglu: k must be a multiple of 16 and hidden of 8 (got k=%d hidden=%d)", k, hidden);
  if (rows == 0 || hidden == 0) return PTX_OK;
  PTX_REQUIRE(x && w_a && w_b && out, PTX_ERR_BAD_ARG, "swiglu: null pointer");
  PTX_REQUIRE(aligned16(x) && aligned16(w_a) && aligned16(w_b) && aligned16(out), PTX_ERR_BAD_ARG,
              "swiglu: pointers must be 16-byte aligned");
  PTX_DISPATCH(dtype, ptx::swiglu_fwd<T>(x, w_a, w_b, out, rows, k, hidden, (hipStream_t)stream));
  return after_launch("swiglu");
}

PTX_API int ptx_single_attention_fwd(const void* q, const void* k, const void* vt, const void* g,
                                     const void* bias, int bias_f32, void* out, int n, int heads,
                                     int d, int64_t ld, int64_t ldt, int64_t ldo, float scale,
                                     int dtype, void* stream) {
  PTX_REQUIRE(dtype_ok(dtype), PTX_ERR_BAD_ARG, "single_attention: unknown dtype %d", dtype);
  PTX_REQUIRE(n >= 0 && heads >= 0, PTX_ERR_BAD_ARG, "single_attention: n=%d heads=%d", n, heads);
  PTX_REQUIRE(d > 0 && d <= 32 && d % 8 == 0, PTX_ERR_UNSUPPORTED,
              "single_attention: head dim must be 8, 16, 24 or 32 (got %d)", d);
  PTX_REQUIRE(n <= 32768 && heads <= 65535, PTX_ERR_UNSUPPORTED, "single_attention: n=%d heads=%d too large",
              n, heads);
  if (n == 0 || heads == 0) return PTX_OK;
  PTX_REQUIRE(q && k && vt && out, PTX_ERR_BAD_ARG, "single_attention: null pointer");
  PTX_REQUIRE(ld % 8 == 0 && ldo % 8 == 0 && ldt % 8 == 0 && ldt >= ((n + 31) / 32) * 32 &&
                  ld >= (int64_t)heads * d && ldo >= (int64_t)heads * d,
              PTX_ERR_BAD_ARG,
              "single_attention: pitches must be multiples of 8, ld / ldo >= heads * d and "
              "ldt >= n rounded up to 32 (ld=%lld ldt=%lld ldo=%lld)",
              (long long)ld, (long long)ldt, (long long)ldo);
  PTX_REQUIRE(aligned16(q) && aligned16(k) && aligned16(vt) && aligned16(out) && (!g || aligned16(g)),
              PTX_ERR_BAD_ARG, "single_attention: pointers must be 16-byte aligned");
  PTX_DISPATCH(dtype, ptx::single_attention_fwd<T>(q, k, vt, g, bias, bias_f32, out, n, heads, d, ld,
                                                   ldt, ldo, scale, (hipStream_t)stream));
  return after_launch("single_attention");
}

PTX_API int ptx_pair_bias_fwd(const void* z, const void* ln_w, const void* ln_b, const void* w, void* bias,
                      int n, int c_z, int heads, int out_f32, float eps, int dtype,
                      void* stream) {
  PTX_REQUIRE(dtype_ok_z(dtype), PTX_ERR_BAD_ARG, "pair_bias: unknown dtype %d", dtype);
  PTX_REQUIRE(n >= 0, PTX_ERR_BAD_ARG, "pair_bias: n=%d", n);
  PTX_REQUIRE(c_z == 128 || (c_z == 256 && dtype != PTX_F32), PTX_ERR_UNSUPPORTED,
              "pair_bias: only c_z = 128, or 256 in bf16 arithmetic, is built (got %d)", c_z);
  PTX_REQUIRE(heads >= 1 && heads <= 32, PTX_ERR_UNSUPPORTED,
              "pair_bias: heads=%d outside 1..32", heads);
  PTX_REQUIRE(n < 32768, PTX_ERR_UNSUPPORTED, "pair_bias: n=%d too large", n);
  if (n == 0) return PTX_OK;
  PTX_REQUIRE(z && w && bias, PTX_ERR_BAD_ARG, "pair_bias: null pointer");
  PTX_REQUIRE(aligned16(z) && aligned16(w) && aligned16(bias) && (!ln_w || aligned16(ln_w)) &&
                  (!ln_b || aligned16(ln_b)),
              PTX_ERR_BAD_ARG, "pair_bias: pointers must be 16-byte aligned");
  PTX_DISPATCH_Z(dtype, (ptx::pair_bias_fwd<T, TZ>)(z, ln_w, ln_b, w, bias, n, c_z, heads, out_f32, eps,
                                            (hipStream_t)stream));
  return after_launch("pair_bias");
}

PTX_API int ptx_hbm_stream(const void* src, void* dst, int64_t bytes, int nontemporal, void* stream) {
  PTX_REQUIRE(bytes >= 0 && bytes % 16 == 0, PTX_ERR_BAD_ARG,
              "hbm_stream: bytes=%lld must be a non-negative multiple of 16", (long long)bytes);
  PTX_REQUIRE(bytes <= ((int64_t)1 << 40), PTX_ERR_UNSUPPORTED, "hbm_stream: more than 1 TiB");
  if (bytes == 0) return PTX_OK;
  PTX_REQUIRE(src || dst, PTX_ERR_BAD_ARG, "hbm_stream: src and dst are both null");
  PTX_REQUIRE(aligned16(src) && aligned16(dst), PTX_ERR_BAD_ARG,
              "hbm_stream: pointers must be 16-byte aligned");
  ptx::hbm_stream(src, dst, bytes, nontemporal, (hipStream_t)stream);
  return after_launch("hbm_stream");
}

}  // extern "C"
