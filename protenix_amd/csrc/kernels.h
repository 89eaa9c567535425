// Host-callable launchers, one per kernel family; api.hip validates arguments
// and dispatches on dtype.  c_z / c: channels of a pair-tensor row: 64 or 128 (hidden
// widths - c_hidden_mul, heads * d - of 128), or 256 in bf16 (hidden widths of 256).  All return 0 after enqueueing on `stream`.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ptx {

// T: arithmetic / weight / workspace type.  TZ (where present): storage type of the pair
// tensor rows the kernel reads (z, x) and of the residual stream it writes (out): T, or float
// with T = bf16 (the fp32 residual stream of autocast inference; rows of 64 or 128 channels).
template <typename T>
int layernorm_fwd(const T* x, const T* gamma, const T* beta, T* y, float* mean, float* rstd,
                  int64_t rows, int cols, float eps, hipStream_t stream);
// LayerNorm backward: dx always; dgamma / dbeta when non-null, through `workspace`
// (layernorm_bwd_workspace_elems fp32 elements).
int64_t layernorm_bwd_workspace_elems(int64_t rows, int cols);
template <typename T>
int layernorm_bwd(const T* dout, const T* x, const float* mean, const float* rstd, const T* gamma,
                  T* dx, T* dgamma, T* dbeta, float* workspace, int64_t rows, int cols,
                  hipStream_t stream);

template <typename T, typename TZ = T>
int trimul_project(const void* z, const void* mask, const void* ln_w, const void* ln_b,
                   const void* w_ap, const void* w_ag, const void* w_bp, const void* w_bg, void* a,
                   void* b, int n, int c_z, int k_pitch, int incoming, float eps,
                   hipStream_t stream);
template <typename T, typename TZ = T>
int trimul_output(const void* x, const void* z, const void* ln_in_w, const void* ln_in_b,
                  const void* ln_out_w, const void* ln_out_b, const void* w_z, const void* w_g,
                  void* out, int n, int c_z, int add_residual, float eps, hipStream_t stream);
template <typename T, typename TZ = T>
int triattn_project(const void* z, const void* ln_w, const void* ln_b, const void* w_q,
                    const void* w_k, const void* w_v, const void* w_g, const void* w_b, void* q,
                    void* k, void* vt, void* g, void* tri_bias, int n, int c_z, int heads, int d,
                    int key_pitch, int transposed, float eps, hipStream_t stream);
template <typename T, typename TZ = T>
int triattn_output(const void* o, const void* w_o, const void* z, void* out, int n, int c_z,
                   int transposed, int add_residual, hipStream_t stream);
// out = [z +] W_o (sigmoid(W_g LN(z)) * o) on rows of 128 channels, 4 heads, 16-bit arithmetic:
// the last stage of the triangle attention with the gate formed here (o ungated, head-major).
template <typename TZ>
int triattn_gate_output(const void* o, const void* z, const void* ln_w, const void* ln_b,
                        const void* w_g, const void* w_o, void* out, int n, int transposed,
                        int add_residual, float eps, hipStream_t stream);
// transition weights -> fragment-ordered chunks of 32 hidden (3 * n_factor*c * c elements)
template <typename T>
int transition_pack(const void* w_a, const void* w_b, const void* w_o, void* packed, int c,
                    int n_factor, hipStream_t stream);
template <typename T, typename TZ = T>
int transition_fwd(const void* x, const void* ln_w, const void* ln_b, const void* packed,
                   void* out, int64_t rows, int c, int n_factor, int add_residual, float eps,
                   hipStream_t stream);
// The transition on rows of 128 channels (16-bit arithmetic) with the pair bias of the single
// attention, bias[h][row] = (W LN_pb(out[row]))[h], formed from the finished rows in its epilogue.
template <typename T, typename TZ = T>
int transition_pair_bias_fwd(const void* x, const void* ln_w, const void* ln_b, const void* packed,
                             void* out, int64_t rows, int n_factor, int add_residual, float eps,
                             const void* pb_ln_w, const void* pb_ln_b, const void* pb_w,
                             void* bias, int heads, int bias_f32, float pb_eps,
                             hipStream_t stream);
// The last stage of a triangle attention (as triattn_gate_output, residual added) and the pair
// transition that follows it (as transition_fwd / transition_pair_bias_fwd, residual added) in
// one launch on rows of 128 channels, 16-bit arithmetic: out = z' + transition(z'),
// z' = z + W_o (sigmoid(W_g LN_att(z)) * o).  `packed` holds both stages' weights
// (triattn_output_transition_pack); pb_w null: no pair bias.
int64_t triattn_output_transition_packed_elems(int n_factor);
template <typename T>
int triattn_output_transition_pack(const void* w_g, const void* w_o, const void* w_a,
                                   const void* w_b, const void* w_to, void* packed, int n_factor,
                                   hipStream_t stream);
template <typename T, typename TZ = T>
int triattn_output_transition_fwd(const void* o, const void* z, const void* att_ln_w,
                                  const void* att_ln_b, const void* packed, const void* ln_w,
                                  const void* ln_b, void* out, int n, int transposed, int n_factor,
                                  float att_eps, float eps, const void* pb_ln_w, const void* pb_ln_b,
                                  const void* pb_w, void* bias, int heads, int bias_f32, float pb_eps,
                                  hipStream_t stream);
template <typename T, typename TZ = T>
int pair_bias_fwd(const void* z, const void* ln_w, const void* ln_b, const void* w, void* bias,
                  int n, int c_z, int heads, int out_f32, float eps, hipStream_t stream);

// Small linear layers of the single-representation track (single.hip):
//   out[rows][n_out] = [res +] x[rows][k] w[n_out][k]^T [+ bias on columns < bias_cols];
//   output columns >= split_col go, transposed, to out_t[n_out - split_col][ldt] instead
//   (rows in [rows, ldt) written as zeros); out then has split_col columns.
template <typename T>
int linear_fwd(const void* x, const void* w, const void* bias, int bias_cols, const void* res,
               void* out, void* out_t, int split_col, int64_t ldt, int rows, int k, int n_out,
               hipStream_t stream);
//   out[rows][hidden] = silu(x w_a^T) * (x w_b^T)
template <typename T>
int swiglu_fwd(const void* x, const void* w_a, const void* w_b, void* out, int rows, int k,
               int hidden, hipStream_t stream);
// out[n][heads*d] = sigmoid(g) * softmax_k(q k^T * scale + bias[h]) v per head; q, k, g rows of
// pitch ld, vt [heads*d][ldt] (keys beyond n hold zeros), bias [heads][n][n] fp32 or T.
template <typename T>
int single_attention_fwd(const void* q, const void* k, const void* vt, const void* g,
                         const void* bias, int bias_f32, void* out, int n, int heads, int d,
                         int64_t ld, int64_t ldt, int64_t ldo, float scale, hipStream_t stream);

// x[c][i][j] = sum_k a[c][i][k] * b[c][j][k] for `batch` independent products;
// a, b rows have pitch k_pitch (a multiple of 64, >= n), x is dense [batch][n][n].
template <typename T>
int nt_gemm_batched(const T* a, const T* b, T* x, int n, int k_pitch, int batch,
                    hipStream_t stream);

// Flash-style triangle attention core (see triattn.hip).
template <typename T>
int triattn_fwd(const T* q, const T* k, const T* vt, const T* g, const T* tri_bias, const T* mask,
                T* o, int n, int heads, int key_pitch, int mask_transposed, float inf,
                int row_begin, int row_count, int n_keys, hipStream_t stream);
// The same core on n_rows rows of n queries / keys, with q / g / o addressed through element
// strides (head, row, query), an optional gate (g may be null), the mask either 0/1 values or
// (mask_is_bias) an additive bias per (row, key), and an optional log2-sum-exp2 output.
// The launch covers rows row_begin .. row_begin + row_count - 1 and lets keys 0 .. n_keys - 1
// take part (keys beyond count as masked: weight exactly zero).
template <typename T>
int triattn_fwd_ex(const T* q, const T* k, const T* vt, const T* g, const T* tri_bias,
                   const T* mask, T* o, int n_rows, int n, int heads, int key_pitch,
                   int mask_transposed, float inf, int mask_is_bias, int64_t sh, int64_t si,
                   int64_t sj, float* lse, int64_t lh, int64_t li, int64_t lj, int row_begin,
                   int row_count, int n_keys, hipStream_t stream);
// Standard-layout K, V [n_rows][n][heads][32] and bias [heads][n][n] -> the core's fragment-
// ordered K, V^T and bias (bias and nothing else multiplied by log2(e)); q [n_rows][n][heads][32]
// -> qs, the same layout multiplied by log2(e).
template <typename T>
int triattn_pack(const T* q, const T* k, const T* v, const T* bias2, T* qs, T* kf, T* vtf, T* bf,
                 int n_rows, int n, int heads, int key_pitch, hipStream_t stream);
// Backward of the standard-layout attention operator: dQ, dK, dV [n_rows][s][heads][32] and,
// when db2 is given, dBias2 [heads][s][s], from Q (scaled), K, V, O, dO, the biases and the
// forward's log2-sum-exp2; delta [n_rows][s][heads] is fp32 scratch.
template <typename T>
int triattn_bwd(const void* q, const void* k, const void* v, const void* b1, const void* b2,
                const void* o, const float* lse, const void* dout, void* dq, void* dk, void* dv,
                void* db2, float* delta, int n_rows, int s, int heads, hipStream_t stream);

// Streams `bytes` (a multiple of 16) from src to dst; src null: write-only, dst null: read-only.
int hbm_stream(const void* src, void* dst, int64_t bytes, int nontemporal, hipStream_t stream);

}  // namespace ptx
