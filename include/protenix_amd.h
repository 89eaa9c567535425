/*
 * protenix_amd.h - C ABI of the MI355X (gfx950) Pairformer pair-stack kernels.
 *
 * One shared library, libprotenix_amd.so.  Every entry point
 *   - takes raw DEVICE pointers, sizes, a dtype code and a hipStream_t (as
 *     void*); no framework types cross the boundary;
 *   - allocates nothing and keeps no state: the caller owns inputs, outputs
 *     and workspaces; work is enqueued on `stream` and not waited for;
 *   - returns PTX_OK or an error code; ptx_last_error_string() describes the
 *     last failure of the calling thread.
 *
 * Tensors are dense, row-major, in the layouts named per function.  `dtype`
 * selects fp32 or bf16 storage for every tensor of the call unless said
 * otherwise; accumulation and statistics are always fp32.  The pair tensor is
 * "z[N][N][c]"; a "logical row" p = outer*N + inner addresses z[outer][inner]
 * (transposed = 0) or z[inner][outer] (transposed = 1), which is how the
 * ending-node attention and the incoming triangle product are served without
 * a transposed copy.
 *
 * Reference interfaces replaced (paths relative to bytedance/Protenix):
 *   protenix/model/layer_norm/kernel/layer_norm_cuda.cpp:142-179 (pybind module
 *     fast_layer_norm_cuda_v2), protenix/model/tri_attention/op.py:37-77
 *     (TriAttentionFunction), protenix/model/triangular/triangular.py:77-90
 *     (triangle_multiplicative_update), and the torch-path arithmetic of
 *     triangular.py:519-566, 657-715, layers.py:276-296, 361-398,
 *     primitives.py:190-230, transformer.py:184-194.
 */
#ifndef PROTENIX_AMD_H_
#define PROTENIX_AMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PTX_ABI_VERSION 3
#define PTX_API __attribute__((visibility("default")))

/*
 * PTX_MIXED: bf16 arithmetic on an fp32 residual stream, the way the reference runs
 * inference (fp32 parameters and activations under torch.autocast(bfloat16),
 * runner/inference.py:214-234): the pair tensor the call reads (z, x of the transition) and
 * the `out` it adds its update to are fp32; weights, masks, workspaces and every other tensor
 * are bf16.  Rows are normalised in fp32 and rounded to bf16 for the matrix products; the
 * update is rounded to bf16 and added to the fp32 row.  Accepted by the entry points that
 * touch the residual stream (rows of 64, 128 or 256 channels); the others (ptx_trimul_contract,
 * ptx_triattn_fwd, ptx_transition_pack) treat it as PTX_BF16, so one code serves a whole
 * update; the LayerNorm entry points refuse it.
 */
enum ptx_dtype { PTX_F32 = 0, PTX_BF16 = 1, PTX_MIXED = 2, PTX_F16 = 3 };
/* PTX_F16 (IEEE half) is taken by the LayerNorm entry points only, which dispatch on float /
 * Half / BFloat16 like the reference's kernel (layer_norm_cuda_kernel.cu:304-330). */

enum ptx_status {
  PTX_OK = 0,
  PTX_ERR_BAD_ARG = 1,     /* null pointer, negative size, unknown dtype       */
  PTX_ERR_UNSUPPORTED = 2, /* a shape this build has no kernel for             */
  PTX_ERR_LAUNCH = 3       /* hipGetLastError() after the launch was not clean */
};

/* ABI version of the loaded library (== PTX_ABI_VERSION it was built with). */
PTX_API int ptx_version(void);

/* Text of the calling thread's last error ("" if none).  Never NULL. */
PTX_API const char* ptx_last_error_string(void);

/*
 * Row pitch (in elements) of the intermediate tensors whose last axis is the
 * contracted / key axis: the smallest multiple of 64 that is >= n.  Padding
 * elements are never read as data and need no initialisation.
 */
PTX_API int ptx_key_pitch(int n);

/*
 * Element counts of the workspaces that travel between the stages of one
 * triangle update.  Their layouts are the library's own (MFMA operand order, so
 * that the consuming kernel reads them in contiguous 1 KB runs); the caller
 * only allocates them, uninitialised, and passes them from stage to stage.
 *   ptx_trimul_operand_elems: one of a, b.  Per channel, rows in blocks of 32 and
 *     K in steps of 16; fragment (c, rb, ks) holds 64 lanes x 8 elements, lane
 *     32*g + r = row 32*rb + r, K = 16*ks + 8*g .. +7:
 *     c_hidden * 32*ceil(n/32) * ptx_key_pitch(n).
 *   ptx_triattn_kv_elems: one of k, vt.  Per (head, row i), keys in tiles of 64, a
 *     tile = 4 fragments of 64 lanes x 8 elements: heads * n * ptx_key_pitch(n) * 32.
 *   ptx_triattn_bias_elems: the triangle bias.  Per head, queries in blocks of 32
 *     and keys in tiles of 64: heads * 32*ceil(n/32) * ptx_key_pitch(n).
 * q, g and o of the attention are head-major, [heads][n][n][d].
 */
PTX_API int64_t ptx_trimul_operand_elems(int n, int c_hidden);
PTX_API int64_t ptx_triattn_kv_elems(int n, int heads);
PTX_API int64_t ptx_triattn_bias_elems(int n, int heads);

/*
 * LayerNorm forward over the last dimension.
 * Replaces fast_layer_norm_cuda_v2.forward_{none,with_bias,with_weight,
 * with_both}_affine (layer_norm_cuda.cpp:142-157; kernel
 * layer_norm_cuda_kernel.cu:145-229): gamma and/or beta may be NULL.
 *   x, y   [rows][cols]     y may alias x
 *   mean, rstd  fp32 [rows], each may be NULL
 */
PTX_API int ptx_layernorm_fwd(const void* x, const void* gamma, const void* beta, void* y,
                      float* mean, float* rstd, int64_t rows, int cols, float eps,
                      int dtype, void* stream);

/*
 * LayerNorm backward.  Replaces fast_layer_norm_cuda_v2.backward_{none,with_bias,with_weight,
 * with_both}_affine (layer_norm_cuda.cpp:159-178; kernels layer_norm_cuda_kernel.cu:395-760,
 * host :860-990), fp32 arithmetic, with xc = x - mean and gd = gamma * dout:
 *   dx     = gd * rstd - sum_c(gd) * rstd / cols - xc * sum_c(gd * xc) * rstd^3 / cols
 *   dgamma = sum_rows dout * xc * rstd          dbeta = sum_rows dout
 *   dout, x, dx [rows][cols] in `dtype` (dx aliases neither);  mean, rstd fp32 [rows] as
 *   written by ptx_layernorm_fwd;  gamma [cols] in `dtype` or NULL (= 1);
 *   dgamma, dbeta [cols] in `dtype`, each may be NULL (not wanted);
 *   workspace: ptx_layernorm_bwd_workspace_elems(rows, cols) fp32 elements of partial sums,
 *   needed unless dgamma and dbeta are both NULL.  The sums run in a fixed order: results are
 *   reproducible bit for bit.  beta does not enter the gradients and is not an argument.
 */
PTX_API int64_t ptx_layernorm_bwd_workspace_elems(int64_t rows, int cols);
PTX_API int ptx_layernorm_bwd(const void* dout, const void* x, const float* mean, const float* rstd,
                      const void* gamma, void* dx, void* dgamma, void* dbeta, float* workspace,
                      int64_t rows, int cols, int dtype, void* stream);

/*
 * ptx_layernorm_bwd without a workspace argument and without any allocation.  No counterpart
 * in the reference; it is for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  The partial sums of
 * dgamma / dbeta live in a buffer built into the library (8 MiB per GPU, kept until the
 * process ends), which bounds the row length: cols <= 1024, else PTX_ERR_UNSUPPORTED.  Same
 * kernels, same summation order and therefore the same bits as ptx_layernorm_bwd.  The
 * buffer's device address is looked up on the first call on each device (call once outside
 * graph capture); the device of `stream` must be the current device.  All calls on one GPU
 * share the buffer: calls that overlap there (different streams or threads) race - serialise
 * them.  Nothing needs clearing between calls: a launch writes every partial row it reads.
 */
PTX_API int ptx_layernorm_bwd_static(const void* dout, const void* x, const float* mean,
                      const float* rstd, const void* gamma, void* dx, void* dgamma, void* dbeta,
                      int64_t rows, int cols, int dtype, void* stream);

/*
 * Triangle multiplication, stage 1 (triangular.py:537-543):
 *   zn = LN(z);  a = mask * sigmoid(W_ag zn) * (W_ap zn);  b likewise,
 * written channel-major so that stage 2 is a plain batched matrix product:
 *   outgoing (incoming = 0):  a[c][i][k] = a(z[i][k])[c]
 *   incoming (incoming = 1):  a[c][i][k] = a(z[k][i])[c]      (same for b)
 *   z [n][n][c_z], mask [n][n] in `dtype` or NULL (= ones),
 *   w_* [c_hidden][c_z]; a, b: workspaces of ptx_trimul_operand_elems(n, c_hidden)
 *   elements each, written in the contraction's operand order (K between n and
 *   k_pitch is written as zeros, rows beyond n stay unwritten);
 *   k_pitch = ptx_key_pitch(n).  Widths: c_z = 64 or 128 with c_hidden = 128, or
 *   (PTX_BF16, PTX_MIXED) c_z = c_hidden = 256.
 */
PTX_API int ptx_trimul_project(const void* z, const void* mask, const void* ln_w, const void* ln_b,
                       const void* w_ap, const void* w_ag, const void* w_bp, const void* w_bg,
                       void* a, void* b, int n, int c_z, int c_hidden, int k_pitch, int incoming,
                       float eps, int dtype, void* stream);

/*
 * Triangle multiplication, stage 2 (triangular.py:123-150): for every channel
 *   x[c][i][j] = sum_k a[c][i][k] * b[c][j][k]
 * which with the stage-1 layouts is 'ikc,jkc->ijc' (outgoing) or
 * 'kic,kjc->ijc' (incoming).  a, b as written by stage 1 (K between n and k_pitch
 * must hold zeros); x [c][n][n] dense.
 */
PTX_API int ptx_trimul_contract(const void* a, const void* b, void* x, int n, int c, int k_pitch,
                        int dtype, void* stream);

/*
 * Triangle multiplication, stage 3 (triangular.py:560-565):
 *   out = [residual z +] W_z LN_out(x) * sigmoid(W_g LN_in(z))
 *   x [c_hidden][n][n] from stage 2, z [n][n][c_z], out [n][n][c_z] (may alias z);
 *   w_z [c_z][c_hidden], w_g [c_z][c_z].  Widths as for stage 1.
 * add_residual = 1 gives z + update (the reference's `_add_with_inplace`).
 */
PTX_API int ptx_trimul_output(const void* x, const void* z, const void* ln_in_w, const void* ln_in_b,
                      const void* ln_out_w, const void* ln_out_b, const void* w_z,
                      const void* w_g, void* out, int n, int c_z, int c_hidden,
                      int add_residual, float eps, int dtype, void* stream);

/*
 * The whole triangle multiplication in one call, with the argument list of the reference's
 * fused operator (triangular.py:26-90, kernel_triangular_mult -> triangle_multiplicative_update;
 * call site triangular.py:497-514): stacked input weights
 *   p_in_weight = [linear_a_p.weight ; linear_b_p.weight]   [2 * c_hidden][c_z]
 *   g_in_weight = [linear_a_g.weight ; linear_b_g.weight]   [2 * c_hidden][c_z]
 *   p_out_weight = linear_z.weight [c_z][c_hidden],  g_out_weight = linear_g.weight [c_z][c_z]
 * x, out [n][n][c_z] (out may alias x);  mask [n][n] or NULL;  incoming = 0: 'outgoing'.
 * out = update, or x + update with add_residual.  Runs ptx_trimul_project,
 * ptx_trimul_contract and ptx_trimul_output on `stream` with their intermediates in
 * `workspace`: ptx_triangle_multiplicative_update_workspace_elems(n, c_hidden) elements of the
 * arithmetic type (bf16 for PTX_MIXED), 16-byte aligned, uninitialised.
 */
PTX_API int64_t ptx_triangle_multiplicative_update_workspace_elems(int n, int c_hidden);
PTX_API int ptx_triangle_multiplicative_update(
    const void* x, int incoming, const void* mask, const void* norm_in_weight,
    const void* norm_in_bias, const void* p_in_weight, const void* g_in_weight,
    const void* norm_out_weight, const void* norm_out_bias, const void* p_out_weight,
    const void* g_out_weight, void* out, void* workspace, int n, int c_z, int c_hidden,
    int add_residual, float eps, int dtype, void* stream);

/*
 * Triangle attention, stage 1 (triangular.py:683-692, layers.py:361-382, 386):
 *   xn = LN(x);  q = W_q xn / sqrt(d);  k = W_k xn;  v = W_v xn;
 *   g = sigmoid(W_g xn);  tri_bias = W_b xn
 * (q and tri_bias are stored multiplied by log2(e): stage 2 exponentiates in base 2)
 * over logical rows p = i*n + j of x = z (transposed = 0) or z^T (transposed = 1).
 *   q, g [heads][n][n][d] (logical row p = i*n + j);  k, vt: workspaces of
 *   ptx_triattn_kv_elems(n, heads) elements;  tri_bias: ptx_triattn_bias_elems(n, heads)
 *   elements;  key_pitch = ptx_key_pitch(n).   d = 32;  c_in = 64 or 128 with 4 heads,
 *   or (PTX_BF16, PTX_MIXED) c_in = 256 with 8 heads  (w_q, w_k, w_v, w_g [heads*d][c_in],
 *   w_b [heads][c_in]).
 * g = NULL (c_in = 128, 4 heads, PTX_BF16 / PTX_MIXED): no gate is written; stage 2 is then
 * called without one and ptx_triattn_gate_output forms it in stage 3.
 */
PTX_API int ptx_triattn_project(const void* z, const void* ln_w, const void* ln_b, const void* w_q,
                        const void* w_k, const void* w_v, const void* w_g, const void* w_b,
                        void* q, void* k, void* vt, void* g, void* tri_bias, int n, int c_in,
                        int heads, int d, int key_pitch, int transposed, float eps, int dtype,
                        void* stream);

/*
 * Triangle attention, stage 2: the fused op of tri_attention/op.py:37-77 with
 * the gate of layers.py:386-390 applied on the way out.  For every row i, head h:
 *   o[i][j][h] = g[i][j][h] * sum_k softmax_k( q[i][j][h].k[i][k][h]
 *                + inf*(mask(i,k)-1) + tri_bias[h][j][k] ) v[i][k][h]
 * The N^3 logits are never materialised.  The two biases are added in the
 * reference's order in fp32, so a fully masked row gives the mean of v, as
 * layers.py:286-291 does.
 *   mask [n][n] in `dtype` or NULL; mask(i,k) = mask[i][k], or mask[k][i] when
 *   mask_transposed = 1.   q, k, vt, g, tri_bias as written by stage 1;
 *   o [heads][n][n][d] (may alias g, not q/k/vt).   g = NULL: no gate (g = 1).
 */
PTX_API int ptx_triattn_fwd(const void* q, const void* k, const void* vt, const void* g,
                    const void* tri_bias, const void* mask, void* o, int n, int heads, int d,
                    int key_pitch, int mask_transposed, float inf, int dtype, void* stream);

/*
 * The same stage on rows row_begin .. row_begin + row_count - 1 only, with keys 0 .. n_keys - 1
 * taking part and the keys from n_keys on treated as masked for every row of the range (weight
 * exactly zero, which is what inf*(mask-1) gives a masked key of a row that has unmasked ones,
 * layers.py:286-291).  For the pair masks of padded batches, mask = m (x) m with the padding at
 * the end (the reference's pair_mask, pairformer.py:103-112 from loss.py:589): the n_valid valid
 * rows go through one call with mask = NULL, n_keys = n_valid, which neither loads a mask nor
 * visits the padded keys; the padded rows, whose keys are all masked, through a second call
 * with the mask and n_keys = n.  All tensors are the whole-tensor ones of ptx_triattn_fwd;
 * ptx_triattn_fwd is this call with row_begin = 0, row_count = n, n_keys = n.
 */
PTX_API int ptx_triattn_fwd_rows(const void* q, const void* k, const void* vt, const void* g,
                                 const void* tri_bias, const void* mask, void* o, int n, int heads,
                                 int d, int key_pitch, int mask_transposed, float inf, int row_begin,
                                 int row_count, int n_keys, int dtype, void* stream);

/*
 * The fused attention operator on standard-layout tensors: the contract of
 * TriAttentionFunction.forward (tri_attention/op.py:37-77, kernel tri_attention/forward.py:22-188)
 * as called from layers.py:539-583.  For every batch b, row i, head h, query position j:
 *   O[b][i][j][h] = sum_k softmax_k( Q[b][i][j][h] . K[b][i][k][h] + Bias1[b][i][k]
 *                                    + Bias2[b][h][j][k] ) V[b][i][k][h]
 *   Q, K, V, O  [batch][n_rows][s][heads][d] contiguous (Q already scaled by 1/sqrt(d), as the
 *               reference's caller does);  d = 32
 *   Bias1       [batch][n_rows][s] (the reference's [B, N, 1, 1, S] mask bias) or NULL
 *   Bias2       [batch][heads][s][s]
 *   lse         fp32 [batch][n_rows][s][heads] or NULL: log2 of the sum over keys of
 *               2^(logit * log2 e), the reference's M (forward.py:185-188)
 *   workspace   ptx_triattn_core_workspace_elems(n_rows, s, heads) elements of `dtype`,
 *               uninitialised (the operands repacked into the core's tile order)
 * The logits are formed as (q.k + Bias1) + Bias2 in fp32 wherever Bias1 is non-zero, the
 * order of layers.py:286-289; they are never materialised.  n_rows may differ from s (a chunk
 * of rows).  dtype PTX_F32 or PTX_BF16.
 */
PTX_API int64_t ptx_triattn_core_workspace_elems(int n_rows, int s, int heads);
PTX_API int ptx_triattn_core_fwd(const void* q, const void* k, const void* v, const void* bias1,
                         const void* bias2, void* o, float* lse, void* workspace, int batch,
                         int n_rows, int s, int heads, int d, int dtype, void* stream);

/*
 * Backward of the operator above: the contract of TriAttentionFunction.backward
 * (tri_attention/op.py:79-163; kernels tri_attention/backward.py:27-609: preprocess, dK/dV,
 * dQ, dBias2).  With P = 2^(S log2 e - lse), S the logits of the forward, and
 * Delta = sum_d O * dO:
 *   dS = P * (dO V^T - Delta),  dV = P^T dO,  dK = dS^T Q,  dQ = dS K   per (batch, row, head)
 *   dBias2[b][h][j][k] = sum over rows of dS[b][i][j][h][k]
 *   q, k, v, o, dout, dq, dk, dv  [batch][n_rows][s][heads][d] contiguous, q as given to the forward
 *   bias1, bias2, lse             as in the forward (lse is required here)
 *   dbias2   [batch][heads][s][s] in `dtype`, or NULL to skip it
 *   delta    fp32 scratch, n_rows * s * heads elements, uninitialised
 * The gradient of Bias1 is not formed: the reference returns an uninitialised tensor for it
 * (op.py:120, 157-163), its Bias1 being a mask that never requires a gradient.  P is
 * recomputed from the logits; sums run in fp32 and every output is rounded once.
 * dtype PTX_F32 or PTX_BF16.
 */
PTX_API int ptx_triattn_core_bwd(const void* q, const void* k, const void* v, const void* bias1,
                         const void* bias2, const void* o, const float* lse, const void* dout,
                         void* dq, void* dk, void* dv, void* dbias2, float* delta, int batch,
                         int n_rows, int s, int heads, int d, int dtype, void* stream);

/*
 * Triangle attention, stage 3 (layers.py:392-396 + the caller's residual add,
 * pairformer.py:189-213):  out(p) = [z(p) +] W_o o[p], where logical row p maps
 * to z[i][j] or, transposed = 1, z[j][i].  o [heads][n][n][d] as written by
 * stage 2; w_o [c_in][heads*d]; out may alias z.  c_in = 64 or 128 (heads*d = 128), or
 * (PTX_BF16, PTX_MIXED) c_in = heads*d = 256.
 */
PTX_API int ptx_triattn_output(const void* o, const void* w_o, const void* z, void* out, int n,
                       int c_in, int transposed, int add_residual, int dtype, void* stream);

/*
 * Stage 3 with the gate of layers.py:386-390 formed here, from rows this stage loads anyway:
 *   out(p) = [z(p) +] W_o ( sigmoid(W_g LN(z(p))) * o[p] )
 * for o written ungated by stage 2 (g = NULL there and in stage 1): the gate tensor is then
 * neither written nor read.  ln_w / ln_b: the LayerNorm of stage 1 (either may be NULL);
 * w_g [heads*d][c_in], w_o [c_in][heads*d]; gate and gated product are rounded to bf16 as the
 * reference's are.  c_in = 128, heads = 4 (d = 32); dtype PTX_BF16 or PTX_MIXED; out may alias z.
 */
PTX_API int ptx_triattn_gate_output(const void* o, const void* z, const void* ln_w, const void* ln_b,
                            const void* w_g, const void* w_o, void* out, int n, int c_in,
                            int heads, int transposed, int add_residual, float eps, int dtype,
                            void* stream);

/*
 * Transition (primitives.py:190-230), one fused kernel:
 *   out = [x +] W_o ( silu(W_a LN(x)) * (W_b LN(x)) )
 * The hidden activations stay on chip, so there is no workspace; instead the three
 * weight matrices are packed once per weight set into the kernel's streaming order
 * (MFMA operand fragments, grouped in chunks of 32 hidden channels):
 *   ptx_transition_pack:  w_a, w_b [n_factor*c][c], w_o [c][n_factor*c]  ->
 *     packed, ptx_transition_packed_elems(c, n_factor) = 3*n_factor*c*c elements.
 *   ptx_transition_fwd:   x, out [rows][c] (out may alias x), ln_w / ln_b may be NULL.
 * a and b stay in fp32 through the activation (the reference rounds them to the
 * storage dtype first); the product is rounded once.   c = 64, 128 or (PTX_BF16, PTX_MIXED) 256;
 * n_factor*c a multiple of 64.
 */
PTX_API int64_t ptx_transition_packed_elems(int c, int n_factor);
PTX_API int ptx_transition_pack(const void* w_a, const void* w_b, const void* w_o, void* packed, int c,
                        int n_factor, int dtype, void* stream);
PTX_API int ptx_transition_fwd(const void* x, const void* ln_w, const void* ln_b, const void* packed,
                       void* out, int64_t rows, int c, int n_factor, int add_residual, float eps,
                       int dtype, void* stream);

/*
 * The pair transition and the pair bias that follows it in a Pairformer block
 * (pairformer.py:215-222: z = z + pair_transition(z); then attention_pair_bias reads z through
 * transformer.py:191-194), in one launch: ptx_transition_fwd, and from the finished rows, while
 * they pass through the kernel's epilogue,
 *   bias[h][row] = (pb_w LN_pb(out[row]))[h]      pb_w [heads][c], heads <= 32
 * as ptx_pair_bias_fwd computes it from the stored tensor (which would read it once more).
 * bias is fp32 when bias_f32 = 1, else bf16.  c = 128; dtype PTX_BF16 or PTX_MIXED.
 */
PTX_API int ptx_transition_pair_bias_fwd(const void* x, const void* ln_w, const void* ln_b,
                                 const void* packed, void* out, int64_t rows, int c, int n_factor,
                                 int add_residual, float eps, const void* pb_ln_w,
                                 const void* pb_ln_b, const void* pb_w, void* bias, int heads,
                                 int bias_f32, float pb_eps, int dtype, void* stream);

/*
 * The last stage of the ending-node triangle attention and the pair transition that follows
 * it in a Pairformer block (pairformer.py:201-217: z = z + tri_att_end(z); z = z +
 * pair_transition(z)), in one launch: what ptx_triattn_gate_output (add_residual = 1) followed
 * by ptx_transition_fwd / ptx_transition_pair_bias_fwd (add_residual = 1) compute, bit for bit,
 * without the pair tensor between the two travelling through memory (both stages are local to
 * a pair position, and nothing else reads that tensor):
 *   z' = z + W_o (sigmoid(W_g LN_att(z)) * o),   out = z' + transition(z')   [, bias from out]
 * o: the attention core's output, head-major [4][n*n][32] (rows in the attention's logical
 * order: with transposed = 1 row (i, j) belongs to z[j][i]); z, out [n][n][128] (out may be z).
 * The weights of both stages are packed once per weight set:
 *   ptx_triattn_output_transition_pack: w_g, w_o [128][128] of the attention, w_a, w_b
 *     [n_factor*128][128], w_to [128][n_factor*128] of the transition -> packed,
 *     ptx_triattn_output_transition_packed_elems(n_factor) elements.
 * pb_w = NULL: no pair bias (bias, pb_* unused).  c_in = 128, heads = 4 (of 32); dtype
 * PTX_BF16 or PTX_MIXED.
 */
PTX_API int64_t ptx_triattn_output_transition_packed_elems(int n_factor);
PTX_API int ptx_triattn_output_transition_pack(const void* w_g, const void* w_o, const void* w_a,
                                       const void* w_b, const void* w_to, void* packed,
                                       int n_factor, int dtype, void* stream);
PTX_API int ptx_triattn_output_transition_fwd(const void* o, const void* z, const void* att_ln_w,
                                      const void* att_ln_b, const void* packed, const void* ln_w,
                                      const void* ln_b, void* out, int n, int c_in, int heads,
                                      int transposed, int n_factor, float att_eps, float eps,
                                      const void* pb_ln_w, const void* pb_ln_b, const void* pb_w,
                                      void* bias, int pb_heads, int bias_f32, float pb_eps,
                                      int dtype, void* stream);

/*
 * Pair bias of the single-representation attention (transformer.py:191-194):
 *   bias[h][i][j] = (W LN(z[i][j]))[h],  W [heads][c_z], heads <= 32, c_z = 128 or
 * (PTX_BF16, PTX_MIXED) 256.
 * ln_b may be NULL.  bias is fp32 when out_f32 = 1, else `dtype`.
 */
PTX_API int ptx_pair_bias_fwd(const void* z, const void* ln_w, const void* ln_b, const void* w,
                      void* bias, int n, int c_z, int heads, int out_f32, float eps, int dtype,
                      void* stream);

/*
 * The single-representation track of a Pairformer block (c_s = 384): small operands that stay
 * in the L2, so these entry points aim at few launches, not at a roofline.
 *
 * ptx_linear_fwd: Linear / LinearNoBias (primitives.py:83-98, F.linear):
 *   out = [res +] x w^T [+ bias]      x [rows][k], w [n_out][k], bias [bias_cols] or NULL (added
 *   to output columns < bias_cols), res [rows][n_out] or NULL, out [rows][split_col].
 *   Output columns >= split_col are stored transposed in out_t [n_out - split_col][ldt] (entries
 *   of rows in [rows, ldt) are written as zeros) - how the attention below wants V; pass
 *   split_col = n_out (and out_t = NULL) for a plain linear layer.  k % 16 == 0, n_out % 8 == 0.
 * ptx_swiglu_fwd: first half of Transition (primitives.py:206-230) for widths the fused
 *   ptx_transition_fwd has no kernel for:  out [rows][hidden] = silu(x w_a^T) * (x w_b^T).
 * ptx_single_attention_fwd: attention with pair bias and gating (transformer.py:196-254,
 *   primitives.py:233-291, 636-879), per head h:
 *   out[i][h] = sigmoid(g[i][h]) * sum_j softmax_j( q[i][h].k[j][h] * scale + bias[h][i][j] ) v[j][h]
 *   q, k, g: rows of pitch ld holding heads * d channels, head-major (g NULL: no gate);
 *   vt [heads * d][ldt], keys in [n, ldt) zero (as ptx_linear_fwd's out_t); bias [heads][n][n],
 *   fp32 (bias_f32 = 1) or `dtype`, or NULL; out rows of pitch ldo.  d = 8, 16, 24 or 32.
 *   Logits and softmax in fp32; the n x n logits are never materialised.
 */
PTX_API int ptx_linear_fwd(const void* x, const void* w, const void* bias, int bias_cols,
                   const void* res, void* out, void* out_t, int split_col, int64_t ldt, int rows,
                   int k, int n_out, int dtype, void* stream);
PTX_API int ptx_swiglu_fwd(const void* x, const void* w_a, const void* w_b, void* out, int rows, int k,
                   int hidden, int dtype, void* stream);
PTX_API int ptx_single_attention_fwd(const void* q, const void* k, const void* vt, const void* g,
                   const void* bias, int bias_f32, void* out, int n, int heads, int d, int64_t ld,
                   int64_t ldt, int64_t ldo, float scale, int dtype, void* stream);

/*
 * Measurement aid with no counterpart in the reference: streams `bytes` (a multiple of 16)
 * through the GPU with plain 16-byte accesses - a copy (src and dst), a read-only pass (dst
 * NULL) or a write-only pass (src NULL), with non-temporal accesses when nontemporal = 1.  Its
 * rate on a tensor of a kernel's size is the ceiling that kernel's achieved HBM bandwidth is
 * reported against (bench.py, `hbm_ceiling`); src and dst must not overlap.
 */
PTX_API int ptx_hbm_stream(const void* src, void* dst, int64_t bytes, int nontemporal, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PROTENIX_AMD_H_ */
