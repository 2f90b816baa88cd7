/*
 * C ABI of libatorch_amd_fp8.so: hand-written gfx950 (MI355X) kernels for the
 * FP8 grouped-linear MoE expert path.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller (the caller
 *     allocates all outputs and workspaces); nothing here allocates device
 *     memory or synchronises the host with the device;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     kernels are only enqueued;
 *   - functions return AAMD_OK (0) or an error code; aamd_last_error() gives
 *     the message of the last failure on the calling thread;
 *   - fp8 tensors are OCP e4m3fn codes, one byte each; scales are fp32
 *     dequantisation scales  s = max(amax, eps) / 448  (0 -> 1);
 *   - `dtype` arguments: AAMD_BF16 or AAMD_F32 (also AAMD_NONE where stated; the inputs of
 *     aamd_quant_1x128, aamd_permute_quant_1x128, aamd_quant_1x128_dual_grouped,
 *     aamd_permute_quant_1x128_dual_grouped and aamd_quant_128x128 may also be AAMD_F16).
 *
 * Each entry point names the reference interface it replaces (paths relative
 * to the reference tree root).
 */
#ifndef ATORCH_AMD_FP8_H
#define ATORCH_AMD_FP8_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default) /* the entry points are the only symbols the library exports */

#define AAMD_OK 0
#define AAMD_ERR_ARG 1 /* bad shape / alignment / dtype */
#define AAMD_ERR_HIP 2 /* the HIP runtime refused the launch */

#define AAMD_NONE (-1)
#define AAMD_BF16 0
#define AAMD_F32 1
#define AAMD_F16 2 /* accepted as the input type of the quantisers only */

/* Layouts of the transposed 1x128 codes q_t of R rows (columns of the quantised tensor) and ld_t padded tokens:
 *   AAMD_QT_ROWS     q_t [R, ld_t]: one row of ld_t bytes per column of x;
 *   AAMD_QT_BLOCKED  q_t [ld_t / 128, R, 128]: token-block-major, byte (r, t) at ((t / 128) * R + r) * 128 + t % 128.
 * The second is what the grouped kernels use among themselves: a 128 x 128 tile of codes is 16 KB of consecutive
 * bytes, which the quantisers write as one sequential sweep and the weight-gradient GEMM loads as whole slabs.
 * The scales s_t [ld_t / 128, R] are the same in both. */
#define AAMD_QT_ROWS 0
#define AAMD_QT_BLOCKED 1

#define AAMD_ABI_VERSION 4

/* Library identity and error text. */
int aamd_abi_version(void);
const char *aamd_last_error(void);

/*
 * 1x128 tile quantisation.
 * Replaces tile_quant / tile_quant_kernel, atorch/modules/fp8/triton_kernel.py:94-140
 * (dispatch: Fp8Quantization.quantize_tilewise, atorch/modules/fp8/quantize.py:176-201).
 *   x [rows, cols] (row stride ldx elements), cols % 128 == 0
 *   q [rows, cols] codes, s [rows, cols/128] fp32, both dense.
 */
int aamd_quant_1x128(const void *x, int x_dtype, int64_t rows, int64_t cols, int64_t ldx, uint8_t *q, float *s,
                     float eps, void *stream);

/*
 * Token permute fused into the 1x128 quantisation: every token row is read and
 * quantised once and written to its topk destination rows.
 * Replaces permute (atorch/modules/moe/token_dispatcher.py:89-116) followed by the
 * per-expert quantize calls of atorch/modules/fp8/quantized_grouped_linear.py:90-101.
 *   x [T, cols]; row_map [T*topk] int32: destination (permuted) row of flat
 *   index token*topk+slot, or -1 when that copy is dropped;
 *   q [M_out, cols], s [M_out, cols/128] dense; rows no map entry points to are not written.
 */
int aamd_permute_quant_1x128(const void *x, int x_dtype, int64_t T, int64_t cols, int64_t ldx,
                             const int32_t *row_map, int topk, int64_t M_out, uint8_t *q, float *s, float eps,
                             void *stream);

/*
 * Token permute without quantisation (rows of bf16 or fp32 copied to their topk permuted
 * positions, each source row read once).
 * Replaces permute, atorch/modules/moe/token_dispatcher.py:89-116 (index_select on the argsort).
 *   x [T, cols] dense; out [M_out, cols] dense; cols * element size must be a multiple of 16.
 */
int aamd_permute_rows(const void *x, int x_dtype, int64_t T, int64_t cols, const int32_t *row_map, int topk,
                      int64_t M_out, void *out, void *stream);

/*
 * Row-wise AND transposed 1x128 quantisation of ragged groups in one pass over x
 * ("return_transpose=True").
 * Replaces quantize_op.quantize(x_i, params, return_transpose=True) per expert,
 * quantized_grouped_linear.py:90-101 and :200-206; the transposed result is defined
 * in-tree as tile_quant(x_i.t().contiguous()), atorch/modules/fp8/scaled_linear.py:402-414,
 * with a partial last token tile zero padded.
 *   x [M, cols]; group_offsets [E+1] int64 (device) exclusive prefix of rows per group;
 *   q [M, cols], s [M, cols/128]              (both may be NULL: transposed only)
 *   q_t, in the layout q_t_layout names: token poff_g + m of column c holds the code of x[off_g + m, c], where
 *       poff_g = sum_{j<g} ceil(M_j/128)*128; pad tokens of a group are written 0
 *   s_t [ld_t/128, cols]: s_t[poff_g/128 + m/128, c]
 *   ld_t % 128 == 0 and ld_t >= poff_E (M + 127*E rounded up to 128 always suffices)
 *   tile_ws: E+1 int32 of scratch.
 */
int aamd_quant_1x128_dual_grouped(const void *x, int x_dtype, int64_t M, int64_t cols, int64_t ldx,
                                  const int64_t *group_offsets, int E, int32_t *tile_ws, uint8_t *q, float *s,
                                  uint8_t *q_t, float *s_t, int64_t ld_t, int q_t_layout, float eps, void *stream);

/*
 * The token permute fused into aamd_quant_1x128_dual_grouped: x holds the tokens in their original order and
 * every output row j (expert-contiguous order) is quantised from token sorted_idx[j] / topk, so the permuted
 * bf16 rows are never written or re-read on the way to the grouped GEMMs of a training step.
 * Replaces permute (atorch/modules/moe/token_dispatcher.py:89-116: argsort, index_select on sorted // topk)
 * followed by the per-expert quantize_op.quantize(x_i, x_params, return_transpose=True) calls of
 * atorch/modules/fp8/quantized_grouped_linear.py:90-101.
 *   x [T, cols] (row stride ldx elements); sorted_idx [M] int64 (device): flat index token*topk+slot of
 *   permuted row j, the sorted_idx of aamd_moe_preprocess (M < T*topk when copies were dropped);
 *   T*topk < 2^31; group_offsets [E+1] int64 exclusive prefix of permuted rows per group;
 *   q [M, cols], s [M, cols/128] (both may be NULL), q_t, s_t [ld_t/128, cols], tile_ws, ld_t and q_t_layout
 *   as for aamd_quant_1x128_dual_grouped.  Results equal aamd_permute_rows followed by
 *   aamd_quant_1x128_dual_grouped bit for bit.
 */
int aamd_permute_quant_1x128_dual_grouped(const void *x, int x_dtype, int64_t T, int64_t cols, int64_t ldx,
                                          const int64_t *sorted_idx, int topk, int64_t M,
                                          const int64_t *group_offsets, int E, int32_t *tile_ws, uint8_t *q, float *s,
                                          uint8_t *q_t, float *s_t, int64_t ld_t, int q_t_layout, float eps,
                                          void *stream);

/*
 * 128x128 block quantisation of E weight matrices, optionally also emitting the
 * transposed codes and scale grid.
 * Replaces block_quant / block_quant_kernel, triton_kernel.py:21-46 (dispatch
 * quantize.py:204-232) and w_fp8.t().contiguous() / scale.t().contiguous(),
 * scaled_linear.py:359-365.
 *   w [E, N, K] (expert stride in elements; rows dense), N % 128 == 0, K % 128 == 0
 *   q [E, N, K], s [E, N/128, K/128]; q_t [E, K, N], s_t [E, K/128, N/128] (q_t/s_t may be NULL).
 */
int aamd_quant_128x128(const void *w, int w_dtype, int64_t E, int64_t N, int64_t K, int64_t expert_stride,
                       uint8_t *q, float *s, uint8_t *q_t, float *s_t, float eps, void *stream);

/*
 * Dequantisation y = code * scale.
 * Replaces dequant, triton_kernel.py:49-91.  tile_scale != 0: s [M, N/128]; else s [M/128, N/128].
 */
int aamd_dequant(const uint8_t *q, const float *s, int64_t M, int64_t N, int tile_scale, void *y, int y_dtype,
                 void *stream);

/*
 * SwiGLU fused into the 1x128 quantisation of the intermediate activations (the step between
 * the two grouped GEMMs of an expert MLP): for rows [a | b] of the first GEMM's output,
 *   h = bf16(bf16(silu(a)) * b)   (silu(x) = x / (1 + exp(-x)) in fp32)
 * is quantised like aamd_quant_1x128 / aamd_quant_1x128_dual_grouped would quantise h, without h
 * making a round trip through memory.
 * Replaces SwiGLUActivatition.forward, atorch/modules/moe/grouped_gemm_moe.py:331-334 (torch.chunk,
 * F.silu, multiply), as used between the gmm calls of compute_moe, :845-850, followed by the
 * per-expert quantize_op.quantize of the next grouped linear, quantized_grouped_linear.py:90-101.
 *   fc1 [rows, 2F] bf16 (row stride ld elements, ld >= 2F), F % 128 == 0
 *   h_out [rows, F] bf16 or NULL (the activation itself, for callers that keep it)
 *   q [rows, F], s [rows, F/128]; the dual form adds q_t / s_t with the layouts, scratch and
 *   group_offsets of aamd_quant_1x128_dual_grouped (q and s may then be NULL).
 */
int aamd_swiglu_quant_1x128(const void *fc1, int64_t rows, int64_t F, int64_t ld, void *h_out, uint8_t *q, float *s,
                            void *stream);
int aamd_swiglu_quant_1x128_dual_grouped(const void *fc1, int64_t M, int64_t F, int64_t ld,
                                         const int64_t *group_offsets, int E, int32_t *tile_ws, void *h_out,
                                         uint8_t *q, float *s, uint8_t *q_t, float *s_t, int64_t ld_t, int q_t_layout,
                                         void *stream);

/*
 * Backward of the gated activation fused into the quantisation of its gradient: for the gradient dh
 * of h and the saved rows [a | b], the rows [da | db] of d(fc1) are quantised 1x128 row-wise and
 * transposed inside the ragged groups without being written in bf16.
 * Replaces what autograd runs for SwiGLUActivatition.forward, atorch/modules/moe/grouped_gemm_moe.py:331-334
 * (the backward of the multiply, then silu_backward) followed by the per-expert quantize_op.quantize
 * calls of the first grouped linear's backward, quantized_grouped_linear.py:202-206.
 *   dh [M, F] bf16 (row stride ld_dh), fc1 [M, 2F] bf16 (row stride ld), F % 128 == 0
 *   g_out [M, 2F] bf16 or NULL (the gradient itself, for callers that keep it)
 *   q [M, 2F], s [M, 2F/128] (both may be NULL), q_t (2F rows), s_t [ld_t/128, 2F];
 *   group_offsets, tile_ws, ld_t, q_t_layout as for aamd_quant_1x128_dual_grouped.
 */
int aamd_swiglu_bwd_quant_1x128_dual_grouped(const void *dh, int64_t ld_dh, const void *fc1, int64_t ld, int64_t M,
                                             int64_t F, const int64_t *group_offsets, int E, int32_t *tile_ws,
                                             void *g_out, uint8_t *q, float *s, uint8_t *q_t, float *s_t,
                                             int64_t ld_t, int q_t_layout, void *stream);

/*
 * GELU, the expert MLP's default activation, fused into the same quantisers:
 *   h = bf16(x/2 * (1 + erf(x / sqrt 2)))  computed in fp32 from bf16 x, quantised like aamd_quant_1x128 /
 *   aamd_quant_1x128_dual_grouped would quantise h; with dh != NULL the dual form quantises the gradient
 *   g = bf16(dh * (cdf(x) + x * pdf(x))) instead (autograd's gelu_backward).
 * Replaces self.activation = torch.nn.functional.gelu, atorch/modules/moe/grouped_gemm_moe.py:449, applied at
 * :849 between the gmm calls, and what autograd runs for it, each followed by the per-expert
 * quantize_op.quantize of the next grouped GEMM's operand (quantized_grouped_linear.py:90-101, 202-206).
 *   x [rows, F] bf16 (row stride ld), F % 128 == 0; dh [rows, F] bf16 with the same row stride ld
 *   h_out [rows, F] bf16 or NULL (h, or g in the backward form); other arguments as the SwiGLU forms.
 */
int aamd_gelu_quant_1x128(const void *x, int64_t rows, int64_t F, int64_t ld, void *h_out, uint8_t *q, float *s,
                          void *stream);
int aamd_gelu_quant_1x128_dual_grouped(const void *x, const void *dh, int64_t M, int64_t F, int64_t ld,
                                       const int64_t *group_offsets, int E, int32_t *tile_ws, void *h_out, uint8_t *q,
                                       float *s, uint8_t *q_t, float *s_t, int64_t ld_t, int q_t_layout, void *stream);

/*
 * Ragged grouped block-scaled GEMM, "NT": for every group g and its rows m,
 *   C[m, n] = sum_kb dot(A[m, kb], B_g[n, kb]) * a_s[m, kb] * b_s_g[n/128 or n, kb]  (+ bias_g[n])
 * fp8 x fp8 MFMA, fp32 accumulation, scales applied per 128-deep block.
 * Replaces fp8_gemm / fp8_gemm_kernel, triton_kernel.py:143-210, and
 * quantize_op.grouped_qgemm for fprop and dgrad, quantized_grouped_linear.py:141-151, 214-223.
 *   a [M, K] codes (row stride lda bytes), a_s [M, K/128]
 *   b [E, N, K] codes dense, b_s [E, N/128, K/128] (b_tile_scaled == 0) or [E, N, K/128] (!= 0)
 *   group_offsets [E+1] int64 device, or NULL for a single group [0, M] (then E must be 1)
 *   c [M, N] of c_dtype (row stride ldc elements, rows 16-byte aligned); rows of empty groups are not touched
 *   bias [E, N] of bias_dtype or NULL (AAMD_NONE); tile_ws: E+1 int32 scratch.
 *   K % 128 == 0, N % 128 == 0.
 */
int aamd_grouped_gemm_fp8_nt(const uint8_t *a, int64_t lda, const float *a_s, const uint8_t *b, const float *b_s,
                             int b_tile_scaled, const int64_t *group_offsets, int E, int32_t *tile_ws, int64_t M,
                             int64_t N, int64_t K, void *c, int c_dtype, int64_t ldc, const void *bias,
                             int bias_dtype, void *stream);

/*
 * aamd_grouped_gemm_fp8_nt for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the same arguments without
 * tile_ws.  No counterpart in the reference.  The E+1 ints of scratch live in a static device array
 * of the library (AAMD_STATIC_MAX_GROUPS + 1 ints per GPU, held until the process ends); the call
 * allocates and frees nothing.  E > AAMD_STATIC_MAX_GROUPS is rejected with AAMD_ERR_ARG.  All calls
 * on one GPU share that array: calls that may overlap on one GPU (different streams) race on it.
 */
#define AAMD_STATIC_MAX_GROUPS 4096
int aamd_grouped_gemm_fp8_nt_static(const uint8_t *a, int64_t lda, const float *a_s, const uint8_t *b,
                                    const float *b_s, int b_tile_scaled, const int64_t *group_offsets, int E,
                                    int64_t M, int64_t N, int64_t K, void *c, int c_dtype, int64_t ldc,
                                    const void *bias, int bias_dtype, void *stream);

/*
 * Grouped weight-gradient GEMM: dW_g[n, k] (+)= sum over the tokens m of group g of
 * dY[m, n] * X[m, k], both operands 1x128-scaled along the tokens (layouts of
 * aamd_quant_1x128_dual_grouped's q_t / s_t).
 * Replaces quantize_op.grouped_qgemm(qdy_t, qx_t, mm_wgrad, ..., accumulate=...),
 * quantized_grouped_linear.py:243-253.
 *   dyt (N rows), sdyt [ld_t/128, N]; xt (K rows), sxt [ld_t/128, K]; both code operands in the layout
 *   q_t_layout names (AAMD_QT_ROWS: [N, ld_t] and [K, ld_t]; AAMD_QT_BLOCKED: [ld_t/128, N, 128] and
 *   [ld_t/128, K, 128])
 *   dw [E, N, K] of dw_dtype (expert stride in elements); an empty group gives zeros,
 *   or leaves dw_g untouched when accumulate != 0.
 *   ld_t must cover the padded token total sum_g ceil(M_g/128)*128, which only the device knows:
 *   a group whose tokens lie beyond ld_t gets NaN in its dw_g instead of a wrong finite gradient.
 */
int aamd_grouped_gemm_fp8_wgrad(const uint8_t *dyt, const float *sdyt, const uint8_t *xt, const float *sxt,
                                int64_t ld_t, int q_t_layout, const int64_t *group_offsets, int E, int32_t *tile_ws,
                                int64_t N, int64_t K, void *dw, int dw_dtype, int64_t expert_stride, int accumulate,
                                void *stream);

/*
 * Inverse permutation + weighted combine in one gather-reduce pass:
 *   out[t, :] = sum_j probs[t, j] * y[row_map[t*topk + j], :]
 * Replaces unpermute, token_dispatcher.py:119-161 (zeros + index_copy_ + multiply + sum).
 * Each product is rounded to the promoted dtype before the fp32 sum, as the reference's
 * separate multiply and sum do (:156-159); the sum adds in the order of torch's GPU reduction
 * (slot j into accumulator j mod 4, then ((a0 + a1) + a2) + a3).
 *   y [M, H] of y_dtype (bf16 or fp32); row_map [T*topk] int32 (-1 = dropped copy, contributes 0)
 *   probs [T, topk] of probs_dtype, or AAMD_NONE (probs ignored); out [T, H] has the promoted type of
 *   rows and probs: bf16 for bf16 rows with bf16 or no probs, fp32 otherwise; H % 8 == 0.
 */
int aamd_unpermute_combine(const void *y, int y_dtype, int64_t M, int64_t H, const int32_t *row_map,
                           const void *probs, int probs_dtype, int64_t T, int topk, void *out, void *stream);

/*
 * The two gradients of that combine, as autograd derives them from the reference's torch ops
 * (token_dispatcher.py:155-159: index_copy_, multiply by probs, sum over topk):
 *   permute_rows_scaled: d_y[row_map[t*topk+j], :] = (out_dtype)(d_out[t, :] * probs[t, j]), the product
 *     formed in fp32 and rounded once; with probs_dtype == AAMD_NONE it is the plain permute with a
 *     conversion.  x [T, cols] of x_dtype, out [M_out, cols] of out_dtype (bf16 -> bf16, fp32 -> bf16,
 *     fp32 -> fp32); cols % 8 == 0; rows no map entry points to are not written.
 *   unpermute_probs_grad: d_probs[t, j] = sum_h d_out[t, h] * y[row_map[t*topk+j], h] in fp32
 *     (0 for a dropped copy); d_probs [T, topk] fp32, the caller casts.
 */
int aamd_permute_rows_scaled(const void *x, int x_dtype, int64_t T, int64_t cols, const int32_t *row_map, int topk,
                             const void *probs, int probs_dtype, int64_t M_out, void *out, int out_dtype,
                             void *stream);
int aamd_unpermute_probs_grad(const void *dout, int dout_dtype, const void *y, int y_dtype, int64_t M, int64_t H,
                              const int32_t *row_map, int64_t T, int topk, float *dprobs, void *stream);

/*
 * Router preprocess on the device, no host round trip: histogram of expert ids,
 * exclusive scan, stable counting sort.
 * Replaces the argsort of permute (token_dispatcher.py:107-112) and the histc + .cpu()
 * of MoEAllToAllTokenDispatcher.preprocess (token_dispatcher.py:297-353).
 *   expert_ids [n] (n = T*topk; int64 when ids_are_i64 != 0, else int32), values in [0, E)
 *   sorted_idx [n] int64: flat index of permuted row j (the reference's sorted_indices); may be NULL
 *   row_map [n] int32: permuted row of flat index i (inverse of sorted_idx)
 *   group_offsets [E+1] int64: exclusive prefix of tokens per expert
 *   ws: aamd_moe_preprocess_ws_ints(n, E) int32 of scratch.
 */
int64_t aamd_moe_preprocess_ws_ints(int64_t n, int E);
int aamd_moe_preprocess(const void *expert_ids, int ids_are_i64, int64_t n, int E, int64_t *sorted_idx,
                        int32_t *row_map, int64_t *group_offsets, int32_t *ws, void *stream);

/*
 * row_map[sorted_idx[j]] = j for j < n_perm, -1 elsewhere (n_flat entries).
 * Adapter from the reference's sorted_indices (token_dispatcher.py:112,136) to row_map.
 */
int aamd_invert_permutation(const int64_t *sorted_idx, int64_t n_perm, int64_t n_flat, int32_t *row_map,
                            void *stream);

/*
 * Per-expert bias on rows tagged with their expert: out[t, :] = inp[t, :] + bias[bin_ids[t], :]
 * (bf16: the fp32 sum rounded to bf16), and its bias gradient bgrad[e, :] = sum of grad[t, :] over
 * the rows with bin_ids[t] == e, accumulated in fp32 (order of the additions unspecified, as with
 * the reference's atomic adds; the caller casts to the gradient's dtype).
 * Replaces bias_gather_add_fw / bias_gather_add_bw, atorch/kernels/triton_jit/bias_gather_add.py:50-66, 101-127.
 *   inp, out, grad [T, H] and bias [E, H] of `dtype`; H * sizeof(dtype) % 16 == 0
 *   bin_ids [T]: int64 when ids_are_i64 != 0, else int32; rows tagged outside [0, E) pass through
 *   unchanged and add nothing to bgrad
 *   bgrad [E, H] fp32, cleared by the call.
 */
int aamd_bias_gather_add(const void *inp, const void *bias, const void *bin_ids, int ids_are_i64, int64_t T,
                         int64_t H, int E, int dtype, void *out, void *stream);
int aamd_bias_gather_add_bgrad(const void *grad, const void *bin_ids, int ids_are_i64, int64_t T, int64_t H, int E,
                               int dtype, float *bgrad, void *stream);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* ATORCH_AMD_FP8_H */
