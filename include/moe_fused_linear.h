/*
 * moe_fused_linear.h -- C ABI of the MI355X (gfx950) moe_fused_linear library.
 *
 * The reference implements this path as in-process Python calls of Triton-JIT
 * kernels; it has no FFI of its own.  Each entry point below replaces one such
 * Python-level kernel wrapper and cites it (paths relative to the reference).
 *
 * Conventions shared by all entry points
 *   - all pointers are DEVICE pointers unless stated otherwise; tensors are dense,
 *     row-major, contiguous;
 *   - `stream` is a hipStream_t passed as void*; every call only enqueues work on
 *     it: no synchronisation, no allocation, no host read of device data;
 *   - return value: 0 = OK, negative = argument error (MFL_ERR_*), positive =
 *     hipError_t of a failed launch;
 *   - global state of the library, all of it: the properties of the device that is current at
 *     the first call (cached read-only: one kind of device per process), one flag per kernel
 *     and device saying that the kernel's launch attribute has been set there (atomic; two
 *     threads racing through a first call both set the same value), and the fixed scratch
 *     array of mfl_expert_sort_static, which is device memory that calls on one GPU share
 *     (see there).  Apart from that array the calls are re-entrant and thread-safe;
 *   - the code objects are built for gfx950 only, and the work distribution of the GEMM
 *     kernels assumes its 8 XCDs (workgroup b runs on XCD b % 8, each XCD with an L2 of its
 *     own): on another part the library does not load its kernels at all.
 */
#ifndef MOE_FUSED_LINEAR_H
#define MOE_FUSED_LINEAR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MFL_ABI_VERSION 1

/* the library is built with hidden visibility: these entry points are all it exports */
#define MFL_API __attribute__((visibility("default")))

/* element types */
#define MFL_BF16 0
#define MFL_F32 1
#define MFL_F16 2
/* index types */
#define MFL_I32 0
#define MFL_I64 1

/* argument errors */
#define MFL_OK 0
#define MFL_ERR_NULL (-1)        /* required pointer is NULL                        */
#define MFL_ERR_SHAPE (-2)       /* negative / zero / inconsistent dimension        */
#define MFL_ERR_DTYPE (-3)       /* unknown or unsupported element / index type     */
#define MFL_ERR_ALIGN (-4)       /* pointer not aligned to its element size         */
#define MFL_ERR_WORKSPACE (-5)   /* workspace missing or too small                  */
#define MFL_ERR_UNSUPPORTED (-6) /* valid request this build has no kernel for      */
#define MFL_ERR_LIMIT (-7)       /* size beyond a fixed maximum of the entry point   */

MFL_API int mfl_abi_version(void);
/* Static, NUL-terminated description of a return code of this library. */
MFL_API const char *mfl_strerror(int code);

/* ---- grouped GEMM ---------------------------------------------------------------
 * Rows of x are grouped by expert, ascending; m_sizes[e] rows belong to expert e and
 * sum(m_sizes) <= R.  Rows past sum(m_sizes) are not written.  m_sizes is read on the
 * device (no host sync).  fp32 accumulation; out = alpha * acc (+ out if accumulate).
 * in_dtype is the type of both x and w; out_dtype the type of the result. */

/* y[m, n] = sum_k w[e(m), n, k] * x[m, k];  x (R,K), w (E,N,K), y (R,N).
 * Replaces grouped_gemm_forward, qwen3_moe_fused/grouped_gemm/forward.py:116-160. */
MFL_API int mfl_gemm_fwd(const void *x, const void *w, const void *m_sizes, int m_sizes_dtype, void *y,
                 int64_t R, int N, int K, int E, int in_dtype, int out_dtype, float alpha,
                 int accumulate, void *stream);

/* dx[m, n] = sum_k w[e(m), k, n] * dy[m, k];  dy (R,K), w (E,K,N), dx (R,N).
 * Replaces grouped_gemm_forward_transposed,
 * qwen3_moe_fused/grouped_gemm/forward_transposed.py:107-151. */
MFL_API int mfl_gemm_dx(const void *dy, const void *w, const void *m_sizes, int m_sizes_dtype, void *dx,
                int64_t R, int N, int K, int E, int in_dtype, int out_dtype, float alpha,
                int accumulate, void *stream);

/* dw[e, n, k] = sum_{m in e} dy[m, n] * x[m, k];  x (R,K), dy (R,N), dw (E,N,K).
 * Every element of dw is written; experts without rows get exact zeros.
 * Replaces grouped_gemm_backward_dw, qwen3_moe_fused/grouped_gemm/backward_dw.py:92-134. */
MFL_API int mfl_gemm_dw(const void *x, const void *dy, const void *m_sizes, int m_sizes_dtype, void *dw,
                int64_t R, int N, int K, int E, int in_dtype, int out_dtype, float alpha,
                int accumulate, void *stream);

/* mfl_gemm_dw for a product with one thin side -- N or K equal to 8, 16, 32 or 64 (the rank of a LoRA adapter,
 * qwen3_moe_fused/lora.py:71-72: the products dA and dB of qwen3_moe_fused/kernels/fast_lora.py:121-125,
 * 139-149), the other side a multiple of 256, bf16 operands, bf16 or fp32 result, at most 512 experts.
 * The rows are dealt out evenly over the workgroups whatever the sizes of the experts; an expert cut by
 * such a border is summed from fp32 partial results in a fixed order (same bits from run to run).
 * Every element of dw is written.  workspace: mfl_gemm_dw_split_workspace(R, N, K, E) bytes of device
 * memory, contents ignored; that function returns 0 for a shape this entry point does not take, and the
 * call then returns MFL_ERR_UNSUPPORTED: use mfl_gemm_dw. */
MFL_API size_t mfl_gemm_dw_split_workspace(int64_t R, int N, int K, int E);
MFL_API int mfl_gemm_dw_split(const void *x, const void *dy, const void *m_sizes, int m_sizes_dtype, void *dw,
                      int64_t R, int N, int K, int E, int in_dtype, int out_dtype, float alpha,
                      void *workspace, size_t ws_bytes, void *stream);

/* Forward GEMM with NF4 weights decoded inside the K loop:
 * w[e, n, k] = code16[nibble] * absmax[(e*N*K + n*K + k) / blocksize], rounded once to
 * in_dtype; byte i of wq holds element 2i in its high nibble, 2i+1 in its low nibble.
 * code16 (16 floats) and absmax (E*N*K/blocksize floats) are device pointers.
 * Replaces grouped_gemm_forward_4bit, qwen3_moe_fused/grouped_gemm/forward_4bit.py:135-208. */
MFL_API int mfl_gemm_fwd_nf4(const void *x, const uint8_t *wq, const float *code16, const float *absmax,
                     int blocksize, const void *m_sizes, int m_sizes_dtype, void *y, int64_t R,
                     int N, int K, int E, int in_dtype, int out_dtype, void *stream);

/* Input-gradient product with NF4 weights: dx[m, n] = sum_k w[e(m), k, n] * dy[m, k] with
 * w (E,K,N) packed as in mfl_gemm_fwd_nf4 (the forward weight (E, out=K, in=N) as stored);
 * out = alpha * acc (+ out if accumulate).  The reference dequantises the whole matrix for this
 * product (qwen3_moe_fused/kernels/fast_lora.py:57-63,127-131; quantize/layer.py:17-22 under
 * autograd).  Returns MFL_ERR_UNSUPPORTED, with nothing enqueued, unless the element type is
 * bf16, K % 64 == 0, N % 32 == 0, blocksize >= 8, E <= 512 and the pointers are 16-byte
 * aligned; the caller then dequantises (mfl_nf4_dequant) and calls mfl_gemm_dx. */
MFL_API int mfl_gemm_dx_nf4(const void *dy, const uint8_t *wq, const float *code16, const float *absmax,
                    int blocksize, const void *m_sizes, int m_sizes_dtype, void *dx, int64_t R,
                    int N, int K, int E, int in_dtype, int out_dtype, float alpha, int accumulate,
                    void *stream);

/* Input gradient with two terms in one kernel: dx = dy1 w1 + dy2 w2 (each term as in
 * mfl_gemm_dx; one reduction over both, one rounding, one pass over dx).  It is the input
 * gradient of the gated unit, de w_gate + dg w_up, which the reference forms as two products
 * and an addition (autograd of modular_qwen3_moe_fused.py:106-108;
 * kernels/fast_lora.py:151-152 with LoRA).  Returns MFL_ERR_UNSUPPORTED, with nothing
 * enqueued, unless the element type is bf16, K % 64 == 0, N % 8 == 0, E <= 512 and the
 * pointers are 16-byte aligned; the caller then calls mfl_gemm_dx twice (accumulate = 1). */
MFL_API int mfl_gemm_dx_dual(const void *dy1, const void *w1, const void *dy2, const void *w2,
                     const void *m_sizes, int m_sizes_dtype, void *dx, int64_t R, int N, int K,
                     int E, int in_dtype, int out_dtype, void *stream);

/* The input gradient of the down projection with the backward of the gated unit in its epilogue:
 * dh = mfl_gemm_dx(dy, w) is not stored; de, dg (and h = silu(e) * g again where h is not NULL) leave the kernel
 * as mfl_silu_mul_bwd computes them from a stored bf16 dh, bit for bit.  dy (R,K), w (E,K,N) as in mfl_gemm_dx;
 * e, g, de, dg, h (R,N); de may be e and dg may be g (in place).  bf16 only.  Saves the (R,N) round trip of dh
 * and one launch per training step (qwen3_moe_fused/kernels/fast_lora.py:133-137 followed by
 * kernels/silu_mul.py:84-111 in the reference).  MFL_ERR_UNSUPPORTED for shapes outside the pipelined kernels:
 * the caller then runs mfl_gemm_dx and mfl_silu_mul_bwd. */
MFL_API int mfl_gemm_dx_silu_bwd(const void *dy, const void *w, const void *e, const void *g,
                         const void *m_sizes, int m_sizes_dtype, void *de, void *dg, void *h, int64_t R,
                         int N, int K, int E, int dtype, void *stream);

/* A product with the rank-r term of a LoRA adapter in the same reduction: one accumulator, one
 * rounding, one pass over the output, where the reference adds the two products
 * (qwen3_moe_fused/lora.py:134; matmul_lora at kernels/fast_lora.py:65-88,127-131,151-152).
 *   mfl_gemm_fwd_lora:  y = x w^T + xt wt^T      x (R,K), w (E,N,K), xt (R,KT), wt (E,N,KT)
 *   mfl_gemm_dx_lora:  dx = dy w (+ dy2 w2) + xt wt    dy, dy2 (R,K), w, w2 (E,K,N), xt (R,KT),
 *                      wt (E,KT,N); dy2 and w2 both NULL or both given (the gated unit's two terms)
 * xt is x A^T (or dy B) already multiplied by the adapter's scaling; KT is the rank, a multiple
 * of 8.  Both return MFL_ERR_UNSUPPORTED, with nothing enqueued, unless the element type is bf16,
 * N, K and KT are multiples of 8 (K % 64 == 0 with dy2), E <= 512 and the pointers are 16-byte
 * aligned; the caller then adds the thin product with a second call (accumulate = 1). */
MFL_API int mfl_gemm_fwd_lora(const void *x, const void *w, const void *xt, const void *wt, int KT,
                      const void *m_sizes, int m_sizes_dtype, void *y, int64_t R, int N, int K,
                      int E, int in_dtype, int out_dtype, void *stream);
MFL_API int mfl_gemm_dx_lora(const void *dy, const void *w, const void *dy2, const void *w2,
                     const void *xt, const void *wt, int KT, const void *m_sizes, int m_sizes_dtype,
                     void *dx, int64_t R, int N, int K, int E, int in_dtype, int out_dtype,
                     void *stream);

/* mfl_gemm_fwd_lora / mfl_gemm_dx_lora over packed NF4 base weights (arguments as in mfl_gemm_fwd_nf4 /
 * mfl_gemm_dx_nf4; the thin term's operands xt, wt are bf16): the QLoRA forms of the same two products
 * (qwen3_moe_fused/kernels/fast_lora.py:57-63,65-88,127-131 dequantise, multiply and add).  Return
 * MFL_ERR_UNSUPPORTED, with nothing enqueued, unless the element type is bf16, K % 64 == 0, N % 8 == 0
 * (dx: N % 32 == 0), KT % 8 == 0, blocksize >= 8, E <= 512 and the pointers are 16-byte aligned. */
MFL_API int mfl_gemm_fwd_nf4_lora(const void *x, const uint8_t *wq, const float *code16,
                          const float *absmax, int blocksize, const void *xt, const void *wt, int KT,
                          const void *m_sizes, int m_sizes_dtype, void *y, int64_t R, int N, int K,
                          int E, int in_dtype, int out_dtype, void *stream);
MFL_API int mfl_gemm_dx_nf4_lora(const void *dy, const uint8_t *wq, const float *code16,
                         const float *absmax, int blocksize, const void *xt, const void *wt, int KT,
                         const void *m_sizes, int m_sizes_dtype, void *dx, int64_t R, int N, int K,
                         int E, int in_dtype, int out_dtype, void *stream);

/* ---- forward products fused with their neighbours in the sparse MLP block ---------
 * The reference names these fusions as future work (modular_qwen3_moe_fused.py:100-101,105).
 * Each call returns MFL_ERR_UNSUPPORTED, with nothing enqueued, for a request the pipelined
 * kernels do not take (element type other than bf16, N or K not a multiple of 8, NF4 with
 * K % 64 != 0 or blocksize < 8, more than 512 experts, pointers not 16-byte aligned, a
 * source matrix of 4 GiB or more); the caller then runs the separate entry points. */

/* y = grouped_gemm_forward(x, w, m_sizes) with x[m, :] = x_src[row_idx[m] / idx_div, :]:
 * the rows are gathered while they are copied into the kernel's staging memory, x is never
 * written.  x_src (src_rows, K); row_idx (R,) int32 with values in [0, src_rows * idx_div).
 * Replaces modular_qwen3_moe_fused.py:95-103 followed by forward.py:116-160. */
MFL_API int mfl_gemm_fwd_gather(const void *x_src, int64_t src_rows, const int32_t *row_idx, int idx_div,
                        const void *w, const void *m_sizes, int m_sizes_dtype, void *y, int64_t R,
                        int N, int K, int E, int in_dtype, int out_dtype, void *stream);

/* The same with NF4 weights (see mfl_gemm_fwd_nf4). */
MFL_API int mfl_gemm_fwd_nf4_gather(const void *x_src, int64_t src_rows, const int32_t *row_idx,
                            int idx_div, const uint8_t *wq, const float *code16,
                            const float *absmax, int blocksize, const void *m_sizes,
                            int m_sizes_dtype, void *y, int64_t R, int N, int K, int E,
                            int in_dtype, int out_dtype, void *stream);

/* h = silu(e) * g with e = grouped_gemm_forward(x, w_gate), g = grouped_gemm_forward(x, w_up),
 * in one kernel: x is read once, e and g stay in registers.  Rounding is that of the separate
 * calls (e and g to bf16, silu in fp32 to bf16, product to bf16), so h is bit-identical to
 * mfl_gemm_fwd x 2 + mfl_silu_mul_fwd.  e_out / g_out (R,N), where not NULL, receive e and g
 * (a training step needs them for the backward pass).  row_idx may be NULL: x is then (R,K)
 * and src_rows, idx_div are ignored; otherwise rows are gathered as in mfl_gemm_fwd_gather.
 * Replaces modular_qwen3_moe_fused.py:105-108 (gate_proj, up_proj, silu_mul). */
MFL_API int mfl_glu_fwd(const void *x, int64_t src_rows, const int32_t *row_idx, int idx_div,
                const void *w_gate, const void *w_up, const void *m_sizes, int m_sizes_dtype,
                void *h, void *e_out, void *g_out, int64_t R, int N, int K, int E, int dtype,
                void *stream);

/* mfl_glu_fwd with the rank-r terms of the gate and up adapters in the two reductions:
 * h = silu(x w_gate^T + xt wt_gate^T) * (x w_up^T + xt wt_up^T), the products themselves to e_out / g_out
 * where not NULL.  xt (R,KT) holds both adapters' scaled activations side by side ([s_g x A_g^T | s_u x A_u^T],
 * KT = the two ranks together); wt_gate and wt_up (E,N,KT) hold each adapter's B over its own columns of xt
 * and zeros over the other's.  The gate and up projections of the LoRA MLP with their SiLU-mul in one launch
 * (qwen3_moe_fused/kernels/fast_lora.py:68-95).  bf16 only; MFL_ERR_UNSUPPORTED as for mfl_glu_fwd. */
MFL_API int mfl_glu_fwd_lora(const void *x, const void *w_gate, const void *w_up, const void *xt,
                     const void *wt_gate, const void *wt_up, int KT, const void *m_sizes,
                     int m_sizes_dtype, void *h, void *e_out, void *g_out, int64_t R, int N, int K,
                     int E, int dtype, void *stream);

/* The same with NF4 weights, each matrix with its own quantisation state. */
MFL_API int mfl_glu_fwd_nf4(const void *x, int64_t src_rows, const int32_t *row_idx, int idx_div,
                    const uint8_t *wq_gate, const float *code16_gate, const float *absmax_gate,
                    int blocksize_gate, const uint8_t *wq_up, const float *code16_up,
                    const float *absmax_up, int blocksize_up, const void *m_sizes,
                    int m_sizes_dtype, void *h, void *e_out, void *g_out, int64_t R, int N, int K,
                    int E, int dtype, void *stream);

/* Tile-ordered scales for decode-sized batches.  At a few rows per expert the NF4 kernels are bound by the
 * number of memory requests, and the 64 scales that a wave needs per 128-wide reduction stage lie in 32
 * different lines of absmax.  mfl_nf4_tile_absmax writes them once more, in the order of consumption:
 * out[((e * ceil(N/32) + t) * (K/128) + s) * 64 + l] = the scale of weight (e, min(32 t + l/2, N-1),
 * 128 s + 64 (l % 2)), mfl_nf4_tiled_absmax_floats floats in all (0: the shape has no such copy -- K not a
 * multiple of 128, or blocks of fewer than 64 weights; mfl_nf4_tile_absmax then returns MFL_ERR_UNSUPPORTED).
 * A caller builds the copy once per quantisation state and hands it to the two entry points below, which
 * are mfl_gemm_fwd_nf4 / mfl_gemm_fwd_nf4_gather (row_idx NULL: x_src is x, src_rows and idx_div ignored)
 * and mfl_glu_fwd_nf4 with one more argument per matrix; absmax_tiled may be NULL (then they are those
 * entry points), and results are bit-identical with and without it.  The kernels that read the copy take the
 * plain product up to 128 rows per expert on average and the gated one up to 384; beyond that it is ignored.
 * No counterpart in the reference, whose
 * 4-bit product (qwen3_moe_fused/grouped_gemm/forward_4bit.py:99-106) reads absmax in place. */
MFL_API int64_t mfl_nf4_tiled_absmax_floats(int blocksize, int N, int K, int E);
MFL_API int mfl_nf4_tile_absmax(const float *absmax, int blocksize, int N, int K, int E, float *out,
                        void *stream);
MFL_API int mfl_gemm_fwd_nf4_tiled(const void *x_src, int64_t src_rows, const int32_t *row_idx, int idx_div,
                           const uint8_t *wq, const float *code16, const float *absmax,
                           const float *absmax_tiled, int blocksize, const void *m_sizes,
                           int m_sizes_dtype, void *y, int64_t R, int N, int K, int E, int in_dtype,
                           int out_dtype, void *stream);
MFL_API int mfl_glu_fwd_nf4_tiled(const void *x, int64_t src_rows, const int32_t *row_idx, int idx_div,
                          const uint8_t *wq_gate, const float *code16_gate, const float *absmax_gate,
                          const float *absmax_tiled_gate, int blocksize_gate, const uint8_t *wq_up,
                          const float *code16_up, const float *absmax_up,
                          const float *absmax_tiled_up, int blocksize_up, const void *m_sizes,
                          int m_sizes_dtype, void *h, void *e_out, void *g_out, int64_t R, int N, int K,
                          int E, int dtype, void *stream);

/* ---- NF4 / blockwise dequantisation ----------------------------------------------- */

/* out[i] = code16[nibble(i)] * absmax[i / blocksize], i < n (n even).  Stands in for the
 * bitsandbytes dequantize_4bit calls at qwen3_moe_fused/quantize/layer.py:21 and
 * qwen3_moe_fused/kernels/fast_lora.py:62. */
MFL_API int mfl_nf4_dequant(const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                    void *out, int64_t n, int out_dtype, void *stream);

/* out[i] = code256[v[i]] * absmax2[i / blocksize2] + offset  (nested absmax),
 * qwen3_moe_fused/grouped_gemm/forward_4bit.py:149-152. */
MFL_API int mfl_dequant_blockwise_u8(const uint8_t *v, const float *code256, const float *absmax2,
                             int blocksize2, float offset, float *out, int64_t n, void *stream);

/* Blockwise NF4 quantiser: absmax[b] = max|block b|, nibble = nearest code16 entry to
 * x / absmax (ties -> lower entry).  w has n elements of w_dtype, n % blocksize == 0.
 * Stands in for bitsandbytes quantize_4bit as used at test_moe_fused_linear.py:40. */
MFL_API int mfl_nf4_quant(const void *w, int w_dtype, int64_t n, int blocksize, const float *code16,
                  uint8_t *wq, float *absmax, void *stream);

/* ---- routing ---------------------------------------------------------------------- */

/* p = softmax_fp32(logits[t, :]); top-k of p, descending, equal values -> lower expert id
 * first; if renorm, weights /= sum(weights).  weights_f32 (T,k) and/or weights_cast (T,k) of
 * cast_dtype may be NULL; idx (T,k) int64 is required.
 * Replaces qwen3_moe_fused/modular_qwen3_moe_fused.py:87-93 (= fast_lora.py:52-58). */
MFL_API int mfl_route_softmax_topk(const void *logits, int logits_dtype, int64_t T, int E, int k,
                           int renorm, float *weights_f32, void *weights_cast, int cast_dtype,
                           int64_t *idx, void *stream);

/* Gradient of mfl_route_softmax_topk's weights with respect to the logits: dlogits (T,E), in the
 * logits' type, from dweights (T,k) of dweights_dtype, the selections idx and the fp32 weights
 * that the forward call wrote; the softmax is recomputed.  E <= 1024.  It is the derivative that
 * autograd forms for qwen3_moe_fused/modular_qwen3_moe_fused.py:87-93 (softmax, topk, the
 * optional renormalisation) from separate tensor operations. */
MFL_API int mfl_route_softmax_topk_bwd(const void *logits, int logits_dtype, int64_t T, int E, int k,
                               int renorm, const int64_t *idx, const float *weights_f32,
                               const void *dweights, int dweights_dtype, void *dlogits,
                               void *stream);

/* mfl_route_softmax_topk followed by mfl_expert_sort of its T * k selections, as ONE launch
 * for decode-sized batches (the three launches of the separate calls cost more than their
 * work there).  Same outputs, bit for bit: weights_f32 / weights_cast / idx as in
 * mfl_route_softmax_topk; counts (E,), sort_idx and inv_sort_idx (T*k,) as in mfl_expert_sort
 * (both index arrays required).  Returns MFL_ERR_UNSUPPORTED, with nothing enqueued, when
 * T > 128, T * k > 8192, E > 512 or T == 0; the caller then makes the two separate calls.
 * Replaces qwen3_moe_fused/modular_qwen3_moe_fused.py:87-93 + kernels/indexing.py:48-65. */
MFL_API int mfl_route_sort_small(const void *logits, int logits_dtype, int64_t T, int E, int k, int renorm,
                         float *weights_f32, void *weights_cast, int cast_dtype, int64_t *idx,
                         int32_t *counts, int32_t *sort_idx, int32_t *inv_sort_idx, void *stream);

/* mfl_route_softmax_topk followed by mfl_expert_sort of its T * k selections, for any T: one launch
 * up to 64 tokens (mfl_route_sort_small), otherwise two (the top-k kernel leaves a histogram of
 * experts per 256 selections, which is the counting pass of the sort), three where the two-launch
 * form does not apply (E > 512, more than 1024 * 256 selections).  Same outputs as the separate
 * calls, bit for bit; both index arrays are required.  workspace: mfl_route_sort_workspace(T, E, k)
 * bytes, 256-byte aligned.
 * Replaces qwen3_moe_fused/modular_qwen3_moe_fused.py:87-93 + kernels/indexing.py:48-65. */
MFL_API size_t mfl_route_sort_workspace(int64_t T, int E, int k);
MFL_API int mfl_route_sort(const void *logits, int logits_dtype, int64_t T, int E, int k, int renorm,
                   float *weights_f32, void *weights_cast, int cast_dtype, int64_t *idx,
                   int32_t *counts, int32_t *sort_idx, int32_t *inv_sort_idx, void *workspace,
                   size_t ws_bytes, void *stream);

/* Stable counting sort of expert ids sel (R,) in [0, E):
 *   counts[e]        = #{j : sel[j] == e}
 *   sort_idx[i]      = j of the i-th row in the stable ascending order
 *   inv_sort_idx[j]  = position of row j in that order
 * sort_idx and inv_sort_idx may both be NULL (counts only).  Ids outside [0, E) are a
 * caller error (they are ignored by the counts and leave their slots unwritten).
 * workspace: mfl_expert_sort_workspace(R, E) bytes of device memory, contents ignored.
 * Replaces get_expert_counts_and_idx / get_expert_counts,
 * qwen3_moe_fused/kernels/indexing.py:18-23,48-65. */
MFL_API size_t mfl_expert_sort_workspace(int64_t R, int E);
MFL_API int mfl_expert_sort(const void *sel, int sel_dtype, int64_t R, int E, int32_t *counts,
                    int32_t *sort_idx, int32_t *inv_sort_idx, void *workspace, size_t ws_bytes,
                    void *stream);

/* mfl_expert_sort without a workspace argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  Same outputs as mfl_expert_sort, bit for bit.  The tables
 * of the sort live in a fixed array of 2 228 224 bytes of device memory that belongs to the
 * library (one copy per GPU the library runs on, held until the process ends); the call
 * allocates nothing, on the device or through any library.  Limit: E <= 512 (any R up to
 * 2^31 - 1); beyond it the call returns MFL_ERR_LIMIT with nothing enqueued.  All calls on one
 * GPU share that GPU's array: calls that may overlap in time on one GPU (different streams,
 * different threads) race and must be serialised by the caller; calls on one stream are safe.
 * The first call on a device looks up the array's address and sets the kernels' launch attributes
 * there (runtime calls that do not belong inside a stream capture): make one call per device
 * before any capture that contains this entry point. */
MFL_API int mfl_expert_sort_static(const void *sel, int sel_dtype, int64_t R, int E, int32_t *counts,
                           int32_t *sort_idx, int32_t *inv_sort_idx, void *stream);

/* dst[j, :] = src[idx[j] / idx_div, :] * (row_scale ? row_scale[idx[j]] : 1), j < R_out.
 * With idx = sort_idx and idx_div = k this is "replicate each token k times, then gather",
 * qwen3_moe_fused/modular_qwen3_moe_fused.py:95-103.  row_scale has `dtype` elements. */
MFL_API int mfl_gather_rows(const void *src, const int32_t *idx, int idx_div, const void *row_scale,
                    void *dst, int64_t R_out, int H, int dtype, void *stream);

/* The same copy written from the source's side: dst[pos[r*k+j], :] = src[r, :] * (row_scale ?
 * row_scale[r*k+j] : 1) for r < R_src, j < k, with pos a permutation of [0, R_src*k) (pos =
 * inv_sort_idx gives what mfl_gather_rows gives with idx = sort_idx, bit for bit).  Every source
 * row is read once instead of k times.  Replaces modular_qwen3_moe_fused.py:95-103 as well. */
MFL_API int mfl_scatter_rows(const void *src, const int32_t *pos, int k, const void *row_scale,
                     void *dst, int64_t R_src, int H, int dtype, void *stream);

/* dst[t, :] = sum_{j<k} src[pos[t*k+j], :] * (weights ? weights[t*k+j] : 1), fp32 accumulate.
 * With pos = inv_sort_idx this is "un-sort, then weighted sum over the k selections",
 * qwen3_moe_fused/modular_qwen3_moe_fused.py:112-115. */
MFL_API int mfl_combine_rows(const void *src, const int32_t *pos, const void *weights, void *dst,
                     int64_t T, int k, int H, int dtype, void *stream);

/* dots[t*k+j] = <a[t, :], b[pos[t*k+j], :]>  (gradient of mfl_combine_rows w.r.t. weights). */
MFL_API int mfl_rows_dot(const void *a, const void *b, const int32_t *pos, void *dots, int64_t T, int k,
                 int H, int dtype, void *stream);

/* ---- SiLU-mul --------------------------------------------------------------------- */

/* h = T(f32(e) * sigmoid(f32(e))) * g.  Replaces silu_mul_forward,
 * qwen3_moe_fused/kernels/silu_mul.py:114-125. */
MFL_API int mfl_silu_mul_fwd(const void *e, const void *g, void *h, int64_t n, int dtype, void *stream);

/* de, dg (and h when h_out != NULL) from dh, e, g.  Outputs may alias inputs element for
 * element (dh->h_out, e->de, g->dg gives the reference's in-place variant).  Replaces
 * silu_mul_backward and silu_mul_backward_inplace,
 * qwen3_moe_fused/kernels/silu_mul.py:128-159. */
MFL_API int mfl_silu_mul_bwd(const void *dh, const void *e, const void *g, void *de, void *dg, void *h_out,
                     int64_t n, int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MOE_FUSED_LINEAR_H */
