// Internal interface between the C ABI (api.hip) and the non-GEMM kernel files.
#pragma once
#include "common.h"

namespace mfl {

int silu_mul_fwd(const void *e, const void *g, void *h, int64_t n, int dtype, hipStream_t stream);
int silu_mul_bwd(const void *dh, const void *e, const void *g, void *de, void *dg, void *h, int64_t n, int dtype,
                 hipStream_t stream);
int scatter_rows(const void *src, const int32_t *pos, int k, const void *row_scale, void *dst, int64_t R_src, int H,
                 int dtype, hipStream_t stream);
int gather_rows(const void *src, const int32_t *idx, int idx_div, const void *row_scale, void *dst, int64_t R_out,
                int H, int dtype, hipStream_t stream);
int combine_rows(const void *src, const int32_t *pos, const void *weights, void *dst, int64_t T, int k, int H,
                 int dtype, hipStream_t stream);
int rows_dot(const void *a, const void *b, const int32_t *pos, void *dots, int64_t T, int k, int H, int dtype,
             hipStream_t stream);
int nf4_dequant(const uint8_t *wq, const float *code16, const float *absmax, int blocksize, void *out, int64_t n,
                int out_dtype, hipStream_t stream);
int dequant_blockwise_u8(const uint8_t *v, const float *code256, const float *absmax2, int blocksize2, float offset,
                         float *out, int64_t n, hipStream_t stream);
int nf4_quant(const void *w, int w_dtype, int64_t n, int blocksize, const float *code16, uint8_t *wq, float *absmax,
              hipStream_t stream);

int route_softmax_topk(const void *logits, int logits_dtype, int64_t T, int E, int k, int renorm, float *w_f32,
                       void *w_cast, int cast_dtype, int64_t *idx, hipStream_t stream);
// d logits of the routing weights (recomputes the softmax; idx and w_f32 as route_softmax_topk wrote them)
int route_softmax_topk_bwd(const void *logits, int logits_dtype, int64_t T, int E, int k, int renorm, const int64_t *idx,
                           const float *w_f32, const void *dw, int dw_dtype, void *dlogits, hipStream_t stream);
int route_sort_small(const void *logits, int logits_dtype, int64_t T, int E, int k, int renorm, float *w_f32,
                     void *w_cast, int cast_dtype, int64_t *idx, int32_t *counts, int32_t *sort_idx,
                     int32_t *inv_sort_idx, hipStream_t stream);
size_t route_sort_workspace(int64_t T, int E, int k);
int route_sort(const void *logits, int logits_dtype, int64_t T, int E, int k, int renorm, float *w_f32, void *w_cast,
               int cast_dtype, int64_t *idx, int32_t *counts, int32_t *sort_idx, int32_t *inv_sort_idx,
               void *workspace, size_t ws_bytes, hipStream_t stream);
size_t expert_sort_workspace(int64_t R, int E);
int expert_sort(const void *sel, int is_i64, int64_t R, int E, int32_t *counts, int32_t *sort_idx,
                int32_t *inv_sort_idx, void *workspace, size_t ws_bytes, hipStream_t stream);
int expert_sort_static(const void *sel, int is_i64, int64_t R, int E, int32_t *counts, int32_t *sort_idx,
                       int32_t *inv_sort_idx, hipStream_t stream);

}  // namespace mfl
