// Internal interface between the C ABI (api.hip) and the grouped-GEMM kernel files.
#pragma once
#include "common.h"

namespace mfl {

enum { MODE_FWD = 0, MODE_DX = 1, MODE_DW = 2 };

// Any shape / any float type; plain FMA.
int gemm_generic(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                 int K, int E, int in_dtype, int out_dtype, float alpha, int accumulate, hipStream_t stream);

// bf16 MFMA kernels.  Returns MFL_ERR_UNSUPPORTED when the shape is not one they take
// (the caller then falls back to gemm_generic).
int gemm_bf16_mfma(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                   int K, int E, int out_dtype, float alpha, int accumulate, hipStream_t stream);

// Pipelined bf16 MFMA kernels (direct global->LDS copies, multi-stage) for aligned shapes.
// Returns MFL_ERR_UNSUPPORTED for the rest.
int gemm_bf16_pipe(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                   int K, int E, int out_dtype, float alpha, int accumulate, hipStream_t stream);

// Forward with NF4 weights for decode-sized batches (at most 32 rows per expert on average):
// weights decoded in registers, no LDS stage.
int gemm_nf4_decode(const void *x, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                    const void *m_sizes, int ms_i64, void *y, int64_t R, int N, int K, int E, int out_dtype,
                    hipStream_t stream);

// Pipelined forward with NF4 weights decoded into LDS one step ahead of the multiply.
int gemm_nf4_pipe(const void *x, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                  const void *m_sizes, int ms_i64, void *y, int64_t R, int N, int K, int E, int out_dtype,
                  hipStream_t stream);

// bf16 MFMA forward with NF4 weights decoded in the K loop.
int gemm_nf4_mfma(const void *x, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                  const void *m_sizes, int ms_i64, void *y, int64_t R, int N, int K, int E, int out_dtype,
                  hipStream_t stream);

}  // namespace mfl
