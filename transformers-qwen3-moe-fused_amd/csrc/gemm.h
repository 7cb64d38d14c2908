// Internal interface between the C ABI (api.hip) and the grouped-GEMM kernel files.
#pragma once
#include "common.h"

namespace mfl {

enum { MODE_FWD = 0, MODE_DX = 1, MODE_DW = 2 };

// Average rows per expert up to which the row-grouped bf16 products run on flat 64 x 128 tiles (the weights are all
// the traffic there; measured cross-over against the 320 x 192 tiles between 48 and 64 rows per expert), and up to
// which the packed-weight forward runs on the streaming / register-decoding kernels instead of the pipelined one
// (gate_proj shape, 128 experts, uniform routing: 68 / 65 / 80 us streaming against 105 / 98 / 95 us pipelined at
// 40 / 48 / 64 rows per expert, 104 against 95 us at 80).
#if defined(MFL_TUNING_BUILD) && defined(MFL_X_FLAT_ROWS)
constexpr int kFlatTileRowsPerExpert = MFL_X_FLAT_ROWS;
#else
constexpr int kFlatTileRowsPerExpert = 48;
#endif
#if defined(MFL_TUNING_BUILD) && defined(MFL_X_NF4_ROWS)
constexpr int kNf4DecodeRowsPerExpert = MFL_X_NF4_ROWS;
#else
constexpr int kNf4DecodeRowsPerExpert = 72;
#endif
// The packed-weight forward stays on the streaming kernel up to this many rows per expert on average (plain / gated
// product); from kNf4StreamTwoBlockRows on its workgroups take 64 rows of an expert.  Gate_proj shape, 128 experts,
// uniform routing, streaming (64-row tiles, two stages) against what ran before (32-row tiles to 72 rows per expert,
// the pipelined kernel beyond): plain 35 / 42 / 44 / 56 / 68 / 77 / 79 / 88 / 100 us against 42 / 51 / 58 / 63 / 73 /
// 103 / 96 / 99 / 103 at 24 / 32 / 40 / 48 / 64 / 80 / 96 / 112 / 128 rows per expert, 115 against 110 at 160;
// gated 68 / 80 / 84 / 118 / 144 / 196 / 257 / 323 against 76 / 94 / 109 / 142 / 227 / 252 / 268 / 334 at
// 24 / 32 / 40 / 64 / 96 / 128 / 192 / 256, 394 / 465 / 598 against 455 / 476 / 527 at 320 / 384 / 512.
constexpr int kNf4StreamRowsPerExpert = 128;
constexpr int kNf4StreamGatedRowsPerExpert = 384;
constexpr int kNf4StreamTwoBlockRows = 20;

// Any shape / any float type; plain FMA.
int gemm_generic(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                 int K, int E, int in_dtype, int out_dtype, float alpha, int accumulate, hipStream_t stream);

// bf16 MFMA kernels.  Returns MFL_ERR_UNSUPPORTED when the shape is not one they take
// (the caller then falls back to gemm_generic).
int gemm_bf16_mfma(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                   int K, int E, int out_dtype, float alpha, int accumulate, hipStream_t stream);

// What a forward product can take over from its neighbours in the sparse MLP block.
struct GemmFusion {
    // gather: row i of the left operand is row row_idx[i] / idx_div of a (src_rows, K) matrix
    const int32_t *row_idx;
    int idx_div;
    int64_t src_rows;
    // gated linear unit: w2 is a second weight matrix of the same shape (the up projection, w being
    // the gate projection); the output is silu(x w^T) * (x w2^T); e_out / g_out, where not null,
    // receive the two products.  With NF4 weights w2 comes with its own quantisation state.
    const void *w2;
    const float *code16_2, *absmax_2;
    int blocksize_2;
    void *e_out, *g_out;
    // input gradient with two terms (DX only): dx = dy w + x2 w2, x2 and w2 shaped like dy and w
    const void *x2;
    // a last term with a reduction length of its own (FWD, DX; bf16 weights): c += xt wt with xt (R, kt) and
    // wt (E, N, kt) in FWD, (E, kt, N) in DX; kt a multiple of 8.  The rank-r term of a LoRA adapter.
    const void *xt, *wt;
    int kt;
    // the same with the gated unit (w2 given, x2 not): thin weights of the second matrix; xt is shared
    const void *wt2;
    // NF4: tile-ordered copies of the scales of w and w2 (see Nf4Matrix), or null
    const float *absmax_tiled, *absmax_tiled_2;
    // DX with the backward of the gated unit in its epilogue (bw_e given): the product dh = dy w is not stored;
    // de, dg (and h = silu(e) g where bw_h is given) are computed from it and the forward products e, g (all
    // (R, N) bf16; de may be e and dg may be g) as silu_mul_bwd computes them from a stored dh
    const void *bw_e, *bw_g;
    void *bw_de, *bw_dg, *bw_h;
};

// Pipelined bf16 MFMA kernels (direct global->LDS copies, multi-stage) for aligned shapes.
// Returns MFL_ERR_UNSUPPORTED for the rest.
int gemm_bf16_pipe(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                   int K, int E, int out_dtype, float alpha, int accumulate, hipStream_t stream,
                   const GemmFusion *fusion = nullptr);

// Four-wave kernels with 128 x 128 wave tiles (bf16 in and out, no accumulation, whole tiles along the weight
// dimensions).  Returns MFL_ERR_UNSUPPORTED for the rest.
// a2, b2 (DX only, shaped like a, b): a second term in the same reduction, c = a b + a2 b2.  at, bt, kthin (FWD,
// DX): a last term with a reduction length of its own, as GemmFusion::xt, wt, kt.
int gemm_bf16_wide(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                   int K, int E, int out_dtype, float alpha, int accumulate, hipStream_t stream,
                   const void *a2 = nullptr, const void *b2 = nullptr, const void *at = nullptr,
                   const void *bt = nullptr, int kthin = 0);

// The weight-gradient product with one thin side (N or K equal to 8, 16, 32 or 64, the other a multiple of 256; bf16 in,
// bf16 or fp32 out): steps of 32 rows dealt out evenly over the workgroups, experts cut by a border finished by
// a second kernel from fp32 partial sums in the workspace.  Takes (a = dy, b = x) like the other kernels.
// gemm_dw_split_workspace returns 0 for a shape the kernel does not take (gemm_dw_split then returns
// MFL_ERR_UNSUPPORTED).
size_t gemm_dw_split_workspace(int64_t R, int N, int K, int E);
int gemm_dw_split(const void *dy, const void *x, const void *m_sizes, int ms_i64, void *dw, int64_t R, int N, int K,
                  int E, int out_dtype, float alpha, void *workspace, size_t ws_bytes, hipStream_t stream);

// One packed NF4 weight matrix with its quantisation state.
struct Nf4Matrix {
    const uint8_t *wq;
    const float *code16;
    const float *absmax;
    int bs_shift;  // log2 of the quantisation block size
    // The scales once more in the order in which the streaming kernel's waves consume them (nf4_tile_absmax),
    // or null: [expert][32-column tile][128-wide reduction stage][column of the tile][half of the stage].
    const float *absmax_tiled = nullptr;
};

// Writes the tile-ordered copy of an (E, N, K) matrix's scales: E * ceil(N / 32) * (K / 128) * 64 floats
// (nf4_tiled_absmax_floats; 0 for a shape without such a copy: K % 128 != 0 or blocks under 64 weights).
int64_t nf4_tiled_absmax_floats(int blocksize, int N, int K, int E);
int nf4_tile_absmax(const float *absmax, int blocksize, int N, int K, int E, float *out, hipStream_t stream);

// The streaming form of gemm_nf4_decode (all operands copied straight to LDS, scale applied per block to the
// partial sums): K % 128 == 0 and blocks of at least 64 weights, MFL_ERR_UNSUPPORTED otherwise.
int gemm_nf4_stream(const bf16_t *x, const int32_t *row_idx, int idx_div, const Nf4Matrix &w0, const Nf4Matrix &w1,
                    bool glu, const void *m_sizes, int ms_i64, void *y, void *e_out, void *g_out, int64_t R, int N,
                    int K, int E, int out_dtype, hipStream_t stream);

// The matrix-vector form of gemm_nf4_decode for at most two rows per expert on average (R <= 2 E): lanes along
// the reduction, rows in registers, no MFMA.  K <= 2048, K a multiple of the quantisation block size;
// MFL_ERR_UNSUPPORTED otherwise.
int gemm_nf4_gemv(const bf16_t *x, const int32_t *row_idx, int idx_div, const Nf4Matrix &w0, const Nf4Matrix &w1,
                  bool glu, const void *m_sizes, int ms_i64, void *y, void *e_out, void *g_out, int64_t R, int N,
                  int K, int E, int out_dtype, hipStream_t stream);

// Forward with NF4 weights for decode-sized batches (at most 32 rows per expert on average):
// weights decoded in registers, no LDS stage.
int gemm_nf4_decode(const void *x, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                    const void *m_sizes, int ms_i64, void *y, int64_t R, int N, int K, int E, int out_dtype,
                    hipStream_t stream, const GemmFusion *fusion = nullptr);

// Pipelined forward with NF4 weights decoded into LDS one step ahead of the multiply.
int gemm_nf4_pipe(const void *x, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                  const void *m_sizes, int ms_i64, void *y, int64_t R, int N, int K, int E, int out_dtype,
                  hipStream_t stream, const GemmFusion *fusion = nullptr);

// Input-gradient product dx = dy w with NF4 weights (w (E, K, N) packed, K the reduction), decoded
// into LDS like the forward.  Needs K % 64 == 0, N % 32 == 0.
int gemm_nf4_pipe_dx(const void *dy, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                     const void *m_sizes, int ms_i64, void *dx, int64_t R, int N, int K, int E, int out_dtype,
                     float alpha, int accumulate, hipStream_t stream, const GemmFusion *fusion = nullptr);

// bf16 MFMA forward with NF4 weights decoded in the K loop.
int gemm_nf4_mfma(const void *x, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                  const void *m_sizes, int ms_i64, void *y, int64_t R, int N, int K, int E, int out_dtype,
                  hipStream_t stream);

}  // namespace mfl
