// extern "C" surface of the library: argument validation and dispatch only.
#include "common.h"
#include "gemm.h"
#include "ops.h"

namespace mfl {

const DeviceInfo &device_info() {
    static const DeviceInfo info = [] {
        DeviceInfo d;
        d.cu_count = 256;
        d.xcd_count = 8;
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
            d.cu_count = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        return d;
    }();
    return info;
}

namespace {

int check_gemm(const void *a, const void *b, const void *m_sizes, int ms_dtype, const void *c, int64_t R, int N, int K,
               int E, int in_dtype, int out_dtype) {
    if (R < 0 || N <= 0 || K <= 0 || E <= 0) return MFL_ERR_SHAPE;
    if (R > 0x7fffffff) return MFL_ERR_SHAPE;
    if (!dtype_ok(in_dtype) || !dtype_ok(out_dtype) || !itype_ok(ms_dtype)) return MFL_ERR_DTYPE;
    if (!m_sizes) return MFL_ERR_NULL;
    if (R > 0 && (!a || !b || !c)) return MFL_ERR_NULL;
    if (!aligned(a, dtype_size(in_dtype)) || !aligned(b, dtype_size(in_dtype)) || !aligned(c, dtype_size(out_dtype)) ||
        !aligned(m_sizes, ms_dtype == MFL_I64 ? 8 : 4))
        return MFL_ERR_ALIGN;
    return MFL_OK;
}

int run_gemm(int mode, const void *a, const void *b, const void *m_sizes, int ms_dtype, void *c, int64_t R, int N, int K,
             int E, int in_dtype, int out_dtype, float alpha, int accumulate, void *stream) {
    int rc = check_gemm(a, b, m_sizes, ms_dtype, c, R, N, K, E, in_dtype, out_dtype);
    if (rc) return rc;
    if (R == 0 && mode != MODE_DW) return MFL_OK;
    if (mode == MODE_DW && !c) return MFL_ERR_NULL;  // dW is written (zeros) even without rows
    hipStream_t s = (hipStream_t)stream;
    const int ms_i64 = ms_dtype == MFL_I64;
    if (in_dtype == MFL_BF16) {
        // weight gradient from about 64 rows per expert on: the four-wave kernel (85.6 against 99.5 us at 64 rows per
        // expert, 156 against 170 us at 256, N = 2048, K = 768, E = 128; below that the eight-wave tiles are ahead)
        // and for the row-grouped products from where the flat tiles end (same box, one after the other, us: gate_proj
        // forward 135.9 against 138.5, down_proj input gradient 135.3 against 138.8, down_proj forward 146.5 against
        // 152.2, skewed routing at 65536 rows 264 against 286 forward and 286 against 302 input gradient; at 48 to 64
        // rows per expert forward 95-97 against 97-99, input gradient with N = 2048, K = 768 91-97 against 102-108)
        // (an output of at most 64 columns stays on the eight-wave kernel's thin tiles: 48 against 99 us for the rank-16
        // product x A^T at 65536 rows)
        const bool wide_rows = mode != MODE_DW && R >= (int64_t)kFlatTileRowsPerExpert * E && N > 64;
        if ((mode == MODE_DW && R >= (int64_t)64 * E) || wide_rows) {
            rc = gemm_bf16_wide(mode, a, b, m_sizes, ms_i64, c, R, N, K, E, out_dtype, alpha, accumulate, s);
            if (rc != MFL_ERR_UNSUPPORTED) return rc;
        }
        rc = gemm_bf16_pipe(mode, a, b, m_sizes, ms_i64, c, R, N, K, E, out_dtype, alpha, accumulate, s);
        if (rc != MFL_ERR_UNSUPPORTED) return rc;
        rc = gemm_bf16_mfma(mode, a, b, m_sizes, ms_i64, c, R, N, K, E, out_dtype, alpha, accumulate, s);
        if (rc != MFL_ERR_UNSUPPORTED) return rc;
    }
    return gemm_generic(mode, a, b, m_sizes, ms_i64, c, R, N, K, E, in_dtype, out_dtype, alpha, accumulate, s);
}

}  // namespace
}  // namespace mfl

using namespace mfl;

extern "C" {

int mfl_abi_version(void) { return MFL_ABI_VERSION; }

const char *mfl_strerror(int code) {
    switch (code) {
        case MFL_OK:
            return "ok";
        case MFL_ERR_NULL:
            return "required pointer is NULL";
        case MFL_ERR_SHAPE:
            return "invalid or inconsistent dimension";
        case MFL_ERR_DTYPE:
            return "unknown or unsupported element/index type";
        case MFL_ERR_ALIGN:
            return "pointer not aligned to its element size";
        case MFL_ERR_WORKSPACE:
            return "workspace missing or too small";
        case MFL_ERR_UNSUPPORTED:
            return "request not supported by this build";
        case MFL_ERR_LIMIT:
            return "size beyond the fixed maximum of this entry point";
        default:
            return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error code";
    }
}

int mfl_gemm_fwd(const void *x, const void *w, const void *m_sizes, int m_sizes_dtype, void *y, int64_t R, int N, int K,
                 int E, int in_dtype, int out_dtype, float alpha, int accumulate, void *stream) {
    return run_gemm(MODE_FWD, x, w, m_sizes, m_sizes_dtype, y, R, N, K, E, in_dtype, out_dtype, alpha, accumulate,
                    stream);
}

int mfl_gemm_dx(const void *dy, const void *w, const void *m_sizes, int m_sizes_dtype, void *dx, int64_t R, int N, int K,
                int E, int in_dtype, int out_dtype, float alpha, int accumulate, void *stream) {
    return run_gemm(MODE_DX, dy, w, m_sizes, m_sizes_dtype, dx, R, N, K, E, in_dtype, out_dtype, alpha, accumulate,
                    stream);
}

int mfl_gemm_dw(const void *x, const void *dy, const void *m_sizes, int m_sizes_dtype, void *dw, int64_t R, int N, int K,
                int E, int in_dtype, int out_dtype, float alpha, int accumulate, void *stream) {
    if (R > 0 && !x) return MFL_ERR_NULL;
    // kernels take (a = dy, b = x)
    return run_gemm(MODE_DW, dy, x, m_sizes, m_sizes_dtype, dw, R, N, K, E, in_dtype, out_dtype, alpha, accumulate,
                    stream);
}

size_t mfl_gemm_dw_split_workspace(int64_t R, int N, int K, int E) { return gemm_dw_split_workspace(R, N, K, E); }

int mfl_gemm_dw_split(const void *x, const void *dy, const void *m_sizes, int m_sizes_dtype, void *dw, int64_t R, int N,
                      int K, int E, int in_dtype, int out_dtype, float alpha, void *workspace, size_t ws_bytes,
                      void *stream) {
    int rc = check_gemm(dy, x, m_sizes, m_sizes_dtype, dw, R, N, K, E, in_dtype, out_dtype);
    if (rc) return rc;
    if (!dw || (R > 0 && !x)) return MFL_ERR_NULL;
    if (in_dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
    return gemm_dw_split(dy, x, m_sizes, m_sizes_dtype == MFL_I64, dw, R, N, K, E, out_dtype, alpha, workspace, ws_bytes,
                         (hipStream_t)stream);
}

// The NF4 forward product, with or without gathered rows (row_idx null: x is (R, K)) and with or without the
// tile-ordered copy of the scales.
static int fwd_nf4(const void *x, int64_t src_rows, const int32_t *row_idx, int idx_div, const uint8_t *wq,
                   const float *code16, const float *absmax, const float *absmax_tiled, int blocksize,
                   const void *m_sizes, int m_sizes_dtype, void *y, int64_t R, int N, int K, int E, int in_dtype,
                   int out_dtype, void *stream) {
    if (R < 0 || N <= 0 || K <= 0 || E <= 0 || R > 0x7fffffff) return MFL_ERR_SHAPE;
    if (blocksize < 2 || (blocksize & (blocksize - 1)) != 0) return MFL_ERR_SHAPE;
    if (K % 2 != 0 || ((int64_t)E * N * K) % blocksize != 0) return MFL_ERR_SHAPE;
    if (!dtype_ok(in_dtype) || !dtype_ok(out_dtype) || !itype_ok(m_sizes_dtype)) return MFL_ERR_DTYPE;
    if (!wq || !code16 || !absmax || !m_sizes || (R > 0 && (!x || !y))) return MFL_ERR_NULL;
    if (R == 0) return MFL_OK;
    if (in_dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
    if (absmax_tiled != nullptr && nf4_tiled_absmax_floats(blocksize, N, K, E) == 0) absmax_tiled = nullptr;
    const int ms_i64 = m_sizes_dtype == MFL_I64;
    GemmFusion fu = {row_idx, idx_div, src_rows, nullptr, nullptr, nullptr, 0, nullptr, nullptr};
    fu.absmax_tiled = absmax_tiled;
    const GemmFusion *pf = (row_idx != nullptr || absmax_tiled != nullptr) ? &fu : nullptr;
    int rc = gemm_nf4_decode(x, wq, code16, absmax, blocksize, m_sizes, ms_i64, y, R, N, K, E, out_dtype,
                             (hipStream_t)stream, pf);
    if (rc != MFL_ERR_UNSUPPORTED) return rc;
    pf = row_idx != nullptr ? &fu : nullptr;
    rc = gemm_nf4_pipe(x, wq, code16, absmax, blocksize, m_sizes, ms_i64, y, R, N, K, E, out_dtype,
                       (hipStream_t)stream, pf);
    if (rc != MFL_ERR_UNSUPPORTED || row_idx != nullptr) return rc;
    return gemm_nf4_mfma(x, wq, code16, absmax, blocksize, m_sizes, ms_i64, y, R, N, K, E, out_dtype,
                         (hipStream_t)stream);
}

int mfl_gemm_fwd_nf4(const void *x, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                     const void *m_sizes, int m_sizes_dtype, void *y, int64_t R, int N, int K, int E, int in_dtype,
                     int out_dtype, void *stream) {
    return fwd_nf4(x, 0, nullptr, 1, wq, code16, absmax, nullptr, blocksize, m_sizes, m_sizes_dtype, y, R, N, K, E,
                   in_dtype, out_dtype, stream);
}

int64_t mfl_nf4_tiled_absmax_floats(int blocksize, int N, int K, int E) {
    return nf4_tiled_absmax_floats(blocksize, N, K, E);
}

int mfl_nf4_tile_absmax(const float *absmax, int blocksize, int N, int K, int E, float *out, void *stream) {
    if (N <= 0 || K <= 0 || E <= 0 || blocksize < 2 || (blocksize & (blocksize - 1)) != 0) return MFL_ERR_SHAPE;
    if (((int64_t)E * N * K) % blocksize != 0) return MFL_ERR_SHAPE;
    if (!absmax || !out) return MFL_ERR_NULL;
    if (!aligned(absmax, 4) || !aligned(out, 4)) return MFL_ERR_ALIGN;
    return nf4_tile_absmax(absmax, blocksize, N, K, E, out, (hipStream_t)stream);
}

namespace {
int check_fused(int64_t src_rows, const int32_t *row_idx, int idx_div, const void *m_sizes, int ms_dtype, int64_t R,
                int N, int K, int E, int in_dtype, int out_dtype);
}

int mfl_gemm_fwd_nf4_tiled(const void *x_src, int64_t src_rows, const int32_t *row_idx, int idx_div, const uint8_t *wq,
                           const float *code16, const float *absmax, const float *absmax_tiled, int blocksize,
                           const void *m_sizes, int m_sizes_dtype, void *y, int64_t R, int N, int K, int E,
                           int in_dtype, int out_dtype, void *stream) {
    if (row_idx != nullptr) {
        const int rc = check_fused(src_rows, row_idx, idx_div, m_sizes, m_sizes_dtype, R, N, K, E, in_dtype, out_dtype);
        if (rc) return rc;
    }
    return fwd_nf4(x_src, src_rows, row_idx, idx_div, wq, code16, absmax, absmax_tiled, blocksize, m_sizes,
                   m_sizes_dtype, y, R, N, K, E, in_dtype, out_dtype, stream);
}

int mfl_gemm_dx_nf4(const void *dy, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                    const void *m_sizes, int m_sizes_dtype, void *dx, int64_t R, int N, int K, int E, int in_dtype,
                    int out_dtype, float alpha, int accumulate, void *stream) {
    if (R < 0 || N <= 0 || K <= 0 || E <= 0 || R > 0x7fffffff) return MFL_ERR_SHAPE;
    if (blocksize < 2 || (blocksize & (blocksize - 1)) != 0) return MFL_ERR_SHAPE;
    if (N % 2 != 0 || ((int64_t)E * N * K) % blocksize != 0) return MFL_ERR_SHAPE;
    if (!dtype_ok(in_dtype) || !dtype_ok(out_dtype) || !itype_ok(m_sizes_dtype)) return MFL_ERR_DTYPE;
    if (!wq || !code16 || !absmax || !m_sizes || (R > 0 && (!dy || !dx))) return MFL_ERR_NULL;
    if (R == 0) return MFL_OK;
    if (in_dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
    return gemm_nf4_pipe_dx(dy, wq, code16, absmax, blocksize, m_sizes, m_sizes_dtype == MFL_I64, dx, R, N, K, E,
                            out_dtype, alpha, accumulate, (hipStream_t)stream);
}

int mfl_gemm_dx_dual(const void *dy1, const void *w1, const void *dy2, const void *w2, const void *m_sizes,
                     int m_sizes_dtype, void *dx, int64_t R, int N, int K, int E, int in_dtype, int out_dtype,
                     void *stream) {
    int rc = check_gemm(dy1, w1, m_sizes, m_sizes_dtype, dx, R, N, K, E, in_dtype, out_dtype);
    if (rc) return rc;
    if (R > 0 && (!dy2 || !w2)) return MFL_ERR_NULL;
    if (R == 0) return MFL_OK;
    if (in_dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
    if (R >= (int64_t)kFlatTileRowsPerExpert * E && N > 64) {
        // the four-wave kernel, as for the one-term product (253 against 268 us at 256 rows per expert, N = 2048,
        // K = 768 per term)
        rc = gemm_bf16_wide(MODE_DX, dy1, w1, m_sizes, m_sizes_dtype == MFL_I64, dx, R, N, K, E, out_dtype, 1.0f, 0,
                            (hipStream_t)stream, dy2, w2);
        if (rc != MFL_ERR_UNSUPPORTED) return rc;
    }
    const GemmFusion fu = {nullptr, 1, 0, w2, nullptr, nullptr, 0, nullptr, nullptr, dy2};
    return gemm_bf16_pipe(MODE_DX, dy1, w1, m_sizes, m_sizes_dtype == MFL_I64, dx, R, N, K, E, out_dtype, 1.0f, 0,
                          (hipStream_t)stream, &fu);
}

int mfl_gemm_dx_silu_bwd(const void *dy, const void *w, const void *e, const void *g, const void *m_sizes,
                         int m_sizes_dtype, void *de, void *dg, void *h, int64_t R, int N, int K, int E, int dtype,
                         void *stream) {
    int rc = check_gemm(dy, w, m_sizes, m_sizes_dtype, de, R, N, K, E, dtype, dtype);
    if (rc) return rc;
    if (R > 0 && (!e || !g || !dg)) return MFL_ERR_NULL;
    if (R == 0) return MFL_OK;
    if (dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
    GemmFusion fu = {nullptr, 1, 0, nullptr, nullptr, nullptr, 0, nullptr, nullptr, nullptr};
    fu.bw_e = e;
    fu.bw_g = g;
    fu.bw_de = de;
    fu.bw_dg = dg;
    fu.bw_h = h;
    return gemm_bf16_pipe(MODE_DX, dy, w, m_sizes, m_sizes_dtype == MFL_I64, nullptr, R, N, K, E, MFL_BF16, 1.0f, 0,
                          (hipStream_t)stream, &fu);
}

int mfl_gemm_fwd_lora(const void *x, const void *w, const void *xt, const void *wt, int KT, const void *m_sizes,
                      int m_sizes_dtype, void *y, int64_t R, int N, int K, int E, int in_dtype, int out_dtype,
                      void *stream) {
    int rc = check_gemm(x, w, m_sizes, m_sizes_dtype, y, R, N, K, E, in_dtype, out_dtype);
    if (rc) return rc;
    if (KT <= 0) return MFL_ERR_SHAPE;
    if (R > 0 && (!xt || !wt)) return MFL_ERR_NULL;
    if (R == 0) return MFL_OK;
    if (in_dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
    if (R >= (int64_t)kFlatTileRowsPerExpert * E && N > 64) {  // the four-wave kernel, as for the product alone
        rc = gemm_bf16_wide(MODE_FWD, x, w, m_sizes, m_sizes_dtype == MFL_I64, y, R, N, K, E, out_dtype, 1.0f, 0,
                            (hipStream_t)stream, nullptr, nullptr, xt, wt, KT);
        if (rc != MFL_ERR_UNSUPPORTED) return rc;
    }
    GemmFusion fu = {nullptr, 1, 0, nullptr, nullptr, nullptr, 0, nullptr, nullptr, nullptr};
    fu.xt = xt, fu.wt = wt, fu.kt = KT;
    return gemm_bf16_pipe(MODE_FWD, x, w, m_sizes, m_sizes_dtype == MFL_I64, y, R, N, K, E, out_dtype, 1.0f, 0,
                          (hipStream_t)stream, &fu);
}

int mfl_gemm_dx_lora(const void *dy, const void *w, const void *dy2, const void *w2, const void *xt, const void *wt,
                     int KT, const void *m_sizes, int m_sizes_dtype, void *dx, int64_t R, int N, int K, int E,
                     int in_dtype, int out_dtype, void *stream) {
    int rc = check_gemm(dy, w, m_sizes, m_sizes_dtype, dx, R, N, K, E, in_dtype, out_dtype);
    if (rc) return rc;
    if (KT <= 0) return MFL_ERR_SHAPE;
    if ((dy2 == nullptr) != (w2 == nullptr)) return MFL_ERR_NULL;
    if (R > 0 && (!xt || !wt)) return MFL_ERR_NULL;
    if (R == 0) return MFL_OK;
    if (in_dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
    if (R >= (int64_t)kFlatTileRowsPerExpert * E && N > 64) {
        rc = gemm_bf16_wide(MODE_DX, dy, w, m_sizes, m_sizes_dtype == MFL_I64, dx, R, N, K, E, out_dtype, 1.0f, 0,
                            (hipStream_t)stream, dy2, w2, xt, wt, KT);
        if (rc != MFL_ERR_UNSUPPORTED) return rc;
    }
    GemmFusion fu = {nullptr, 1, 0, w2, nullptr, nullptr, 0, nullptr, nullptr, dy2};
    fu.xt = xt, fu.wt = wt, fu.kt = KT;
    return gemm_bf16_pipe(MODE_DX, dy, w, m_sizes, m_sizes_dtype == MFL_I64, dx, R, N, K, E, out_dtype, 1.0f, 0,
                          (hipStream_t)stream, &fu);
}

namespace {

int check_nf4_lora(const void *a, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                   const void *xt, const void *wt, int KT, const void *m_sizes, int ms_dtype, const void *c, int64_t R,
                   int N, int K, int E, int in_dtype, int out_dtype) {
    if (R < 0 || N <= 0 || K <= 0 || E <= 0 || KT <= 0 || R > 0x7fffffff) return MFL_ERR_SHAPE;
    if (blocksize < 2 || (blocksize & (blocksize - 1)) != 0) return MFL_ERR_SHAPE;
    if (((int64_t)E * N * K) % blocksize != 0 || ((int64_t)E * N * K) % 2 != 0) return MFL_ERR_SHAPE;
    if (!dtype_ok(in_dtype) || !dtype_ok(out_dtype) || !itype_ok(ms_dtype)) return MFL_ERR_DTYPE;
    if (!wq || !code16 || !absmax || !m_sizes || (R > 0 && (!a || !c || !xt || !wt))) return MFL_ERR_NULL;
    return MFL_OK;
}

}  // namespace

int mfl_gemm_fwd_nf4_lora(const void *x, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                          const void *xt, const void *wt, int KT, const void *m_sizes, int m_sizes_dtype, void *y,
                          int64_t R, int N, int K, int E, int in_dtype, int out_dtype, void *stream) {
    int rc = check_nf4_lora(x, wq, code16, absmax, blocksize, xt, wt, KT, m_sizes, m_sizes_dtype, y, R, N, K, E, in_dtype,
                            out_dtype);
    if (rc) return rc;
    if (R == 0) return MFL_OK;
    if (in_dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
    GemmFusion fu = {nullptr, 1, 0, nullptr, nullptr, nullptr, 0, nullptr, nullptr, nullptr};
    fu.xt = xt, fu.wt = wt, fu.kt = KT;
    return gemm_nf4_pipe(x, wq, code16, absmax, blocksize, m_sizes, m_sizes_dtype == MFL_I64, y, R, N, K, E, out_dtype,
                         (hipStream_t)stream, &fu);
}

int mfl_gemm_dx_nf4_lora(const void *dy, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                         const void *xt, const void *wt, int KT, const void *m_sizes, int m_sizes_dtype, void *dx,
                         int64_t R, int N, int K, int E, int in_dtype, int out_dtype, void *stream) {
    int rc = check_nf4_lora(dy, wq, code16, absmax, blocksize, xt, wt, KT, m_sizes, m_sizes_dtype, dx, R, N, K, E,
                            in_dtype, out_dtype);
    if (rc) return rc;
    if (R == 0) return MFL_OK;
    if (in_dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
    GemmFusion fu = {nullptr, 1, 0, nullptr, nullptr, nullptr, 0, nullptr, nullptr, nullptr};
    fu.xt = xt, fu.wt = wt, fu.kt = KT;
    return gemm_nf4_pipe_dx(dy, wq, code16, absmax, blocksize, m_sizes, m_sizes_dtype == MFL_I64, dx, R, N, K, E,
                            out_dtype, 1.0f, 0, (hipStream_t)stream, &fu);
}

/* ---- forward products fused with their neighbours in the sparse MLP block ---- */

namespace {

int check_fused(int64_t src_rows, const int32_t *row_idx, int idx_div, const void *m_sizes, int ms_dtype, int64_t R,
                int N, int K, int E, int in_dtype, int out_dtype) {
    if (R < 0 || N <= 0 || K <= 0 || E <= 0 || R > 0x7fffffff) return MFL_ERR_SHAPE;
    if (row_idx != nullptr && (idx_div <= 0 || src_rows <= 0)) return MFL_ERR_SHAPE;
    if (!dtype_ok(in_dtype) || !dtype_ok(out_dtype) || !itype_ok(ms_dtype)) return MFL_ERR_DTYPE;
    if (!m_sizes) return MFL_ERR_NULL;
    return MFL_OK;
}

}  // namespace

int mfl_gemm_fwd_gather(const void *x_src, int64_t src_rows, const int32_t *row_idx, int idx_div, const void *w,
                        const void *m_sizes, int m_sizes_dtype, void *y, int64_t R, int N, int K, int E, int in_dtype,
                        int out_dtype, void *stream) {
    int rc = check_fused(src_rows, row_idx, idx_div, m_sizes, m_sizes_dtype, R, N, K, E, in_dtype, out_dtype);
    if (rc) return rc;
    if (R > 0 && (!x_src || !row_idx || !w || !y)) return MFL_ERR_NULL;
    if (R == 0) return MFL_OK;
    if (in_dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
    const GemmFusion fu = {row_idx, idx_div, src_rows, nullptr, nullptr, nullptr, 0, nullptr, nullptr};
    return gemm_bf16_pipe(MODE_FWD, x_src, w, m_sizes, m_sizes_dtype == MFL_I64, y, R, N, K, E, out_dtype, 1.0f, 0,
                          (hipStream_t)stream, &fu);
}

int mfl_gemm_fwd_nf4_gather(const void *x_src, int64_t src_rows, const int32_t *row_idx, int idx_div, const uint8_t *wq,
                            const float *code16, const float *absmax, int blocksize, const void *m_sizes,
                            int m_sizes_dtype, void *y, int64_t R, int N, int K, int E, int in_dtype, int out_dtype,
                            void *stream) {
    int rc = check_fused(src_rows, row_idx, idx_div, m_sizes, m_sizes_dtype, R, N, K, E, in_dtype, out_dtype);
    if (rc) return rc;
    if (blocksize < 2 || (blocksize & (blocksize - 1)) != 0) return MFL_ERR_SHAPE;
    if (K % 2 != 0 || ((int64_t)E * N * K) % blocksize != 0) return MFL_ERR_SHAPE;
    if (!wq || !code16 || !absmax || (R > 0 && (!x_src || !row_idx || !y))) return MFL_ERR_NULL;
    if (R == 0) return MFL_OK;
    if (in_dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
    const GemmFusion fu = {row_idx, idx_div, src_rows, nullptr, nullptr, nullptr, 0, nullptr, nullptr};
    const int ms_i64 = m_sizes_dtype == MFL_I64;
    rc = gemm_nf4_decode(x_src, wq, code16, absmax, blocksize, m_sizes, ms_i64, y, R, N, K, E, out_dtype,
                         (hipStream_t)stream, &fu);
    if (rc != MFL_ERR_UNSUPPORTED) return rc;
    return gemm_nf4_pipe(x_src, wq, code16, absmax, blocksize, m_sizes, ms_i64, y, R, N, K, E, out_dtype,
                         (hipStream_t)stream, &fu);
}

int mfl_glu_fwd(const void *x, int64_t src_rows, const int32_t *row_idx, int idx_div, const void *w_gate,
                const void *w_up, const void *m_sizes, int m_sizes_dtype, void *h, void *e_out, void *g_out, int64_t R,
                int N, int K, int E, int dtype, void *stream) {
    int rc = check_fused(src_rows, row_idx, idx_div, m_sizes, m_sizes_dtype, R, N, K, E, dtype, dtype);
    if (rc) return rc;
    if (R > 0 && (!x || !w_gate || !w_up || !h)) return MFL_ERR_NULL;
    if (R == 0) return MFL_OK;
    if (dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
    const GemmFusion fu = {row_idx, idx_div, src_rows, w_up, nullptr, nullptr, 0, e_out, g_out};
    return gemm_bf16_pipe(MODE_FWD, x, w_gate, m_sizes, m_sizes_dtype == MFL_I64, h, R, N, K, E, MFL_BF16, 1.0f, 0,
                          (hipStream_t)stream, &fu);
}

int mfl_glu_fwd_lora(const void *x, const void *w_gate, const void *w_up, const void *xt, const void *wt_gate,
                     const void *wt_up, int KT, const void *m_sizes, int m_sizes_dtype, void *h, void *e_out, void *g_out,
                     int64_t R, int N, int K, int E, int dtype, void *stream) {
    int rc = check_fused(0, nullptr, 1, m_sizes, m_sizes_dtype, R, N, K, E, dtype, dtype);
    if (rc) return rc;
    if (KT <= 0) return MFL_ERR_SHAPE;
    if (R > 0 && (!x || !w_gate || !w_up || !h || !xt || !wt_gate || !wt_up)) return MFL_ERR_NULL;
    if (R == 0) return MFL_OK;
    if (dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
    GemmFusion fu = {nullptr, 1, 0, w_up, nullptr, nullptr, 0, e_out, g_out, nullptr};
    fu.xt = xt, fu.wt = wt_gate, fu.kt = KT, fu.wt2 = wt_up;
    return gemm_bf16_pipe(MODE_FWD, x, w_gate, m_sizes, m_sizes_dtype == MFL_I64, h, R, N, K, E, MFL_BF16, 1.0f, 0,
                          (hipStream_t)stream, &fu);
}

int mfl_glu_fwd_nf4_tiled(const void *x, int64_t src_rows, const int32_t *row_idx, int idx_div, const uint8_t *wq_gate,
                          const float *code16_gate, const float *absmax_gate, const float *absmax_tiled_gate,
                          int blocksize_gate, const uint8_t *wq_up, const float *code16_up, const float *absmax_up,
                          const float *absmax_tiled_up, int blocksize_up, const void *m_sizes, int m_sizes_dtype,
                          void *h, void *e_out, void *g_out, int64_t R, int N, int K, int E, int dtype, void *stream) {
    int rc = check_fused(src_rows, row_idx, idx_div, m_sizes, m_sizes_dtype, R, N, K, E, dtype, dtype);
    if (rc) return rc;
    for (int bs : {blocksize_gate, blocksize_up}) {
        if (bs < 2 || (bs & (bs - 1)) != 0 || ((int64_t)E * N * K) % bs != 0) return MFL_ERR_SHAPE;
    }
    if (K % 2 != 0) return MFL_ERR_SHAPE;
    if (!wq_gate || !code16_gate || !absmax_gate || !wq_up || !code16_up || !absmax_up || (R > 0 && (!x || !h)))
        return MFL_ERR_NULL;
    if (R == 0) return MFL_OK;
    if (dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
    GemmFusion fu = {row_idx, idx_div, src_rows, wq_up, code16_up, absmax_up, blocksize_up, e_out, g_out};
    // the tile-ordered scales serve where both matrices have them
    if (absmax_tiled_gate != nullptr && absmax_tiled_up != nullptr &&
        nf4_tiled_absmax_floats(blocksize_gate, N, K, E) != 0 && nf4_tiled_absmax_floats(blocksize_up, N, K, E) != 0) {
        fu.absmax_tiled = absmax_tiled_gate;
        fu.absmax_tiled_2 = absmax_tiled_up;
    }
    const int ms_i64 = m_sizes_dtype == MFL_I64;
    rc = gemm_nf4_decode(x, wq_gate, code16_gate, absmax_gate, blocksize_gate, m_sizes, ms_i64, h, R, N, K, E, MFL_BF16,
                         (hipStream_t)stream, &fu);
    if (rc != MFL_ERR_UNSUPPORTED) return rc;
    return gemm_nf4_pipe(x, wq_gate, code16_gate, absmax_gate, blocksize_gate, m_sizes, ms_i64, h, R, N, K, E, MFL_BF16,
                         (hipStream_t)stream, &fu);
}

int mfl_glu_fwd_nf4(const void *x, int64_t src_rows, const int32_t *row_idx, int idx_div, const uint8_t *wq_gate,
                    const float *code16_gate, const float *absmax_gate, int blocksize_gate, const uint8_t *wq_up,
                    const float *code16_up, const float *absmax_up, int blocksize_up, const void *m_sizes,
                    int m_sizes_dtype, void *h, void *e_out, void *g_out, int64_t R, int N, int K, int E, int dtype,
                    void *stream) {
    return mfl_glu_fwd_nf4_tiled(x, src_rows, row_idx, idx_div, wq_gate, code16_gate, absmax_gate, nullptr,
                                 blocksize_gate, wq_up, code16_up, absmax_up, nullptr, blocksize_up, m_sizes,
                                 m_sizes_dtype, h, e_out, g_out, R, N, K, E, dtype, stream);
}

int mfl_nf4_dequant(const uint8_t *wq, const float *code16, const float *absmax, int blocksize, void *out, int64_t n,
                    int out_dtype, void *stream) {
    if (n < 0 || n % 2 != 0 || blocksize < 2 || n % blocksize != 0) return MFL_ERR_SHAPE;
    if (!dtype_ok(out_dtype)) return MFL_ERR_DTYPE;
    if (n > 0 && (!wq || !code16 || !absmax || !out)) return MFL_ERR_NULL;
    if (!aligned(out, dtype_size(out_dtype))) return MFL_ERR_ALIGN;
    return nf4_dequant(wq, code16, absmax, blocksize, out, n, out_dtype, (hipStream_t)stream);
}

int mfl_dequant_blockwise_u8(const uint8_t *v, const float *code256, const float *absmax2, int blocksize2, float offset,
                             float *out, int64_t n, void *stream) {
    if (n < 0 || blocksize2 <= 0) return MFL_ERR_SHAPE;
    if (n > 0 && (!v || !code256 || !absmax2 || !out)) return MFL_ERR_NULL;
    return dequant_blockwise_u8(v, code256, absmax2, blocksize2, offset, out, n, (hipStream_t)stream);
}

int mfl_nf4_quant(const void *w, int w_dtype, int64_t n, int blocksize, const float *code16, uint8_t *wq, float *absmax,
                  void *stream) {
    if (n < 0 || blocksize < 2 || blocksize % 2 != 0 || n % blocksize != 0) return MFL_ERR_SHAPE;
    if (!dtype_ok(w_dtype)) return MFL_ERR_DTYPE;
    if (n > 0 && (!w || !code16 || !wq || !absmax)) return MFL_ERR_NULL;
    return nf4_quant(w, w_dtype, n, blocksize, code16, wq, absmax, (hipStream_t)stream);
}

int mfl_route_softmax_topk(const void *logits, int logits_dtype, int64_t T, int E, int k, int renorm, float *weights_f32,
                           void *weights_cast, int cast_dtype, int64_t *idx, void *stream) {
    if (T < 0 || E <= 0 || k <= 0 || k > E || k > 64) return MFL_ERR_SHAPE;
    if (!dtype_ok(logits_dtype) || (weights_cast && !dtype_ok(cast_dtype))) return MFL_ERR_DTYPE;
    if (T > 0 && (!logits || !idx)) return MFL_ERR_NULL;
    return route_softmax_topk(logits, logits_dtype, T, E, k, renorm, weights_f32, weights_cast,
                              weights_cast ? cast_dtype : MFL_F32, idx, (hipStream_t)stream);
}

int mfl_route_softmax_topk_bwd(const void *logits, int logits_dtype, int64_t T, int E, int k, int renorm,
                               const int64_t *idx, const float *weights_f32, const void *dweights, int dweights_dtype,
                               void *dlogits, void *stream) {
    if (T < 0 || E <= 0 || k <= 0 || k > E || k > 64) return MFL_ERR_SHAPE;
    if (!dtype_ok(logits_dtype) || !dtype_ok(dweights_dtype)) return MFL_ERR_DTYPE;
    if (T > 0 && (!logits || !idx || !weights_f32 || !dweights || !dlogits)) return MFL_ERR_NULL;
    return route_softmax_topk_bwd(logits, logits_dtype, T, E, k, renorm, idx, weights_f32, dweights, dweights_dtype,
                                  dlogits, (hipStream_t)stream);
}

int mfl_route_sort_small(const void *logits, int logits_dtype, int64_t T, int E, int k, int renorm, float *weights_f32,
                         void *weights_cast, int cast_dtype, int64_t *idx, int32_t *counts, int32_t *sort_idx,
                         int32_t *inv_sort_idx, void *stream) {
    if (T < 0 || E <= 0 || k <= 0 || k > E || k > 64) return MFL_ERR_SHAPE;
    if (!dtype_ok(logits_dtype) || (weights_cast && !dtype_ok(cast_dtype))) return MFL_ERR_DTYPE;
    if (!counts || (T > 0 && (!logits || !idx))) return MFL_ERR_NULL;
    return route_sort_small(logits, logits_dtype, T, E, k, renorm, weights_f32, weights_cast,
                            weights_cast ? cast_dtype : MFL_F32, idx, counts, sort_idx, inv_sort_idx,
                            (hipStream_t)stream);
}

size_t mfl_route_sort_workspace(int64_t T, int E, int k) {
    if (T < 0 || E <= 0 || k <= 0) return 0;
    return route_sort_workspace(T, E, k);
}

int mfl_route_sort(const void *logits, int logits_dtype, int64_t T, int E, int k, int renorm, float *weights_f32,
                   void *weights_cast, int cast_dtype, int64_t *idx, int32_t *counts, int32_t *sort_idx,
                   int32_t *inv_sort_idx, void *workspace, size_t ws_bytes, void *stream) {
    if (T < 0 || E <= 0 || k <= 0 || k > E || k > 64 || T * k > 0x7fffffff) return MFL_ERR_SHAPE;
    if (!dtype_ok(logits_dtype) || (weights_cast && !dtype_ok(cast_dtype))) return MFL_ERR_DTYPE;
    if (!counts || (T > 0 && (!logits || !idx || !sort_idx || !inv_sort_idx))) return MFL_ERR_NULL;
    if (T == 0) return expert_sort(idx, 1, 0, E, counts, sort_idx, inv_sort_idx, workspace, ws_bytes, (hipStream_t)stream);
    return route_sort(logits, logits_dtype, T, E, k, renorm, weights_f32, weights_cast,
                      weights_cast ? cast_dtype : MFL_F32, idx, counts, sort_idx, inv_sort_idx, workspace, ws_bytes,
                      (hipStream_t)stream);
}

size_t mfl_expert_sort_workspace(int64_t R, int E) { return expert_sort_workspace(R, E); }

int mfl_expert_sort(const void *sel, int sel_dtype, int64_t R, int E, int32_t *counts, int32_t *sort_idx,
                    int32_t *inv_sort_idx, void *workspace, size_t ws_bytes, void *stream) {
    if (R < 0 || E <= 0 || R > 0x7fffffff) return MFL_ERR_SHAPE;
    if (!itype_ok(sel_dtype)) return MFL_ERR_DTYPE;
    if (!counts || (R > 0 && !sel)) return MFL_ERR_NULL;
    return expert_sort(sel, sel_dtype == MFL_I64, R, E, counts, sort_idx, inv_sort_idx, workspace, ws_bytes,
                       (hipStream_t)stream);
}

int mfl_expert_sort_static(const void *sel, int sel_dtype, int64_t R, int E, int32_t *counts, int32_t *sort_idx,
                           int32_t *inv_sort_idx, void *stream) {
    if (R < 0 || E <= 0 || R > 0x7fffffff) return MFL_ERR_SHAPE;
    if (!itype_ok(sel_dtype)) return MFL_ERR_DTYPE;
    if (!counts || (R > 0 && !sel)) return MFL_ERR_NULL;
    return expert_sort_static(sel, sel_dtype == MFL_I64, R, E, counts, sort_idx, inv_sort_idx, (hipStream_t)stream);
}

int mfl_gather_rows(const void *src, const int32_t *idx, int idx_div, const void *row_scale, void *dst, int64_t R_out,
                    int H, int dtype, void *stream) {
    if (R_out < 0 || H <= 0 || idx_div <= 0) return MFL_ERR_SHAPE;
    if (!dtype_ok(dtype)) return MFL_ERR_DTYPE;
    if (R_out > 0 && (!src || !idx || !dst)) return MFL_ERR_NULL;
    return gather_rows(src, idx, idx_div, row_scale, dst, R_out, H, dtype, (hipStream_t)stream);
}

int mfl_scatter_rows(const void *src, const int32_t *pos, int k, const void *row_scale, void *dst, int64_t R_src, int H,
                     int dtype, void *stream) {
    if (R_src < 0 || H <= 0 || k <= 0 || R_src * k > 0x7fffffff) return MFL_ERR_SHAPE;
    if (!dtype_ok(dtype)) return MFL_ERR_DTYPE;
    if (R_src > 0 && (!src || !pos || !dst)) return MFL_ERR_NULL;
    return scatter_rows(src, pos, k, row_scale, dst, R_src, H, dtype, (hipStream_t)stream);
}

int mfl_combine_rows(const void *src, const int32_t *pos, const void *weights, void *dst, int64_t T, int k, int H,
                     int dtype, void *stream) {
    if (T < 0 || H <= 0 || k <= 0) return MFL_ERR_SHAPE;
    if (!dtype_ok(dtype)) return MFL_ERR_DTYPE;
    if (T > 0 && (!src || !pos || !dst)) return MFL_ERR_NULL;
    return combine_rows(src, pos, weights, dst, T, k, H, dtype, (hipStream_t)stream);
}

int mfl_rows_dot(const void *a, const void *b, const int32_t *pos, void *dots, int64_t T, int k, int H, int dtype,
                 void *stream) {
    if (T < 0 || H <= 0 || k <= 0) return MFL_ERR_SHAPE;
    if (!dtype_ok(dtype)) return MFL_ERR_DTYPE;
    if (T > 0 && (!a || !b || !pos || !dots)) return MFL_ERR_NULL;
    return rows_dot(a, b, pos, dots, T, k, H, dtype, (hipStream_t)stream);
}

int mfl_silu_mul_fwd(const void *e, const void *g, void *h, int64_t n, int dtype, void *stream) {
    if (n < 0) return MFL_ERR_SHAPE;
    if (!dtype_ok(dtype)) return MFL_ERR_DTYPE;
    if (n > 0 && (!e || !g || !h)) return MFL_ERR_NULL;
    return silu_mul_fwd(e, g, h, n, dtype, (hipStream_t)stream);
}

int mfl_silu_mul_bwd(const void *dh, const void *e, const void *g, void *de, void *dg, void *h_out, int64_t n, int dtype,
                     void *stream) {
    if (n < 0) return MFL_ERR_SHAPE;
    if (!dtype_ok(dtype)) return MFL_ERR_DTYPE;
    if (n > 0 && (!dh || !e || !g || !de || !dg)) return MFL_ERR_NULL;
    return silu_mul_bwd(dh, e, g, de, dg, h_out, n, dtype, (hipStream_t)stream);
}

}  // extern "C"
