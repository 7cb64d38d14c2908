// Shape- and type-generic grouped GEMM (plain FMA, fp32 accumulate).
//
// This is the path for fp32 / fp16 inputs and for bf16 shapes the MFMA kernels do not
// take (dimensions that are not multiples of 8, tiny experts): every dimension is
// masked, nothing is assumed about alignment beyond the element size.
//
//   MODE_FWD : c[m, n]    = sum_k a[m, k] * b[e(m), n, k]     a = x (R,K),  b = w (E,N,K)
//   MODE_DX  : c[m, n]    = sum_k a[m, k] * b[e(m), k, n]     a = dy (R,K), b = w (E,K,N)
//   MODE_DW  : c[e, n, k] = sum_{m in e} a[m, n] * b[m, k]    a = dy (R,N), b = x (R,K)
#include "common.h"
#include "gemm.h"

namespace mfl {

namespace {

constexpr int GT = 64;   // output tile edge
constexpr int GK = 16;   // reduction step
constexpr int GPAD = 4;  // LDS row padding (floats)

// Loads a GT x GK operand tile into lds[k][i].
//   red_contig  : element (i, r) lives at base[i * ld + r]
//   !red_contig : element (i, r) lives at base[r * ld + i]
template <typename TI, bool RED_CONTIG>
__device__ __forceinline__ void load_tile(float (*lds)[GT + GPAD], const TI *base, int64_t ld, int i0,
                                          int i_end, int r0, int r_end, int tid) {
    if (RED_CONTIG) {
        const int i = tid >> 2, rq = (tid & 3) * 4;
        const bool iok = (i0 + i) < i_end;
        const TI *p = base + (int64_t)(i0 + i) * ld + r0 + rq;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            float v = 0.f;
            if (iok && (r0 + rq + u) < r_end) v = to_f32(p[u]);
            lds[rq + u][i] = v;
        }
    } else {
        const int r = tid >> 4, iq = (tid & 15) * 4;
        const bool rok = (r0 + r) < r_end;
        const TI *p = base + (int64_t)(r0 + r) * ld + i0 + iq;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            float v = 0.f;
            if (rok && (i0 + iq + u) < i_end) v = to_f32(p[u]);
            lds[r][iq + u] = v;
        }
    }
}

template <typename TI, typename TO, int MODE>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TI *__restrict__ a, const TI *__restrict__ b,
                                                           const void *__restrict__ m_sizes, int ms_i64,
                                                           TO *c, int64_t R, int N, int K, int E, float alpha,
                                                           int accumulate) {
    __shared__ float As[GK][GT + GPAD];
    __shared__ float Bs[GK][GT + GPAD];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;

    // Output tile [i0, i_end) x [j0, j_end), reduction range [r_begin, r_end).
    int i0, i_end, j0, j_end, r_begin, r_end;
    const TI *a_base;
    const TI *b_base;
    int64_t lda, ldb, ldc;
    TO *c_base;

    if (MODE == MODE_DW) {
        const int e = blockIdx.z;
        int m_start = 0;
        for (int q = 0; q < e; ++q) m_start += load_msize(m_sizes, ms_i64, q);
        const int m_size = load_msize(m_sizes, ms_i64, e);
        i0 = blockIdx.y * GT, i_end = N;
        j0 = blockIdx.x * GT, j_end = K;
        r_begin = m_start, r_end = m_start + m_size;
        if ((int64_t)r_end > R) r_end = (int)R;
        a_base = a, lda = N;
        b_base = b, ldb = K;
        c_base = c + (int64_t)e * N * K, ldc = K;
    } else {
        // blockIdx.x enumerates (expert, m-tile) pairs in expert order; slots past the last
        // real tile exit.
        int slot = blockIdx.x, m_start = 0, e = 0, m_size = 0;
        bool found = false;
        for (; e < E; ++e) {
            m_size = load_msize(m_sizes, ms_i64, e);
            const int t = ceil_div(m_size, GT);
            if (slot < t) {
                found = true;
                break;
            }
            slot -= t;
            m_start += m_size;
        }
        if (!found) return;
        i0 = m_start + slot * GT;
        i_end = m_start + m_size;
        if ((int64_t)i_end > R) i_end = (int)R;
        j0 = blockIdx.y * GT, j_end = N;
        r_begin = 0, r_end = K;
        a_base = a, lda = K;
        b_base = b + (int64_t)e * N * K;
        ldb = (MODE == MODE_FWD) ? K : N;
        c_base = c, ldc = N;
    }

    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int r0 = r_begin; r0 < r_end; r0 += GK) {
        load_tile<TI, MODE != MODE_DW>(As, a_base, lda, i0, i_end, r0, r_end, tid);
        load_tile<TI, MODE == MODE_FWD>(Bs, b_base, ldb, j0, j_end, r0, r_end, tid);
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GK; ++k) {
            float av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = As[k][ty + 16 * i];
#pragma unroll
            for (int j = 0; j < 4; ++j) bv[j] = Bs[k][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = i0 + ty + 16 * i;
        if (row >= i_end) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = j0 + tx + 16 * j;
            if (col >= j_end) continue;
            TO *p = c_base + (int64_t)row * ldc + col;
            float v = alpha * acc[i][j];
            if (accumulate) v += to_f32(*p);
            *p = from_f32<TO>(v);
        }
    }
}

template <typename TI, typename TO>
int launch_generic(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R,
                   int N, int K, int E, float alpha, int accumulate, hipStream_t stream) {
    if (mode == MODE_DW) {
        if (ceil_div(N, GT) > 65535 || E > 65535) return MFL_ERR_UNSUPPORTED;
        dim3 grid(ceil_div(K, GT), ceil_div(N, GT), E);
        gemm_generic_kernel<TI, TO, MODE_DW><<<grid, 256, 0, stream>>>((const TI *)a, (const TI *)b, m_sizes, ms_i64,
                                                                       (TO *)c, R, N, K, E, alpha, accumulate);
    } else {
        const int64_t slots = (R + GT - 1) / GT + E;
        if (slots > 0x7fffffff || ceil_div(N, GT) > 65535) return MFL_ERR_UNSUPPORTED;
        dim3 grid((unsigned)slots, ceil_div(N, GT), 1);
        if (mode == MODE_FWD)
            gemm_generic_kernel<TI, TO, MODE_FWD><<<grid, 256, 0, stream>>>(
                (const TI *)a, (const TI *)b, m_sizes, ms_i64, (TO *)c, R, N, K, E, alpha, accumulate);
        else
            gemm_generic_kernel<TI, TO, MODE_DX><<<grid, 256, 0, stream>>>(
                (const TI *)a, (const TI *)b, m_sizes, ms_i64, (TO *)c, R, N, K, E, alpha, accumulate);
    }
    return launch_status();
}

}  // namespace

int gemm_generic(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                 int K, int E, int in_dtype, int out_dtype, float alpha, int accumulate, hipStream_t stream) {
    int rc = MFL_ERR_DTYPE;
    MFL_DISPATCH_FLOAT(in_dtype, TI, MFL_DISPATCH_FLOAT(out_dtype, TO, rc = (launch_generic<TI, TO>(
        mode, a, b, m_sizes, ms_i64, c, R, N, K, E, alpha, accumulate, stream))));
    return rc;
}

}  // namespace mfl
