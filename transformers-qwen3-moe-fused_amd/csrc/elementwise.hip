// Bandwidth-bound kernels: SiLU-mul, row gather / combine, NF4 and 8-bit blockwise
// (de)quantisation.  All of them stream 16-byte vectors per lane where alignment allows
// and fall back to element-wise access otherwise.
#include "common.h"
#include "ops.h"

namespace mfl {

namespace {

template <typename T>
struct Vec {
    static constexpr int N = 16 / sizeof(T);
    T v[N];
};

// (the loads fill their destination in place: returning the vector by value made the compiler
// take it apart into elements and pack it again)
template <typename T>
__device__ __forceinline__ void ld_vec(Vec<T> &r, const T *p) {
    *(uint4_t *)r.v = *(const uint4_t *)p;
}
// 16-byte load of data that is read once (non-temporal: does not displace what the caches hold).
// It pays where rows are picked at random (combine: 50 -> 27 us); the contiguous sweeps of the
// SiLU kernels were 10 % slower with it.
template <typename T>
__device__ __forceinline__ void ld_vec_stream(Vec<T> &r, const T *p) {
    *(uint4_t *)r.v = __builtin_nontemporal_load((const uint4_t *)p);
}
template <typename T>
__device__ __forceinline__ void st_vec(T *p, const Vec<T> &r) {
    *(uint4_t *)p = *(const uint4_t *)r.v;
}

// ---------------------------------------------------------------- SiLU-mul

template <typename T>
__global__ __launch_bounds__(256) void silu_fwd_kernel(const T *e, const T *g, T *h, int64_t n, int vec_ok) {
    constexpr int V = Vec<T>::N;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (vec_ok) {
        const int64_t nv = n / V;
        for (int64_t q = i; q < nv; q += stride) {
            Vec<T> ve, vg, vh;
            ld_vec(ve, e + q * V);
            ld_vec(vg, g + q * V);
#pragma unroll
            for (int u = 0; u < V; ++u) vh.v[u] = silu_fwd_one(ve.v[u], vg.v[u]);
            st_vec(h + q * V, vh);
        }
        for (int64_t q = nv * V + i; q < n; q += stride) h[q] = silu_fwd_one(e[q], g[q]);
    } else {
        for (int64_t q = i; q < n; q += stride) h[q] = silu_fwd_one(e[q], g[q]);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void silu_bwd_kernel(const T *dh, const T *e, const T *g, T *de, T *dg, T *h,
                                                       int64_t n, int vec_ok) {
    constexpr int V = Vec<T>::N;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (vec_ok) {
        const int64_t nv = n / V;
        for (int64_t q = i; q < nv; q += stride) {
            Vec<T> vdh, ve, vg, vh, vde, vdg;
            ld_vec(vdh, dh + q * V);
            ld_vec(ve, e + q * V);
            ld_vec(vg, g + q * V);
#pragma unroll
            for (int u = 0; u < V; ++u) silu_bwd_one(vdh.v[u], ve.v[u], vg.v[u], vh.v[u], vde.v[u], vdg.v[u]);
            if (h) st_vec(h + q * V, vh);
            st_vec(de + q * V, vde);
            st_vec(dg + q * V, vdg);
        }
        i += nv * V;
    }
    for (int64_t q = i; q < n; q += stride) {
        T vh, vde, vdg;
        silu_bwd_one(dh[q], e[q], g[q], vh, vde, vdg);
        if (h) h[q] = vh;
        de[q] = vde;
        dg[q] = vdg;
    }
}

inline int stream_grid(int64_t n_items) {
    const int64_t blocks = (n_items + 255) / 256;
    const int64_t cap = (int64_t)device_info().cu_count * 16;
    return (int)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

// ---------------------------------------------------------------- row gather / combine

// One wave per destination row.
template <typename T>
__global__ __launch_bounds__(256) void gather_rows_kernel(const T *src, const int32_t *idx, int idx_div,
                                                          const T *row_scale, T *dst, int64_t R_out, int H,
                                                          int vec_ok) {
    constexpr int V = Vec<T>::N;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= R_out) return;
    const int32_t j = idx[row];
    const T *s = src + (int64_t)(j / idx_div) * H;
    T *d = dst + row * H;
    const bool scaled = row_scale != nullptr;
    const float sc = scaled ? to_f32(row_scale[j]) : 1.0f;
    if (vec_ok) {
        // four vectors per lane in flight before the first store
        constexpr int U = 4;
        for (int c0 = lane * V; c0 < H; c0 += 64 * V * U) {
            Vec<T> v[U];
#pragma unroll
            for (int q = 0; q < U; ++q)
                if (c0 + q * 64 * V < H) ld_vec(v[q], s + c0 + q * 64 * V);
#pragma unroll
            for (int q = 0; q < U; ++q) {
                if (c0 + q * 64 * V >= H) continue;
                if (scaled) {
#pragma unroll
                    for (int u = 0; u < V; ++u) v[q].v[u] = from_f32<T>(to_f32(v[q].v[u]) * sc);
                }
                st_vec(d + c0 + q * 64 * V, v[q]);
            }
        }
    } else {
        for (int c = lane; c < H; c += 64) d[c] = scaled ? from_f32<T>(to_f32(s[c]) * sc) : s[c];
    }
}

// The same copy from the source's side: one wave per source row, read once, written to the k places
// pos[row * k + j] (times row_scale[row * k + j]).  The gather form reads a source row k times, from k
// workgroups that run at different times: 1.7 times the source's bytes came from HBM at 4096 tokens.
template <typename T>
__global__ __launch_bounds__(256) void scatter_rows_kernel(const T *src, const int32_t *pos, int k,
                                                           const T *row_scale, T *dst, int64_t R_src, int H,
                                                           int vec_ok) {
    constexpr int V = Vec<T>::N;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= R_src) return;
    const T *s = src + row * H;
    const int32_t *p = pos + row * k;
    const bool scaled = row_scale != nullptr;
    if (vec_ok) {
        constexpr int U = 4;
        for (int c0 = lane * V; c0 < H; c0 += 64 * V * U) {
            Vec<T> v[U];
#pragma unroll
            for (int q = 0; q < U; ++q)
                if (c0 + q * 64 * V < H) ld_vec(v[q], s + c0 + q * 64 * V);
            for (int j = 0; j < k; ++j) {
                T *d = dst + (int64_t)p[j] * H;
                const float sc = scaled ? to_f32(row_scale[row * k + j]) : 1.0f;
#pragma unroll
                for (int q = 0; q < U; ++q) {
                    if (c0 + q * 64 * V >= H) continue;
                    Vec<T> o = v[q];
                    if (scaled) {
#pragma unroll
                        for (int u = 0; u < V; ++u) o.v[u] = from_f32<T>(to_f32(o.v[u]) * sc);
                    }
                    st_vec(d + c0 + q * 64 * V, o);
                }
            }
        }
    } else {
        for (int j = 0; j < k; ++j) {
            T *d = dst + (int64_t)p[j] * H;
            const float sc = scaled ? to_f32(row_scale[row * k + j]) : 1.0f;
            for (int c = lane; c < H; c += 64) d[c] = scaled ? from_f32<T>(to_f32(s[c]) * sc) : s[c];
        }
    }
}

// One wave per token; fp32 accumulation over the k selected rows.
template <typename T>
__global__ __launch_bounds__(256) void combine_rows_kernel(const T *src, const int32_t *pos, const T *weights,
                                                           T *dst, int64_t Tn, int k, int H, int vec_ok) {
    constexpr int V = Vec<T>::N;
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= Tn) return;
    const int32_t *p = pos + t * k;
    T *d = dst + t * H;
    if (vec_ok) {
        // A lane owns CC chunks of V columns, 64 * V apart, so that the wave reads whole rows (a
        // row is one contiguous run in memory): U rows at a time, all chunks of a row together,
        // before they are added (in order: the sum is the same as one row after the other).
        // Every row is read exactly once: streaming loads, which leave the caches to the writes.
        // (Measured at 4096 tokens x 8 rows of 2048: a 1 KiB piece of each of 8 rows per pass
        // with ordinary loads, 55 us; this, 27 us.)
        constexpr int CC = 4, U = 4;
        for (int c0 = lane * V; c0 < H; c0 += CC * 64 * V) {
            float acc[CC][V];
#pragma unroll
            for (int cc = 0; cc < CC; ++cc)
#pragma unroll
                for (int u = 0; u < V; ++u) acc[cc][u] = 0.f;
            for (int j0 = 0; j0 < k; j0 += U) {
                Vec<T> v[U][CC];
                float w[U];
#pragma unroll
                for (int q = 0; q < U; ++q) {
                    if (j0 + q >= k) continue;
                    w[q] = weights ? to_f32(weights[t * k + j0 + q]) : 1.0f;
                    const T *row = src + (int64_t)p[j0 + q] * H + c0;
#pragma unroll
                    for (int cc = 0; cc < CC; ++cc)
                        if (c0 + cc * 64 * V < H) ld_vec_stream(v[q][cc], row + cc * 64 * V);
                }
#pragma unroll
                for (int q = 0; q < U; ++q) {
                    if (j0 + q >= k) continue;
#pragma unroll
                    for (int cc = 0; cc < CC; ++cc)
#pragma unroll
                        for (int u = 0; u < V; ++u) acc[cc][u] = fmaf(to_f32(v[q][cc].v[u]), w[q], acc[cc][u]);
                }
            }
#pragma unroll
            for (int cc = 0; cc < CC; ++cc) {
                if (c0 + cc * 64 * V >= H) continue;
                Vec<T> o;
#pragma unroll
                for (int u = 0; u < V; ++u) o.v[u] = from_f32<T>(acc[cc][u]);
                st_vec(d + c0 + cc * 64 * V, o);
            }
        }
    } else {
        for (int c = lane; c < H; c += 64) {
            float acc = 0.f;
            for (int j = 0; j < k; ++j) {
                const float w = weights ? to_f32(weights[t * k + j]) : 1.0f;
                acc = fmaf(to_f32(src[(int64_t)p[j] * H + c]), w, acc);
            }
            d[c] = from_f32<T>(acc);
        }
    }
}

// One wave per token: dots[t, j] = <a[t, :], b[pos[t*k+j], :]>.  Like the combine kernel it reads
// whole rows of b, U at a time with streaming loads (each is read exactly once); the token's own
// row of a comes from the cache after the first group.
template <typename T>
__global__ __launch_bounds__(256) void rows_dot_kernel(const T *a, const T *b, const int32_t *pos, T *dots,
                                                       int64_t Tn, int k, int H, int vec_ok) {
    constexpr int V = Vec<T>::N;
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= Tn) return;
    const T *pa = a + t * H;
    const int32_t *p = pos + t * k;
    constexpr int CC = 4, U = 4;
    for (int j0 = 0; j0 < k; j0 += U) {
        float acc[U];
#pragma unroll
        for (int q = 0; q < U; ++q) acc[q] = 0.f;
        if (vec_ok) {
            for (int c0 = lane * V; c0 < H; c0 += CC * 64 * V) {
                Vec<T> va[CC], vb[U][CC];
#pragma unroll
                for (int q = 0; q < U; ++q) {
                    if (j0 + q >= k) continue;
                    const T *row = b + (int64_t)p[j0 + q] * H + c0;
#pragma unroll
                    for (int cc = 0; cc < CC; ++cc)
                        if (c0 + cc * 64 * V < H) ld_vec_stream(vb[q][cc], row + cc * 64 * V);
                }
#pragma unroll
                for (int cc = 0; cc < CC; ++cc)
                    if (c0 + cc * 64 * V < H) ld_vec(va[cc], pa + c0 + cc * 64 * V);
#pragma unroll
                for (int q = 0; q < U; ++q) {
                    if (j0 + q >= k) continue;
#pragma unroll
                    for (int cc = 0; cc < CC; ++cc) {
                        if (c0 + cc * 64 * V >= H) continue;
#pragma unroll
                        for (int u = 0; u < V; ++u)
                            acc[q] = fmaf(to_f32(va[cc].v[u]), to_f32(vb[q][cc].v[u]), acc[q]);
                    }
                }
            }
        } else {
            for (int q = 0; q < U && j0 + q < k; ++q) {
                const T *pb = b + (int64_t)p[j0 + q] * H;
                for (int c = lane; c < H; c += 64) acc[q] = fmaf(to_f32(pa[c]), to_f32(pb[c]), acc[q]);
            }
        }
#pragma unroll
        for (int q = 0; q < U; ++q) {
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) acc[q] += __shfl_xor(acc[q], off);
            if (lane == 0 && j0 + q < k) dots[t * k + j0 + q] = from_f32<T>(acc[q]);
        }
    }
}

// ---------------------------------------------------------------- NF4

// Vector path (blocksize >= 8, aligned pointers): a lane decodes one packed dword (8 elements that
// share one absmax) into one 16-byte chunk of bf16 (two of fp32), and the 64 lanes of a wave take 64
// consecutive dwords, so a wave's loads and stores are whole contiguous runs (256 bytes in, 1 KiB
// out per instruction); four such groups per iteration keep four loads in flight per lane.  The
// output is written once and read by a later kernel: streaming stores.
template <typename T>
__global__ __launch_bounds__(256) void nf4_dequant_kernel(const uint8_t *__restrict__ wq,
                                                          const float *__restrict__ code16,
                                                          const float *__restrict__ absmax, int bs_shift,
                                                          T *__restrict__ out, int64_t n, int vec_ok) {
    __shared__ float code[16];
    if (threadIdx.x < 16) code[threadIdx.x] = code16[threadIdx.x];
    __syncthreads();
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t nbytes = n / 2;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (vec_ok) {
        constexpr int U = 4;
        const int64_t nchunks = nbytes / 4;  // packed dwords
        const int lane = threadIdx.x & 63;
        const int64_t wave = i >> 6, nwaves = stride >> 6;
        for (int64_t base = wave * (64 * U); base < nchunks; base += nwaves * (64 * U)) {
            uint32_t pk[U];
            float am[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t c = base + u * 64 + lane;
                if (c < nchunks) {
                    pk[u] = __builtin_nontemporal_load((const uint32_t *)wq + c);
                    am[u] = absmax[(c * 8) >> bs_shift];
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t c = base + u * 64 + lane;
                if (c >= nchunks) continue;
                union {
                    T e[8];
                    uint4_t v[sizeof(T) / 2];
                } vals;
#pragma unroll
                for (int bt = 0; bt < 4; ++bt) {
                    const uint32_t byte = (pk[u] >> (8 * bt)) & 0xffu;
                    vals.e[2 * bt] = from_f32<T>(code[byte >> 4] * am[u]);
                    vals.e[2 * bt + 1] = from_f32<T>(code[byte & 15u] * am[u]);
                }
                uint4_t *o = (uint4_t *)(out + c * 8);
#pragma unroll
                for (int v = 0; v < (int)sizeof(T) / 2; ++v) __builtin_nontemporal_store(vals.v[v], o + v);
            }
        }
        i += nchunks * 4;
    }
    for (int64_t q = i; q < nbytes; q += stride) {
        const uint32_t byte = wq[q];
        out[2 * q] = from_f32<T>(code[byte >> 4] * absmax[(2 * q) >> bs_shift]);
        out[2 * q + 1] = from_f32<T>(code[byte & 15u] * absmax[(2 * q + 1) >> bs_shift]);
    }
}

__global__ __launch_bounds__(256) void dequant_u8_kernel(const uint8_t *__restrict__ v,
                                                         const float *__restrict__ code256,
                                                         const float *__restrict__ absmax2, int blocksize2,
                                                         float offset, float *__restrict__ out, int64_t n) {
    __shared__ float code[256];
    code[threadIdx.x] = code256[threadIdx.x];
    __syncthreads();
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        out[i] = code[v[i]] * absmax2[i / blocksize2] + offset;
}

// One wave per quantisation block.
template <typename T>
__global__ __launch_bounds__(256) void nf4_quant_kernel(const T *__restrict__ w, int64_t nblocks, int blocksize,
                                                        const float *__restrict__ code16,
                                                        uint8_t *__restrict__ wq, float *__restrict__ absmax) {
    __shared__ float code[16];
    if (threadIdx.x < 16) code[threadIdx.x] = code16[threadIdx.x];
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int64_t blk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blk >= nblocks) return;
    const T *src = w + blk * blocksize;
    float am = 0.f;
    for (int i = lane; i < blocksize; i += 64) am = fmaxf(am, fabsf(to_f32(src[i])));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) am = fmaxf(am, __shfl_xor(am, off));
    if (lane == 0) absmax[blk] = am;
    const float inv = am > 0.f ? 1.0f / am : 0.f;
    for (int p = lane; p < blocksize / 2; p += 64) {
        uint32_t nib[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float v = to_f32(src[2 * p + h]) * inv;
            int best = 0;
            float bd = fabsf(v - code[0]);
#pragma unroll
            for (int c = 1; c < 16; ++c) {
                const float d = fabsf(v - code[c]);
                if (d < bd) {
                    bd = d;
                    best = c;
                }
            }
            nib[h] = (uint32_t)best;
        }
        wq[(blk * blocksize) / 2 + p] = (uint8_t)((nib[0] << 4) | nib[1]);
    }
}

inline int log2_exact(int v) {
    int s = 0;
    while ((1 << s) < v) ++s;
    return (1 << s) == v ? s : -1;
}

}  // namespace

int silu_mul_fwd(const void *e, const void *g, void *h, int64_t n, int dtype, hipStream_t stream) {
    if (n == 0) return MFL_OK;
    const int vec_ok = aligned(e, 16) && aligned(g, 16) && aligned(h, 16);
    MFL_DISPATCH_FLOAT(dtype, T, (silu_fwd_kernel<T><<<stream_grid(n / Vec<T>::N + 1), 256, 0, stream>>>(
                                     (const T *)e, (const T *)g, (T *)h, n, vec_ok)));
    return launch_status();
}

int silu_mul_bwd(const void *dh, const void *e, const void *g, void *de, void *dg, void *h, int64_t n, int dtype,
                 hipStream_t stream) {
    if (n == 0) return MFL_OK;
    const int vec_ok = aligned(dh, 16) && aligned(e, 16) && aligned(g, 16) && aligned(de, 16) && aligned(dg, 16) &&
                       (h == nullptr || aligned(h, 16));
    MFL_DISPATCH_FLOAT(dtype, T, (silu_bwd_kernel<T><<<stream_grid(n / Vec<T>::N + 1), 256, 0, stream>>>(
                                     (const T *)dh, (const T *)e, (const T *)g, (T *)de, (T *)dg, (T *)h, n, vec_ok)));
    return launch_status();
}

int scatter_rows(const void *src, const int32_t *pos, int k, const void *row_scale, void *dst, int64_t R_src, int H,
                 int dtype, hipStream_t stream) {
    if (R_src == 0) return MFL_OK;
    const size_t es = dtype_size(dtype);
    const int vec_ok = aligned(src, 16) && aligned(dst, 16) && ((size_t)H * es) % 16 == 0;
    const unsigned grid = (unsigned)((R_src + 3) / 4);
    MFL_DISPATCH_FLOAT(dtype, T, (scatter_rows_kernel<T><<<grid, 256, 0, stream>>>(
                                     (const T *)src, pos, k, (const T *)row_scale, (T *)dst, R_src, H, vec_ok)));
    return launch_status();
}

int gather_rows(const void *src, const int32_t *idx, int idx_div, const void *row_scale, void *dst, int64_t R_out,
                int H, int dtype, hipStream_t stream) {
    if (R_out == 0) return MFL_OK;
    const size_t es = dtype_size(dtype);
    const int vec_ok = aligned(src, 16) && aligned(dst, 16) && ((size_t)H * es) % 16 == 0;
    const unsigned grid = (unsigned)((R_out + 3) / 4);
    MFL_DISPATCH_FLOAT(dtype, T, (gather_rows_kernel<T><<<grid, 256, 0, stream>>>(
                                     (const T *)src, idx, idx_div, (const T *)row_scale, (T *)dst, R_out, H, vec_ok)));
    return launch_status();
}

int combine_rows(const void *src, const int32_t *pos, const void *weights, void *dst, int64_t T_, int k, int H,
                 int dtype, hipStream_t stream) {
    if (T_ == 0) return MFL_OK;
    const size_t es = dtype_size(dtype);
    const int vec_ok = aligned(src, 16) && aligned(dst, 16) && ((size_t)H * es) % 16 == 0;
    const unsigned grid = (unsigned)((T_ + 3) / 4);
    MFL_DISPATCH_FLOAT(dtype, T, (combine_rows_kernel<T><<<grid, 256, 0, stream>>>(
                                     (const T *)src, pos, (const T *)weights, (T *)dst, T_, k, H, vec_ok)));
    return launch_status();
}

int rows_dot(const void *a, const void *b, const int32_t *pos, void *dots, int64_t T_, int k, int H, int dtype,
             hipStream_t stream) {
    if (T_ * k == 0) return MFL_OK;
    const size_t es = dtype_size(dtype);
    const int vec_ok = aligned(a, 16) && aligned(b, 16) && ((size_t)H * es) % 16 == 0;
    const unsigned grid = (unsigned)((T_ + 3) / 4);
    MFL_DISPATCH_FLOAT(dtype, T, (rows_dot_kernel<T><<<grid, 256, 0, stream>>>((const T *)a, (const T *)b, pos,
                                                                               (T *)dots, T_, k, H, vec_ok)));
    return launch_status();
}

int nf4_dequant(const uint8_t *wq, const float *code16, const float *absmax, int blocksize, void *out, int64_t n,
                int out_dtype, hipStream_t stream) {
    if (n == 0) return MFL_OK;
    const int shift = log2_exact(blocksize);
    if (shift < 1) return MFL_ERR_SHAPE;
    const int vec_ok = aligned(wq, 4) && aligned(out, 16) && blocksize >= 8;
    MFL_DISPATCH_FLOAT(out_dtype, T, (nf4_dequant_kernel<T><<<stream_grid(n / 32 + 1), 256, 0, stream>>>(
                                         wq, code16, absmax, shift, (T *)out, n, vec_ok)));
    return launch_status();
}

int dequant_blockwise_u8(const uint8_t *v, const float *code256, const float *absmax2, int blocksize2, float offset,
                         float *out, int64_t n, hipStream_t stream) {
    if (n == 0) return MFL_OK;
    dequant_u8_kernel<<<stream_grid(n), 256, 0, stream>>>(v, code256, absmax2, blocksize2, offset, out, n);
    return launch_status();
}

int nf4_quant(const void *w, int w_dtype, int64_t n, int blocksize, const float *code16, uint8_t *wq, float *absmax,
              hipStream_t stream) {
    if (n == 0) return MFL_OK;
    const int64_t nblocks = n / blocksize;
    const unsigned grid = (unsigned)((nblocks + 3) / 4);
    MFL_DISPATCH_FLOAT(w_dtype, T, (nf4_quant_kernel<T><<<grid, 256, 0, stream>>>((const T *)w, nblocks, blocksize,
                                                                                  code16, wq, absmax)));
    return launch_status();
}

}  // namespace mfl
