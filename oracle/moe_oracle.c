/*
 * CPU restatement of the reference's moe_fused_linear hot path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the
 * smoke check and the benchmark's cpu_baseline leg may load it; the product
 * path (the HIP library) never calls into it and has no CPU fallback.
 *
 * Every function cites the reference file:line whose arithmetic it restates
 * (paths relative to the reference checkout).  Floating-point reductions
 * accumulate in double and round once to float, so the oracle sits closer to
 * the exact value than any fp32 summation order would.
 *
 * Pinning status (what independently checks each function is listed in
 * tests/test_oracle_*.py):
 *   orc_linear_*            pinned: einsum closed forms, autograd, brute force
 *   orc_expert_counts_*     pinned: bincount + stable argsort, invariants
 *   orc_softmax_topk        pinned: library softmax/topk on tie-free inputs,
 *                           declared tie rule (lower index first) tested apart
 *   orc_silu_mul_*          pinned: library silu + autograd in fp64
 *   orc_nf4_dequant/quant   PARITY UNPINNED against bitsandbytes (the package
 *                           is not installed and is not vendored by the
 *                           reference).  Pinned only against the reference's
 *                           own restatement of the format
 *                           (grouped_gemm/forward_4bit.py:99-104), the
 *                           published 16-entry table, its closed form to
 *                           1.2e-7, and quantise/dequantise round trips.
 *   orc_dequant_blockwise_u8 same status as NF4 (nested absmax path).
 *
 * Build: see oracle/Makefile  (gcc -O2 -fopenmp -shared -fPIC).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ bf16 */

static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even, NaN kept quiet */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

void orc_f32_to_bf16(const float *src, uint16_t *dst, int64_t n) {
    for (int64_t i = 0; i < n; ++i) dst[i] = f32_to_bf16(src[i]);
}

void orc_bf16_to_f32(const uint16_t *src, float *dst, int64_t n) {
    for (int64_t i = 0; i < n; ++i) dst[i] = bf16_to_f32(src[i]);
}

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------- naive linear trio (a1/a2) */

/* qwen3_moe_fused/functional.py:7-33
 * out[b, o] = sum_i weight[sel[b], o, i] * input[b, i]   (one mat-vec per row) */
void orc_linear_fwd_f32(const float *x, const float *w, const int64_t *sel, float *out,
                        int64_t B, int N, int K) {
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < B; ++b) {
        const float *wb = w + (size_t)sel[b] * N * K;
        const float *xb = x + (size_t)b * K;
        for (int o = 0; o < N; ++o) {
            const float *wr = wb + (size_t)o * K;
            double acc = 0.0;
#pragma omp simd reduction(+ : acc)
            for (int i = 0; i < K; ++i) acc += (double)wr[i] * (double)xb[i];
            out[(size_t)b * N + o] = (float)acc;
        }
    }
}

/* qwen3_moe_fused/functional.py:37-48
 * grad_input[b, i] = sum_o weight[sel[b], o, i] * grad_output[b, o] */
void orc_linear_bwd_input_f32(const float *dy, const float *w, const int64_t *sel, float *dx,
                              int64_t B, int N, int K) {
#pragma omp parallel
    {
        double *acc = (double *)malloc(sizeof(double) * (size_t)K);
#pragma omp for schedule(static)
        for (int64_t b = 0; b < B; ++b) {
            const float *wb = w + (size_t)sel[b] * N * K;
            const float *dyb = dy + (size_t)b * N;
            for (int i = 0; i < K; ++i) acc[i] = 0.0;
            for (int o = 0; o < N; ++o) {
                const double g = (double)dyb[o];
                const float *wr = wb + (size_t)o * K;
#pragma omp simd
                for (int i = 0; i < K; ++i) acc[i] += g * (double)wr[i];
            }
            for (int i = 0; i < K; ++i) dx[(size_t)b * K + i] = (float)acc[i];
        }
        free(acc);
    }
}

/* qwen3_moe_fused/functional.py:52-61
 * grad_weight = zeros; grad_weight[sel[b]] += grad_output[b, :, None] * input[b, None, :]
 * Rows are visited in ascending b for every (e, o) slice, as in the reference loop;
 * threads split the output rows o, never the reduction over b. */
void orc_linear_bwd_weight_f32(const float *dy, const float *x, const int64_t *sel, float *dw,
                               int64_t B, int N, int K, int E) {
    memset(dw, 0, sizeof(float) * (size_t)E * N * K);
    /* rows of each expert in ascending b (a bucket pass, so the loops below do not rescan sel) */
    int64_t *start = (int64_t *)calloc((size_t)E + 1, sizeof(int64_t));
    int64_t *fill = (int64_t *)calloc((size_t)E, sizeof(int64_t));
    int64_t *rows = (int64_t *)malloc(sizeof(int64_t) * (size_t)(B > 0 ? B : 1));
    for (int64_t b = 0; b < B; ++b) start[sel[b] + 1] += 1;
    for (int e = 0; e < E; ++e) start[e + 1] += start[e];
    for (int64_t b = 0; b < B; ++b) rows[start[sel[b]] + fill[sel[b]]++] = b;
#pragma omp parallel
    {
        double *acc = (double *)malloc(sizeof(double) * (size_t)K);
#pragma omp for schedule(dynamic, 8) collapse(2)
        for (int e = 0; e < E; ++e) {
            for (int o = 0; o < N; ++o) {
                if (start[e + 1] == start[e]) continue;
                for (int i = 0; i < K; ++i) acc[i] = 0.0;
                for (int64_t r = start[e]; r < start[e + 1]; ++r) {
                    const int64_t b = rows[r];
                    const double g = (double)dy[(size_t)b * N + o];
                    const float *xb = x + (size_t)b * K;
#pragma omp simd
                    for (int i = 0; i < K; ++i) acc[i] += g * (double)xb[i];
                }
                float *dst = dw + ((size_t)e * N + o) * K;
                for (int i = 0; i < K; ++i) dst[i] = (float)acc[i];
            }
        }
        free(acc);
    }
    free(start);
    free(fill);
    free(rows);
}

/* ------------------------------------------------- expert counting sort (a9) */

/* qwen3_moe_fused/kernels/indexing.py:48-65  (get_expert_counts_and_idx)
 *   counts[e]  = #{j : s[j] == e}                                  (:53)
 *   rank[j]    = inclusive running count of s[j] up to j           (:56-57)
 *   offsets[e] = exclusive prefix of counts                        (:58)
 *   idx[j]     = rank[j] + offsets[s[j]] - 1                       (:59)
 *   inv_idx[idx[j]] = j                                            (:61-62)
 * The reference returns (counts, inv_idx, idx); its caller names them
 * (m_sizes, sort_idx, inv_sort_idx)  (modular_qwen3_moe_fused.py:102).
 * Returns 0, or -1 when an id lies outside [0, E). */
int orc_expert_counts_and_idx(const int64_t *s, int64_t R, int E, int32_t *counts,
                              int32_t *sort_idx, int32_t *inv_sort_idx) {
    int32_t *offsets = (int32_t *)calloc((size_t)E, sizeof(int32_t));
    int32_t *running = (int32_t *)calloc((size_t)E, sizeof(int32_t));
    for (int e = 0; e < E; ++e) counts[e] = 0;
    for (int64_t j = 0; j < R; ++j) {
        if (s[j] < 0 || s[j] >= E) {
            free(offsets);
            free(running);
            return -1;
        }
        counts[s[j]] += 1;
    }
    int32_t acc = 0;
    for (int e = 0; e < E; ++e) {
        acc += counts[e];
        offsets[e] = acc - counts[e];
    }
    for (int64_t j = 0; j < R; ++j) {
        const int64_t e = s[j];
        running[e] += 1; /* inclusive cumsum of the compare row */
        const int32_t idx = running[e] + offsets[e] - 1;
        inv_sort_idx[j] = idx;
        sort_idx[idx] = (int32_t)j;
    }
    free(offsets);
    free(running);
    return 0;
}

/* qwen3_moe_fused/kernels/indexing.py:18-23 */
void orc_expert_counts(const int64_t *s, int64_t R, int E, int32_t *counts) {
    for (int e = 0; e < E; ++e) counts[e] = 0;
    for (int64_t j = 0; j < R; ++j) counts[s[j]] += 1;
}

/* ------------------------------------------------- softmax + top-k routing (a10) */

/* qwen3_moe_fused/modular_qwen3_moe_fused.py:87-91 (same at fast_lora.py:52-56)
 *   p = softmax(logits, dim=1) in fp32; (w, idx) = topk(p, k) sorted descending;
 *   if renorm: w /= sum(w).
 * Tie rule (the library leaves it open): equal probabilities -> lower expert id first. */
void orc_softmax_topk(const float *logits, int64_t T, int E, int k, int renorm, float *weights,
                      int64_t *idx) {
#pragma omp parallel
    {
        float *p = (float *)malloc(sizeof(float) * (size_t)E);
        char *taken = (char *)malloc((size_t)E);
#pragma omp for schedule(static)
        for (int64_t t = 0; t < T; ++t) {
            const float *row = logits + (size_t)t * E;
            float mx = row[0];
            for (int e = 1; e < E; ++e) mx = row[e] > mx ? row[e] : mx;
            float sum = 0.0f;
            for (int e = 0; e < E; ++e) {
                p[e] = expf(row[e] - mx);
                sum += p[e];
            }
            for (int e = 0; e < E; ++e) p[e] = p[e] / sum;
            memset(taken, 0, (size_t)E);
            float wsum = 0.0f;
            for (int j = 0; j < k; ++j) {
                int best = -1;
                for (int e = 0; e < E; ++e) {
                    if (taken[e]) continue;
                    if (best < 0 || p[e] > p[best]) best = e;
                }
                taken[best] = 1;
                weights[(size_t)t * k + j] = p[best];
                idx[(size_t)t * k + j] = best;
                wsum += p[best];
            }
            if (renorm)
                for (int j = 0; j < k; ++j) weights[(size_t)t * k + j] /= wsum;
        }
        free(p);
        free(taken);
    }
}

/* ------------------------------------------------- SiLU-mul (a12) */

static inline float sigmoidf_(float e) { return 1.0f / (1.0f + expf(-e)); }

/* qwen3_moe_fused/kernels/silu_mul.py:34-39
 *   f = bf16(e32 * sigmoid(e32));  h = bf16(f * g) */
void orc_silu_mul_fwd_bf16(const uint16_t *e, const uint16_t *g, uint16_t *h, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        const float e32 = bf16_to_f32(e[i]);
        const float f = bf16_to_f32(f32_to_bf16(e32 * sigmoidf_(e32)));
        h[i] = f32_to_bf16(f * bf16_to_f32(g[i]));
    }
}

void orc_silu_mul_fwd_f32(const float *e, const float *g, float *h, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) h[i] = (e[i] * sigmoidf_(e[i])) * g[i];
}

/* qwen3_moe_fused/kernels/silu_mul.py:62-73
 *   se = sigmoid(e32); ese = e32*se; f = bf16(ese); df = bf16(dh*g); dg = bf16(f*dh)
 *   de = bf16(f32(df) * se * (1 + e32 - ese)) */
void orc_silu_mul_bwd_bf16(const uint16_t *dh, const uint16_t *e, const uint16_t *g, uint16_t *de,
                           uint16_t *dg, uint16_t *h_or_null, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        const float e32 = bf16_to_f32(e[i]);
        const float g32 = bf16_to_f32(g[i]);
        const float dh32 = bf16_to_f32(dh[i]);
        const float se = sigmoidf_(e32);
        const float ese = e32 * se;
        const float f = bf16_to_f32(f32_to_bf16(ese));
        const float df = bf16_to_f32(f32_to_bf16(dh32 * g32));
        const uint16_t dg_i = f32_to_bf16(f * dh32);
        const uint16_t de_i = f32_to_bf16(df * se * (1.0f + e32 - ese));
        if (h_or_null) h_or_null[i] = f32_to_bf16(f * g32); /* :103 in-place variant also yields h */
        de[i] = de_i;
        dg[i] = dg_i;
    }
}

void orc_silu_mul_bwd_f32(const float *dh, const float *e, const float *g, float *de, float *dg,
                          float *h_or_null, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        const float se = sigmoidf_(e[i]);
        const float ese = e[i] * se;
        const float df = dh[i] * g[i];
        const float dg_i = ese * dh[i];
        const float de_i = df * se * (1.0f + e[i] - ese);
        if (h_or_null) h_or_null[i] = ese * g[i];
        de[i] = de_i;
        dg[i] = dg_i;
    }
}

/* ------------------------------------------------- NF4 (a7/a8) */

/* The 16-entry NF4 code book that bitsandbytes hard-codes and stores in
 * quant_state.code; the reference kernel receives it as data
 * (qwen3_moe_fused/grouped_gemm/forward_4bit.py:146-147). */
static const float NF4_CODE[16] = {
    -1.0f,
    -0.6961928009986877f,
    -0.5250730514526367f,
    -0.39491748809814453f,
    -0.28444138169288635f,
    -0.18477343022823334f,
    -0.09105003625154495f,
    0.0f,
    0.07958029955625534f,
    0.16093020141124725f,
    0.24611230194568634f,
    0.33791524171829224f,
    0.44070982933044434f,
    0.5626170039176941f,
    0.7229568362236023f,
    1.0f,
};

void orc_nf4_code(float *out16) { memcpy(out16, NF4_CODE, sizeof(NF4_CODE)); }

/* qwen3_moe_fused/grouped_gemm/forward_4bit.py:99-104
 *   byte i holds element 2i in its high nibble and element 2i+1 in its low nibble (:100)
 *   value = code[nibble] * absmax[element_index / blocksize] in fp32 (:101-102),
 *   rounded once to the output type (:104). */
void orc_nf4_dequant_f32(const uint8_t *q, const float *code16, const float *absmax, int blocksize,
                         int64_t n_elems, float *out) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n_elems / 2; ++i) {
        const uint8_t b = q[i];
        out[2 * i] = code16[b >> 4] * absmax[(2 * i) / blocksize];
        out[2 * i + 1] = code16[b & 15] * absmax[(2 * i + 1) / blocksize];
    }
}

void orc_nf4_dequant_bf16(const uint8_t *q, const float *code16, const float *absmax,
                          int blocksize, int64_t n_elems, uint16_t *out) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n_elems / 2; ++i) {
        const uint8_t b = q[i];
        out[2 * i] = f32_to_bf16(code16[b >> 4] * absmax[(2 * i) / blocksize]);
        out[2 * i + 1] = f32_to_bf16(code16[b & 15] * absmax[(2 * i + 1) / blocksize]);
    }
}

/* Blockwise NF4 quantiser used to build test inputs: absmax = max|block|,
 * nibble = nearest code entry to x/absmax (ties -> lower code index).
 * The reference obtains its inputs from bitsandbytes' quantize_nf4
 * (test_moe_fused_linear.py:40); this is the same published scheme, with the
 * midpoint tie rule being this file's own choice. */
void orc_nf4_quant_f32(const float *w, int64_t n_elems, int blocksize, uint8_t *q, float *absmax) {
    const int64_t nblocks = n_elems / blocksize;
#pragma omp parallel for schedule(static)
    for (int64_t blk = 0; blk < nblocks; ++blk) {
        const float *src = w + blk * blocksize;
        float am = 0.0f;
        for (int i = 0; i < blocksize; ++i) {
            const float a = fabsf(src[i]);
            am = a > am ? a : am;
        }
        absmax[blk] = am;
        const float inv = am > 0.0f ? 1.0f / am : 0.0f;
        for (int i = 0; i < blocksize; i += 2) {
            int nib[2];
            for (int h = 0; h < 2; ++h) {
                const float v = src[i + h] * inv;
                int best = 0;
                float bd = fabsf(v - NF4_CODE[0]);
                for (int c = 1; c < 16; ++c) {
                    const float d = fabsf(v - NF4_CODE[c]);
                    if (d < bd) {
                        bd = d;
                        best = c;
                    }
                }
                nib[h] = best;
            }
            q[(blk * blocksize + i) / 2] = (uint8_t)((nib[0] << 4) | nib[1]);
        }
    }
}

/* Nested absmax: qwen3_moe_fused/grouped_gemm/forward_4bit.py:149-152
 *   absmax = dequantize_blockwise(absmax_u8, state2) + offset
 * with dequantize_blockwise(v)[i] = code256[v[i]] * absmax2[i / blocksize2]. */
void orc_dequant_blockwise_u8(const uint8_t *v, const float *code256, const float *absmax2,
                              int blocksize2, float offset, int64_t n, float *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = code256[v[i]] * absmax2[i / blocksize2] + offset;
}
