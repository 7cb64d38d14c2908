// Token routing: fused softmax + top-k, and the stable counting sort of expert ids.
//
// Both are latency/bandwidth-bound integer-heavy kernels built from wavefront ballots,
// cross-lane shuffles and LDS histograms; neither uses atomics, so results are
// deterministic and the index outputs are reproducible bit for bit.
#include "common.h"
#include "ops.h"

namespace mfl {

namespace {

// ---------------------------------------------------------------- softmax + top-k

// One wave per token.  Lane l holds experts l, l+64, l+128, ... (VPL of them).
template <typename TI, typename TC, int VPL>
__global__ __launch_bounds__(256) void softmax_topk_kernel(const TI *__restrict__ logits, int64_t T, int E, int k,
                                                           int renorm, float *__restrict__ w_f32,
                                                           TC *__restrict__ w_cast, int64_t *__restrict__ idx) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    const TI *row = logits + t * E;

    float p[VPL];
    float mx = -INFINITY;
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
        const int e = lane + 64 * v;
        p[v] = e < E ? to_f32(row[e]) : -INFINITY;
        mx = fmaxf(mx, p[v]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    float sum = 0.f;
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
        const int e = lane + 64 * v;
        p[v] = e < E ? expf(p[v] - mx) : 0.f;
        sum += p[v];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
        const int e = lane + 64 * v;
        p[v] = e < E ? p[v] / sum : -1.0f;  // -1 marks "not selectable"
    }

    float my_w = 0.f, wsum = 0.f;
    int my_i = 0;
    for (int j = 0; j < k; ++j) {
        // lane-local best: larger p, then lower expert id (v ascending = id ascending)
        float bp = -2.0f;
        int bi = 0x7fffffff;
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
            if (p[v] > bp) {
                bp = p[v];
                bi = lane + 64 * v;
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float op = __shfl_xor(bp, off);
            const int oi = __shfl_xor(bi, off);
            if (op > bp || (op == bp && oi < bi)) {
                bp = op;
                bi = oi;
            }
        }
        // the owner retires the winner
#pragma unroll
        for (int v = 0; v < VPL; ++v)
            if (bi == lane + 64 * v) p[v] = -1.0f;
        if (lane == j) {
            my_w = bp;
            my_i = bi;
        }
        wsum += bp;
    }
    if (lane < k) {
        const float w = renorm ? my_w / wsum : my_w;
        if (w_f32) w_f32[t * k + lane] = w;
        if (w_cast) w_cast[t * k + lane] = from_f32<TC>(w);
        idx[t * k + lane] = my_i;
    }
}

template <typename TI, typename TC>
int launch_topk(const void *logits, int64_t T, int E, int k, int renorm, float *w_f32, void *w_cast, int64_t *idx,
                hipStream_t stream) {
    const unsigned grid = (unsigned)((T + 3) / 4);
    const int vpl = ceil_div(E, 64);
#define MFL_TOPK(V)                                                                                        \
    softmax_topk_kernel<TI, TC, V><<<grid, 256, 0, stream>>>((const TI *)logits, T, E, k, renorm, w_f32, \
                                                             (TC *)w_cast, idx)
    if (vpl <= 1)
        MFL_TOPK(1);
    else if (vpl <= 2)
        MFL_TOPK(2);
    else if (vpl <= 4)
        MFL_TOPK(4);
    else if (vpl <= 8)
        MFL_TOPK(8);
    else if (vpl <= 16)
        MFL_TOPK(16);
    else
        return MFL_ERR_UNSUPPORTED;
#undef MFL_TOPK
    return launch_status();
}

// ---------------------------------------------------------------- stable counting sort

constexpr int kSortMaxE = 4096;

__device__ __forceinline__ int64_t load_key(const void *sel, int is_i64, int64_t j) {
    return is_i64 ? ((const int64_t *)sel)[j] : (int64_t)((const int32_t *)sel)[j];
}

// Phase 1 for one wave: walk its segment [seg_begin, seg_end) in batches of 64 in order,
// count keys into the wave-private histogram `hist` (LDS, E ints, zeroed by the caller) and,
// when `local_rank` is given, store each row's rank among the rows of the same key seen so
// far by this wave.  Within a batch, lanes sharing a key are found with one ballot per key
// bit; their order is the lane order, which keeps the sort stable.
__device__ __forceinline__ void wave_count(const void *sel, int is_i64, int E, int key_bits, int64_t seg_begin,
                                           int64_t seg_end, int *hist, int32_t *local_rank, int lane) {
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    for (int64_t base = seg_begin; base < seg_end; base += 64) {
        const int64_t j = base + lane;
        bool valid = j < seg_end;
        int key = 0;
        if (valid) {
            const int64_t k64 = load_key(sel, is_i64, j);
            valid = k64 >= 0 && k64 < E;
            key = valid ? (int)k64 : 0;
        }
        uint64_t same = __ballot(valid);
        for (int b = 0; b < key_bits; ++b) {
            const uint64_t bal = __ballot((key >> b) & 1);
            same &= ((key >> b) & 1) ? bal : ~bal;
        }
        if (valid) {
            const int before = hist[key];
            const int rank = before + __popcll(same & lt_mask);
            if (local_rank) local_rank[j] = rank;
            // the last lane of each key group publishes the new running count
            if ((same >> lane) == 1ull) hist[key] = before + __popcll(same);
        }
    }
}

__device__ __forceinline__ void segment_of(int w, int n_waves, int64_t R, int64_t &b, int64_t &e) {
    int64_t seg = (R + n_waves - 1) / n_waves;
    seg = (seg + 63) / 64 * 64;
    b = (int64_t)w * seg;
    e = b + seg;
    if (b > R) b = R;
    if (e > R) e = R;
}

// Whole sort in one workgroup (n_waves <= 16): the (wave, expert) table lives in LDS.
__global__ __launch_bounds__(1024) void sort_single_kernel(const void *__restrict__ sel, int is_i64, int64_t R,
                                                           int E, int key_bits, int32_t *__restrict__ counts,
                                                           int32_t *__restrict__ sort_idx,
                                                           int32_t *__restrict__ inv_sort_idx) {
    extern __shared__ int lds[];  // [n_waves][E] table, then [E] totals
    const int n_waves = blockDim.x >> 6;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int *table = lds;
    int *totals = lds + n_waves * E;
    for (int i = threadIdx.x; i < n_waves * E; i += blockDim.x) table[i] = 0;
    __syncthreads();
    int64_t sb, se;
    segment_of(wave, n_waves, R, sb, se);
    wave_count(sel, is_i64, E, key_bits, sb, se, table + wave * E, inv_sort_idx, lane);
    __syncthreads();
    // exclusive scan over waves for every expert, totals per expert
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        int run = 0;
        for (int w = 0; w < n_waves; ++w) {
            const int c = table[w * E + e];
            table[w * E + e] = run;
            run += c;
        }
        totals[e] = run;
        counts[e] = run;
    }
    __syncthreads();
    if (sort_idx == nullptr && inv_sort_idx == nullptr) return;
    // exclusive scan of totals over experts (wave 0, 64 experts per step)
    if (wave == 0) {
        int carry = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            const int v = e < E ? totals[e] : 0;
            int inc = v;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int o = __shfl_up(inc, off);
                if (lane >= off) inc += o;
            }
            if (e < E) totals[e] = carry + inc - v;
            carry += __shfl(inc, 63);
        }
    }
    __syncthreads();
    for (int64_t base = sb; base < se; base += 64) {
        const int64_t j = base + lane;
        if (j < se) {
            const int64_t k64 = load_key(sel, is_i64, j);
            if (k64 >= 0 && k64 < E) {
                const int pos = inv_sort_idx[j] + table[wave * E + (int)k64] + totals[(int)k64];
                inv_sort_idx[j] = pos;
                if (sort_idx) sort_idx[pos] = (int32_t)j;
            }
        }
    }
}

// Multi-workgroup path: count -> scan -> scatter, table in global workspace.
__global__ __launch_bounds__(256) void sort_count_kernel(const void *__restrict__ sel, int is_i64, int64_t R, int E,
                                                         int key_bits, int n_waves, int32_t *__restrict__ table,
                                                         int32_t *__restrict__ local_rank) {
    extern __shared__ int lds[];  // [4][E]
    const int wave_in_block = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + wave_in_block;
    int *hist = lds + wave_in_block * E;
    for (int i = lane; i < E; i += 64) hist[i] = 0;
    if (wave >= n_waves) return;
    int64_t sb, se;
    segment_of(wave, n_waves, R, sb, se);
    wave_count(sel, is_i64, E, key_bits, sb, se, hist, local_rank, lane);
    for (int i = lane; i < E; i += 64) table[(int64_t)wave * E + i] = hist[i];
}

__global__ __launch_bounds__(1024) void sort_scan_kernel(int32_t *__restrict__ table, int n_waves, int E,
                                                         int32_t *__restrict__ counts) {
    __shared__ int totals[kSortMaxE];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        int run = 0;
        for (int w0 = 0; w0 < n_waves; w0 += 8) {
            int c[8];  // loads first, so the eight are in flight together
#pragma unroll
            for (int u = 0; u < 8; ++u) c[u] = (w0 + u) < n_waves ? table[(int64_t)(w0 + u) * E + e] : 0;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if ((w0 + u) < n_waves) table[(int64_t)(w0 + u) * E + e] = run;
                run += c[u];
            }
        }
        totals[e] = run;
        counts[e] = run;
    }
    __syncthreads();
    if (wave == 0) {
        int carry = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            const int v = e < E ? totals[e] : 0;
            int inc = v;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int o = __shfl_up(inc, off);
                if (lane >= off) inc += o;
            }
            if (e < E) totals[e] = carry + inc - v;
            carry += __shfl(inc, 63);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n_waves * E; i += blockDim.x) table[i] += totals[i % E];
}

__global__ __launch_bounds__(256) void sort_scatter_kernel(const void *__restrict__ sel, int is_i64, int64_t R,
                                                           int E, int n_waves, const int32_t *__restrict__ table,
                                                           int32_t *__restrict__ sort_idx,
                                                           int32_t *__restrict__ inv_sort_idx) {
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wave >= n_waves) return;
    int64_t sb, se;
    segment_of(wave, n_waves, R, sb, se);
    for (int64_t base = sb; base < se; base += 64) {
        const int64_t j = base + lane;
        if (j < se) {
            const int64_t k64 = load_key(sel, is_i64, j);
            if (k64 >= 0 && k64 < E) {
                const int pos = inv_sort_idx[j] + table[(int64_t)wave * E + (int)k64];
                inv_sort_idx[j] = pos;
                if (sort_idx) sort_idx[pos] = (int32_t)j;
            }
        }
    }
}

constexpr int64_t kSingleBlockMaxR = 65536;

inline int multi_waves(int64_t R) {
    int64_t w = (R + 2047) / 2048;
    if (w > 128) w = 128;
    if (w < 1) w = 1;
    return (int)w;
}

}  // namespace

int route_softmax_topk(const void *logits, int logits_dtype, int64_t T, int E, int k, int renorm, float *w_f32,
                       void *w_cast, int cast_dtype, int64_t *idx, hipStream_t stream) {
    if (T == 0) return MFL_OK;
    int rc = MFL_ERR_DTYPE;
    MFL_DISPATCH_FLOAT(logits_dtype, TI, MFL_DISPATCH_FLOAT(cast_dtype, TC, rc = (launch_topk<TI, TC>(
        logits, T, E, k, renorm, w_f32, w_cast, idx, stream))));
    return rc;
}

size_t expert_sort_workspace(int64_t R, int E) {
    // table for the multi-workgroup path + a rank buffer used when inv_sort_idx is not requested
    const size_t table = R > kSingleBlockMaxR ? (size_t)multi_waves(R) * (size_t)E * 4 : 0;
    const size_t ranks = (size_t)(R > 0 ? R : 0) * 4;
    return ((table + 255) / 256) * 256 + ((ranks + 255) / 256) * 256 + 256;
}

int expert_sort(const void *sel, int is_i64, int64_t R, int E, int32_t *counts, int32_t *sort_idx,
                int32_t *inv_sort_idx, void *workspace, size_t ws_bytes, hipStream_t stream) {
    if (E > kSortMaxE) return MFL_ERR_UNSUPPORTED;
    int key_bits = 0;
    while ((1 << key_bits) < E) ++key_bits;
    const size_t table_bytes = ((R > kSingleBlockMaxR ? (size_t)multi_waves(R) * (size_t)E * 4 : 0) + 255) / 256 * 256;
    int32_t *table = (int32_t *)workspace;
    int32_t *rank_buf = inv_sort_idx;
    if (sort_idx != nullptr && inv_sort_idx == nullptr) {
        if (workspace == nullptr || ws_bytes < table_bytes + (size_t)R * 4) return MFL_ERR_WORKSPACE;
        rank_buf = (int32_t *)((char *)workspace + table_bytes);
    }
    if (R <= kSingleBlockMaxR) {
        int n_waves = (int)((R + 2047) / 2048);
        if (n_waves < 1) n_waves = 1;
        if (n_waves > 16) n_waves = 16;
        while (n_waves > 1 && (size_t)(n_waves + 1) * E * 4 > 64 * 1024) --n_waves;
        const size_t lds = (size_t)(n_waves + 1) * E * 4;
        sort_single_kernel<<<1, n_waves * 64, lds, stream>>>(sel, is_i64, R, E, key_bits, counts, sort_idx, rank_buf);
        return launch_status();
    }
    const int n_waves = multi_waves(R);
    if (workspace == nullptr || ws_bytes < table_bytes) return MFL_ERR_WORKSPACE;
    const unsigned blocks = (unsigned)ceil_div(n_waves, 4);
    sort_count_kernel<<<blocks, 256, (size_t)4 * E * 4, stream>>>(sel, is_i64, R, E, key_bits, n_waves, table,
                                                                   rank_buf);
    int rc = launch_status();
    if (rc) return rc;
    sort_scan_kernel<<<1, 1024, 0, stream>>>(table, n_waves, E, counts);
    rc = launch_status();
    if (rc || rank_buf == nullptr) return rc;
    sort_scatter_kernel<<<blocks, 256, 0, stream>>>(sel, is_i64, R, E, n_waves, table, sort_idx, rank_buf);
    return launch_status();
}

}  // namespace mfl
