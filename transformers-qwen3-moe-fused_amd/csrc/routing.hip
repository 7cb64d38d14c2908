// Token routing: fused softmax + top-k, and the stable counting sort of expert ids.
//
// Both are latency/bandwidth-bound integer-heavy kernels built from wavefront ballots,
// cross-lane shuffles and LDS histograms; neither uses atomics, so results are
// deterministic and the index outputs are reproducible bit for bit.
#include <mutex>

#include "common.h"
#include "ops.h"

namespace mfl {

namespace {

// ---------------------------------------------------------------- softmax + top-k

// Maximum over the 64 lanes of a wave, the same value in every lane: data-parallel-primitive moves
// inside the vector ALU (two quad permutes, two rotations inside each row of 16 lanes, two row
// broadcasts), then a read of lane 63.  A butterfly of six cross-lane shuffles goes through the
// LDS crossbar six times instead.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_max_step(float x) {
    const int xi = __builtin_bit_cast(int, x);
    // lanes that the move does not write keep x: max(x, x) = x
    const int yi = __builtin_amdgcn_update_dpp(xi, xi, CTRL, ROW_MASK, 0xf, false);
    return fmaxf(x, __builtin_bit_cast(float, yi));
}
__device__ __forceinline__ float wave_max_f32(float x) {
    x = dpp_max_step<0xb1, 0xf>(x);   // quad_perm [1,0,3,2]
    x = dpp_max_step<0x4e, 0xf>(x);   // quad_perm [2,3,0,1]
    x = dpp_max_step<0x124, 0xf>(x);  // row_ror 4
    x = dpp_max_step<0x128, 0xf>(x);  // row_ror 8: every lane holds the maximum of its row
    x = dpp_max_step<0x142, 0xa>(x);  // row_bcast 15: rows 1 and 3 take in rows 0 and 2
    x = dpp_max_step<0x143, 0xc>(x);  // row_bcast 31: rows 2 and 3 take in rows 0..1
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
}

// One wave per token.  Lane l holds experts l, l+64, l+128, ... (VPL of them).
template <typename TI, typename TC, int VPL>
__device__ __forceinline__ int topk_one_token(const TI *__restrict__ logits, int64_t t, int E, int k, int renorm,
                                               float *__restrict__ w_f32, TC *__restrict__ w_cast,
                                               int64_t *__restrict__ idx, int lane) {
    const TI *row = logits + t * E;

    float p[VPL];
    float mx = -INFINITY;
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
        const int e = lane + 64 * v;
        p[v] = e < E ? to_f32(row[e]) : -INFINITY;
        mx = fmaxf(mx, p[v]);
    }
    mx = wave_max_f32(mx);
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
        // the wave's best: the maximum, then its owner; several lanes with the same value (rare)
        // settle for the lowest expert id the slow way
        const float m = wave_max_f32(bp);
        const uint64_t owners = __ballot(bp == m);
        if (__popcll(owners) == 1) {
            bi = __builtin_amdgcn_readlane(bi, __ffsll((unsigned long long)owners) - 1);
        } else {
            if (bp != m) bi = 0x7fffffff;
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const int oi = __shfl_xor(bi, off);
                if (oi < bi) bi = oi;
            }
        }
        bp = m;
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
    return my_i;  // lanes below k: the lane's selection
}

template <typename TI, typename TC, int VPL>
__global__ __launch_bounds__(256) void softmax_topk_kernel(const TI *__restrict__ logits, int64_t T, int E, int k,
                                                           int renorm, float *__restrict__ w_f32,
                                                           TC *__restrict__ w_cast, int64_t *__restrict__ idx) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    topk_one_token<TI, TC, VPL>(logits, t, E, k, renorm, w_f32, w_cast, idx, lane);
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

// Gradient of the routing weights with respect to the logits: a wave per token recomputes the softmax, spreads the
// k incoming gradients over the selected experts and applies the softmax Jacobian:
//   renorm:  w_j = p_sel_j / s, s = sum_j p_sel_j   ->   dp_sel_j = (dw_j - sum_i dw_i w_i) / s
//   dlogits_e = p_e (dp_e - sum_j dp_sel_j p_sel_j),  dp_e = dp_sel_j where e is the j-th selection, else 0
// (the derivative of modular_qwen3_moe_fused.py:87-93 that autograd forms there from five tensor operations).
template <typename TI, typename TG, int VPL>
__global__ __launch_bounds__(256) void softmax_topk_bwd_kernel(const TI *__restrict__ logits, int64_t T, int E, int k,
                                                               int renorm, const int64_t *__restrict__ idx,
                                                               const float *__restrict__ w_f32,
                                                               const TG *__restrict__ dw, TI *__restrict__ dlogits) {
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
    mx = wave_max_f32(mx);
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
    for (int v = 0; v < VPL; ++v) p[v] = p[v] / sum;

    // lane j < k: the j-th selection, its probability, weight and incoming gradient
    const int my_i = lane < k ? (int)idx[t * k + lane] : 0;
    const float my_w = lane < k ? w_f32[t * k + lane] : 0.f;
    float my_g = lane < k ? to_f32(dw[t * k + lane]) : 0.f;
    float my_p = 0.f, s = 0.f;
    for (int j = 0; j < k; ++j) {
        const int ij = __builtin_amdgcn_readlane(my_i, j);
        float pv = 0.f;
#pragma unroll
        for (int v = 0; v < VPL; ++v)
            if ((ij >> 6) == v) pv = p[v];
        const float pj = __shfl(pv, ij & 63);
        if (lane == j) my_p = pj;
        s += pj;
    }
    if (renorm) {
        float c = my_g * my_w;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off);
        my_g = (my_g - c) / s;
    }
    float tsum = lane < k ? my_g * my_p : 0.f;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) tsum += __shfl_xor(tsum, off);
    float dp[VPL];
#pragma unroll
    for (int v = 0; v < VPL; ++v) dp[v] = 0.f;
    for (int j = 0; j < k; ++j) {
        const int ij = __builtin_amdgcn_readlane(my_i, j);
        const float gj = __shfl(my_g, j);
#pragma unroll
        for (int v = 0; v < VPL; ++v)
            if (ij == lane + 64 * v) dp[v] += gj;
    }
    TI *out = dlogits + t * E;
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
        const int e = lane + 64 * v;
        if (e < E) out[e] = from_f32<TI>(p[v] * (dp[v] - tsum));
    }
}

template <typename TI, typename TG>
int launch_topk_bwd(const void *logits, int64_t T, int E, int k, int renorm, const int64_t *idx, const float *w_f32,
                    const void *dw, void *dlogits, hipStream_t stream) {
    const unsigned grid = (unsigned)((T + 3) / 4);
    const int vpl = ceil_div(E, 64);
#define MFL_TOPKB(V)                                                                                          \
    softmax_topk_bwd_kernel<TI, TG, V><<<grid, 256, 0, stream>>>((const TI *)logits, T, E, k, renorm, idx, w_f32, \
                                                                 (const TG *)dw, (TI *)dlogits)
    if (vpl <= 1)
        MFL_TOPKB(1);
    else if (vpl <= 2)
        MFL_TOPKB(2);
    else if (vpl <= 4)
        MFL_TOPKB(4);
    else if (vpl <= 8)
        MFL_TOPKB(8);
    else if (vpl <= 16)
        MFL_TOPKB(16);
    else
        return MFL_ERR_UNSUPPORTED;
#undef MFL_TOPKB
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
constexpr int kSortChunk = 16;  // batches of 64 keys whose loads are issued together

__device__ __forceinline__ void wave_count(const void *sel, int is_i64, int E, int key_bits, int64_t seg_begin,
                                           int64_t seg_end, int *hist, int32_t *local_rank, int lane) {
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    for (int64_t chunk = seg_begin; chunk < seg_end; chunk += 64 * kSortChunk) {
        // all loads of the chunk first: their latencies overlap instead of adding up
        int keys[kSortChunk];
#pragma unroll
        for (int u = 0; u < kSortChunk; ++u) {
            const int64_t j = chunk + u * 64 + lane;
            int key = -1;
            if (j < seg_end) {
                const int64_t k64 = load_key(sel, is_i64, j);
                key = (k64 >= 0 && k64 < E) ? (int)k64 : -1;
            }
            keys[u] = key;
        }
#pragma unroll
        for (int u = 0; u < kSortChunk; ++u) {
            if (chunk + u * 64 >= seg_end) break;  // wave-uniform
            const int key = keys[u];
            const bool valid = key >= 0;
            uint64_t same = __ballot(valid);
            for (int b = 0; b < key_bits; ++b) {
                const uint64_t bal = __ballot((key >> b) & 1);
                same &= ((key >> b) & 1) ? bal : ~bal;
            }
            if (valid) {
                const int before = hist[key];
                const int rank = before + __popcll(same & lt_mask);
                if (local_rank) local_rank[chunk + u * 64 + lane] = rank;
                // the last lane of each key group publishes the new running count
                if ((same >> lane) == 1ull) hist[key] = before + __popcll(same);
            }
        }
    }
}

// Phase 3 for one wave: final position = rank within the wave's segment + global offset of
// (wave, key); writes inv_sort_idx in place of the rank and scatters sort_idx.
__device__ __forceinline__ void wave_scatter(const void *sel, int is_i64, int E, int64_t seg_begin, int64_t seg_end,
                                             const int *offsets, const int *offsets2, int32_t *sort_idx,
                                             int32_t *rank_io, int lane) {
    for (int64_t chunk = seg_begin; chunk < seg_end; chunk += 64 * kSortChunk) {
        int keys[kSortChunk], ranks[kSortChunk];
#pragma unroll
        for (int u = 0; u < kSortChunk; ++u) {
            const int64_t j = chunk + u * 64 + lane;
            int key = -1, rank = 0;
            if (j < seg_end) {
                const int64_t k64 = load_key(sel, is_i64, j);
                key = (k64 >= 0 && k64 < E) ? (int)k64 : -1;
                rank = rank_io[j];
            }
            keys[u] = key;
            ranks[u] = rank;
        }
#pragma unroll
        for (int u = 0; u < kSortChunk; ++u) {
            const int64_t j = chunk + u * 64 + lane;
            if (keys[u] >= 0) {
                const int pos = ranks[u] + offsets[keys[u]] + (offsets2 ? offsets2[keys[u]] : 0);
                rank_io[j] = pos;
                if (sort_idx) sort_idx[pos] = (int32_t)j;
            }
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

// Whole sort in one workgroup (n_waves <= 16): the (wave, expert) table lives in LDS
// (lds: [n_waves][E] table, then [E] totals).
__device__ __forceinline__ void sort_single_body(const void *__restrict__ sel, int is_i64, int64_t R, int E,
                                                 int key_bits, int32_t *__restrict__ counts,
                                                 int32_t *__restrict__ sort_idx, int32_t *__restrict__ inv_sort_idx,
                                                 int *lds) {
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
    wave_scatter(sel, is_i64, E, sb, se, table + wave * E, totals, sort_idx, inv_sort_idx, lane);
}

__global__ __launch_bounds__(1024) void sort_single_kernel(const void *__restrict__ sel, int is_i64, int64_t R,
                                                           int E, int key_bits, int32_t *__restrict__ counts,
                                                           int32_t *__restrict__ sort_idx,
                                                           int32_t *__restrict__ inv_sort_idx) {
    extern __shared__ int lds[];
    sort_single_body(sel, is_i64, R, E, key_bits, counts, sort_idx, inv_sort_idx, lds);
}

// Decode-sized batches: softmax + top-k of every token and the stable expert sort of the T * k
// selections in ONE launch of one workgroup (three launches otherwise, each a few microseconds of
// work): the waves take the tokens round robin, then sort what they wrote.
template <typename TI, typename TC, int VPL>
__global__ __launch_bounds__(1024) void route_sort_small_kernel(const TI *__restrict__ logits, int64_t T, int E,
                                                                int k, int renorm, float *__restrict__ w_f32,
                                                                TC *__restrict__ w_cast, int64_t *__restrict__ idx,
                                                                int key_bits, int32_t *__restrict__ counts,
                                                                int32_t *__restrict__ sort_idx,
                                                                int32_t *__restrict__ inv_sort_idx) {
    extern __shared__ int lds[];
    const int lane = threadIdx.x & 63, n_waves = blockDim.x >> 6;
    for (int64_t t = threadIdx.x >> 6; t < T; t += n_waves)
        topk_one_token<TI, TC, VPL>(logits, t, E, k, renorm, w_f32, w_cast, idx, lane);
    __threadfence();  // the selections are read back from memory by other waves of the workgroup
    __syncthreads();
    sort_single_body(idx, 1, T * k, E, key_bits, counts, sort_idx, inv_sort_idx, lds);
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
    wave_scatter(sel, is_i64, E, sb, se, table + (int64_t)wave * E, nullptr, sort_idx, inv_sort_idx, lane);
}

// ---- two-kernel sort (E <= 512) ------------------------------------------------------------
//
// Many short segments (256 keys per wave) instead of a few long ones: the ballot ranking of a
// batch depends on the LDS histogram left by the batch before it, so a wave is a serial chain
// and the parallelism has to come from the number of waves.  Workgroups of 16 waves.
//   kernel 1: every wave counts its segment; the workgroup turns its 16 histograms into
//             exclusive prefixes over its waves (table[wave][e]) and a workgroup total
//             (wg_tot[block][e]).
//   kernel 2: a workgroup reads the (small) wg_tot table, derives the global offset of each of
//             its (wave, expert) pairs -- experts before e, workgroups before it, waves before
//             it -- then ranks its keys again (cheaper than a round trip of the ranks through
//             memory) and scatters.  Workgroup 0 also writes the counts.

constexpr int kFastBatches = 4;   // 64-key batches per chunk: 256 keys
constexpr int kFastWaves = 16;    // waves per workgroup
constexpr int kFastMaxBlocks = 64;

template <int NBATCH>
__device__ __forceinline__ void wave_rank_chunk(const void *sel, int is_i64, int E, int key_bits, int64_t begin,
                                                int64_t seg_end, int *hist, int (&keys)[NBATCH],
                                                int (&ranks)[NBATCH], int lane) {
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
    for (int u = 0; u < NBATCH; ++u) {
        const int64_t j = begin + u * 64 + lane;
        int key = -1;
        if (j < seg_end) {
            const int64_t k64 = load_key(sel, is_i64, j);
            key = (k64 >= 0 && k64 < E) ? (int)k64 : -1;
        }
        keys[u] = key;
    }
#pragma unroll
    for (int u = 0; u < NBATCH; ++u) {
        const int key = keys[u];
        const bool valid = key >= 0;
        uint64_t same = __ballot(valid);
        for (int b = 0; b < key_bits; ++b) {
            const uint64_t bal = __ballot((key >> b) & 1);
            same &= ((key >> b) & 1) ? bal : ~bal;
        }
        int rank = 0;
        if (valid) {
            const int before = hist[key];
            rank = before + __popcll(same & lt_mask);
            if ((same >> lane) == 1ull) hist[key] = before + __popcll(same);
        }
        ranks[u] = rank;
    }
}

__global__ __launch_bounds__(1024) void fast_count_kernel(const void *__restrict__ sel, int is_i64, int64_t R, int E,
                                                          int key_bits, int n_waves, int32_t *__restrict__ table,
                                                          int32_t *__restrict__ wg_tot) {
    extern __shared__ int lds[];  // [16][E]
    const int wib = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int wave = blockIdx.x * kFastWaves + wib;
    int *hist = lds + wib * E;
    for (int i = lane; i < E; i += 64) hist[i] = 0;
    if (wave < n_waves) {
        int64_t sb, se;
        segment_of(wave, n_waves, R, sb, se);
        for (int64_t c = sb; c < se; c += 64 * kFastBatches) {
            int keys[kFastBatches], ranks[kFastBatches];
            wave_rank_chunk<kFastBatches>(sel, is_i64, E, key_bits, c, se, hist, keys, ranks, lane);
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        int run = 0;
#pragma unroll
        for (int w = 0; w < kFastWaves; ++w) {
            const int cnt = lds[w * E + e];
            lds[w * E + e] = run;
            run += cnt;
        }
        wg_tot[blockIdx.x * E + e] = run;
    }
    __syncthreads();
    if (wave < n_waves)
        for (int i = lane; i < E; i += 64) table[(int64_t)wave * E + i] = hist[i];
}

__global__ __launch_bounds__(1024) void fast_scatter_kernel(const void *__restrict__ sel, int is_i64, int64_t R,
                                                            int E, int key_bits, int n_waves, int n_blocks,
                                                            const int32_t *__restrict__ table,
                                                            const int32_t *__restrict__ wg_tot,
                                                            int32_t *__restrict__ counts,
                                                            int32_t *__restrict__ sort_idx,
                                                            int32_t *__restrict__ inv_sort_idx) {
    extern __shared__ int lds[];  // base [E], offsets [16][E], histograms [16][E]
    int *base = lds;
    int *offs = base + E;
    int *hists = offs + kFastWaves * E;
    const int tid = threadIdx.x, wib = tid >> 6, lane = tid & 63;
    // base[e] = rows of experts before e + rows of e in workgroups before this one
    for (int e = tid; e < E; e += blockDim.x) {
        int total = 0, before = 0;
        for (int blk = 0; blk < n_blocks; ++blk) {
            const int v = wg_tot[blk * E + e];
            if (blk < (int)blockIdx.x) before += v;
            total += v;
        }
        base[e] = total;
        offs[e] = before;  // parked in the first offsets row until the scan is done
        if (blockIdx.x == 0) counts[e] = total;
    }
    __syncthreads();
    if (sort_idx == nullptr && inv_sort_idx == nullptr) return;
    if (wib == 0) {  // exclusive scan of the totals over the experts, plus the workgroup part
        int carry = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            const int v = e < E ? base[e] : 0;
            int inc = v;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int up = __shfl_up(inc, o);
                if (lane >= o) inc += up;
            }
            if (e < E) base[e] = carry + inc - v + offs[e];
            carry += __shfl(inc, 63);
        }
    }
    __syncthreads();
    const int wave = blockIdx.x * kFastWaves + wib;
    if (wave >= n_waves) return;
    int *hist = hists + wib * E;
    int *my_off = offs + wib * E;
    for (int i = lane; i < E; i += 64) {
        hist[i] = 0;
        my_off[i] = base[i] + table[(int64_t)wave * E + i];
    }
    int64_t sb, se;
    segment_of(wave, n_waves, R, sb, se);
    for (int64_t c = sb; c < se; c += 64 * kFastBatches) {
        int keys[kFastBatches], ranks[kFastBatches];
        wave_rank_chunk<kFastBatches>(sel, is_i64, E, key_bits, c, se, hist, keys, ranks, lane);
#pragma unroll
        for (int u = 0; u < kFastBatches; ++u) {
            if (keys[u] < 0) continue;
            const int64_t j = c + u * 64 + lane;
            const int pos = ranks[u] + my_off[keys[u]];
            if (inv_sort_idx) inv_sort_idx[j] = pos;
            if (sort_idx) sort_idx[pos] = (int32_t)j;
        }
    }
}

// ---- routing in two launches: softmax + top-k that also counts, then the scatter
// route_count_kernel: one workgroup per segment of tokens_per_seg tokens (at most 256 selections, the
// segment one wave of the scatter kernel ranks), one wave per token (in turn, where a segment has more
// tokens than the workgroup has waves).  Besides the routing weights and the selections it leaves the
// segment's histogram of experts in table_raw[segment][E] (LDS atomics on integers: the sums do not depend
// on their order).
template <typename TI, typename TC, int VPL>
__global__ __launch_bounds__(1024) void route_count_kernel(const TI *__restrict__ logits, int64_t T, int E, int k,
                                                           int renorm, float *__restrict__ w_f32,
                                                           TC *__restrict__ w_cast, int64_t *__restrict__ idx,
                                                           int tokens_per_seg, int32_t *__restrict__ table_raw) {
    extern __shared__ int lds[];  // [E]
    const int wib = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < E; i += blockDim.x) lds[i] = 0;
    __syncthreads();
    for (int tt = wib; tt < tokens_per_seg; tt += kFastWaves) {
        const int64_t t = (int64_t)blockIdx.x * tokens_per_seg + tt;
        if (t >= T) break;
        const int sel = topk_one_token<TI, TC, VPL>(logits, t, E, k, renorm, w_f32, w_cast, idx, lane);
        // a row of NaN (or of -inf throughout) selects nothing: its lanes keep the "no expert" id, which the
        // scatter pass skips like any key outside [0, E); it must not reach the histogram either
        if (lane < k && (unsigned)sel < (unsigned)E) atomicAdd(&lds[sel], 1);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < E; i += blockDim.x) table_raw[(int64_t)blockIdx.x * E + i] = lds[i];
}

// fast_scatter_kernel on the raw histograms of route_count_kernel: wave w of the launch ranks segment w
// (seg_keys selections, at most 256).  Everything the workgroup needs from global memory is requested at the
// start, in one go: its waves' selections, the n_segs raw histograms (for the totals per expert and the rows
// in earlier workgroups, which fast_count_kernel would have left in its tables) and, once more, the 16
// histograms of its own segments; what follows works in LDS.
__global__ __launch_bounds__(1024) void route_scatter_kernel(const int64_t *__restrict__ sel, int64_t R, int E,
                                                             int key_bits, int seg_keys, int n_segs,
                                                             const int32_t *__restrict__ table_raw,
                                                             int32_t *__restrict__ counts,
                                                             int32_t *__restrict__ sort_idx,
                                                             int32_t *__restrict__ inv_sort_idx) {
    extern __shared__ int lds[];  // base [E], before [E], offsets [16][E], histograms [16][E]
    int *base = lds;
    int *befo = base + E;
    int *offs = befo + E;
    int *hists = offs + kFastWaves * E;
    const int tid = threadIdx.x, wib = tid >> 6, lane = tid & 63;
    const int seg = blockIdx.x * kFastWaves + wib;
    const int first_seg = blockIdx.x * kFastWaves;
    const int64_t sb = (int64_t)seg * seg_keys;
    int64_t se = sb + seg_keys;
    if (se > R) se = R;
    int keys[kFastBatches];
#pragma unroll
    for (int u = 0; u < kFastBatches; ++u) {
        const int64_t j = sb + u * 64 + lane;
        int key = -1;
        if (seg < n_segs && j < se) {
            const int64_t k64 = sel[j];
            key = (k64 >= 0 && k64 < E) ? (int)k64 : -1;
        }
        keys[u] = key;
    }
    // the raw histograms of this workgroup's segments
    for (int i = tid; i < kFastWaves * E; i += blockDim.x) {
        const int w = i / E;
        offs[i] = first_seg + w < n_segs ? table_raw[(int64_t)first_seg * E + i] : 0;
    }
    // Totals and rows in earlier workgroups, per expert: column sums of the n_segs x E table.  The threads
    // split the rows among them, load eight rows at a time before they add any (a loop of load-then-add
    // pays the L2 latency once per row: 15 us for 256 rows) and meet in LDS (integer atomics).
    for (int e = tid; e < 2 * E; e += blockDim.x) base[e] = 0;  // base and befo
    __syncthreads();
    if ((E & 3) == 0) {
        const int EV = E >> 2, rpp = blockDim.x / EV;
        const int r0 = tid / EV, c = tid - r0 * EV;
        if (r0 < rpp) {
            const int4 *t4 = (const int4 *)table_raw;
            int4 total = {0, 0, 0, 0}, before = {0, 0, 0, 0};
            for (int s0 = r0; s0 < n_segs; s0 += 8 * rpp) {
                int4 v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int sgm = s0 + u * rpp;
                    v[u] = sgm < n_segs ? t4[(int64_t)sgm * EV + c] : int4{0, 0, 0, 0};
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    total.x += v[u].x, total.y += v[u].y, total.z += v[u].z, total.w += v[u].w;
                    if (s0 + u * rpp < first_seg)
                        before.x += v[u].x, before.y += v[u].y, before.z += v[u].z, before.w += v[u].w;
                }
            }
            atomicAdd(&base[4 * c + 0], total.x), atomicAdd(&base[4 * c + 1], total.y);
            atomicAdd(&base[4 * c + 2], total.z), atomicAdd(&base[4 * c + 3], total.w);
            if (first_seg > 0) {
                atomicAdd(&befo[4 * c + 0], before.x), atomicAdd(&befo[4 * c + 1], before.y);
                atomicAdd(&befo[4 * c + 2], before.z), atomicAdd(&befo[4 * c + 3], before.w);
            }
        }
    } else {
        const int rpp = blockDim.x / E;
        const int r0 = tid / E, e = tid - r0 * E;
        if (r0 < rpp) {
            int total = 0, before = 0;
            for (int s0 = r0; s0 < n_segs; s0 += 8 * rpp) {
                int v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int sgm = s0 + u * rpp;
                    v[u] = sgm < n_segs ? table_raw[(int64_t)sgm * E + e] : 0;
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    total += v[u];
                    if (s0 + u * rpp < first_seg) before += v[u];
                }
            }
            atomicAdd(&base[e], total);
            if (first_seg > 0) atomicAdd(&befo[e], before);
        }
    }
    __syncthreads();
    if (blockIdx.x == 0)
        for (int e = tid; e < E; e += blockDim.x) counts[e] = base[e];
    if (sort_idx == nullptr && inv_sort_idx == nullptr) return;
    if (wib == 0) {  // exclusive scan of the totals over the experts, plus the part of earlier workgroups
        int carry = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            const int v = e < E ? base[e] : 0;
            int inc = v;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int up = __shfl_up(inc, o);
                if (lane >= o) inc += up;
            }
            if (e < E) befo[e] = carry + inc - v + befo[e];  // base stays: workgroup 0 may still be copying it to counts
            carry += __shfl(inc, 63);
        }
    }
    int *hist = hists + wib * E;
    for (int i = lane; i < E; i += 64) hist[i] = 0;
    __syncthreads();
    // offsets of this workgroup's waves: first row of the expert, plus its rows in the workgroup's earlier segments
    for (int e = tid; e < E; e += blockDim.x) {
        int run = befo[e];
#pragma unroll
        for (int w = 0; w < kFastWaves; ++w) {
            const int c = offs[w * E + e];
            offs[w * E + e] = run;
            run += c;
        }
    }
    __syncthreads();
    if (seg >= n_segs) return;
    const int *my_off = offs + wib * E;
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
    for (int u = 0; u < kFastBatches; ++u) {
        const int key = keys[u];
        const bool valid = key >= 0;
        uint64_t same = __ballot(valid);
        if (same == 0) continue;  // past the end of the segment
        for (int b = 0; b < key_bits; ++b) {
            const uint64_t bal = __ballot((key >> b) & 1);
            same &= ((key >> b) & 1) ? bal : ~bal;
        }
        if (valid) {
            const int before = hist[key];
            const int pos = before + __popcll(same & lt_mask) + my_off[key];
            if ((same >> lane) == 1ull) hist[key] = before + __popcll(same);
            const int64_t j = sb + u * 64 + lane;
            if (inv_sort_idx) inv_sort_idx[j] = pos;
            if (sort_idx) sort_idx[pos] = (int32_t)j;
        }
    }
}

inline int fast_waves(int64_t R) {
    int64_t w = (R + 64 * kFastBatches - 1) / (64 * kFastBatches);
    if (w > kFastMaxBlocks * kFastWaves) w = kFastMaxBlocks * kFastWaves;
    if (w < 1) w = 1;
    return (int)w;
}

inline bool fast_sort_ok(int E) { return E <= 512; }  // (2 * 16 + 1) * E ints of LDS

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

int route_softmax_topk_bwd(const void *logits, int logits_dtype, int64_t T, int E, int k, int renorm, const int64_t *idx,
                           const float *w_f32, const void *dw, int dw_dtype, void *dlogits, hipStream_t stream) {
    if (T == 0) return MFL_OK;
    int rc = MFL_ERR_DTYPE;
    MFL_DISPATCH_FLOAT(logits_dtype, TI, MFL_DISPATCH_FLOAT(dw_dtype, TG, rc = (launch_topk_bwd<TI, TG>(
        logits, T, E, k, renorm, idx, w_f32, dw, dlogits, stream))));
    return rc;
}

namespace {

template <typename TI, typename TC>
int launch_route_sort_small(const void *logits, int64_t T, int E, int k, int renorm, float *w_f32, void *w_cast,
                            int64_t *idx, int32_t *counts, int32_t *sort_idx, int32_t *inv_sort_idx,
                            hipStream_t stream) {
    int key_bits = 0;
    while ((1 << key_bits) < E) ++key_bits;
    const int n_waves = 16;
    const size_t lds = (size_t)(n_waves + 1) * E * 4;
    const int vpl = ceil_div(E, 64);
#define MFL_RS(V)                                                                                              \
    route_sort_small_kernel<TI, TC, V><<<1, n_waves * 64, lds, stream>>>(                                      \
        (const TI *)logits, T, E, k, renorm, w_f32, (TC *)w_cast, idx, key_bits, counts, sort_idx, inv_sort_idx)
    if (vpl <= 1)
        MFL_RS(1);
    else if (vpl <= 2)
        MFL_RS(2);
    else if (vpl <= 4)
        MFL_RS(4);
    else
        MFL_RS(8);
#undef MFL_RS
    return launch_status();
}

}  // namespace

int route_sort_small(const void *logits, int logits_dtype, int64_t T, int E, int k, int renorm, float *w_f32,
                     void *w_cast, int cast_dtype, int64_t *idx, int32_t *counts, int32_t *sort_idx,
                     int32_t *inv_sort_idx, hipStream_t stream) {
    // one workgroup does everything: worth it only while the tokens are few
    if (T > 128 || T * k > 8192 || E > 512 || inv_sort_idx == nullptr || sort_idx == nullptr)
        return MFL_ERR_UNSUPPORTED;
    if (T == 0) return MFL_ERR_UNSUPPORTED;  // the separate entry points define the empty case
    int rc = MFL_OK;
    MFL_DISPATCH_FLOAT(logits_dtype, TI, MFL_DISPATCH_FLOAT(cast_dtype, TC, rc = (launch_route_sort_small<TI, TC>(
        logits, T, E, k, renorm, w_f32, w_cast, idx, counts, sort_idx, inv_sort_idx, stream))));
    return rc;
}

namespace {

// Segments of the two-launch routing: whole tokens, at most 256 selections; a token per wave of the top-k
// workgroup (16) while that keeps the segments under 1024, more tokens per segment beyond.  0: does not apply.
inline int route_tokens_per_seg(int64_t T, int E, int k) {
    if (T <= 0 || E > 512 || k > 64 || T * k > 0x7fffffff) return 0;
    const int most = 256 / k;  // k <= 64
    int64_t tps = (T + kFastMaxBlocks * kFastWaves - 1) / (kFastMaxBlocks * kFastWaves);
    if (tps < kFastWaves) tps = kFastWaves;
    if (tps > most) tps = most;
    return (T + tps - 1) / tps <= kFastMaxBlocks * kFastWaves ? (int)tps : 0;
}

template <typename TI, typename TC>
int launch_route_count(const void *logits, int64_t T, int E, int k, int renorm, float *w_f32, void *w_cast,
                       int64_t *idx, int tps, int n_segs, int32_t *table_raw, hipStream_t stream) {
    const int vpl = ceil_div(E, 64);
    const size_t lds = (size_t)E * 4;
#define MFL_RC(V)                                                                                         \
    route_count_kernel<TI, TC, V><<<n_segs, kFastWaves * 64, lds, stream>>>(                              \
        (const TI *)logits, T, E, k, renorm, w_f32, (TC *)w_cast, idx, tps, table_raw)
    if (vpl <= 1)
        MFL_RC(1);
    else if (vpl <= 2)
        MFL_RC(2);
    else if (vpl <= 4)
        MFL_RC(4);
    else
        MFL_RC(8);
#undef MFL_RC
    return launch_status();
}

}  // namespace

size_t route_sort_workspace(int64_t T, int E, int k) {
    if (const int tps = route_tokens_per_seg(T, E, k)) {
        return (((size_t)((T + tps - 1) / tps) * (size_t)E * 4) + 255) / 256 * 256;
    }
    return expert_sort_workspace(T * k, E);
}

int route_sort(const void *logits, int logits_dtype, int64_t T, int E, int k, int renorm, float *w_f32, void *w_cast,
               int cast_dtype, int64_t *idx, int32_t *counts, int32_t *sort_idx, int32_t *inv_sort_idx,
               void *workspace, size_t ws_bytes, hipStream_t stream) {
    // up to 64 tokens one workgroup does it all in one launch (above, its single workgroup is the slower way)
    int rc = T <= 64 ? route_sort_small(logits, logits_dtype, T, E, k, renorm, w_f32, w_cast, cast_dtype, idx, counts,
                                        sort_idx, inv_sort_idx, stream)
                     : MFL_ERR_UNSUPPORTED;
    if (rc != MFL_ERR_UNSUPPORTED) return rc;
    const int tps = route_tokens_per_seg(T, E, k);
    if (tps == 0) {
        rc = route_softmax_topk(logits, logits_dtype, T, E, k, renorm, w_f32, w_cast, cast_dtype, idx, stream);
        if (rc) return rc;
        return expert_sort(idx, 1, T * k, E, counts, sort_idx, inv_sort_idx, workspace, ws_bytes, stream);
    }
    const int n_segs = (int)((T + tps - 1) / tps);
    if (workspace == nullptr || ws_bytes < (size_t)n_segs * E * 4) return MFL_ERR_WORKSPACE;
    int32_t *table_raw = (int32_t *)workspace;
    rc = MFL_ERR_DTYPE;
    MFL_DISPATCH_FLOAT(logits_dtype, TI, MFL_DISPATCH_FLOAT(cast_dtype, TC, rc = (launch_route_count<TI, TC>(
        logits, T, E, k, renorm, w_f32, w_cast, idx, tps, n_segs, table_raw, stream))));
    if (rc) return rc;
    int key_bits = 0;
    while ((1 << key_bits) < E) ++key_bits;
    static PerDeviceOnce attr;
    const hipError_t e = attr.run([] {
        return hipFuncSetAttribute((const void *)route_scatter_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   34 * 512 * 4);
    });
    if (e != hipSuccess) return (int)e;
    const size_t lds2 = (size_t)(2 * kFastWaves + 2) * E * 4;
    route_scatter_kernel<<<ceil_div(n_segs, kFastWaves), kFastWaves * 64, lds2, stream>>>(
        idx, T * k, E, key_bits, tps * k, n_segs, table_raw, counts, sort_idx, inv_sort_idx);
    return launch_status();
}

size_t expert_sort_workspace(int64_t R, int E) {
    if (fast_sort_ok(E)) {
        const int n_waves = fast_waves(R);
        return ((size_t)(n_waves + ceil_div(n_waves, kFastWaves)) * (size_t)E * 4 + 255) / 256 * 256;
    }
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
    if (fast_sort_ok(E)) {
        const int n_waves = fast_waves(R);
        const int n_blocks = ceil_div(n_waves, kFastWaves);
        if (workspace == nullptr || ws_bytes < (size_t)(n_waves + n_blocks) * E * 4) return MFL_ERR_WORKSPACE;
        int32_t *table = (int32_t *)workspace;
        int32_t *wg_tot = table + (size_t)n_waves * E;
        const size_t lds1 = (size_t)kFastWaves * E * 4, lds2 = (size_t)(2 * kFastWaves + 1) * E * 4;
        static PerDeviceOnce attr;
        const hipError_t e = attr.run([] {
            return hipFuncSetAttribute((const void *)fast_scatter_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       33 * 512 * 4);
        });
        if (e != hipSuccess) return (int)e;
        fast_count_kernel<<<n_blocks, kFastWaves * 64, lds1, stream>>>(sel, is_i64, R, E, key_bits, n_waves, table,
                                                                       wg_tot);
        int rc = launch_status();
        if (rc) return rc;
        fast_scatter_kernel<<<n_blocks, kFastWaves * 64, lds2, stream>>>(sel, is_i64, R, E, key_bits, n_waves,
                                                                         n_blocks, table, wg_tot, counts, sort_idx,
                                                                         inv_sort_idx);
        return launch_status();
    }
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

// ---- expert sort that allocates nothing ----------------------------------------------------
//
// The tables of the two-kernel sort (per-wave histograms and per-workgroup totals) live in a
// file-scope device array instead of a caller-supplied workspace.  The array's name is a host-side
// stand-in, not a device address: its address on the current device is looked up once per device
// with hipGetSymbolAddress and kept; kernels get that pointer as an argument, like a workspace.
// Every call on a device shares that device's array: calls that overlap in time on one device race
// (calls on one stream are ordered and safe).  Nothing needs clearing between calls: the count
// kernel writes every table entry that the scatter kernel reads.
namespace {

constexpr size_t kStaticSortBytes =
    (size_t)(kFastMaxBlocks * kFastWaves + kFastMaxBlocks) * 512 * sizeof(int32_t);  // 2 228 224 bytes
static __device__ __align__(256) unsigned char scratch[kStaticSortBytes];

constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;

}  // namespace

int expert_sort_static(const void *sel, int is_i64, int64_t R, int E, int32_t *counts, int32_t *sort_idx,
                       int32_t *inv_sort_idx, hipStream_t stream) {
    if (!fast_sort_ok(E)) return MFL_ERR_LIMIT;  // the tables of more experts do not fit the fixed array
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return MFL_ERR_LIMIT;
    void *ptr;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (g_scratch_ptr[dev] == nullptr) {
            void *p = nullptr;
            e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
            if (e != hipSuccess) return (int)e;
            if (p == nullptr) return (int)hipErrorInvalidSymbol;
            g_scratch_ptr[dev] = p;
        }
        ptr = g_scratch_ptr[dev];
    }
    return expert_sort(sel, is_i64, R, E, counts, sort_idx, inv_sort_idx, ptr, kStaticSortBytes, stream);
}

}  // namespace mfl
