// bf16 grouped GEMM on the CDNA4 matrix cores (v_mfma_f32_32x32x16_bf16), fp32 accumulate.
//
// One kernel template covers the three products of the moe_fused_linear path.  With
// C[i, j] = sum_r A(i, r) * B(j, r):
//
//   MODE_FWD : i = row m, j = out feature n, r = in feature k
//              A = x  (R,K)   reduction-contiguous     B = w[e] (N,K) reduction-contiguous
//   MODE_DX  : i = row m, j = in feature n,  r = out feature k
//              A = dy (R,K)   reduction-contiguous     B = w[e] (K,N) reduction-strided
//   MODE_DW  : i = out feature n, j = in feature k, r = row m of expert e
//              A = dy (R,N)   reduction-strided        B = x  (R,K)   reduction-strided
//
// A reduction-contiguous operand tile sits in LDS as [i][BK + 8] and is read as MFMA
// fragments with one 128-bit LDS read per lane.  A reduction-strided tile sits in LDS the
// way it lies in memory, [r][BI + 32], and is read with ds_read_b64_tr_b16, which hands
// each lane four consecutive r for its own i: the transpose costs no extra pass.
//
// Scheduling.  Rows per expert are only known on the device, so the grid is an upper bound
// on the number of tiles; every wave derives (expert, tile) for its workgroup from m_sizes
// with a shuffle scan and surplus workgroups exit.  Workgroup b runs on XCD b % 8, so
// logical tiles are dealt out in eight contiguous runs: the tiles of one expert (which
// share its weight matrix and its rows) land on one XCD and meet in that XCD's L2.
#include "common.h"
#include "gemm.h"

namespace mfl {

namespace {

constexpr int kPadRC = 8;   // elements of padding after a reduction-contiguous LDS row
constexpr int kPadRS = 32;  // elements of padding after a reduction-strided LDS row
constexpr int kXcd = 8;

typedef __attribute__((address_space(3))) short4_t *lds_short4_ptr;

template <int BI, int BK, bool RC>
struct TileLayout {
    static constexpr int kRowElems = RC ? (BK + kPadRC) : (BI + kPadRS);
    static constexpr int kRows = RC ? BI : BK;
    static constexpr int kBytes = kRows * kRowElems * 2;
    static constexpr int kChunks = BI * BK / 8;  // 16-byte chunks in the tile
};

// Global -> registers for one operand tile.  Chunks outside [i0, i_end) x [r0, r_end) read
// as zero.  ld is the stride (in elements) between consecutive rows of the 2-D view.
template <int BI, int BK, bool RC, int NT>
__device__ __forceinline__ void load_stage(uint4_t (&stage)[BI * BK / 8 / NT], const bf16_t *base, int64_t ld,
                                           int i0, int i_end, int r0, int r_end, int tid) {
    constexpr int CPT = BI * BK / 8 / NT;
#pragma unroll
    for (int u = 0; u < CPT; ++u) {
        const int c = tid + NT * u;
        uint4_t v = {0u, 0u, 0u, 0u};
        if (RC) {
            const int row = c / (BK / 8), kc = c % (BK / 8);
            const int i = i0 + row, r = r0 + kc * 8;
            if (i < i_end && r < r_end) v = *(const uint4_t *)(base + (int64_t)i * ld + r);
        } else {
            const int row = c / (BI / 8), ic = c % (BI / 8);
            const int r = r0 + row, i = i0 + ic * 8;
            if (r < r_end && i < i_end) v = *(const uint4_t *)(base + (int64_t)r * ld + i);
        }
        stage[u] = v;
    }
}

template <int BI, int BK, bool RC, int NT>
__device__ __forceinline__ void store_stage(const uint4_t (&stage)[BI * BK / 8 / NT], unsigned char *lds, int tid) {
    constexpr int CPT = BI * BK / 8 / NT;
    constexpr int ROW = TileLayout<BI, BK, RC>::kRowElems;
#pragma unroll
    for (int u = 0; u < CPT; ++u) {
        const int c = tid + NT * u;
        int off;
        if (RC) {
            const int row = c / (BK / 8), kc = c % (BK / 8);
            off = (row * ROW + kc * 8) * 2;
        } else {
            const int row = c / (BI / 8), ic = c % (BI / 8);
            off = (row * ROW + ic * 8) * 2;
        }
        *(uint4_t *)(lds + off) = stage[u];
    }
}

// NF4 weight tile (forward only): each 16-byte LDS chunk of 8 weights comes from 4 packed
// bytes and one absmax.  Element 2i sits in the high nibble of byte i, 2i+1 in the low one.
struct Nf4Args {
    const float *code16;
    const float *absmax;
    int bs_shift;
};

template <int BN, int BK, int NT>
__device__ __forceinline__ void load_stage_nf4(uint32_t (&q)[BN * BK / 8 / NT], float (&am)[BN * BK / 8 / NT],
                                               const uint8_t *wq, const float *absmax, int bs_shift,
                                               int64_t elem_base, int K, int j0, int j_end, int r0, int r_end,
                                               int tid) {
    constexpr int CPT = BN * BK / 8 / NT;
#pragma unroll
    for (int u = 0; u < CPT; ++u) {
        const int c = tid + NT * u;
        const int row = c / (BK / 8), kc = c % (BK / 8);
        const int n = j0 + row, k = r0 + kc * 8;
        uint32_t word = 0x77777777u;  // code entry 7 is 0.0
        float a = 0.f;
        if (n < j_end && k < r_end) {
            const int64_t idx = elem_base + (int64_t)n * K + k;
            word = *(const uint32_t *)(wq + (idx >> 1));
            a = absmax[idx >> bs_shift];
        }
        q[u] = word;
        am[u] = a;
    }
}

template <int BN, int BK, int NT>
__device__ __forceinline__ void store_stage_nf4(const uint32_t (&q)[BN * BK / 8 / NT],
                                                const float (&am)[BN * BK / 8 / NT], const float *code,
                                                unsigned char *lds, int tid) {
    constexpr int CPT = BN * BK / 8 / NT;
    constexpr int ROW = TileLayout<BN, BK, true>::kRowElems;
#pragma unroll
    for (int u = 0; u < CPT; ++u) {
        const int c = tid + NT * u;
        const int row = c / (BK / 8), kc = c % (BK / 8);
        bf16x8 v;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t nib = (q[u] >> (8 * (j >> 1) + ((j & 1) ? 0 : 4))) & 15u;
            v[j] = (bf16_t)(code[nib] * am[u]);
        }
        *(bf16x8 *)(lds + (row * ROW + kc * 8) * 2) = v;
    }
}

// MFMA operand fragment for the 32 (i) x 16 (r) block at (ib, ks*16): lane l gets
// i = ib + l % 32 and r = ks*16 + 8*(l/32) .. +7.
template <int BI, int BK, bool RC>
__device__ __forceinline__ bf16x8 load_frag(const unsigned char *lds, int ib, int ks, int lane) {
    constexpr int ROW = TileLayout<BI, BK, RC>::kRowElems;
    if (RC) {
        const int off = ((ib + (lane & 31)) * ROW + ks * 16 + 8 * (lane >> 5)) * 2;
        return *(const bf16x8 *)(lds + off);
    } else {
        // Transposing read: in each group of 16 lanes, lanes 4q..4q+3 address row q (16
        // consecutive i, four per lane) and lane t receives column t of rows 0..3.
        const int g = lane >> 4, il = lane & 15;
        const int r = ks * 16 + 8 * (g >> 1) + (il >> 2);
        const int i = ib + 16 * (g & 1) + 4 * (il & 3);
        const int off = (r * ROW + i) * 2;
        const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(lds + off));
        const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(lds + off + 4 * ROW * 2));
        union {
            short4_t h[2];
            bf16x8 v;
        } u;
        u.h[0] = lo;
        u.h[1] = hi;
        return u.v;
    }
}

struct TileCoord {
    int expert;
    int i0, i_end;  // rows of C covered / valid bound
    int j0;
    int r_begin, r_end;
    bool valid;
};

// (expert, m-tile, n-tile) of logical tile L for the row-grouped modes.  Every wave runs
// this redundantly (no LDS, no barrier): 64 experts per step, shuffle prefix sums.
template <int BM>
__device__ __forceinline__ TileCoord find_tile_rows(const void *m_sizes, int ms_i64, int E, int n_tiles_n,
                                                    int64_t R, int lane) {
    TileCoord tc;
    tc.valid = false;
    // pass 1: total number of tiles
    int total = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
        const int e = e0 + lane;
        int t = e < E ? ceil_div(load_msize(m_sizes, ms_i64, e), BM) * n_tiles_n : 0;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) t += __shfl_xor(t, off);
        total += t;
    }
    const int chunk = ceil_div(total, kXcd);
    const int xcd = blockIdx.x % kXcd, slot = blockIdx.x / kXcd;
    const int L = xcd * chunk + slot;
    if (slot >= chunk || L >= total) return tc;
    // pass 2: locate L
    int tile_carry = 0, row_carry = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
        const int e = e0 + lane;
        const int m = e < E ? load_msize(m_sizes, ms_i64, e) : 0;
        const int t = ceil_div(m, BM) * n_tiles_n;
        int tinc = t, minc = m;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int ot = __shfl_up(tinc, off), om = __shfl_up(minc, off);
            if (lane >= off) {
                tinc += ot;
                minc += om;
            }
        }
        const int tbeg = tile_carry + tinc - t;
        const bool hit = L >= tbeg && L < tbeg + t;
        const uint64_t hits = __ballot(hit);
        if (hits) {
            const int src = __ffsll((unsigned long long)hits) - 1;
            const int local = L - __shfl(tbeg, src);
            const int m_start = row_carry + __shfl(minc - m, src);
            const int m_size = __shfl(m, src);
            tc.expert = e0 + src;
            tc.i0 = m_start + (local / n_tiles_n) * BM;
            tc.i_end = m_start + m_size;
            if ((int64_t)tc.i_end > R) tc.i_end = (int)R;
            tc.j0 = local % n_tiles_n;  // tile index; scaled by the caller
            tc.valid = true;
            return tc;
        }
        tile_carry += __shfl(tinc, 63);
        row_carry += __shfl(minc, 63);
    }
    return tc;
}

template <typename TO>
__device__ __forceinline__ void store_out(TO *p, float v, float alpha, int accumulate) {
    v *= alpha;
    if (accumulate) v += to_f32(*p);
    *p = from_f32<TO>(v);
}

template <int BM, int BN, int BK, int WGM, int WGN, int OCC, int MODE, bool NF4, typename TO>
__global__ __launch_bounds__(WGM *WGN * 64) __attribute__((amdgpu_waves_per_eu(OCC *WGM *WGN / 4, OCC *WGM *WGN / 4)))
void gemm_mfma_kernel(const bf16_t *__restrict__ a, const bf16_t *__restrict__ b, const void *__restrict__ m_sizes,
                      int ms_i64, TO *__restrict__ c, int64_t R, int N, int K, int E, float alpha, int accumulate,
                      Nf4Args nf4) {
    static_assert(!NF4 || MODE == MODE_FWD, "NF4 weights are a forward-only operand");
    constexpr int NT = WGM * WGN * 64;
    constexpr bool A_RC = MODE != MODE_DW;
    constexpr bool B_RC = MODE == MODE_FWD;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    typedef TileLayout<BM, BK, A_RC> LA;
    typedef TileLayout<BN, BK, B_RC> LB;
    static_assert(LA::kChunks % NT == 0 && LB::kChunks % NT == 0, "tile does not split over the workgroup");
    static_assert(LA::kBytes + LB::kBytes <= 64 * 1024, "static LDS limit");

    __shared__ __attribute__((aligned(16))) unsigned char lds_a[LA::kBytes];
    __shared__ __attribute__((aligned(16))) unsigned char lds_b[LB::kBytes];
    __shared__ float lds_code[16];
    if (NF4 && threadIdx.x < 16) lds_code[threadIdx.x] = nf4.code16[threadIdx.x];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;

    // ---- which tile
    int i0, i_end, j0, j_end, r_begin, r_end;
    const bf16_t *a_base;
    const bf16_t *b_base;
    int64_t lda, ldb, ldc, nf4_base = 0;
    TO *c_base;
    if (MODE == MODE_DW) {
        const int tn = ceil_div(N, BM), tk = ceil_div(K, BN);
        const int per_expert = tn * tk;
        const int total = E * per_expert;
        const int chunk = ceil_div(total, kXcd);
        const int xcd = blockIdx.x % kXcd, slot = blockIdx.x / kXcd;
        const int L = xcd * chunk + slot;
        if (slot >= chunk || L >= total) return;
        const int e = L / per_expert, local = L % per_expert;
        // rows of expert e: prefix over m_sizes (wave-redundant shuffle reduction)
        int before = 0, mine = 0;
        for (int e0 = 0; e0 <= e; e0 += 64) {
            const int q = e0 + lane;
            const int m = q < E ? load_msize(m_sizes, ms_i64, q) : 0;
            int part = q < e ? m : 0;
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) part += __shfl_xor(part, off);
            before += part;
            if (e - e0 < 64) mine = __shfl(m, e - e0);
        }
        i0 = (local / tk) * BM, i_end = N;
        j0 = (local % tk) * BN, j_end = K;
        r_begin = before, r_end = before + mine;
        if ((int64_t)r_end > R) r_end = (int)R;
        if (r_begin > r_end) r_begin = r_end;
        a_base = a, lda = N;
        b_base = b, ldb = K;
        c_base = c + (int64_t)e * N * K, ldc = K;
    } else {
        const int n_tiles_n = ceil_div(N, BN);
        const TileCoord tc = find_tile_rows<BM>(m_sizes, ms_i64, E, n_tiles_n, R, lane);
        if (!tc.valid) return;
        i0 = tc.i0, i_end = tc.i_end;
        j0 = tc.j0 * BN, j_end = N;
        r_begin = 0, r_end = K;
        a_base = a, lda = K;
        b_base = NF4 ? b : b + (int64_t)tc.expert * N * K;
        nf4_base = (int64_t)tc.expert * N * K;
        ldb = B_RC ? K : N;
        c_base = c, ldc = N;
    }

    floatx16 acc[TM][TN];
#pragma unroll
    for (int bi = 0; bi < TM; ++bi)
#pragma unroll
        for (int bj = 0; bj < TN; ++bj)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[bi][bj][r] = 0.f;

    // 32-row blocks of this wave that hold at least one valid row (wave-uniform)
    bool blk_on[TM];
#pragma unroll
    for (int bi = 0; bi < TM; ++bi) blk_on[bi] = (i0 + wm * WTM + bi * 32) < i_end;

    uint4_t stage_a[LA::kChunks / NT], stage_b[NF4 ? 1 : LB::kChunks / NT];
    uint32_t stage_q[NF4 ? LB::kChunks / NT : 1];
    float stage_am[NF4 ? LB::kChunks / NT : 1];
    const uint8_t *wq = (const uint8_t *)b;
    if (r_begin < r_end) {
        load_stage<BM, BK, A_RC, NT>(stage_a, a_base, lda, i0, i_end, r_begin, r_end, tid);
        if constexpr (NF4)
            load_stage_nf4<BN, BK, NT>(stage_q, stage_am, wq, nf4.absmax, nf4.bs_shift, nf4_base, K, j0, j_end,
                                       r_begin, r_end, tid);
        else
            load_stage<BN, BK, B_RC, NT>(stage_b, b_base, ldb, j0, j_end, r_begin, r_end, tid);
    }
    for (int r0 = r_begin; r0 < r_end; r0 += BK) {
        __syncthreads();  // everyone is done reading the previous tile
        store_stage<BM, BK, A_RC, NT>(stage_a, lds_a, tid);
        if constexpr (NF4)
            store_stage_nf4<BN, BK, NT>(stage_q, stage_am, lds_code, lds_b, tid);
        else
            store_stage<BN, BK, B_RC, NT>(stage_b, lds_b, tid);
        __syncthreads();
        if (r0 + BK < r_end) {  // next tile travels while this one is multiplied
            load_stage<BM, BK, A_RC, NT>(stage_a, a_base, lda, i0, i_end, r0 + BK, r_end, tid);
            if constexpr (NF4)
                load_stage_nf4<BN, BK, NT>(stage_q, stage_am, wq, nf4.absmax, nf4.bs_shift, nf4_base, K, j0, j_end,
                                           r0 + BK, r_end, tid);
            else
                load_stage<BN, BK, B_RC, NT>(stage_b, b_base, ldb, j0, j_end, r0 + BK, r_end, tid);
        }
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            bf16x8 fb[TN];
#pragma unroll
            for (int bj = 0; bj < TN; ++bj) fb[bj] = load_frag<BN, BK, B_RC>(lds_b, wn * WTN + bj * 32, ks, lane);
#pragma unroll
            for (int bi = 0; bi < TM; ++bi) {
                if (!blk_on[bi]) continue;
                const bf16x8 fa = load_frag<BM, BK, A_RC>(lds_a, wm * WTM + bi * 32, ks, lane);
#pragma unroll
                for (int bj = 0; bj < TN; ++bj)
                    acc[bi][bj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb[bj], acc[bi][bj], 0, 0, 0);
            }
        }
    }

    // ---- epilogue: lane l of a 32x32 block holds column l%32, rows 8*(r/4) + 4*(l/32) + r%4
#pragma unroll
    for (int bi = 0; bi < TM; ++bi) {
        if (!blk_on[bi]) continue;
#pragma unroll
        for (int bj = 0; bj < TN; ++bj) {
            const int col = j0 + wn * WTN + bj * 32 + (lane & 31);
            if (col >= j_end) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = i0 + wm * WTM + bi * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (row < i_end) store_out<TO>(c_base + (int64_t)row * ldc + col, acc[bi][bj][r], alpha, accumulate);
            }
        }
    }
}

template <int BM, int BN, int BK, int WGM, int WGN, int OCC, typename TO>
int launch_mfma(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                int K, int E, float alpha, int accumulate, const Nf4Args *nf4, hipStream_t stream) {
    constexpr int NT = WGM * WGN * 64;
    int64_t tiles;
    if (mode == MODE_DW) {
        tiles = (int64_t)E * ceil_div(N, BM) * ceil_div(K, BN);
    } else {
        const int64_t m_tiles = R / BM + (R < E ? R : E);
        tiles = m_tiles * ceil_div(N, BN);
    }
    if (tiles == 0) return MFL_OK;
    const int64_t grid = (tiles + kXcd - 1) / kXcd * kXcd + kXcd;
    if (grid > 0x7fffffff) return MFL_ERR_UNSUPPORTED;
    const bf16_t *pa = (const bf16_t *)a, *pb = (const bf16_t *)b;
    TO *pc = (TO *)c;
    const Nf4Args none = {nullptr, nullptr, 0};
#define MFL_KERNEL(MODE, NF4)                                                                        \
    gemm_mfma_kernel<BM, BN, BK, WGM, WGN, OCC, MODE, NF4, TO><<<(unsigned)grid, NT, 0, stream>>>( \
        pa, pb, m_sizes, ms_i64, pc, R, N, K, E, alpha, accumulate, NF4 ? *nf4 : none)
    if (nf4 != nullptr) {
        MFL_KERNEL(MODE_FWD, true);
    } else if (mode == MODE_FWD) {
        MFL_KERNEL(MODE_FWD, false);
    } else if (mode == MODE_DX) {
        MFL_KERNEL(MODE_DX, false);
    } else {
        MFL_KERNEL(MODE_DW, false);
    }
#undef MFL_KERNEL
    return launch_status();
}

}  // namespace

// Tile configuration: 0 = the default below; a variable only in tuning builds.
#ifdef MFL_TUNING_BUILD
int g_mfma_config = 0;
#else
namespace {
constexpr int g_mfma_config = 0;
}
#endif

namespace {

int dispatch_mfma(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                  int K, int E, int out_dtype, float alpha, int accumulate, const Nf4Args *nf4, hipStream_t stream) {
#define MFL_LAUNCH(BM, BN, BK, WGM, WGN, OCC)                                                                  \
    (out_dtype == MFL_BF16                                                                                     \
         ? launch_mfma<BM, BN, BK, WGM, WGN, OCC, bf16_t>(mode, a, b, m_sizes, ms_i64, c, R, N, K, E, alpha,  \
                                                          accumulate, nf4, stream)                             \
         : launch_mfma<BM, BN, BK, WGM, WGN, OCC, float>(mode, a, b, m_sizes, ms_i64, c, R, N, K, E, alpha,   \
                                                         accumulate, nf4, stream))
    switch (g_mfma_config) {
        case 1:
            return MFL_LAUNCH(128, 128, 64, 2, 2, 2);
        case 2:
            return MFL_LAUNCH(256, 128, 64, 2, 2, 1);
        case 3:
            return MFL_LAUNCH(128, 128, 32, 2, 2, 2);
        default:
            return MFL_LAUNCH(128, 128, 64, 2, 2, 2);
    }
#undef MFL_LAUNCH
}

}  // namespace

int gemm_bf16_mfma(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                   int K, int E, int out_dtype, float alpha, int accumulate, hipStream_t stream) {
    // 16-byte chunks along every contiguous dimension
    // thin LoRA shapes (N or K = rank) run here too: the tile edges are masked, and those
    // products are bound by streaming the wide operand, not by the matrix cores
    if (N % 8 != 0 || K % 8 != 0 || N < 8 || K < 8) return MFL_ERR_UNSUPPORTED;
    if (!aligned(a, 16) || !aligned(b, 16) || !aligned(c, 4)) return MFL_ERR_UNSUPPORTED;
    if (out_dtype != MFL_BF16 && out_dtype != MFL_F32) return MFL_ERR_UNSUPPORTED;
    return dispatch_mfma(mode, a, b, m_sizes, ms_i64, c, R, N, K, E, out_dtype, alpha, accumulate, nullptr, stream);
}

int gemm_nf4_mfma(const void *x, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                  const void *m_sizes, int ms_i64, void *y, int64_t R, int N, int K, int E, int out_dtype,
                  hipStream_t stream) {
    int shift = 0;
    while ((1 << shift) < blocksize) ++shift;
    // a 16-byte LDS chunk (8 weights along K) must not straddle two absmax blocks
    if (K % 8 != 0 || blocksize < 8 || N < 1) return MFL_ERR_UNSUPPORTED;
    if (!aligned(x, 16) || !aligned(wq, 4) || !aligned(y, 4)) return MFL_ERR_UNSUPPORTED;
    if (out_dtype != MFL_BF16 && out_dtype != MFL_F32) return MFL_ERR_UNSUPPORTED;
    const Nf4Args nf4 = {code16, absmax, shift};
    return dispatch_mfma(MODE_FWD, x, wq, m_sizes, ms_i64, y, R, N, K, E, out_dtype, 1.0f, 0, &nf4, stream);
}

}  // namespace mfl
