// Pipelined bf16 grouped GEMM for CDNA4: global -> LDS copies that bypass the register file
// (global_load_lds_dwordx4), a ring of S LDS stages so several K steps are in flight per
// compute unit, XOR-swizzled stage layouts (no padding: the copy engine writes 1 KiB of
// consecutive LDS per wave instruction), v_mfma_f32_32x32x16_bf16, persistent workgroups.
//
// Operand conventions are those of gemm_bf16_mfma.hip: C[i, j] = sum_r A(i, r) * B(j, r) with
// each operand either reduction-contiguous (RC, memory [i][r]) or reduction-strided
// (RS, memory [r][i]).
//
//   RC stage: row i holds BK elements (BK*2 bytes); 16-byte chunk c of row i is stored at
//             chunk c ^ ((i / rows_per_256B) % chunks_per_row): the 16 rows one half-wave reads
//             for an MFMA fragment then fall in 16 different bank groups.
//   RS stage: row r holds BI elements; chunk c of row r is stored at c ^ ((r & 3) << 1): the
//             four rows a transposing read (ds_read_b64_tr_b16) touches fall in different banks.
//
// Shapes this kernel takes (the caller falls back to gemm_bf16_mfma.hip otherwise):
//   FWD, DX: K % BK == 0, N % 8 == 0.   DW: N % 8 == 0, K % 8 == 0.
// Rows or columns past a tile's valid range are loaded from a clamped (valid) address and never
// stored; in DW the rows of the last, partial reduction step are zeroed in LDS before use.
#include "common.h"
#include "gemm.h"

namespace mfl {

namespace {

constexpr int kXcd = 8;

typedef __attribute__((address_space(3))) void *lds_void_ptr;
typedef const __attribute__((address_space(1))) void *global_void_ptr;
typedef __attribute__((address_space(3))) short4_t *lds_short4_ptr;

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | 0x70 | 0xF00 | ((N >> 4) << 14));
}

template <int BI, int BK, bool RC>
struct Stage {
    static constexpr int kRowBytes = RC ? BK * 2 : BI * 2;
    static constexpr int kRows = RC ? BI : BK;
    static constexpr int kBytes = BI * BK * 2;
    static constexpr int kWaveLoads = kBytes / 1024;       // 1 KiB per wave-wide copy
    static constexpr int kRowsPerLoad = 1024 / kRowBytes;  // rows covered by one copy
    static constexpr int kChunksPerRow = kRowBytes / 16;
    static constexpr int kRowsPer256 = kRowBytes >= 256 ? 1 : 256 / kRowBytes;
    static_assert(kRowBytes <= 1024 && 1024 % kRowBytes == 0, "row must divide a 1 KiB copy");

    // physical 16-byte chunk of logical chunk c in row `row`
    __device__ static __forceinline__ int swz(int row, int c) {
        if (RC) return c ^ ((row / kRowsPer256) % kChunksPerRow);
        return c ^ ((row & 3) << 1);
    }
};

// Per-lane byte offset (relative to the operand's tile origin in global memory at reduction
// step 0) of the 16 bytes this lane copies in wave-load `load`.  `i_lim` is the number of valid
// rows (RC) or columns (RS) from the tile origin; lanes outside are clamped inside.
template <int BI, int BK, bool RC>
__device__ __forceinline__ int64_t lane_src_offset(int load, int lane, int64_t ld, int i_lim) {
    typedef Stage<BI, BK, RC> S;
    const int row = load * S::kRowsPerLoad + lane / S::kChunksPerRow;  // stage row
    const int phys = lane % S::kChunksPerRow;
    const int c = S::swz(row, phys);  // XOR swizzle is its own inverse
    if (RC) {
        int i = row;
        if (i >= i_lim) i = i_lim - 1;
        return ((int64_t)i * ld + c * 8) * 2;
    } else {
        int i = c * 8;
        if (i >= i_lim) i = i_lim - 8;
        return ((int64_t)row * ld + i) * 2;  // rows past the reduction range are pulled back at issue time
    }
}

struct RowTile {
    int expert, i0, i_end, jt;
};

// Number of tiles of the row-grouped modes: sum over experts of ceil(m_e / BM) * n_tiles_n.
template <int BM>
__device__ __forceinline__ int count_row_tiles(const void *m_sizes, int ms_i64, int E, int n_tiles_n, int lane) {
    int total = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
        const int e = e0 + lane;
        int t = e < E ? ceil_div(load_msize(m_sizes, ms_i64, e), BM) * n_tiles_n : 0;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) t += __shfl_xor(t, off);
        total += t;
    }
    return total;
}

// (expert, first row, row bound, n-tile) of logical tile L < total.  Within an expert the
// m-tiles of one n-tile are consecutive: workgroups that share a slice of the weight matrix
// run side by side, and a boundary between scheduling rounds costs a re-read of the expert's
// rows (small) rather than of its weights (large).
template <int BM>
__device__ __forceinline__ RowTile locate_row_tile(const void *m_sizes, int ms_i64, int E, int n_tiles_n, int64_t R,
                                                   int L, int lane) {
    RowTile rt = {0, 0, 0, 0};
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
        const uint64_t hits = __ballot(L >= tbeg && L < tbeg + t);
        if (hits) {
            const int src = __ffsll((unsigned long long)hits) - 1;
            const int local = L - __shfl(tbeg, src);
            const int m_start = row_carry + __shfl(minc - m, src);
            const int m_size = __shfl(m, src);
            const int m_tiles = ceil_div(m_size, BM);
            rt.expert = e0 + src;
            rt.i0 = m_start + (local % m_tiles) * BM;
            rt.i_end = m_start + m_size;
            if ((int64_t)rt.i_end > R) rt.i_end = (int)R;
            rt.jt = local / m_tiles;
            return rt;
        }
        tile_carry += __shfl(tinc, 63);
        row_carry += __shfl(minc, 63);
    }
    return rt;
}

// Per-lane LDS byte offsets (within an operand's part of a stage) of the MFMA fragment reads.
// RC: one offset per 16-wide reduction sub-step (the row block adds a constant).
// RS: one offset per 32-row block of the tile (the sub-step adds a constant).
template <int BI, int BK, bool RC, int TB>
struct FragOffsets {
    static constexpr int kCount = RC ? BK / 16 : TB;
    int off[kCount];

    __device__ __forceinline__ void init(int wave_row0, int lane) {
        typedef Stage<BI, BK, RC> S;
        if (RC) {
            const int row = wave_row0 + (lane & 31);
#pragma unroll
            for (int ks = 0; ks < kCount; ++ks)
                off[ks] = row * S::kRowBytes + S::swz(row, ks * 2 + (lane >> 5)) * 16;
        } else {
            const int g = lane >> 4, il = lane & 15;
            const int r = 8 * (g >> 1) + (il >> 2);
#pragma unroll
            for (int bi = 0; bi < kCount; ++bi) {
                const int i = wave_row0 + bi * 32 + 16 * (g & 1) + 4 * (il & 3);
                off[bi] = r * S::kRowBytes + S::swz(r, i >> 3) * 16 + (i & 7) * 2;
            }
        }
    }

    // fragment of row block bi at sub-step ks; `base` points at the operand's part of the stage
    __device__ __forceinline__ bf16x8 load(const unsigned char *base, int bi, int ks) const {
        typedef Stage<BI, BK, RC> S;
        if (RC) {
            return *(const bf16x8 *)(base + off[ks] + bi * 32 * S::kRowBytes);
        } else {
            const unsigned char *p = base + off[bi] + ks * 16 * S::kRowBytes;
            const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)p);
            const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(p + 4 * S::kRowBytes));
            union {
                short4_t h[2];
                bf16x8 v;
            } u;
            u.h[0] = lo;
            u.h[1] = hi;
            return u.v;
        }
    }
};

// One more wave than the WGM x WGN that multiply runs ahead of them when PF > 0: it touches
// one dword of every 128-byte line of reduction step kt + S - 1 + PF (a 4-byte copy per lane into
// a scratch corner of LDS) so that the copies proper find their data in L2.  Tiles share
// operands (rows of an expert are read by every n-tile, weights by every m-tile), so only a
// fraction of the bytes the stages hold in flight is new to L2; with its own memory counter the
// extra wave keeps many more first-touch misses in flight than the stage ring can.
template <int BI, int BK, bool RC>
__device__ __forceinline__ void touch_lines(const unsigned char *tile, int ld, int lim, int kt, int red, int lane,
                                            unsigned char *scratch) {
    constexpr int LINES = BI * BK * 2 / 128;
#pragma unroll
    for (int j = 0; j < LINES / 64; ++j) {
        const int idx = j * 64 + lane;
        const unsigned char *p;
        if (RC) {
            int row = idx / (BK * 2 / 128), seg = idx % (BK * 2 / 128);
            if (row >= lim) row = lim - 1;
            p = tile + ((int64_t)row * ld + kt * BK) * 2 + seg * 128;
        } else {
            constexpr int SEGS = BI * 2 / 128 > 0 ? BI * 2 / 128 : 1;
            int r = kt * BK + idx / SEGS, seg = idx % SEGS;
            if (r >= red) r = red - 1;
            int col = seg * 64;
            if (col >= lim) col = lim - 8;
            p = tile + ((int64_t)r * ld + col) * 2;
        }
        __builtin_amdgcn_global_load_lds((global_void_ptr)p, (lds_void_ptr)scratch, 4, 0, 0);
    }
}

template <int BM, int BN, int BK, int S, int WGM, int WGN, int PF, int MODE, typename TO>
__global__ __launch_bounds__((WGM * WGN + (PF > 0 ? 1 : 0)) * 64) void gemm_pipe_kernel(const bf16_t *__restrict__ a,
                                                                  const bf16_t *__restrict__ b,
                                                                  const void *__restrict__ m_sizes, int ms_i64,
                                                                  TO *__restrict__ c, int64_t R, int N, int K, int E,
                                                                  float alpha, int accumulate) {
    constexpr int NW = WGM * WGN;
    constexpr bool A_RC = MODE != MODE_DW;
    constexpr bool B_RC = MODE == MODE_FWD;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int KS = BK / 16;
    typedef Stage<BM, BK, A_RC> SA;
    typedef Stage<BN, BK, B_RC> SB;
    constexpr int LA = SA::kWaveLoads / NW, LB = SB::kWaveLoads / NW;  // copies per wave per step
    static_assert(SA::kWaveLoads % NW == 0 && SB::kWaveLoads % NW == 0, "copies must split over the waves");
    constexpr int LPW = LA + LB;
    constexpr int STAGE_BYTES = SA::kBytes + SB::kBytes;
    static_assert((S - 2) * LPW < 64, "vmcnt range");

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;

    FragOffsets<BM, BK, A_RC, TM> fo_a;
    FragOffsets<BN, BK, B_RC, TN> fo_b;
    fo_a.init(wm * WTM, lane);
    fo_b.init(wn * WTN, lane);

    // ---- tile range of this workgroup: XCD x owns logical tiles [x*chunk, (x+1)*chunk)
    int total, tiles_n = 0, per_expert = 0;
    if (MODE == MODE_DW) {
        tiles_n = ceil_div(K, BN);
        per_expert = ceil_div(N, BM) * tiles_n;
        total = E * per_expert;
    } else {
        tiles_n = ceil_div(N, BN);
        total = __builtin_amdgcn_readfirstlane(count_row_tiles<BM>(m_sizes, ms_i64, E, tiles_n, lane));
    }
    const int chunk = ceil_div(total, kXcd);
    const int xcd = blockIdx.x % kXcd;
    const int per_xcd = gridDim.x / kXcd;
    int L_end = (xcd + 1) * chunk;
    if (L_end > total) L_end = total;

    for (int L = xcd * chunk + blockIdx.x / kXcd; L < L_end; L += per_xcd) {
        // ---- tile coordinates
        int i0, i_end, j0, j_end, r_begin, r_end;
        const unsigned char *a_tile;
        const unsigned char *b_tile;
        int lda, ldb;
        int64_t ldc;
        TO *c_base;
        if (MODE == MODE_DW) {
            const int e = L / per_expert, local = L % per_expert;
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
            i0 = (local / tiles_n) * BM, i_end = N;
            j0 = (local % tiles_n) * BN, j_end = K;
            r_begin = __builtin_amdgcn_readfirstlane(before), r_end = r_begin + __builtin_amdgcn_readfirstlane(mine);
            if ((int64_t)r_end > R) r_end = (int)R;
            if (r_begin > r_end) r_begin = r_end;
            lda = N, ldb = K, ldc = K;
            a_tile = (const unsigned char *)(a + (int64_t)r_begin * lda + i0);
            b_tile = (const unsigned char *)(b + (int64_t)r_begin * ldb + j0);
            c_base = c + (int64_t)e * N * K;
        } else {
            const RowTile rt = locate_row_tile<BM>(m_sizes, ms_i64, E, tiles_n, R, L, lane);
            i0 = __builtin_amdgcn_readfirstlane(rt.i0), i_end = __builtin_amdgcn_readfirstlane(rt.i_end);
            j0 = __builtin_amdgcn_readfirstlane(rt.jt) * BN, j_end = N;
            const int expert = __builtin_amdgcn_readfirstlane(rt.expert);
            r_begin = 0, r_end = K;
            lda = K, ldc = N;
            a_tile = (const unsigned char *)(a + (int64_t)i0 * lda);
            if (B_RC) {
                ldb = K;
                b_tile = (const unsigned char *)(b + (int64_t)expert * N * K + (int64_t)j0 * ldb);
            } else {
                ldb = N;
                b_tile = (const unsigned char *)(b + (int64_t)expert * N * K + j0);
            }
            c_base = c;
        }
        const int red = r_end - r_begin;
        const int KT = ceil_div(red, BK);
        const int i_lim = i_end - i0 < BM ? i_end - i0 : BM;  // valid rows (or columns) of A from the tile origin
        const int j_lim = j_end - j0 < BN ? j_end - j0 : BN;

        if (PF > 0 && wave == NW) {
            // ---- the wave that runs ahead: same barrier sequence as the others, no arithmetic
            unsigned char *scratch = smem + S * STAGE_BYTES;
            auto touch = [&](int step) {
                if (step < KT) {
                    touch_lines<BM, BK, A_RC>(a_tile, lda, i_lim, step, red, lane, scratch);
#ifndef MFL_EXP_PF_A_ONLY
                    touch_lines<BN, BK, B_RC>(b_tile, ldb, j_lim, step, red, lane, scratch);
#endif
                    wait_vmcnt<40>();
                }
            };
            __builtin_amdgcn_s_barrier();
            for (int step = S - 1; step < S - 1 + PF; ++step) touch(step);
            for (int kt = 0; kt < KT; ++kt) {
                __builtin_amdgcn_s_barrier();
                touch(kt + S - 1 + PF);
                if (MODE == MODE_DW && (kt + 1) * BK > red) __builtin_amdgcn_s_barrier();
            }
            if (sizeof(TO) == 2 && !accumulate) __builtin_amdgcn_s_barrier();
            continue;
        }

        // per-lane 32-bit source offsets of this wave's copies (tile origin, reduction step 0);
        // the step advances a wave-uniform base pointer
        uint32_t lane_off[LPW];
#pragma unroll
        for (int q = 0; q < LA; ++q)
            lane_off[q] = (uint32_t)lane_src_offset<BM, BK, A_RC>(wave * LA + q, lane, lda, i_lim);
#pragma unroll
        for (int q = 0; q < LB; ++q)
            lane_off[LA + q] = (uint32_t)lane_src_offset<BN, BK, B_RC>(wave * LB + q, lane, ldb, j_lim);
        const int64_t step_a = A_RC ? (int64_t)BK * 2 : (int64_t)BK * lda * 2;
        const int64_t step_b = B_RC ? (int64_t)BK * 2 : (int64_t)BK * ldb * 2;

        auto issue = [&](int kt) {
#ifdef MFL_EXP_NOLOAD
            return;
#endif
            unsigned char *st = smem + (kt % S) * STAGE_BYTES;
#ifdef MFL_EXP_ROT
            const int kk = MODE == MODE_DW ? kt : (kt + (L * MFL_EXP_ROT) % KT) % KT;
#else
            const int kk = kt;
#endif
            const unsigned char *pa = a_tile + kk * step_a;
            const unsigned char *pb = b_tile + kk * step_b;
            // In DW the last step may be partial: lanes whose row lies past the end re-read the
            // last valid row; those rows are zeroed in LDS before use.
            const bool tail = MODE == MODE_DW && (kt + 1) * BK > red;
#pragma unroll
            for (int q = 0; q < LA; ++q) {
                uint32_t o = lane_off[q];
                if (!A_RC && tail) {
                    const int row = (wave * LA + q) * SA::kRowsPerLoad + lane / SA::kChunksPerRow + kt * BK;
                    if (row >= red) o -= (uint32_t)(row - (red - 1)) * (uint32_t)lda * 2u;
                }
                __builtin_amdgcn_global_load_lds((global_void_ptr)(pa + o), (lds_void_ptr)(st + (wave * LA + q) * 1024),
                                                 16, 0, 0);
            }
#pragma unroll
            for (int q = 0; q < LB; ++q) {
                uint32_t o = lane_off[LA + q];
                if (!B_RC && tail) {
                    const int row = (wave * LB + q) * SB::kRowsPerLoad + lane / SB::kChunksPerRow + kt * BK;
                    if (row >= red) o -= (uint32_t)(row - (red - 1)) * (uint32_t)ldb * 2u;
                }
                __builtin_amdgcn_global_load_lds((global_void_ptr)(pb + o),
                                                 (lds_void_ptr)(st + SA::kBytes + (wave * LB + q) * 1024), 16, 0, 0);
            }
        };

        floatx16 acc[TM][TN];
#pragma unroll
        for (int bi = 0; bi < TM; ++bi)
#pragma unroll
            for (int bj = 0; bj < TN; ++bj)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[bi][bj][r] = 0.f;
        bool blk_on[TM];
#pragma unroll
        for (int bi = 0; bi < TM; ++bi) blk_on[bi] = (wm * WTM + bi * 32) < i_lim;

        // every store of the previous tile has left, every wave is done with the stages
        wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();

        // ---- prologue: S-1 steps in flight
#pragma unroll
        for (int s = 0; s < S - 1; ++s)
            if (s < KT) issue(s);

        for (int kt = 0; kt < KT; ++kt) {
            // step kt has landed for this wave's copies; the barrier extends that to all waves
            // and tells us everybody finished reading step kt-1, whose stage is refilled next
            if (kt + S - 2 < KT)
                wait_vmcnt<(S - 2) * LPW>();
            else
                wait_vmcnt<0>();
#ifndef MFL_EXP_NOBARRIER
            __builtin_amdgcn_s_barrier();
#endif
            if (kt + S - 1 < KT) issue(kt + S - 1);

            unsigned char *st = smem + (kt % S) * STAGE_BYTES;
            if (MODE == MODE_DW && (kt + 1) * BK > red) {
                // zero the rows of A past the end of the expert (B's are multiplied by them)
                const int first = red - kt * BK;
                for (int q = tid; q < (BK - first) * SA::kChunksPerRow; q += NW * 64)
                    *(uint4_t *)(st + first * SA::kRowBytes + q * 16) = uint4_t{0u, 0u, 0u, 0u};
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
            }
            const unsigned char *sa = st, *sb = st + SA::kBytes;
#ifndef MFL_EXP_NOLDS
            {
                // Every wave multiplies, also one whose rows all lie past the tile edge: a branch
                // here makes the compiler shuttle the accumulators between register files.
                // Fragments of sub-step ks+1 are fetched while sub-step ks is multiplied.
                bf16x8 fa[2][TM], fb[2][TN];
#pragma unroll
                for (int bj = 0; bj < TN; ++bj) fb[0][bj] = fo_b.load(sb, bj, 0);
#pragma unroll
                for (int bi = 0; bi < TM; ++bi) fa[0][bi] = fo_a.load(sa, bi, 0);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    if (ks + 1 < KS) {
#pragma unroll
                        for (int bj = 0; bj < TN; ++bj) fb[(ks + 1) & 1][bj] = fo_b.load(sb, bj, ks + 1);
#pragma unroll
                        for (int bi = 0; bi < TM; ++bi) fa[(ks + 1) & 1][bi] = fo_a.load(sa, bi, ks + 1);
                    }
#pragma unroll
                    for (int bi = 0; bi < TM; ++bi)
#pragma unroll
                        for (int bj = 0; bj < TN; ++bj)
#ifdef MFL_EXP_NOMFMA
                            acc[bi][bj][0] += (float)fa[ks & 1][bi][0] + (float)fb[ks & 1][bj][0];
#else
                            acc[bi][bj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ks & 1][bi], fb[ks & 1][bj],
                                                                                  acc[bi][bj], 0, 0, 0);
#endif
                }
            }
#endif
        }

        // ---- epilogue
        if (sizeof(TO) == 2 && !accumulate) {
            // Stage the wave's tile in LDS as bf16, then write full rows: 8 lanes x 16 bytes per
            // row instead of 2-byte stores scattered over 32 rows.
            __builtin_amdgcn_s_barrier();  // all waves are done reading the last stage
            constexpr int ROWB = WTN * 2 + 16;  // padded row, bytes
            unsigned char *ep = smem + wave * (WTM * ROWB);
#pragma unroll
            for (int bi = 0; bi < TM; ++bi) {
                if (!blk_on[bi]) continue;
#pragma unroll
                for (int bj = 0; bj < TN; ++bj)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int row = bi * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                        const int col = bj * 32 + (lane & 31);
                        *(bf16_t *)(ep + row * ROWB + col * 2) = (bf16_t)(acc[bi][bj][r] * alpha);
                    }
            }
            // same wave reads back what it wrote: LDS ops of one wave complete in order
            constexpr int LPR = WTN / 8;        // lanes per row
            constexpr int RPI = 64 / LPR;       // rows per wave instruction
            const int lrow = lane / LPR, lcol = (lane % LPR) * 8;
#pragma unroll
            for (int r0 = 0; r0 < WTM; r0 += RPI) {
                const int row_l = r0 + lrow;
                const int row = i0 + wm * WTM + row_l;
                const int col = j0 + wn * WTN + lcol;
                if (!blk_on[r0 / 32] || row >= i_end || col >= j_end) continue;
                const uint4_t v = *(const uint4_t *)(ep + row_l * ROWB + lcol * 2);
                bf16_t *dst = (bf16_t *)c_base + (int64_t)row * ldc + col;
                if (col + 8 <= j_end) {
                    *(uint4_t *)dst = v;
                } else {
                    const bf16_t *pv = (const bf16_t *)&v;
                    for (int u = 0; u < j_end - col; ++u) dst[u] = pv[u];
                }
            }
        } else {
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
                        if (row >= i_end) continue;
                        TO *p = c_base + (int64_t)row * ldc + col;
                        float v = alpha * acc[bi][bj][r];
                        if (accumulate) v += to_f32(*p);
                        *p = from_f32<TO>(v);
                    }
                }
            }
        }
    }
}

template <int BM, int BN, int BK, int S, int WGM, int WGN, int PF, typename TO>
int launch_pipe(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                int K, int E, float alpha, int accumulate, hipStream_t stream) {
    constexpr int NT = (WGM * WGN + (PF > 0 ? 1 : 0)) * 64;
    constexpr int STAGE_BYTES = (BM + BN) * BK * 2;
    constexpr int EP_BYTES = WGM * WGN * (BM / WGM) * ((BN / WGN) * 2 + 16);
    constexpr int LDS_BYTES = (S * STAGE_BYTES > EP_BYTES ? S * STAGE_BYTES : EP_BYTES) + 1024;  // + scratch corner
    static_assert(LDS_BYTES <= 160 * 1024, "LDS capacity of a CDNA4 compute unit");
    const bf16_t *pa = (const bf16_t *)a, *pb = (const bf16_t *)b;
    TO *pc = (TO *)c;
    const int grid = device_info().cu_count / kXcd * kXcd;  // one persistent workgroup per CU
#define MFL_PIPE(MODE)                                                                                          \
    {                                                                                                           \
        auto kern = gemm_pipe_kernel<BM, BN, BK, S, WGM, WGN, PF, MODE, TO>;                                        \
        static bool attr_set = false;                                                                           \
        if (!attr_set) {                                                                                        \
            hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,  \
                                               LDS_BYTES);                                                      \
            if (e != hipSuccess) return (int)e;                                                                 \
            attr_set = true;                                                                                    \
        }                                                                                                       \
        kern<<<grid, NT, LDS_BYTES, stream>>>(pa, pb, m_sizes, ms_i64, pc, R, N, K, E, alpha, accumulate);      \
    }
    if (mode == MODE_FWD) MFL_PIPE(MODE_FWD)
    else if (mode == MODE_DX) MFL_PIPE(MODE_DX)
    else MFL_PIPE(MODE_DW)
#undef MFL_PIPE
    return launch_status();
}

}  // namespace

int g_pipe_config = 0;

int gemm_bf16_pipe(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                   int K, int E, int out_dtype, float alpha, int accumulate, hipStream_t stream) {
    if (g_pipe_config < 0) return MFL_ERR_UNSUPPORTED;
    if (!aligned(a, 16) || !aligned(b, 16) || !aligned(c, 16)) return MFL_ERR_UNSUPPORTED;
    if (out_dtype != MFL_BF16 && out_dtype != MFL_F32) return MFL_ERR_UNSUPPORTED;
    if (mode == MODE_FWD && (K % 64 != 0 || N % 8 != 0 || N < 8)) return MFL_ERR_UNSUPPORTED;
    if (mode == MODE_DX && (K % 64 != 0 || N % 8 != 0 || N < 8)) return MFL_ERR_UNSUPPORTED;
    if (mode == MODE_DW && (N % 8 != 0 || K % 8 != 0 || N < 8 || K < 8)) return MFL_ERR_UNSUPPORTED;
    if (mode != MODE_DW && R <= 0) return MFL_OK;
#define MFL_LAUNCH(BM, BN, BK, S, WGM, WGN, PF)                                                                  \
    (out_dtype == MFL_BF16 ? launch_pipe<BM, BN, BK, S, WGM, WGN, PF, bf16_t>(mode, a, b, m_sizes, ms_i64, c, R, \
                                                                              N, K, E, alpha, accumulate, stream) \
                           : launch_pipe<BM, BN, BK, S, WGM, WGN, PF, float>(mode, a, b, m_sizes, ms_i64, c, R,  \
                                                                             N, K, E, alpha, accumulate, stream))
    // Tile table (BM, BN, BK, stages, waves along M, waves along N, run-ahead distance).  The
    // default per product was picked from timings at the Qwen3-30B-A3B expert shapes.
    int cfg = g_pipe_config;
    if (cfg == 0) {
        if (mode == MODE_DX) return MFL_ERR_UNSUPPORTED;  // the register-staged kernel is faster there
        cfg = 8;
    }
    switch (cfg) {
        case 1:
            return MFL_LAUNCH(128, 128, 64, 4, 2, 2, 0);
        case 2:
            return MFL_LAUNCH(256, 128, 64, 3, 4, 2, 0);
        case 4:
            return MFL_LAUNCH(256, 128, 64, 3, 4, 2, 4);
        case 7:
            return MFL_LAUNCH(256, 256, 32, 4, 2, 4, 0);
        default:
            return MFL_LAUNCH(256, 256, 64, 2, 2, 4, 0);
    }
#undef MFL_LAUNCH
}

}  // namespace mfl
