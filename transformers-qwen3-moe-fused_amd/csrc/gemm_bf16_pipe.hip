// Pipelined bf16 grouped GEMM for CDNA4: global -> LDS copies that bypass the register file
// (global_load_lds_dwordx4), a ring of S LDS stages so several reduction steps are in flight per
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
//   RS stage: row r holds BI elements; chunk c of row r is stored at c ^ ((r & 3) << s), s = 1 or
//             2 by row length: the four rows a transposing read (ds_read_b64_tr_b16) touches
//             fall in different banks.
//
// Tiles.  A tile is MB x NB blocks of 32 x 32.  The WGM x WGN waves of a workgroup split the
// columns in contiguous runs and take the 32-row blocks round robin (wave row w owns blocks
// w, w + WGM, ...).  In the row-grouped products (FWD, DX) a tile covers up to 32*MB rows of ONE
// expert; MB is chosen so that a typical expert fits in one tile: its weights are then streamed
// by exactly one workgroup per column slice, and a few rows more or less change the number of
// active blocks, not the number of tiles.  Experts with more rows are cut into equal parts.
// The reduction loop is instantiated once per number of active row blocks of a wave, so blocks
// past the last row cost no MFMA and there is no branch inside the loop.
//
// Shapes this kernel takes (the caller falls back to gemm_bf16_mfma.hip otherwise):
//   N % 8 == 0, K % 8 == 0 (NF4 weights: K % BK == 0).
// Rows or columns past a tile's valid range are loaded from a clamped (valid) address (or, with
// two stages, not copied at all) and never stored; in DW the rows of A in the last, partial
// reduction step are copied from a chunk of zeros.
//
// Variants of the same kernel:
//   NF4 weights (FWD, DX): the packed weights travel through registers and are decoded into the
//     weight part of the stage, one step ahead of the multiply.
//   FWD with gathered rows: the copy of row i reads row row_idx[i] / idx_div of the source.
//   FWD with two weight matrices (gate, up) and a silu(gate) * up epilogue.
//   DX with two terms: the reduction runs over a second pair of operands after the first.
// Memory hints: weights of the row-grouped products are copied non-temporal (each is read by one
// workgroup), the output leaves with streaming stores.
#include "pipe_parts.h"

namespace mfl {

namespace {

// NF4 weights (forward and input-gradient products): b points at the packed bytes; byte i holds
// element 2i in its high nibble and 2i+1 in its low one; value = code16[nibble] *
// absmax[element >> bs_shift], rounded once to bf16.
struct Nf4Params {
    const float *code16;
    const float *absmax;
    int bs_shift;
};

// Fusions of the forward product with its neighbours in the sparse MLP block.
//   Gather: row i of A is row row_idx[i] / idx_div of `a` (the replicate-and-sort of the tokens
//   never materialises).
//   Two-term DX: see a2 below (the input gradient of the gated unit, de w_gate + dg w_up).
//   GLU: two weight matrices b (gate) and b2 (up) of the same shape; the output is
//   silu(A b^T) * (A b2^T), rounded like the separate kernels round (each product to bf16, silu
//   in fp32 to bf16, product to bf16); the two products are stored too where c_e / c_g are given.
struct FwdFusion {
    const int32_t *row_idx;
    int idx_div;
    const void *b2;
    Nf4Params nf4_2;
    void *c_e, *c_g;
    // Two-term input gradient (DX only): the reduction runs over (a, b) and then over (a2, b2),
    // same shapes, one accumulator, one epilogue: dx = a b + a2 b2.
    const void *a2;
    // A last term with a reduction length of its own (FWD, DX; the rank of a LoRA adapter), after the one or
    // two terms above, in the same accumulator: c += at bt, at (R, kt), bt (E, N, kt) in FWD and (E, kt, N)
    // in DX.
    const void *at, *bt;
    int kthin;
    // with the GLU epilogue: the thin weights of the second (up) matrix; at is shared (its columns are the two
    // adapters' activations side by side, and each matrix's thin weights are zero over the other's columns)
    const void *bt2;
    // DX: the backward of the gated unit in the epilogue (see GemmFusion::bw_e)
    const void *bw_e, *bw_g;
    void *bw_de, *bw_dg, *bw_h;
};

// FUSE: 0 plain, 1 two weight matrices and the silu(gate) * up epilogue, 2 a thin last term in the reduction (built
// as a kernel of its own: the test for it in every step cost the plain products 3-5 %), 3 both: each of the two
// matrices with thin weights of its own, against one thin left operand; 4 the input gradient with the gated unit's
// backward in its epilogue (a kernel of its own: its epilogue holds pieces of e and g in registers beside the
// accumulators, which the plain input gradient has no room for).
template <int MB, int NB, int BK, int S, int WGM, int WGN, int MODE, bool NF4, int FUSE, typename TO>
__global__ __launch_bounds__(WGM *WGN * 64) void gemm_pipe_kernel(const bf16_t *__restrict__ a,
                                                                  const bf16_t *__restrict__ b,
                                                                  const void *__restrict__ m_sizes, int ms_i64,
                                                                  TO *__restrict__ c, int64_t R, int N, int K, int E,
                                                                  float alpha, int accumulate, Nf4Params nf4,
                                                                  FwdFusion fu) {
    constexpr bool GLU = FUSE == 1 || FUSE == 3, THIN = FUSE == 2 || FUSE == 3, BWG = FUSE == 4;
    static_assert(!BWG || (MODE == MODE_DX && sizeof(TO) == 2), "the gated unit's backward: input gradient, bf16");
    static_assert(!THIN || MODE != MODE_DW, "the thin last term belongs to the row-grouped products");
    static_assert(!NF4 || (MODE != MODE_DW && S == 2 && BK == 64), "NF4 weights: row-grouped products, two stages");
    static_assert(!GLU || (MODE == MODE_FWD && WGN % 2 == 0 && sizeof(TO) == 2 && BK == 64),
                  "GLU: forward product, bf16 output, the waves along N split in a gate half and an up half");
    constexpr int BM = MB * 32, BN = NB * 32;
    // GLU: the weight stage holds BNH rows of the gate matrix and the same BNH rows of the up
    // matrix.  Wave column wn < WGN/2 multiplies gate rows, wn >= WGN/2 the up rows of the same
    // output columns as wave wn - WGN/2.
    constexpr int BNH = GLU ? BN / 2 : BN;  // output columns of a tile
    constexpr int HW = GLU ? WGN / 2 : WGN;
    constexpr int NW = WGM * WGN;
    constexpr bool A_RC = MODE != MODE_DW;
    constexpr bool B_RC = MODE == MODE_FWD;
    constexpr int TM = (MB + WGM - 1) / WGM;  // row blocks per wave (the last may not exist)
    static_assert(NB % WGN == 0, "column blocks must split evenly over the waves");
    constexpr int TN = NB / WGN;
    constexpr int WTN = TN * 32;
    constexpr int KS = BK / 16;
    typedef Stage<BM, BK, A_RC> SA;
    typedef Stage<BN, BK, B_RC> SB;
    constexpr int LA = SA::kWaveLoads / NW, LB = NF4 ? 0 : SB::kWaveLoads / NW;  // copies per wave per step
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
    fo_a.init(wm * 32, WGM * 32, lane);
    fo_b.init(wn * WTN, 32, lane);
    // GLU: weight-stage row -> (matrix, column of the tile).  A copy fills 8 whole stage rows and
    // WTN is a multiple of 32, so the matrix is the same for all lanes of a copy.
    auto glu_up = [](int stage_row) { return (stage_row / WTN) / HW; };
    auto glu_col = [](int stage_row) { return ((stage_row / WTN) % HW) * WTN + stage_row % WTN; };

    // ---- per-expert prefix tables in LDS, behind the stages and the NF4 code tables (every wave
    // computes them, wave 0 writes them): rows, tiles and work before expert e.  The work of a
    // tile is its number of reduction-side units (32-row blocks, or reduction steps in DW) plus a
    // constant for what every tile costs whatever its height (streaming its weights, the epilogue).
    int *tab_rows = (int *)(smem + S * STAGE_BYTES + 128);
    int *tab_tiles = tab_rows + (kMaxTableExperts + 1);
    int *tab_work = tab_tiles + (kMaxTableExperts + 1);
    constexpr int kTileConstWork = MODE == MODE_DW ? 3 : 6;
    auto tile_work = [&](int m) {
        return (MODE == MODE_DW ? ceil_div(m, BK) : tile_rows_of<BM>(m) / 32) + kTileConstWork;
    };
    const int tiles_n = MODE == MODE_DW ? ceil_div(K, BN) : ceil_div(N, BNH);
    const int per_expert = MODE == MODE_DW ? ceil_div(N, BM) * tiles_n : 0;
    {
        int row_carry = 0, tile_carry = 0, work_carry = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            const int m = e < E ? load_msize(m_sizes, ms_i64, e) : 0;
            const int t = e >= E ? 0 : MODE == MODE_DW ? per_expert : m_tiles_of<BM>(m) * tiles_n;
            const int w = t * tile_work(m);
            const int minc = wave_inclusive_scan(m), tinc = wave_inclusive_scan(t), winc = wave_inclusive_scan(w);
            if (wave == 0 && e <= E) {  // entry E comes from the lane behind the last expert, or from below
                tab_rows[e] = row_carry + minc - m;
                tab_tiles[e] = tile_carry + tinc - t;
                tab_work[e] = work_carry + winc - w;
            }
            row_carry += wave_last(minc);
            tile_carry += wave_last(tinc);
            work_carry += wave_last(winc);
        }
        if (wave == 0 && lane == 0 && E % 64 == 0) {
            tab_rows[E] = row_carry;
            tab_tiles[E] = tile_carry;
            tab_work[E] = work_carry;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
    }
    const int total = __builtin_amdgcn_readfirstlane(tab_tiles[E]);

    // ---- tile range of this workgroup.  XCD x owns a contiguous run of logical tiles, so the
    // tiles of one expert meet in one L2.  With few tiles per workgroup the runs hold equal
    // numbers of tiles (one tile more on an XCD is a whole extra round there); with many, as
    // under skewed routing, the runs hold equal work, and the strided deal within a run mixes
    // tall and flat tiles over its workgroups.
    const int xcd = blockIdx.x % kXcd;
    const int per_xcd = gridDim.x / kXcd;
    int L_begin, L_end;
    if (total < 3 * (int)gridDim.x) {
        const int chunk = ceil_div(total, kXcd);
        L_begin = xcd * chunk;
        L_end = (xcd + 1) * chunk;
    } else {
        const int total_work = __builtin_amdgcn_readfirstlane(tab_work[E]);
        // first tile whose work prefix reaches total_work * x / kXcd
        auto boundary = [&](int x) {
            if (x >= kXcd) return total;
            const int target = (int)((int64_t)total_work * x / kXcd);
            int found = total;
            for (int e0 = 0; e0 < E; e0 += 64) {
                const int e = e0 + lane < E ? e0 + lane : E - 1;
                const int wb = tab_work[e], we = tab_work[e + 1];
                const uint64_t hits = __ballot(e0 + lane < E && target >= wb && target < we);
                if (hits) {
                    const int src = __ffsll((unsigned long long)hits) - 1;
                    const int ex = e0 + src;
                    const int m = tab_rows[ex + 1] - tab_rows[ex];
                    found = tab_tiles[ex] + (target - __shfl(wb, src)) / tile_work(m);
                    break;
                }
            }
            return __builtin_amdgcn_readfirstlane(found);
        };
        L_begin = boundary(xcd);
        L_end = boundary(xcd + 1);
    }
    if (L_end > total) L_end = total;

    // ---- state of the tile that is being copied and multiplied (set by setup_tile)
    int i0 = 0, i_end = 0, j0 = 0, j_end = 0, r_begin = 0, r_end = 0;
    const unsigned char *a_tile = nullptr, *b_tile = nullptr;
    const unsigned char *b2_tile = nullptr;
    const unsigned char *a2_tile = nullptr;  // two-term DX: second pair of operands
    const unsigned char *at_tile = nullptr, *bt_tile = nullptr, *bt2_tile = nullptr;  // the thin last term
    int KT_thin = 0;
    int lda = 0, ldb = 0;
    int64_t ldc = 0, nf4_base = 0;
    TO *c_base = nullptr;
    int red = 0, KT1 = 0, KT = 0, i_lim = 0, j_lim = 0, active = 0;
    int64_t step_a = 0, step_b = 0;
    uint32_t lane_off[LPW];
    auto setup_tile = [&](int L) {
        // ---- tile coordinates
        b2_tile = nullptr, a2_tile = nullptr, nf4_base = 0;
        if (MODE == MODE_DW) {
            const int e = L / per_expert, local = L % per_expert;
            i0 = (local / tiles_n) * BM, i_end = N;
            j0 = (local % tiles_n) * BN, j_end = K;
            r_begin = __builtin_amdgcn_readfirstlane(tab_rows[e]);
            r_end = __builtin_amdgcn_readfirstlane(tab_rows[e + 1]);
            if ((int64_t)r_end > R) r_end = (int)R;
            if (r_begin > r_end) r_begin = r_end;
            lda = N, ldb = K, ldc = K;
            a_tile = (const unsigned char *)(a + (int64_t)r_begin * lda + i0);
            b_tile = (const unsigned char *)(b + (int64_t)r_begin * ldb + j0);
            c_base = c + (int64_t)(L / per_expert) * N * K;
        } else {
            // expert whose tile range holds L.  Within an expert the m-tiles of one n-tile are
            // consecutive, so workgroups that share a slice of the weight matrix run side by side.
            int expert = 0;
            for (int e0 = 0; e0 < E; e0 += 64) {
                const int e = e0 + lane < E ? e0 + lane : E - 1;
                const uint64_t hits = __ballot(e0 + lane < E && L >= tab_tiles[e] && L < tab_tiles[e + 1]);
                if (hits) {
                    expert = e0 + __ffsll((unsigned long long)hits) - 1;
                    break;
                }
            }
            expert = __builtin_amdgcn_readfirstlane(expert);
            const int m_start = __builtin_amdgcn_readfirstlane(tab_rows[expert]);
            const int m_size = __builtin_amdgcn_readfirstlane(tab_rows[expert + 1]) - m_start;
            const int local = L - __builtin_amdgcn_readfirstlane(tab_tiles[expert]);
            const int m_tiles = m_tiles_of<BM>(m_size);
            const int rows = tile_rows_of<BM>(m_size);
            // Which of an expert's tiles run side by side.  Few row tiles: those of one column slice (they share
            // the slice of the weights, and the expert's rows stay in L2 from one slice to the next).  Many row
            // tiles (an expert of thousands of rows): the column slices of one row tile (they share its rows; the
            // expert's whole weight matrix is what stays in L2 from one row tile to the next).
            // (65536 rows under Zipf(1.2) routing: forward 273 -> 266 us; 131072 rows: 506 -> 469 us; uniform
            // routing unchanged; switching earlier, from two or three row tiles on, gains nothing)
            const bool n_fast = m_tiles > tiles_n;
            const int mi = n_fast ? local / tiles_n : local % m_tiles;
            const int ni = n_fast ? local % tiles_n : local / m_tiles;
            i0 = m_start + mi * rows;
            i_end = m_start + m_size;
            if (i_end > i0 + rows) i_end = i0 + rows;
            if ((int64_t)i_end > R) i_end = (int)R;
            if (i0 > i_end) i0 = i_end;
            j0 = ni * BNH, j_end = N;
            r_begin = 0, r_end = K;
            lda = K, ldc = N;
            a_tile = (const unsigned char *)(a + (int64_t)i0 * lda);
            // first weight element of the tile: rows j0.. of the (N, K) matrix in FWD, columns j0..
            // of the (K, N) matrix in DX
            nf4_base = B_RC ? ((int64_t)expert * N + j0) * K : (int64_t)expert * N * K + j0;
            if (B_RC) {
                ldb = K;
                b_tile = (const unsigned char *)(b + (int64_t)expert * N * K + (int64_t)j0 * ldb);
                if (GLU) b2_tile = (const unsigned char *)((const bf16_t *)fu.b2 + (int64_t)expert * N * K + (int64_t)j0 * ldb);
            } else {
                ldb = N;
                b_tile = (const unsigned char *)(b + (int64_t)expert * N * K + j0);
                if (fu.a2 != nullptr) {
                    a2_tile = (const unsigned char *)((const bf16_t *)fu.a2 + (int64_t)i0 * lda);
                    b2_tile = (const unsigned char *)((const bf16_t *)fu.b2 + (int64_t)expert * N * K + j0);
                }
            }
            if constexpr (THIN) {
                at_tile = (const unsigned char *)((const bf16_t *)fu.at + (int64_t)i0 * fu.kthin);
                bt_tile = (const unsigned char *)((const bf16_t *)fu.bt + (B_RC ? ((int64_t)expert * N + j0) * fu.kthin
                                                                               : (int64_t)expert * N * fu.kthin + j0));
                if constexpr (GLU)
                    bt2_tile = (const unsigned char *)((const bf16_t *)fu.bt2 + ((int64_t)expert * N + j0) * fu.kthin);
            }
            c_base = c;
        }
        red = r_end - r_begin;
        KT1 = ceil_div(red, BK);                                      // steps of one term
        KT = MODE == MODE_DX && fu.a2 != nullptr ? 2 * KT1 : KT1;  // the host checked K % BK == 0
        KT_thin = KT;  // first step of the thin term
        if constexpr (THIN) KT += ceil_div(fu.kthin, BK);
        i_lim = i_end - i0 < BM ? i_end - i0 : BM;  // valid rows (or columns) of A from the tile origin
        j_lim = j_end - j0 < BNH ? j_end - j0 : BNH;

        // per-lane 32-bit source offsets of this wave's copies (tile origin, reduction step 0);
        // the step advances a wave-uniform base pointer
#pragma unroll
        for (int q = 0; q < LA; ++q)
            lane_off[q] = (uint32_t)lane_src_offset<BM, BK, A_RC>(wave * LA + q, lane, lda, i_lim);
        if (MODE == MODE_FWD && fu.row_idx != nullptr) {
            // gathered rows: offsets from the start of the source matrix (the host checked that
            // it is smaller than 4 GiB)
#pragma unroll
            for (int q = 0; q < LA; ++q) {
                const int load = wave * LA + q;
                const int row = SA::row_of(load, lane);
                const int ch = SA::swz(row, SA::phys_of(load, lane));
                const int i = row < i_lim ? row : i_lim - 1;
                const uint32_t src = (uint32_t)fu.row_idx[i0 + i] / (uint32_t)fu.idx_div;
                lane_off[q] = (src * (uint32_t)lda + ch * 8) * 2;
            }
            a_tile = (const unsigned char *)a;
        }
#pragma unroll
        for (int q = 0; q < LB; ++q) {
            if (GLU) {
                const int load = wave * LB + q;
                const int row = SB::row_of(load, lane);
                const int ch = SB::swz(row, SB::phys_of(load, lane));
                int col = glu_col(row);
                if (col >= j_lim) col = j_lim - 1;
                lane_off[LA + q] = (uint32_t)(((int64_t)col * ldb + ch * 8) * 2);
            } else {
                lane_off[LA + q] = (uint32_t)lane_src_offset<BN, BK, B_RC>(wave * LB + q, lane, ldb, j_lim);
            }
        }
        step_a = A_RC ? (int64_t)BK * 2 : (int64_t)BK * lda * 2;
        step_b = B_RC ? (int64_t)BK * 2 : (int64_t)BK * ldb * 2;
        // row blocks of this wave that hold at least one valid row: blocks wm, wm+WGM, ... below
        // ceil(i_lim / 32)
        const int n_blocks = ceil_div(i_lim, 32);
        active = n_blocks > wm ? ceil_div(n_blocks - wm, WGM) : 0;
        if (active > TM) active = TM;
    };

    // ---- dW, two stages, whole tiles: the tiles of a workgroup form ONE stream of reduction steps.  A tile of dW
    // has only a handful of steps (rows of the expert / BK), so a pipeline that drains at every tile end and
    // fills again after the epilogue spends a third of its time doing one or the other.  Here the first step of
    // the NEXT tile is requested where a step of the current tile would be, at the top of its last step, into the
    // stage that step frees; the epilogue stages its output in the other stage, the one the last step was read
    // from.  Only scalars change from tile to tile when every tile is whole (N % BM == 0, K % BN == 0): the
    // per-lane source offsets of the copies are computed once, which is what keeps the accumulators out of
    // scratch memory (a second call of the whole set-up with live accumulators spilled 500-760 bytes per lane).
    constexpr bool XT = MODE == MODE_DW && S == 2 && !NF4 && NW * 32 * ((NB / WGN) * 64 + 16) <= STAGE_BYTES;
    const bool xt = XT && N % BM == 0 && K % BN == 0 && !(accumulate && sizeof(TO) == 2);
    int xt_g = 0;             // stage of the current tile's step 0
    bool xt_fetched = false;  // the current tile's step 0 has been requested already
    int n_i0 = 0, n_j0 = 0, n_red = 0;
    const unsigned char *n_a = nullptr, *n_b = nullptr;
    TO *n_c = nullptr;
    auto dw_next = [&](int L) {  // coordinates of dW tile L: scalars only
        const int e = L / per_expert, local = L % per_expert;
        n_i0 = (local / tiles_n) * BM;
        n_j0 = (local % tiles_n) * BN;
        int rb = __builtin_amdgcn_readfirstlane(tab_rows[e]);
        int re = __builtin_amdgcn_readfirstlane(tab_rows[e + 1]);
        if ((int64_t)re > R) re = (int)R;
        if (rb > re) rb = re;
        n_a = (const unsigned char *)(a + (int64_t)rb * N + n_i0);
        n_b = (const unsigned char *)(b + (int64_t)rb * K + n_j0);
        n_c = c + (int64_t)e * N * K;
        n_red = re - rb;
    };

    for (int L = L_begin + blockIdx.x / kXcd; L < L_end; L += per_xcd) {
        if (XT && xt_fetched) {
            // set-up of a tile whose first step is on its way: what dw_next computed
            i0 = n_i0, j0 = n_j0, a_tile = n_a, b_tile = n_b, c_base = n_c, red = n_red;
            r_begin = 0, r_end = n_red;
            KT1 = KT = ceil_div(red, BK);
        } else {
            setup_tile(L);
        }
        // the tile after this one, if its first step is to be requested under this one's last step
        bool xt_next = false;
        if (XT && xt && KT > 0 && L + per_xcd < L_end) {
            dw_next(L + per_xcd);
            xt_next = n_red > 0;
        }

        // Cache policy of the weight copies in the row-grouped products: a weight is read by exactly
        // one workgroup, so it is fetched non-temporal (bit 1 of the instruction's cache-policy
        // field) and leaves the L2 to the rows, which the workgroups of an expert share
        // (fwd 146.6 -> 140.5 us, dX 161.4 -> 157.3 us; the same hint on the rows costs 5-10 %).
        constexpr int B_POLICY = MODE == MODE_DW ? 0 : 2;
        // dW with square tiles: the dy panel of a tile is shared by fewer tiles (K / BN) than its x
        // panel (N / BM); fetching it non-temporal gains 2 % (195 -> 191.5 us); on x it costs 3 %.
        constexpr int A_POLICY = MODE == MODE_DW && NB > 2 ? 2 : 0;
        constexpr bool SKIP_A = A_RC && S == 2;
        // products with a reduction-strided operand read it with transposing LDS reads
        constexpr bool ASM_COPY = MODE != MODE_FWD;
        constexpr int SA_ROWS_PER_COPY = 64 / SA::kChunksPerRow;
        // A step of the last term, the one with a reduction length of its own: source offsets from that term's leading
        // dimensions, worked out here (the term is one or two steps of a tile's many); chunks past the end of a
        // reduction-contiguous row come from a chunk of zeros, rows past the end of a reduction-strided operand
        // re-read its last row (they meet zeros of the other operand).
        auto issue_second = [&](int ks, unsigned char *st) {
            static_assert(MODE == MODE_DW || A_RC, "the left operand of a row-grouped product");
            const int k2 = fu.kthin;
            // the lane number behind a barrier for the optimiser: what follows is worked out here, once or twice
            // per tile, and not kept in registers across the tile's other steps
            int ln = lane;
            asm volatile("" : "+v"(ln));
#pragma unroll
            for (int q = 0; q < LA; ++q) {
                const int load = wave * LA + q;
                int i = SA::row_of(load, ln);
                const int c = SA::swz(i, SA::phys_of(load, ln));
                if (i >= i_lim) i = i_lim - 1;
                const int r = ks * BK + c * 8;
                const unsigned char *p = r >= k2 ? (const unsigned char *)&g_zero_chunk : at_tile + ((int64_t)i * k2 + r) * 2;
                copy_to_lds<0, ASM_COPY>(p, st + load * 1024);
            }
            // (with NF4 weights the other steps fill the weight stage by decoding; this one copies bf16)
            constexpr int LBT = SB::kWaveLoads / NW;
#pragma unroll
            for (int q = 0; q < LBT; ++q) {
                const int load = wave * LBT + q;
                const int row = SB::row_of(load, ln);
                const int c = SB::swz(row, SB::phys_of(load, ln));
                const unsigned char *p;
                if (B_RC) {
                    // GLU: the stage row belongs to the gate or to the up matrix, each with its own thin weights
                    const int col = GLU ? glu_col(row) : row;
                    const unsigned char *bt_m = GLU && glu_up(row) ? bt2_tile : bt_tile;
                    const int j = col < j_lim ? col : j_lim - 1;
                    const int r = ks * BK + c * 8;
                    p = r >= k2 ? (const unsigned char *)&g_zero_chunk : bt_m + ((int64_t)j * k2 + r) * 2;
                } else {
                    int r = ks * BK + row;
                    if (r >= k2) r = k2 - 1;
                    int j = c * 8;
                    if (j >= j_lim) j = j_lim - 8;
                    p = bt_tile + ((int64_t)r * N + j) * 2;
                }
                copy_to_lds<0, ASM_COPY>(p, st + SA::kBytes + load * 1024);
            }
        };
        // next_tile (XT only): step 0 of the tile after this one, into the stage after this tile's last
        auto issue = [&](int kt, bool next_tile = false) {
            unsigned char *st = smem + ((XT ? xt_g + kt : kt) % S) * STAGE_BYTES;
            if constexpr (THIN) {
                if (kt >= KT_thin) {
                    issue_second(kt - KT_thin, st);
                    return;
                }
            }
            // step of the term that is being reduced (two-term DX: the second term follows the first)
            int ks = kt;
            const unsigned char *a_term = a_tile, *b_term = b_tile;
            int red = r_end - r_begin;  // shadows the tile's: the reduction length the tail handling goes by
            if (XT && next_tile) {
                ks = 0;
                a_term = n_a;
                b_term = n_b;
                red = n_red;
            }
            if (MODE == MODE_DX && kt >= KT1) {
                ks = kt - KT1;
                a_term = a2_tile;
                b_term = b2_tile;
            }
            const unsigned char *pa = a_term + ks * step_a;
            const unsigned char *pb = b_term + ks * step_b;
            const unsigned char *pb2 = GLU ? b2_tile + ks * step_b : pb;
            // weight matrix of the wave's q-th copy (wave-uniform)
            auto b_src = [&](int q) { return GLU && glu_up((wave * LB + q) * (64 / SB::kChunksPerRow)) ? pb2 : pb; };
            // The last step may be partial.  Reduction-strided operand: lanes whose row lies past
            // the end re-read the last valid row (in DW those rows of A are copied from a chunk of
            // zeros instead; in DX they meet zeros of A).  Reduction-contiguous operand: chunks past the
            // end of the row are copied from a chunk of zeros.
            const bool tail = (ks + 1) * BK > red;
            if (!tail) {
#pragma unroll
                for (int q = 0; q < LA; ++q) {
                    // a copy fills whole stage rows; rows past the tile's last one feed nothing that
                    // is stored (with two stages every wait is for all copies, so leaving some out
                    // does not disturb the counting)
                    if (SKIP_A && (wave * LA + q) * SA_ROWS_PER_COPY >= i_lim) continue;
                    copy_to_lds<A_POLICY, ASM_COPY>(pa + lane_off[q], st + (wave * LA + q) * 1024);
                }
#pragma unroll
                for (int q = 0; q < LB; ++q)
                    copy_to_lds<B_POLICY, ASM_COPY>(b_src(q) + lane_off[LA + q], st + SA::kBytes + (wave * LB + q) * 1024);
                return;
            }
            // DW, two stages: the last step multiplies only the 16-row sub-steps that hold rows, and
            // copies that lie wholly past them are left out (every wait is for all copies, so the
            // counting is not disturbed)
            const int tail_rows = MODE == MODE_DW && S == 2 ? ceil_div(red - ks * BK, 16) * 16 : BK;
#pragma unroll
            for (int q = 0; q < LA; ++q) {
                const int load = wave * LA + q;
                if (MODE == MODE_DW && SA::row_of(load, 0) >= tail_rows) continue;
                const unsigned char *p = pa + lane_off[q];
                if (A_RC) {
                    const int c = SA::swz(SA::row_of(load, lane), SA::phys_of(load, lane));
                    if (ks * BK + c * 8 >= red) p = (const unsigned char *)&g_zero_chunk;
                } else {
                    // rows past the end: zeros in DW (the rows of B that meet them are re-reads of
                    // the last valid row: finite data), the last valid row again in DX
                    const int row = SA::row_of(load, lane) + ks * BK;
                    if (row >= red) {
                        if (MODE == MODE_DW)
                            p = (const unsigned char *)&g_zero_chunk;
                        else
                            p -= (int64_t)(row - (red - 1)) * lda * 2;
                    }
                }
                copy_to_lds<0, ASM_COPY>(p, st + load * 1024);
            }
#pragma unroll
            for (int q = 0; q < LB; ++q) {
                const int load = wave * LB + q;
                if (MODE == MODE_DW && SB::row_of(load, 0) >= tail_rows) continue;
                const unsigned char *p = b_src(q) + lane_off[LA + q];
                if (B_RC) {
                    const int c = SB::swz(SB::row_of(load, lane), SB::phys_of(load, lane));
                    if (ks * BK + c * 8 >= red) p = (const unsigned char *)&g_zero_chunk;
                } else {
                    const int row = SB::row_of(load, lane) + ks * BK;
                    if (row >= red) p -= (int64_t)(row - (red - 1)) * ldb * 2;
                }
                copy_to_lds<0, ASM_COPY>(p, st + SA::kBytes + load * 1024);
            }
        };

        floatx16 acc[TM][TN];
#pragma unroll
        for (int t = 0; t < TM; ++t)
#pragma unroll
            for (int bj = 0; bj < TN; ++bj)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[t][bj][r] = 0.f;

        if (!(XT && xt_fetched)) {
            // every store of the previous tile has left, every wave is done with the stages
            wait_vmcnt<0>();
            __builtin_amdgcn_s_barrier();

            // ---- prologue: S-1 steps in flight
#pragma unroll
            for (int s = 0; s < S - 1; ++s)
                if (s < KT) issue(s);
        }

        // ---- reduction loop, instantiated per number of row blocks that are multiplied.  The
        // MFMA operands are swapped (B first): the accumulator of a lane then holds, for output
        // row lane % 32 of the block, the columns 8g + 4*(lane / 32) + {0..3}, g = 0..3.
        auto k_loop = [&](auto ta_tag) {
            constexpr int TA = decltype(ta_tag)::value;
            // The partial last step of DW multiplies only the 16-row sub-steps that hold rows.
            const int ks_last = MODE == MODE_DW ? ceil_div(red - (KT - 1) * BK, 16) : KS;
            for (int kt = 0; kt < KT; ++kt) {
                // step kt has landed for this wave's copies; the barrier extends that to all
                // waves and tells us everybody finished reading step kt-1, whose stage is
                // refilled next
                // A tile whose first step was requested under the previous tile: that tile's output stores were
                // issued after those copies, the memory counter counts down in order of issue, so "at most as
                // many outstanding as there were stores" means the copies have landed, and the stores' way to
                // memory is not waited for.
                constexpr int XT_STORES = TM * (WTN / 16);  // per wave, bf16 output staged through LDS, whole tiles
                if (XT && XT_STORES < 64 && sizeof(TO) == 2 && !accumulate && xt_fetched && kt == 0)
                    wait_vmcnt<(XT_STORES < 64 ? XT_STORES : 0)>();
                else if (kt + S - 2 < KT)
                    wait_vmcnt<(S - 2) * LPW>();
                else
                    wait_vmcnt<0>();
                __builtin_amdgcn_s_barrier();
                if (kt + S - 1 < KT)
                    issue(kt + S - 1);
                else if (XT && xt_next)
                    issue(KT, true);

                unsigned char *st = smem + ((XT ? xt_g + kt : kt) % S) * STAGE_BYTES;
                const unsigned char *sa = st, *sb = st + SA::kBytes;
                const int ks_lim = MODE == MODE_DW && kt == KT - 1 ? ks_last : KS;
                // fragments of sub-step ks+1 are fetched while sub-step ks is multiplied
                bf16x8 fa[2][TA], fb[2][TN];
#pragma unroll
                for (int bj = 0; bj < TN; ++bj) fb[0][bj] = fo_b.load(sb, bj, 0);
#pragma unroll
                for (int t = 0; t < TA; ++t) fa[0][t] = fo_a.load(sa, t, 0);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    if (MODE == MODE_DW && ks >= ks_lim) break;
                    if (ks + 1 < KS) {
#pragma unroll
                        for (int bj = 0; bj < TN; ++bj) fb[(ks + 1) & 1][bj] = fo_b.load(sb, bj, ks + 1);
#pragma unroll
                        for (int t = 0; t < TA; ++t) fa[(ks + 1) & 1][t] = fo_a.load(sa, t, ks + 1);
                    }
#pragma unroll
                    for (int t = 0; t < TA; ++t)
#pragma unroll
                        for (int bj = 0; bj < TN; ++bj)
                            acc[t][bj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[ks & 1][bj], fa[ks & 1][t],
                                                                                 acc[t][bj], 0, 0, 0);
                }
            }
        };
        // ---- NF4 weights: packed words travel through registers two steps ahead and are decoded
        // into the other stage while the current one is multiplied.  A thread owns 32 consecutive
        // weights of one row of the weight stage: 16 packed bytes (one load) = four 16-byte LDS
        // chunks.  FWD: a stage row is an output column, 64 weights along the reduction, two
        // threads.  DX: a stage row is a reduction index, BN weights along the output columns,
        // BN / 32 threads.
        // The 16 fp32 codes sit in LDS: whatever the nibbles, a wave's lookups fall in 16 different
        // banks (a 256-entry table of code pairs, one lookup per byte, was 2x slower: bank conflicts).
        constexpr int NT_ = NW * 64;
        static_assert(!NF4 || BN * 2 <= NT_, "one thread per half row of the weight stage");
        float *lut = (float *)(smem + S * STAGE_BYTES);
        // whole waves decode (a wave is 32 stage rows): a wave-uniform condition, no lane mask
        static_assert((BN * 2) % 64 == 0, "decoding threads are whole waves");
        const bool nf4_on = wave < BN * 2 / 64;
        constexpr int NF4_SEGS = B_RC ? 2 : BN / 32;  // threads per stage row
        const int nf4_row = tid / NF4_SEGS, nf4_half = tid % NF4_SEGS;
        // GLU: the thread's stage row belongs to the gate or to the up matrix, each with its own
        // packed bytes, absmax, block size and code table
        const bool nf4_up = GLU && glu_up(nf4_row);
        const unsigned char *nf4_w = (const unsigned char *)(nf4_up ? fu.b2 : (const void *)b);
        const float *nf4_am = nf4_up ? fu.nf4_2.absmax : nf4.absmax;
        const int nf4_shift = nf4_up ? fu.nf4_2.bs_shift : nf4.bs_shift;
        const float *nf4_lut = lut + (nf4_up ? 16 : 0);
        struct Nf4Regs {
            uint4_t w;
            float am[4];
        };
        auto nf4_load = [&](int kt, Nf4Regs &r) {
            if (!nf4_on) return;
            int64_t el;
            if (B_RC) {
                int row = GLU ? glu_col(nf4_row) : nf4_row;
                if (row >= j_lim) row = j_lim - 1;
                el = nf4_base + (int64_t)row * K + kt * BK + nf4_half * 32;
            } else {
                int col = nf4_half * 32;  // the host checked N % 32 == 0: a segment is inside or outside as a whole
                if (col >= j_lim) col = j_lim - 32;
                el = nf4_base + (int64_t)(kt * BK + nf4_row) * N + col;
            }
            r.w = *(const uint4_t *)(nf4_w + (el >> 1));
            if (nf4_shift >= 5) {
                r.am[0] = nf4_am[el >> nf4_shift];
            } else {
#pragma unroll
                for (int u = 0; u < 4; ++u) r.am[u] = nf4_am[(el + 8 * u) >> nf4_shift];
            }
        };
        // one packed dword (8 weights, one 16-byte chunk of the stage) of the thread's 32
        auto nf4_decode_part = [&](int kt, const Nf4Regs &r, int u) {
            unsigned char *sb = smem + (kt % S) * STAGE_BYTES + SA::kBytes + nf4_row * SB::kRowBytes;
            const float am = nf4_shift >= 5 ? r.am[0] : r.am[u];
            bf16x8 v;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t nib = (r.w[u] >> (8 * (j >> 1) + ((j & 1) ? 0 : 4))) & 15u;
                v[j] = (bf16_t)(nf4_lut[nib] * am);
            }
            *(bf16x8 *)(sb + SB::swz(nf4_row, nf4_half * 4 + u) * 16) = v;
        };
        auto nf4_decode = [&](int kt, const Nf4Regs &r) {
            if (!nf4_on) return;
#pragma unroll
            for (int u = 0; u < 4; ++u) nf4_decode_part(kt, r, u);
        };
        auto k_loop_nf4 = [&](auto ta_tag) {
            constexpr int TA = decltype(ta_tag)::value;
            Nf4Regs r0, r1;
            if (tid < 16) lut[tid] = nf4.code16[tid];
            if (GLU && tid >= 16 && tid < 32) lut[tid] = fu.nf4_2.code16[tid - 16];
            // steps from KT_thin on (a thin last term) copy bf16 weights: nothing to load or decode for them
            if (KT_thin > 0) nf4_load(0, r0);
            if (KT_thin > 1) nf4_load(1, r1);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();  // the code table is in LDS
            if (KT_thin > 0) nf4_decode(0, r0);
            auto step = [&](int kt, Nf4Regs &r_even, Nf4Regs &r_odd) {
                // on entry: r_odd holds step kt+1 (in flight or landed), r_even is free
                wait_vmcnt<0>();
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");  // decoded weights of step kt are written
                __builtin_amdgcn_s_barrier();
                if (kt + 1 < KT) issue(kt + 1);
                if (kt + 2 < KT_thin) nf4_load(kt + 2, r_even);
                const unsigned char *sa = smem + (kt % S) * STAGE_BYTES, *sb = sa + SA::kBytes;
                // The decode of the next step's weights (vector ALU) is spread over the four
                // sub-steps, so that it runs under this step's matrix instructions instead of
                // ahead of them: the two waves of a SIMD move in lock step from barrier to
                // barrier and would otherwise both decode first and both multiply after.
                // (Forcing a finer interleave with scheduling barriers, or one straight-line
                // variant of the step per case, made the register allocator spill.)
                static_assert(KS == 4, "one packed dword per sub-step");
                const bool dec = nf4_on && kt + 1 < KT_thin;
                bf16x8 fa[2][TA], fb[2][TN];
#pragma unroll
                for (int bj = 0; bj < TN; ++bj) fb[0][bj] = fo_b.load(sb, bj, 0);
#pragma unroll
                for (int t = 0; t < TA; ++t) fa[0][t] = fo_a.load(sa, t, 0);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    if (ks + 1 < KS) {
#pragma unroll
                        for (int bj = 0; bj < TN; ++bj) fb[(ks + 1) & 1][bj] = fo_b.load(sb, bj, ks + 1);
#pragma unroll
                        for (int t = 0; t < TA; ++t) fa[(ks + 1) & 1][t] = fo_a.load(sa, t, ks + 1);
                    }
                    if (dec) nf4_decode_part(kt + 1, r_odd, ks);
#pragma unroll
                    for (int t = 0; t < TA; ++t)
#pragma unroll
                        for (int bj = 0; bj < TN; ++bj)
                            acc[t][bj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[ks & 1][bj], fa[ks & 1][t],
                                                                                 acc[t][bj], 0, 0, 0);
                }
            };
            for (int kt = 0; kt < KT; kt += 2) {
                step(kt, r0, r1);
                if (kt + 1 < KT) step(kt + 1, r1, r0);
            }
        };
        // a wave without valid rows still copies, and multiplies one block nobody stores
        auto run = [&](auto ta_tag) {
            if constexpr (NF4)
                k_loop_nf4(ta_tag);
            else
                k_loop(ta_tag);
        };
        if (TM == 1 || active <= 1)
            run(IC<1>{});
        else if (TM == 2 || active == 2)
            run(IC<(TM >= 2 ? 2 : 1)>{});
        else if (TM == 3 || active == 3)
            run(IC<(TM >= 3 ? 3 : 1)>{});
        else
            run(IC<TM>{});

        // ---- epilogue
        const int h = lane >> 5, rl = lane & 31;
        // where the output is staged: the stages are idle, except (XT) the one that receives the next tile's
        // first step; the other one is the stage the last step was read from
        unsigned char *const ep_base = smem + (XT && xt_next ? ((xt_g + KT + 1) & 1) * STAGE_BYTES : 0);
        if (XT) {
            xt_g = (xt_g + KT) & 1;
            xt_fetched = xt_next;
        }
        if constexpr (GLU) {
            // Each wave stages its 32-row block of one product in LDS as bf16; the wave that holds
            // the other product of the same rows and columns does the same; then each of the two
            // takes 16 of the 32 rows, reads both products back as whole 16-byte chunks, and
            // stores silu(gate) * up (and the products themselves where the caller wants them).
            __builtin_amdgcn_s_barrier();  // all waves are done reading the last stage
            constexpr int ROWB = WTN * 2 + 16;  // padded row, bytes
            constexpr int CPR = WTN / 8;        // 16-byte chunks per row
            const int up = wn / HW, cw = wn % HW;
            unsigned char *ep = smem + wave * (32 * ROWB);
            const unsigned char *ep_e = smem + (wm * WGN + cw) * (32 * ROWB);
            const unsigned char *ep_g = smem + (wm * WGN + cw + HW) * (32 * ROWB);
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                if (t < active) {
#pragma unroll
                    for (int bj = 0; bj < TN; ++bj)
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            union {
                                bf16_t e[4];
                                uint2_t v;
                            } pk;
#pragma unroll
                            for (int u = 0; u < 4; ++u) pk.e[u] = (bf16_t)acc[t][bj][4 * g + u];
                            *(uint2_t *)(ep + rl * ROWB + (bj * 32 + 8 * g + 4 * h) * 2) = pk.v;
                        }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_s_barrier();  // both products of the block are staged
                if (t < active) {
                    for (int q = lane; q < 16 * CPR; q += 64) {
                        const int row_l = 16 * up + q / CPR, lcol = (q % CPR) * 8;
                        const int row = i0 + (wm + WGM * t) * 32 + row_l;
                        const int col = j0 + cw * WTN + lcol;
                        if (row >= i_end || col >= j_end) continue;
                        const bf16x8 e8 = *(const bf16x8 *)(ep_e + row_l * ROWB + lcol * 2);
                        const bf16x8 g8 = *(const bf16x8 *)(ep_g + row_l * ROWB + lcol * 2);
                        bf16x8 h8;
#pragma unroll
                        for (int u = 0; u < 8; ++u) h8[u] = silu_fwd_one<bf16_t>(e8[u], g8[u]);
                        const int64_t o = (int64_t)row * ldc + col;
                        __builtin_nontemporal_store(h8, (bf16x8 *)((bf16_t *)c_base + o));
                        if (fu.c_e) __builtin_nontemporal_store(e8, (bf16x8 *)((bf16_t *)fu.c_e + o));
                        if (fu.c_g) __builtin_nontemporal_store(g8, (bf16x8 *)((bf16_t *)fu.c_g + o));
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_s_barrier();  // the staging areas are free again
            }
        } else if (sizeof(TO) == 2 && !accumulate) {
            // One 32-row block of the wave at a time: stage it in LDS as bf16 (8 bytes per lane and
            // write), then store whole rows, 16 bytes per lane, instead of short stores scattered
            // over 32 rows.
            __builtin_amdgcn_s_barrier();  // all waves are done reading the last stage
            constexpr int ROWB = WTN * 2 + 16;  // padded row, bytes
            constexpr int CPR = WTN / 8;        // 16-byte chunks per row
            unsigned char *ep = ep_base + wave * (32 * ROWB);
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                if (t >= active) continue;
#pragma unroll
                for (int bj = 0; bj < TN; ++bj)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        union {
                            bf16_t e[4];
                            uint2_t v;
                        } pk;
#pragma unroll
                        for (int u = 0; u < 4; ++u) pk.e[u] = (bf16_t)(acc[t][bj][4 * g + u] * alpha);
                        *(uint2_t *)(ep + rl * ROWB + (bj * 32 + 8 * g + 4 * h) * 2) = pk.v;
                    }
                // the same wave reads back what it wrote: LDS operations of one wave complete in order
                const int row_base = i0 + (wm + WGM * t) * 32;
                if constexpr (BWG) {
                    // the product is the gradient of h = silu(e) g: its pieces meet the same pieces of e and g
                    // (requested for the whole block first) and leave as de and dg, h where asked for
                    // One piece at a time: with two in flight the 320 x 192 tile spills ten registers, with a whole
                    // block's twelve loads fifty, and either is slower.
                    constexpr int NQ = (32 * CPR + 63) / 64, QB = 1;  // pieces per lane; requested QB at a time
#pragma unroll
                    for (int q0 = 0; q0 < NQ; q0 += QB) {
                        uint4_t e_in[QB], g_in[QB];
#pragma unroll
                        for (int qi = 0; qi < QB; ++qi) {
                            const int q = (q0 + qi) * 64 + lane, row = row_base + q / CPR, col = j0 + wn * WTN + (q % CPR) * 8;
                            if (q0 + qi >= NQ || q >= 32 * CPR || row >= i_end || col >= j_end) continue;
                            const int64_t o = (int64_t)row * ldc + col;
                            e_in[qi] = __builtin_nontemporal_load((const uint4_t *)((const bf16_t *)fu.bw_e + o));
                            g_in[qi] = __builtin_nontemporal_load((const uint4_t *)((const bf16_t *)fu.bw_g + o));
                        }
#pragma unroll
                        for (int qi = 0; qi < QB; ++qi) {
                            const int q = (q0 + qi) * 64 + lane, row_l = q / CPR, lcol = (q % CPR) * 8;
                            const int row = row_base + row_l, col = j0 + wn * WTN + lcol;
                            if (q0 + qi >= NQ || q >= 32 * CPR || row >= i_end || col >= j_end) continue;
                            union {
                                uint4_t u;
                                bf16x8 v;
                            } dh8, e8, g8, h8, de8, dg8;
                            dh8.u = *(const uint4_t *)(ep + row_l * ROWB + lcol * 2);
                            e8.u = e_in[qi];
                            g8.u = g_in[qi];
#pragma unroll
                            for (int u = 0; u < 8; ++u) {
                                bf16_t h1, de1, dg1;
                                silu_bwd_one<bf16_t>(dh8.v[u], e8.v[u], g8.v[u], h1, de1, dg1);
                                h8.v[u] = h1;
                                de8.v[u] = de1;
                                dg8.v[u] = dg1;
                            }
                            const int64_t o = (int64_t)row * ldc + col;
                            __builtin_nontemporal_store(de8.u, (uint4_t *)((bf16_t *)fu.bw_de + o));
                            __builtin_nontemporal_store(dg8.u, (uint4_t *)((bf16_t *)fu.bw_dg + o));
                            if (fu.bw_h) __builtin_nontemporal_store(h8.u, (uint4_t *)((bf16_t *)fu.bw_h + o));
                        }
                    }
                    continue;
                }
                for (int q = lane; q < 32 * CPR; q += 64) {
                    const int row_l = q / CPR, lcol = (q % CPR) * 8;
                    const int row = row_base + row_l;
                    const int col = j0 + wn * WTN + lcol;
                    if (row >= i_end || col >= j_end) continue;
                    // the output width is a multiple of 8: a chunk is inside or outside as a whole
                    // written once, read by a later kernel: streaming store (dW 205 -> 199 us)
                    __builtin_nontemporal_store(*(const uint4_t *)(ep + row_l * ROWB + lcol * 2),
                                                (uint4_t *)((bf16_t *)c_base + (int64_t)row * ldc + col));
                }
            }
        } else if (sizeof(TO) == 2) {
            // accumulate into a bf16 output: the products are staged in fp32, the old values are
            // read as whole rows, and the sum is rounded once
            __builtin_amdgcn_s_barrier();  // all waves are done reading the last stage
            constexpr int ROWF = WTN * 4 + 16;  // padded row of floats, bytes
            constexpr int CPR = WTN / 8;        // 16-byte output chunks per row
            static_assert(NW * 32 * ROWF <= S * STAGE_BYTES, "fp32 output staging must fit in the stages");
            unsigned char *ep = ep_base + wave * (32 * ROWF);
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                if (t >= active) continue;
#pragma unroll
                for (int bj = 0; bj < TN; ++bj)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        floatx4 v;
#pragma unroll
                        for (int u = 0; u < 4; ++u) v[u] = acc[t][bj][4 * g + u] * alpha;
                        *(floatx4 *)(ep + rl * ROWF + (bj * 32 + 8 * g + 4 * h) * 4) = v;
                    }
                const int row_base = i0 + (wm + WGM * t) * 32;
                for (int q = lane; q < 32 * CPR; q += 64) {
                    const int row_l = q / CPR, lcol = (q % CPR) * 8;
                    const int row = row_base + row_l;
                    const int col = j0 + wn * WTN + lcol;
                    if (row >= i_end || col >= j_end) continue;
                    bf16x8 *dst = (bf16x8 *)((bf16_t *)c_base + (int64_t)row * ldc + col);
                    const bf16x8 old = *dst;
                    const floatx4 lo = *(const floatx4 *)(ep + row_l * ROWF + lcol * 4);
                    const floatx4 hi = *(const floatx4 *)(ep + row_l * ROWF + lcol * 4 + 16);
                    bf16x8 out;
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        out[u] = (bf16_t)(lo[u] + (float)old[u]);
                        out[4 + u] = (bf16_t)(hi[u] + (float)old[4 + u]);
                    }
                    *dst = out;
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                if (t >= active) continue;
                const int row = i0 + (wm + WGM * t) * 32 + rl;
                if (row >= i_end) continue;
#pragma unroll
                for (int bj = 0; bj < TN; ++bj)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int col = j0 + wn * WTN + bj * 32 + 8 * g + 4 * h;
                        TO *p = c_base + (int64_t)row * ldc + col;
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            if (col + u >= j_end) continue;
                            float v = alpha * acc[t][bj][4 * g + u];
                            if (accumulate) v += to_f32(p[u]);
                            p[u] = from_f32<TO>(v);
                        }
                    }
            }
        }
    }
}

// MODES: bit 0 FWD (and NF4), bit 1 DX, bit 2 DW -- the products a tile configuration is built for.
template <int MB, int NB, int BK, int S, int WGM, int WGN, int MODES, typename TO>
int launch_pipe(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                int K, int E, float alpha, int accumulate, const Nf4Params *nf4, const FwdFusion *fusion,
                hipStream_t stream) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int STAGE_BYTES = (MB + NB) * 32 * BK * 2;
    constexpr int EP_BYTES = WGM * WGN * 32 * ((NB / WGN) * 64 + 16);
    static_assert(EP_BYTES <= S * STAGE_BYTES, "the output staging reuses the stages");
    // stages | two NF4 code tables | three per-expert prefix tables
    constexpr int LDS_BYTES = S * STAGE_BYTES + 128 + 3 * (kMaxTableExperts + 1) * 4;
    static_assert(LDS_BYTES <= 160 * 1024, "LDS capacity of a CDNA4 compute unit");
    const bf16_t *pa = (const bf16_t *)a, *pb = (const bf16_t *)b;
    TO *pc = (TO *)c;
    // one persistent workgroup per CU, two where two fit (the small rings of the thin products)
    constexpr int PER_CU = LDS_BYTES <= 80 * 1024 ? 2 : 1;
    const int grid = device_info().cu_count / kXcd * kXcd * PER_CU;
    const Nf4Params none = {nullptr, nullptr, 0};
    const FwdFusion no_fusion = {nullptr, 1, nullptr, none, nullptr, nullptr, nullptr, nullptr, nullptr, 0, nullptr};
    const FwdFusion fu = fusion ? *fusion : no_fusion;
    const bool glu = fu.b2 != nullptr && fu.a2 == nullptr;
    if ((glu || fu.row_idx) && mode != MODE_FWD) return MFL_ERR_UNSUPPORTED;
    if (fu.a2 != nullptr && (mode != MODE_DX || nf4 != nullptr || fu.b2 == nullptr)) return MFL_ERR_UNSUPPORTED;
    if (fu.at != nullptr && (mode == MODE_DW || fu.bt == nullptr || (glu && (fu.bt2 == nullptr || nf4 != nullptr)))) return MFL_ERR_UNSUPPORTED;
#define MFL_PIPE(MODE, NF4, GLU)                                                                                \
    {                                                                                                           \
        auto kern = gemm_pipe_kernel<MB, NB, BK, S, WGM, WGN, MODE, NF4, GLU, TO>;                              \
        static PerDeviceOnce attr;                                                                              \
        const hipError_t e = attr.run([&] {                                                                     \
            return hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,          \
                                       LDS_BYTES);                                                              \
        });                                                                                                     \
        if (e != hipSuccess) return (int)e;                                                                     \
        kern<<<grid, NT, LDS_BYTES, stream>>>(pa, pb, m_sizes, ms_i64, pc, R, N, K, E, alpha, accumulate,       \
                                              NF4 ? *nf4 : none, fu);                                           \
    }
    // MODES bit 3: the configuration is also built with the GLU epilogue (bf16 output only)
    constexpr bool GLU_OK = (MODES & 8) && WGN % 2 == 0 && sizeof(TO) == 2 && BK == 64;
    if (glu && fu.at != nullptr) {
        if constexpr (GLU_OK && (MODES & 16) != 0) MFL_PIPE(MODE_FWD, false, 3)
        else return MFL_ERR_UNSUPPORTED;
    } else if (glu) {
        if constexpr (GLU_OK) {
            if (nf4 != nullptr) {
                if constexpr (S == 2 && NB * 64 <= NT) MFL_PIPE(MODE_FWD, true, true)
                else return MFL_ERR_UNSUPPORTED;
            } else {
                MFL_PIPE(MODE_FWD, false, true)
            }
        } else {
            return MFL_ERR_UNSUPPORTED;
        }
    } else if (fu.at != nullptr) {
        // MODES bit 4: the configuration is also built with the thin last term
        if constexpr ((MODES & 16) != 0 && (MODES & 3) == 3) {
            if (nf4 != nullptr) {
                if constexpr (S == 2 && BK == 64 && NB * 64 <= NT) {
                    if (mode == MODE_FWD) MFL_PIPE(MODE_FWD, true, 2)
                    else MFL_PIPE(MODE_DX, true, 2)
                } else {
                    return MFL_ERR_UNSUPPORTED;
                }
            } else if (mode == MODE_FWD) {
                MFL_PIPE(MODE_FWD, false, 2)
            } else {
                MFL_PIPE(MODE_DX, false, 2)
            }
        } else {
            return MFL_ERR_UNSUPPORTED;
        }
    } else if (fu.bw_e != nullptr) {
        // the gated unit's backward in the epilogue: built with the configurations that have the GLU epilogue
        if constexpr ((MODES & 8) != 0 && (MODES & 2) != 0 && sizeof(TO) == 2) {
            if (mode != MODE_DX || nf4 != nullptr || accumulate) return MFL_ERR_UNSUPPORTED;
            MFL_PIPE(MODE_DX, false, 4)
        } else {
            return MFL_ERR_UNSUPPORTED;
        }
    } else if (nf4 != nullptr && mode == MODE_DX) {
        if constexpr ((MODES & 2) && S == 2 && BK == 64 && NB * 64 <= NT) MFL_PIPE(MODE_DX, true, false)
        else return MFL_ERR_UNSUPPORTED;
    } else if (nf4 != nullptr) {
        if constexpr ((MODES & 1) && S == 2 && BK == 64 && NB * 64 <= NT) MFL_PIPE(MODE_FWD, true, false)
        else return MFL_ERR_UNSUPPORTED;
    } else if (mode == MODE_FWD) {
        if constexpr (MODES & 1) MFL_PIPE(MODE_FWD, false, false)
        else return MFL_ERR_UNSUPPORTED;
    } else if (mode == MODE_DX) {
        if constexpr (MODES & 2) MFL_PIPE(MODE_DX, false, false)
        else return MFL_ERR_UNSUPPORTED;
    } else {
        if constexpr (MODES & 4) MFL_PIPE(MODE_DW, false, false)
        else return MFL_ERR_UNSUPPORTED;
    }
#undef MFL_PIPE
    return launch_status();
}

}  // namespace

// Tile configuration of every launch: 0 = the built-in table below.  A variable only in tuning builds
// (the library proper has no switch and no mutable state here).
#ifdef MFL_TUNING_BUILD
int g_pipe_config = 0;
#else
namespace {
constexpr int g_pipe_config = 0;
}
#endif

namespace {

int dispatch_pipe(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                  int K, int E, int out_dtype, float alpha, int accumulate, const Nf4Params *nf4,
                  const FwdFusion *fusion, hipStream_t stream) {
#define MFL_LAUNCH(MB, NB, BK, S, WGM, WGN, MODES)                                                              \
    (out_dtype == MFL_BF16                                                                                     \
         ? launch_pipe<MB, NB, BK, S, WGM, WGN, MODES, bf16_t>(mode, a, b, m_sizes, ms_i64, c, R, N, K, E, alpha, \
                                                               accumulate, nf4, fusion, stream)                \
         : launch_pipe<MB, NB, BK, S, WGM, WGN, MODES, float>(mode, a, b, m_sizes, ms_i64, c, R, N, K, E, alpha,  \
                                                              accumulate, nf4, fusion, stream))
    // Tile table (row blocks, column blocks, BK, stages, waves along M, waves along N, products).
    // The default per product was picked from timings at the Qwen3-30B-A3B expert shapes.
    // Row-grouped products at a few hundred rows per expert: 320 x 192 tiles, i.e. every expert of
    // up to 320 rows is one tile per 192-column slice (4 slices of N = 768: 512 tiles, two per CU).
    // From about 512 rows per expert on, and in DW: square 256 x 256 tiles (fewer bytes per flop).
    // Rank-r LoRA products (one side of the output at most 64 wide) are bound by streaming the
    // wide operand: small stages, many of them, so that a CU keeps 100 KiB and more in flight.
    // Products with the GLU epilogue (bit 3): the configurations whose waves along N split in two halves.
    const bool glu = fusion != nullptr && fusion->b2 != nullptr && fusion->a2 == nullptr;
    int cfg = g_pipe_config;
    if (glu && (cfg == 0 || nf4 != nullptr)) {
        cfg = R >= (int64_t)512 * E ? 8 : (R <= (int64_t)kFlatTileRowsPerExpert * E && nf4 == nullptr) ? 15 : 3;
    } else if (cfg == 0 || nf4 != nullptr) {
        if (mode == MODE_DW)
            cfg = (N <= 64 || K <= 64) ? 11 : 8;
        else {
            // packed weights with an output of 1024 columns and more that is a multiple of 256 wide, up to 232 rows per
            // expert: 256 x 256 tiles as well (8 column slices an expert instead of 11 of 192 columns)
            const bool nf4_wide = nf4 != nullptr && N % 256 == 0 && N >= 1024 && R <= (int64_t)232 * E;
            cfg = (N <= 64 && nf4 == nullptr) ? 10
                  : (R <= (int64_t)kFlatTileRowsPerExpert * E && nf4 == nullptr) ? 15
                  : (R >= (int64_t)512 * E || nf4_wide) ? 8 : 3;
        }
    }
    switch (cfg) {
        case 1:
            return MFL_LAUNCH(4, 4, 64, 4, 2, 2, 7);
        case 2:
            return MFL_LAUNCH(8, 4, 64, 3, 4, 2, 7);
        case 3:
            return MFL_LAUNCH(10, 6, 64, 2, 4, 2, 31);
        case 4:
            return MFL_LAUNCH(10, 4, 64, 2, 4, 2, 7);
        case 15:  // a few rows per expert (decode): the weights are all the traffic; flat 64 x 128 tiles,
                  // 3 stages of 24 KiB, two workgroups per CU (one with 6 stages: 85 instead of 77 us for
                  // 2048 rows over 128 experts, N = 768, K = 2048)
            return MFL_LAUNCH(2, 4, 64, 3, 2, 4, 27);
        case 10:  // thin output of a row-grouped product: 128 rows x 64 columns, 3 stages of 24 KiB, two
                  // workgroups per CU (one's set-up and epilogue under the other's loop; one workgroup with 6
                  // stages: x A^T 57 instead of 53 us, dy B 28.5 instead of 23.5 us at 65536 rows)
            return MFL_LAUNCH(4, 2, 64, 3, 4, 1, 19);
        case 11:  // dW with a thin side: 64 x 64 tiles (an expert's reduction is spread over as many
                  // workgroups as its wide side has 64-column slices), 8 stages of 16 KiB
            return MFL_LAUNCH(2, 2, 64, 8, 2, 2, 4);
        default:
            return MFL_LAUNCH(8, 8, 64, 2, 2, 4, 31);
    }
#undef MFL_LAUNCH
}

}  // namespace

namespace {

// Checks the fusion request of a forward product and translates it for the kernel.
// Returns MFL_ERR_UNSUPPORTED for what the pipelined kernels do not take.
int make_fusion(const GemmFusion *f, int K, bool nf4, FwdFusion *out) {
    *out = FwdFusion{nullptr, 1, nullptr, Nf4Params{nullptr, nullptr, 0}, nullptr, nullptr, nullptr, nullptr, nullptr, 0, nullptr};
    if (f == nullptr) return MFL_OK;
    if (f->row_idx != nullptr) {
        // the kernel addresses the source rows with 32-bit byte offsets
        if (f->idx_div <= 0 || f->src_rows <= 0 || f->src_rows * (int64_t)K * 2 > 0xffffffffll)
            return MFL_ERR_UNSUPPORTED;
        out->row_idx = f->row_idx;
        out->idx_div = f->idx_div;
    }
    if (f->xt != nullptr) {
        // with a second weight matrix and no second left operand (the gated unit) the thin term needs thin weights
        // for that matrix too
        const bool glu_thin = f->w2 != nullptr && f->x2 == nullptr;
        if (f->wt == nullptr || f->kt < 8 || f->kt % 8 != 0 || !aligned(f->xt, 16) || !aligned(f->wt, 16) ||
            f->row_idx != nullptr || (glu_thin && (nf4 || f->wt2 == nullptr || !aligned(f->wt2, 16))))
            return MFL_ERR_UNSUPPORTED;
        out->at = f->xt;
        out->bt = f->wt;
        out->bt2 = glu_thin ? f->wt2 : nullptr;
        out->kthin = f->kt;
    }
    if (f->bw_e != nullptr) {
        if (nf4 || f->bw_g == nullptr || f->bw_de == nullptr || f->bw_dg == nullptr || f->row_idx != nullptr ||
            f->x2 != nullptr || f->w2 != nullptr || f->xt != nullptr || !aligned(f->bw_e, 16) || !aligned(f->bw_g, 16) ||
            !aligned(f->bw_de, 16) || !aligned(f->bw_dg, 16) || !aligned(f->bw_h, 16))
            return MFL_ERR_UNSUPPORTED;
        out->bw_e = f->bw_e;
        out->bw_g = f->bw_g;
        out->bw_de = f->bw_de;
        out->bw_dg = f->bw_dg;
        out->bw_h = f->bw_h;
    }
    if (f->x2 != nullptr) {
        // two-term input gradient: whole reduction steps only, bf16 weights
        if (nf4 || f->w2 == nullptr || K % 64 != 0 || !aligned(f->x2, 16) || !aligned(f->w2, 16) ||
            f->row_idx != nullptr)
            return MFL_ERR_UNSUPPORTED;
        out->a2 = f->x2;
        out->b2 = f->w2;
        return MFL_OK;
    }
    if (f->w2 != nullptr) {
        out->b2 = f->w2;
        out->c_e = f->e_out;
        out->c_g = f->g_out;
        if (!aligned(f->w2, nf4 ? 4 : 16) || !aligned(f->e_out, 16) || !aligned(f->g_out, 16)) return MFL_ERR_UNSUPPORTED;
        if (nf4) {
            int shift = 0;
            while ((1 << shift) < f->blocksize_2) ++shift;
            if (f->blocksize_2 < 8 || f->code16_2 == nullptr || f->absmax_2 == nullptr) return MFL_ERR_UNSUPPORTED;
            out->nf4_2 = Nf4Params{f->code16_2, f->absmax_2, shift};
        }
    }
    return MFL_OK;
}

}  // namespace

int gemm_bf16_pipe(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                   int K, int E, int out_dtype, float alpha, int accumulate, hipStream_t stream,
                   const GemmFusion *fusion) {
    if (g_pipe_config < 0 || E > kMaxTableExperts) return MFL_ERR_UNSUPPORTED;
    if (!aligned(a, 16) || !aligned(b, 16) || !aligned(c, 16)) return MFL_ERR_UNSUPPORTED;
    if (out_dtype != MFL_BF16 && out_dtype != MFL_F32) return MFL_ERR_UNSUPPORTED;
    if (mode != MODE_DW && (K % 8 != 0 || K < 8 || N % 8 != 0 || N < 8)) return MFL_ERR_UNSUPPORTED;
    if (mode == MODE_DW && (N % 8 != 0 || K % 8 != 0 || N < 8 || K < 8)) return MFL_ERR_UNSUPPORTED;
    FwdFusion fu;
    if (fusion != nullptr) {
        // two full terms: DX; a thin last term: FWD or DX; everything else: FWD
        if (mode == MODE_DW || (fusion->x2 != nullptr && mode != MODE_DX) ||
            (mode == MODE_DX && fusion->x2 == nullptr && fusion->xt == nullptr && fusion->bw_e == nullptr))
            return MFL_ERR_UNSUPPORTED;
        // the gated unit's backward sits in the bf16, non-accumulating epilogue of DX
        if (fusion->bw_e != nullptr && (mode != MODE_DX || out_dtype != MFL_BF16 || accumulate || alpha != 1.0f))
            return MFL_ERR_UNSUPPORTED;
        if (fusion->x2 == nullptr && fusion->w2 != nullptr && (out_dtype != MFL_BF16 || accumulate || alpha != 1.0f))
            return MFL_ERR_UNSUPPORTED;
        const int rc = make_fusion(fusion, K, false, &fu);
        if (rc) return rc;
    }
    if (mode != MODE_DW && R <= 0) return MFL_OK;
    return dispatch_pipe(mode, a, b, m_sizes, ms_i64, c, R, N, K, E, out_dtype, alpha, accumulate, nullptr,
                         fusion ? &fu : nullptr, stream);
}

int gemm_nf4_pipe(const void *x, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                  const void *m_sizes, int ms_i64, void *y, int64_t R, int N, int K, int E, int out_dtype,
                  hipStream_t stream, const GemmFusion *fusion) {
    if (g_pipe_config < 0 || E > kMaxTableExperts) return MFL_ERR_UNSUPPORTED;
    int shift = 0;
    while ((1 << shift) < blocksize) ++shift;
    // a 16-byte LDS chunk (8 weights along K) must not straddle two absmax blocks
    if (K % 64 != 0 || N % 8 != 0 || N < 8 || blocksize < 8) return MFL_ERR_UNSUPPORTED;
    // With few rows per expert the streaming kernel (32-row tiles, weights decoded once per tile from packed
    // bytes in LDS) is ahead; the caller tries it first.
    if (R < (int64_t)kNf4DecodeRowsPerExpert * E && fusion == nullptr) return MFL_ERR_UNSUPPORTED;
    if (!aligned(x, 16) || !aligned(wq, 4) || !aligned(y, 16)) return MFL_ERR_UNSUPPORTED;
    if (out_dtype != MFL_BF16 && out_dtype != MFL_F32) return MFL_ERR_UNSUPPORTED;
    FwdFusion fu;
    if (fusion != nullptr) {
        if (fusion->w2 != nullptr && out_dtype != MFL_BF16) return MFL_ERR_UNSUPPORTED;
        const int rc = make_fusion(fusion, K, true, &fu);
        if (rc) return rc;
    }
    if (R <= 0) return MFL_OK;
    const Nf4Params nf4 = {code16, absmax, shift};
    return dispatch_pipe(MODE_FWD, x, wq, m_sizes, ms_i64, y, R, N, K, E, out_dtype, 1.0f, 0, &nf4,
                         fusion ? &fu : nullptr, stream);
}

int gemm_nf4_pipe_dx(const void *dy, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                     const void *m_sizes, int ms_i64, void *dx, int64_t R, int N, int K, int E, int out_dtype,
                     float alpha, int accumulate, hipStream_t stream, const GemmFusion *fusion) {
    if (g_pipe_config < 0 || E > kMaxTableExperts) return MFL_ERR_UNSUPPORTED;
    int shift = 0;
    while ((1 << shift) < blocksize) ++shift;
    // a thread decodes 32 consecutive output columns of one reduction row: whole segments only
    if (K % 64 != 0 || N % 32 != 0 || N < 32 || blocksize < 8) return MFL_ERR_UNSUPPORTED;
    if (!aligned(dy, 16) || !aligned(wq, 16) || !aligned(dx, 16)) return MFL_ERR_UNSUPPORTED;
    if (out_dtype != MFL_BF16 && out_dtype != MFL_F32) return MFL_ERR_UNSUPPORTED;
    FwdFusion fu;
    if (fusion != nullptr) {
        // only the thin last term
        if (fusion->xt == nullptr || fusion->x2 != nullptr || fusion->w2 != nullptr || fusion->row_idx != nullptr ||
            accumulate || alpha != 1.0f)
            return MFL_ERR_UNSUPPORTED;
        const int rc = make_fusion(fusion, K, true, &fu);
        if (rc) return rc;
    }
    if (R <= 0) return MFL_OK;
    const Nf4Params nf4 = {code16, absmax, shift};
    return dispatch_pipe(MODE_DX, dy, wq, m_sizes, ms_i64, dx, R, N, K, E, out_dtype, alpha, accumulate, &nf4,
                         fusion ? &fu : nullptr, stream);
}

}  // namespace mfl
