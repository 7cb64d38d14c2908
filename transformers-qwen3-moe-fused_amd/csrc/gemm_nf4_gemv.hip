// Fused NF4 grouped product for batches of a few rows per expert (256 < K <= 2048): a matrix-vector form.
//
// With one or two rows per expert there is nothing for a matrix core to share: a 32-row MFMA tile would
// be 3 to 6 % full, and what the launch has to do is pull every routed expert's packed weights through
// the chip once.  So no tile and no LDS stage:
//   * a wave owns two output columns at a time, 16 apart (one in the gated form, where the second matrix takes
//     the registers).  Its 64 lanes lie along the reduction: load i of a column gives lane l the dword of 8
//     packed weights k = (64 i + l) * 8 .., i.e. a wave reads 256 consecutive bytes per load and a column of
//     K = 2048 in four.  The scale of those 8 weights is one float (blocks
//     of at least 8 weights, K a multiple of the block size).
//   * the rows of the group (up to two of one expert) stay in registers for all columns of the group: 16
//     bytes per lane, load and row.
//   * a byte of packed weights is two weights and one dword of bf16 pairs: a 256-entry table in LDS holds
//     the finished pair, and v_dot2_f32_bf16 multiplies it with the row's pair.  An entry is 256 bytes: 32
//     copies for the first matrix, 32 for the second of the gated form; lane l reads copy l & 31, so the 64
//     lookups of a wave meet no bank conflict, and the address 256 * byte + 4 * copy is ONE byte permute.
//     One vector instruction per byte for the address, one per byte and row for the product; the scale goes
//     onto the partial sum of the 8 weights in fp32.
//   * the 64 partial sums of each of the two columns become 32 + 32 in one swap of half waves
//     (v_permlane32_swap) and an add, and five data-parallel-primitive adds finish both at once; lanes 31 and
//     63 store.
//   * one workgroup of 16 waves per CU, as many workgroups as CUs, and the (row group, 32 columns) units of
//     the launch (16 columns in the gated form) dealt out in equal contiguous shares: no second round of
//     workgroups, and a workgroup changes rows once or twice.  Each wave keeps the loads of four columns ahead
//     in registers.
//   * rows of at most 1024 elements: 32 lanes to a column, the wave's second column (16 further on) in lanes
//     32..63, loads of 128 bytes per half wave, no swap before the five adds.
//   What the loop is short of, with 16 waves to a CU, is issue slots, scalar ones first: addresses move by
//   increments, the row count is branched on once per column, and the lookups of a dword wait once.
//
// The product is sum over 8-weight pieces of absmax * (x . bf16(code)), as in the streaming form.
#include <mutex>
#include <type_traits>

#include "common.h"
#include "gemm.h"

namespace mfl {

namespace {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((address_space(3))) void *lds_void_ptr;
typedef const __attribute__((address_space(3))) uint32_t *lds_u32_ptr;

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_fadd_step(float x) {
    // lanes without a source, and rows that the mask leaves out, add 0
    const int y = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, ROW_MASK, 0xf, true);
    return x + __builtin_bit_cast(float, y);
}
// a: 64 partial sums of one column, b: of another.  Returns the first column's sum in lane 31 and the second's in
// lane 63: v_permlane32_swap exchanges lanes 32..63 of its first operand with lanes 0..31 of its second, so the
// sum of the two holds a[l] + a[l + 32] in lanes 0..31 and b[l - 32] + b[l] in lanes 32..63.  (Written out: through
// __builtin_amdgcn_permlane32_swap, with both results feeding one add, the compiler added the first result to
// itself.  The no-ops keep the wait states that the swap and the moves after it need from their neighbours.)
__device__ __forceinline__ float two_sums_to_31_and_63(float a, float b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    float x = a + b;
    x = dpp_fadd_step<0x111, 0xf>(x);  // row_shr 1
    x = dpp_fadd_step<0x112, 0xf>(x);  // row_shr 2
    x = dpp_fadd_step<0x114, 0xf>(x);  // row_shr 4
    x = dpp_fadd_step<0x118, 0xf>(x);  // row_shr 8
    x = dpp_fadd_step<0x142, 0xa>(x);  // row_bcast 15 into rows 1 and 3
    return x;
}

// lanes 0..31 hold the partial sums of one column, lanes 32..63 of another: the sums in lanes 31 and 63
__device__ __forceinline__ float half_sums_to_31_and_63(float x) {
    x = dpp_fadd_step<0x111, 0xf>(x);  // row_shr 1
    x = dpp_fadd_step<0x112, 0xf>(x);  // row_shr 2
    x = dpp_fadd_step<0x114, 0xf>(x);  // row_shr 4
    x = dpp_fadd_step<0x118, 0xf>(x);  // row_shr 8
    x = dpp_fadd_step<0x142, 0xa>(x);  // row_bcast 15 into rows 1 and 3
    return x;
}

__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
}

// Four table reads and one wait for all of them, written out: the compiler would wait before each use, and with
// 16 waves to a CU the issue slots of those waits are not free.  The addresses count from LDS address 0.
__device__ __forceinline__ void lookup4(uint32_t (&pr)[4], uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3) {
    asm volatile(
        "ds_read_b32 %0, %4\n\tds_read_b32 %1, %5\n\tds_read_b32 %2, %6\n\tds_read_b32 %3, %7\n\ts_waitcnt lgkmcnt(0)"
        : "=&v"(pr[0]), "=&v"(pr[1]), "=&v"(pr[2]), "=&v"(pr[3])
        : "v"(a0), "v"(a1), "v"(a2), "v"(a3));
}

constexpr int kGemvThreads = 1024;
constexpr int kGemvTable = 65536;


// The LDS address of the pair of packed byte `B` of w: 256 * byte + lane_copy (the lane's copy of the table, one
// byte), put together by one byte permute.
template <int B>
__device__ __forceinline__ uint32_t pair_address(uint32_t w, uint32_t lane_copy) {
    // byte 0 of the result: byte 0 of lane_copy; byte 1: byte B of w; bytes 2 and 3: zero
    return __builtin_amdgcn_perm(w, lane_copy, 0x0c0c0000u | ((4u + B) << 8));
}

// NL: loads per column (K <= 512 NL); ROWS: rows per group; D: columns whose loads a wave keeps in flight
template <int NL, int ROWS, int D, bool GLU, bool EXACT, bool HALF, typename TO>
__global__ __launch_bounds__(kGemvThreads) void nf4_gemv_kernel(const bf16_t *__restrict__ x,
                                                                const int32_t *__restrict__ row_idx, int idx_div,
                                                                Nf4Matrix w0, Nf4Matrix w1,
                                                                const void *__restrict__ m_sizes, int ms_i64,
                                                                TO *__restrict__ y, TO *__restrict__ e_out,
                                                                TO *__restrict__ g_out, int64_t R, int N, int K,
                                                                int E, int units_n, int max_groups) {
    constexpr int CB = GLU ? 2 : 1;
    // Columns per wave and unit: two, 16 apart, for the plain product (the loop's scalar work and the sum over the
    // lanes are shared by both); one for the gated form, whose second matrix leaves no registers for a second column.
    constexpr int COLS = (GLU || HALF) ? 1 : 2;
    // HALF (rows of at most 1024 elements): 32 lanes to a column, the wave's second column (16 further on) in its
    // upper 32 lanes instead of in registers of its own: a load serves both, and the sums need no swap.
    constexpr int UCOLS = HALF ? 32 : 16 * COLS;  // columns of a unit per wave-column: 16 waves x UCOLS / 16
    static_assert(!(HALF && EXACT), "");
    static_assert(D % CB == 0, "the matrix of a ring slot is fixed");
    extern __shared__ __attribute__((aligned(256))) unsigned char smem[];
    unsigned char *const table = smem;                      // kGemvTable bytes
    int *const grp_e = (int *)(smem + kGemvTable);          // expert | rows << 16
    int *const grp_r = grp_e + max_groups;                  // first row
    int *const n_groups_s = grp_r + max_groups;
    int *const ms_s = n_groups_s + 1;                       // the E counts
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // the lookups address the table from LDS address 0: the kernel has no static LDS in front of the dynamic
    // (the launcher asks the runtime and does not launch a build that has)
    // the counts, asked for first: their latency runs under the filling of the table
    int ms_own[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int e = tid + j * kGemvThreads;
        ms_own[j] = e < E ? load_msize(m_sizes, ms_i64, e) : 0;
    }
    // ---- pair table: entry b = bf16(code[b >> 4]) in the low half (the first of the two weights is the high
    // nibble), bf16(code[b & 15]) in the high half.  Entry b is the 256 bytes at 256 b: 32 copies for the first
    // matrix, 32 for the second; thread t writes 64 of the bytes of entry t & 255.
    {
        const int b = tid & 255, part = tid >> 8;
        if (part < 2 * CB) {
            const float *const code = part < 2 ? w0.code16 : w1.code16;
            union {
                bf16_t e[2];
                uint32_t u;
            } pr;
            pr.e[0] = (bf16_t)code[b >> 4];
            pr.e[1] = (bf16_t)code[b & 15];
            const uint4_t v = {pr.u, pr.u, pr.u, pr.u};
            uint4_t *const dst = (uint4_t *)(table + b * 256 + part * 64);
#pragma unroll
            for (int j = 0; j < 4; ++j) dst[j] = v;
        }
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int e = tid + j * kGemvThreads;
        if (e < E) ms_s[e] = ms_own[j];
    }
    __syncthreads();
    // ---- row groups in the order of the experts: group g = rows grp_r[g] .. of expert grp_e[g] & 0xffff
    if (wave == 0) {
        int row_carry = 0, grp_carry = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            int m = e < E ? ms_s[e] : 0;
            if (m < 0) m = 0;
            const int minc = wave_inclusive_scan(m);
            const int64_t start = (int64_t)row_carry + minc - m;
            if (start + m > R) m = start < R ? (int)(R - start) : 0;  // counts that run past the rows given
            const int g = ceil_div(m, ROWS);
            const int ginc = wave_inclusive_scan(g);
            const int gb = grp_carry + ginc - g;
            for (int q = 0; q < g && gb + q < max_groups; ++q) {
                const int rows = m - q * ROWS < ROWS ? m - q * ROWS : ROWS;
                grp_e[gb + q] = e | (rows << 16);
                grp_r[gb + q] = (int)start + q * ROWS;
            }
            row_carry += wave_last(minc);
            grp_carry += wave_last(ginc);
        }
        if (lane == 0) *n_groups_s = grp_carry < max_groups ? grp_carry : max_groups;
    }
    __syncthreads();

    // ---- this workgroup's share of the units (row group, 16 columns), row group major
    // (equal shares, the first U % gridDim.x workgroups one unit more; the host keeps U below 2^31)
    const uint32_t U = (uint32_t)*n_groups_s * (uint32_t)units_n;
    const uint32_t share = U / gridDim.x, extra = U % gridDim.x;
    const uint32_t u_begin = blockIdx.x * share + (blockIdx.x < extra ? blockIdx.x : extra);
    const uint32_t u_end = u_begin + share + (blockIdx.x < extra ? 1 : 0);
    if (u_begin >= u_end) return;
    const int n_items = (int)(u_end - u_begin) * CB;  // (unit, matrix) pairs, matrix minor

    // ---- what a lane reads of a column: dword (64 i + lane) of its packed row, if that is inside the row
    // EXACT (K a multiple of 512): load i is inside the row for all lanes or for none, and the lane's offsets are
    // lane * 8 plus constants; otherwise they are kept per load, clamped to 0 where the lane is past the row.
    uint32_t x_off[NL];
    bool inside[NL];
    const Nf4Matrix mat[2] = {w0, w1};
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int k = HALF ? (i * 32 + (lane & 31)) * 8 : (i * 64 + lane) * 8;
        inside[i] = EXACT ? i * 512 < K : k < K;
        x_off[i] = EXACT ? (uint32_t)(lane * 8 + (i * 512 < K ? i * 512 : 0)) : (uint32_t)(inside[i] ? k : 0);
    }
    const uint32_t copy_off = (lane & 31) * 4;  // + 128 for the second matrix

    // ---- the ring of columns ahead
    uint32_t ring_w[D][COLS][NL];  // a slot: the wave's columns of a unit
    float ring_a[D][COLS][NL];
    // Cursor of the loads: the wave's column of unit ic of group ig.  The pointers move on by 16 columns per unit
    // (N % 16 == 0: every unit is whole) and are set up afresh when the group changes: a handful of scalar
    // instructions per column instead of the 64-bit products, which with 16 waves to a CU are what the scalar
    // unit has no time for.
    const int ig0 = (int)(u_begin / (uint32_t)units_n), ic0 = (int)(u_begin % (uint32_t)units_n);
    int ig = ig0, ic = ic0;
    int i_units_left = (int)(u_end - u_begin);
    const uint32_t *i_wp[CB];
    const float *i_ap[CB];
    auto point_loads = [&]() {
        const int expert = __builtin_amdgcn_readfirstlane(grp_e[ig]) & 0xffff;
        const int64_t base = ((int64_t)expert * N + ic * UCOLS + wave) * K;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            i_wp[cb] = (const uint32_t *)(mat[cb].wq + (base >> 1));
            i_ap[cb] = mat[cb].absmax + (base >> mat[cb].bs_shift);
        }
    };
    point_loads();
    const int w_step = 2 * K;  // dwords of 16 columns
    int a_step[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) a_step[cb] = (16 * K) >> mat[cb].bs_shift;
    auto issue = [&](int d) {
        const int cb = d % CB;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const uint32_t w_idx = (x_off[i] >> 3) + (HALF ? (lane >> 5) * w_step : 0);
            ring_w[d][0][i] = i_wp[cb][w_idx];
            // (computed here: a register per load and matrix less)
            const uint32_t a_off = (x_off[i] >> mat[cb].bs_shift) + (HALF ? (lane >> 5) * a_step[cb] : 0);
            ring_a[d][0][i] = i_ap[cb][a_off];
            if constexpr (COLS == 2) {
                ring_w[d][1][i] = i_wp[cb][w_step + w_idx];
                ring_a[d][1][i] = i_ap[cb][a_step[cb] + a_off];
            }
        }
        // past the end the cursor stays on the last unit: loads that nobody uses
        if (cb == CB - 1 && i_units_left > 1) {
            --i_units_left;
            if (++ic == units_n) {
                ic = 0;
                ++ig;
                point_loads();
            } else {
#pragma unroll
                for (int c2 = 0; c2 < CB; ++c2) {
                    i_wp[c2] += (UCOLS / 16) * w_step;
                    i_ap[c2] += (UCOLS / 16) * a_step[c2];
                }
            }
        }
    };
#pragma unroll
    for (int d = 0; d < D; ++d) issue(d);

    // ---- the loop over the columns
    uint4_t xr[ROWS][NL];
    int cg = ig0, cc = ic0;  // cursor of the arithmetic
    int rows = 0, row0 = 0, o_col = cc * UCOLS;
    int64_t o_row[ROWS];  // where the wave's column of unit 0 is in the output, per row of the group
    bool fresh = true;
    float first[ROWS];  // the gate projection's sums, until the up projection's are there
    // One column: the arithmetic on ring slot d, then (in the loop) the loads of the column D further on into it.
    auto column = [&](const int d, const bool more) {
            const int cb = d % CB;
            if (fresh) {
                fresh = false;
                const int ge = __builtin_amdgcn_readfirstlane(grp_e[cg]);
                rows = ge >> 16;
                row0 = __builtin_amdgcn_readfirstlane(grp_r[cg]);
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    o_row[r] = (int64_t)(row0 + r) * N + wave + (UCOLS == 32 ? (lane >> 5) * 16 : 0);  // lanes 32..63 end up with the second column
                    int64_t src_row = row0 + (r < rows ? r : rows - 1);
                    if (row_idx != nullptr) src_row = (uint32_t)row_idx[src_row] / (uint32_t)idx_div;
                    const bf16_t *const xp = x + src_row * K;
#pragma unroll
                    for (int i = 0; i < NL; ++i) {
                        const uint4_t v = *(const uint4_t *)(xp + x_off[i]);
                        const uint4_t zero = {0, 0, 0, 0};
                        xr[r][i] = inside[i] ? v : zero;
                    }
                }
            }
            const uint32_t lane_copy = copy_off + cb * 128;
            // The slot's values move to registers of the column and the slot is asked for again right away, in one
            // place for all row counts: were the loads issued inside the branches below, the branches would load
            // into different registers, and the copy that reconciles them would wait for the load just issued.
            // (the next loads are asked for behind the arithmetic, in one place for all row counts: asked for inside
            // the branches below they would land in different registers per branch, and the copy that reconciles
            // them would wait for the load just issued)
            // the arithmetic of the two columns for RN rows: one branch on the number of rows per unit, none inside
            auto arithmetic = [&](auto RN) {
                constexpr int rn = decltype(RN)::value;
                float acc[COLS][rn];
#pragma unroll
                for (int c = 0; c < COLS; ++c)
#pragma unroll
                    for (int r = 0; r < rn; ++r) acc[c][r] = 0.f;
#pragma unroll
                for (int i = 0; i < NL; ++i) {
#pragma unroll
                    for (int c = 0; c < COLS; ++c) {
                        uint32_t pr[4];
                        lookup4(pr, pair_address<0>(ring_w[d][c][i], lane_copy), pair_address<1>(ring_w[d][c][i], lane_copy),
                                pair_address<2>(ring_w[d][c][i], lane_copy), pair_address<3>(ring_w[d][c][i], lane_copy));
#pragma unroll
                        for (int r = 0; r < rn; ++r) {
                            float s = dot2_bf16(pr[0], xr[r][i][0], 0.f);
                            s = dot2_bf16(pr[1], xr[r][i][1], s);
                            s = dot2_bf16(pr[2], xr[r][i][2], s);
                            s = dot2_bf16(pr[3], xr[r][i][3], s);
                            acc[c][r] = __builtin_fmaf(ring_a[d][c][i], s, acc[c][r]);
                        }
                    }
                }
                // the two columns' 64 partial sums each become 32 + 32 in one swap of half waves and one add, and
                // five data-parallel-primitive adds finish both: the first column's sum in lane 31, the second's in 63
                float tot[rn];
#pragma unroll
                for (int r = 0; r < rn; ++r) {
                    // (one column: summed in the same order as each of two, so that the gated form's products are
                    // bit for bit those of the plain one; its sum is in lane 31 and in lane 63)
                    if constexpr (HALF)
                        tot[r] = half_sums_to_31_and_63(acc[0][r]);
                    else
                        tot[r] = two_sums_to_31_and_63(acc[0][r], acc[COLS - 1][r]);
                }
                if (GLU && cb == 0) {
#pragma unroll
                    for (int r = 0; r < rn; ++r) first[r] = tot[r];
                    return;
                }
                if (UCOLS == 32 ? (lane & 31) == 31 : lane == 63) {  // one lane per column
#pragma unroll
                    for (int r = 0; r < rn; ++r) {
                        const int64_t o = o_row[r] + o_col;
                        if constexpr (GLU) {
                            const bf16_t pe = (bf16_t)first[r], pg = (bf16_t)tot[r];
                            ((bf16_t *)y)[o] = silu_fwd_one<bf16_t>(pe, pg);
                            if (e_out) ((bf16_t *)e_out)[o] = pe;
                            if (g_out) ((bf16_t *)g_out)[o] = pg;
                        } else {
                            y[o] = from_f32<TO>(tot[r]);
                        }
                    }
                }
            };
            if (rows == 1)
                arithmetic(std::integral_constant<int, 1>());
            else if (ROWS == 2 || rows == 2)
                arithmetic(std::integral_constant<int, 2>());
            else if (ROWS == 4 && rows == 3)
                arithmetic(std::integral_constant<int, (ROWS > 2 ? 3 : 1)>());
            else
                arithmetic(std::integral_constant<int, ROWS>());
            if (more) issue(d);
            if (cb == CB - 1) {
                o_col += UCOLS;
                if (++cc == units_n) {
                    cc = 0;
                    o_col = 0;
                    ++cg;
                    fresh = true;
                }
            }
    };
    // Whole rounds of the ring in a loop without a way out of its middle, the rest behind it: with an exit
    // between two columns the compiler sees a path from a column's loads straight to the head of the loop,
    // where they would be the youngest in flight, and waits for every load at every column.
    const int rounds = n_items / D, rest = n_items % D;
    for (int q = 0; q < rounds; ++q) {
#pragma unroll
        for (int d = 0; d < D; ++d) column(d, true);
    }
#pragma unroll
    for (int d = 0; d < D - 1; ++d)
        if (d < rest) column(d, false);
}

template <int NL, int ROWS, int D, bool GLU, bool EXACT, bool HALF, typename TO>
int launch_gemv(const bf16_t *x, const int32_t *row_idx, int idx_div, const Nf4Matrix &w0, const Nf4Matrix &w1,
                const void *m_sizes, int ms_i64, TO *y, TO *e_out, TO *g_out, int64_t R, int N, int K, int E,
                hipStream_t stream) {
    const int64_t max_groups = R / ROWS + (R < E ? R : E);  // upper bound on sum over experts of ceil(m / ROWS)
    const int lds = kGemvTable + (int)max_groups * 8 + 16 + E * 4;
    auto *kernel = nf4_gemv_kernel<NL, ROWS, D, GLU, EXACT, HALF, TO>;
    static PerDeviceOnce attr;
    // The table lookups take the dynamic LDS to start at address 0; static LDS in this kernel would move it, so
    // such a build is left to the kernels that decode in registers.
    static std::atomic<int> static_lds{-1};
    const hipError_t e = attr.run([&] {
        hipFuncAttributes fa;
        const hipError_t e1 = hipFuncGetAttributes(&fa, (const void *)kernel);
        if (e1 != hipSuccess) return e1;
        static_lds.store((int)fa.sharedSizeBytes, std::memory_order_release);
        return hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kGemvTable + 4096 * 8 + 16 + 2048 * 4);
    });
    if (e != hipSuccess) return (int)e;
    if (static_lds.load(std::memory_order_acquire) != 0) return MFL_ERR_UNSUPPORTED;
    kernel<<<(unsigned)device_info().cu_count, kGemvThreads, lds, stream>>>(x, row_idx, idx_div, w0, w1, m_sizes, ms_i64,
                                                                            y, e_out, g_out, R, N, K, E,
                                                                            N / ((GLU && !HALF) ? 16 : 32), (int)max_groups);
    return launch_status();
}

template <int NL, int ROWS, bool HALF>
int dispatch_gemv(const bf16_t *x, const int32_t *row_idx, int idx_div, const Nf4Matrix &w0, const Nf4Matrix &w1,
                  bool glu, const void *m_sizes, int ms_i64, void *y, void *e_out, void *g_out, int64_t R, int N,
                  int K, int E, int out_dtype, hipStream_t stream) {
    const bool exact = !HALF && K % 512 == 0;
#define MFL_GEMV(GLU, EXACT, TO, Y, EO, GO)                                                                         \
    launch_gemv<NL, ROWS, ((GLU || HALF) ? 4 : 2), GLU, (EXACT && !HALF), HALF, TO>(x, row_idx, idx_div, w0, w1, m_sizes, \
                                                                                 ms_i64, Y, EO, GO, R, N, K, E, stream)
    if (glu)
        return exact ? MFL_GEMV(true, true, bf16_t, (bf16_t *)y, (bf16_t *)e_out, (bf16_t *)g_out)
                     : MFL_GEMV(true, false, bf16_t, (bf16_t *)y, (bf16_t *)e_out, (bf16_t *)g_out);
    if (out_dtype == MFL_BF16)
        return exact ? MFL_GEMV(false, true, bf16_t, (bf16_t *)y, nullptr, nullptr)
                     : MFL_GEMV(false, false, bf16_t, (bf16_t *)y, nullptr, nullptr);
    return exact ? MFL_GEMV(false, true, float, (float *)y, nullptr, nullptr)
                 : MFL_GEMV(false, false, float, (float *)y, nullptr, nullptr);
#undef MFL_GEMV
}

}  // namespace

int gemm_nf4_gemv(const bf16_t *x, const int32_t *row_idx, int idx_div, const Nf4Matrix &w0, const Nf4Matrix &w1,
                  bool glu, const void *m_sizes, int ms_i64, void *y, void *e_out, void *g_out, int64_t R, int N,
                  int K, int E, int out_dtype, hipStream_t stream) {
    if (R <= 0 || R > 2 * (int64_t)E || E > 2048) return MFL_ERR_UNSUPPORTED;  // a few rows per expert only
    const bool half = K <= 1024;  // 32 lanes to a column
    // (short rows: ahead of the streaming form only up to a row per expert: 23.5 against 25.5 us at 16 tokens of 8
    // experts each for K = 768, N = 2048, 35.0 against 30.4 us at 32 tokens)
    if (half && R > E) return MFL_ERR_UNSUPPORTED;
    if (K % 8 != 0 || K > 2048 || K <= 256) return MFL_ERR_UNSUPPORTED;
    // whole units (32 columns; 16 in the gated form with 64 lanes to a column); fewer than 2^31 units in all
    if (N % ((glu && !half) ? 16 : 32) != 0 || N > (1 << 18)) return MFL_ERR_UNSUPPORTED;
    const Nf4Matrix *mats[2] = {&w0, &w1};
    for (int cb = 0; cb < (glu ? 2 : 1); ++cb) {
        const Nf4Matrix &m = *mats[cb];
        // a lane's 8 weights under one scale, and every column starts a quantisation block
        if (m.bs_shift < 3 || (K & ((1 << m.bs_shift) - 1)) != 0) return MFL_ERR_UNSUPPORTED;
        if (!aligned(m.absmax, 4) || !aligned(m.wq, 4)) return MFL_ERR_UNSUPPORTED;
    }
    if (!aligned(x, 16)) return MFL_ERR_UNSUPPORTED;
#define MFL_GEMV_D(NL, ROWS, HALF) \
    dispatch_gemv<NL, ROWS, HALF>(x, row_idx, idx_div, w0, w1, glu, m_sizes, ms_i64, y, e_out, g_out, R, N, K, E, out_dtype, stream)
    if (!half) return MFL_GEMV_D(4, 2, false);
    return K <= 768 ? MFL_GEMV_D(3, 2, true) : MFL_GEMV_D(4, 2, true);
#undef MFL_GEMV_D
}

}  // namespace mfl
