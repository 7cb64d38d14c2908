// Fused NF4 grouped GEMM for decode-sized batches, streaming form (K % 128 == 0, quantisation blocks of at
// least 64 weights): everything a workgroup reads arrives in LDS by direct copies (global_load_lds), in a ring
// of stages of 128 reduction elements, so that the only vector-memory operations in the reduction loop are
// copies with one and the same lead.  The wave's memory counter completes in order: a register load of rows
// or scales issued after a copy would, when waited for, hold the wave until the copy has landed too, and the
// copies would never be further ahead than those loads.
//
// A workgroup (4 waves) owns 32 MR rows of one expert (MR = 1 at decode sizes, 2 from some twenty rows per expert
// on: the weights are streamed and decoded once per row tile) and 128 output columns, a wave 32 of the columns (of
// both matrices in the gated linear unit) for all of the rows.
//   stage = rows     32 MR x 128 bf16 (8 KiB a block of 32, shared by the four waves; chunk c of row r at c ^ (r & 15))
//         + weights  per wave and matrix 32 columns x 64 packed bytes (2 KiB; chunk c of row r at c ^ ((r >> 2) & 3))
//         + scales   per wave and matrix 32 columns x 2 floats (one per 64 reduction elements)
//   One barrier per stage: it publishes the rows that the other waves copied and frees the slot of the
//   stage before for the next copies.  Three stages of 32-row tiles are 52 KiB, two stages of 64-row tiles 51 KiB:
//   three workgroups share a CU (two of the gated form), and what counts is how many workgroups of the launch
//   are resident at once: a workgroup's loop is a chain of latencies (about 1.1 us per stage whatever is taken
//   out of it), so a second round of workgroups doubles the time of the launch.
//
// Decoding costs about one vector instruction per weight instead of three and a half:
//   * a byte of packed weights is two weights, and two bf16 are one dword of an MFMA operand: a 256-entry
//     table in LDS, indexed by the byte, holds the finished pair.  One shift-by-two of a byte (SDWA) and one
//     LDS read per pair; the table lies at LDS address 0, so the shifted byte is the address.  (A copy of the table per bank, 64 KiB, takes the bank conflicts of the lookups
//     away and the second and third workgroup of the CU with them: slower.)
//   * the table holds the bare code values (rounded to bf16 once).  The scale of a quantisation block is
//     applied to the block's partial sum in fp32: with the weights as the SECOND MFMA operand a lane's 16
//     accumulators all belong to one output column, whose scale the lane holds, so a 64-wide step is four
//     MFMAs into a fresh accumulator and 16 multiply-adds into the running sum.
//   The product is therefore sum over blocks of absmax * (x . bf16(code)) instead of x . bf16(code * absmax): the
//   same one rounding to bf16 per weight, taken before the scale rather than after it.  The two differ by
//   rounding noise of the size that either has against exact arithmetic.
#include "common.h"
#include "gemm.h"

namespace mfl {

namespace {

typedef __attribute__((address_space(3))) void *lds_void_ptr;
typedef const __attribute__((address_space(3))) uint32_t *lds_u32_ptr;

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | 0x70 | 0xF00 | ((N >> 4) << 14));
}

// Wave-wide copies from global memory to consecutive LDS (16 or 4 bytes per lane), written out by hand: the
// compiler orders LDS reads behind every copy to LDS that it knows to be in flight, i.e. behind the stages
// just requested.  M0 carries the LDS address of lane 0's piece; nothing else in the kernel uses M0.
__device__ __forceinline__ void copy16_to_lds(const void *src, unsigned char *dst) {
    const uint32_t lds_addr = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_void_ptr)dst);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(lds_addr) : "memory");
}
__device__ __forceinline__ void copy4_to_lds(const void *src, unsigned char *dst) {
    const uint32_t lds_addr = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_void_ptr)dst);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" : : "v"(src), "s"(lds_addr) : "memory");
}

// (byte `B` of w) << 2: the LDS byte offset of the pair-table entry of two packed weights, in one instruction.
template <int B>
__device__ __forceinline__ uint32_t byte_times_4(uint32_t w) {
    uint32_t r;
    const uint32_t two = 2;
    if constexpr (B == 0)
        asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0" : "=v"(r) : "v"(two), "v"(w));
    else if constexpr (B == 1)
        asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_1" : "=v"(r) : "v"(two), "v"(w));
    else if constexpr (B == 2)
        asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_2" : "=v"(r) : "v"(two), "v"(w));
    else
        asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_3" : "=v"(r) : "v"(two), "v"(w));
    return r;
}

template <bool GLU, int MR, int RING_>
struct StreamShape {
    static constexpr int CB = GLU ? 2 : 1;     // weight matrices per wave
    static constexpr int RING = RING_;         // stages in LDS; all but one of them in flight
    static constexpr int kX = MR * 32 * 256;   // rows of a stage: MR blocks of 32
    static constexpr int kW = 32 * 64;         // packed weights of a stage, per wave and matrix
    static constexpr int kA = 32 * 2 * 4;      // scales of a stage, per wave and matrix
    static constexpr int kStage = kX + 4 * CB * (kW + kA);
    static constexpr int kTable = CB * 256 * 4;
    // RING 3, MR 1: 53248, three workgroups per CU; gated: 81920, two.  RING 2, MR 2: 52224, three; gated: 71680, two.
    static constexpr int kLds = RING * kStage + kTable;
    static constexpr int kWOps = 2 * CB + CB;  // copies of weights and scales per wave and stage (the rows: up to 2 MR more)
};

// at most OPS + xc (xc = 0 .. XMAX, wave-uniform) vector-memory operations outstanding
template <int OPS, int XMAX>
__device__ __forceinline__ void wait_stage_ops(int xc) {
    if constexpr (XMAX == 0) {
        wait_vmcnt<OPS>();
    } else {
        if (xc == XMAX) wait_vmcnt<OPS + XMAX>();
        else wait_stage_ops<OPS, XMAX - 1>(xc);
    }
}

template <bool GLU, bool TILED, int MR, int RING_, typename TO>
__global__ __launch_bounds__(256) void nf4_stream_kernel(const bf16_t *__restrict__ x,
                                                         const int32_t *__restrict__ row_idx, int idx_div,
                                                         Nf4Matrix w0, Nf4Matrix w1,
                                                         const void *__restrict__ m_sizes, int ms_i64,
                                                         TO *__restrict__ y, TO *__restrict__ e_out,
                                                         TO *__restrict__ g_out, int64_t R, int N, int K, int E,
                                                         int tiles_n) {
    using S = StreamShape<GLU, MR, RING_>;
    constexpr int CB = S::CB, RING = S::RING, TR = 32 * MR;  // TR: rows of a workgroup's tile
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    // the pair table first, at LDS address 0 (the kernel has no static LDS, which the launcher checks): a lookup's address is then the shifted
    // byte itself plus a constant that fits the instruction's offset field, no add
    unsigned char *const table = smem;
    unsigned char *const ring = smem + S::kTable;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, h = lane >> 5;

    // ---- pair table: entry b = bf16(code[b >> 4]) in the low half (the first of the two weights is the high
    // nibble), bf16(code[b & 15]) in the high half
    {
        const Nf4Matrix *mats[2] = {&w0, &w1};
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            union {
                bf16_t e[2];
                uint32_t u;
            } pr;
            pr.e[0] = (bf16_t)mats[cb]->code16[tid >> 4];
            pr.e[1] = (bf16_t)mats[cb]->code16[tid & 15];
            ((uint32_t *)table)[cb * 256 + tid] = pr.u;
        }
    }

    // ---- which 32 rows: row tile blockIdx.x / tiles_n in the order of the experts
    // Workgroup b runs on XCD b % 8.  Row tiles are dealt to the XCDs round robin, and all column tiles of a row
    // tile to the same XCD, one after the other: the tile's rows come over the fabric once and are shared in
    // that XCD's L2 (dealt by workgroup number, every XCD that holds one of the column tiles fetches the rows
    // for itself), while all XCDs still work on neighbouring experts at any one time.
    const int xcd_idx = blockIdx.x >> 3;
    const int ct = xcd_idx % tiles_n, rt = (xcd_idx / tiles_n) * 8 + (blockIdx.x & 7);
    int expert = -1, m_start = 0, m_size = 0, t_begin = 0;
    {
        int row_carry = 0, tile_carry = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            const int m = e < E ? load_msize(m_sizes, ms_i64, e) : 0;
            const int t = ceil_div(m, TR);
            const int minc = wave_inclusive_scan(m), tinc = wave_inclusive_scan(t);
            const int tb = tile_carry + tinc - t;
            const uint64_t hits = __ballot(rt >= tb && rt < tb + t);
            if (hits) {
                const int src = __ffsll((unsigned long long)hits) - 1;
                expert = e0 + src;
                m_start = row_carry + __shfl(minc - m, src);
                m_size = __shfl(m, src);
                t_begin = __shfl(tb, src);
                break;
            }
            row_carry += wave_last(minc);
            tile_carry += wave_last(tinc);
        }
    }
    // every wave of the workgroup takes the same path here: the values above are the same in all of them
    if (expert < 0) return;
    expert = __builtin_amdgcn_readfirstlane(expert);
    const int i0 = __builtin_amdgcn_readfirstlane(m_start) + (rt - __builtin_amdgcn_readfirstlane(t_begin)) * TR;
    int i_end = __builtin_amdgcn_readfirstlane(m_start) + __builtin_amdgcn_readfirstlane(m_size);
    if ((int64_t)i_end > R) i_end = (int)R;
    const int rows = i_end - i0 < TR ? i_end - i0 : TR;
    if (rows <= 0) return;

    // ---- sources of this lane's pieces of a stage
    const int j0 = (ct * 4 + wave) * 32;  // first column of the wave
    const Nf4Matrix mat[2] = {w0, w1};
    const unsigned char *w_src[CB][2];  // copy j: columns 16j .. 16j+15 of the wave, four lanes to a column
    int64_t a_el[CB];                   // first weight under the lane's scale of stage 0: lane i brings scale i & 1 of column i >> 1
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int r = 16 * j + (lane >> 2);
            const int c = (lane & 3) ^ ((r >> 2) & 3);
            int col = j0 + r;
            if (col >= N) col = N - 1;  // copied, multiplied, never stored
            w_src[cb][j] = mat[cb].wq + ((((int64_t)expert * N + col) * K) >> 1) + c * 16;
        }
        int col = j0 + (lane >> 1);
        if (col >= N) col = N - 1;
        a_el[cb] = ((int64_t)expert * N + col) * K + (lane & 1) * 64;
    }
    const bf16_t *x_src[2 * MR];  // copy j: rows 32 (j / 2) + 8 wave + 4 (j % 2) .. + 3, sixteen lanes to a row
#pragma unroll
    for (int j = 0; j < 2 * MR; ++j) {
        const int r = 32 * (j >> 1) + 8 * wave + 4 * (j & 1) + (lane >> 4);
        const int c = (lane & 15) ^ (r & 15);
        int64_t src_row = i0 + (r < rows ? r : rows - 1);
        if (row_idx != nullptr) src_row = (uint32_t)row_idx[src_row] / (uint32_t)idx_div;
        x_src[j] = x + src_row * K + c * 8;
    }
    const int NS = K / 128, tiles32 = (N + 31) / 32;
    // a wave whose 32 columns all lie past N (N not a multiple of 128) takes the scales of the last tile of its
    // expert: copied, multiplied, never stored, and inside the array also for the last expert
    const int a_tile = j0 / 32 < tiles32 ? j0 / 32 : tiles32 - 1;
    // A copy of rows whose four rows all lie past the tile's last row is left out (nobody stores what the MFMAs
    // make of that part of the stage): the first x_copies of the wave's 2 MR (their rows ascend with j), the same
    // number in every stage.
    int x_copies = 0;
#pragma unroll
    for (int j = 0; j < 2 * MR; ++j) x_copies += rows > 32 * (j >> 1) + 8 * wave + 4 * (j & 1) ? 1 : 0;
    x_copies = __builtin_amdgcn_readfirstlane(x_copies);
    const int m_blocks = ceil_div(rows, 32);  // 32-row blocks of the tile that hold rows
    auto issue = [&](int stg) {
        unsigned char *const base = ring + (stg % RING) * S::kStage;
#pragma unroll
        for (int j = 0; j < 2 * MR; ++j)
            if (j < x_copies) copy16_to_lds(x_src[j] + (int64_t)stg * 128, base + ((j >> 1) * 8 + wave * 2 + (j & 1)) * 1024);
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
                copy16_to_lds(w_src[cb][j] + (int64_t)stg * 64, base + S::kX + (wave * CB + cb) * S::kW + j * 1024);
            // the wave's 64 scales of the stage: 256 consecutive bytes of the tile-ordered copy where the caller
            // brought one (two lines per copy), else two neighbours out of each column's own run (32 lines)
            const float *a_src = TILED ? mat[cb].absmax_tiled + ((((int64_t)expert * tiles32 + a_tile) * NS + stg) * 64 + lane)
                                       : mat[cb].absmax + ((a_el[cb] + (int64_t)stg * 128) >> mat[cb].bs_shift);
            copy4_to_lds(a_src, base + S::kX + 4 * CB * S::kW + (wave * CB + cb) * S::kA);
        }
    };
    // ---- where this lane reads a stage: its 16 bytes of packed weights of step s2, its 16 bytes of row n for
    // MFMA ks of step s2
    int w_rd[2], x_rd[2][4];
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
        w_rd[s2] = n * 64 + (((2 * s2 + h) ^ ((n >> 2) & 3)) << 4);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) x_rd[s2][ks] = n * 256 + (((8 * s2 + 4 * h + ks) ^ (n & 15)) << 4);
    }

    floatx16 tot[MR][CB];
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
            for (int r = 0; r < 16; ++r) tot[m][cb][r] = 0.f;

    // Every wave issues the same number of copies per stage (S::kWOps and the row copies it does not leave out),
    // unconditionally (past the end they repeat the last stage, into a slot that is free), so "at most RING - 2
    // stages' worth of my copies outstanding" means that the stage about to be read has landed.
#pragma unroll
    for (int q = 0; q < RING - 1; ++q) issue(q < NS ? q : NS - 1);
    for (int q = 0; q < NS; ++q) {
        // at most (RING - 2) stages' worth of this wave's copies outstanding
        if constexpr (RING == 3) wait_stage_ops<S::kWOps, 2 * MR>(x_copies);
        else wait_vmcnt<0>();
        __syncthreads();  // stage q is whole (the first time round: so is the pair table); nobody reads stage q - 1 any more
        const unsigned char *const base = ring + (q % RING) * S::kStage;
        // the stage's packed weights and scales are asked of the LDS before the next copies are set up (some
        // forty scalar and vector instructions), so that their latency runs under that
        uint4_t wl2[2][CB];
        float am2[2][CB];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                wl2[s2][cb] = *(const uint4_t *)(base + S::kX + (wave * CB + cb) * S::kW + w_rd[s2]);
                am2[s2][cb] = *(const float *)(base + S::kX + 4 * CB * S::kW + (wave * CB + cb) * S::kA + (n * 2 + s2) * 4);
            }
        issue(q + RING - 1 < NS ? q + RING - 1 : NS - 1);
        // The eight MFMA steps of the stage in one sequence, the operands of a step (16 bytes of the rows, four
        // table lookups per matrix) asked of the LDS one step ahead: asked for right in front of their MFMA, every
        // step would wait out the LDS latency and the stage would be a chain of eight of them.
        struct StepOps {
            uint4_t xa[MR];
            uint4_t wf[CB];
        };
        auto fetch = [&](int step, StepOps &o) {
            const int s2 = step >> 2, ks = step & 3;
#pragma unroll
            for (int m = 0; m < MR; ++m)
                if (m == 0 || m < m_blocks) o.xa[m] = *(const uint4_t *)(base + m * 8192 + x_rd[s2][ks]);
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                const uint32_t w = wl2[s2][cb][ks];
                o.wf[cb][0] = *(lds_u32_ptr)(uintptr_t)(byte_times_4<0>(w) + cb * 1024);
                o.wf[cb][1] = *(lds_u32_ptr)(uintptr_t)(byte_times_4<1>(w) + cb * 1024);
                o.wf[cb][2] = *(lds_u32_ptr)(uintptr_t)(byte_times_4<2>(w) + cb * 1024);
                o.wf[cb][3] = *(lds_u32_ptr)(uintptr_t)(byte_times_4<3>(w) + cb * 1024);
            }
        };
        constexpr int AHEAD = 1;  // two steps ahead: no faster; the gated form would pass the 15 LDS reads that can be in flight
        StepOps ops[AHEAD + 1];
#pragma unroll
        for (int a = 0; a < AHEAD; ++a) fetch(a, ops[a]);
        floatx16 blk[MR][CB];
#pragma unroll
        for (int step = 0; step < 8; ++step) {
            if (step + AHEAD < 8) fetch(step + AHEAD, ops[(step + AHEAD) % (AHEAD + 1)]);
            const StepOps &o = ops[step % (AHEAD + 1)];
            const int s2 = step >> 2, ks = step & 3;
            // a block past the tile's last row (wave-uniform) is neither read nor multiplied
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                if (m > 0 && m >= m_blocks) continue;
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    union {
                        uint4_t u;
                        bf16x8 v;
                    } xa, wf;
                    xa.u = o.xa[m];
                    wf.u = o.wf[cb];
                    if (ks == 0) {
                        floatx16 zero;
#pragma unroll
                        for (int r = 0; r < 16; ++r) zero[r] = 0.f;
                        blk[m][cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa.v, wf.v, zero, 0, 0, 0);
                    } else {
                        blk[m][cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa.v, wf.v, blk[m][cb], 0, 0, 0);
                    }
                }
                if (ks == 3) {
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            tot[m][cb][r] = __builtin_fmaf(am2[s2][cb], blk[m][cb][r], tot[m][cb][r]);
                }
            }
        }
    }
    wait_vmcnt<0>();  // the repeated copies of the last stage must not land in LDS that another workgroup owns by then

    // ---- output: a lane holds column n, rows 8g + 4h + u
    const int col = j0 + n;
    if (col >= N) return;
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = 32 * m + 8 * (r >> 2) + 4 * h + (r & 3);
            if (row >= rows) continue;
            const int64_t o = (int64_t)(i0 + row) * N + col;
            if constexpr (GLU) {
                const bf16_t pe = (bf16_t)tot[m][0][r], pg = (bf16_t)tot[m][1][r];
                ((bf16_t *)y)[o] = silu_fwd_one<bf16_t>(pe, pg);
                if (e_out) ((bf16_t *)e_out)[o] = pe;
                if (g_out) ((bf16_t *)g_out)[o] = pg;
            } else {
                y[o] = from_f32<TO>(tot[m][0][r]);
            }
        }
}

template <bool GLU, bool TILED, int MR, int RING_, typename TO>
int launch_stream(const bf16_t *x, const int32_t *row_idx, int idx_div, const Nf4Matrix &w0, const Nf4Matrix &w1,
                  const void *m_sizes, int ms_i64, TO *y, TO *e_out, TO *g_out, int64_t R, int N, int K, int E,
                  hipStream_t stream) {
    using S = StreamShape<GLU, MR, RING_>;
    constexpr int kLds = S::kLds;
    const int tiles_n = ceil_div(N, 128);
    const int64_t row_tiles = R / (32 * MR) + (R < E ? R : E);  // upper bound on sum over experts of ceil(m / (32 MR))
    const int64_t grid = (row_tiles + 7) / 8 * 8 * tiles_n;  // row tiles in eights: one per XCD
    if (grid > 0x7fffffff) return MFL_ERR_UNSUPPORTED;
    auto *kernel = nf4_stream_kernel<GLU, TILED, MR, RING_, TO>;
    static PerDeviceOnce attr;
    // The kernel's table lookups take the dynamic LDS to start at address 0: any static LDS in this kernel
    // (a later __shared__ variable, an inlined helper that brings one) would move it, so the launcher asks the
    // runtime once and leaves such a build to the register-decoding kernel.
    static std::atomic<int> static_lds{-1};
    const hipError_t e = attr.run([&] {
        hipFuncAttributes fa;
        const hipError_t e1 = hipFuncGetAttributes(&fa, (const void *)kernel);
        if (e1 != hipSuccess) return e1;
        static_lds.store((int)fa.sharedSizeBytes, std::memory_order_release);
        return hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    });
    if (e != hipSuccess) return (int)e;
    if (static_lds.load(std::memory_order_acquire) != 0) return MFL_ERR_UNSUPPORTED;
    kernel<<<(unsigned)grid, 256, kLds, stream>>>(x, row_idx, idx_div, w0, w1, m_sizes, ms_i64, y, e_out, g_out,
                                                          R, N, K, E, tiles_n);
    return launch_status();
}

// out[((e * tiles32 + t) * NS + s) * 64 + l] = the scale of column 32 t + (l >> 1) (the last column past N), weights
// 128 s + 64 (l & 1) .. + 63 of its reduction
__global__ __launch_bounds__(256) void nf4_tile_absmax_kernel(const float *__restrict__ absmax, int bs_shift, int N, int K,
                                                              int tiles32, int64_t total, float *__restrict__ out) {
    const int NS = K / 128;
    for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < total; i += gridDim.x * 256ll) {
        const int l = (int)(i & 63);
        const int64_t q = i >> 6;
        const int s = (int)(q % NS);
        const int64_t et = q / NS;
        const int t = (int)(et % tiles32);
        const int64_t e = et / tiles32;
        int col = 32 * t + (l >> 1);
        if (col >= N) col = N - 1;
        out[i] = absmax[((e * N + col) * K + 128 * s + 64 * (l & 1)) >> bs_shift];
    }
}

}  // namespace

int64_t nf4_tiled_absmax_floats(int blocksize, int N, int K, int E) {
    if (blocksize < 64 || (blocksize & (blocksize - 1)) != 0 || K % 128 != 0 || N <= 0 || E <= 0) return 0;
    return (int64_t)E * ceil_div(N, 32) * (K / 128) * 64;
}

int nf4_tile_absmax(const float *absmax, int blocksize, int N, int K, int E, float *out, hipStream_t stream) {
    const int64_t total = nf4_tiled_absmax_floats(blocksize, N, K, E);
    if (total == 0) return MFL_ERR_UNSUPPORTED;
    int shift = 0;
    while ((1 << shift) < blocksize) ++shift;
    const int64_t blocks = (total + 255) / 256;
    nf4_tile_absmax_kernel<<<(unsigned)(blocks < 65536 ? blocks : 65536), 256, 0, stream>>>(absmax, shift, N, K,
                                                                                          ceil_div(N, 32), total, out);
    return launch_status();
}

int gemm_nf4_stream(const bf16_t *x, const int32_t *row_idx, int idx_div, const Nf4Matrix &w0, const Nf4Matrix &w1,
                    bool glu, const void *m_sizes, int ms_i64, void *y, void *e_out, void *g_out, int64_t R, int N,
                    int K, int E, int out_dtype, hipStream_t stream) {
    // a 64-wide step must lie inside one quantisation block, and the scales are copied four bytes at a time
    if (K % 128 != 0 || w0.bs_shift < 6 || w1.bs_shift < 6) return MFL_ERR_UNSUPPORTED;
    if (!aligned(w0.absmax, 4) || !aligned(w1.absmax, 4)) return MFL_ERR_UNSUPPORTED;
    // the tile-ordered scales are used where the caller brought them for every matrix of the product
    const bool tiled = w0.absmax_tiled != nullptr && (!glu || w1.absmax_tiled != nullptr) &&
                       aligned(w0.absmax_tiled, 4) && (!glu || aligned(w1.absmax_tiled, 4));
    // Tile height and ring depth.  Up to kNf4StreamTwoBlockRows rows per expert on average: 32-row tiles, three
    // stages.  Above: 64-row tiles (an expert's weights are streamed and decoded once per row tile) with two stages,
    // which leaves the plain product its three workgroups per CU and the gated one its two: residency counts for
    // more than a second stage in flight (plain product, 40 rows per expert: 43 us against 55 with three stages
    // and two workgroups per CU, 59 with 32-row tiles).  The bits are the same whatever the tile height.
    const bool two = R > (int64_t)kNf4StreamTwoBlockRows * E;
#define MFL_STREAM_MR(GLU, MR, RG, TO, Y, EO, GO)                                                                              \
    (tiled ? launch_stream<GLU, true, MR, RG, TO>(x, row_idx, idx_div, w0, w1, m_sizes, ms_i64, Y, EO, GO, R, N, K, E, stream) \
           : launch_stream<GLU, false, MR, RG, TO>(x, row_idx, idx_div, w0, w1, m_sizes, ms_i64, Y, EO, GO, R, N, K, E, stream))
#define MFL_STREAM(GLU, TO, Y, EO, GO) (two ? MFL_STREAM_MR(GLU, 2, 2, TO, Y, EO, GO) : MFL_STREAM_MR(GLU, 1, 3, TO, Y, EO, GO))
    if (glu) return MFL_STREAM(true, bf16_t, (bf16_t *)y, (bf16_t *)e_out, (bf16_t *)g_out);
    if (out_dtype == MFL_BF16) return MFL_STREAM(false, bf16_t, (bf16_t *)y, nullptr, nullptr);
    return MFL_STREAM(false, float, (float *)y, nullptr, nullptr);
#undef MFL_STREAM
#undef MFL_STREAM_MR
}

}  // namespace mfl
