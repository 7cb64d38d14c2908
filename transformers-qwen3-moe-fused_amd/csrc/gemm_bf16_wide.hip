// bf16 grouped GEMM for CDNA4 with four waves per workgroup, one per SIMD, each holding a wave tile of up to
// 128 x 128 outputs in its 256 accumulation registers.  Against the eight-wave tiles of gemm_bf16_pipe.hip a wave
// reads a third fewer LDS fragment bytes per MFMA, which is what the weight-gradient product (both operands read
// with transposing LDS reads, half the rate of plain ones) and the matrix-bound shapes of the other two products
// are limited by.
//
// Operand conventions are those of gemm_bf16_pipe.hip: C[i, j] = sum_r A(i, r) * B(j, r), each operand
// reduction-contiguous (RC) or reduction-strided (RS); FWD = RC x RC, DX = RC x RS, DW = RS x RS; the stage
// layouts, copies and fragment reads come from pipe_parts.h.
//
// One stream of reduction steps per workgroup.  The tiles of a persistent workgroup are not separate pipelines:
// a producer cursor walks (tile, step) ahead of the consumer cursor, so the copies of the next tile's first steps
// are in flight while the current tile is multiplied and its output stored.  The ring holds SR stages.  In step g
// the wave multiplies all sub-steps but the last, then (point P) waits for its own copies of step g+1, meets the
// other waves at the one barrier of the step -- after it stage g is free and stage g+1 complete for everybody --
// requests the fragments of step g+1's first sub-step, and multiplies the last sub-step of step g with the copies
// of step g+SR dealt out between its MFMAs.  With one wave per SIMD nothing else hides a wait, so neither the
// fragment reads nor the copies are ever asked for right before they are needed.
//
// The vector-memory counter of a wave counts down in order of issue; the kernel keeps the number of operations it
// has issued (copies and output stores) and, per ring slot, that number after the slot's last copy: "step g+1 has
// landed" is a wait for at most (issued - mark) outstanding operations, whatever was issued in between.
//
// Shapes: bf16 in, bf16 out, no accumulation, no scaling; E <= 512; FWD/DX: N % 8 == 0, K % 64 == 0; DW: N % BM == 0,
// K % BN == 0 (any number of rows per expert).  The caller falls back to gemm_bf16_pipe.hip otherwise.
#include "pipe_parts.h"

namespace mfl {

namespace {

constexpr int kWideOutRowsPerExpert = 152, kWideMidRowsPerExpert = 232;

// Tuning builds can take parts of the kernel out (timing experiments only; the results are then wrong).
#ifdef MFL_TUNING_BUILD
#ifndef MFL_X_NO_STORE
#define MFL_X_NO_STORE 0
#endif
#ifndef MFL_X_NO_COPY
#define MFL_X_NO_COPY 0
#endif
#ifndef MFL_X_NO_MFMA
#define MFL_X_NO_MFMA 0
#endif
#ifndef MFL_X_NO_READ
#define MFL_X_NO_READ 0
#endif
constexpr bool kNoStore = MFL_X_NO_STORE, kNoCopy = MFL_X_NO_COPY, kNoMfma = MFL_X_NO_MFMA, kNoRead = MFL_X_NO_READ;
#else
constexpr bool kNoStore = false, kNoCopy = false, kNoMfma = false, kNoRead = false;
#endif

#if defined(MFL_TUNING_BUILD) && defined(MFL_X_TRACE)
// time stamps of one workgroup's first wave, kept in LDS (behind everything else) and copied out at the end
__device__ unsigned int g_wide_trace[4096];
__device__ int g_wide_trace_n;
#define MFL_TR_LDS 155648
#define MFL_TR(tag)                                                                                          \
    if (blockIdx.x == MFL_X_TRACE && wave == 0 && tr_n < 1000) {                                               \
        if (lane == 0) {                                                                                     \
            ((unsigned int *)(smem + MFL_TR_LDS))[2 * tr_n] = (tag);                                          \
            ((unsigned int *)(smem + MFL_TR_LDS))[2 * tr_n + 1] = (unsigned int)__builtin_readcyclecounter(); \
        }                                                                                                    \
        ++tr_n;                                                                                              \
    }
#else
#define MFL_TR(tag)
#endif

// s_waitcnt vmcnt(min(n, 63)), n wave-uniform.  Exact, not rounded down: a wait for a few operations fewer than
// necessary also waits for the first copies of the step after the one that is needed.  The instruction takes its
// count as an immediate only, so this is a computed jump into a table of 64 of them (8 bytes an entry; the three
// instructions between s_getpc_b64 and the table are 12 bytes).
__device__ __forceinline__ void wait_vmcnt_upto(int n) {
    uint32_t t;
    n = __builtin_amdgcn_readfirstlane(n);
    asm volatile(
        "s_min_u32 %[t], %[n], 63\n\ts_lshl_b32 %[t], %[t], 3\n\ts_add_u32 %[t], %[t], 12\n\t"
        "s_getpc_b64 s[98:99]\n\ts_add_u32 s98, s98, %[t]\n\ts_addc_u32 s99, s99, 0\n\ts_setpc_b64 s[98:99]\n\t"
        "s_waitcnt vmcnt(0)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(1)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(2)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(3)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(4)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(5)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(6)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(7)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(8)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(9)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(10)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(11)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(12)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(13)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(14)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(15)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(16)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(17)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(18)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(19)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(20)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(21)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(22)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(23)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(24)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(25)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(26)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(27)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(28)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(29)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(30)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(31)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(32)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(33)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(34)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(35)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(36)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(37)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(38)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(39)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(40)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(41)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(42)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(43)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(44)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(45)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(46)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(47)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(48)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(49)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(50)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(51)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(52)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(53)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(54)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(55)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(56)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(57)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(58)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(59)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(60)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(61)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(62)\n\ts_branch .Lwv_end_%=\n\t"
        "s_waitcnt vmcnt(63)\n\ts_branch .Lwv_end_%=\n\t"
        ".Lwv_end_%=:"
        : [t] "=&s"(t)
        : [n] "s"(n)
        : "memory", "scc", "s98", "s99");
}

// f(IC<0>{}), ..., f(IC<N-1>{}): a loop whose index is a constant expression inside the body
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(IC<I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// 16 bytes per lane from a per-lane address to 1 KiB of consecutive LDS; POLICY 2 = non-temporal.  The copy is
// issued when `on` (wave-uniform) is not zero.  The test sits inside the statement: a branch in the source around a
// copy between two MFMAs cuts the sub-step into basic blocks, and two variants of a sub-step (with and without
// copies) make the register allocator move accumulators between them.
template <int POLICY>
__device__ __forceinline__ void wide_copy(const unsigned char *src, uint32_t lds_addr) {
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);  // wave-uniform by construction; the asm needs an SGPR
    if constexpr (kNoCopy)
        asm volatile("s_nop 0" : : "v"(src), "s"(lds_addr) : "memory");
    else if constexpr (POLICY == 2)
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" : : "v"(src), "s"(lds_addr) : "memory");
    else
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(lds_addr) : "memory");
}
template <int POLICY>
__device__ __forceinline__ void wide_copy_if(const unsigned char *src, uint32_t lds_addr, int on) {
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    if constexpr (kNoCopy)
        asm volatile("s_nop 0" : : "v"(src), "s"(lds_addr), "s"(on) : "memory");
    else if constexpr (POLICY == 2)
        asm volatile(
            "s_cmp_eq_u32 %2, 0\n\ts_cbranch_scc1 .Lwc_skip_%=\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\t"
            "global_load_lds_dwordx4 %0, off nt\n.Lwc_skip_%=:"
            :
            : "v"(src), "s"(lds_addr), "s"(on)
            : "memory", "scc");
    else
        asm volatile(
            "s_cmp_eq_u32 %2, 0\n\ts_cbranch_scc1 .Lwc_skip_%=\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\t"
            "global_load_lds_dwordx4 %0, off\n.Lwc_skip_%=:"
            :
            : "v"(src), "s"(lds_addr), "s"(on)
            : "memory", "scc");
}

// Up to four copies of the wave as one statement: 16 bytes per lane each, from base + voff[q] + q * 1024 (the
// instruction's offset field, which the hardware adds to the global and to the LDS address alike) to the 1 KiB
// of LDS at lds_addr + q * 1024.  One M0 write for the group, no vector-ALU instruction; issued if `on`
// (wave-uniform).  The callers fold "- q * 1024 + kCopyBias" into voff and "- kCopyBias" into base.
constexpr int kCopyBias = 4096;
#define MFL_WC_HEAD "s_cmp_eq_u32 %[on], 0\n\ts_cbranch_scc1 .Lwg_skip_%=\n\ts_mov_b32 m0, %[lds]\n\ts_nop 0\n\t"
#define MFL_WC_LOAD(V, OFF, NT) "global_load_lds_dwordx4 %[" V "], %[base] offset:" OFF NT "\n\t"
#define MFL_WC_TAIL ".Lwg_skip_%=:"
template <int POLICY>
__device__ __forceinline__ void wide_copy4(uint64_t base, uint32_t v0, uint32_t v1, uint32_t v2, uint32_t v3,
                                           uint32_t lds_addr, int on) {
    on = __builtin_amdgcn_readfirstlane(on);  // wave-uniform by construction; the statement needs scalar registers
    if constexpr (kNoCopy)
        asm volatile("s_nop 0" : : [base] "s"(base), [v0] "v"(v0), [v1] "v"(v1), [v2] "v"(v2), [v3] "v"(v3),
                     [lds] "s"(lds_addr), [on] "s"(on) : "memory");
    else if constexpr (POLICY == 2)
        asm volatile(MFL_WC_HEAD MFL_WC_LOAD("v0", "0", " nt") MFL_WC_LOAD("v1", "1024", " nt")
                     MFL_WC_LOAD("v2", "2048", " nt") MFL_WC_LOAD("v3", "3072", " nt") MFL_WC_TAIL
                     : : [base] "s"(base), [v0] "v"(v0), [v1] "v"(v1), [v2] "v"(v2), [v3] "v"(v3), [lds] "s"(lds_addr),
                     [on] "s"(on) : "memory", "scc");
    else
        asm volatile(MFL_WC_HEAD MFL_WC_LOAD("v0", "0", "") MFL_WC_LOAD("v1", "1024", "") MFL_WC_LOAD("v2", "2048", "")
                     MFL_WC_LOAD("v3", "3072", "") MFL_WC_TAIL
                     : : [base] "s"(base), [v0] "v"(v0), [v1] "v"(v1), [v2] "v"(v2), [v3] "v"(v3), [lds] "s"(lds_addr),
                     [on] "s"(on) : "memory", "scc");
}
template <int POLICY>
__device__ __forceinline__ void wide_copy2(uint64_t base, uint32_t v0, uint32_t v1, uint32_t lds_addr, int on) {
    on = __builtin_amdgcn_readfirstlane(on);
    if constexpr (kNoCopy)
        asm volatile("s_nop 0" : : [base] "s"(base), [v0] "v"(v0), [v1] "v"(v1), [lds] "s"(lds_addr), [on] "s"(on) : "memory");
    else if constexpr (POLICY == 2)
        asm volatile(MFL_WC_HEAD MFL_WC_LOAD("v0", "0", " nt") MFL_WC_LOAD("v1", "1024", " nt") MFL_WC_TAIL
                     : : [base] "s"(base), [v0] "v"(v0), [v1] "v"(v1), [lds] "s"(lds_addr), [on] "s"(on) : "memory", "scc");
    else
        asm volatile(MFL_WC_HEAD MFL_WC_LOAD("v0", "0", "") MFL_WC_LOAD("v1", "1024", "") MFL_WC_TAIL
                     : : [base] "s"(base), [v0] "v"(v0), [v1] "v"(v1), [lds] "s"(lds_addr), [on] "s"(on) : "memory", "scc");
}
#undef MFL_WC_HEAD
#undef MFL_WC_LOAD
#undef MFL_WC_TAIL

// a 64-bit value that is the same in every lane, held in scalar registers
__device__ __forceinline__ uint64_t uniform64(uint64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
}

// One accumulator element, fetched from its accumulation register where the statement stands.  (Left to itself
// the compiler copies all 256 of a tile into vector registers at the top of the epilogue, and spills what else
// is live there: the fragments and addresses of the next tile's first step.)
__device__ __forceinline__ float acc_read(float v) {
    float r;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(r) : "a"(v));
    return r;
}

template <int MODE, int MB, int NB, int BK, int SR, bool THIN, typename TO>
__global__ __launch_bounds__(256) void gemm_wide_kernel(const bf16_t *__restrict__ a, const bf16_t *__restrict__ b,
                                                        const void *__restrict__ m_sizes, int ms_i64,
                                                        TO *__restrict__ c, int64_t R, int N, int K, int E,
                                                        const bf16_t *__restrict__ a2, const bf16_t *__restrict__ b2,
                                                        const bf16_t *__restrict__ at, const bf16_t *__restrict__ bt,
                                                        int kthin) {
    static_assert(!THIN || MODE != MODE_DW, "the thin last term belongs to the row-grouped products");
    static_assert(sizeof(TO) == 2, "bf16 output");
    constexpr int WGM = 2, WGN = 2, NW = 4;
    constexpr int BM = MB * 32, BN = NB * 32;
    constexpr bool A_RC = MODE != MODE_DW, B_RC = MODE == MODE_FWD;
    constexpr int TM = (MB + WGM - 1) / WGM;  // row blocks per wave, dealt round robin (the last may not exist)
    static_assert(NB % WGN == 0, "column blocks must split evenly over the waves");
    constexpr int TN = NB / WGN, WTN = TN * 32, KS = BK / 16;
    static_assert(KS % 2 == 0, "fragment buffers alternate by sub-step");
    typedef Stage<BM, BK, A_RC> SA;
    typedef Stage<BN, BK, B_RC> SB;
    static_assert(SA::kWaveLoads % NW == 0 && SB::kWaveLoads % NW == 0, "copies must split over the waves");
    constexpr int LA = SA::kWaveLoads / NW, LB = SB::kWaveLoads / NW, LPW = LA + LB;
    static_assert((SR - 2) * LPW < 64, "the steady-state wait fits the 6-bit counter");
    constexpr int STAGE_BYTES = SA::kBytes + SB::kBytes;
    constexpr int RING_BYTES = SR * STAGE_BYTES;
    // output staging, per wave: 32 rows of EPC columns
    constexpr int EPC = WTN % 64 == 0 ? 64 : WTN;
    constexpr int EP_ROWB = EPC * 2 + (EPC == 64 ? 16 : 8);
    constexpr int EP_WAVE = 32 * EP_ROWB;
    constexpr int STORES = TM * (WTN / EPC) * (EPC / 8 * 32 / 64);  // 16-byte stores per lane and tile
    static_assert((EPC / 8 * 32) % 64 == 0, "whole wave stores");

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
#if defined(MFL_TUNING_BUILD) && defined(MFL_X_TRACE)
    int tr_n = 0;
#endif

    FragOffsets<BM, BK, A_RC, TM> fo_a;
    FragOffsets<BN, BK, B_RC, TN> fo_b;
    fo_a.init(wm * 32, WGM * 32, lane);
    fo_b.init(wn * WTN, 32, lane);

    // ---- per-expert prefix tables in LDS behind the ring and the staging area: rows and tiles before expert e
    int *tab_rows = (int *)(smem + RING_BYTES + NW * EP_WAVE);
    int *tab_tiles = tab_rows + (kMaxTableExperts + 1);
    const int tiles_n = MODE == MODE_DW ? K / BN : ceil_div(N, BN);  // row-grouped products: the last may be partial
    const int per_expert = MODE == MODE_DW ? (N / BM) * tiles_n : 0;
    {
        int row_carry = 0, tile_carry = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            const int m = e < E ? load_msize(m_sizes, ms_i64, e) : 0;
            const int t = e >= E ? 0 : MODE == MODE_DW ? per_expert : m_tiles_of<BM>(m) * tiles_n;
            const int minc = wave_inclusive_scan(m), tinc = wave_inclusive_scan(t);
            if (wave == 0 && e <= E) {
                tab_rows[e] = row_carry + minc - m;
                tab_tiles[e] = tile_carry + tinc - t;
            }
            row_carry += wave_last(minc);
            tile_carry += wave_last(tinc);
        }
        if (wave == 0 && lane == 0 && E % 64 == 0) {
            tab_rows[E] = row_carry;
            tab_tiles[E] = tile_carry;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
    }
    const int total = __builtin_amdgcn_readfirstlane(tab_tiles[E]);

    // ---- tile range of this workgroup: XCD x owns a contiguous run of logical tiles (the tiles of an expert meet
    // in one L2), dealt out with a stride inside the run
    const int xcd = blockIdx.x % kXcd;
    const int per_xcd = gridDim.x / kXcd;
    const int chunk = ceil_div(total, kXcd);
    const int L_first = xcd * chunk + blockIdx.x / kXcd;
    int L_end = (xcd + 1) * chunk;
    if (L_end > total) L_end = total;

    // ---- what a cursor knows about a tile; every field wave-uniform
    // DX with a second term (a2, b2 shaped like a, b): the tile's reduction runs over (a, b) and goes on over
    // (a2, b2), in one accumulator: dx = a b + a2 b2 (the input gradient of the gated unit, de w_gate + dg w_up)
    const bool two_term = MODE == MODE_DX && a2 != nullptr;
    const int64_t second_a = (int64_t)((intptr_t)a2 - (intptr_t)a), second_b = (int64_t)((intptr_t)b2 - (intptr_t)b);
    // THIN: a last term with a reduction length of its own (the rank of a LoRA adapter), after the one or two
    // terms above, in the same accumulator: c += at bt with at (R, kthin) and bt (E, N, kthin) in FWD, (E, kthin, N)
    // in DX; kthin a multiple of 8.  Its steps come last in the tile's reduction; chunks past kthin are zeros.
    const int thin_steps = THIN ? ceil_div(kthin, BK) : 0;
    struct Tile {
        int i0, i_end, j0, red, KT, expert;
        const unsigned char *pa, *pb;
        TO *pc;
    };
    auto tile_at = [&](int L, Tile &t) {
        if (MODE == MODE_DW) {
            const int e = L / per_expert, local = L % per_expert;
            t.i0 = (local / tiles_n) * BM;
            t.i_end = t.i0 + BM;
            t.j0 = (local % tiles_n) * BN;
            int rb = __builtin_amdgcn_readfirstlane(tab_rows[e]);
            int re = __builtin_amdgcn_readfirstlane(tab_rows[e + 1]);
            if ((int64_t)re > R) re = (int)R;
            if (rb > re) rb = re;
            t.red = re - rb;
            t.KT = ceil_div(t.red, BK);
            t.pa = (const unsigned char *)(a + (int64_t)rb * N + t.i0);
            t.pb = (const unsigned char *)(b + (int64_t)rb * K + t.j0);
            t.pc = c + (int64_t)e * N * K;
        } else {
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
            // few row tiles: those of one column slice run side by side (they share the slice of the weights);
            // many: the column slices of one row tile (they share its rows)
#if defined(MFL_TUNING_BUILD) && defined(MFL_X_ORDER)
            const bool n_fast = MFL_X_ORDER == 1;
#else
            const bool n_fast = m_tiles > tiles_n;
#endif
            const int mi = n_fast ? local / tiles_n : local % m_tiles;
            const int ni = n_fast ? local % tiles_n : local / m_tiles;
            t.i0 = m_start + mi * rows;
            t.i_end = m_start + m_size;
            if (t.i_end > t.i0 + rows) t.i_end = t.i0 + rows;
            if ((int64_t)t.i_end > R) t.i_end = (int)R;
            if (t.i0 > t.i_end) t.i0 = t.i_end;
            t.j0 = ni * BN;
            t.red = K;
            t.KT = t.i_end > t.i0 ? (two_term ? 2 : 1) * (K / BK) + thin_steps : 0;
            t.expert = expert;
            t.pa = (const unsigned char *)(a + (int64_t)t.i0 * K);
            t.pb = B_RC ? (const unsigned char *)(b + (int64_t)expert * N * K + (int64_t)t.j0 * K)
                        : (const unsigned char *)(b + (int64_t)expert * N * K + t.j0);
            t.pc = c;
        }
    };
    const int lda = MODE == MODE_DW ? N : K;
    const int ldb = MODE == MODE_FWD ? K : MODE == MODE_DX ? N : K;
    const int64_t ldc = MODE == MODE_DW ? K : N;
    const int64_t step_a = A_RC ? (int64_t)BK * 2 : (int64_t)BK * lda * 2;
    const int64_t step_b = B_RC ? (int64_t)BK * 2 : (int64_t)BK * ldb * 2;

    // ---- producer: the (tile, step) whose copies are issued next.  A step's copies go out in groups of up to
    // four (one statement, one M0 write, scalar base + per-lane 32-bit offset + the instruction's offset field).
    constexpr int GS = 4;  // copies per group (groups of two and of one were measured: no faster)
    static_assert(LA % 2 == 0 && LB % 2 == 0, "copy groups hold two or four copies");
    constexpr int GA = (LA + GS - 1) / GS, GB = (LB + GS - 1) / GS, NG = GA + GB;  // groups per step: A's first, then B's
    // With three stages or more a step's copies have two steps to land: the second half of the groups goes out in
    // the first sub-step of the consumer's next step, so that no sub-step carries more than half of them.  With two
    // stages the second half then has three sub-steps to land instead of four: the 256 x 256 tiles, which run where
    // experts have many rows and the MFMAs of one sub-step do not cover the issue of a whole step's copies, do it
    // (4 % faster at 1024 rows per expert); the 320 x 192 tiles do not (the same at 256 rows per expert, 4-7 %
    // slower at 48-128, where the weights, whose groups come second, are most of the traffic).
    constexpr bool SPLIT = NG >= 2 && (SR >= 3 || MB * NB >= 64);
    constexpr int NG1 = SPLIT ? (NG + 1) / 2 : NG;  // groups in the sub-step after point P
    Tile pt;
    int pL = L_first, pk = 0, p_full = 0;  // p_full: steps of the producer's tile that are whole
    // Row-grouped products: copy groups of A whose stage rows all lie past the tile's last row are left out (nothing
    // that is stored reads them): bit j of p_amask says that this wave issues group j, p_copies how many copies
    // a step of the producer's tile comes to for this wave.
    unsigned p_amask = ~0u;
    int p_copies = LPW;
    bool p_more = false;
    uint64_t pa_cur = 0, pb_cur = 0;  // operand addresses of the producer's step, minus kCopyBias
    uint32_t lane_off[LPW];           // per-lane source offsets of the wave's copies (tile origin, step 0)
    uint32_t voff[LPW];               // the same, prepared for the grouped copies
    auto prep_voff = [&](int q0, int q1) {
#pragma unroll
        for (int q = 0; q < LPW; ++q)
            if (q >= q0 && q < q1) voff[q] = lane_off[q] + kCopyBias - ((q < LA ? q : q - LA) % GS) * 1024;
    };
    auto prod_offsets = [&]() {  // row-grouped products: rows past the tile's last and columns past N are clamped
        const int i_lim = pt.i_end - pt.i0 < BM ? pt.i_end - pt.i0 : BM;
        const int j_lim = N - pt.j0 < BN ? N - pt.j0 : BN;
#pragma unroll
        for (int q = 0; q < LA; ++q) lane_off[q] = (uint32_t)lane_src_offset<BM, BK, A_RC>(wave * LA + q, lane, lda, i_lim);
#pragma unroll
        for (int q = 0; q < LB; ++q)
            lane_off[LA + q] = (uint32_t)lane_src_offset<BN, BK, B_RC>(wave * LB + q, lane, ldb, j_lim);
        prep_voff(0, LPW);
        p_amask = 0, p_copies = LB;
#pragma unroll
        for (int j = 0; j < GA; ++j) {
            const int first_row = SA::row_of(wave * LA + GS * j, 0);
            if (first_row < i_lim) {
                p_amask |= 1u << j;
                p_copies += LA - GS * j >= GS ? GS : LA - GS * j;
            }
        }
    };
    auto prod_seek = [&]() {  // first tile from pL on that has steps
        p_more = false;
        while (pL < L_end) {
            tile_at(pL, pt);
            if (pt.KT > 0) {
                p_more = true;
                if (MODE != MODE_DW) prod_offsets();
                break;
            }
            pL += per_xcd;
        }
        pk = 0;
        p_full = MODE == MODE_DW ? pt.red / BK : pt.KT - thin_steps;
        pa_cur = uniform64((uint64_t)(uintptr_t)pt.pa - kCopyBias);
        pb_cur = uniform64((uint64_t)(uintptr_t)pt.pb - kCopyBias);
    };
#pragma unroll
    for (int q = 0; q < LB; ++q) lane_off[LA + q] = (uint32_t)lane_src_offset<BN, BK, B_RC>(wave * LB + q, lane, ldb, BN);
    if (MODE == MODE_DW) {
#pragma unroll
        for (int q = 0; q < LA; ++q) lane_off[q] = (uint32_t)lane_src_offset<BM, BK, A_RC>(wave * LA + q, lane, lda, BM);
    }
    prep_voff(0, LPW);
    prod_seek();

    // `issued` counts the vector-memory operations of this wave (copies and output stores); mark[s] is its value
    // after the last copy into ring slot s.
    unsigned issued = 0, pg = 0;  // pg: steps whose copies have been issued
    unsigned mark[SR];
#pragma unroll
    for (int s = 0; s < SR; ++s) mark[s] = 0;
    const uint32_t ring_lds = (uint32_t)(uintptr_t)(lds_void_ptr)smem;
    const uint32_t wave_a_lds = ring_lds + wave * LA * 1024, wave_b_lds = ring_lds + SA::kBytes + wave * LB * 1024;

    // Cache policy: the weights of the row-grouped products are read by one workgroup per column slice
    // (non-temporal, the L2 is left to the rows); DW: both panels are shared by the tiles of an expert.
#if defined(MFL_TUNING_BUILD) && defined(MFL_X_DW_POLICY)
    constexpr int A_POLICY = MODE == MODE_DW ? (MFL_X_DW_POLICY & 1) * 2 : 0;
    constexpr int B_POLICY = MODE == MODE_DW ? (MFL_X_DW_POLICY >> 1) * 2 : 2;
#elif defined(MFL_TUNING_BUILD) && defined(MFL_X_AB_POLICY)
    constexpr int A_POLICY = MODE == MODE_DW ? 0 : (MFL_X_AB_POLICY & 1) * 2;
    constexpr int B_POLICY = MODE == MODE_DW ? 0 : (MFL_X_AB_POLICY >> 1) * 2;
#else
    constexpr int A_POLICY = 0;
    constexpr int B_POLICY = MODE == MODE_DW ? 0 : 2;
#endif

    // group j of the producer's step (a whole step) into the ring slot at byte offset slot_off
    auto copy_group = [&](auto j_tag, uint32_t slot_off, int on) {
        constexpr int j = decltype(j_tag)::value;
        if constexpr (j < GA) {
            constexpr int q = GS * j, n = LA - q >= GS ? GS : LA - q;
            const uint32_t lds = __builtin_amdgcn_readfirstlane(wave_a_lds + slot_off + q * 1024);
            const uint64_t base = uniform64(pa_cur);
            if constexpr (A_RC) on = on & (int)((p_amask >> j) & 1u);
            if constexpr (n == 4) wide_copy4<A_POLICY>(base, voff[q], voff[q + 1], voff[q + 2], voff[q + 3], lds, on);
            else wide_copy2<A_POLICY>(base, voff[q], voff[q + 1], lds, on);
        } else {
            constexpr int qb = GS * (j - GA), q = LA + qb, n = LB - qb >= GS ? GS : LB - qb;
            const uint32_t lds = __builtin_amdgcn_readfirstlane(wave_b_lds + slot_off + qb * 1024);
            const uint64_t base = uniform64(pb_cur);
            if constexpr (n == 4) wide_copy4<B_POLICY>(base, voff[q], voff[q + 1], voff[q + 2], voff[q + 3], lds, on);
            else wide_copy2<B_POLICY>(base, voff[q], voff[q + 1], lds, on);
        }
    };
    // a partial last step of DW: rows of A past the end come from a chunk of zeros, rows of B past the end
    // re-read the last row (finite values that meet zeros); per-lane addresses, all copies at once
    auto copy_tail = [&](uint32_t slot_off) {
        const uint32_t st = ring_lds + slot_off;
        const int valid = pt.red - pk * BK;  // 1 .. BK - 1 rows
        const unsigned char *pa = (const unsigned char *)(uintptr_t)(pa_cur + kCopyBias);
        const unsigned char *pb = (const unsigned char *)(uintptr_t)(pb_cur + kCopyBias);
#pragma unroll
        for (int q = 0; q < LA; ++q) {
            const int row = SA::row_of(wave * LA + q, lane);
            const unsigned char *p = pa + lane_off[q];
            if (row >= valid) p = (const unsigned char *)&g_zero_chunk;
            wide_copy<0>(p, st + (wave * LA + q) * 1024);
        }
#pragma unroll
        for (int q = 0; q < LB; ++q) {
            const int row = SB::row_of(wave * LB + q, lane);
            const unsigned char *p = pb + lane_off[LA + q];
            if (row >= valid) p -= (int64_t)(row - (valid - 1)) * ldb * 2;
            wide_copy<0>(p, st + SA::kBytes + (wave * LB + q) * 1024);
        }
    };
    // a step of the thin last term: per-lane addresses from that term's own leading dimensions, all copies at once
    auto copy_thin = [&](uint32_t slot_off) {
        if constexpr (THIN) {
            const uint32_t st = ring_lds + slot_off;
            const int ks = pk - p_full;
            const int i_lim = pt.i_end - pt.i0 < BM ? pt.i_end - pt.i0 : BM;
            const int j_lim = N - pt.j0 < BN ? N - pt.j0 : BN;
            const unsigned char *at_tile = (const unsigned char *)(at + (int64_t)pt.i0 * kthin);
            const unsigned char *bt_tile =
                (const unsigned char *)(bt + (B_RC ? ((int64_t)pt.expert * N + pt.j0) * kthin
                                                   : (int64_t)pt.expert * N * kthin + pt.j0));
            // the lane number behind a barrier for the optimiser: what follows is worked out here, once or twice per
            // tile, and not kept in registers across the tile's other steps
            int ln = lane;
            asm volatile("" : "+v"(ln));
#pragma unroll
            for (int q = 0; q < LA; ++q) {
                const int load = wave * LA + q;
                int i = SA::row_of(load, ln);
                const int r = ks * BK + SA::swz(i, SA::phys_of(load, ln)) * 8;
                if (i >= i_lim) i = i_lim - 1;
                const unsigned char *p = r >= kthin ? (const unsigned char *)&g_zero_chunk : at_tile + ((int64_t)i * kthin + r) * 2;
                wide_copy<0>(p, st + load * 1024);
            }
#pragma unroll
            for (int q = 0; q < LB; ++q) {
                const int load = wave * LB + q;
                const int row = SB::row_of(load, ln);
                const int c = SB::swz(row, SB::phys_of(load, ln));
                const unsigned char *p;
                if (B_RC) {
                    const int j = row < j_lim ? row : j_lim - 1;
                    const int r = ks * BK + c * 8;
                    p = r >= kthin ? (const unsigned char *)&g_zero_chunk : bt_tile + ((int64_t)j * kthin + r) * 2;
                } else {
                    // rows past the end of the term re-read its last row: they meet zeros of the left operand
                    int r = ks * BK + row;
                    if (r >= kthin) r = kthin - 1;
                    int j = c * 8;
                    if (j >= j_lim) j = j_lim - 8;
                    p = bt_tile + ((int64_t)r * N + j) * 2;
                }
                wide_copy<0>(p, st + SA::kBytes + load * 1024);
            }
        }
    };
    auto prod_advance = [&](bool all_copies = false) {  // after the last copy of a step
        issued += all_copies ? LPW : p_copies;
        mark[pg % SR] = issued;
        ++pg;
        pa_cur += step_a;
        pb_cur += step_b;
        if (++pk == pt.KT) {
            pL += per_xcd;
            prod_seek();
        } else if (MODE == MODE_DX && two_term && pk == K / BK) {
            // the second term starts at the beginning of its own operands
            pa_cur = uniform64((uint64_t)((intptr_t)pt.pa + second_a) - kCopyBias);
            pb_cur = uniform64((uint64_t)((intptr_t)pt.pb + second_b) - kCopyBias);
        }
    };
    auto issue_all = [&]() {  // one whole step, back to back
        const uint32_t slot_off = (pg % SR) * STAGE_BYTES;
        bool tail = false;
        if constexpr (MODE == MODE_DW || THIN) tail = pk >= p_full;
        if (tail) {
            if constexpr (MODE == MODE_DW) copy_tail(slot_off);
            else copy_thin(slot_off);
        } else {
            static_for<NG>([&](auto j_tag) { copy_group(j_tag, slot_off, 1); });
        }
        prod_advance(tail);
    };

    // ---- consumer
    Tile ct;
    int cL = L_first;
    unsigned g = 0;  // steps multiplied so far (of the whole workgroup)
    bf16x8 fa[2][TM], fb[2][TN];  // carried from step to step, across tiles
    // The fragment offsets carry the ring slot they read: moved on by one stage at point P.
#pragma unroll
    for (int i = 0; i < decltype(fo_b)::kCount; ++i) fo_b.off[i] += SA::kBytes;
    auto frags_to_next_slot = [&]() {
        const int delta = (g + 1) % SR == 0 ? -(SR - 1) * STAGE_BYTES : STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < decltype(fo_a)::kCount; ++i) fo_a.off[i] += delta;
#pragma unroll
        for (int i = 0; i < decltype(fo_b)::kCount; ++i) fo_b.off[i] += delta;
    };
    auto load_frags = [&](int ks, int buf) {
#pragma unroll
        for (int bj = 0; bj < TN; ++bj) fb[buf][bj] = fo_b.load(smem, bj, ks);
#pragma unroll
        for (int t = 0; t < TM; ++t) fa[buf][t] = fo_a.load(smem, t, ks);
    };
    // second half of a step's copy groups, owed to the next sub-step 0 (SPLIT)
    int owed = 0;
    uint32_t owed_slot = 0;

    // prologue: SR steps in flight, the first one landed and its first fragments requested
#pragma unroll 1
    for (int s = 0; s < SR; ++s)
        if (p_more) issue_all();
    if (pg > 0) {
        wait_vmcnt_upto(issued - mark[0]);
        __builtin_amdgcn_s_barrier();
        load_frags(0, 0);
    }

    const int h = lane >> 5, rl = lane & 31;
    unsigned char *const ep = smem + RING_BYTES + wave * EP_WAVE;

    // Store u of a part covers pieces 64 u .. 64 u + 63 of its 32 x CPR pieces (row-major); the lanes' places
    // repeat every NPER stores, RPP rows further down.
    constexpr int CPR = EPC / 8, NST = 32 * CPR / 64;
    constexpr int NPER = CPR % 8 == 0 ? 1 : CPR % 4 == 0 ? CPR / 4 : CPR % 2 == 0 ? CPR / 2 : CPR;
    constexpr int RPP = 64 * NPER / CPR;
    static_assert(NST % NPER == 0 && (64 * NPER) % CPR == 0, "whole periods");
    uint32_t st_voff[NPER], st_lds[NPER], st_rc[NPER];  // global offset, LDS address, row | column << 8
#pragma unroll
    for (int e = 0; e < NPER; ++e) {
        const int q = e * 64 + lane, row = q / CPR, col = (q % CPR) * 8;
        st_voff[e] = (uint32_t)((row * (int)ldc + col) * 2);
        st_lds[e] = (uint32_t)(uintptr_t)(lds_void_ptr)(ep + row * EP_ROWB + col * 2);
        st_rc[e] = (uint32_t)(row | col << 8);
    }

    constexpr int PPT = WTN / EPC;  // parts (32 rows x EPC columns) per row block

#pragma unroll 1
    for (; cL < L_end; cL += per_xcd) {
        tile_at(cL, ct);
        const int i_lim = ct.i_end - ct.i0 < BM ? ct.i_end - ct.i0 : BM;
        const int n_blocks = ceil_div(i_lim, 32);
        int active = n_blocks > wm ? ceil_div(n_blocks - wm, WGM) : 0;
        if (active > TM || MODE == MODE_DW) active = TM;

        if (ct.KT == 0) {
            // no reduction steps: an expert without rows (DW) writes zeros, a tile without rows nothing
            if (MODE == MODE_DW) {
                const uint4_t z = {0u, 0u, 0u, 0u};
                for (int q = lane; q < TM * 32 * (WTN / 8); q += 64) {
                    const int rr = q / (WTN / 8), cc = (q % (WTN / 8)) * 8;
                    const int row = ct.i0 + (wm + WGM * (rr / 32)) * 32 + rr % 32;
                    const int col = ct.j0 + wn * WTN + cc;
                    __builtin_nontemporal_store(z, (uint4_t *)((bf16_t *)ct.pc + (int64_t)row * ldc + col));
                }
                issued += TM * 32 * (WTN / 8) / 64;
            }
            continue;
        }

        // The body of a tile for a wave with TA row blocks that hold rows (a wave without any multiplies one block
        // that nobody stores): zeroing, steps, epilogue.  One instance per TA, so that blocks past the tile's last row
        // cost no MFMA and no branch stands between the MFMAs.
        auto tile_body = [&](auto ta_tag) {
        constexpr int TA = decltype(ta_tag)::value;
        floatx16 acc[TA][TN];
        // One reduction step.  The order of the instructions inside a sub-step is pinned: a wave that is alone on
        // its SIMD overlaps nothing by itself, and a batch of LDS reads ahead of a batch of MFMAs costs the sum of
        // the two (the reads of a batch queue up behind those of the other three waves while the matrix unit idles).
        // So the NM MFMAs of sub-step ks alternate with the NU fragment reads of the sub-step after it -- after the
        // step's barrier those of the next step's first sub-step -- and in the last sub-step also with the copies of
        // step g+SR.  A partial last step of DW multiplies all its sub-steps: rows past the end are zeros in A.
        constexpr int NM = TA * TN, NU = TM + TN;
        auto read_unit = [&](auto u_tag, int rks, int buf) {
            constexpr int U = decltype(u_tag)::value;
            if constexpr (kNoRead) {
                asm volatile("" : "+v"(fb[buf][0]));
                return;
            }
            if constexpr (U < TN)
                fb[buf][U] = fo_b.load(smem, U, rks);
            else
                fa[buf][U - TN] = fo_a.load(smem, U - TN, rks);
        };
        // Sub-step ks: its MFMAs, the fragment reads of sub-step rks (of this step, or after point P of the next
        // one) and the copy groups [G0, G1) of the producer's step, issued if `on`.
        auto substep = [&](auto ks_tag, auto g0_tag, auto g1_tag, int rks, uint32_t slot_off, int on) {
            constexpr int ks = decltype(ks_tag)::value, G0 = decltype(g0_tag)::value, G1 = decltype(g1_tag)::value;
            static_for<NM>([&](auto i_tag) {
                constexpr int I = decltype(i_tag)::value, t = I / TN, bj = I % TN;
                if (!kNoMfma)
                    acc[t][bj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[ks & 1][bj], fa[ks & 1][t], acc[t][bj], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                // read unit u follows MFMA u * NM / NU
                static_for<NU>([&](auto u_tag) {
                    if constexpr (decltype(u_tag)::value * NM / NU == I) read_unit(u_tag, rks, (ks + 1) & 1);
                });
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (G1 > G0) {
                    // copy group j follows MFMA (j - G0) * NM / (G1 - G0)
                    static_for<NG>([&](auto j_tag) {
                        constexpr int J = decltype(j_tag)::value;
                        if constexpr (J >= G0 && J < G1 && (J - G0) * NM / (G1 - G0) == I) copy_group(j_tag, slot_off, on);
                    });
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
        };
        auto step = [&]() {
            MFL_TR(1)
            // first sub-step: with it the copy groups that the previous step's point P left for later
            if constexpr (SPLIT) {
                substep(IC<0>{}, IC<NG1>{}, IC<NG>{}, 1, owed_slot, owed);
                if (owed) prod_advance();
                owed = 0;
            } else {
                substep(IC<0>{}, IC<0>{}, IC<0>{}, 1, 0, 0);
            }
            static_for<KS - 2>([&](auto k_tag) {
                constexpr int ks = decltype(k_tag)::value + 1;
                substep(IC<ks>{}, IC<0>{}, IC<0>{}, ks + 1, 0, 0);
            });
            // ---- point P: my reads of this stage are done, my copies of the next step have landed
            MFL_TR(2)
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (g + 1 < pg) {
                const unsigned n = issued - mark[(g + 1) % SR];
                if (n == (SR - 2) * LPW) wait_vmcnt<(SR - 2) * LPW>();  // the steady state
                else wait_vmcnt_upto((int)n);
            }
            MFL_TR(3)
            __builtin_amdgcn_s_barrier();
            MFL_TR(4)
            // (past the workgroup's last step the reads fetch a stage nobody uses)
            frags_to_next_slot();
            int spread = 0;
            const uint32_t slot_off = (pg % SR) * STAGE_BYTES;
            if (p_more) {
                bool tail = false;
                if constexpr (MODE == MODE_DW || THIN) tail = pk >= p_full;
                if (tail) {
                    if constexpr (MODE == MODE_DW) copy_tail(slot_off);
                    else copy_thin(slot_off);
                    prod_advance(true);
                } else {
                    spread = 1;
                }
            }
            spread = __builtin_amdgcn_readfirstlane(spread);
            substep(IC<KS - 1>{}, IC<0>{}, IC<NG1>{}, 0, slot_off, spread);
            if (spread) {
                if constexpr (SPLIT) {
                    owed = 1;
                    owed_slot = slot_off;
                } else {
                    prod_advance();
                }
            }
            ++g;
        };
        {
            // zeros from the matrix unit: 0 x 0 + 0 (one instruction per 16 registers instead of 16 moves)
            const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            bf16x8 zf;
#pragma unroll
            for (int u = 0; u < 8; ++u) zf[u] = (bf16_t)0.f;
#pragma unroll
            for (int t = 0; t < TA; ++t)
#pragma unroll
                for (int bj = 0; bj < TN; ++bj) {
                    asm volatile("" : "+v"(zf));  // sixteen instructions, not one and fifteen copies of its result
                    acc[t][bj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(zf, zf, zero, 0, 0, 0);
                }
        }
        {
            int kc = 0;  // KT >= 1 here
#pragma unroll 1
            do step();
            while (++kc < ct.KT);
        }
        MFL_TR(5)

        // ---- epilogue: a 32-row block of EPC columns at a time through the wave's own staging area (8 bytes per
        // lane and write), then whole 16-byte pieces of rows, streaming stores from a scalar base plus a per-lane
        // offset that is the same for every tile.  Accumulators are fetched sixteen at a time into registers of their
        // own, so that converting and writing one group does not wait for the fetch of the next.
        const uint64_t c_tile = uniform64((uint64_t)(uintptr_t)ct.pc +
                                          (((int64_t)(ct.i0 + wm * 32)) * ldc + ct.j0 + wn * WTN) * 2);
        // Part p (a 32-row block of one row block t, EPC columns) is fetched while the staged pieces of part p - 1
        // are on their way back from LDS, and converted and staged after the stores of part p - 1 have gone out.
        constexpr int NP = TA * PPT, BPP = EPC / 32;  // parts, 32-column blocks per part
        float v[BPP][16];
        uint4_t piece[NST];
        auto fetch = [&](auto p_tag) {
            constexpr int p = decltype(p_tag)::value, t = p / PPT, part = p % PPT;
#pragma unroll
            for (int bq = 0; bq < BPP; ++bq)
#pragma unroll
                for (int u = 0; u < 16; ++u) v[bq][u] = acc_read(acc[t][part * BPP + bq][u]);
        };
        auto stage = [&]() {
#pragma unroll
            for (int bq = 0; bq < BPP; ++bq)
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    union {
                        bf16_t e[4];
                        uint2_t v;
                    } pk4;
#pragma unroll
                    for (int u = 0; u < 4; ++u) pk4.e[u] = (bf16_t)v[bq][4 * gq + u];
                    *(uint2_t *)(ep + rl * EP_ROWB + (bq * 32 + 8 * gq + 4 * h) * 2) = pk4.v;
                }
        };
        auto store = [&](auto p_tag) {
            constexpr int p = decltype(p_tag)::value, t = p / PPT, part = p % PPT;
            const int row_base = ct.i0 + (wm + WGM * t) * 32;
            const int col0 = ct.j0 + wn * WTN + part * EPC;
            const uint64_t c_part = c_tile + ((int64_t)t * (WGM * 32) * ldc + part * EPC) * 2;
#pragma unroll
            for (int u = 0; u < NST; ++u) {
                // a store whose rows all lie past the tile's last one, or whose columns all lie past N, is left
                // out, and not counted
                if (MODE != MODE_DW && (row_base + u * 64 / CPR >= ct.i_end || col0 >= N)) continue;
                if (kNoStore) continue;
#if defined(MFL_TUNING_BUILD) && defined(MFL_X_HALF_STORE)
                if (p >= NP / 2) continue;
#endif
                ++issued;
                const int down = (u / NPER) * RPP;
                const uint64_t c_rows = c_part + (int64_t)down * ldc * 2;
                const uint32_t off = st_voff[u % NPER];  // (operands of a statement in a nested lambda: its own locals)
                const uint4_t data = piece[u];
                const int st_row = (int)(st_rc[u % NPER] & 255u), st_col = (int)(st_rc[u % NPER] >> 8);
                if (MODE == MODE_DW || (row_base + down + st_row < ct.i_end && col0 + st_col < N))
                    asm volatile("global_store_dwordx4 %0, %1, %2 nt" : : "v"(off), "v"(data), "s"(c_rows) : "memory");
            }
        };
        if (active > 0) {
            fetch(IC<0>{});
            stage();
            static_for<NP>([&](auto p_tag) {
                constexpr int p = decltype(p_tag)::value;
                __builtin_amdgcn_sched_barrier(0);
                // the same wave reads back what it wrote: LDS operations of one wave complete in order
#pragma unroll
                for (int u = 0; u < NST; ++u)
                    piece[u] = *(const __attribute__((address_space(3))) uint4_t *)(st_lds[u % NPER] + (u / NPER) * RPP * EP_ROWB);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (p + 1 < NP) fetch(IC<p + 1>{});
                __builtin_amdgcn_sched_barrier(0);
                store(p_tag);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (p + 1 < NP) stage();
            });
        }
        MFL_TR(6)
        };  // tile_body
        if (MODE == MODE_DW)
            tile_body(IC<TM>{});
        else if (TM == 1 || active <= 1)
            tile_body(IC<1>{});
        else if (TM == 2 || active == 2)
            tile_body(IC<(TM >= 2 ? 2 : 1)>{});
        else if (TM == 3 || active == 3)
            tile_body(IC<(TM >= 3 ? 3 : 1)>{});
        else if (TM == 4 || active == 4)
            tile_body(IC<(TM >= 4 ? 4 : 1)>{});
        else
            tile_body(IC<TM>{});
    }
#if defined(MFL_TUNING_BUILD) && defined(MFL_X_TRACE)
    if (blockIdx.x == MFL_X_TRACE && wave == 0) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        for (int i = lane; i < 2 * tr_n; i += 64) g_wide_trace[i] = ((unsigned int *)(smem + MFL_TR_LDS))[i];
        if (lane == 0) g_wide_trace_n = tr_n;
    }
#endif
}

template <int MODE, int MB, int NB, int BK, int SR, bool THIN = false>
int launch_wide(const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N, int K,
                int E, hipStream_t stream, const void *a2 = nullptr, const void *b2 = nullptr, const void *at = nullptr,
                const void *bt = nullptr, int kthin = 0) {
    constexpr int STAGE_BYTES = (MB + NB) * 32 * BK * 2;
    constexpr int WTN = NB / 2 * 32;
    constexpr int EPC = WTN % 64 == 0 ? 64 : WTN;
    constexpr int EP_ROWB = EPC * 2 + (EPC == 64 ? 16 : 8);
#if defined(MFL_TUNING_BUILD) && defined(MFL_X_TRACE)
    constexpr int LDS_BYTES = 160 * 1024;
#else
    constexpr int LDS_BYTES = SR * STAGE_BYTES + 4 * 32 * EP_ROWB + 2 * (kMaxTableExperts + 1) * 4;
#endif
    static_assert(LDS_BYTES <= 160 * 1024, "LDS capacity of a CDNA4 compute unit");
    auto kern = gemm_wide_kernel<MODE, MB, NB, BK, SR, THIN, bf16_t>;
    static PerDeviceOnce attr;
    const hipError_t e = attr.run(
        [&] { return hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES); });
    if (e != hipSuccess) return (int)e;
    const int grid = device_info().cu_count / kXcd * kXcd;
    kern<<<grid, 256, LDS_BYTES, stream>>>((const bf16_t *)a, (const bf16_t *)b, m_sizes, ms_i64, (bf16_t *)c, R, N, K, E,
                                           (const bf16_t *)a2, (const bf16_t *)b2, (const bf16_t *)at, (const bf16_t *)bt, kthin);
    return launch_status();
}

}  // namespace

#ifdef MFL_TUNING_BUILD
int g_wide_variant = 0;  // 0: 320 x 192 tiles where N allows, 1: 256 x 256 tiles, 3: 192 x 256 tiles, -1: the library's choice
#endif

int gemm_bf16_wide(int mode, const void *a, const void *b, const void *m_sizes, int ms_i64, void *c, int64_t R, int N,
                   int K, int E, int out_dtype, float alpha, int accumulate, hipStream_t stream, const void *a2,
                   const void *b2, const void *at, const void *bt, int kthin) {
    if (out_dtype != MFL_BF16 || accumulate || alpha != 1.0f || E > kMaxTableExperts || E < 1) return MFL_ERR_UNSUPPORTED;
    if (!aligned(a, 16) || !aligned(b, 16) || !aligned(c, 16)) return MFL_ERR_UNSUPPORTED;
    if ((a2 != nullptr) != (b2 != nullptr) || (a2 != nullptr && mode != MODE_DX) || !aligned(a2, 16) || !aligned(b2, 16))
        return MFL_ERR_UNSUPPORTED;
    if (mode == MODE_DW) {
        if (N % 256 != 0 || K % 256 != 0 || N < 256 || K < 256) return MFL_ERR_UNSUPPORTED;
        return launch_wide<MODE_DW, 8, 8, 32, 4>(a, b, m_sizes, ms_i64, c, R, N, K, E, stream);
    }
    if (K % 64 != 0 || K < 64 || R <= 0) return R <= 0 ? MFL_OK : MFL_ERR_UNSUPPORTED;
    // 320 x 192 tiles (an expert of up to 320 rows is one tile per column slice) up to about 512 rows per expert,
    // 256 x 256 beyond (fewer bytes per flop).  Outputs that are wide and a multiple of 256 columns, up to 152 rows
    // per expert on average (few experts then hold more than 192 rows): 192 x 256 tiles, a quarter fewer tiles and
    // reduction steps per CU than with 192-column slices (N = 2048, K = 768, 128 experts: 8 slices an expert
    // instead of 11, 4 tiles a CU instead of 5.5; 88 / 91 / 97 / 106 / 110 us against 95 / 100 / 107 / 118 / 124 at
    // 48 / 64 / 96 / 128 / 160 rows per expert, forward and input gradient alike; 154 against 137 at 192).
    // From there to 232 rows per expert such outputs take the 256 x 256 tiles (few experts hold more than 256 rows;
    // 8 slices an expert again): 111 / 114 / 118 / 139 us against 120 / 127 / 134 / 147 at 168 / 184 / 192 / 224 rows
    // per expert (and against 120 at 168 on the 192 x 256 tiles), 164 against 158 at 256.
    const bool wide_n = N % 256 == 0 && N >= 1024;
    const bool wide_out = wide_n && R <= (int64_t)kWideOutRowsPerExpert * E && at == nullptr;
    const bool wide_mid = wide_n && R > (int64_t)kWideOutRowsPerExpert * E && R <= (int64_t)kWideMidRowsPerExpert * E;
#ifdef MFL_TUNING_BUILD
    const int v = g_wide_variant >= 0 ? g_wide_variant : (R >= (int64_t)512 * E || wide_mid ? 1 : wide_out ? 3 : 0);
#else
    const int v = R >= (int64_t)512 * E || wide_mid ? 1 : wide_out ? 3 : 0;
#endif
    if (N % 8 != 0 || N < 8) return MFL_ERR_UNSUPPORTED;
    if (at != nullptr) {
        // the thin last term: kernels of their own (its test in every step would cost the plain products)
        if (bt == nullptr || kthin < 8 || kthin % 8 != 0 || !aligned(at, 16) || !aligned(bt, 16)) return MFL_ERR_UNSUPPORTED;
        if (v == 0) {
            if (mode == MODE_FWD)
                return launch_wide<MODE_FWD, 10, 6, 64, 2, true>(a, b, m_sizes, ms_i64, c, R, N, K, E, stream, nullptr,
                                                                 nullptr, at, bt, kthin);
            return launch_wide<MODE_DX, 10, 6, 64, 2, true>(a, b, m_sizes, ms_i64, c, R, N, K, E, stream, a2, b2, at, bt, kthin);
        }
        if (mode == MODE_FWD)
            return launch_wide<MODE_FWD, 8, 8, 64, 2, true>(a, b, m_sizes, ms_i64, c, R, N, K, E, stream, nullptr, nullptr,
                                                            at, bt, kthin);
        return launch_wide<MODE_DX, 8, 8, 64, 2, true>(a, b, m_sizes, ms_i64, c, R, N, K, E, stream, a2, b2, at, bt, kthin);
    }
#ifdef MFL_TUNING_BUILD
    // 256 x 256 tiles with four stages of 32 reduction indices (96 KiB in flight instead of 64; rows of 64 bytes in
    // the stages of the operands that are contiguous along the reduction): measured 9 % slower in the forward
    // product at 1024 rows per expert (twice the barriers, half-line requests), 3 % faster in dX
    if (v == 2) {
        if (mode == MODE_FWD) return launch_wide<MODE_FWD, 8, 8, 32, 4>(a, b, m_sizes, ms_i64, c, R, N, K, E, stream);
        return launch_wide<MODE_DX, 8, 8, 32, 4>(a, b, m_sizes, ms_i64, c, R, N, K, E, stream, a2, b2);
    }
#endif
    if (v == 3) {
        if (mode == MODE_FWD) return launch_wide<MODE_FWD, 6, 8, 64, 2>(a, b, m_sizes, ms_i64, c, R, N, K, E, stream);
        return launch_wide<MODE_DX, 6, 8, 64, 2>(a, b, m_sizes, ms_i64, c, R, N, K, E, stream, a2, b2);
    }
    if (v == 0) {
        if (mode == MODE_FWD) return launch_wide<MODE_FWD, 10, 6, 64, 2>(a, b, m_sizes, ms_i64, c, R, N, K, E, stream);
        return launch_wide<MODE_DX, 10, 6, 64, 2>(a, b, m_sizes, ms_i64, c, R, N, K, E, stream, a2, b2);
    }
    if (mode == MODE_FWD) return launch_wide<MODE_FWD, 8, 8, 64, 2>(a, b, m_sizes, ms_i64, c, R, N, K, E, stream);
    return launch_wide<MODE_DX, 8, 8, 64, 2>(a, b, m_sizes, ms_i64, c, R, N, K, E, stream, a2, b2);
}

}  // namespace mfl
