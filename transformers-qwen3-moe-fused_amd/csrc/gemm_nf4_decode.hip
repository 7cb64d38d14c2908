// Fused NF4 grouped GEMM for decode-sized batches (a few rows per expert): the packed weights are
// all the traffic, so the kernel is built around streaming them.
//
// A workgroup (4 waves) owns 32 rows of one expert and 128 output columns; every wave owns one
// 32-column block and works alone: no LDS stage, no barrier in the reduction loop.
//   * v_mfma_f32_32x32x16_bf16 takes from lane l of its first operand 8 reduction elements of
//     column l % 32 (group l / 32): 8 weights = one packed dword.  The reduction index is
//     permuted (the same way for both operands, which leaves the sum unchanged) so that a lane
//     owns 32 consecutive weights of its column per 64-wide step: ONE 16-byte load per lane and
//     step feeds 4 MFMAs.  The weights are decoded in registers (16-entry code table in LDS,
//     code * absmax in fp32, one rounding to bf16) straight into the fragment layout.
//   * the rows are multiplied the same way: lane l holds 32 consecutive elements of row l % 32
//     (64 bytes).  They are loaded eight lanes to a row and change hands in a 4 KiB LDS stage of
//     the wave: a load of one row per lane costs the L1 one tag lookup per lane.
//   * loads run DEPTH steps ahead in registers, and two or three workgroups share a CU: tens of
//     KiB of packed weights in flight per CU.
// The accumulator of a lane holds output row l % 32, columns 8g + 4*(l / 32) + {0..3}.
//
// Two fusions with the neighbours of the product in the sparse MLP block:
//   * gathered rows: row i of x is row row_idx[i] / idx_div of the token matrix;
//   * gated linear unit: the wave multiplies the same rows with the same columns of a second
//     weight matrix (gate = first, up = second) and stores silu(gate) * up, rounded the way the
//     separate kernels round.
#include "common.h"
#include "gemm.h"

namespace mfl {

namespace {

constexpr int kDepth = 4;  // steps in flight

// SUPER (K % 256 == 0): the reduction index is permuted over 256-wide super-steps so that a lane
// owns 128 consecutive weights of its column (64 packed bytes: one half of a 128-byte line) per
// super-step and fetches them with four back-to-back loads, once every four steps.  With one
// 16-byte load per step instead, the four touches of a line were four steps apart and the L1
// had lost the line each time: 875 MB of requests to L2 per launch for 113 MB of weights and 8 MB
// of rows at 256 tokens.
// AM1 (quantisation blocks of at least 32 weights): the 32 weights of a lane and step share one
// scale, fetched with one load instead of four.  Every lane reads its own line of the scales, so a
// load instruction costs the L1 as many tag lookups as it has lanes, and those lookups, not bytes,
// are what the kernel runs out of.
template <bool GLU, bool SUPER, bool AM1, bool XSTAGE, typename TO>
__global__ __launch_bounds__(256) void nf4_decode_kernel(const bf16_t *__restrict__ x,
                                                         const int32_t *__restrict__ row_idx, int idx_div,
                                                         Nf4Matrix w0, Nf4Matrix w1,
                                                         const void *__restrict__ m_sizes, int ms_i64,
                                                         TO *__restrict__ y, TO *__restrict__ e_out,
                                                         TO *__restrict__ g_out, int64_t R, int N, int K, int E,
                                                         int tiles_n) {
    constexpr int CB = GLU ? 2 : 1;  // products per wave: block cb uses weight matrix cb
    __shared__ float lut[16 * CB];
    // 4 KiB per wave: the rows of one step on their way from the layout they are loaded in (eight
    // lanes per row) to the layout the MFMA takes them in (a lane per row and half)
    __shared__ __attribute__((aligned(16))) unsigned char x_stage[XSTAGE ? 4 : 1][XSTAGE ? 4096 : 16];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, h = lane >> 5;
    if (tid < 16) lut[tid] = w0.code16[tid];
    if (GLU && tid >= 16 && tid < 32) lut[tid] = w1.code16[tid - 16];

    // ---- which 32 rows: row tile blockIdx.x / tiles_n in the order of the experts
    const int ct = blockIdx.x % tiles_n, rt = blockIdx.x / tiles_n;
    int expert = -1, m_start = 0, m_size = 0, t_begin = 0;
    {
        int row_carry = 0, tile_carry = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            const int m = e < E ? load_msize(m_sizes, ms_i64, e) : 0;
            const int t = ceil_div(m, 32);
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
    __syncthreads();  // the code table is in LDS (every wave of the workgroup takes the same path below)
    if (expert < 0) return;
    expert = __builtin_amdgcn_readfirstlane(expert);
    const int i0 = __builtin_amdgcn_readfirstlane(m_start) + (rt - __builtin_amdgcn_readfirstlane(t_begin)) * 32;
    int i_end = __builtin_amdgcn_readfirstlane(m_start) + __builtin_amdgcn_readfirstlane(m_size);
    if ((int64_t)i_end > R) i_end = (int)R;
    const int rows = i_end - i0 < 32 ? i_end - i0 : 32;
    if (rows <= 0) return;

    // ---- this lane's sources
    const int j0 = (ct * 4 + wave) * 32;  // first column of the wave
    int64_t w_el;                         // first weight of the lane in step 0
    {
        int col = j0 + n;
        if (col >= N) col = N - 1;  // loaded, multiplied, never stored
        w_el = ((int64_t)expert * N + col) * K + h * (SUPER ? 128 : 32);
    }
    // element offset of reduction step kt from the lane's first element
    auto step_off = [](int kt) { return SUPER ? (kt >> 2) * 256 + (kt & 3) * 32 : kt * 64; };
    // XSTAGE (more than a row or two per expert; with fewer, the lanes of a load that reads one
    // row per lane mostly hit the same lines anyway, and the detour costs 2 us at 16 tokens).
    // Rows: load u of a step brings rows 8u .. 8u+7, eight lanes per row: four lanes per 64-byte
    // piece (the piece of half 0 and the piece of half 1), so an instruction touches 8 or 16 lines
    // instead of 64.  The lanes pass the chunks on through the wave's LDS stage (no barrier: LDS
    // operations of one wave complete in order); chunk c of row r sits at c ^ ((r >> 1) & 7), which
    // keeps the reads of 16 lanes in 16 different bank groups.
    const bf16_t *x_src[4];
    int x_wr[4], x_rd[4];
    unsigned char *xl = x_stage[wave];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        // without the stage: lane l loads 64 bytes of row l % 32 itself, chunk u with load u
        const int r = XSTAGE ? 8 * u + (lane >> 3) : n, p = XSTAGE ? (lane >> 2) & 1 : h, q = XSTAGE ? lane & 3 : u;
        int64_t src_row = i0 + (r < rows ? r : rows - 1);
        if (row_idx != nullptr) src_row = (uint32_t)row_idx[src_row] / (uint32_t)idx_div;
        x_src[u] = x + src_row * K + p * (SUPER ? 128 : 32) + q * 8;
        x_wr[u] = r * 128 + (((p * 4 + q) ^ ((r >> 1) & 7)) << 4);
        x_rd[u] = n * 128 + (((h * 4 + u) ^ ((n >> 1) & 7)) << 4);
    }
    const int KT = K / 64;
    const uint8_t *wq_of[2] = {w0.wq, w1.wq};
    const float *am_of[2] = {w0.absmax, w1.absmax};
    const int shift_of[2] = {w0.bs_shift, w1.bs_shift};

    struct Step {
        uint4_t w[CB];
        float am[CB][4];
        uint4_t xs[4];
    };
    auto load = [&](int kt, Step &s) {
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            const int64_t el = w_el + step_off(kt);
            if (!SUPER) s.w[cb] = *(const uint4_t *)(wq_of[cb] + (el >> 1));
            if (AM1) {
                s.am[cb][0] = am_of[cb][el >> shift_of[cb]];
            } else {
#pragma unroll
                for (int u = 0; u < 4; ++u) s.am[cb][u] = am_of[cb][(el + 8 * u) >> shift_of[cb]];
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) s.xs[u] = *(const uint4_t *)(x_src[u] + step_off(kt));
    };

    floatx16 acc[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[cb][r] = 0.f;

    // packed weights of a whole super-step: [matrix][step of the super-step]
    struct SuperW {
        uint4_t w[CB][4];
    };
    auto load_w = [&](int super, SuperW &sw) {
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            const uint4_t *p = (const uint4_t *)(wq_of[cb] + ((w_el + (int64_t)super * 256) >> 1));
#pragma unroll
            for (int d = 0; d < 4; ++d) sw.w[cb][d] = p[d];
        }
    };

    auto multiply = [&](const Step &s, const SuperW &sw, int d) {
        if (XSTAGE) {
#pragma unroll
            for (int u = 0; u < 4; ++u) *(uint4_t *)(xl + x_wr[u]) = s.xs[u];
            // lanes read below what other lanes of the wave wrote: say so (no instructions; without it the compiler
            // may treat the reads as reads of this lane's own writes only)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            union {
                uint4_t u;
                bf16x8 v;
            } xa;
            xa.u = XSTAGE ? *(const uint4_t *)(xl + x_rd[ks]) : s.xs[ks];
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                const uint32_t w = SUPER ? sw.w[cb][d][ks] : s.w[cb][ks];
                const float am = AM1 ? s.am[cb][0] : s.am[cb][ks];
                bf16x8 wf;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t nib = (w >> (8 * (j >> 1) + ((j & 1) ? 0 : 4))) & 15u;
                    wf[j] = (bf16_t)(lut[16 * cb + nib] * am);
                }
                acc[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xa.v, acc[cb], 0, 0, 0);
            }
        }
    };

    Step st[kDepth];  // st[j] holds a step congruent to j modulo kDepth
#pragma unroll
    for (int d = 0; d < kDepth; ++d)
        if (d < KT) load(d, st[d]);
    static_assert(kDepth == 4, "a super-step is kDepth steps");
    SuperW sw0, sw1;
    if (SUPER) {
        load_w(0, sw0);
        load_w(KT > 4 ? 1 : 0, sw1);
    }
    // four steps: one super-step, whose weights sit in sw; when it is done sw is refilled for the
    // super-step after the next
    auto four_steps = [&](int kt, SuperW &sw) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            if (kt + d < KT) {
                multiply(st[d], sw, d);
                if (kt + d + kDepth < KT) load(kt + d + kDepth, st[d]);
            }
        }
        if (SUPER && kt + 8 < KT) load_w(kt / 4 + 2, sw);
    };
    if (SUPER) {
        // One super-step per iteration, the loop body one straight run of code: every load is
        // issued unconditionally (past the end it re-reads the last step), so that the waits the
        // compiler places count exactly the loads that may still be in flight.  With loads under
        // "if (step < KT)" it waited for ALL outstanding loads at the top of every iteration, which
        // cut the prefetch distance from four steps to about one.
        const int n_super = KT / 4;
        for (int sp = 0; sp < n_super; ++sp) {
#pragma unroll
            for (int d = 0; d < kDepth; ++d) {
                multiply(st[d], sw0, d);
                const int nxt = 4 * sp + d + kDepth;
                load(nxt < KT ? nxt : KT - 1, st[d]);
            }
            sw0 = sw1;
            load_w(sp + 2 < n_super ? sp + 2 : n_super - 1, sw1);
        }
    } else {
        for (int kt = 0; kt < KT; kt += 2 * kDepth) {
            four_steps(kt, sw0);
            if (kt + kDepth < KT) four_steps(kt + kDepth, sw1);
        }
    }

    // ---- output: lane = row n, 4 consecutive columns per group
    if (n < rows) {
        const int64_t o_row = (int64_t)(i0 + n) * N;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int col = j0 + 8 * g + 4 * h;
            if (col >= N) continue;  // N is a multiple of 8: a group of 4 is inside or outside as a whole
            if constexpr (GLU) {
                union {
                    bf16_t e[4];
                    uint2_t v;
                } pe, pg, ph;
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    pe.e[u] = (bf16_t)acc[0][4 * g + u];
                    pg.e[u] = (bf16_t)acc[1][4 * g + u];
                    ph.e[u] = silu_fwd_one<bf16_t>(pe.e[u], pg.e[u]);
                }
                *(uint2_t *)((bf16_t *)y + o_row + col) = ph.v;
                if (e_out) *(uint2_t *)((bf16_t *)e_out + o_row + col) = pe.v;
                if (g_out) *(uint2_t *)((bf16_t *)g_out + o_row + col) = pg.v;
            } else if (sizeof(TO) == 2) {
                union {
                    bf16_t e[4];
                    uint2_t v;
                } pk;
#pragma unroll
                for (int u = 0; u < 4; ++u) pk.e[u] = (bf16_t)acc[0][4 * g + u];
                *(uint2_t *)((bf16_t *)y + o_row + col) = pk.v;
            } else {
#pragma unroll
                for (int u = 0; u < 4; ++u) y[o_row + col + u] = from_f32<TO>(acc[0][4 * g + u]);
            }
        }
    }
}

}  // namespace

int gemm_nf4_decode(const void *x, const uint8_t *wq, const float *code16, const float *absmax, int blocksize,
                    const void *m_sizes, int ms_i64, void *y, int64_t R, int N, int K, int E, int out_dtype,
                    hipStream_t stream, const GemmFusion *fusion) {
    // up to where the streaming kernel (64-row tiles) is ahead of the pipelined one: with more rows per expert every
    // row tile streams and decodes the weights again
    const bool gated = fusion != nullptr && fusion->w2 != nullptr;
    if (R <= 0) return MFL_OK;
    if (R > (int64_t)(gated ? kNf4StreamGatedRowsPerExpert : kNf4StreamRowsPerExpert) * E) return MFL_ERR_UNSUPPORTED;
    int shift = 0;
    while ((1 << shift) < blocksize) ++shift;
    if (K % 64 != 0 || N % 8 != 0 || N < 8 || blocksize < 8) return MFL_ERR_UNSUPPORTED;
    if (!aligned(x, 16) || !aligned(wq, 16) || !aligned(y, 16)) return MFL_ERR_UNSUPPORTED;
    if (out_dtype != MFL_BF16 && out_dtype != MFL_F32) return MFL_ERR_UNSUPPORTED;
    Nf4Matrix w0 = {wq, code16, absmax, shift};
    if (fusion != nullptr) w0.absmax_tiled = fusion->absmax_tiled;
    Nf4Matrix w1 = w0;
    const int32_t *row_idx = nullptr;
    int idx_div = 1;
    void *e_out = nullptr, *g_out = nullptr;
    bool glu = false;
    if (fusion != nullptr) {
        if (fusion->row_idx != nullptr) {
            if (fusion->idx_div <= 0 || fusion->src_rows <= 0) return MFL_ERR_UNSUPPORTED;
            row_idx = fusion->row_idx;
            idx_div = fusion->idx_div;
        }
        if (fusion->w2 != nullptr) {
            int shift2 = 0;
            while ((1 << shift2) < fusion->blocksize_2) ++shift2;
            if (out_dtype != MFL_BF16 || fusion->blocksize_2 < 8 || !fusion->code16_2 || !fusion->absmax_2 ||
                !aligned(fusion->w2, 16) || !aligned(fusion->e_out, 8) || !aligned(fusion->g_out, 8))
                return MFL_ERR_UNSUPPORTED;
            glu = true;
            w1 = Nf4Matrix{(const uint8_t *)fusion->w2, fusion->code16_2, fusion->absmax_2, shift2, fusion->absmax_tiled_2};
            e_out = fusion->e_out;
            g_out = fusion->g_out;
        }
    }
    // 128 columns per workgroup: the most workgroups per expert (two blocks per wave: slower)
    const int tiles_n = ceil_div(N, 128);
    const int64_t row_tiles = R / 32 + (R < E ? R : E);  // upper bound on sum over experts of ceil(m / 32)
    const int64_t grid = row_tiles * tiles_n;
    if (grid > 0x7fffffff) return MFL_ERR_UNSUPPORTED;
    const bf16_t *px = (const bf16_t *)x;
    {
        const int rc = gemm_nf4_gemv(px, row_idx, idx_div, w0, w1, glu, m_sizes, ms_i64, y, e_out, g_out, R, N, K, E,
                                     out_dtype, stream);
        if (rc != MFL_ERR_UNSUPPORTED) return rc;
    }
    {
        const int rc = gemm_nf4_stream(px, row_idx, idx_div, w0, w1, glu, m_sizes, ms_i64, y, e_out, g_out, R, N, K, E,
                                       out_dtype, stream);
        if (rc != MFL_ERR_UNSUPPORTED) return rc;
    }
    if (R > (int64_t)kNf4DecodeRowsPerExpert * E) return MFL_ERR_UNSUPPORTED;  // 32-row tiles from here on
    const bool wide = K % 256 == 0;  // 64 packed bytes per lane and super-step
    const bool am1 = w0.bs_shift >= 5 && w1.bs_shift >= 5;  // one scale per lane and step
    const bool xstage = R > 2 * (int64_t)E;                   // rows change hands in LDS
#define MFL_DECODE_K(GLU, SUPER, AM1, XS, TO, Y, EO, GO)                                        \
    nf4_decode_kernel<GLU, SUPER, AM1, XS, TO><<<(unsigned)grid, 256, 0, stream>>>(                \
        px, row_idx, idx_div, w0, w1, m_sizes, ms_i64, Y, EO, GO, R, N, K, E, tiles_n)
#define MFL_DECODE(GLU, SUPER, TO, Y, EO, GO)                                                   \
    do {                                                                                        \
        if (am1 && xstage)                                                                      \
            MFL_DECODE_K(GLU, SUPER, true, true, TO, Y, EO, GO);                                \
        else if (am1)                                                                           \
            MFL_DECODE_K(GLU, SUPER, true, false, TO, Y, EO, GO);                               \
        else if (xstage)                                                                        \
            MFL_DECODE_K(GLU, SUPER, false, true, TO, Y, EO, GO);                               \
        else                                                                                    \
            MFL_DECODE_K(GLU, SUPER, false, false, TO, Y, EO, GO);                              \
    } while (0)
    if (glu) {
        if (wide)
            MFL_DECODE(true, true, bf16_t, (bf16_t *)y, (bf16_t *)e_out, (bf16_t *)g_out);
        else
            MFL_DECODE(true, false, bf16_t, (bf16_t *)y, (bf16_t *)e_out, (bf16_t *)g_out);
    } else if (out_dtype == MFL_BF16) {
        if (wide)
            MFL_DECODE(false, true, bf16_t, (bf16_t *)y, nullptr, nullptr);
        else
            MFL_DECODE(false, false, bf16_t, (bf16_t *)y, nullptr, nullptr);
    } else {
        if (wide)
            MFL_DECODE(false, true, float, (float *)y, nullptr, nullptr);
        else
            MFL_DECODE(false, false, float, (float *)y, nullptr, nullptr);
    }
#undef MFL_DECODE
#undef MFL_DECODE_K
    return launch_status();
}

}  // namespace mfl
