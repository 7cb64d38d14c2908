// Weight-gradient product with one thin side, the reduction dealt out evenly over the workgroups.
//
//   dw[e, n, k] = alpha * sum_{m in expert e} dy[m, n] * x[m, k]
//   (qwen3_moe_fused/grouped_gemm/backward_dw.py:64-89)
//
// with N or K equal to 8, 16, 32 or 64 -- the rank of a LoRA adapter (qwen3_moe_fused/lora.py:71-72), i.e. the
// products dA and dB of qwen3_moe_fused/kernels/fast_lora.py:121-125,139-149 -- and the other side a multiple
// of 256.  Such a product does nothing but stream its wide operand once, and a tile per (expert, slice) as in
// the general kernel makes the expert with the most rows the last to finish, however the tiles are dealt:
// under skewed routing one workgroup then streams a sixteenth of all rows.  Here the unit of work is a step of
// 32 consecutive rows of one expert, all steps of the launch are numbered in row order, and workgroup
// (chunk c, slice s) takes steps [c * spc, (c + 1) * spc) of the 256 columns s of the wide operand: every
// workgroup streams the same number of bytes, in pieces of 512 contiguous bytes per row.
//   * an expert whose steps all lie in one chunk is finished by that workgroup and written in the output type;
//   * an expert cut by a chunk border leaves one fp32 partial sum per chunk it touches in the workspace (a
//     chunk has at most two such experts: the one it starts in and the one it ends in), and a second kernel
//     adds an expert's partial sums in chunk order, scales and rounds once.  The order of the additions is
//     fixed by the sizes alone: results are the same from run to run, there are no atomics.  Which expert a
//     border cuts, and where its partial sums lie, the first kernel leaves in the workspace too (one entry per
//     border), so that the second one starts without reading the sizes;
//   * the zeros of an expert without rows are written by the workgroups that pass it: those that hold the last
//     step of the expert before it (chunk 0 for experts with no rows before them).
// Both operands have the reduction index as their slow one, so both go to LDS as they lie in memory (copies
// that bypass the registers, a ring of stages) and are read with transposing reads (ds_read_b64_tr_b16) into
// v_mfma_f32_32x32x16_bf16 fragments: the thin operand is the first MFMA operand (8, 16 or 32 of its values index the
// accumulator registers of a block; rank 64 is two blocks), the 32 columns of a block of the wide operand the second (they index the lanes).
// Rows of a step past the end of the expert are copied from a block of zeros.
#include <type_traits>

#include "common.h"
#include "gemm.h"

namespace mfl {

namespace {

typedef __attribute__((address_space(3))) void *lds_void_ptr;
typedef __attribute__((address_space(3))) short4_t *lds_short4_ptr;

constexpr int kSplitThreads = 256;  // four waves: wave w owns columns 64 w .. 64 w + 63 of the slice
constexpr int kSplitWaves = kSplitThreads / 64;
constexpr int kStepRows = 32;
constexpr int kSliceCols = 256;
// Two workgroups per compute unit with four stages each (one's set-up and drain under the other's loop) measured
// ahead of one with six or eight: dA of a rank-16 adapter at 65536 rows 58 against 61-63 us.
constexpr int kSplitStages = 4;
constexpr int kSplitPerCu = 2;
constexpr int kWideRowBytes = kSliceCols * 2;
constexpr int kWideStageBytes = kStepRows * kWideRowBytes;  // 16 KiB
constexpr int kWideCopies = kWideStageBytes / 1024 / kSplitWaves;  // per wave and step
constexpr int kCopiesPerWave = kWideCopies + 1;                    // and one (partial) copy of thin rows
constexpr int kSplitMaxExperts = 512;
constexpr int kMinStepsPerChunk = 8;

constexpr int split_stage_bytes(int th) { return kWideStageBytes + kStepRows * th * 2; }
// rank 64: three stages, so that two workgroups still fit in a compute unit's LDS
constexpr int split_stages(int th) { return th == 64 ? 3 : kSplitStages; }
constexpr int split_lds_bytes(int th) { return split_stages(th) * split_stage_bytes(th) + 2 * (kSplitMaxExperts + 1) * 4; }

__device__ uint4_t g_split_zeros = {0u, 0u, 0u, 0u};

template <int N>
__device__ __forceinline__ void split_wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | 0x70 | 0xF00 | ((N >> 4) << 14));
}

// 16 bytes per active lane from global memory to LDS address lds_addr + 16 * lane.  Written out by hand: the
// compiler orders transposing LDS reads behind every copy it knows of; the kernel waits for its copies itself.
// M0 is used by nothing else in this kernel.
__device__ __forceinline__ void split_copy(const unsigned char *src, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(lds_addr) : "memory");
}

__device__ __forceinline__ bf16x8 split_tr_fragment(const unsigned char *p, int row_bytes) {
    union {
        short4_t h[2];
        bf16x8 v;
    } u;
    u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)p);
    u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(p + 4 * row_bytes));
    return u.v;
}

__device__ __forceinline__ int split_steps_of(int m) { return m <= 0 ? 0 : ceil_div(m, kStepRows); }

// Partial sum that the chunk [c * spc, ...) holds for an expert whose first step is `first`: slot 0 of the
// chunk if the expert's part starts with the chunk, slot 1 if it starts inside it.
__device__ __forceinline__ int split_slot(int chunk, int spc, int first) { return 2 * chunk + (first <= chunk * spc ? 0 : 1); }

// TH: width of the thin operand.  THIN_N: the thin operand is dy (dw is (E, TH, WIDE), wide index contiguous);
// otherwise it is x (dw is (E, WIDE, TH), thin index contiguous).
template <int TH, bool THIN_N, typename TO>
__global__ __launch_bounds__(kSplitThreads) void dw_split_kernel(const bf16_t *__restrict__ thin,
                                                                 const bf16_t *__restrict__ wide,
                                                                 const void *__restrict__ m_sizes, int ms_i64,
                                                                 TO *__restrict__ out, float *__restrict__ partial,
                                                                 int4 *__restrict__ plan, int64_t R, int WIDE, int E,
                                                                 int chunks, float alpha) {
    static_assert(TH == 8 || TH == 16 || TH == 32 || TH == 64, "one or two MFMA blocks of thin values");
    constexpr int TB = TH == 64 ? 2 : 1;  // thin blocks of 32
    constexpr int THB = TH / TB;          // thin values per block
    constexpr int STAGE = split_stage_bytes(TH);
    constexpr int STAGES = split_stages(TH);
    constexpr int THIN_ROW = TH * 2;
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    int *tab_rows = (int *)(smem + STAGES * STAGE);
    int *tab_steps = tab_rows + (kSplitMaxExperts + 1);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slices = WIDE / kSliceCols;
    const int slice = blockIdx.x % slices, chunk = blockIdx.x / slices;
    const int col0 = slice * kSliceCols;

    // ---- rows and steps before every expert (every wave computes, wave 0 writes)
    {
        int row_carry = 0, step_carry = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            int m = e < E ? load_msize(m_sizes, ms_i64, e) : 0;
            if (m < 0) m = 0;
            const int st = split_steps_of(m);
            const int minc = wave_inclusive_scan(m), sinc = wave_inclusive_scan(st);
            if (wave == 0 && e <= E) {
                tab_rows[e] = row_carry + minc - m;
                tab_steps[e] = step_carry + sinc - st;
            }
            row_carry += wave_last(minc);
            step_carry += wave_last(sinc);
        }
        if (wave == 0 && lane == 0 && E % 64 == 0) {
            tab_rows[E] = row_carry;
            tab_steps[E] = step_carry;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
    }
    const int64_t mat = (int64_t)TH * WIDE;
    // this workgroup's 256 columns of the matrix of an expert without rows
    auto zero_slice = [&](int e) {
        constexpr int ROW16 = kSliceCols * (int)sizeof(TO) / 16;  // 16-byte pieces of a row of the slice (THIN_N)
        const uint4_t z = {0u, 0u, 0u, 0u};
        if (THIN_N) {
            for (int q = tid; q < TH * ROW16; q += kSplitThreads)
                *(uint4_t *)((unsigned char *)(out + (int64_t)e * mat + (int64_t)(q / ROW16) * WIDE + col0) + (q % ROW16) * 16) = z;
        } else {
            for (int q = tid; q < kSliceCols * TH * (int)sizeof(TO) / 16; q += kSplitThreads)
                *(uint4_t *)((unsigned char *)(out + (int64_t)e * mat + (int64_t)col0 * TH) + q * 16) = z;
        }
    };
    const int total = __builtin_amdgcn_readfirstlane(tab_steps[E]);
    const int spc = total == 0 ? 0 : ceil_div(total, chunks);
    const int s0 = chunk * spc;
    const int s1 = s0 + spc < total ? s0 + spc : total;
    if (s0 >= s1) {
        // no steps: nothing to add at this border; without any rows at all chunk 0 writes every matrix
        if (slice == 0 && tid == 0 && chunk >= 1) plan[chunk] = make_int4(-1, 0, 0, 0);
        if (total == 0 && chunk == 0)
            for (int e = 0; e < E; ++e) zero_slice(e);
        return;
    }
    const int KT = s1 - s0;

    // ---- the expert that holds step s0
    struct Cursor {
        int e, b, nb, row0, m;
    };
    auto load_expert = [&](Cursor &c) {
        c.row0 = __builtin_amdgcn_readfirstlane(tab_rows[c.e]);
        c.m = __builtin_amdgcn_readfirstlane(tab_rows[c.e + 1]) - c.row0;
        c.nb = split_steps_of(c.m);
    };
    auto advance = [&](Cursor &c) {
        if (++c.b < c.nb) return;
        c.b = 0;
        do {
            if (++c.e >= E) {
                c.e = E, c.nb = 0, c.m = 0;
                return;
            }
            load_expert(c);
        } while (c.nb == 0);
    };
    Cursor ci;
    {
        int found = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane < E ? e0 + lane : E - 1;
            const uint64_t hits = __ballot(e0 + lane < E && s0 >= tab_steps[e] && s0 < tab_steps[e + 1]);
            if (hits) {
                found = e0 + __ffsll((unsigned long long)hits) - 1;
                break;
            }
        }
        ci.e = __builtin_amdgcn_readfirstlane(found);
        load_expert(ci);
        ci.b = s0 - __builtin_amdgcn_readfirstlane(tab_steps[ci.e]);
    }
    Cursor cc = ci;
    if (slice == 0 && tid == 0 && chunk >= 1) {
        // the border before this chunk cuts expert ci.e if that expert started earlier; the first border that
        // cuts an expert adds its partial sums: first slot, then slot 0 of each of the `later` chunks after it
        const int sb = tab_steps[ci.e], se = tab_steps[ci.e + 1];
        int4 p = make_int4(-1, 0, 0, 0);
        if (sb < s0 && sb / spc + 1 == chunk) p = make_int4(ci.e, split_slot(chunk - 1, spc, sb), (se - 1) / spc - (chunk - 1), 0);
        plan[chunk] = p;
    }
    if (chunk == 0)
        for (int e = 0; e < ci.e; ++e) zero_slice(e);  // no rows, and no expert with rows before them

    // ---- per-lane constants of the copies: wave w copies rows 8 w .. 8 w + 7 of a step, two rows of the wide
    // operand per copy (16-byte chunk c of row r lies at chunk c ^ ((r & 3) << 2): the four rows that a
    // transposing read touches start 64 bytes apart), its eight thin rows with its first TH lanes
    const int wrow = 8 * wave + (lane >> 5);
    uint32_t woff[kWideCopies];
#pragma unroll
    for (int q = 0; q < kWideCopies; ++q) {
        const int row = wrow + 2 * q;
        const int c = (lane & 31) ^ ((row & 3) << 2);
        woff[q] = (uint32_t)(((int64_t)row * WIDE + c * 8) * 2);
    }
    constexpr int TCH = TH / 8;  // 16-byte chunks of a thin row
    const int trow = 8 * wave + lane / TCH;
    const uint32_t toff = (uint32_t)((trow * TH + (lane % TCH) * 8) * 2);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_void_ptr)smem;
    const unsigned char *zeros = (const unsigned char *)&g_split_zeros;

    auto issue = [&](const Cursor &c, int slot) {
        const int64_t base = (int64_t)c.row0 + kStepRows * c.b;
        int valid = c.m - kStepRows * c.b;
        if (valid > kStepRows) valid = kStepRows;
        if (base + valid > R) valid = (int)(R - base);  // sizes that sum to more than R rows: nothing past row R is read
        const unsigned char *wbase = (const unsigned char *)(wide + base * WIDE + col0);
        const unsigned char *tbase = (const unsigned char *)(thin + base * TH);
        const uint32_t st = lds0 + slot * STAGE;
#pragma unroll
        for (int q = 0; q < kWideCopies; ++q)
            split_copy(wrow + 2 * q < valid ? wbase + woff[q] : zeros, st + (wave * kWideCopies + q) * 1024);
        if (lane < TH) split_copy(trow < valid ? tbase + toff : zeros, st + kWideStageBytes + wave * (8 * THIN_ROW));
    };

    // ---- per-lane offsets of the fragment reads
    const int g = lane >> 4, il = lane & 15;
    const int fr = 8 * (g >> 1) + (il >> 2);
    const int thin_off = fr * THIN_ROW + ((16 * (g & 1) + 4 * (il & 3)) % THB) * 2;  // block tb: + 64 bytes
    int wide_off[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int i = (2 * wave + t) * 32 + 16 * (g & 1) + 4 * (il & 3);
        wide_off[t] = fr * kWideRowBytes + (((i >> 3) ^ ((fr & 3) << 2)) * 16) + (i & 7) * 2;
    }

    floatx16 acc[2][TB];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][tb][r] = 0.f;

    const int h = lane >> 5;
    auto store_block = [&](auto *dst, float scale) {
        typedef std::remove_pointer_t<decltype(dst)> T;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int j = col0 + (2 * wave + t) * 32 + (lane & 31);
#pragma unroll
            for (int tb = 0; tb < TB; ++tb) {
#pragma unroll
                for (int gg = 0; gg < THB / 8; ++gg) {
                    const int i0 = 32 * tb + 8 * gg + 4 * h;
                    if (THIN_N) {
#pragma unroll
                        for (int u = 0; u < 4; ++u)
                            dst[(int64_t)(i0 + u) * WIDE + j] = (T)(acc[t][tb][4 * gg + u] * scale);
                    } else {
                        typedef T vec4 __attribute__((ext_vector_type(4)));
                        vec4 v;
#pragma unroll
                        for (int u = 0; u < 4; ++u) v[u] = (T)(acc[t][tb][4 * gg + u] * scale);
                        *(vec4 *)(dst + (int64_t)j * TH + i0) = v;
                    }
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[t][tb][r] = 0.f;
            }
        }
    };
    auto flush = [&](int e) {
        const int sb = __builtin_amdgcn_readfirstlane(tab_steps[e]);
        const int se = __builtin_amdgcn_readfirstlane(tab_steps[e + 1]);
        if (sb >= s0 && se <= s1)
            store_block(out + (int64_t)e * mat, alpha);
        else
            store_block(partial + (int64_t)split_slot(chunk, spc, sb) * mat, 1.0f);
    };

    // ---- ring of stages: STAGES - 1 steps in flight
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < KT) {
            issue(ci, s);
            advance(ci);
        }
    for (int kt = 0; kt < KT; ++kt) {
        // this wave's copies of step kt have landed; the barrier extends that to all waves and says that
        // everybody is done with step kt - 1, whose stage is filled next
        if (kt + STAGES - 2 < KT)
            split_wait_vmcnt<(STAGES - 2) * kCopiesPerWave>();
        else
            split_wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
        if (kt + STAGES - 1 < KT) {
            issue(ci, (kt + STAGES - 1) % STAGES);
            advance(ci);
        }
        const unsigned char *sw = smem + (kt % STAGES) * STAGE, *stn = sw + kWideStageBytes;
#pragma unroll
        for (int ks = 0; ks < kStepRows / 16; ++ks) {
            bf16x8 tf[TB];
#pragma unroll
            for (int tb = 0; tb < TB; ++tb) tf[tb] = split_tr_fragment(stn + thin_off + tb * 64 + ks * 16 * THIN_ROW, THIN_ROW);
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const bf16x8 wf = split_tr_fragment(sw + wide_off[t] + ks * 16 * kWideRowBytes, kWideRowBytes);
#pragma unroll
                for (int tb = 0; tb < TB; ++tb)
                    acc[t][tb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tf[tb], wf, acc[t][tb], 0, 0, 0);
            }
        }
        if (cc.b + 1 == cc.nb || kt == KT - 1) flush(cc.e);
        if (cc.b + 1 == cc.nb) {
            // the expert's last step: the experts without rows that follow it are this workgroup's to write
            for (int e = cc.e + 1; e < E && tab_steps[e + 1] == tab_steps[e]; ++e) zero_slice(e);
        }
        advance(cc);
    }
}

// The experts cut by a chunk border.  Workgroup (border b, part p) takes 1024 elements p of the matrix of the
// expert that the first kernel noted for border b (the border between chunks b - 1 and b), if any, and adds its
// partial sums in chunk order.
template <typename TO>
__global__ __launch_bounds__(256) void dw_split_finish_kernel(const float *__restrict__ partial,
                                                              const int4 *__restrict__ plan, TO *__restrict__ out,
                                                              int mat, float alpha) {
    const int parts = mat / 1024;
    const int part = blockIdx.x % parts, border = 1 + blockIdx.x / parts;
    const int4 p = plan[border];
    if (p.x < 0) return;
    const int idx = part * 1024 + threadIdx.x * 4;
    floatx4 sum = *(const floatx4 *)(partial + (int64_t)p.y * mat + idx);
    // every chunk after the expert's first holds its part in slot 0
    const float *src = partial + (int64_t)(2 * border) * mat + idx;
#pragma unroll 8
    for (int c = 0; c < p.z; ++c, src += 2 * (int64_t)mat) sum += *(const floatx4 *)src;
    typedef TO vec4 __attribute__((ext_vector_type(4)));
    vec4 v;
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = (TO)(sum[u] * alpha);
    *(vec4 *)(out + (int64_t)p.x * mat + idx) = v;
}

int split_chunks(int64_t R, int wide) {
    const int slices = wide / kSliceCols;
    int chunks = device_info().cu_count * kSplitPerCu / slices;
    const int64_t most = R / (kStepRows * kMinStepsPerChunk);
    if (chunks > most) chunks = (int)most;
    return chunks < 1 ? 1 : chunks;
}

bool split_thin(int n) { return n == 8 || n == 16 || n == 32 || n == 64; }

bool split_shape_ok(int64_t R, int N, int K, int E) {
    if (R <= 0 || R > 0x7fffffff || E <= 0 || E > kSplitMaxExperts) return false;
    const bool thin_n = split_thin(N);
    const bool thin_k = split_thin(K);
    if (thin_n == thin_k) return false;
    const int wide = thin_n ? K : N;
    return wide % kSliceCols == 0 && wide / kSliceCols <= 256;
}

template <int TH, bool THIN_N, typename TO>
int launch_split(const bf16_t *thin, const bf16_t *wide_p, const void *m_sizes, int ms_i64, TO *out, float *partial,
                 int64_t R, int wide, int E, int chunks, float alpha, hipStream_t stream) {
    static PerDeviceOnce once;
    auto kernel = dw_split_kernel<TH, THIN_N, TO>;
    const hipError_t err = once.run([&] {
        return hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, split_lds_bytes(TH));
    });
    if (err != hipSuccess) return (int)err;
    const int slices = wide / kSliceCols;
    const int mat = TH * wide;
    int4 *plan = (int4 *)(partial + (size_t)chunks * 2 * mat);
    hipLaunchKernelGGL(kernel, dim3(slices * chunks), dim3(kSplitThreads), split_lds_bytes(TH), stream, thin, wide_p,
                       m_sizes, ms_i64, out, partial, plan, R, wide, E, chunks, alpha);
    int rc = launch_status();
    if (rc != MFL_OK || chunks == 1) return rc;
    hipLaunchKernelGGL(dw_split_finish_kernel<TO>, dim3((chunks - 1) * (mat / 1024)), dim3(256), 0, stream, partial,
                       plan, out, mat, alpha);
    return launch_status();
}

}  // namespace

size_t gemm_dw_split_workspace(int64_t R, int N, int K, int E) {
    if (!split_shape_ok(R, N, K, E)) return 0;
    const bool thin_n = split_thin(N);
    const int wide = thin_n ? K : N, th = thin_n ? N : K;
    // two partial sums and one border entry per chunk
    return (size_t)split_chunks(R, wide) * (2 * (size_t)th * wide * sizeof(float) + sizeof(int4));
}

int gemm_dw_split(const void *dy, const void *x, const void *m_sizes, int ms_i64, void *dw, int64_t R, int N, int K,
                  int E, int out_dtype, float alpha, void *workspace, size_t ws_bytes, hipStream_t stream) {
    if (!split_shape_ok(R, N, K, E)) return MFL_ERR_UNSUPPORTED;
    if (out_dtype != MFL_BF16 && out_dtype != MFL_F32) return MFL_ERR_UNSUPPORTED;
    if (!aligned(dy, 16) || !aligned(x, 16) || !aligned(dw, 16) || !aligned(workspace, 16)) return MFL_ERR_ALIGN;
    if (!workspace || ws_bytes < gemm_dw_split_workspace(R, N, K, E)) return MFL_ERR_WORKSPACE;
    const bool thin_n = split_thin(N);
    const int wide = thin_n ? K : N, th = thin_n ? N : K;
    const bf16_t *thin_p = (const bf16_t *)(thin_n ? dy : x), *wide_p = (const bf16_t *)(thin_n ? x : dy);
    const int chunks = split_chunks(R, wide);
    float *partial = (float *)workspace;
#define MFL_SPLIT(TH_, TN_)                                                                                          \
    (out_dtype == MFL_BF16 ? launch_split<TH_, TN_, bf16_t>(thin_p, wide_p, m_sizes, ms_i64, (bf16_t *)dw, partial, R,  \
                                                           wide, E, chunks, alpha, stream)                            \
                           : launch_split<TH_, TN_, float>(thin_p, wide_p, m_sizes, ms_i64, (float *)dw, partial, R,   \
                                                          wide, E, chunks, alpha, stream))
    if (thin_n)
        return th == 8 ? MFL_SPLIT(8, true) : th == 16 ? MFL_SPLIT(16, true) : th == 32 ? MFL_SPLIT(32, true) : MFL_SPLIT(64, true);
    return th == 8 ? MFL_SPLIT(8, false) : th == 16 ? MFL_SPLIT(16, false) : th == 32 ? MFL_SPLIT(32, false) : MFL_SPLIT(64, false);
#undef MFL_SPLIT
}

}  // namespace mfl
