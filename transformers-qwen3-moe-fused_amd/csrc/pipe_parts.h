// Building blocks shared by the pipelined bf16 grouped-GEMM kernels (gemm_bf16_pipe.hip, gemm_bf16_wide.hip):
// the direct global -> LDS copy, the XOR-swizzled stage layouts, the per-lane source offsets of the copies, the
// per-lane LDS offsets of the MFMA fragment reads, and the cut of an expert's rows into tiles.
// Everything sits in an anonymous namespace: each translation unit gets its own copy.
#pragma once
#include <type_traits>

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

// One wave-wide copy of 16 bytes per lane from global memory to 1 KiB of consecutive LDS.
// ASM: the instruction is written out by hand.  The compiler orders every transposing LDS read
// (ds_read_b64_tr_b16) behind all copies it knows to be in flight, i.e. it waits for the stage it
// has just requested before it reads the current one; a copy it does not see leaves the waiting
// to the kernel's own s_waitcnt vmcnt.  M0 holds the LDS address of the wave's 1 KiB; nothing else
// in the kernels built with ASM uses M0 (no builtin copy, no message, no indexed move), so it is
// set in the same statement as the copy and not saved.
template <int POLICY, bool ASM>
__device__ __forceinline__ void copy_to_lds(const unsigned char *src, unsigned char *dst) {
    if constexpr (ASM) {
        const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_void_ptr)dst;
        if constexpr (POLICY == 2)
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt"
                         :
                         : "v"(src), "s"(lds_addr)
                         : "memory");
        else
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                         :
                         : "v"(src), "s"(lds_addr)
                         : "memory");
    } else {
        __builtin_amdgcn_global_load_lds((global_void_ptr)src, (lds_void_ptr)dst, 16, 0, POLICY);
    }
}

template <int BI, int BK, bool RC>
struct Stage {
    static constexpr int kRowBytes = RC ? BK * 2 : BI * 2;
    static constexpr int kBytes = BI * BK * 2;
    static constexpr int kWaveLoads = kBytes / 1024;       // 1 KiB per wave-wide copy
    static constexpr int kChunksPerRow = kRowBytes / 16;
    static constexpr int kRowsPer256 = kRowBytes >= 256 ? 1 : 256 / kRowBytes;
    // RS rows: a transposing read touches 4 consecutive rows, and the two 16-lane groups that the
    // LDS serves together read 32 bytes each of every row, 32 bytes apart.  Rows whose length is
    // a multiple of 256 bytes start in the same bank: they are spread 64 bytes apart (4 rows x 64
    // bytes = all 64 banks).  Other row lengths (384 bytes) already differ by 128 bytes from row to
    // row, and a 32-byte spread keeps the XOR inside the row.
    static constexpr int kRsShift = kChunksPerRow % 16 == 0 ? 2 : 1;
    static_assert(kBytes % 1024 == 0 && kChunksPerRow % (RC ? 4 : 8) == 0,
                  "stage must be whole copies; rows of 64 bytes or more along the reduction, of whole 128 B across it");

    // stage row and physical chunk that lane `lane` of wave-load `load` fills (a copy covers 64
    // consecutive chunks of the stage, whatever the row length)
    __device__ static __forceinline__ int row_of(int load, int lane) { return (load * 64 + lane) / kChunksPerRow; }
    __device__ static __forceinline__ int phys_of(int load, int lane) { return (load * 64 + lane) % kChunksPerRow; }

    // physical 16-byte chunk of logical chunk c in row `row`
    __device__ static __forceinline__ int swz(int row, int c) {
        if (RC) return c ^ ((row / kRowsPer256) % kChunksPerRow);
        return c ^ ((row & 3) << kRsShift);
    }
};

// Per-lane byte offset (relative to the operand's tile origin in global memory at reduction
// step 0) of the 16 bytes this lane copies in wave-load `load`.  `i_lim` is the number of valid
// rows (RC) or columns (RS) from the tile origin; lanes outside are clamped inside.
template <int BI, int BK, bool RC>
__device__ __forceinline__ int64_t lane_src_offset(int load, int lane, int64_t ld, int i_lim) {
    typedef Stage<BI, BK, RC> S;
    const int row = S::row_of(load, lane);
    const int phys = S::phys_of(load, lane);
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

// Per-lane LDS byte offsets (within an operand's part of a stage) of the MFMA fragment reads of
// the wave's blocks: block t of the wave starts at row first + t * stride.
// RC: one offset per 16-wide reduction sub-step (the block adds a constant).
// RS: one offset per block (the sub-step adds a constant).
template <int BI, int BK, bool RC, int TB>
struct FragOffsets {
    static constexpr int kCount = RC ? BK / 16 : TB;
    int off[kCount];
    int block_bytes;  // RC only: byte distance between consecutive blocks of the wave

    __device__ __forceinline__ void init(int first, int stride, int lane) {
        typedef Stage<BI, BK, RC> S;
        block_bytes = stride * S::kRowBytes;
        if (RC) {
            const int row = first + (lane & 31);
#pragma unroll
            for (int ks = 0; ks < kCount; ++ks)
                off[ks] = row * S::kRowBytes + S::swz(row, ks * 2 + (lane >> 5)) * 16;
        } else {
            const int g = lane >> 4, il = lane & 15;
            const int r = 8 * (g >> 1) + (il >> 2);
#pragma unroll
            for (int t = 0; t < kCount; ++t) {
                const int i = first + t * stride + 16 * (g & 1) + 4 * (il & 3);
                off[t] = r * S::kRowBytes + S::swz(r, i >> 3) * 16 + (i & 7) * 2;
            }
        }
    }

    // fragment of the wave's block t at sub-step ks; `base` points at the operand's part of the stage
    __device__ __forceinline__ bf16x8 load(const unsigned char *base, int t, int ks) const {
        typedef Stage<BI, BK, RC> S;
        if (RC) {
            return *(const bf16x8 *)(base + off[ks] + t * block_bytes);
        } else {
            const unsigned char *p = base + off[t] + ks * 16 * S::kRowBytes;
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

// ---- tile enumeration of the row-grouped products -------------------------------------------

// An expert with m rows is cut into ceil(m / BM) parts of equal height (a multiple of 32).
template <int BM>
__device__ __forceinline__ int m_tiles_of(int m) {
    return ceil_div(m, BM);
}
template <int BM>
__device__ __forceinline__ int tile_rows_of(int m) {
    const int t = ceil_div(m, BM);
    return t == 0 ? 0 : ceil_div(ceil_div(m, t), 32) * 32;
}

constexpr int kMaxTableExperts = 512;  // per-expert prefix tables live in LDS

template <int V>
using IC = std::integral_constant<int, V>;

// Source of the 16-byte chunks that lie past the end of a reduction-contiguous row in the last,
// partial reduction step (K not a multiple of BK).
__device__ uint4_t g_zero_chunk = {0u, 0u, 0u, 0u};

}  // namespace

}  // namespace mfl
