// Shared device/host helpers for the gfx950 moe_fused_linear library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/moe_fused_linear.h"

namespace mfl {

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(2))) float floatx2;
typedef __attribute__((ext_vector_type(16))) float floatx16;
typedef __attribute__((ext_vector_type(4))) uint32_t uint4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t uint2_t;

constexpr int kWave = 64;

template <typename T>
__device__ __forceinline__ float to_f32(T v) {
    return (float)v;
}
template <typename T>
__device__ __forceinline__ T from_f32(float v) {
    return (T)v;  // bf16/f16: one round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950)
}

// 1 / (1 + 2^(-x log2 e)) on the hardware exp2 and reciprocal instructions (about an ulp of
// error each, far below the bf16 rounding that follows).  The library's expf and an IEEE
// division cost about ten times as many instructions, which made the SiLU as expensive as its
// memory traffic.  Large |x|: 2^t overflows to +inf (sigmoid 0) or flushes to 0 (sigmoid 1).
__device__ __forceinline__ float sigmoid_f32(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504088896341f));
}

// h = silu(e) * g with the rounding chain of the reference (qwen3_moe_fused/kernels/silu_mul.py:34-39):
// silu in fp32, rounded to the storage type, then the product in the storage type.
template <typename T>
__device__ __forceinline__ T silu_fwd_one(T e, T g) {
    const float e32 = to_f32(e);
    if (sizeof(T) == 4) return from_f32<T>((e32 * sigmoid_f32(e32)) * to_f32(g));
    const T f = from_f32<T>(e32 * sigmoid_f32(e32));
    return from_f32<T>(to_f32(f) * to_f32(g));
}

// Backward of h = silu(e) * g for one element: h again, de and dg from dh (the rounding chain of the reference's
// kernel, qwen3_moe_fused/kernels/silu_mul.py:84-111).
template <typename T>
__device__ __forceinline__ void silu_bwd_one(T dh, T e, T g, T &h, T &de, T &dg) {
    const float e32 = to_f32(e), g32 = to_f32(g), dh32 = to_f32(dh);
    const float se = sigmoid_f32(e32);
    const float ese = e32 * se;
    const float f = to_f32(from_f32<T>(ese));
    const float df = to_f32(from_f32<T>(dh32 * g32));
    h = from_f32<T>(f * g32);
    dg = from_f32<T>(f * dh32);
    de = from_f32<T>(df * se * (1.0f + e32 - ese));
}

__device__ __forceinline__ int load_msize(const void *m_sizes, int is_i64, int e) {
    return is_i64 ? (int)((const int64_t *)m_sizes)[e] : ((const int32_t *)m_sizes)[e];
}

__host__ __device__ constexpr int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Inclusive prefix sum over the 64 lanes of a wave (all lanes active) on data-parallel-primitive
// moves: a Kogge-Stone scan inside each row of 16 lanes (shifts by 1, 2, 4, 8; lanes without a
// source add 0), then the last lane of rows 0 and 2 is added to rows 1 and 3, and lane 31 to rows
// 2 and 3.  Six vector-ALU instructions instead of six trips through the LDS crossbar.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_add_step(int x) {
    return x + __builtin_amdgcn_update_dpp(0, x, CTRL, ROW_MASK, 0xf, true);
}
__device__ __forceinline__ int wave_inclusive_scan(int x) {
    x = dpp_add_step<0x111, 0xf>(x);  // row_shr 1
    x = dpp_add_step<0x112, 0xf>(x);  // row_shr 2
    x = dpp_add_step<0x114, 0xf>(x);  // row_shr 4
    x = dpp_add_step<0x118, 0xf>(x);  // row_shr 8
    x = dpp_add_step<0x142, 0xa>(x);  // row_bcast 15 into rows 1 and 3
    x = dpp_add_step<0x143, 0xc>(x);  // row_bcast 31 into rows 2 and 3
    return x;
}
// value of lane 63, in every lane
__device__ __forceinline__ int wave_last(int x) { return __builtin_amdgcn_readlane(x, 63); }

inline size_t dtype_size(int dt) { return dt == MFL_F32 ? 4 : 2; }
inline bool dtype_ok(int dt) { return dt == MFL_BF16 || dt == MFL_F32 || dt == MFL_F16; }
inline bool itype_ok(int it) { return it == MFL_I32 || it == MFL_I64; }
inline bool aligned(const void *p, size_t a) { return ((uintptr_t)p % a) == 0; }

inline int launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? MFL_OK : (int)e;
}

// Runs `f` (a per-device set-up call such as hipFuncSetAttribute) once for every device that a kernel
// is launched on; safe under concurrent first calls (f must be idempotent: two threads that meet in
// the first call on a device may both run it).
struct PerDeviceOnce {
    std::atomic<uint64_t> done{0};
    template <typename F>
    hipError_t run(F &&f) {
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        const uint64_t bit = 1ull << (dev & 63);
        if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
        e = f();
        if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
        return e;
    }
};

struct DeviceInfo {
    int cu_count;
    int xcd_count;
};
const DeviceInfo &device_info();

// dispatch helpers -----------------------------------------------------------------
#define MFL_DISPATCH_FLOAT(dt, T, ...)          \
    switch (dt) {                               \
        case MFL_BF16: {                        \
            typedef ::mfl::bf16_t T;            \
            __VA_ARGS__;                        \
        } break;                                \
        case MFL_F16: {                         \
            typedef ::mfl::f16_t T;             \
            __VA_ARGS__;                        \
        } break;                                \
        default: {                              \
            typedef float T;                    \
            __VA_ARGS__;                        \
        } break;                                \
    }

}  // namespace mfl
