// Building blocks shared by the MFMA block-product kernels (gfx950, wave64).
//
// One wavefront computes one 32 x 32 output block with v_mfma_f32_32x32x2_f32.  Lane l feeds
// A[i = l % 32][k] and B[k][j = l % 32]; inside a 32-wide k chunk, MFMA step s pairs k = s
// (lanes 0-31) with k = 16 + s (lanes 32-63), so a row-contiguous operand is a run of 16
// consecutive values per lane.  Accumulator register r of lane l is output element
// (row 8*(r/4) + 4*(l/32) + r%4, column l % 32).
#pragma once

#include <stdint.h>

#include <type_traits>

#include "sswin_common.hpp"

namespace sswin {

typedef float f32x4_u __attribute__((ext_vector_type(4), aligned(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// 16 consecutive values of one operand row, zero beyond `valid` (0..16).
template <typename T>
__device__ __forceinline__ void load_run16(const T* __restrict__ p, int valid, float (&x)[16]) {
    if (valid >= 16) {
        if (std::is_same<T, float>::value) {
            const f32x4_u* q = reinterpret_cast<const f32x4_u*>(p);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const f32x4_u t = q[v];
                x[4 * v] = t.x; x[4 * v + 1] = t.y; x[4 * v + 2] = t.z; x[4 * v + 3] = t.w;
            }
        } else {
#pragma unroll
            for (int s = 0; s < 16; ++s) x[s] = to_acc(p[s]);
        }
    } else if (valid == 8 && std::is_same<T, float>::value) {   // half of a 16-channel reduction
        const f32x4_u* q = reinterpret_cast<const f32x4_u*>(p);
#pragma unroll
        for (int v = 0; v < 2; ++v) {
            const f32x4_u t = q[v];
            x[4 * v] = t.x; x[4 * v + 1] = t.y; x[4 * v + 2] = t.z; x[4 * v + 3] = t.w;
        }
#pragma unroll
        for (int s = 8; s < 16; ++s) x[s] = 0.f;
    } else {
#pragma unroll
        for (int s = 0; s < 16; ++s) x[s] = s < valid ? to_acc(p[s]) : 0.f;
    }
}

// 16 consecutive values, all valid
template <typename T>
__device__ __forceinline__ void load_run16_full(const T* __restrict__ p, float (&x)[16]) {
    if (std::is_same<T, float>::value) {
        const f32x4_u* q = reinterpret_cast<const f32x4_u*>(p);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const f32x4_u t = q[v];
            x[4 * v] = t.x; x[4 * v + 1] = t.y; x[4 * v + 2] = t.z; x[4 * v + 3] = t.w;
        }
    } else {
#pragma unroll
        for (int s = 0; s < 16; ++s) x[s] = to_acc(p[s]);
    }
}

// Workgroups that share the 32 x 32 blocks of a workgroup's groups (the y extent of a block-product launch), from the
// mean group size.  A workgroup deals the blocks of `groups_per_wg` consecutive groups to its wavefronts, which take
// them one after the other, so windows of many blocks (7^3 positions: up to 64 blocks per group) would leave a few
// workgroups running long after the rest.  About 2.5 blocks per workgroup and slice measured best on windows of 5^3
// (30 tokens a group on average), 7^3 (60) and dense 5^3 windows (110).  square: the blocks tile a [c x c] result,
// otherwise a [c x C] one.
inline unsigned block_task_slices(double mean_c, int C, bool square, int groups_per_wg) {
    if (!(mean_c > 0)) return 1;
    const double nb = mean_c / 32.0 + 0.5;                              // 32-wide blocks along a side of c tokens
    const double per_group = square ? nb * nb : nb * (double)((C + 31) / 32);
    const int y = (int)(groups_per_wg * per_group / 2.5 + 0.5);
    return (unsigned)(y < 1 ? 1 : (y > 8 ? 8 : y));
}

// ---- blocks addressed through buffer descriptors ----
// A descriptor of exactly a block's size (base and size are scalars) lets the memory pipeline do the bounds checks: a
// lane whose row, column or reduction index lies outside the block forms the offset BUF_OUTSIDE, loads zero and has
// its store dropped, so ragged blocks need no clamp, select or branch, and an access costs one vector add for its
// offset.  Sizes stay at or below 2^31 bytes so that BUF_OUTSIDE plus any offset inside the block is still outside.
typedef uint32_t u32x4_b __attribute__((ext_vector_type(4)));
constexpr uint32_t BUF_OUTSIDE = 0x80000000u;

template <typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buf_of(const T* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(base), 0, (int)bytes, 0x00020000);
}
// one value of a float, half or bfloat16 array at byte offset off
template <typename T>
__device__ __forceinline__ float buf_load1(const __amdgpu_buffer_rsrc_t& r, uint32_t off) {
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0));
    } else {
        const uint16_t u = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0);
        return to_acc(__builtin_bit_cast(T, u));
    }
}
// N consecutive values (8 or 16) from byte offset off, all inside or all outside the buffer, in 16-byte loads
template <typename T, int N>
__device__ __forceinline__ void buf_load_run(const __amdgpu_buffer_rsrc_t& r, uint32_t off, float (&x)[16]) {
    constexpr int PER = 16 / (int)sizeof(T);                 // values per load
#pragma unroll
    for (int v = 0; v < N / PER; ++v) {
        const u32x4_b t = __builtin_amdgcn_raw_buffer_load_b128(r, off + 16u * v, 0, 0);
        const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if constexpr (sizeof(T) == 4) {
                x[4 * v + e] = __builtin_bit_cast(float, w[e]);
            } else {
                const uint16_t lo = (uint16_t)(w[e] & 0xffffu), hi = (uint16_t)(w[e] >> 16);
                x[8 * v + 2 * e] = to_acc(__builtin_bit_cast(T, lo));
                x[8 * v + 2 * e + 1] = to_acc(__builtin_bit_cast(T, hi));
            }
        }
    }
}
template <typename T>
__device__ __forceinline__ void buf_store1(const __amdgpu_buffer_rsrc_t& r, uint32_t off, float v) {
    if constexpr (sizeof(T) == 4) {
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), r, off, 0, 0);
    } else {
        const T t = from_acc<T>(v);
        __builtin_amdgcn_raw_buffer_store_b16((short)__builtin_bit_cast(uint16_t, t), r, off, 0, 0);
    }
}

__device__ __forceinline__ int clamp16(int v) { return v < 0 ? 0 : (v > 16 ? 16 : v); }

__device__ __forceinline__ int acc_row(int r, int half) { return 8 * (r >> 2) + 4 * half + (r & 3); }

}  // namespace sswin
