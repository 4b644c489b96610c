// Shared host/device helpers of the sswin3d library (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/sswin3d.h"

namespace sswin {

// ------------------------------------------------------------------------------------------
// host: error reporting
// ------------------------------------------------------------------------------------------
char* error_buffer();                       // thread-local, 512 bytes
int fail(const char* fmt, ...);             // formats into error_buffer(), returns 1

#define SSWIN_CHECK(cond, ...)                       \
    do {                                             \
        if (!(cond)) return ::sswin::fail(__VA_ARGS__); \
    } while (0)

#define SSWIN_HIP(expr)                                                              \
    do {                                                                             \
        hipError_t _e = (expr);                                                      \
        if (_e != hipSuccess)                                                        \
            return ::sswin::fail("%s failed: %s", #expr, hipGetErrorString(_e));     \
    } while (0)

inline int launch_ok(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("launch of %s failed: %s", what, hipGetErrorString(e));
    return 0;
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Carves aligned pieces out of a caller-provided workspace.
struct Carver {
    char* base;
    size_t size, used = 0;
    Carver(void* p, size_t n) : base(static_cast<char*>(p)), size(n) {}
    template <typename T>
    T* take(size_t count) {
        used = align_up(used, 256);
        T* p = reinterpret_cast<T*>(base + used);
        used += count * sizeof(T);
        return p;
    }
    bool ok() const { return used <= size; }
};

// ------------------------------------------------------------------------------------------
// device: wave64 cross-lane primitives.  Reductions inside a 16-lane DPP row use DPP
// modifiers (no LDS traffic); the two cross-row steps use ds_bpermute via __shfl_xor.
// ------------------------------------------------------------------------------------------
// (the controls used here give every lane a source lane, so no lane keeps an old value: the move form without one
// lets the compiler fold the cross-lane read into the instruction that uses it)
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
    return __builtin_amdgcn_mov_dpp(v, CTRL, 0xf, 0xf, true);
}

// DPP controls: quad_perm[1,0,3,2]=0xB1, quad_perm[2,3,0,1]=0x4E, row_half_mirror=0x141,
// row_mirror=0x140.  After the four steps every lane of a 16-lane row holds the row total;
// the operands of each step are exchanged symmetrically, so all lanes agree bit for bit.
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_f32<0xB1>(v);
    v += dpp_f32<0x4E>(v);
    v += dpp_f32<0x141>(v);
    v += dpp_f32<0x140>(v);
    return v;
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_f32<0xB1>(v));
    v = fmaxf(v, dpp_f32<0x4E>(v));
    v = fmaxf(v, dpp_f32<0x141>(v));
    v = fmaxf(v, dpp_f32<0x140>(v));
    return v;
}
__device__ __forceinline__ double row16_sum(double v) {
    // 64-bit values have no single DPP move; shuffle the halves.
    for (int m = 1; m < 16; m <<= 1) v += __shfl_xor(v, m, 64);
    return v;
}
__device__ __forceinline__ double row16_max(double v) {
    for (int m = 1; m < 16; m <<= 1) v = fmax(v, __shfl_xor(v, m, 64));
    return v;
}

__device__ __forceinline__ int row16_sum_i32(int v) {
    v += dpp_i32<0xB1>(v);
    v += dpp_i32<0x4E>(v);
    v += dpp_i32<0x141>(v);
    v += dpp_i32<0x140>(v);
    return v;
}

__device__ __forceinline__ int wave_sum_i32(int v) {
    v += dpp_i32<0xB1>(v);
    v += dpp_i32<0x4E>(v);
    v += dpp_i32<0x141>(v);
    v += dpp_i32<0x140>(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
__device__ __forceinline__ int wave_max_i32(int v) {
    v = max(v, dpp_i32<0xB1>(v));
    v = max(v, dpp_i32<0x4E>(v));
    v = max(v, dpp_i32<0x141>(v));
    v = max(v, dpp_i32<0x140>(v));
    v = max(v, __shfl_xor(v, 16, 64));
    v = max(v, __shfl_xor(v, 32, 64));
    return v;
}

// value type traits: storage type -> accumulate type
template <typename T> struct acc_of { using type = float; };
template <> struct acc_of<double> { using type = double; };

__device__ __forceinline__ float to_acc(float v) { return v; }
__device__ __forceinline__ double to_acc(double v) { return v; }
__device__ __forceinline__ float to_acc(__half v) { return __half2float(v); }
__device__ __forceinline__ float to_acc(__hip_bfloat16 v) { return __bfloat162float(v); }

template <typename T> __device__ __forceinline__ T from_acc(typename acc_of<T>::type v);
template <> __device__ __forceinline__ float from_acc<float>(float v) { return v; }
template <> __device__ __forceinline__ double from_acc<double>(double v) { return v; }
template <> __device__ __forceinline__ __half from_acc<__half>(float v) { return __float2half(v); }
template <> __device__ __forceinline__ __hip_bfloat16 from_acc<__hip_bfloat16>(float v) {
    return __float2bfloat16(v);
}

// Zeros by a kernel instead of hipMemsetAsync: callers may capture these entry points into a HIP graph, and memset
// nodes have given wrong results on replays of a captured graph.
template <typename T>
__global__ __launch_bounds__(256) void zero_fill_kernel(T* __restrict__ p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) p[i] = T(0);
}
template <typename T>
inline void zero_fill(T* p, int64_t n, hipStream_t s) {
    if (n <= 0) return;
    const unsigned blocks = (unsigned)((n + 255) / 256 < 1024 ? (n + 255) / 256 : 1024);
    hipLaunchKernelGGL((zero_fill_kernel<T>), dim3(blocks), dim3(256), 0, s, p, n);
}

}  // namespace sswin
