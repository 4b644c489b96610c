// Index glue of the shifted-window stage on int32 voxel coordinates: what the reference does with a
// chain of small tensor operations per block (pad, roll, partition; a dense int8 mask volume cut into
// 27 regions; sparse_swin/swin3d_base.py:336-372, 416-452, 501-554) and with spconv's strided
// convolution between stages (:950-976), as single passes over the voxel list.
//
//   window_indices   (batch, d, h, w) -> (window slot, position inside the window) after the cyclic
//                    shift, one 16-byte load and one 8-byte store per voxel
//   shift_mask       region ids [windows, positions] of the shifted grid, computed from the position
//                    instead of 27 slice assignments and a permuted copy of a dense volume
//   pool_windows     rows of the voxels of a window, in (window, position) order, reduced to one row
//                    (mean, or sum of per-position weights applied outside); with windows of 2x2x2
//                    this is the floor(coord / 2) merge between stages.  The token plan supplies the
//                    order, so the sum runs in a fixed order without atomics.
#include <stdint.h>

#include "sswin_common.hpp"

namespace sswin {

struct Grid3 {
    int dim[3];     // padded extent
    int win[3];     // window extent
    int shift[3];   // cyclic shift (subtracted)
    int nwin[3];    // windows per axis
};

__global__ __launch_bounds__(256) void window_indices_kernel(const int4* __restrict__ coords, int64_t N, Grid3 g,
                                                             int2* __restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N) return;
    const int4 c = coords[i];                                // batch, d, h, w
    int z = c.y - g.shift[0], y = c.z - g.shift[1], x = c.w - g.shift[2];
    z += z < 0 ? g.dim[0] : 0;                               // 0 <= shift < extent and 0 <= coordinate < extent
    y += y < 0 ? g.dim[1] : 0;
    x += x < 0 ? g.dim[2] : 0;
    const int wz = z / g.win[0], wy = y / g.win[1], wx = x / g.win[2];
    const int pz = z - wz * g.win[0], py = y - wy * g.win[1], px = x - wx * g.win[2];
    int2 o;
    o.x = ((c.x * g.nwin[0] + wz) * g.nwin[1] + wy) * g.nwin[2] + wx;
    o.y = (pz * g.win[1] + py) * g.win[2] + px;
    out[i] = o;
}

// the three slices of the reference along one axis, later assignments winning:
// [0, D - ws) -> 0, [D - ws, D - s) -> 1, [D - s, D) -> 2; with s == 0 the last slice is the whole axis
__device__ __forceinline__ int axis_region(int v, int extent, int ws, int s) {
    if (s == 0) return 2;
    return v < extent - ws ? 0 : (v < extent - s ? 1 : 2);
}

// Region id of entry i = window * n + pos and of the three entries behind it.  The (window, position) pair is
// decomposed once per thread (five 32-bit divisions; the quotient i / n in 64 bits only when the array is
// that large) and then advanced by carries: position -> (pz, py, px), window -> (wz, wy, wx).
struct MaskCursor {
    int wz, wy, wx, pz, py, px;
};
__device__ __forceinline__ MaskCursor mask_cursor(const Grid3& g, int n, int64_t i, bool small) {
    uint32_t w, pos;
    if (small) {
        w = (uint32_t)i / (uint32_t)n;
        pos = (uint32_t)i - w * (uint32_t)n;
    } else {
        w = (uint32_t)(i / n);
        pos = (uint32_t)(i - (int64_t)w * n);
    }
    MaskCursor c;
    const uint32_t wyz = w / (uint32_t)g.nwin[2];
    c.wx = (int)(w - wyz * (uint32_t)g.nwin[2]);
    c.wz = (int)(wyz / (uint32_t)g.nwin[1]);
    c.wy = (int)(wyz - (uint32_t)c.wz * (uint32_t)g.nwin[1]);
    const uint32_t pzy = pos / (uint32_t)g.win[2];
    c.px = (int)(pos - pzy * (uint32_t)g.win[2]);
    c.pz = (int)(pzy / (uint32_t)g.win[1]);
    c.py = (int)(pzy - (uint32_t)c.pz * (uint32_t)g.win[1]);
    return c;
}
__device__ __forceinline__ int mask_region(const Grid3& g, const MaskCursor& c) {
    const int rz = axis_region(c.wz * g.win[0] + c.pz, g.dim[0], g.win[0], g.shift[0]);
    const int ry = axis_region(c.wy * g.win[1] + c.py, g.dim[1], g.win[1], g.shift[1]);
    const int rx = axis_region(c.wx * g.win[2] + c.px, g.dim[2], g.win[2], g.shift[2]);
    return 9 * rz + 3 * ry + rx;
}
__device__ __forceinline__ void mask_advance(const Grid3& g, MaskCursor& c) {
    if (++c.px < g.win[2]) return;
    c.px = 0;
    if (++c.py < g.win[1]) return;
    c.py = 0;
    if (++c.pz < g.win[0]) return;
    c.pz = 0;                                                // next window
    if (++c.wx < g.nwin[2]) return;
    c.wx = 0;
    if (++c.wy < g.nwin[1]) return;
    c.wy = 0;
    ++c.wz;
}

// four consecutive entries per thread, one 32-bit store (the array is 4-byte aligned); the last
// thread finishes a total that is not a multiple of four byte by byte
__global__ __launch_bounds__(256) void shift_mask_kernel(Grid3 g, int n, int64_t total, int8_t* __restrict__ mask) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= total) return;
    MaskCursor c = mask_cursor(g, n, i, total < ((int64_t)1 << 31));
    if (i + 4 <= total) {
        uint32_t v = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            v |= (uint32_t)mask_region(g, c) << (8 * k);
            mask_advance(g, c);
        }
        *reinterpret_cast<uint32_t*>(mask + i) = v;
    } else {
        for (int64_t k = i; k < total; ++k) {
            mask[k] = (int8_t)mask_region(g, c);
            mask_advance(g, c);
        }
    }
}

// ------------------------------------------------------------------------------------------
// pooling over the tokens of a window (token plan with one head: group = non-empty window)
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ void unpack4(const float4& v, float (&x)[4]) { x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w; }
__device__ __forceinline__ float4 pack4(const float (&x)[4], float) { return float4{x[0], x[1], x[2], x[3]}; }
template <typename T>
__device__ __forceinline__ void unpack4_16(const uint2& v, float (&x)[4]) {
    const T* p = reinterpret_cast<const T*>(&v);
#pragma unroll
    for (int k = 0; k < 4; ++k) x[k] = to_acc(p[k]);
}
template <typename T>
__device__ __forceinline__ uint2 pack4_16(const float (&x)[4]) {
    uint2 v;
    T* p = reinterpret_cast<T*>(&v);
#pragma unroll
    for (int k = 0; k < 4; ++k) p[k] = from_acc<T>(x[k]);
    return v;
}
template <typename T>
__device__ __forceinline__ void load4(const T* p, float (&x)[4]);
template <> __device__ __forceinline__ void load4<float>(const float* p, float (&x)[4]) {
    unpack4(*reinterpret_cast<const float4*>(p), x);
}
template <typename T>
__device__ __forceinline__ void load4(const T* p, float (&x)[4]) { unpack4_16<T>(*reinterpret_cast<const uint2*>(p), x); }
template <typename T>
__device__ __forceinline__ void store4(T* p, const float (&x)[4]);
template <> __device__ __forceinline__ void store4<float>(float* p, const float (&x)[4]) {
    *reinterpret_cast<float4*>(p) = pack4(x, 0.f);
}
template <typename T>
__device__ __forceinline__ void store4(T* p, const float (&x)[4]) { *reinterpret_cast<uint2*>(p) = pack4_16<T>(x); }

// plan rows: c [g_cap], row_start [g_cap], (sq_start), window [g_cap]; tokens row 0: voxel of rank r
template <typename T>
__global__ __launch_bounds__(256) void pool_windows_kernel(const int32_t* __restrict__ plan, int64_t g_cap, int64_t M,
                                                           const int32_t* __restrict__ order, const T* __restrict__ x,
                                                           int64_t x_stride, int C4, int mean, T* __restrict__ out,
                                                           int64_t out_stride) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= M * C4) return;
    const int64_t m = i / C4;
    const int ch = (int)(i - m * C4) * 4;
    const int c = plan[m], first = plan[g_cap + m];
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < c; ++k) {                            // position order: a fixed order of summation
        float v[4];
        load4<T>(x + (int64_t)order[first + k] * x_stride + ch, v);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += v[e];
    }
    if (mean) {
        const float inv = 1.0f / (float)c;
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] *= inv;
    }
    store4<T>(out + m * out_stride + ch, acc);
}

// gradient of the pooling: every voxel of a window receives the window's row (divided by the count)
template <typename T>
__global__ __launch_bounds__(256) void pool_windows_grad_kernel(const int32_t* __restrict__ plan, int64_t g_cap, int64_t M,
                                                                const int32_t* __restrict__ order,
                                                                const T* __restrict__ g_out, int64_t g_stride, int C4,
                                                                int mean, T* __restrict__ g_x, int64_t x_stride) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= M * C4) return;
    const int64_t m = i / C4;
    const int ch = (int)(i - m * C4) * 4;
    const int c = plan[m], first = plan[g_cap + m];
    float v[4];
    load4<T>(g_out + m * g_stride + ch, v);
    if (mean) {
        const float inv = 1.0f / (float)c;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] *= inv;
    }
    for (int k = 0; k < c; ++k) store4<T>(g_x + (int64_t)order[first + k] * x_stride + ch, v);
}

// coordinates of the windows themselves: (batch, wz, wy, wx) of every non-empty window
__global__ __launch_bounds__(256) void window_coords_kernel(const int32_t* __restrict__ plan, int64_t g_cap, int64_t M,
                                                            Grid3 g, int4* __restrict__ out) {
    const int64_t m = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (m >= M) return;
    int w = plan[3 * g_cap + m];
    int4 o;
    o.w = w % g.nwin[2];
    w /= g.nwin[2];
    o.z = w % g.nwin[1];
    w /= g.nwin[1];
    o.y = w % g.nwin[0];
    o.x = w / g.nwin[0];
    out[m] = o;
}

static int make_grid(const char* who, const int32_t* dims, const int32_t* window, const int32_t* shift, Grid3* g) {
    SSWIN_CHECK(dims && window, "%s: null grid description", who);
    for (int a = 0; a < 3; ++a) {
        g->dim[a] = dims[a];
        g->win[a] = window[a];
        g->shift[a] = shift ? shift[a] : 0;
        SSWIN_CHECK(window[a] > 0 && dims[a] > 0 && dims[a] % window[a] == 0,
                    "%s: extent %d of axis %d is not a positive multiple of the window %d", who, dims[a], a, window[a]);
        SSWIN_CHECK(g->shift[a] >= 0 && g->shift[a] < dims[a], "%s: shift %d of axis %d is outside [0, extent)", who,
                    g->shift[a], a);
        g->nwin[a] = dims[a] / window[a];
    }
    return 0;
}

template <typename T>
static void launch_pool(const int32_t* plan, int64_t g_cap, int64_t M, const int32_t* order, const void* x,
                        int64_t x_stride, int C, int mean, void* out, int64_t out_stride, int backward,
                        hipStream_t s) {
    const int64_t total = M * (C / 4);
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (!backward)
        hipLaunchKernelGGL((pool_windows_kernel<T>), dim3(blocks), dim3(256), 0, s, plan, g_cap, M, order,
                           static_cast<const T*>(x), x_stride, C / 4, mean, static_cast<T*>(out), out_stride);
    else
        hipLaunchKernelGGL((pool_windows_grad_kernel<T>), dim3(blocks), dim3(256), 0, s, plan, g_cap, M, order,
                           static_cast<const T*>(x), x_stride, C / 4, mean, static_cast<T*>(out), out_stride);
}

}  // namespace sswin

using namespace sswin;

extern "C" {

int sswin_window_indices(const int32_t* coords, int64_t N, int batch_size, const int32_t* dims, const int32_t* window,
                         const int32_t* shift, int32_t* indices, void* stream) {
    Grid3 g;
    if (make_grid("window_indices", dims, window, shift, &g)) return 1;
    SSWIN_CHECK(N >= 0 && batch_size > 0, "window_indices: bad sizes");
    const int64_t slots = (int64_t)batch_size * g.nwin[0] * g.nwin[1] * g.nwin[2];
    SSWIN_CHECK(slots < ((int64_t)1 << 31) && (int64_t)window[0] * window[1] * window[2] < ((int64_t)1 << 31),
                "window_indices: %lld window slots do not fit int32", (long long)slots);
    if (N == 0) return 0;
    SSWIN_CHECK(coords && indices, "window_indices: null pointer");
    SSWIN_CHECK(((uintptr_t)coords % 16) == 0 && ((uintptr_t)indices % 8) == 0, "window_indices: misaligned pointers");
    hipLaunchKernelGGL(window_indices_kernel, dim3((unsigned)((N + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), reinterpret_cast<const int4*>(coords), N, g,
                       reinterpret_cast<int2*>(indices));
    return launch_ok("window_indices");
}

int sswin_shift_mask(const int32_t* dims, const int32_t* window, const int32_t* shift, int8_t* mask, void* stream) {
    Grid3 g;
    if (make_grid("shift_mask", dims, window, shift, &g)) return 1;
    const int64_t n = (int64_t)window[0] * window[1] * window[2];
    const int64_t total = n * g.nwin[0] * g.nwin[1] * g.nwin[2];
    SSWIN_CHECK(n < (1 << 24) && total < ((int64_t)1 << 40), "shift_mask: grid too large");
    SSWIN_CHECK(mask && ((uintptr_t)mask % 4) == 0, "shift_mask: null or misaligned pointer");
    hipLaunchKernelGGL(shift_mask_kernel, dim3((unsigned)((total + 1023) / 1024)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), g, (int)n, total, mask);
    return launch_ok("shift_mask");
}

int sswin_window_coords(const int32_t* plan, int64_t g_cap, int64_t M, const int32_t* dims, const int32_t* window,
                        int32_t* coords_out, void* stream) {
    Grid3 g;
    if (make_grid("window_coords", dims, window, nullptr, &g)) return 1;
    SSWIN_CHECK(M >= 0 && M <= g_cap, "window_coords: %lld windows, capacity %lld", (long long)M, (long long)g_cap);
    if (M == 0) return 0;
    SSWIN_CHECK(plan && coords_out && ((uintptr_t)coords_out % 16) == 0, "window_coords: null or misaligned pointer");
    hipLaunchKernelGGL(window_coords_kernel, dim3((unsigned)((M + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), plan, g_cap, M, g, reinterpret_cast<int4*>(coords_out));
    return launch_ok("window_coords");
}

int sswin_pool_windows(int dtype, int backward, int mean, const int32_t* plan, int64_t g_cap, int64_t M,
                       const int32_t* tokens, int64_t N, const void* src, int64_t src_stride, int C, void* dst,
                       int64_t dst_stride, void* stream) {
    SSWIN_CHECK(M >= 0 && M <= g_cap && N >= 0, "pool_windows: bad sizes");
    SSWIN_CHECK(C > 0 && C % 4 == 0, "pool_windows: %d channels are not a multiple of 4", C);
    SSWIN_CHECK(dtype == SSWIN_F32 || dtype == SSWIN_F16 || dtype == SSWIN_BF16, "pool_windows: unsupported dtype %d", dtype);
    if (M == 0 || N == 0) return 0;
    SSWIN_CHECK(plan && tokens && src && dst, "pool_windows: null pointer");
    const int64_t esz = dtype == SSWIN_F32 ? 4 : 2;
    SSWIN_CHECK(src_stride >= C && dst_stride >= C && (src_stride * esz) % (4 * esz) == 0 &&
                    (dst_stride * esz) % (4 * esz) == 0 && ((uintptr_t)src % (4 * esz)) == 0 &&
                    ((uintptr_t)dst % (4 * esz)) == 0,
                "pool_windows: rows must be aligned to four channels");
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case SSWIN_F32: launch_pool<float>(plan, g_cap, M, tokens, src, src_stride, C, mean, dst, dst_stride, backward, s); break;
        case SSWIN_F16: launch_pool<__half>(plan, g_cap, M, tokens, src, src_stride, C, mean, dst, dst_stride, backward, s); break;
        default: launch_pool<__hip_bfloat16>(plan, g_cap, M, tokens, src, src_stride, C, mean, dst, dst_stride, backward, s); break;
    }
    return launch_ok("pool_windows");
}

}  // extern "C"
