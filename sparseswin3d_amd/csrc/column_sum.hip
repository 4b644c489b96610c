// Column sums of a tall [N, P] matrix (fp32, fp16 or bf16; sums in fp32): the bias gradient of the
// qkv / proj projections (nn.Linear of sparse_swin/swin3d_base.py:606-610 with bias; autograd
// computes it as grad_out.sum(0)).  Two stages with a fixed summation order: workgroup (w, y) adds
// the rows w, w + W, ... of the columns of chunk y (at most 1024 columns per chunk, four columns
// per thread, one row per chunk_width/4 threads), the second stage adds the W partial rows per
// column.
#include <algorithm>

#include "sswin_common.hpp"

namespace sswin {

typedef float cs_f4 __attribute__((ext_vector_type(4)));

constexpr int CS_THREADS = 256;

template <typename T>
__device__ __forceinline__ cs_f4 load_cols4(const T* p);
template <>
__device__ __forceinline__ cs_f4 load_cols4<float>(const float* p) { return *reinterpret_cast<const cs_f4*>(p); }
template <typename T>
__device__ __forceinline__ cs_f4 load_cols4(const T* p) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    const T* e = reinterpret_cast<const T*>(&v);
    return cs_f4{to_acc(e[0]), to_acc(e[1]), to_acc(e[2]), to_acc(e[3])};
}

// threads are laid out as (row lane, group of four columns): rows_per_pass = CS_THREADS / (chunk/4)
template <typename T>
__global__ __launch_bounds__(CS_THREADS) void column_sum_partial_kernel(const T* __restrict__ x, int64_t N, int P,
                                                                        int chunk, float* __restrict__ partial) {
    __shared__ cs_f4 acc_s[CS_THREADS];
    const int col0 = blockIdx.y * chunk;
    const int width = P - col0 < chunk ? P - col0 : chunk;    // columns of this chunk
    const int c4n = chunk >> 2;                               // column groups per row lane
    const int rpp = CS_THREADS / c4n;                         // rows per pass
    const int rl = threadIdx.x / c4n, c4 = threadIdx.x - rl * c4n;
    cs_f4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = a0, a2 = a0, a3 = a0;
    if (rl < rpp && 4 * c4 < width) {
        const int64_t stride = (int64_t)gridDim.x * rpp;
        int64_t r = (int64_t)blockIdx.x * rpp + rl;
        const T* p = x + col0 + 4 * c4;
        // four independent chains keep four loads in flight
        for (; r + 3 * stride < N; r += 4 * stride) {
            a0 += load_cols4<T>(p + r * P);
            a1 += load_cols4<T>(p + (r + stride) * P);
            a2 += load_cols4<T>(p + (r + 2 * stride) * P);
            a3 += load_cols4<T>(p + (r + 3 * stride) * P);
        }
        for (; r < N; r += stride) a0 += load_cols4<T>(p + r * P);
    }
    acc_s[threadIdx.x] = (a0 + a1) + (a2 + a3);
    __syncthreads();
    if (threadIdx.x < c4n && 4 * threadIdx.x < width) {
        cs_f4 t = acc_s[threadIdx.x];
        for (int k = 1; k < rpp; ++k) t += acc_s[k * c4n + threadIdx.x];
        *reinterpret_cast<cs_f4*>(partial + (int64_t)blockIdx.x * P + col0 + 4 * threadIdx.x) = t;
    }
}

// out[c] = sum over parts of partial[part][c]: 64 chains per column (four loads in flight each),
// then the 64 chain sums are added in chain order
__global__ __launch_bounds__(1024) void column_sum_final_kernel(const float* __restrict__ partial, int parts, int P,
                                                                float* __restrict__ out) {
    __shared__ float part[64][17];
    const int cl = threadIdx.x & 15, q = threadIdx.x >> 4;
    const int c = blockIdx.x * 16 + cl;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (c < P) {
        const float* src = partial + c;
        int k = q;
        for (; k + 192 < parts; k += 256) {
            s0 += src[(int64_t)k * P];
            s1 += src[(int64_t)(k + 64) * P];
            s2 += src[(int64_t)(k + 128) * P];
            s3 += src[(int64_t)(k + 192) * P];
        }
        for (; k < parts; k += 64) s0 += src[(int64_t)k * P];
    }
    part[q][cl] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (q == 0 && c < P) {
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < 64; ++k) t += part[k][cl];
        out[c] = t;
    }
}

// columns per chunk: all of them up to 1024, else 1024 (the last chunk may be narrower)
static int column_sum_chunk(int P) { return P <= 4 * CS_THREADS ? P : 4 * CS_THREADS; }

static int column_sum_parts(int64_t N, int P) {
    const int rpp = CS_THREADS / (column_sum_chunk(P) / 4);
    const int64_t useful = std::max<int64_t>(1, N / (4 * rpp));
    return (int)std::min<int64_t>(1024, useful);
}

}  // namespace sswin

using namespace sswin;

extern "C" {

size_t sswin_column_sum_workspace_bytes(int64_t N, int P) {
    if (P <= 0 || (P % 4)) return 0;
    return (size_t)column_sum_parts(N, P) * P * sizeof(float) + 256;
}

int sswin_column_sum(const void* x, int dtype, int64_t N, int P, float* out, void* ws, size_t ws_bytes, void* stream) {
    SSWIN_CHECK(N >= 0 && P > 0 && (P % 4) == 0, "column_sum: %d columns are not supported (a multiple of 4)", P);
    SSWIN_CHECK(dtype == SSWIN_F32 || dtype == SSWIN_F16 || dtype == SSWIN_BF16, "column_sum: unsupported dtype %d", dtype);
    SSWIN_CHECK(out, "column_sum: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (N == 0) {
        zero_fill(out, (int64_t)P, s);
        return launch_ok("column_sum");
    }
    SSWIN_CHECK(x && ws, "column_sum: null pointer");
    SSWIN_CHECK(((uintptr_t)x % 16) == 0, "column_sum: the matrix is not 16-byte aligned");
    SSWIN_CHECK(ws_bytes >= sswin_column_sum_workspace_bytes(N, P), "column_sum: workspace too small");
    const int parts = column_sum_parts(N, P), chunk = column_sum_chunk(P);
    const dim3 grid((unsigned)parts, (unsigned)((P + chunk - 1) / chunk));
    float* partial = static_cast<float*>(ws);
    switch (dtype) {
        case SSWIN_F32:
            hipLaunchKernelGGL(column_sum_partial_kernel<float>, grid, dim3(CS_THREADS), 0, s, static_cast<const float*>(x), N, P, chunk, partial);
            break;
        case SSWIN_F16:
            hipLaunchKernelGGL(column_sum_partial_kernel<__half>, grid, dim3(CS_THREADS), 0, s, static_cast<const __half*>(x), N, P, chunk, partial);
            break;
        default:
            hipLaunchKernelGGL(column_sum_partial_kernel<__hip_bfloat16>, grid, dim3(CS_THREADS), 0, s,
                               static_cast<const __hip_bfloat16*>(x), N, P, chunk, partial);
            break;
    }
    hipLaunchKernelGGL(column_sum_final_kernel, dim3((unsigned)((P + 15) / 16)), dim3(1024), 0, s, partial, parts, P, out);
    return launch_ok("column_sum");
}

}  // extern "C"
