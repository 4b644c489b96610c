// Y = X W^T + b for a very tall fp32 X [N, K] (N = voxels, K = channels <= 192) and a small weight
// W [P, K]: the qkv and proj projections of the window attention (nn.Linear of
// sparse_swin/swin3d_base.py:606-610, applied at :658 and :676).
//
// On gfx950 the fp32 matrix instruction runs on the vector ALU's own multipliers (64 FLOP per clock
// and SIMD, and it blocks the ALU while it runs), so an fp32 GEMM cannot get past the packed-FMA rate;
// the bf16 matrix cores are sixteen times faster and sit idle.  This kernel uses them without giving
// up fp32 accuracy: every fp32 operand is split exactly into three bf16 pieces (x = h + m + l, 8 + 8 +
// 8 significant bits, by truncation and exact subtraction) and a product is the sum of the six
// piece products whose weight is at least 2^-16 of the leading one (hh, hm, mh, mm, hl, lh), all
// accumulated in fp32 by v_mfma_f32_32x32x16_bf16.  What is dropped (ml, lm, ll) is below 2^-23 of
// the product, i.e. at the level of fp32 rounding itself.
//
// Layout: a workgroup owns one group of 96 output columns and keeps the three bf16 planes of those
// columns of W in LDS in MFMA operand order (split by the workgroup itself when it starts); it
// walks over blocks of 128 rows, one 32-row tile per wave.  Per 16-wide k step a lane reads its
// 8 fp32 of X (row l % 32, k group l / 32), splits them, and feeds 3 column tiles x 6 products.
#include <stdint.h>

#include <algorithm>

#include "mfma_block.hpp"
#include "sswin_common.hpp"

namespace sswin {

typedef __bf16 tl_bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t tl_u32x4 __attribute__((ext_vector_type(4)));
typedef float tl_f32x4 __attribute__((ext_vector_type(4)));

constexpr int TL_COLS = 96;          // output columns per workgroup (3 MFMA tiles)
constexpr int TL_MAX_K = 192;

// exact split of two fp32 values into bf16 pieces, packed (low half = first value)
struct Split2 {
    uint32_t h, m, l;
};
__device__ __forceinline__ Split2 split2(float x0, float x1) {
    const uint32_t u0 = __builtin_bit_cast(uint32_t, x0), u1 = __builtin_bit_cast(uint32_t, x1);
    const float r0 = x0 - __builtin_bit_cast(float, u0 & 0xffff0000u);
    const float r1 = x1 - __builtin_bit_cast(float, u1 & 0xffff0000u);
    const uint32_t v0 = __builtin_bit_cast(uint32_t, r0), v1 = __builtin_bit_cast(uint32_t, r1);
    const float s0 = r0 - __builtin_bit_cast(float, v0 & 0xffff0000u);
    const float s1 = r1 - __builtin_bit_cast(float, v1 & 0xffff0000u);
    Split2 o;
    o.h = __builtin_amdgcn_perm(u1, u0, 0x07060302u);       // {u1.hi16, u0.hi16}
    o.m = __builtin_amdgcn_perm(v1, v0, 0x07060302u);
    o.l = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, s1), __builtin_bit_cast(uint32_t, s0), 0x07060302u);
    return o;
}

__device__ __forceinline__ tl_bf16x8 as_bf16x8(const tl_u32x4& v) { return __builtin_bit_cast(tl_bf16x8, v); }

struct APlanes {
    tl_bf16x8 h, m, l;
};
__device__ __forceinline__ APlanes split8(const tl_f32x4& c0, const tl_f32x4& c1) {
    const Split2 s0 = split2(c0.x, c0.y), s1 = split2(c0.z, c0.w), s2 = split2(c1.x, c1.y), s3 = split2(c1.z, c1.w);
    APlanes a;
    a.h = as_bf16x8(tl_u32x4{s0.h, s1.h, s2.h, s3.h});
    a.m = as_bf16x8(tl_u32x4{s0.m, s1.m, s2.m, s3.m});
    a.l = as_bf16x8(tl_u32x4{s0.l, s1.l, s2.l, s3.l});
    return a;
}

// The workgroup's 96 columns of W, split and laid out in LDS in operand order:
// [k step][column tile 3][plane 3][lane 64][8 bf16]
template <int THREADS>
__device__ __forceinline__ void fill_w_planes(const float* __restrict__ w, int K, int ksteps, int cg, tl_u32x4* w_s) {
    for (int it = threadIdx.x; it < ksteps * 3 * 64; it += THREADS) {
        const int lane = it & 63, ct = (it >> 6) % 3, ks = (it >> 6) / 3;
        const int col = cg * TL_COLS + ct * 32 + (lane & 31);
        const tl_f32x4* src = reinterpret_cast<const tl_f32x4*>(w + (int64_t)col * K + ks * 16 + (lane >> 5) * 8);
        const tl_f32x4 c0 = src[0], c1 = src[1];
        const Split2 s0 = split2(c0.x, c0.y), s1 = split2(c0.z, c0.w), s2 = split2(c1.x, c1.y), s3 = split2(c1.z, c1.w);
        tl_u32x4* dst = w_s + (ks * 3 + ct) * 3 * 64 + lane;
        dst[0] = tl_u32x4{s0.h, s1.h, s2.h, s3.h};
        dst[64] = tl_u32x4{s0.m, s1.m, s2.m, s3.m};
        dst[128] = tl_u32x4{s0.l, s1.l, s2.l, s3.l};
    }
}

// Workgroups b, b + 8, b + 16 ... run on the same XCD and share its L2: the column groups of one set
// of rows are dealt to such workgroups, so X comes from HBM once.  Returns the column group and the
// row slot (0 .. gridDim.x / groups - 1) of this workgroup.
__device__ __forceinline__ void group_and_slot(int groups, int& cg, int& slot) {
    const int b = blockIdx.x, chunk = 8 * groups, full = gridDim.x / chunk * chunk;
    if (b < full) {
        cg = (b / 8) % groups;
        slot = b / chunk * 8 + b % 8;
    } else {
        cg = (b - full) % groups;
        slot = full / groups + (b - full) / groups;
    }
}

// the three planes of the workgroup's three column tiles for one k step, as read from LDS
struct BPlanes {
    tl_bf16x8 h[3], m[3], l[3];
};
__device__ __forceinline__ BPlanes read_b(const tl_u32x4* wk) {
    BPlanes b;
#pragma unroll
    for (int ct = 0; ct < 3; ++ct) {
        b.h[ct] = as_bf16x8(wk[(ct * 3 + 0) * 64]);
        b.m[ct] = as_bf16x8(wk[(ct * 3 + 1) * 64]);
        b.l[ct] = as_bf16x8(wk[(ct * 3 + 2) * 64]);
    }
    return b;
}

// one 16-wide k step of a 32-row tile against the workgroup's 96 columns: 3 tiles x 6 products.
// Small terms first; the three column tiles alternate so that no product waits for the previous one
// into the same accumulator.
__device__ __forceinline__ void k_products(const APlanes& a, const BPlanes& b, f32x16 (&acc)[3]) {
#pragma unroll
    for (int ct = 0; ct < 3; ++ct) acc[ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.l, b.h[ct], acc[ct], 0, 0, 0);
#pragma unroll
    for (int ct = 0; ct < 3; ++ct) acc[ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.h, b.l[ct], acc[ct], 0, 0, 0);
#pragma unroll
    for (int ct = 0; ct < 3; ++ct) acc[ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.m, b.m[ct], acc[ct], 0, 0, 0);
#pragma unroll
    for (int ct = 0; ct < 3; ++ct) acc[ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.m, b.h[ct], acc[ct], 0, 0, 0);
#pragma unroll
    for (int ct = 0; ct < 3; ++ct) acc[ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.h, b.m[ct], acc[ct], 0, 0, 0);
#pragma unroll
    for (int ct = 0; ct < 3; ++ct) acc[ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.h, b.h[ct], acc[ct], 0, 0, 0);
}
__device__ __forceinline__ void k_step(const APlanes& a, const tl_u32x4* wk, f32x16 (&acc)[3]) {
    k_products(a, read_b(wk), acc);
}

// any supported K; the next k step's 8 values are in flight during the current one
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void tall_linear_forward_kernel(
    const float* __restrict__ x, int64_t N, int K, const float* __restrict__ w, int groups, const float* __restrict__ bias,
    float* __restrict__ y, int P, int64_t row_blocks) {
    extern __shared__ __attribute__((aligned(16))) tl_u32x4 w_s[];      // [k step][tile][plane][lane]
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    const int ksteps = K / 16;
    int cg, slot;
    group_and_slot(groups, cg, slot);
    const int64_t wg = slot, wgs = gridDim.x / groups;
    fill_w_planes<256>(w, K, ksteps, cg, w_s);
    __syncthreads();
    float bcol[3];
#pragma unroll
    for (int ct = 0; ct < 3; ++ct) bcol[ct] = bias ? bias[cg * TL_COLS + ct * 32 + l32] : 0.f;

    for (int64_t rb = wg; rb < row_blocks; rb += wgs) {
        const int64_t row0 = rb * 128 + wave * 32;
        f32x16 acc[3];
#pragma unroll
        for (int ct = 0; ct < 3; ++ct) acc[ct] = f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        int64_t row = row0 + l32;
        row = row < N ? row : N - 1;                                     // padding rows read the last row
        const tl_f32x4* xp = reinterpret_cast<const tl_f32x4*>(x + row * K + half * 8);
        tl_f32x4 c0 = xp[0], c1 = xp[1];
        for (int ks = 0; ks < ksteps; ++ks) {
            const APlanes a = split8(c0, c1);
            if (ks + 1 < ksteps) c0 = xp[(ks + 1) * 4], c1 = xp[(ks + 1) * 4 + 1];
            k_step(a, w_s + ks * 9 * 64 + lane, acc);
        }
        if (row0 >= N) continue;
        // accumulator register r of lane l: row acc_row(r, half), column l % 32
#pragma unroll
        for (int ct = 0; ct < 3; ++ct) {
            float* yp = y + (int64_t)cg * TL_COLS + ct * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t orow = row0 + acc_row(r, half);
                if (orow < N) yp[orow * P] = acc[ct][r] + bcol[ct];
            }
        }
    }
}

// The same product with the rows of X read the way they lie in memory.  The kernel above reads a
// row per lane, 16 bytes at a time: every such instruction touches 64 cache lines and the texture
// path, not the matrix cores, sets its pace.  Here a wave reads its 32 x K tile as one contiguous
// run (16 bytes per lane, 8 lines per instruction), one block ahead, parks it in a private LDS tile
// (pitch K + 4 floats, so 8 rows hit 8 different bank groups) and takes its operands from there.
// One workgroup of 8 waves per CU shares the planes of W: K <= 96 fits 160 KB of LDS.
constexpr int TL_STAGED_MAX_KS = 6;
template <int KS>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void tall_linear_forward_staged_kernel(
    const float* __restrict__ x, int64_t N, const float* __restrict__ w, int groups, const float* __restrict__ bias,
    float* __restrict__ y, int P, int64_t row_tiles) {
    constexpr int K = KS * 16, PITCH = K + 4, C4 = K / 4, NI = 2 * KS;   // 16-byte chunks per row; loads per lane and tile
    extern __shared__ __attribute__((aligned(16))) tl_u32x4 w_s[];      // [k step][tile][plane][lane], then the X tiles
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    int cg, slot;
    group_and_slot(groups, cg, slot);
    const int64_t first = (int64_t)slot * 8 + wave, stride = (int64_t)(gridDim.x / groups) * 8;
    constexpr int n16 = KS * 9 * 64;
    fill_w_planes<512>(w, K, KS, cg, w_s);
    float* xs = reinterpret_cast<float*>(w_s + n16) + wave * 32 * PITCH;
    __syncthreads();
    float bcol[3];
#pragma unroll
    for (int ct = 0; ct < 3; ++ct) bcol[ct] = bias ? bias[cg * TL_COLS + ct * 32 + l32] : 0.f;

    tl_f32x4 xn[NI];
    auto fetch = [&](int64_t t) {
        const int64_t e0 = t * 32 * K, end = N * K;                      // the tile is 32 K consecutive floats
        const tl_f32x4* xp = reinterpret_cast<const tl_f32x4*>(x + e0);
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int q = i * 64 + lane;
            xn[i] = e0 + q * 4 < end ? xp[q] : tl_f32x4{0.f, 0.f, 0.f, 0.f};
        }
    };
    if (first < row_tiles) fetch(first);
    for (int64_t t = first; t < row_tiles; t += stride) {
        const int64_t row0 = t * 32;
        __builtin_amdgcn_wave_barrier();                                 // the previous tile's operand reads are done
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int q = i * 64 + lane;
            *reinterpret_cast<tl_f32x4*>(xs + (q / C4) * PITCH + (q % C4) * 4) = xn[i];
        }
        __builtin_amdgcn_wave_barrier();
        if (t + stride < row_tiles) fetch(t + stride);
        f32x16 acc[3];
#pragma unroll
        for (int ct = 0; ct < 3; ++ct) acc[ct] = f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        const float* xr = xs + l32 * PITCH + half * 8;
        // the operands of step ks + 1 are read and split while the products of step ks run
        APlanes a[2];
        BPlanes b[2];
        a[0] = split8(*reinterpret_cast<const tl_f32x4*>(xr), *reinterpret_cast<const tl_f32x4*>(xr + 4));
        b[0] = read_b(w_s + lane);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (ks + 1 < KS) {
                b[(ks + 1) & 1] = read_b(w_s + (ks + 1) * 9 * 64 + lane);
                a[(ks + 1) & 1] = split8(*reinterpret_cast<const tl_f32x4*>(xr + (ks + 1) * 16),
                                         *reinterpret_cast<const tl_f32x4*>(xr + (ks + 1) * 16 + 4));
            }
            k_products(a[ks & 1], b[ks & 1], acc);
            __builtin_amdgcn_sched_barrier(0);                           // keeps the operands of later steps out of registers
        }
#pragma unroll
        for (int ct = 0; ct < 3; ++ct) {
            float* yp = y + (int64_t)cg * TL_COLS + ct * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t orow = row0 + acc_row(r, half);
                if (orow < N) yp[orow * P] = acc[ct][r] + bcol[ct];
            }
        }
    }
}

}  // namespace sswin

using namespace sswin;

static int staged_lds_bytes(int ksteps) {
    return ksteps * 9 * 64 * (int)sizeof(tl_u32x4) + 8 * 32 * (ksteps * 16 + 4) * (int)sizeof(float);
}

extern "C" {

int sswin_tall_linear_supported(int P, int K) {
    return P > 0 && K > 0 && (P % TL_COLS) == 0 && (K % 16) == 0 && K <= TL_MAX_K;
}

int sswin_tall_linear_forward(const float* x, int64_t N, int K, const float* w, const float* bias, int P, float* y,
                              void* stream) {
    SSWIN_CHECK(N >= 0 && K > 0 && P > 0, "tall_linear_forward: bad sizes");
    SSWIN_CHECK(K % 16 == 0 && K <= TL_MAX_K, "tall_linear_forward: %d input channels are not supported (a multiple of 16, at most %d)",
                K, TL_MAX_K);
    SSWIN_CHECK(P % TL_COLS == 0, "tall_linear_forward: %d output channels are not a multiple of %d", P, TL_COLS);
    if (N == 0) return 0;
    SSWIN_CHECK(x && w && y, "tall_linear_forward: null pointer");
    SSWIN_CHECK(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0, "tall_linear_forward: x and w must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int groups = P / TL_COLS, ksteps = K / 16;
    int cus = 256;
    {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            cus = n;
    }
    static bool configured = false;
    if (!configured) {
        const int max_lds = TL_MAX_K / 16 * 9 * 64 * (int)sizeof(tl_u32x4);
        SSWIN_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(tall_linear_forward_kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, max_lds));
        const void* staged[] = {reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<1>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<2>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<3>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<4>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<5>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<6>)};
        for (int ks = 1; ks <= TL_STAGED_MAX_KS; ++ks)
            SSWIN_HIP(hipFuncSetAttribute(staged[ks - 1], hipFuncAttributeMaxDynamicSharedMemorySize, staged_lds_bytes(ks)));
        configured = true;
    }
    if (ksteps <= TL_STAGED_MAX_KS) {
        const int64_t row_tiles = (N + 31) / 32;
        const int64_t per_group = std::min<int64_t>((row_tiles + 7) / 8, std::max<int64_t>(1, cus / groups));
        const dim3 grid((unsigned)(per_group * groups)), block(512);
        const size_t lds = staged_lds_bytes(ksteps);
#define SSWIN_TL_STAGED(KS)                                                                                                  \
    case KS:                                                                                                                 \
        hipLaunchKernelGGL(tall_linear_forward_staged_kernel<KS>, grid, block, lds, s, x, N, w, groups, bias, y, P,          \
                           row_tiles);                                                                                       \
        break;
        switch (ksteps) {
            SSWIN_TL_STAGED(1) SSWIN_TL_STAGED(2) SSWIN_TL_STAGED(3) SSWIN_TL_STAGED(4) SSWIN_TL_STAGED(5) SSWIN_TL_STAGED(6)
        }
#undef SSWIN_TL_STAGED
        return launch_ok("tall_linear_forward");
    }
    const size_t lds = (size_t)ksteps * 9 * 64 * sizeof(tl_u32x4);
    const int64_t row_blocks = (N + 127) / 128;
    const int per_cu = lds <= 64 * 1024 ? 2 : 1;                          // workgroups that fit a CU's LDS
    int64_t per_group = std::min<int64_t>(row_blocks, std::max<int64_t>(1, (int64_t)cus * per_cu / groups));
    hipLaunchKernelGGL(tall_linear_forward_kernel, dim3((unsigned)(per_group * groups)), dim3(256), lds, s, x, N, K, w, groups,
                       bias, y, P, row_blocks);
    return launch_ok("tall_linear_forward");
}

}  // extern "C"
