// The qkv and proj projections of the window attention (nn.Linear of sparse_swin/swin3d_base.py:606-610,
// applied at :658 and :676) for fp32 tokens: Y = X W^T + b for a very tall X [N, K] (N = voxels) and a
// small weight W [P, K], the input gradient dX = dY W and the weight / bias gradient dW = dY^T X,
// db = column sums of dY.
//
// On gfx950 the fp32 matrix instruction runs on the vector ALU's own multipliers (64 FLOP per clock
// and SIMD, and it blocks the ALU while it runs), so an fp32 GEMM cannot get past the packed-FMA rate;
// the bf16 matrix cores are sixteen times faster and sit idle.  These kernels use them without giving
// up fp32 accuracy: every fp32 operand is split exactly into three bf16 pieces (x = h + m + l, 8 + 8 +
// 8 significant bits, by truncation and exact subtraction) and a product is the sum of the six
// piece products whose weight is at least 2^-16 of the leading one (hh, hm, mh, mm, hl, lh), all
// accumulated in fp32 by v_mfma_f32_32x32x16_bf16.  What is dropped (ml, lm, ll) is below 2^-23 of
// the product, i.e. at the level of fp32 rounding itself.  Inputs are taken to be finite (the pieces
// of an infinity are infinity and NaN).
//
// Common layout of the row-streaming kernels (forward, input gradient): a workgroup owns one group of
// 96 output columns and keeps the three bf16 planes of those columns of W in LDS in MFMA operand order
// (it splits them itself when it starts); its waves walk over 32-row tiles.  Per 16-wide k step a
// lane holds 8 fp32 of X (row l % 32, k group l / 32), splits them, and feeds 3 column tiles x 6
// products.  Kernels, by shape:
//   tall_linear_forward_staged_kernel   K <= 96 (also dX of a 96-column dY, W read transposed)
//   tall_linear_forward_kernel          96 < K <= 192
//   tall_linear_wide_kernel             dX for 192..288 columns of dY: all of W on the CU
//   tall_linear_chunked_kernel          dX for more columns of dY: W in chunks of 96 rows
//   tall_linear_wgrad_kernel (+ reduce) dW and db, the reduction over the rows
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
// TRANSPOSED: the operand is W^T of a [K, P] array (w[k * P + col]: the input gradient of a layer whose
// weight is stored [out, in]); otherwise w[col * K + k].
template <int THREADS, bool TRANSPOSED = false>
__device__ __forceinline__ void fill_w_planes(const float* __restrict__ w, int K, int ksteps, int cg, tl_u32x4* w_s, int P = 0) {
    for (int it = threadIdx.x; it < ksteps * 3 * 64; it += THREADS) {
        const int lane = it & 63, ct = (it >> 6) % 3, ks = (it >> 6) / 3;
        const int col = cg * TL_COLS + ct * 32 + (lane & 31), k0 = ks * 16 + (lane >> 5) * 8;
        float v[8];
        if (TRANSPOSED) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = w[(int64_t)(k0 + e) * P + col];
        } else {
            const tl_f32x4* src = reinterpret_cast<const tl_f32x4*>(w + (int64_t)col * K + k0);
            const tl_f32x4 c0 = src[0], c1 = src[1];
            v[0] = c0.x; v[1] = c0.y; v[2] = c0.z; v[3] = c0.w; v[4] = c1.x; v[5] = c1.y; v[6] = c1.z; v[7] = c1.w;
        }
        const Split2 s0 = split2(v[0], v[1]), s1 = split2(v[2], v[3]), s2 = split2(v[4], v[5]), s3 = split2(v[6], v[7]);
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
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave: a scalar
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
// SMALL: fewer than 32 rows in all (one ragged tile, guarded).  Otherwise a last ragged tile is moved
// back to end at row N: it recomputes a few rows of its neighbour (same inputs, same arithmetic, the
// same bits stored twice) and every tile takes the unguarded path.
template <int KS, bool SMALL, bool TRANSPOSED = false>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void tall_linear_forward_staged_kernel(
    const float* __restrict__ x, int64_t N, const float* __restrict__ w, int groups, const float* __restrict__ bias,
    float* __restrict__ y, int P, int64_t row_tiles) {
    constexpr int K = KS * 16, PITCH = K + 4, C4 = K / 4, NI = 2 * KS;   // 16-byte chunks per row; loads per lane and tile
    extern __shared__ __attribute__((aligned(16))) tl_u32x4 w_s[];      // [k step][tile][plane][lane], then the X tiles
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave: a scalar
    const int half = lane >> 5, l32 = lane & 31;
    int cg, slot;
    group_and_slot(groups, cg, slot);
    const int64_t first = (int64_t)slot * 8 + wave, stride = (int64_t)(gridDim.x / groups) * 8;
    constexpr int n16 = KS * 9 * 64;
    fill_w_planes<512, TRANSPOSED>(w, K, KS, cg, w_s, P);
    float* xs = reinterpret_cast<float*>(w_s + n16) + wave * 32 * PITCH;
    __syncthreads();
    float bcol[3];
#pragma unroll
    for (int ct = 0; ct < 3; ++ct) bcol[ct] = bias ? bias[cg * TL_COLS + ct * 32 + l32] : 0.f;

    // A load instruction covers 64 / GW rows x GW 16-byte chunks (GW x 16 contiguous bytes per row), so
    // that global and LDS addresses are a per-lane part, computed once, plus a compile-time part.
    constexpr int GW = (C4 % 8 == 0) ? 8 : 4, RPI = 64 / GW, CGS = C4 / GW;   // rows per instruction, chunk groups per row
    static_assert(NI == (32 / RPI) * CGS, "loads per tile");
    const int lr = lane / GW, lc = lane % GW;
    const uint32_t g_lane = (uint32_t)(lr * K + lc * 4);                 // floats, within the tile
    const uint32_t s_lane = (uint32_t)(lr * PITCH + lc * 4);
    const uint32_t y_lane = (uint32_t)(4 * half * P + l32);              // accumulator rows start at 4 * half
    tl_f32x4 xn[NI];
    auto tile_row0 = [&](int64_t t) { return SMALL ? 0 : (t * 32 + 32 <= N ? t * 32 : N - 32); };
    auto fetch = [&](int64_t t) {
        const float* xt = x + tile_row0(t) * K;                          // uniform; the tile is 32 K consecutive floats
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const tl_f32x4* src = reinterpret_cast<const tl_f32x4*>(xt + ((i / CGS) * RPI * K + (i % CGS) * GW * 4) + g_lane);
            if (SMALL)
                xn[i] = (i / CGS) * RPI + lr < N ? *src : tl_f32x4{0.f, 0.f, 0.f, 0.f};
            else
                xn[i] = *src;
        }
    };
    if (first < row_tiles) fetch(first);
    for (int64_t t = first; t < row_tiles; t += stride) {
        const int64_t row0 = tile_row0(t);
        __builtin_amdgcn_wave_barrier();                                 // the previous tile's operand reads are done
#pragma unroll
        for (int i = 0; i < NI; ++i)
            *reinterpret_cast<tl_f32x4*>(xs + ((i / CGS) * RPI * PITCH + (i % CGS) * GW * 4) + s_lane) = xn[i];
        __builtin_amdgcn_wave_barrier();
        if (t + stride < row_tiles) fetch(t + stride);
        f32x16 acc[3];
#pragma unroll
        for (int ct = 0; ct < 3; ++ct) acc[ct] = f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        const float* xr = xs + l32 * PITCH + half * 8;
        // Software pipeline over the k steps: during the 18 products of step ks the planes of W for step
        // ks + 1 and the 8 values of X for step ks + 2 are read from LDS, and the values of step ks + 1
        // (read one step earlier) are split, three vector instructions after every MFMA, so that the
        // vector ALU works in the shadow of the matrix core.
        APlanes a[2];
        BPlanes b[2];
        tl_f32x4 raw[2][2];
        raw[0][0] = *reinterpret_cast<const tl_f32x4*>(xr);
        raw[0][1] = *reinterpret_cast<const tl_f32x4*>(xr + 4);
        b[0] = read_b(w_s + lane);
        if (KS > 1) {
            raw[1][0] = *reinterpret_cast<const tl_f32x4*>(xr + 16);
            raw[1][1] = *reinterpret_cast<const tl_f32x4*>(xr + 20);
        }
        a[0] = split8(raw[0][0], raw[0][1]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (ks + 1 < KS) b[(ks + 1) & 1] = read_b(w_s + (ks + 1) * 9 * 64 + lane);
            if (ks + 2 < KS) {
                raw[ks & 1][0] = *reinterpret_cast<const tl_f32x4*>(xr + (ks + 2) * 16);
                raw[ks & 1][1] = *reinterpret_cast<const tl_f32x4*>(xr + (ks + 2) * 16 + 4);
            }
            k_products(a[ks & 1], b[ks & 1], acc);
            if (ks + 1 < KS) a[(ks + 1) & 1] = split8(raw[(ks + 1) & 1][0], raw[(ks + 1) & 1][1]);
            // order inside the step: the LDS reads, then MFMA / vector / vector / vector ...
            __builtin_amdgcn_sched_group_barrier(0x100, 11, 0);
#pragma unroll
            for (int q = 0; q < 18; ++q) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
            }
            __builtin_amdgcn_sched_barrier(0);                           // keeps the operands of later steps out of registers
        }
        // accumulator register r of lane l: row 8 (r / 4) + 4 half + r % 4, column l % 32
        float* yt = y + row0 * P + cg * TL_COLS;                         // uniform
#pragma unroll
        for (int ct = 0; ct < 3; ++ct)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (!SMALL || acc_row(r, half) < N)                      // the bias last: the small terms are summed first
                    (yt + (8 * (r >> 2) + (r & 3)) * P + ct * 32)[y_lane] = acc[ct][r] + bcol[ct];
    }
}

// ------------------------------------------------------------------------------------------
// More than 96 input channels: y[N, 96 G] = x[N, 96 C] Wop, C chunks of 96 channels, accumulators kept
// in registers over the chunks.  The planes of one chunk of W (54 KB) are double buffered in LDS: the
// values of the next chunk are requested before the products of the current one and split and
// stored after them, one barrier per chunk.  One workgroup of 8 waves per CU, one 32-row tile per
// wave; the lane's 48 values of the next chunk of X are in flight during the products.
// TRANSPOSED: Wop[k][col] = w[k * out + col] (input gradient dX = dY W of the layer, W [P, K] as
// stored); otherwise Wop[k][col] = w[col * in + k] (the forward with W [P, K]).
// ------------------------------------------------------------------------------------------
constexpr int CH_KS = 6, CH_ITEMS = CH_KS * 3 * 64, CH_SLOTS = (CH_ITEMS + 511) / 512;

template <bool TRANSPOSED>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void tall_linear_chunked_kernel(
    const float* __restrict__ x, int64_t N, int in, const float* __restrict__ w, int groups, const float* __restrict__ bias,
    float* __restrict__ y, int out, int64_t row_tiles) {
    extern __shared__ __attribute__((aligned(16))) tl_u32x4 w_s[];      // [buffer 2][k step 6][tile 3][plane 3][lane 64]
    constexpr int BUF = CH_KS * 9 * 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave: a scalar
    const int half = lane >> 5, l32 = lane & 31;
    const int chunks = in / 96;
    int cg, slot;
    group_and_slot(groups, cg, slot);
    const int64_t first = (int64_t)slot * 8 + wave, stride = (int64_t)(gridDim.x / groups) * 8;
    // every wave of the workgroup runs the same number of rounds (barriers inside)
    const int64_t wg_first = (int64_t)slot * 8;
    const int rounds = wg_first < row_tiles ? (int)((row_tiles - wg_first + stride - 1) / stride) : 0;

    // --- the chunk of W that comes next: raw values in registers, then planes in LDS
    float wraw[CH_SLOTS][8];
    auto w_request = [&](int chunk) {
#pragma unroll
        for (int q = 0; q < CH_SLOTS; ++q) {
            const int it = threadIdx.x + q * 512;
            if (it < CH_ITEMS) {
                const int ln = it & 63, ct = (it >> 6) % 3, ks = (it >> 6) / 3;
                const int col = cg * TL_COLS + ct * 32 + (ln & 31), k0 = chunk * 96 + ks * 16 + (ln >> 5) * 8;
                if (TRANSPOSED) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) wraw[q][e] = w[(int64_t)(k0 + e) * out + col];
                } else {
                    const tl_f32x4* src = reinterpret_cast<const tl_f32x4*>(w + (int64_t)col * in + k0);
                    const tl_f32x4 c0 = src[0], c1 = src[1];
                    wraw[q][0] = c0.x; wraw[q][1] = c0.y; wraw[q][2] = c0.z; wraw[q][3] = c0.w;
                    wraw[q][4] = c1.x; wraw[q][5] = c1.y; wraw[q][6] = c1.z; wraw[q][7] = c1.w;
                }
            }
        }
    };
    auto w_store = [&](tl_u32x4* buf) {
#pragma unroll
        for (int q = 0; q < CH_SLOTS; ++q) {
            const int it = threadIdx.x + q * 512;
            if (it < CH_ITEMS) {
                const Split2 s0 = split2(wraw[q][0], wraw[q][1]), s1 = split2(wraw[q][2], wraw[q][3]);
                const Split2 s2 = split2(wraw[q][4], wraw[q][5]), s3 = split2(wraw[q][6], wraw[q][7]);
                tl_u32x4* dst = buf + (it >> 6) * 3 * 64 + (it & 63);
                dst[0] = tl_u32x4{s0.h, s1.h, s2.h, s3.h};
                dst[64] = tl_u32x4{s0.m, s1.m, s2.m, s3.m};
                dst[128] = tl_u32x4{s0.l, s1.l, s2.l, s3.l};
            }
        }
    };
    // --- the lane's 48 values of one chunk of its row (row l % 32 of the tile, k group l / 32)
    tl_f32x4 xn[CH_KS][2];
    auto x_request = [&](int64_t tile, int chunk) {
        int64_t row = tile * 32 + l32;
        row = row < N ? row : N - 1;                                     // padding rows read the last row
        const tl_f32x4* xp = reinterpret_cast<const tl_f32x4*>(x + row * in + chunk * 96 + half * 8);
#pragma unroll
        for (int ks = 0; ks < CH_KS; ++ks) xn[ks][0] = xp[ks * 4], xn[ks][1] = xp[ks * 4 + 1];
    };
    float bcol[3];
#pragma unroll
    for (int ct = 0; ct < 3; ++ct) bcol[ct] = bias ? bias[cg * TL_COLS + ct * 32 + l32] : 0.f;

    if (rounds > 0) {
        w_request(0);
        w_store(w_s);
        x_request(first < row_tiles ? first : row_tiles - 1, 0);
    }
    __syncthreads();
    int it = 0;                                                          // chunk iterations so far: buffer it & 1 is current
    for (int r = 0; r < rounds; ++r) {
        const int64_t tile = first + (int64_t)r * stride;
        const int64_t my_tile = tile < row_tiles ? tile : row_tiles - 1; // a wave past the end repeats the last tile, stores nothing
        f32x16 acc[3];
#pragma unroll
        for (int ct = 0; ct < 3; ++ct) acc[ct] = f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        for (int c = 0; c < chunks; ++c, ++it) {
            tl_f32x4 xc[CH_KS][2];
#pragma unroll
            for (int ks = 0; ks < CH_KS; ++ks) xc[ks][0] = xn[ks][0], xc[ks][1] = xn[ks][1];
            const bool last = r + 1 == rounds && c + 1 == chunks;
            const int next_c = c + 1 < chunks ? c + 1 : 0;
            if (!last) {
                w_request(next_c);
                int64_t nt = c + 1 < chunks ? my_tile : tile + stride;
                x_request(nt < row_tiles ? nt : row_tiles - 1, next_c);
            }
            const tl_u32x4* cur = w_s + (it & 1) * BUF + lane;
#pragma unroll
            for (int ks = 0; ks < CH_KS; ++ks) {
                k_step(split8(xc[ks][0], xc[ks][1]), cur + ks * 9 * 64, acc);
                __builtin_amdgcn_sched_barrier(0);                       // keeps the operands of later steps out of registers
            }
            if (!last) w_store(w_s + ((it + 1) & 1) * BUF);
            __syncthreads();
        }
        if (tile < row_tiles) {
            const int64_t row0 = tile * 32;
#pragma unroll
            for (int ct = 0; ct < 3; ++ct) {
                float* yp = y + (int64_t)cg * TL_COLS + ct * 32 + l32;
#pragma unroll
                for (int rr = 0; rr < 16; ++rr) {
                    const int64_t orow = row0 + acc_row(rr, half);
                    if (orow < N) yp[orow * out] = acc[ct][rr] + bcol[ct];
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// 96 < input channels <= 288 without chunk barriers: the planes of all of W for the workgroup's 96 columns
// stay in LDS (9 KB per k step, at most 17 steps = 153 KB); with 18 steps (288 channels: the input
// gradient of the qkv layer of a 96-channel stage) the planes of the last step stay in registers, 36
// per lane.  After the fill nothing is shared any more: every wave streams its 32-row tiles on its
// own, the lane's 48 values of the next 96 channels in flight during the products.
// ------------------------------------------------------------------------------------------
constexpr int WIDE_LDS_KS = 17, WIDE_MAX_KS = 18;

template <bool TRANSPOSED>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void tall_linear_wide_kernel(
    const float* __restrict__ x, int64_t N, int in, const float* __restrict__ w, int groups, const float* __restrict__ bias,
    float* __restrict__ y, int out, int64_t row_tiles) {
    extern __shared__ __attribute__((aligned(16))) tl_u32x4 w_s[];      // [k step][tile 3][plane 3][lane 64]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    const int ksteps = in / 16, chunks = in / 96;
    const int lds_ks = ksteps < WIDE_LDS_KS ? ksteps : WIDE_LDS_KS;
    int cg, slot;
    group_and_slot(groups, cg, slot);
    const int64_t first = (int64_t)slot * 8 + wave, stride = (int64_t)(gridDim.x / groups) * 8;

    // 8 values of Wop for (column, k0 .. k0 + 7)
    auto w_load = [&](int col, int k0, float (&v)[8]) {
        if (TRANSPOSED) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = w[(int64_t)(k0 + e) * out + col];
        } else {
            const tl_f32x4* src = reinterpret_cast<const tl_f32x4*>(w + (int64_t)col * in + k0);
            const tl_f32x4 c0 = src[0], c1 = src[1];
            v[0] = c0.x; v[1] = c0.y; v[2] = c0.z; v[3] = c0.w; v[4] = c1.x; v[5] = c1.y; v[6] = c1.z; v[7] = c1.w;
        }
    };
    auto w_split = [&](const float (&v)[8], tl_u32x4& h, tl_u32x4& m, tl_u32x4& l) {
        const Split2 s0 = split2(v[0], v[1]), s1 = split2(v[2], v[3]), s2 = split2(v[4], v[5]), s3 = split2(v[6], v[7]);
        h = tl_u32x4{s0.h, s1.h, s2.h, s3.h};
        m = tl_u32x4{s0.m, s1.m, s2.m, s3.m};
        l = tl_u32x4{s0.l, s1.l, s2.l, s3.l};
    };
    // The fill is a chain of memory latencies if it goes item by item, so all of a thread's values (at
    // most 7 items of the LDS part and the 3 of the register part) are requested first.
    constexpr int FILL_ITEMS = (WIDE_LDS_KS * 3 * 64 + 511) / 512;
    const int total = lds_ks * 3 * 64;
    float wv[FILL_ITEMS][8], wr[3][8];
#pragma unroll
    for (int q = 0; q < FILL_ITEMS; ++q) {
        const int it = threadIdx.x + q * 512;
        if (it < total) w_load(cg * TL_COLS + ((it >> 6) % 3) * 32 + (it & 31), ((it >> 6) / 3) * 16 + ((it & 63) >> 5) * 8, wv[q]);
    }
    if (ksteps > WIDE_LDS_KS) {
#pragma unroll
        for (int ct = 0; ct < 3; ++ct) w_load(cg * TL_COLS + ct * 32 + l32, WIDE_LDS_KS * 16 + half * 8, wr[ct]);
    }
#pragma unroll
    for (int q = 0; q < FILL_ITEMS; ++q) {
        const int it = threadIdx.x + q * 512;
        if (it < total) {
            tl_u32x4 h, m, l;
            w_split(wv[q], h, m, l);
            tl_u32x4* dst = w_s + (it >> 6) * 3 * 64 + (it & 63);
            dst[0] = h;
            dst[64] = m;
            dst[128] = l;
        }
    }
    BPlanes breg;                                                        // planes of k step 17, this lane's operand slots
    if (ksteps > WIDE_LDS_KS) {
#pragma unroll
        for (int ct = 0; ct < 3; ++ct) {
            tl_u32x4 h, m, l;
            w_split(wr[ct], h, m, l);
            breg.h[ct] = as_bf16x8(h);
            breg.m[ct] = as_bf16x8(m);
            breg.l[ct] = as_bf16x8(l);
        }
    }
    float bcol[3];
#pragma unroll
    for (int ct = 0; ct < 3; ++ct) bcol[ct] = bias ? bias[cg * TL_COLS + ct * 32 + l32] : 0.f;
    __syncthreads();

    // the lane's 48 values of 96 channels of its row (row l % 32 of the tile, k group l / 32)
    tl_f32x4 xn[CH_KS][2];
    auto x_request = [&](int64_t tile, int chunk) {
        int64_t row = tile * 32 + l32;
        row = row < N ? row : N - 1;                                     // padding rows read the last row
        const tl_f32x4* xp = reinterpret_cast<const tl_f32x4*>(x + row * in + chunk * 96 + half * 8);
#pragma unroll
        for (int ks = 0; ks < CH_KS; ++ks) xn[ks][0] = xp[ks * 4], xn[ks][1] = xp[ks * 4 + 1];
    };
    if (first < row_tiles) x_request(first, 0);
    for (int64_t tile = first; tile < row_tiles; tile += stride) {
        f32x16 acc[3];
#pragma unroll
        for (int ct = 0; ct < 3; ++ct) acc[ct] = f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        for (int c = 0; c < chunks; ++c) {
            tl_f32x4 xc[CH_KS][2];
#pragma unroll
            for (int ks = 0; ks < CH_KS; ++ks) xc[ks][0] = xn[ks][0], xc[ks][1] = xn[ks][1];
            if (c + 1 < chunks)
                x_request(tile, c + 1);
            else if (tile + stride < row_tiles)
                x_request(tile + stride, 0);
            const tl_u32x4* cur = w_s + c * CH_KS * 9 * 64 + lane;
#pragma unroll
            for (int ks = 0; ks < CH_KS; ++ks) {
                const APlanes a = split8(xc[ks][0], xc[ks][1]);
                if (c * CH_KS + ks < WIDE_LDS_KS)
                    k_step(a, cur + ks * 9 * 64, acc);
                else
                    k_products(a, breg, acc);
                __builtin_amdgcn_sched_barrier(0);                       // keeps the operands of later steps out of registers
            }
        }
        const int64_t row0 = tile * 32;
#pragma unroll
        for (int ct = 0; ct < 3; ++ct) {
            float* yp = y + (int64_t)cg * TL_COLS + ct * 32 + l32;
#pragma unroll
            for (int rr = 0; rr < 16; ++rr) {
                const int64_t orow = row0 + acc_row(rr, half);
                if (orow < N) yp[orow * out] = acc[ct][rr] + bcol[ct];
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// Weight and bias gradient of the same layers: dW[P,K] = dY^T X, db[P] = column sums of dY, for
// dY [N,P] and X [N,K] (autograd of the nn.Linear at swin3d_base.py:606-610).
//
// The reduction runs over the rows, so both operands carry rows in their k slots: a lane reads 8 rows
// of one column with 8 dword loads (32 lanes = 128 contiguous bytes of a row) and splits them in
// registers.  A workgroup has 12 waves = 4 row quarters x 3 waves; a wave owns one 32-column tile of dY
// (within the workgroup's group of 96 columns of dY) against all of X's column tiles.  The split planes
// of X are shared among the 3 waves of a quarter through LDS (each wave splits one tile of X), double
// buffered with one barrier per 16-row step.  The quarters are added through LDS at the end in a
// fixed order, every workgroup writes one partial dW / db, and a second kernel adds the partials in
// workgroup order: no atomics, the same bits on every run.
// ------------------------------------------------------------------------------------------
constexpr int WG_QUARTERS = 4, WG_WAVES = 12, WG_STEP_ROWS = 16 * WG_QUARTERS;

struct Raw8 {
    float v[8];
};
__device__ __forceinline__ APlanes split_raw8(const Raw8& r) {
    const Split2 s0 = split2(r.v[0], r.v[1]), s1 = split2(r.v[2], r.v[3]), s2 = split2(r.v[4], r.v[5]), s3 = split2(r.v[6], r.v[7]);
    APlanes a;
    a.h = as_bf16x8(tl_u32x4{s0.h, s1.h, s2.h, s3.h});
    a.m = as_bf16x8(tl_u32x4{s0.m, s1.m, s2.m, s3.m});
    a.l = as_bf16x8(tl_u32x4{s0.l, s1.l, s2.l, s3.l});
    return a;
}

// XT = K / 32 column tiles of X (1..3); PITCHED: x has more columns than this pass takes (row pitch
// x_pitch), otherwise its rows are K long and the row offsets are compile-time constants
// PC: the number of columns of dy when it is known at compile time (row offsets become constants), else 0
template <int XT, bool PITCHED, int PC = 0>
__global__ __launch_bounds__(WG_WAVES * 64) __attribute__((amdgpu_waves_per_eu(3, 3))) void tall_linear_wgrad_kernel(
    const float* __restrict__ dy, const float* __restrict__ x, int x_pitch, int64_t N, int P_rt, int groups,
    int64_t rows_per_chunk, float* __restrict__ part_w, float* __restrict__ part_b) {
    constexpr int K = XT * 32;                                           // columns of X in this pass (x: their first column)
    const int xp = PITCHED ? x_pitch : K;
    const int P = PC ? PC : P_rt;
    // X planes: [buffer 2][quarter 4][tile XT][plane 3][lane 64] x 16 bytes; reused for the final sums
    extern __shared__ __attribute__((aligned(16))) tl_u32x4 lds[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave: a scalar
    const int half = lane >> 5, l32 = lane & 31;
    const int quarter = wave / 3, t = wave % 3;                          // t: this wave's column tile of dY (and of X)
    int g, chunk;
    group_and_slot(groups, g, chunk);                                    // the groups of one row chunk share an XCD's L2
    const int64_t row_begin = (int64_t)chunk * rows_per_chunk;
    const int64_t row_end = row_begin + rows_per_chunk < N ? row_begin + rows_per_chunk : N;
    const int steps = (int)((row_end - row_begin + WG_STEP_ROWS - 1) / WG_STEP_ROWS);
    const int ycol = g * 96 + t * 32 + l32, xcol = t * 32 + l32;
    constexpr int BUF = WG_QUARTERS * XT * 3 * 64;                       // 16-byte units per buffer

    f32x16 acc[XT];
#pragma unroll
    for (int xt = 0; xt < XT; ++xt) acc[xt] = f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    float bsum = 0.f;
    // rows are requested two steps ahead (loaded HBM latency is about two steps of products)
    Raw8 ry[2], rx[2];
    // addresses: a uniform part (scalar arithmetic) plus a per-lane offset computed once
    const uint32_t y_lane = (uint32_t)(half * 8 * P + ycol), x_lane = (uint32_t)(half * 8 * xp + xcol);
    auto fetch = [&](int s, Raw8& y8, Raw8& x8) {
        const int64_t r0 = row_begin + (int64_t)s * WG_STEP_ROWS + quarter * 16;
        const float* yb = dy + r0 * P;
        const float* xb = x + r0 * xp;
        if (r0 + 16 <= row_end) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                y8.v[e] = (yb + e * P)[y_lane];
                if (t < XT) x8.v[e] = (xb + e * xp)[x_lane];
            }
        } else {                                                         // the ragged end of the rows: zeros past it
            const int nvalid = (int)(row_end - r0) - half * 8;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                y8.v[e] = e < nvalid ? (yb + e * P)[y_lane] : 0.f;
                if (t < XT) x8.v[e] = e < nvalid ? (xb + e * xp)[x_lane] : 0.f;
            }
        }
    };
    auto step = [&](int s, Raw8& y8, Raw8& x8) {
        tl_u32x4* buf = lds + (s & 1) * BUF + quarter * XT * 3 * 64;
        if (t < XT) {
            const APlanes xp = split_raw8(x8);
            tl_u32x4* dst = buf + t * 3 * 64 + lane;
            dst[0] = __builtin_bit_cast(tl_u32x4, xp.h);
            dst[64] = __builtin_bit_cast(tl_u32x4, xp.m);
            dst[128] = __builtin_bit_cast(tl_u32x4, xp.l);
        }
        const APlanes a = split_raw8(y8);
#pragma unroll
        for (int e = 0; e < 8; ++e) bsum += y8.v[e];
        if (s + 2 < steps) fetch(s + 2, y8, x8);
        __syncthreads();
#pragma unroll
        for (int xt = 0; xt < XT; ++xt) {
            const tl_bf16x8 bh = as_bf16x8(buf[(xt * 3 + 0) * 64 + lane]);
            const tl_bf16x8 bm = as_bf16x8(buf[(xt * 3 + 1) * 64 + lane]);
            const tl_bf16x8 bl = as_bf16x8(buf[(xt * 3 + 2) * 64 + lane]);
            acc[xt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.l, bh, acc[xt], 0, 0, 0);
            acc[xt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.h, bl, acc[xt], 0, 0, 0);
            acc[xt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.m, bm, acc[xt], 0, 0, 0);
            acc[xt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.m, bh, acc[xt], 0, 0, 0);
            acc[xt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.h, bm, acc[xt], 0, 0, 0);
            acc[xt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.h, bh, acc[xt], 0, 0, 0);
        }
    };
    fetch(0, ry[0], rx[0]);
    if (steps > 1) fetch(1, ry[1], rx[1]);
    for (int s = 0; s < steps; s += 2) {
        step(s, ry[0], rx[0]);
        if (s + 1 < steps) step(s + 1, ry[1], rx[1]);
    }
    // quarters: (0 + 2) + (1 + 3), through LDS; values of a wave at [slot][value][lane]
    float* red = reinterpret_cast<float*>(lds);
    constexpr int VALS = XT * 16 + 1;                                    // accumulators and the bias sum
    auto put = [&](int slot) {
        float* dst = red + (slot * VALS) * 64 + lane;
#pragma unroll
        for (int xt = 0; xt < XT; ++xt)
#pragma unroll
            for (int r = 0; r < 16; ++r) dst[(xt * 16 + r) * 64] = acc[xt][r];
        dst[XT * 16 * 64] = bsum;
    };
    auto add = [&](int slot) {
        const float* src = red + (slot * VALS) * 64 + lane;
#pragma unroll
        for (int xt = 0; xt < XT; ++xt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[xt][r] += src[(xt * 16 + r) * 64];
        bsum += src[XT * 16 * 64];
    };
    __syncthreads();
    if (quarter >= 2) put((quarter - 2) * 3 + t);
    __syncthreads();
    if (quarter < 2) add(quarter * 3 + t);
    __syncthreads();
    if (quarter == 1) put(t);
    __syncthreads();
    if (quarter == 0) {
        add(t);
        float* pw = part_w + (int64_t)chunk * P * K + (int64_t)(g * 96 + t * 32) * K + l32;
#pragma unroll
        for (int xt = 0; xt < XT; ++xt)
#pragma unroll
            for (int r = 0; r < 16; ++r) pw[(int64_t)acc_row(r, half) * K + xt * 32] = acc[xt][r];
        bsum += __shfl_xor(bsum, 32);                                    // the two k groups of a column
        if (half == 0) part_b[(int64_t)chunk * P + ycol] = bsum;
    }
}

// out[e] = sum over chunks of part[chunk][e].  A block handles 16 x 4 consecutive outputs; 16 threads
// share an output quadruple, each adds every 16th chunk in order, and the 16 sums are added in a fixed
// tree.  part_w and part_b are contiguous ([chunks][PK] then [chunks][P]), so e runs over both.
__global__ __launch_bounds__(256) void tall_linear_wgrad_reduce_kernel(const float* __restrict__ part_w,
                                                                       const float* __restrict__ part_b, int chunks, int PK,
                                                                       int P, int K, float* __restrict__ dw, int dw_pitch,
                                                                       float* __restrict__ db) {
    __shared__ tl_f32x4 sums[16][17];
    const int el = threadIdx.x & 15, cl = threadIdx.x >> 4;
    const int e = (blockIdx.x * 16 + el) * 4;
    const bool weight = e < PK, valid = weight || (db && e - PK < P);
    tl_f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    if (valid) {
        const float* src = weight ? part_w + e : part_b + (e - PK);
        const int64_t pitch = weight ? PK : P;
        for (int c = cl; c < chunks; c += 16) sum += *reinterpret_cast<const tl_f32x4*>(src + c * pitch);
    }
    sums[cl][el] = sum;
    __syncthreads();
#pragma unroll
    for (int w = 8; w >= 1; w >>= 1) {
        if (cl < w) sums[cl][el] += sums[cl + w][el];
        __syncthreads();
    }
    if (cl == 0 && valid)                                                // dw: this pass's K columns of rows of dw_pitch
        *reinterpret_cast<tl_f32x4*>(weight ? dw + (int64_t)(e / K) * dw_pitch + e % K : db + (e - PK)) = sums[0][el];
}

}  // namespace sswin

using namespace sswin;

static int staged_lds_bytes(int ksteps) {
    return ksteps * 9 * 64 * (int)sizeof(tl_u32x4) + 8 * 32 * (ksteps * 16 + 4) * (int)sizeof(float);
}

static int device_cus() {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
        n > 0)
        return n;
    return 256;
}

template <bool TRANSPOSED>
static int launch_chunked(const float* x, int64_t N, int in, const float* w, const float* bias, int out, float* y, int cus,
                          hipStream_t s, const char* what) {
    if (in / 16 <= WIDE_MAX_KS) {                                        // all of W stays on the CU
        const int lds_ks = std::min(in / 16, WIDE_LDS_KS);
        const size_t lds = (size_t)lds_ks * 9 * 64 * sizeof(tl_u32x4);
        static bool configured_wide = false;
        if (!configured_wide) {
            SSWIN_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(tall_linear_wide_kernel<TRANSPOSED>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize,
                                          WIDE_LDS_KS * 9 * 64 * (int)sizeof(tl_u32x4)));
            configured_wide = true;
        }
        const int groups = out / TL_COLS;
        const int64_t row_tiles = (N + 31) / 32;
        const int64_t per_group = std::min<int64_t>((row_tiles + 7) / 8, std::max<int64_t>(1, cus / groups));
        hipLaunchKernelGGL(tall_linear_wide_kernel<TRANSPOSED>, dim3((unsigned)(per_group * groups)), dim3(512), lds, s, x, N, in,
                           w, groups, bias, y, out, row_tiles);
        return launch_ok(what);
    }
    const size_t lds = 2 * (size_t)CH_KS * 9 * 64 * sizeof(tl_u32x4);
    static bool configured = false;
    if (!configured) {
        SSWIN_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(tall_linear_chunked_kernel<TRANSPOSED>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        configured = true;
    }
    const int groups = out / TL_COLS;
    const int64_t row_tiles = (N + 31) / 32;
    const int64_t per_group = std::min<int64_t>((row_tiles + 7) / 8, std::max<int64_t>(1, cus / groups));
    hipLaunchKernelGGL(tall_linear_chunked_kernel<TRANSPOSED>, dim3((unsigned)(per_group * groups)), dim3(512), lds, s, x, N, in, w,
                       groups, bias, y, out, row_tiles);
    return launch_ok(what);
}

extern "C" {

int sswin_tall_linear_input_grad_supported(int P, int K) {
    return P > 0 && K > 0 && (P % 96) == 0 && (K % TL_COLS) == 0;
}

int sswin_tall_linear_input_grad(const float* dy, int64_t N, int P, const float* w, int K, float* dx, void* stream) {
    SSWIN_CHECK(N >= 0 && K > 0 && P > 0, "tall_linear_input_grad: bad sizes");
    SSWIN_CHECK(P % 96 == 0, "tall_linear_input_grad: %d output channels are not a multiple of 96", P);
    SSWIN_CHECK(K % TL_COLS == 0, "tall_linear_input_grad: %d input channels are not a multiple of %d", K, TL_COLS);
    if (N == 0) return 0;
    SSWIN_CHECK(dy && w && dx, "tall_linear_input_grad: null pointer");
    SSWIN_CHECK(((uintptr_t)dy % 16) == 0, "tall_linear_input_grad: dy must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int cus = device_cus();
    if (P == 96 && N >= 32) {
        // 96 channels of dY: the staged kernel of the forward with W read transposed
        SSWIN_CHECK(((uintptr_t)w % 16) == 0, "tall_linear_input_grad: w must be 16-byte aligned");
        static bool configured = false;
        if (!configured) {
            SSWIN_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<6, false, true>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, staged_lds_bytes(6)));
            configured = true;
        }
        const int groups = K / TL_COLS;
        const int64_t row_tiles = (N + 31) / 32;
        const int64_t per_group = std::min<int64_t>((row_tiles + 7) / 8, std::max<int64_t>(1, cus / groups));
        hipLaunchKernelGGL((tall_linear_forward_staged_kernel<6, false, true>), dim3((unsigned)(per_group * groups)), dim3(512),
                           staged_lds_bytes(6), s, dy, N, w, groups, static_cast<const float*>(nullptr), dx, K, row_tiles);
        return launch_ok("tall_linear_input_grad");
    }
    return launch_chunked<true>(dy, N, P, w, nullptr, K, dx, cus, s, "tall_linear_input_grad");
}

int sswin_tall_linear_supported(int P, int K) {
    return P > 0 && K > 0 && (P % TL_COLS) == 0 && (K % 16) == 0 && (K <= TL_MAX_K || ((K % 96) == 0 && K <= 768));
}

int sswin_tall_linear_forward(const float* x, int64_t N, int K, const float* w, const float* bias, int P, float* y,
                              void* stream) {
    SSWIN_CHECK(N >= 0 && K > 0 && P > 0, "tall_linear_forward: bad sizes");
    SSWIN_CHECK(K % 16 == 0 && (K <= TL_MAX_K || (K % 96 == 0 && K <= 768)),
                "tall_linear_forward: %d input channels are not supported (a multiple of 16 up to %d, or of 96 up to 768)", K,
                TL_MAX_K);
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
        const void* staged[] = {reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<1, false>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<2, false>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<3, false>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<4, false>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<5, false>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<6, false>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<1, true>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<2, true>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<3, true>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<4, true>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<5, true>),
                                reinterpret_cast<const void*>(tall_linear_forward_staged_kernel<6, true>)};
        for (int q = 0; q < 12; ++q)
            SSWIN_HIP(hipFuncSetAttribute(staged[q], hipFuncAttributeMaxDynamicSharedMemorySize, staged_lds_bytes(q % 6 + 1)));
        configured = true;
    }
    if (ksteps <= TL_STAGED_MAX_KS) {
        const int64_t row_tiles = (N + 31) / 32;
        const int64_t per_group = std::min<int64_t>((row_tiles + 7) / 8, std::max<int64_t>(1, cus / groups));
        const dim3 grid((unsigned)(per_group * groups)), block(512);
        const size_t lds = staged_lds_bytes(ksteps);
#define SSWIN_TL_STAGED(KS)                                                                                                  \
    case KS:                                                                                                                 \
        if (N < 32)                                                                                                          \
            hipLaunchKernelGGL((tall_linear_forward_staged_kernel<KS, true>), grid, block, lds, s, x, N, w, groups, bias, y, \
                               P, row_tiles);                                                                                \
        else                                                                                                                 \
            hipLaunchKernelGGL((tall_linear_forward_staged_kernel<KS, false>), grid, block, lds, s, x, N, w, groups, bias,   \
                               y, P, row_tiles);                                                                             \
        break;
        switch (ksteps) {
            SSWIN_TL_STAGED(1) SSWIN_TL_STAGED(2) SSWIN_TL_STAGED(3) SSWIN_TL_STAGED(4) SSWIN_TL_STAGED(5) SSWIN_TL_STAGED(6)
        }
#undef SSWIN_TL_STAGED
        return launch_ok("tall_linear_forward");
    }
    if (K > TL_MAX_K) return launch_chunked<false>(x, N, K, w, bias, P, y, cus, s, "tall_linear_forward");
    const size_t lds = (size_t)ksteps * 9 * 64 * sizeof(tl_u32x4);
    const int64_t row_blocks = (N + 127) / 128;
    const int per_cu = lds <= 64 * 1024 ? 2 : 1;                          // workgroups that fit a CU's LDS
    int64_t per_group = std::min<int64_t>(row_blocks, std::max<int64_t>(1, (int64_t)cus * per_cu / groups));
    hipLaunchKernelGGL(tall_linear_forward_kernel, dim3((unsigned)(per_group * groups)), dim3(256), lds, s, x, N, K, w, groups,
                       bias, y, P, row_blocks);
    return launch_ok("tall_linear_forward");
}

}  // extern "C"

static void wgrad_split(int64_t N, int groups, int cus, int64_t* rows_per_chunk, int* chunks) {
    const int64_t want = std::max<int64_t>(1, cus / groups);
    int64_t rows = (N + want - 1) / want;
    rows = std::max<int64_t>(WG_STEP_ROWS, (rows + WG_STEP_ROWS - 1) / WG_STEP_ROWS * WG_STEP_ROWS);
    *rows_per_chunk = rows;
    *chunks = (int)std::max<int64_t>(1, (N + rows - 1) / rows);
}

extern "C" {

static bool wgrad_shape_ok(int P, int K) {
    // up to 96 input channels in one pass, more in passes of 96
    return P > 0 && K > 0 && (P % 96) == 0 && (K % 32) == 0 && (K <= 96 || ((K % 96) == 0 && K <= 768));
}

size_t sswin_tall_linear_weight_grad_workspace_bytes(int64_t N, int P, int K) {
    if (N <= 0 || !wgrad_shape_ok(P, K)) return 0;
    int64_t rows;
    int chunks;
    wgrad_split(N, P / 96, device_cus(), &rows, &chunks);
    const int kp = std::min(K, 96);
    return (size_t)chunks * ((size_t)P * kp + P) * sizeof(float) + 256;
}

int sswin_tall_linear_weight_grad(const float* dy, const float* x, int64_t N, int P, int K, float* dw, float* db, void* ws,
                                  size_t ws_bytes, void* stream) {
    SSWIN_CHECK(N > 0 && P > 0 && K > 0, "tall_linear_weight_grad: bad sizes");
    SSWIN_CHECK(P % 96 == 0, "tall_linear_weight_grad: %d output channels are not a multiple of 96", P);
    SSWIN_CHECK(wgrad_shape_ok(P, K),
                "tall_linear_weight_grad: %d input channels are not supported (32, 64, 96 or a multiple of 96 up to 768)", K);
    SSWIN_CHECK(dy && x && dw && ws, "tall_linear_weight_grad: null pointer");
    SSWIN_CHECK(((uintptr_t)dw % 16) == 0 && ((uintptr_t)db % 16) == 0 && ((uintptr_t)ws % 16) == 0,
                "tall_linear_weight_grad: dw, db and the workspace must be 16-byte aligned");
    SSWIN_CHECK(ws_bytes >= sswin_tall_linear_weight_grad_workspace_bytes(N, P, K), "tall_linear_weight_grad: workspace too small");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int groups = P / 96, kp = std::min(K, 96), xt = kp / 32, passes = K / kp;
    int64_t rows;
    int chunks;
    wgrad_split(N, groups, device_cus(), &rows, &chunks);
    float* part_w = static_cast<float*>(ws);
    float* part_b = part_w + (size_t)chunks * P * kp;
    // LDS: the double-buffered planes of X, or the two rounds of the final sums, whichever is larger
    const size_t planes = 2 * (size_t)WG_QUARTERS * xt * 3 * 64 * sizeof(tl_u32x4);
    const size_t sums = 6 * (size_t)(xt * 16 + 1) * 64 * sizeof(float);
    const size_t lds = std::max(planes, sums);
    static bool configured = false;
    if (!configured) {
        const int max_lds = 96 * 1024;
        const void* all[] = {reinterpret_cast<const void*>(tall_linear_wgrad_kernel<1, false>),
                             reinterpret_cast<const void*>(tall_linear_wgrad_kernel<2, false>),
                             reinterpret_cast<const void*>(tall_linear_wgrad_kernel<3, false>),
                             reinterpret_cast<const void*>(tall_linear_wgrad_kernel<3, true>),
                             reinterpret_cast<const void*>(tall_linear_wgrad_kernel<3, false, 96>),
                             reinterpret_cast<const void*>(tall_linear_wgrad_kernel<3, false, 288>)};
        for (const void* k : all) SSWIN_HIP(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, max_lds));
        configured = true;
    }
    const dim3 grid((unsigned)(chunks * groups)), block(WG_WAVES * 64);
    const int PK = P * kp, total4 = (PK + P) / 4;
    // one pass per 96 columns of X: the partial buffer is reused, the column sums of dy come from the first
    for (int pass = 0; pass < passes; ++pass) {
        const float* xp = x + pass * kp;
        if (passes > 1)
            hipLaunchKernelGGL((tall_linear_wgrad_kernel<3, true>), grid, block, lds, s, dy, xp, K, N, P, groups, rows, part_w, part_b);
        else if (xt == 1)
            hipLaunchKernelGGL((tall_linear_wgrad_kernel<1, false>), grid, block, lds, s, dy, xp, K, N, P, groups, rows, part_w, part_b);
        else if (xt == 2)
            hipLaunchKernelGGL((tall_linear_wgrad_kernel<2, false>), grid, block, lds, s, dy, xp, K, N, P, groups, rows, part_w, part_b);
        else if (P == 96)
            hipLaunchKernelGGL((tall_linear_wgrad_kernel<3, false, 96>), grid, block, lds, s, dy, xp, K, N, P, groups, rows, part_w, part_b);
        else if (P == 288)
            hipLaunchKernelGGL((tall_linear_wgrad_kernel<3, false, 288>), grid, block, lds, s, dy, xp, K, N, P, groups, rows, part_w, part_b);
        else
            hipLaunchKernelGGL((tall_linear_wgrad_kernel<3, false>), grid, block, lds, s, dy, xp, K, N, P, groups, rows, part_w, part_b);
        if (int rc = launch_ok("tall_linear_weight_grad")) return rc;
        hipLaunchKernelGGL(tall_linear_wgrad_reduce_kernel, dim3((unsigned)((total4 + 15) / 16)), dim3(256), 0, s, part_w, part_b,
                           chunks, PK, P, kp, dw + pass * kp, K, pass == 0 ? db : nullptr);
        if (int rc = launch_ok("tall_linear_weight_grad reduce")) return rc;
    }
    return 0;
}

}  // extern "C"
