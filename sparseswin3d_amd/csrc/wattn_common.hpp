// Pieces shared by the window-resident attention kernels (gfx950, wave64): task lookup, 32-bit token
// addressing, wave-private LDS tiles and tables, coalesced row loads and stores.
#pragma once

#include <math.h>
#include <stdint.h>

#include <type_traits>

#include "mfma_block.hpp"
#include "sswin_common.hpp"

namespace sswin {

struct TokenTensor32 {      // rows addressed by voxel, columns col0 + h*32 + ch
    const void* base;
    int64_t stride;
    int col0;
};

struct WAttnCommon {
    const int4* tasks;      // [4][g_cap] descriptors {T, c | head << 8, window, sq_start} by bucket
    int64_t g_cap;
    int64_t first[5];       // first task id of bucket 3, 2, 1, 0 (heaviest first) and the task total
    const int32_t* order;   // voxel of token rank r
    const int32_t* tok_pos; // position inside the window of token rank r
    const int2* recs;       // token records: [record][32] {voxel, pos}, a record per (window, tile), in task order
    int64_t rec_first[4];   // first record of bucket 3, 2, 1, 0
    int H, n;
    float scale;
    const float* bias;      // [H, n, n]
    const int8_t* mask;     // [nmw, n] region ids or null
    int nmw;
};

struct GroupCtx {
    int Tk, c, h, w, sq;
};

// task id -> (group descriptor, 32-row block inside the group, token record of that block); false past the last task.
// Nothing is read from memory: the descriptor and the records of the group's tiles (rec - blk + t) can be requested
// together.
__device__ __forceinline__ bool locate(const WAttnCommon& a, int64_t task, int64_t& d, int& blk, int64_t& rec) {
    if (task >= a.first[4]) return false;
    int q = 0;                                   // 0 = bucket 3 (four tiles) ... 3 = bucket 0 (one tile)
#pragma unroll
    for (int k = 1; k < 4; ++k) q += task >= a.first[k] ? 1 : 0;
    const int nt = 4 - q;
    const uint32_t local = (uint32_t)(task - a.first[q]);
    const uint32_t grp = local / (uint32_t)nt;   // the bucket's groups: H per window, windows in window order
    blk = (int)(local - grp * (uint32_t)nt);
    d = (int64_t)(nt - 1) * a.g_cap + grp;
    rec = a.rec_first[q] + (int64_t)(grp / (uint32_t)a.H) * nt + blk;
    return true;
}
// entry l32 of a token record: .x = voxel, .y = position inside the window
__device__ __forceinline__ int2 token_entry(const WAttnCommon& a, int64_t rec, int l32) { return a.recs[rec * 32 + l32]; }

__device__ __forceinline__ GroupCtx load_group(const int4* __restrict__ tasks, int64_t d) {
    const int4 t = tasks[d];
    GroupCtx g;
    g.Tk = __builtin_amdgcn_readfirstlane(t.x);
    g.c = __builtin_amdgcn_readfirstlane(t.y & 0xff);
    g.h = __builtin_amdgcn_readfirstlane(t.y >> 8);
    g.w = __builtin_amdgcn_readfirstlane(t.z);
    g.sq = __builtin_amdgcn_readfirstlane(t.w);
    return g;
}

// ------------------------------------------------------------------------------------------
// Addressing.  Every token tensor is reached as  uniform byte base (tensor base + head columns)
// + 32-bit byte offset of the row: one full-rate 24-bit multiply per token and no 64-bit vector
// arithmetic.  The host checks that row offsets fit 32 bits and that rows are 16-byte aligned.
// ------------------------------------------------------------------------------------------
typedef float f32x4_a __attribute__((ext_vector_type(4)));               // naturally aligned
typedef uint32_t u32x4_a __attribute__((ext_vector_type(4)));

constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

template <typename T>
__device__ __forceinline__ const char* head_base(const TokenTensor32& t, int h) {
    return static_cast<const char*>(t.base) + (int64_t)(t.col0 + h * 32) * sizeof(T);
}
template <typename T>
__device__ __forceinline__ uint32_t pitch_of(const TokenTensor32& t) { return (uint32_t)t.stride * (uint32_t)sizeof(T); }

__device__ __forceinline__ void unpack2(uint32_t u, float& lo, float& hi, __half) {
    const __half2 h2 = __builtin_bit_cast(__half2, u);
    lo = __low2float(h2);
    hi = __high2float(h2);
}
__device__ __forceinline__ void unpack2(uint32_t u, float& lo, float& hi, __hip_bfloat16) {
    lo = __builtin_bit_cast(float, u << 16);
    hi = __builtin_bit_cast(float, u & 0xffff0000u);
}
__device__ __forceinline__ uint32_t pack2(float lo, float hi, __half) {
    return __builtin_bit_cast(uint32_t, __floats2half2_rn(lo, hi));
}
__device__ __forceinline__ uint32_t pack2(float lo, float hi, __hip_bfloat16) {
    const uint32_t a = __builtin_bit_cast(uint16_t, __float2bfloat16(lo));
    const uint32_t b = __builtin_bit_cast(uint16_t, __float2bfloat16(hi));
    return a | (b << 16);
}

// ------------------------------------------------------------------------------------------
// Wave-private LDS.  A "tile" holds 32 token rows of 32 fp32 channels at a pitch of 36 dwords
// (16-byte rows stay aligned, and 16-byte accesses of neighbouring rows fall into different
// banks); it turns the row-major global loads into the column-major MFMA operand of the second
// product and the accumulators back into rows for wide stores.  A "table" holds one 32-bit value
// per token of the tile; the 16 entries a lane needs (rows acc_row(r, half)) are four runs of
// four, fetched with four 16-byte reads.  Only the owning wavefront touches its tiles and tables;
// LDS operations of one wavefront execute in order, so no barrier is involved.
// ------------------------------------------------------------------------------------------
constexpr int TILE_LD = 36;
constexpr int TILE_WORDS = 32 * TILE_LD;

__device__ __forceinline__ void tile_put_rows(float* tile, int l32, int half, const float (&x)[16]) {
    f32x4_a* p = reinterpret_cast<f32x4_a*>(tile + l32 * TILE_LD + half * 16);
#pragma unroll
    for (int v = 0; v < 4; ++v) p[v] = f32x4_a{x[4 * v], x[4 * v + 1], x[4 * v + 2], x[4 * v + 3]};
}
__device__ __forceinline__ void tile_get_rows(const float* tile, int l32, int half, float (&x)[16]) {
    const f32x4_a* p = reinterpret_cast<const f32x4_a*>(tile + l32 * TILE_LD + half * 16);
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const f32x4_a t = p[v];
        x[4 * v] = t.x; x[4 * v + 1] = t.y; x[4 * v + 2] = t.z; x[4 * v + 3] = t.w;
    }
}
// x[r] = tile[row acc_row(r, half)][column l32]
__device__ __forceinline__ void tile_get_cols(const float* tile, int l32, int half, float (&x)[16]) {
    const float* p = tile + 4 * half * TILE_LD + l32;
#pragma unroll
    for (int r = 0; r < 16; ++r) x[r] = p[(8 * (r >> 2) + (r & 3)) * TILE_LD];
}
__device__ __forceinline__ void tile_put_acc(float* tile, int l32, int half, const f32x16& acc) {
    float* p = tile + 4 * half * TILE_LD + l32;
#pragma unroll
    for (int r = 0; r < 16; ++r) p[(8 * (r >> 2) + (r & 3)) * TILE_LD] = acc[r];
}
__device__ __forceinline__ void table_put(uint32_t* tab, int l32, uint32_t v) { tab[l32] = v; }
__device__ __forceinline__ void table_get(const uint32_t* tab, int half, uint32_t (&x)[16]) {
    const u32x4_a* p = reinterpret_cast<const u32x4_a*>(tab + 4 * half);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const u32x4_a t = p[2 * q];
        x[4 * q] = t.x; x[4 * q + 1] = t.y; x[4 * q + 2] = t.z; x[4 * q + 3] = t.w;
    }
}
// A table kept in the spare columns of a tile: rows are 36 dwords wide and only 32 of them carry
// values, so the four spare dwords of eight consecutive rows hold 32 entries, entries 4k .. 4k+3
// in row k.  A tile has room for four such tables (rows 0-7, 8-15, 16-23, 24-31); the 16-byte
// reads of table_get fall on whole rows' spare columns.  The backward kernels keep their tables
// there, which leaves LDS for the exchange tiles of the two-tile groups.
struct PadTab {
    uint32_t* p;
    __device__ __forceinline__ void put(int e, uint32_t v) const { p[(e >> 2) * TILE_LD + (e & 3)] = v; }
    __device__ __forceinline__ uint32_t get(int e) const { return p[(e >> 2) * TILE_LD + (e & 3)]; }
    __device__ __forceinline__ u32x4_a chunk(int ch) const { return *reinterpret_cast<const u32x4_a*>(p + ch * TILE_LD); }
};
__device__ __forceinline__ PadTab pad_tab(float* tile, int k) {
    return PadTab{reinterpret_cast<uint32_t*>(tile) + 8 * k * TILE_LD + 32};
}
__device__ __forceinline__ void table_put(const PadTab& tab, int l32, uint32_t v) { tab.put(l32, v); }
__device__ __forceinline__ void table_get(const PadTab& tab, int half, uint32_t (&x)[16]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const u32x4_a t = tab.chunk(2 * q + half);
        x[4 * q] = t.x; x[4 * q + 1] = t.y; x[4 * q + 2] = t.z; x[4 * q + 3] = t.w;
    }
}
__device__ __forceinline__ uint32_t f2u(float v) { return __builtin_bit_cast(uint32_t, v); }
__device__ __forceinline__ float u2f(uint32_t v) { return __builtin_bit_cast(float, v); }
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// ------------------------------------------------------------------------------------------
// One MFMA product step over the reduction slots a lane holds.  fp32 tokens: one
// v_mfma_f32_32x32x2_f32 per slot (the lane pair l, l + 32 supplies k = 2 values).  16-bit tokens:
// the operands are rounded to the token type and eight slots go into one v_mfma_f32_32x32x16
// (k = 16: eight slots of lanes 0-31, eight of lanes 32-63) - an eighth of the matrix-core
// passes.  A and B use the same slot -> reduction index mapping, which is all a product needs.
// ------------------------------------------------------------------------------------------
template <typename T> struct LowPrec;
template <> struct LowPrec<__hip_bfloat16> {
    typedef __bf16 elem;
    typedef __bf16 vec __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ f32x16 mma(vec a, vec b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct LowPrec<__half> {
    typedef _Float16 elem;
    typedef _Float16 vec __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ f32x16 mma(vec a, vec b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};
// the same, starting from the instruction's zero operand instead of a cleared accumulator
template <typename T, int N, typename A, typename B>
__device__ __forceinline__ f32x16 mma_slots_first(const A& a, const B& b) {
    const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    f32x16 acc;
    if constexpr (std::is_same<T, float>::value) {
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b[0], zero, 0, 0, 0);
#pragma unroll
        for (int s = 1; s < N; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[s], acc, 0, 0, 0);
    } else {
        typename LowPrec<T>::vec va, vb;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            va[i] = (typename LowPrec<T>::elem)a[i];
            vb[i] = (typename LowPrec<T>::elem)b[i];
        }
        acc = LowPrec<T>::mma(va, vb, zero);
#pragma unroll
        for (int m = 1; m < N / 8; ++m) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                va[i] = (typename LowPrec<T>::elem)a[8 * m + i];
                vb[i] = (typename LowPrec<T>::elem)b[8 * m + i];
            }
            acc = LowPrec<T>::mma(va, vb, acc);
        }
    }
    return acc;
}
// eight slots: a[OFF .. OFF + 8) against b[0 .. 8)
template <typename T, int OFF, typename A, typename B>
__device__ __forceinline__ void mma_slots8_off(const A& a, const B& b, f32x16& acc) {
    typename LowPrec<T>::vec va, vb;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        va[i] = (typename LowPrec<T>::elem)a[OFF + i];
        vb[i] = (typename LowPrec<T>::elem)b[i];
    }
    acc = LowPrec<T>::mma(va, vb, acc);
}
template <typename T, int OFF, int N, typename A, typename B>
__device__ __forceinline__ void mma_slots(const A& a, const B& b, f32x16& acc) {
    if constexpr (std::is_same<T, float>::value) {
#pragma unroll
        for (int s = 0; s < N; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[OFF + s], b[OFF + s], acc, 0, 0, 0);
    } else {
        static_assert(N % 8 == 0, "16-bit products take eight slots per step");
#pragma unroll
        for (int m = 0; m < N / 8; ++m) {
            typename LowPrec<T>::vec va, vb;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                va[i] = (typename LowPrec<T>::elem)a[OFF + 8 * m + i];
                vb[i] = (typename LowPrec<T>::elem)b[OFF + 8 * m + i];
            }
            acc = LowPrec<T>::mma(va, vb, acc);
        }
    }
}

// ------------------------------------------------------------------------------------------
// Coalesced token rows.  A head's slice of a token row is 32 channels = CH chunks of 16 bytes
// (8 for fp32, 4 for 16-bit values).  One load instruction fetches 64 / CH whole slices: lane l
// reads chunk l % CH of the row l / CH of its group, so the lanes of a slice read one contiguous
// 128- or 64-byte piece and the memory pipeline sees a quarter of the requests a row-per-lane
// load makes.  The pieces are turned into the row-per-lane MFMA operand through an LDS tile.
// ------------------------------------------------------------------------------------------
template <typename T>
struct RowLoad {
    static constexpr int CH = 32 * (int)sizeof(T) / 16;      // chunks per row slice
    static constexpr int ROWS = 64 / CH;                     // rows per instruction
    static constexpr int NI = 32 / ROWS;                     // instructions per 32 rows
    u32x4_a v[NI];
};

// vox_lane: voxel of row l32, held by lanes l32 and l32 + 32
// STREAM: the rows belong to a group of one tile, so no other task reads them: loaded with the streaming hint (the
// key-side task of one-tile groups in the backward: 0.1203 -> 0.1187 ms on cfg2, 0.096 -> 0.095 on cfg3).  Rows of
// larger groups are read by up to eight tasks and must stay cached: with the hint on all loads the bf16 backward of
// 100-125-token windows went from 0.097 to 0.156 ms and the forward from 0.049 to 0.062; in the forward the hint for
// one-tile groups alone was no gain either (cfg2 0.0568 against 0.0572 ms, cfg3 0.0441 against 0.0425).
template <typename T, bool STREAM = false>
__device__ __forceinline__ void rows_load(const char* __restrict__ base, uint32_t pitch, uint32_t vox_lane, int lane,
                                          RowLoad<T>& r) {
    constexpr int CH = RowLoad<T>::CH, ROWS = RowLoad<T>::ROWS;
#pragma unroll
    for (int v = 0; v < RowLoad<T>::NI; ++v) {
        const uint32_t vox = (uint32_t)__shfl((int)vox_lane, v * ROWS + lane / CH, 64);
        const u32x4_a* p = reinterpret_cast<const u32x4_a*>(base + (__umul24(vox, pitch) + (uint32_t)(lane % CH) * 16u));
        r.v[v] = STREAM ? __builtin_nontemporal_load(p) : *p;
    }
}
template <typename T>
__device__ __forceinline__ void rows_to_tile(float* tile, int lane, const RowLoad<T>& r);
template <>
__device__ __forceinline__ void rows_to_tile<float>(float* tile, int lane, const RowLoad<float>& r) {
#pragma unroll
    for (int v = 0; v < RowLoad<float>::NI; ++v)
        *reinterpret_cast<u32x4_a*>(tile + (v * 8 + lane / 8) * TILE_LD + (lane % 8) * 4) = r.v[v];
}
template <typename T>
__device__ __forceinline__ void rows_to_tile(float* tile, int lane, const RowLoad<T>& r) {
#pragma unroll
    for (int v = 0; v < RowLoad<T>::NI; ++v) {
        float x[8];
        unpack2(r.v[v].x, x[0], x[1], T());
        unpack2(r.v[v].y, x[2], x[3], T());
        unpack2(r.v[v].z, x[4], x[5], T());
        unpack2(r.v[v].w, x[6], x[7], T());
        f32x4_a* p = reinterpret_cast<f32x4_a*>(tile + (v * 16 + lane / 4) * TILE_LD + (lane % 4) * 8);
        p[0] = f32x4_a{x[0], x[1], x[2], x[3]};
        p[1] = f32x4_a{x[4], x[5], x[6], x[7]};
    }
}
// tile rows -> global rows, the same lane assignment; rows at or beyond `rows` are padding
template <typename T>
__device__ __forceinline__ void tile_store_rows(const float* tile, char* __restrict__ base, uint32_t pitch,
                                                uint32_t vox_lane, int rows, int lane);
template <>
__device__ __forceinline__ void tile_store_rows<float>(const float* tile, char* __restrict__ base, uint32_t pitch,
                                                       uint32_t vox_lane, int rows, int lane) {
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int R = v * 8 + lane / 8;
        const uint32_t vox = (uint32_t)__shfl((int)vox_lane, R, 64);
        const u32x4_a x = *reinterpret_cast<const u32x4_a*>(tile + R * TILE_LD + (lane % 8) * 4);
        if (R < rows) *reinterpret_cast<u32x4_a*>(base + (__umul24(vox, pitch) + (uint32_t)(lane % 8) * 16u)) = x;
    }
}
template <typename T>
__device__ __forceinline__ void tile_store_rows(const float* tile, char* __restrict__ base, uint32_t pitch,
                                                uint32_t vox_lane, int rows, int lane) {
#pragma unroll
    for (int v = 0; v < 2; ++v) {
        const int R = v * 16 + lane / 4;
        const uint32_t vox = (uint32_t)__shfl((int)vox_lane, R, 64);
        const f32x4_a* p = reinterpret_cast<const f32x4_a*>(tile + R * TILE_LD + (lane % 4) * 8);
        const f32x4_a lo = p[0], hi = p[1];
        const u32x4_a x = {pack2(lo.x, lo.y, T()), pack2(lo.z, lo.w, T()), pack2(hi.x, hi.y, T()), pack2(hi.z, hi.w, T())};
        if (R < rows) *reinterpret_cast<u32x4_a*>(base + (__umul24(vox, pitch) + (uint32_t)(lane % 4) * 16u)) = x;
    }
}

// table[row] = x_row . y_row for the 32 rows two loads hold: per-chunk dot products, summed over
// the CH lanes of a row by DPP steps inside groups of 4 and 8 lanes
template <typename T>
__device__ __forceinline__ float chunk_dot(const u32x4_a& x, const u32x4_a& y);
template <>
__device__ __forceinline__ float chunk_dot<float>(const u32x4_a& x, const u32x4_a& y) {
    float d = u2f(x.x) * u2f(y.x);
    d = fmaf(u2f(x.y), u2f(y.y), d);
    d = fmaf(u2f(x.z), u2f(y.z), d);
    return fmaf(u2f(x.w), u2f(y.w), d);
}
template <typename T>
__device__ __forceinline__ float chunk_dot(const u32x4_a& x, const u32x4_a& y) {
    const uint32_t xs[4] = {x.x, x.y, x.z, x.w}, ys[4] = {y.x, y.y, y.z, y.w};
    float d = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        float a0, a1, b0, b1;
        unpack2(xs[k], a0, a1, T());
        unpack2(ys[k], b0, b1, T());
        d = fmaf(a0, b0, d);
        d = fmaf(a1, b1, d);
    }
    return d;
}
template <typename T>
__device__ __forceinline__ void rows_dot_to_table(const PadTab& tab, int lane, const RowLoad<T>& x, const RowLoad<T>& y) {
    constexpr int CH = RowLoad<T>::CH, ROWS = RowLoad<T>::ROWS;
#pragma unroll
    for (int v = 0; v < RowLoad<T>::NI; ++v) {
        float d = chunk_dot<T>(x.v[v], y.v[v]);
        d += dpp_f32<0xB1>(d);                               // lanes 0..3 of a quad
        d += dpp_f32<0x4E>(d);
        if (CH == 8) d += dpp_f32<0x141>(d);                 // the two quads of 8 lanes
        if (lane % CH == 0) tab.put(v * ROWS + lane / CH, f2u(d));
    }
}

// The whole backward in one launch.  Workgroups (four wavefronts, one task each) are numbered through
// four segments, each starting at a workgroup boundary:
//   1. query-side tasks of the groups of three and four tiles
//   2. their key-side tasks (KV_ONLY); 1 and 2 are interleaved in runs of eight workgroups (see the kernel)
//   3. key-side tasks of the groups of two tiles, the two tasks of a group side by side (KV_PAIR)
//   4. key-side tasks of the groups of one tile (KV_SINGLE)
// Heaviest tasks first, so the long ones start first and the short ones fill the tail.
// Workgroups are dealt to the eight XCDs round robin: workgroup b runs on XCD b % 8, and every XCD has an L2 of its own.
// xcd_run_order turns the workgroup number into a work number such that every XCD takes whole runs of XCD_RUN consecutive
// work numbers, one after the other: neighbours in the work order (the heads of a window, the two sides of a group) run on
// one XCD at about the same time and share what they read.  With 16-bit tokens the 64-byte slices of two heads of a
// token share a 128-byte line: dealt to different XCDs, every line leaves memory twice (measured on 24 heads of bf16
// tokens: 176 MB read for 62 MB of rows).  The launch holds xcd_run_grid(n) workgroups; work numbers >= n do nothing.
constexpr int XCD_RUN = 16;
__device__ __forceinline__ int64_t xcd_run_order(int64_t b) {
    const int64_t k = b >> 3;
    return ((k / XCD_RUN) * 8 + (b & 7)) * XCD_RUN + k % XCD_RUN;
}
inline int64_t xcd_run_grid(int64_t n) { return (n + 8 * XCD_RUN - 1) / (8 * XCD_RUN) * (8 * XCD_RUN); }

struct BwdSegments {
    int64_t wg_kv, wg_pair, wg_single;   // first workgroup of segments 2, 3, 4
    int64_t n_big;                       // tasks per side of the groups of three and four tiles
    int64_t n_pair;                      // key-side tasks of the groups of two tiles (even)
    int64_t wgs;                         // workgroups of the launch
};
// pairs: segments 1 and 2 interleaved workgroup by workgroup (work order of xcd_run_order) instead of in runs of eight
inline BwdSegments make_segments(const WAttnCommon& a, bool pairs = false) {
    BwdSegments sg;
    sg.n_big = a.first[2];
    sg.n_pair = a.first[3] - a.first[2];
    const int64_t n_single = a.first[4] - a.first[3];
    const int64_t wg_big = (sg.n_big + 3) / 4;
    sg.wg_kv = wg_big;
    sg.wg_pair = pairs ? 2 * wg_big : 16 * ((wg_big + 7) / 8);   // both sides, interleaved
    sg.wg_single = sg.wg_pair + (sg.n_pair + 3) / 4;
    sg.wgs = sg.wg_single + (n_single + 3) / 4;
    return sg;
}


}  // namespace sswin
