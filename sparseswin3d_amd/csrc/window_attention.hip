// Window-resident attention: forward and backward of one (window, head) group without ever
// materialising the attention matrix in HBM.
//
// The reference computes S = Q K^T as a COO product, runs a sparse softmax over it and multiplies
// by V in a second COO product (sparse_swin/swin3d_base.py:660-672); its backward composes the
// gradient products and transposes (:119-134) with the softmax backward (ops.cu:169-194).  All of
// these exchange [c x c] blocks through memory.  A window holds at most 125 tokens, so a whole
// attention row fits into the registers of one wavefront:
//
//   forward    per (group, 32 queries): S^T tiles = K Q^T on MFMA, + bias + mask, softmax in
//              registers, O = P V with P fed to the MFMA straight from the accumulators;
//              writes O rows in voxel order and one log-sum-exp per attention row.
//   backward, query side, per (group, 32 queries): recomputes S^T, dP^T = V dO^T, dS = P (dP - D)
//              with D_i = dO_i . O_i, dQ = scale dS K.
//   backward, key side, per (group, 32 keys): recomputes S and dP = dO V^T in the other orientation,
//              dV = P^T dO, dK = scale dS^T Q; optionally stores dS for the bias gradient.  For a
//              group of at most 32 tokens it also produces dQ from the dS it already holds.
//   The whole backward is one launch: query-side tasks of the larger groups, then key-side tasks.
//
// Orientation trick: v_mfma_f32_32x32x2_f32 leaves output column l%32 in lane l and 16 rows in
// its registers.  Computing S transposed (keys as rows, queries as columns) puts a whole
// attention row into one lane pair (l, l+32): the softmax needs no cross-lane reduction beyond
// one exchange between the two halves, and accumulator register r of a lane is exactly the A
// operand of the P V product for the key pair (acc_row(r,0), acc_row(r,1)).
//
// Softmax semantics are the operator's (ops.cu:128-167): m = max(0, rowmax), y = e / (sum + 1e-8).
// Groups are bucketed by their number of 32-token tiles (1..4).  One launch covers all buckets:
// tasks (group, 32-row block) are numbered with the heaviest bucket first, so the long tasks start
// first and the short ones fill the tail; the loop over tiles is a run-time loop with a register
// budget that does not depend on the tile count.
//
// Global memory is touched in whole row slices only: eight (fp32) or four (16-bit) neighbouring
// lanes read or write the 128 or 64 contiguous bytes a head occupies in a token row, and a
// wave-private LDS tile turns these pieces into the row-per-lane MFMA operands (RowLoad,
// rows_to_tile, tile_store_rows).  A row-per-lane load would touch 64 different cache lines per
// instruction for 16 bytes each; the vector memory pipeline of a compute unit is shared by all
// its waves and was the busiest unit of these kernels before.
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
    int H, n;
    float scale;
    const float* bias;      // [H, n, n]
    const int8_t* mask;     // [nmw, n] region ids or null
    int nmw;
};

struct GroupCtx {
    int Tk, c, h, w, sq;
};

// task id -> (group descriptor, 32-row block inside the group); false past the last task
__device__ __forceinline__ bool locate(const WAttnCommon& a, int64_t task, int64_t& d, int& blk) {
    if (task >= a.first[4]) return false;
    int q = 0;                                   // 0 = bucket 3 (four tiles) ... 3 = bucket 0 (one tile)
#pragma unroll
    for (int k = 1; k < 4; ++k) q += task >= a.first[k] ? 1 : 0;
    const int nt = 4 - q;
    const int64_t local = task - a.first[q];
    const int64_t grp = local / nt;
    blk = (int)(local - grp * nt);
    d = (int64_t)(nt - 1) * a.g_cap + grp;
    return true;
}

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

// ------------------------------------------------------------------------------------------
// forward: rows = 32 queries of a group, tiles = its keys
// ------------------------------------------------------------------------------------------
// What a forward task needs before it can ask for token rows: its group, its block of 32 queries, and the
// voxels and window positions of its queries and of its first key tile.  Fetching them takes two dependent
// memory round trips (descriptor, then indices); they are fetched in one place so that a caller can fetch them ahead of the task.
struct KIdx {
    uint32_t vox;        // voxel of key t*32 + l32 (clamped to the last token)
    int pos;
};
struct FwdIdx {
    uint32_t vox_i;      // voxel of query bi*32 + l32 (clamped to the last token)
    int pos_i;
    KIdx k0;
};
__device__ __forceinline__ GroupCtx decode_group(const int4& t) {
    GroupCtx g;
    g.Tk = __builtin_amdgcn_readfirstlane(t.x);
    g.c = __builtin_amdgcn_readfirstlane(t.y & 0xff);
    g.h = __builtin_amdgcn_readfirstlane(t.y >> 8);
    g.w = __builtin_amdgcn_readfirstlane(t.z);
    g.sq = __builtin_amdgcn_readfirstlane(t.w);
    return g;
}
__device__ __forceinline__ FwdIdx fwd_indices(const WAttnCommon& a, const GroupCtx& g, int bi, int l32) {
    const int32_t* order = a.order + g.Tk;
    const int32_t* tok_pos = a.tok_pos + g.Tk;
    const int i_q = bi * 32 + l32;
    const int i_c = i_q < g.c ? i_q : g.c - 1;
    const int j_c = l32 < g.c ? l32 : g.c - 1;
    FwdIdx x;
    x.vox_i = order[i_c];
    x.pos_i = tok_pos[i_c];
    x.k0 = KIdx{(uint32_t)order[j_c], tok_pos[j_c]};
    return x;
}

// One forward task on one wavefront.  `mid` runs once between the last key tile and the write-out (a hook for
// work that should overlap the write-out; the plain kernel passes nothing).
template <typename T, bool MASK, typename Mid>
__device__ __forceinline__ void fwd_task(const WAttnCommon& a, const GroupCtx& g, const int bi, const FwdIdx& fi,
                                         float* tile, float* tile_x, uint32_t* tab_key, uint32_t* tab_alpha,
                                         const TokenTensor32& tq, const TokenTensor32& tk, const TokenTensor32& tv,
                                         const TokenTensor32& to, float* __restrict__ lse, Mid&& mid) {
    const int lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    const int c = g.c, h = g.h;
    const int nt = (c + 31) >> 5;
    const int32_t* order = a.order + g.Tk;
    const int32_t* tok_pos = a.tok_pos + g.Tk;
    const int8_t* mrow = MASK ? a.mask + (int64_t)(g.w % a.nmw) * a.n : nullptr;
    const char* qbase = head_base<T>(tq, h);
    const char* kbase = head_base<T>(tk, h);
    const char* vbase = head_base<T>(tv, h);
    const uint32_t qpitch = pitch_of<T>(tq), kpitch = pitch_of<T>(tk), vpitch = pitch_of<T>(tv);

    // query side: lane l32 owns query bi*32 + l32 (both halves), clamped to the last token
    const int i_q = bi * 32 + l32;
    const uint32_t vox_i = fi.vox_i;
    const int pos_i = fi.pos_i;
    // The memory round trips of a task depend on one another (descriptor -> token indices -> rows ->
    // bias) and a task is short, so the indices of the first key tile are requested together with the
    // query indices, and its K and V rows together with the Q rows.
    auto load_kidx = [&](const int t) {
        const int j = t * 32 + l32;
        const int j_c = j < c ? j : c - 1;
        return KIdx{(uint32_t)order[j_c], tok_pos[j_c]};
    };
    KIdx kcur = fi.k0;
    const int reg_i = MASK ? mrow[pos_i] : 0;
    RowLoad<T> rk, rv;
    float qb[16];
    {
        RowLoad<T> rq;
        rows_load<T>(qbase, qpitch, vox_i, lane, rq);
        rows_load<T>(kbase, kpitch, kcur.vox, lane, rk);
        rows_load<T>(vbase, vpitch, kcur.vox, lane, rv);
        __builtin_amdgcn_wave_barrier();
        rows_to_tile<T>(tile_x, lane, rq);
        __builtin_amdgcn_wave_barrier();
        tile_get_rows(tile_x, l32, half, qb);
    }
    const float qscale = a.scale * LOG2E;                    // scores are kept in units of log 2
#pragma unroll
    for (int s = 0; s < 16; ++s) qb[s] *= qscale;
    const char* bias_h = reinterpret_cast<const char*>(a.bias + (int64_t)h * a.n * a.n);
    const uint32_t brow = (uint32_t)(pos_i * a.n) * 4u;

    float m = 0.f;                                           // the operator's max(0, rowmax)
    float l = 0.f;                                           // this lane half's share of the row sum
    f32x16 o;
    // one tile of keys.  The first tile is a separate instantiation: its accumulators start from the
    // instruction's zero operand and nothing has to be rescaled (most groups have one tile only).
    // rk, rv hold the K and V rows of key tile t (requested by the caller), ki its indices.
    auto tile_step = [&](auto first_tag, const int t, const KIdx& ki) {
        constexpr bool FIRST = decltype(first_tag)::value;
        uint32_t pk = (uint32_t)ki.pos * 4u;
        if (MASK) pk |= (uint32_t)mrow[ki.pos] << 16;
        __builtin_amdgcn_wave_barrier();
        table_put(tab_key, l32, pk);
        rows_to_tile<T>(tile_x, lane, rk);
        rows_to_tile<T>(tile, lane, rv);
        __builtin_amdgcn_wave_barrier();
        // the bias gathers are requested before the score product, which covers part of their latency
        uint32_t pkr[16];
        table_get(tab_key, half, pkr);
        float bv[16];
#pragma unroll
        for (int r = 0; r < 16; ++r)
            bv[r] = *reinterpret_cast<const float*>(bias_h + (brow + (MASK ? (pkr[r] & 0xffffu) : pkr[r])));
        float ka[16];
        tile_get_rows(tile_x, l32, half, ka);
        // S^T tile: rows = keys, columns = queries
        f32x16 S = mma_slots_first<T, 16>(ka, qb);
        float vb[16];
        tile_get_cols(tile, l32, half, vb);                  // V[key acc_row(r, half)][channel l32]

        const int jlim = c - t * 32 - 4 * half;              // keys acc_row(r, 0) >= jlim are padding
        float mt = m;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float s = fmaf(bv[r], LOG2E, S[r]);
            if (MASK && (int)(pkr[r] >> 16) != reg_i) s += -100.0f * LOG2E;
            s = (8 * (r >> 2) + (r & 3)) < jlim ? s : -INFINITY;
            S[r] = s;
            mt = fmaxf(mt, s);
        }
        mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
        if constexpr (!FIRST) {                              // rescale what earlier tiles accumulated
            const float alpha = exp2_fast(m - mt);
            l *= alpha;
            table_put(tab_alpha, l32, f2u(alpha));
            __builtin_amdgcn_wave_barrier();
            uint32_t ar[16];
            table_get(tab_alpha, half, ar);
#pragma unroll
            for (int r = 0; r < 16; ++r) o[r] *= u2f(ar[r]);
        }
        m = mt;
        if constexpr (std::is_same<T, float>::value) {
            // P V by blocks of eight key rows (registers 4q .. 4q + 3 hold rows 8q + k and 8q + k + 4 of the two
            // lane halves): a block that lies wholly behind the last key is padding and is skipped, exponentials
            // and matrix steps alike (windows of 5^3 positions hold 20 to 30 tokens on average)
            const int kleft = c - t * 32;
            if constexpr (FIRST) o = f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (q > 0 && 8 * q >= kleft) break;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int r = 4 * q + k;
                    const float pr = exp2_fast(S[r] - m);
                    l += pr;
                    o = __builtin_amdgcn_mfma_f32_32x32x2f32(pr, vb[r], o, 0, 0, 0);
                }
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                S[r] = exp2_fast(S[r] - m);
                l += S[r];
            }
            if constexpr (FIRST)
                o = mma_slots_first<T, 16>(S, vb);
            else
                mma_slots<T, 0, 16>(S, vb, o);
        }
    };
    tile_step(std::true_type{}, 0, kcur);
#pragma unroll 1
    for (int t = 1; t < nt; ++t) {
        kcur = load_kidx(t);
        rows_load<T>(kbase, kpitch, kcur.vox, lane, rk);
        rows_load<T>(vbase, vpitch, kcur.vox, lane, rv);
        tile_step(std::false_type{}, t, kcur);
    }
    mid();
    l += __shfl_xor(l, 32, 64);
    l += 1e-8f;
    if (half == 0 && i_q < c) lse[(int64_t)a.H * g.Tk + h * c + i_q] = (m + __builtin_amdgcn_logf(l)) * LN2;
    // normalise (one factor per query row, through the table), accumulators -> LDS rows -> coalesced stores
    __builtin_amdgcn_wave_barrier();
    table_put(tab_alpha, l32, f2u(1.0f / l));
    __builtin_amdgcn_wave_barrier();
    uint32_t ir[16];
    table_get(tab_alpha, half, ir);
#pragma unroll
    for (int r = 0; r < 16; ++r) o[r] *= u2f(ir[r]);
    tile_put_acc(tile, l32, half, o);
    __builtin_amdgcn_wave_barrier();
    tile_store_rows<T>(tile, const_cast<char*>(head_base<T>(to, h)), pitch_of<T>(to), vox_i, c - bi * 32, lane);
}


// ------------------------------------------------------------------------------------------
// forward of a group of at most 16 tokens (fp32) on 16 x 16 tiles: v_mfma_f32_16x16x4_f32 instead of the
// 32 x 32 x 2 instruction, whose tile would be three quarters padding for such a group.  S^T = K Q^T takes 8
// matrix steps of 32 cycles instead of 16 of 64, P V two blocks of 4 steps instead of up to 8 steps of 64, and the
// softmax works on 4 scores per lane instead of 16.
// Lane l: column col = l % 16, slice g = l / 16.  An operand's reduction index may be permuted freely as long
// as A and B use the same permutation: for S^T slice g carries channels 8g .. 8g + 7 (two 16-byte LDS reads
// per operand), for P V it carries keys 4g .. 4g + 3 - exactly the keys whose scores the lane's accumulator
// holds, so P goes from the accumulator into the second product without leaving its registers.
// ------------------------------------------------------------------------------------------
typedef float f32x4_v __attribute__((ext_vector_type(4)));

template <bool MASK>
__device__ __forceinline__ void fwd_task_small(const WAttnCommon& a, const GroupCtx& g, const FwdIdx& fi, float* tile,
                                               float* tile_x, uint32_t* tab_key, uint32_t* tab_inv,
                                               const TokenTensor32& tq, const TokenTensor32& tk, const TokenTensor32& tv,
                                               const TokenTensor32& to, float* __restrict__ lse) {
    const int lane = threadIdx.x & 63;
    const int col = lane & 15, sl = lane >> 4;
    const int c = g.c, h = g.h;
    const int8_t* mrow = MASK ? a.mask + (int64_t)(g.w % a.nmw) * a.n : nullptr;
    // token col of the group (clamped): query of this lane's column and one of its keys' rows
    const uint32_t vox = (uint32_t)__shfl((int)fi.vox_i, col, 64);       // lanes 0-31 of fi hold tokens 0-31
    const int pos = __shfl(fi.pos_i, col, 64);
    const int reg = MASK ? mrow[pos] : 0;
    u32x4_a rq[2], rk[2], rv[2];
    const char* qbase = head_base<float>(tq, h);
    const char* kbase = head_base<float>(tk, h);
    const char* vbase = head_base<float>(tv, h);
    const uint32_t qpitch = pitch_of<float>(tq), kpitch = pitch_of<float>(tk), vpitch = pitch_of<float>(tv);
#pragma unroll
    for (int v = 0; v < 2; ++v) {                            // eight rows per instruction, 16 bytes per lane
        const uint32_t vr = (uint32_t)__shfl((int)vox, v * 8 + lane / 8, 64);
        const uint32_t off = (uint32_t)(lane % 8) * 16u;
        rq[v] = *reinterpret_cast<const u32x4_a*>(qbase + (__umul24(vr, qpitch) + off));
        rk[v] = *reinterpret_cast<const u32x4_a*>(kbase + (__umul24(vr, kpitch) + off));
        rv[v] = *reinterpret_cast<const u32x4_a*>(vbase + (__umul24(vr, vpitch) + off));
    }
    uint32_t pk = (uint32_t)pos * 4u;
    if (MASK) pk |= (uint32_t)reg << 16;
    __builtin_amdgcn_wave_barrier();
    if (sl == 0) tab_key[col] = pk;
    float* tile_k = tile_x + 16 * TILE_LD;                   // rows 16-31 of the second tile hold K
#pragma unroll
    for (int v = 0; v < 2; ++v) {
        const int at = (v * 8 + lane / 8) * TILE_LD + (lane % 8) * 4;
        *reinterpret_cast<u32x4_a*>(tile_x + at) = rq[v];
        *reinterpret_cast<u32x4_a*>(tile_k + at) = rk[v];
        *reinterpret_cast<u32x4_a*>(tile + at) = rv[v];
    }
    __builtin_amdgcn_wave_barrier();
    // bias gathers first: keys 4 sl .. 4 sl + 3 of query col
    const u32x4_a pkq = *reinterpret_cast<const u32x4_a*>(tab_key + 4 * sl);
    const uint32_t pkr[4] = {pkq.x, pkq.y, pkq.z, pkq.w};
    const char* bias_h = reinterpret_cast<const char*>(a.bias + (int64_t)h * a.n * a.n);
    const uint32_t brow = (uint32_t)(pos * a.n) * 4u;
    float bv[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) bv[r] = *reinterpret_cast<const float*>(bias_h + (brow + (MASK ? (pkr[r] & 0xffffu) : pkr[r])));
    float qb[8], ka[8];
    {
        const f32x4_a* pq = reinterpret_cast<const f32x4_a*>(tile_x + col * TILE_LD + 8 * sl);
        const f32x4_a* pk4 = reinterpret_cast<const f32x4_a*>(tile_k + col * TILE_LD + 8 * sl);
#pragma unroll
        for (int v = 0; v < 2; ++v) {
            const f32x4_a x = pq[v], y = pk4[v];
            qb[4 * v] = x.x; qb[4 * v + 1] = x.y; qb[4 * v + 2] = x.z; qb[4 * v + 3] = x.w;
            ka[4 * v] = y.x; ka[4 * v + 1] = y.y; ka[4 * v + 2] = y.z; ka[4 * v + 3] = y.w;
        }
    }
    const float qscale = a.scale * LOG2E;
    f32x4_v S = {0, 0, 0, 0};                                // S^T[key 4 sl + r][query col]
#pragma unroll
    for (int m = 0; m < 8; ++m) S = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[m], qb[m] * qscale, S, 0, 0, 0);
    float vb[2][4];                                          // V[key 4 sl + r][channel 16 b + col]
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        vb[0][r] = tile[(4 * sl + r) * TILE_LD + col];
        vb[1][r] = tile[(4 * sl + r) * TILE_LD + 16 + col];
    }
    float mx = 0.f;                                          // the operator's max(0, rowmax)
    float sc[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        float x = fmaf(bv[r], LOG2E, S[r]);
        if (MASK && (int)(pkr[r] >> 16) != reg) x += -100.0f * LOG2E;
        x = 4 * sl + r < c ? x : -INFINITY;
        sc[r] = x;
        mx = fmaxf(mx, x);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    float l = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        sc[r] = exp2_fast(sc[r] - mx);
        l += sc[r];
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    l += 1e-8f;
    if (sl == 0 && col < c) lse[(int64_t)a.H * g.Tk + h * c + col] = (mx + __builtin_amdgcn_logf(l)) * LN2;
    f32x4_v o0 = {0, 0, 0, 0}, o1 = {0, 0, 0, 0};            // O[query 4 sl + r][channel col], [16 + col]
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        if (m > 0 && m >= c) break;                          // step m carries keys m, 4 + m, 8 + m, 12 + m
        // step m of slice sl carries key 4 sl + m: A = P[query col][that key], B = V[that key][channel]
        o0 = __builtin_amdgcn_mfma_f32_16x16x4f32(sc[m], vb[0][m], o0, 0, 0, 0);
        o1 = __builtin_amdgcn_mfma_f32_16x16x4f32(sc[m], vb[1][m], o1, 0, 0, 0);
    }
    __builtin_amdgcn_wave_barrier();
    if (sl == 0) tab_inv[col] = f2u(1.0f / l);
    __builtin_amdgcn_wave_barrier();
    const u32x4_a iv = *reinterpret_cast<const u32x4_a*>(tab_inv + 4 * sl);
    const float inv[4] = {u2f(iv.x), u2f(iv.y), u2f(iv.z), u2f(iv.w)};
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        tile[(4 * sl + r) * TILE_LD + col] = o0[r] * inv[r];
        tile[(4 * sl + r) * TILE_LD + 16 + col] = o1[r] * inv[r];
    }
    __builtin_amdgcn_wave_barrier();
    char* obase = const_cast<char*>(head_base<float>(to, h));
    const uint32_t opitch = pitch_of<float>(to);
#pragma unroll
    for (int v = 0; v < 2; ++v) {
        const int R = v * 8 + lane / 8;
        const uint32_t vr = (uint32_t)__shfl((int)vox, R, 64);
        const u32x4_a x = *reinterpret_cast<const u32x4_a*>(tile + R * TILE_LD + (lane % 8) * 4);
        if (R < c) *reinterpret_cast<u32x4_a*>(obase + (__umul24(vr, opitch) + (uint32_t)(lane % 8) * 16u)) = x;
    }
}

template <typename T, bool MASK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void wattn_fwd_kernel(WAttnCommon a, TokenTensor32 tq, TokenTensor32 tk,
                                                        TokenTensor32 tv, TokenTensor32 to,
                                                        float* __restrict__ lse) {
    __shared__ __attribute__((aligned(16))) float tiles[4][2][TILE_WORDS];
    __shared__ __attribute__((aligned(16))) uint32_t tabs[4][2][32];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    int64_t d;
    int bi;
    if (!locate(a, (int64_t)blockIdx.x * 4 + wave, d, bi)) return;
    const GroupCtx g = load_group(a.tasks, d);
    const FwdIdx fi = fwd_indices(a, g, bi, lane & 31);
    if constexpr (std::is_same<T, float>::value) {
        if (g.c <= 16) {
            fwd_task_small<MASK>(a, g, fi, tiles[wave][0], tiles[wave][1], tabs[wave][0], tabs[wave][1], tq, tk, tv, to, lse);
            return;
        }
    }
    fwd_task<T, MASK>(a, g, bi, fi, tiles[wave][0], tiles[wave][1], tabs[wave][0], tabs[wave][1], tq, tk, tv, to, lse, [] {});
}

// ------------------------------------------------------------------------------------------
// backward, query side: dQ
// ------------------------------------------------------------------------------------------
// One task of the query side on one wavefront.  tile: K of the tile (read back by column); tile_x:
// rows in transit to the operand layout, then dQ; two 32-entry tables.
template <typename T, bool MASK>
__device__ __forceinline__ void bwd_q_task(const WAttnCommon& a, int64_t task, float* tile, float* tile_x,
                                           const TokenTensor32& tq,
                                           const TokenTensor32& tk, const TokenTensor32& tv, const TokenTensor32& to,
                                           const TokenTensor32& tdo, const float* __restrict__ lse,
                                           const TokenTensor32& tdq) {
    const int lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    int64_t d;
    int bi;
    if (!locate(a, task, d, bi)) return;
    const PadTab tab_key = pad_tab(tile, 0), tab_D = pad_tab(tile, 1);
    const GroupCtx g = load_group(a.tasks, d);
    const int c = g.c, h = g.h;
    const int nt = (c + 31) >> 5;
    const int32_t* order = a.order + g.Tk;
    const int32_t* tok_pos = a.tok_pos + g.Tk;
    const int8_t* mrow = MASK ? a.mask + (int64_t)(g.w % a.nmw) * a.n : nullptr;
    const char* kbase = head_base<T>(tk, h);
    const char* vbase = head_base<T>(tv, h);
    const uint32_t kpitch = pitch_of<T>(tk), vpitch = pitch_of<T>(tv);

    const int i_q = bi * 32 + l32;
    const int i_c = i_q < c ? i_q : c - 1;
    const uint32_t vox_i = order[i_c];
    const int pos_i = tok_pos[i_c];
    // indices of the first key tile: requested in the same round trip as the query indices
    int jn_c = l32 < c ? l32 : c - 1;
    uint32_t vox_n = order[jn_c];
    int pos_n = tok_pos[jn_c];
    const int reg_i = MASK ? mrow[pos_i] : 0;
    const float L2 = lse[(int64_t)a.H * g.Tk + h * c + i_c] * LOG2E;
    float qb[16], dob[16];
    {
        RowLoad<T> rq, rdo, ro;
        rows_load<T>(head_base<T>(tq, h), pitch_of<T>(tq), vox_i, lane, rq);
        rows_load<T>(head_base<T>(tdo, h), pitch_of<T>(tdo), vox_i, lane, rdo);
        rows_load<T>(head_base<T>(to, h), pitch_of<T>(to), vox_i, lane, ro);
        rows_to_tile<T>(tile_x, lane, rq);
        __builtin_amdgcn_wave_barrier();
        tile_get_rows(tile_x, l32, half, qb);
        __builtin_amdgcn_wave_barrier();
        rows_to_tile<T>(tile_x, lane, rdo);
        rows_dot_to_table<T>(tab_D, lane, rdo, ro);          // D_i = dO_i . O_i
        __builtin_amdgcn_wave_barrier();
        tile_get_rows(tile_x, l32, half, dob);
    }
    const float D = u2f(tab_D.get(l32));
    const float qscale = a.scale * LOG2E;
#pragma unroll
    for (int s = 0; s < 16; ++s) qb[s] *= qscale;
    const char* bias_h = reinterpret_cast<const char*>(a.bias + (int64_t)h * a.n * a.n);
    const uint32_t brow = (uint32_t)(pos_i * a.n) * 4u;

    f32x16 dq = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 1
    for (int t = 0; t < nt; ++t) {
        const uint32_t vox_j = vox_n;
        const int pos_j = pos_n;
        RowLoad<T> rk, rv;
        rows_load<T>(kbase, kpitch, vox_j, lane, rk);
        rows_load<T>(vbase, vpitch, vox_j, lane, rv);
        uint32_t pk = (uint32_t)pos_j * 4u;
        if (MASK) pk |= (uint32_t)mrow[pos_j] << 16;
        {                                                    // indices of the next key tile, a tile ahead
            const int j = (t + 1) * 32 + l32;
            jn_c = j < c ? j : c - 1;
            vox_n = order[jn_c];
            pos_n = tok_pos[jn_c];
        }
        __builtin_amdgcn_wave_barrier();
        table_put(tab_key, l32, pk);
        rows_to_tile<T>(tile, lane, rk);                     // K rows, read back by column for dQ
        rows_to_tile<T>(tile_x, lane, rv);
        __builtin_amdgcn_wave_barrier();
        float ka[16], va[16];
        tile_get_rows(tile, l32, half, ka);
        tile_get_rows(tile_x, l32, half, va);
        uint32_t pkr[16];
        table_get(tab_key, half, pkr);
        float bv[16];
#pragma unroll
        for (int r = 0; r < 16; ++r)
            bv[r] = *reinterpret_cast<const float*>(bias_h + (brow + (MASK ? (pkr[r] & 0xffffu) : pkr[r])));
        f32x16 St = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        f32x16 dPt = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        mma_slots<T, 0, 16>(ka, qb, St);
        mma_slots<T, 0, 16>(va, dob, dPt);
        float kb[16];
        tile_get_cols(tile, l32, half, kb);                  // K[key acc_row(r, half)][channel l32]
        const int jlim = c - t * 32 - 4 * half;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            // fp32: a block of eight key rows wholly behind the last key is padding and is skipped
            if (std::is_same<T, float>::value && (r & 3) == 0 && r > 0 && 2 * r >= c - t * 32) break;
            float s = fmaf(bv[r], LOG2E, St[r]);
            if (MASK && (int)(pkr[r] >> 16) != reg_i) s += -100.0f * LOG2E;
            const float pr = (8 * (r >> 2) + (r & 3)) < jlim ? exp2_fast(s - L2) : 0.f;
            const float ds = pr * (dPt[r] - D);
            if constexpr (std::is_same<T, float>::value)
                dq = __builtin_amdgcn_mfma_f32_32x32x2f32(ds, kb[r], dq, 0, 0, 0);
            else
                St[r] = ds;
        }
        if constexpr (!std::is_same<T, float>::value) mma_slots<T, 0, 16>(St, kb, dq);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) dq[r] *= a.scale;
    __builtin_amdgcn_wave_barrier();
    tile_put_acc(tile_x, l32, half, dq);
    __builtin_amdgcn_wave_barrier();
    tile_store_rows<T>(tile_x, const_cast<char*>(head_base<T>(tdq, h)), pitch_of<T>(tdq), vox_i, c - bi * 32, lane);
}

template <typename T, bool MASK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void wattn_bwd_q_kernel(
    WAttnCommon a, TokenTensor32 tq, TokenTensor32 tk, TokenTensor32 tv, TokenTensor32 to, TokenTensor32 tdo,
    const float* __restrict__ lse, TokenTensor32 tdq) {
    __shared__ __attribute__((aligned(16))) float tiles[4][2][TILE_WORDS];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    bwd_q_task<T, MASK>(a, (int64_t)blockIdx.x * 4 + wave, tiles[wave][0], tiles[wave][1], tq, tk, tv, to, tdo, lse, tdq);
}

// ------------------------------------------------------------------------------------------
// backward, key side: dK, dV (and dS for the bias gradient)
// ------------------------------------------------------------------------------------------
// What a key-side task does about dQ:
//   KV_ONLY    nothing (the group has query-side tasks of its own)
//   KV_SINGLE  a group of one tile: dS is already in registers; transposed through LDS it is the A
//              operand of dQ = dS K, which saves the group its whole query-side task
//   KV_PAIR    a group of two tiles, its two key-side tasks on neighbouring wavefronts of one
//              workgroup: each forms dS K for both query tiles, hands the partial result of the other
//              wavefront's tile over through an LDS exchange tile, and after one workgroup barrier adds
//              the two partial results of its own tile.  S and dP of the group are then computed once
//              instead of twice (320 instead of 448 MFMA steps of 32x32x2 per group) and the five
//              operands are read once.
enum { KV_ONLY = 0, KV_SINGLE = 1, KV_PAIR = 2 };

// xch: this wavefront's exchange tile (KV_PAIR), xch_peer: the other wavefront's; accumulator layout
// (piece q of lane l at 16-byte slot q*64 + l: neighbouring lanes touch neighbouring slots)
__device__ __forceinline__ void xch_put(float* xch, int lane, const f32x16& v) {
    f32x4_a* p = reinterpret_cast<f32x4_a*>(xch) + lane;
#pragma unroll
    for (int q = 0; q < 4; ++q) p[q * 64] = f32x4_a{v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]};
}
__device__ __forceinline__ void xch_add(const float* xch, int lane, f32x16& v) {
    const f32x4_a* p = reinterpret_cast<const f32x4_a*>(xch) + lane;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const f32x4_a t = p[q * 64];
        v[4 * q] += t.x; v[4 * q + 1] += t.y; v[4 * q + 2] += t.z; v[4 * q + 3] += t.w;
    }
}

// ------------------------------------------------------------------------------------------
// backward of a group of at most 16 tokens (fp32) on 16 x 16 tiles (v_mfma_f32_16x16x4_f32; lane l: column
// col = l % 16, slice sl = l / 16; see the forward).  S and dP are formed with queries as rows
// (accumulator rows 4 sl + r) and keys as columns (col), so the lane's P and dS are the A operand of
// dV = P^T dO and dK = dS^T Q as they stand (step m of slice sl carries query 4 sl + m); dQ = dS K takes dS
// through a 16 x 16 LDS transpose.  40 matrix steps of 32 cycles instead of 80 of 64, ten row loads instead
// of twenty, a softmax pass over 4 values per lane instead of 16.
// LDS: rows 0-15 of tile_q hold Q, rows 16-31 K; rows 0-15 of tile_do hold dO, rows 16-31 V, later dS.
// ------------------------------------------------------------------------------------------
template <bool MASK>
__device__ __forceinline__ void bwd_task_small(const WAttnCommon& a, const GroupCtx& g, float* tile_q, float* tile_do,
                                               const TokenTensor32& tq, const TokenTensor32& tk, const TokenTensor32& tv,
                                               const TokenTensor32& to, const TokenTensor32& tdo,
                                               const float* __restrict__ lse, const TokenTensor32& tdq,
                                               const TokenTensor32& tdk, const TokenTensor32& tdv,
                                               float* __restrict__ ds_out) {
    const int lane = threadIdx.x & 63;
    const int col = lane & 15, sl = lane >> 4;
    const int c = g.c, h = g.h;
    const int8_t* mrow = MASK ? a.mask + (int64_t)(g.w % a.nmw) * a.n : nullptr;
    const PadTab tab_pos = pad_tab(tile_q, 0), tab_L = pad_tab(tile_q, 1), tab_D = pad_tab(tile_q, 2);
    // token col of the group (clamped to the last one): key of this lane's column
    const int t_c = col < c ? col : c - 1;
    const uint32_t vox = (uint32_t)a.order[g.Tk + t_c];
    const int pos = a.tok_pos[g.Tk + t_c];
    const float L2 = col < c ? lse[(int64_t)a.H * g.Tk + h * c + t_c] * LOG2E : INFINITY;   // padding queries: P = 0
    const int reg = MASK ? mrow[pos] : 0;
    u32x4_a rq[2], rk[2], rv[2], rdo[2], ro[2];
#pragma unroll
    for (int v = 0; v < 2; ++v) {                            // eight rows per instruction, 16 bytes per lane
        const uint32_t vr = (uint32_t)__shfl((int)vox, v * 8 + lane / 8, 64);
        const uint32_t off = (uint32_t)(lane % 8) * 16u;
        rk[v] = *reinterpret_cast<const u32x4_a*>(head_base<float>(tk, h) + (__umul24(vr, pitch_of<float>(tk)) + off));
        rv[v] = *reinterpret_cast<const u32x4_a*>(head_base<float>(tv, h) + (__umul24(vr, pitch_of<float>(tv)) + off));
        rq[v] = *reinterpret_cast<const u32x4_a*>(head_base<float>(tq, h) + (__umul24(vr, pitch_of<float>(tq)) + off));
        rdo[v] = *reinterpret_cast<const u32x4_a*>(head_base<float>(tdo, h) + (__umul24(vr, pitch_of<float>(tdo)) + off));
        ro[v] = *reinterpret_cast<const u32x4_a*>(head_base<float>(to, h) + (__umul24(vr, pitch_of<float>(to)) + off));
    }
    uint32_t pi = (uint32_t)(pos * a.n) * 4u;                // byte offset of bias row pos (< 2^16)
    if (MASK) pi |= (uint32_t)reg << 16;
    float* tile_k = tile_q + 16 * TILE_LD;
    float* tile_v = tile_do + 16 * TILE_LD;
    __builtin_amdgcn_wave_barrier();
    if (sl == 0) {
        tab_pos.put(col, pi);
        tab_L.put(col, f2u(L2));
    }
#pragma unroll
    for (int v = 0; v < 2; ++v) {
        const int at = (v * 8 + lane / 8) * TILE_LD + (lane % 8) * 4;
        *reinterpret_cast<u32x4_a*>(tile_q + at) = rq[v];
        *reinterpret_cast<u32x4_a*>(tile_k + at) = rk[v];
        *reinterpret_cast<u32x4_a*>(tile_do + at) = rdo[v];
        *reinterpret_cast<u32x4_a*>(tile_v + at) = rv[v];
        float d = chunk_dot<float>(rdo[v], ro[v]);           // D_i = dO_i . O_i, summed over the 8 lanes of a row
        d += dpp_f32<0xB1>(d);
        d += dpp_f32<0x4E>(d);
        d += dpp_f32<0x141>(d);
        if (lane % 8 == 0) tab_D.put(v * 8 + lane / 8, f2u(d));
    }
    __builtin_amdgcn_wave_barrier();
    // bias[h][pos of query 4 sl + r][pos of key col]: gathers first, the products cover their latency
    const u32x4_a piq = tab_pos.chunk(sl);
    const uint32_t pir[4] = {piq.x, piq.y, piq.z, piq.w};
    const char* bias_h = reinterpret_cast<const char*>(a.bias + (int64_t)h * a.n * a.n);
    const uint32_t bcol = (uint32_t)pos * 4u;
    float bv[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) bv[r] = *reinterpret_cast<const float*>(bias_h + (bcol + (MASK ? (pir[r] & 0xffffu) : pir[r])));
    auto row8 = [&](const float* t, float (&x)[8]) {         // channels 8 sl .. 8 sl + 7 of row col
        const f32x4_a* p4 = reinterpret_cast<const f32x4_a*>(t + col * TILE_LD + 8 * sl);
        const f32x4_a u = p4[0], w = p4[1];
        x[0] = u.x; x[1] = u.y; x[2] = u.z; x[3] = u.w; x[4] = w.x; x[5] = w.y; x[6] = w.z; x[7] = w.w;
    };
    f32x4_v S = {0, 0, 0, 0}, dP = {0, 0, 0, 0};            // [query 4 sl + r][key col]
    {
        float qa[8], kb[8];
        row8(tile_q, qa);
        row8(tile_k, kb);
#pragma unroll
        for (int m = 0; m < 8; ++m) S = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[m], kb[m], S, 0, 0, 0);
        float doa[8], vb[8];
        row8(tile_do, doa);
        row8(tile_v, vb);
#pragma unroll
        for (int m = 0; m < 8; ++m) dP = __builtin_amdgcn_mfma_f32_16x16x4f32(doa[m], vb[m], dP, 0, 0, 0);
    }
    const u32x4_a Lq = tab_L.chunk(sl), Dq = tab_D.chunk(sl);
    const float Lr[4] = {u2f(Lq.x), u2f(Lq.y), u2f(Lq.z), u2f(Lq.w)};
    const float Dr[4] = {u2f(Dq.x), u2f(Dq.y), u2f(Dq.z), u2f(Dq.w)};
    const float sscale = a.scale * LOG2E;
    float pr[4], ds[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        float x = fmaf(S[r], sscale, bv[r] * LOG2E);
        if (MASK && (int)(pir[r] >> 16) != reg) x += -100.0f * LOG2E;
        pr[r] = col < c ? exp2_fast(x - Lr[r]) : 0.f;        // padding keys and (L = inf) padding queries: 0
        ds[r] = pr[r] * (dP[r] - Dr[r]);
    }
    if (ds_out && col < c) {
        float* ds_g = ds_out + g.sq + col;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (4 * sl + r < c) ds_g[(4 * sl + r) * c] = ds[r];
    }
    // dV = P^T dO, dK = dS^T Q: step m of slice sl carries query 4 sl + m
    f32x4_v dv0 = {0, 0, 0, 0}, dv1 = {0, 0, 0, 0}, dk0 = {0, 0, 0, 0}, dk1 = {0, 0, 0, 0};
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        if (m > 0 && m >= c) break;
        const float* rdo_ = tile_do + (4 * sl + m) * TILE_LD + col;
        const float* rq_ = tile_q + (4 * sl + m) * TILE_LD + col;
        dv0 = __builtin_amdgcn_mfma_f32_16x16x4f32(pr[m], rdo_[0], dv0, 0, 0, 0);
        dv1 = __builtin_amdgcn_mfma_f32_16x16x4f32(pr[m], rdo_[16], dv1, 0, 0, 0);
        dk0 = __builtin_amdgcn_mfma_f32_16x16x4f32(ds[m], rq_[0], dk0, 0, 0, 0);
        dk1 = __builtin_amdgcn_mfma_f32_16x16x4f32(ds[m], rq_[16], dk1, 0, 0, 0);
    }
    // dQ = dS K: dS[query][key] through LDS (the V rows are no longer needed), read back a query row per column
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int r = 0; r < 4; ++r) tile_v[(4 * sl + r) * TILE_LD + col] = ds[r];
    __builtin_amdgcn_wave_barrier();
    const f32x4_a dsq = *reinterpret_cast<const f32x4_a*>(tile_v + col * TILE_LD + 4 * sl);   // dS[query col][keys 4 sl ..]
    const float dsr[4] = {dsq.x, dsq.y, dsq.z, dsq.w};
    f32x4_v dq0 = {0, 0, 0, 0}, dq1 = {0, 0, 0, 0};
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        if (m > 0 && m >= c) break;
        const float* rk_ = tile_k + (4 * sl + m) * TILE_LD + col;
        dq0 = __builtin_amdgcn_mfma_f32_16x16x4f32(dsr[m], rk_[0], dq0, 0, 0, 0);
        dq1 = __builtin_amdgcn_mfma_f32_16x16x4f32(dsr[m], rk_[16], dq1, 0, 0, 0);
    }
    // accumulators (rows 4 sl + r, channels col and 16 + col) -> LDS rows -> 16-byte row stores
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int at = (4 * sl + r) * TILE_LD + col;
        tile_q[at] = dq0[r] * a.scale;                       // Q, K, dO rows have all been read
        tile_q[at + 16] = dq1[r] * a.scale;
        tile_k[at] = dk0[r] * a.scale;
        tile_k[at + 16] = dk1[r] * a.scale;
        tile_do[at] = dv0[r];
        tile_do[at + 16] = dv1[r];
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int v = 0; v < 2; ++v) {
        const int R = v * 8 + lane / 8;
        const uint32_t vr = (uint32_t)__shfl((int)vox, R, 64);
        const int at = R * TILE_LD + (lane % 8) * 4;
        const uint32_t off = (uint32_t)(lane % 8) * 16u;
        if (R < c) {
            *reinterpret_cast<u32x4_a*>(const_cast<char*>(head_base<float>(tdq, h)) + (__umul24(vr, pitch_of<float>(tdq)) + off)) =
                *reinterpret_cast<const u32x4_a*>(tile_q + at);
            *reinterpret_cast<u32x4_a*>(const_cast<char*>(head_base<float>(tdk, h)) + (__umul24(vr, pitch_of<float>(tdk)) + off)) =
                *reinterpret_cast<const u32x4_a*>(tile_k + at);
            *reinterpret_cast<u32x4_a*>(const_cast<char*>(head_base<float>(tdv, h)) + (__umul24(vr, pitch_of<float>(tdv)) + off)) =
                *reinterpret_cast<const u32x4_a*>(tile_do + at);
        }
    }
}

// `live` = false (KV_PAIR only): a wavefront without a task that still has to meet the barrier.
template <typename T, bool MASK, int DQ>
__device__ __forceinline__ void bwd_kv_task(const WAttnCommon& a, int64_t task, bool live, float* tile_q, float* tile_do,
                                            float* xch, const float* xch_peer,
                                            const TokenTensor32& tq, const TokenTensor32& tk, const TokenTensor32& tv,
                                            const TokenTensor32& to, const TokenTensor32& tdo,
                                            const float* __restrict__ lse, const TokenTensor32& tdk,
                                            const TokenTensor32& tdv, float* __restrict__ ds_out,
                                            const TokenTensor32& tdq) {
    const int lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    int64_t d;
    int bj;
    if (!live || !locate(a, task, d, bj)) {
        if (DQ == KV_PAIR) __syncthreads();
        return;
    }
    const PadTab tab_pos = pad_tab(tile_q, 0), tab_L = pad_tab(tile_q, 1), tab_D = pad_tab(tile_q, 2);
    const GroupCtx g = load_group(a.tasks, d);
    if constexpr (DQ == KV_SINGLE && std::is_same<T, float>::value) {
        if (g.c <= 16) {
            bwd_task_small<MASK>(a, g, tile_q, tile_do, tq, tk, tv, to, tdo, lse, tdq, tdk, tdv, ds_out);
            return;
        }
    }
    const int c = g.c, h = g.h;
    const int nt = (c + 31) >> 5;
    const int32_t* order = a.order + g.Tk;
    const int32_t* tok_pos = a.tok_pos + g.Tk;
    const int8_t* mrow = MASK ? a.mask + (int64_t)(g.w % a.nmw) * a.n : nullptr;
    const char* qbase = head_base<T>(tq, h);
    const char* obase = head_base<T>(to, h);
    const char* dobase = head_base<T>(tdo, h);
    const uint32_t qpitch = pitch_of<T>(tq), opitch = pitch_of<T>(to), dopitch = pitch_of<T>(tdo);
    const float* lse_g = lse + (int64_t)a.H * g.Tk + h * c;

    // Memory round trips of a task depend on one another (descriptor -> token indices -> rows -> bias), and
    // a task is short, so everything that can be requested in the same round trip is: the indices of the
    // first query tile go out with the key indices, and its rows with the K and V rows.
    struct QIdx {
        uint32_t vox;        // voxel of query t*32 + l32 (clamped to the last token)
        int pos;
        float L2;            // its log-sum-exp in units of log 2; +inf for padding queries: P and dS exactly zero
    };
    auto load_qidx = [&](const int t) {
        const int i = t * 32 + l32;
        const int i_c = i < c ? i : c - 1;
        QIdx q;
        q.vox = order[i_c];
        q.pos = tok_pos[i_c];
        q.L2 = i < c ? lse_g[i_c] * LOG2E : INFINITY;
        return q;
    };
    // key side: lane l32 owns key bj*32 + l32
    const int j_k = bj * 32 + l32;
    const int j_c = j_k < c ? j_k : c - 1;
    const uint32_t vox_j = order[j_c];
    const int pos_j = tok_pos[j_c];
    const int t_first = DQ == KV_PAIR ? 1 - bj : 0;           // KV_PAIR: the other wavefront's query tile first
    QIdx qcur = load_qidx(t_first);
    const int reg_j = MASK ? mrow[pos_j] : 0;
    RowLoad<T> rq, rdo, ro;
    float kb[16], vb[16];
    {
        RowLoad<T> rk, rv;
        constexpr bool ONCE = DQ == KV_SINGLE;                // a group of one tile: nobody else reads these rows
        rows_load<T, ONCE>(head_base<T>(tk, h), pitch_of<T>(tk), vox_j, lane, rk);
        rows_load<T, ONCE>(head_base<T>(tv, h), pitch_of<T>(tv), vox_j, lane, rv);
        rows_load<T, ONCE>(qbase, qpitch, qcur.vox, lane, rq);
        rows_load<T, ONCE>(dobase, dopitch, qcur.vox, lane, rdo);
        rows_load<T, ONCE>(obase, opitch, qcur.vox, lane, ro);
        rows_to_tile<T>(tile_q, lane, rk);
        rows_to_tile<T>(tile_do, lane, rv);
        __builtin_amdgcn_wave_barrier();
        tile_get_rows(tile_q, l32, half, kb);
        tile_get_rows(tile_do, l32, half, vb);
    }
    const float kscale = a.scale * LOG2E;                    // scores in units of log 2
#pragma unroll
    for (int s = 0; s < 16; ++s) kb[s] *= kscale;
    const char* bias_h = reinterpret_cast<const char*>(a.bias + (int64_t)h * a.n * a.n);
    const uint32_t bcol = (uint32_t)pos_j * 4u;
    float* ds_g = ds_out ? ds_out + g.sq + j_k : nullptr;

    f32x16 dk = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    f32x16 dv = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    f32x16 dq_own;                                            // KV_PAIR: dS K of this wavefront's own query tile
    // One query tile t against this task's keys.  What happens to dS K of the tile (dq_tag): 0 = not
    // formed, 1 = written out as dQ of a one-tile group, 2 = handed to the other wavefront of the pair,
    // 3 = kept in dq_own.
    // rq, rdo, ro hold the rows of query tile t (requested by the caller), qi its indices.
    auto tile_pass = [&](const int t, const QIdx& qi, auto dq_tag) {
        constexpr int DQ_USE = decltype(dq_tag)::value;
        uint32_t pi = (uint32_t)(qi.pos * a.n) * 4u;         // byte offset of bias row pos_i (< 2^16)
        if (MASK) pi |= (uint32_t)mrow[qi.pos] << 16;
        __builtin_amdgcn_wave_barrier();
        table_put(tab_pos, l32, pi);
        table_put(tab_L, l32, f2u(qi.L2));
        rows_dot_to_table<T>(tab_D, lane, rdo, ro);          // D_i = dO_i . O_i
        rows_to_tile<T>(tile_q, lane, rq);                   // both are read back by row and by column
        rows_to_tile<T>(tile_do, lane, rdo);
        __builtin_amdgcn_wave_barrier();
        // P and dS of the tile: rows = queries acc_row(r, half), column = this lane's key.
        // The bias gathers of all 16 rows are requested between the two score products (the second
        // one covers their latency, and the operand registers of the first are free by then);
        // everything else is fetched from LDS four rows at a time, right before it is used, to keep
        // the register footprint low.
        f32x16 St, dPt;
        {
            float qa[16];
            tile_get_rows(tile_q, l32, half, qa);
            St = mma_slots_first<T, 16>(qa, kb);
        }
        float bv[16];
        uint32_t differ = 0;                                  // bit r: regions of the row and the key differ
        {
            uint32_t pir[16];
            table_get(tab_pos, half, pir);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                bv[r] = *reinterpret_cast<const float*>(bias_h + (bcol + (MASK ? (pir[r] & 0xffffu) : pir[r])));
                if (MASK) differ |= ((int)(pir[r] >> 16) != reg_j ? 1u : 0u) << r;
            }
        }
        {
            float doa[16];
            tile_get_rows(tile_do, l32, half, doa);
            dPt = mma_slots_first<T, 16>(doa, vb);
        }
        float* ds_t = ds_g ? ds_g + (int64_t)(t * 32 + 4 * half) * c : nullptr;
        const int ilim = c - t * 32 - 4 * half;
        const float* do_col = tile_do + 4 * half * TILE_LD + l32;
        const float* q_col = tile_q + 4 * half * TILE_LD + l32;
        float dob8[8], qbr8[8];                              // 16-bit tokens: operands of eight slots
        const int qleft = c - t * 32;                         // queries of this tile
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if constexpr (std::is_same<T, float>::value) {
                // a block of eight query rows that lies wholly behind the last query is padding: P and dS
                // are zero there, so its exponentials, LDS reads and matrix steps are skipped
                if (q > 0 && 8 * q >= qleft) {
                    if (DQ_USE != 0) {
#pragma unroll
                        for (int qq = q; qq < 4; ++qq)
#pragma unroll
                            for (int k = 0; k < 4; ++k) dPt[4 * qq + k] = 0.f;
                    }
                    break;
                }
            }
            const u32x4_a Lq = tab_L.chunk(2 * q + half), Dq = tab_D.chunk(2 * q + half);
            const uint32_t Lr[4] = {Lq.x, Lq.y, Lq.z, Lq.w}, Dr[4] = {Dq.x, Dq.y, Dq.z, Dq.w};
            float dob[4], qbr[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                dob[k] = do_col[(8 * q + k) * TILE_LD];      // dO[query acc_row(r, half)][channel l32]
                qbr[k] = q_col[(8 * q + k) * TILE_LD];       // Q [query acc_row(r, half)][channel l32]
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int r = 4 * q + k;
                float s = fmaf(bv[r], LOG2E, St[r]);
                if (MASK && (differ >> r & 1u)) s += -100.0f * LOG2E;
                const float pr = exp2_fast(s - u2f(Lr[k]));
                const float ds = pr * (dPt[r] - u2f(Dr[k]));
                const int row = 8 * q + k;
                if (ds_t && row < ilim && j_k < c) ds_t[row * c] = ds;
                if constexpr (std::is_same<T, float>::value) {
                    dv = __builtin_amdgcn_mfma_f32_32x32x2f32(pr, dob[k], dv, 0, 0, 0);     // dV += P^T dO
                    dk = __builtin_amdgcn_mfma_f32_32x32x2f32(ds, qbr[k], dk, 0, 0, 0);     // dK += dS^T Q
                    if (DQ_USE != 0) dPt[r] = ds;
                } else {                                     // collected: eight slots per 16-bit step
                    St[r] = pr;
                    dPt[r] = ds;
                    dob8[4 * (q & 1) + k] = dob[k];
                    qbr8[4 * (q & 1) + k] = qbr[k];
                }
            }
            if constexpr (!std::is_same<T, float>::value) {
                if (q & 1) {
                    if (q == 1) {
                        mma_slots<T, 0, 8>(St, dob8, dv);
                        mma_slots<T, 0, 8>(dPt, qbr8, dk);
                    } else {
                        mma_slots8_off<T, 8>(St, dob8, dv);
                        mma_slots8_off<T, 8>(dPt, qbr8, dk);
                    }
                }
            }
        }
        if constexpr (DQ_USE != 0) {
            // dS of this tile (rows = queries by register, column = this lane's key; padding keys
            // zeroed) -> LDS -> one query row per lane; K rows (still scaled by scale * log2 e) go back
            // to LDS for the column reads.  dQ = scale dS K = (dS K_scaled) ln 2.
#pragma unroll
            for (int r = 0; r < 16; ++r) dPt[r] = j_k < c ? dPt[r] : 0.f;
            __builtin_amdgcn_wave_barrier();
            tile_put_acc(tile_do, l32, half, dPt);
            tile_put_rows(tile_q, l32, half, kb);
            __builtin_amdgcn_wave_barrier();
            float dsr[16], kc[16];
            tile_get_rows(tile_do, l32, half, dsr);              // dS[query l32][keys 16 * half + s]
            const float* k_col = tile_q + 16 * half * TILE_LD + l32;
#pragma unroll
            for (int s = 0; s < 16; ++s) kc[s] = k_col[s * TILE_LD];  // K[key 16 * half + s][channel l32]
            f32x16 dq;
            if constexpr (std::is_same<T, float>::value) {
                // slot s carries keys s and 16 + s of this task's tile: slots behind the last key are padding
                const int kleft = c - bj * 32;
                dq = f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (int sb = 0; sb < 4; ++sb) {
                    if (sb > 0 && 4 * sb >= kleft) break;
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        dq = __builtin_amdgcn_mfma_f32_32x32x2f32(dsr[4 * sb + k], kc[4 * sb + k], dq, 0, 0, 0);
                }
            } else {
                dq = mma_slots_first<T, 16>(dsr, kc);
            }
            if constexpr (DQ_USE == 2) {
                xch_put(xch, lane, dq);
                __builtin_amdgcn_wave_barrier();
            } else if constexpr (DQ_USE == 3) {
                dq_own = dq;
                __builtin_amdgcn_wave_barrier();
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) dq[r] *= LN2;
                __builtin_amdgcn_wave_barrier();
                tile_put_acc(tile_do, l32, half, dq);
                __builtin_amdgcn_wave_barrier();
                tile_store_rows<T>(tile_do, const_cast<char*>(head_base<T>(tdq, h)), pitch_of<T>(tdq), vox_j, c, lane);
                __builtin_amdgcn_wave_barrier();
            }
        }
    };
    // the indices of the next query tile are requested before the current one is worked on
    auto request_rows = [&](const QIdx& qi) {
        rows_load<T>(qbase, qpitch, qi.vox, lane, rq);
        rows_load<T>(dobase, dopitch, qi.vox, lane, rdo);
        rows_load<T>(obase, opitch, qi.vox, lane, ro);
    };
    if constexpr (DQ == KV_PAIR) {
        // the other wavefront's query tile first, the own one last (its result stays in registers)
        const QIdx qown = load_qidx(bj);
        tile_pass(1 - bj, qcur, std::integral_constant<int, 2>{});
        request_rows(qown);
        tile_pass(bj, qown, std::integral_constant<int, 3>{});
    } else if constexpr (DQ == KV_SINGLE) {
        tile_pass(0, qcur, std::integral_constant<int, 1>{});     // groups of one tile only
    } else {
        tile_pass(0, qcur, std::integral_constant<int, 0>{});
#pragma unroll 1
        for (int t = 1; t < nt; ++t) {
            const QIdx qi = load_qidx(t);
            request_rows(qi);
            tile_pass(t, qi, std::integral_constant<int, 0>{});
        }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) dk[r] *= a.scale;
    __builtin_amdgcn_wave_barrier();
    tile_put_acc(tile_q, l32, half, dk);
    tile_put_acc(tile_do, l32, half, dv);
    __builtin_amdgcn_wave_barrier();
    tile_store_rows<T>(tile_q, const_cast<char*>(head_base<T>(tdk, h)), pitch_of<T>(tdk), vox_j, c - bj * 32, lane);
    tile_store_rows<T>(tile_do, const_cast<char*>(head_base<T>(tdv, h)), pitch_of<T>(tdv), vox_j, c - bj * 32, lane);
    if (DQ == KV_PAIR) {
        __syncthreads();                                     // both partial results of every pair are in LDS
        xch_add(xch_peer, lane, dq_own);
#pragma unroll
        for (int r = 0; r < 16; ++r) dq_own[r] *= LN2;
        tile_put_acc(tile_do, l32, half, dq_own);
        __builtin_amdgcn_wave_barrier();
        tile_store_rows<T>(tile_do, const_cast<char*>(head_base<T>(tdq, h)), pitch_of<T>(tdq), vox_j, c - bj * 32, lane);
    }
}

template <typename T, bool MASK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void wattn_bwd_kv_kernel(
    WAttnCommon a, TokenTensor32 tq, TokenTensor32 tk, TokenTensor32 tv, TokenTensor32 to, TokenTensor32 tdo,
    const float* __restrict__ lse, TokenTensor32 tdk, TokenTensor32 tdv, float* __restrict__ ds_out) {
    __shared__ __attribute__((aligned(16))) float tiles[4][2][TILE_WORDS];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    bwd_kv_task<T, MASK, KV_ONLY>(a, (int64_t)blockIdx.x * 4 + wave, true, tiles[wave][0], tiles[wave][1], nullptr, nullptr,
                                  tq, tk, tv, to, tdo, lse, tdk, tdv, ds_out, tdk);
}

// The whole backward in one launch.  Workgroups (four wavefronts, one task each) are numbered through
// four segments, each starting at a workgroup boundary:
//   1. query-side tasks of the groups of three and four tiles
//   2. their key-side tasks (KV_ONLY); 1 and 2 are interleaved in runs of eight workgroups (see the kernel)
//   3. key-side tasks of the groups of two tiles, the two tasks of a group side by side (KV_PAIR)
//   4. key-side tasks of the groups of one tile (KV_SINGLE)
// Heaviest tasks first, so the long ones start first and the short ones fill the tail.
struct BwdSegments {
    int64_t wg_kv, wg_pair, wg_single;   // first workgroup of segments 2, 3, 4
    int64_t n_big;                       // tasks per side of the groups of three and four tiles
    int64_t n_pair;                      // key-side tasks of the groups of two tiles (even)
};

template <typename T, bool MASK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void wattn_bwd_all_kernel(
    WAttnCommon a, BwdSegments sg, TokenTensor32 tq, TokenTensor32 tk, TokenTensor32 tv, TokenTensor32 to,
    TokenTensor32 tdo, const float* __restrict__ lse, TokenTensor32 tdq, TokenTensor32 tdk, TokenTensor32 tdv,
    float* __restrict__ ds_out) {
    __shared__ __attribute__((aligned(16))) float tiles[4][2][TILE_WORDS];
    __shared__ __attribute__((aligned(16))) float xch[4][64 * 16];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t wg = blockIdx.x;
    float* t0 = tiles[wave][0];
    float* t1 = tiles[wave][1];
    if (wg < sg.wg_pair) {
        // Segments 1 and 2 interleaved in runs of eight workgroups: workgroups 16 k .. 16 k + 7 take the query side
        // of eight consecutive task quadruples, workgroups 16 k + 8 .. 16 k + 15 the key side of the same ones.
        // Workgroups are dealt to the eight XCDs round robin, so both sides of a group run on one XCD at about the
        // same time and the second one finds the group's rows in that XCD's L2.
        const int64_t quad = (wg >> 4) * 8 + (wg & 7);
        const int64_t task = quad * 4 + wave;
        if (task < sg.n_big) {
            if ((wg & 8) == 0)
                bwd_q_task<T, MASK>(a, task, t0, t1, tq, tk, tv, to, tdo, lse, tdq);
            else
                bwd_kv_task<T, MASK, KV_ONLY>(a, task, true, t0, t1, nullptr, nullptr, tq, tk, tv, to, tdo, lse, tdk, tdv,
                                              ds_out, tdq);
        }
    } else if (wg < sg.wg_single) {
        const int64_t task = (wg - sg.wg_pair) * 4 + wave;
        bwd_kv_task<T, MASK, KV_PAIR>(a, sg.n_big + task, task < sg.n_pair, t0, t1, xch[wave], xch[wave ^ 1], tq, tk, tv, to,
                                      tdo, lse, tdk, tdv, ds_out, tdq);
    } else {
        const int64_t task = (wg - sg.wg_single) * 4 + wave;
        bwd_kv_task<T, MASK, KV_SINGLE>(a, sg.n_big + sg.n_pair + task, true, t0, t1, nullptr, nullptr, tq, tk, tv, to, tdo,
                                        lse, tdk, tdv, ds_out, tdq);
    }
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
constexpr int WATTN_BUCKETS = 4;

template <typename T>
static int run_forward(const WAttnCommon& a, const TokenTensor32& q, const TokenTensor32& k, const TokenTensor32& v,
                       const TokenTensor32& o, float* lse, hipStream_t s) {
    const unsigned blocks = (unsigned)((a.first[4] + 3) / 4);
    if (a.mask)
        hipLaunchKernelGGL((wattn_fwd_kernel<T, true>), dim3(blocks), dim3(256), 0, s, a, q, k, v, o, lse);
    else
        hipLaunchKernelGGL((wattn_fwd_kernel<T, false>), dim3(blocks), dim3(256), 0, s, a, q, k, v, o, lse);
    return launch_ok("window attention forward");
}

template <typename T, bool MASK>
static void launch_backward(const WAttnCommon& a, const TokenTensor32& q, const TokenTensor32& k,
                            const TokenTensor32& v, const TokenTensor32& o, const TokenTensor32& d_o, const float* lse,
                            const TokenTensor32& dq, const TokenTensor32& dk, const TokenTensor32& dv, float* ds_out,
                            int sides, hipStream_t s) {
    if (sides == 3) {
        BwdSegments sg;
        sg.n_big = a.first[2];
        sg.n_pair = a.first[3] - a.first[2];
        const int64_t n_single = a.first[4] - a.first[3];
        const int64_t wg_big = (sg.n_big + 3) / 4;
        sg.wg_kv = wg_big;
        sg.wg_pair = 16 * ((wg_big + 7) / 8);              // both sides, interleaved in runs of eight workgroups
        sg.wg_single = sg.wg_pair + (sg.n_pair + 3) / 4;
        const int64_t wgs = sg.wg_single + (n_single + 3) / 4;
        hipLaunchKernelGGL((wattn_bwd_all_kernel<T, MASK>), dim3((unsigned)wgs), dim3(256), 0, s, a, sg, q, k, v, o, d_o, lse,
                           dq, dk, dv, ds_out);
        return;
    }
    const unsigned blocks = (unsigned)((a.first[4] + 3) / 4);
    if (sides & 1)
        hipLaunchKernelGGL((wattn_bwd_q_kernel<T, MASK>), dim3(blocks), dim3(256), 0, s, a, q, k, v, o, d_o, lse, dq);
    if (sides & 2)
        hipLaunchKernelGGL((wattn_bwd_kv_kernel<T, MASK>), dim3(blocks), dim3(256), 0, s, a, q, k, v, o, d_o, lse, dk,
                           dv, ds_out);
}

template <typename T>
static int run_backward(const WAttnCommon& a, const TokenTensor32& q, const TokenTensor32& k, const TokenTensor32& v,
                        const TokenTensor32& o, const TokenTensor32& d_o, const float* lse, const TokenTensor32& dq,
                        const TokenTensor32& dk, const TokenTensor32& dv, float* ds_out, int sides, hipStream_t s) {
    if (a.mask)
        launch_backward<T, true>(a, q, k, v, o, d_o, lse, dq, dk, dv, ds_out, sides, s);
    else
        launch_backward<T, false>(a, q, k, v, o, d_o, lse, dq, dk, dv, ds_out, sides, s);
    return launch_ok("window attention backward");
}

// rows must be reachable with 32-bit byte offsets and 16-byte vector accesses
static int check_tensor(const char* who, const char* name, const void* base, int64_t stride, int col0, int64_t N,
                        int H, int dtype) {
    const int64_t esz = dtype == SSWIN_F32 ? 4 : 2;
    SSWIN_CHECK(stride >= (int64_t)H * 32 + col0 && col0 >= 0, "%s: %s has %lld columns per row, fewer than col0 + H*32",
                who, name, (long long)stride);
    SSWIN_CHECK(N * stride * esz < ((int64_t)1 << 32) && stride * esz < (1 << 24) && N < (1 << 24),
                "%s: %s is too large for 32-bit row offsets", who, name);
    SSWIN_CHECK(((uintptr_t)base % 16) == 0 && (stride * esz) % 16 == 0 && (col0 * esz) % 16 == 0,
                "%s: %s rows are not 16-byte aligned", who, name);
    return 0;
}

static WAttnCommon make_common(const int32_t* tasks, int64_t g_cap, const int64_t* counts, const int32_t* tokens,
                               int64_t N, int H, int n, float scale, const float* bias, const int8_t* mask, int nmw) {
    WAttnCommon a;
    a.tasks = reinterpret_cast<const int4*>(tasks);
    a.g_cap = g_cap;
    a.first[0] = 0;
    for (int q = 0; q < 4; ++q) a.first[q + 1] = a.first[q] + counts[3 - q] * (4 - q);
    a.order = tokens;
    a.tok_pos = tokens + 3 * N;
    a.H = H;
    a.n = n;
    a.scale = scale;
    a.bias = bias;
    a.mask = mask;
    a.nmw = nmw;
    return a;
}

static int check_common(const char* who, int dtype, const int32_t* tasks, int64_t g_cap, const int64_t* counts,
                        const int32_t* tokens, int64_t N, int H, int hd, const float* bias, int n, const int8_t* mask,
                        int nmw, int64_t* total) {
    SSWIN_CHECK(hd == 32, "%s: head dimension %d is not supported (32 only)", who, hd);
    SSWIN_CHECK(dtype == SSWIN_F32 || dtype == SSWIN_F16 || dtype == SSWIN_BF16, "%s: unsupported token dtype %d", who, dtype);
    SSWIN_CHECK(N >= 0 && H > 0 && H < (1 << 23) && g_cap > 0, "%s: bad sizes", who);
    SSWIN_CHECK(n > 0 && n <= 128, "%s: windows of %d positions are not supported (128 at most)", who, n);
    SSWIN_CHECK(counts, "%s: bucket counts are null", who);
    *total = 0;
    for (int b = 0; b < WATTN_BUCKETS; ++b) {
        SSWIN_CHECK(counts[b] >= 0 && counts[b] <= g_cap, "%s: bucket %d holds %lld groups, capacity %lld", who, b,
                    (long long)counts[b], (long long)g_cap);
        *total += counts[b];
    }
    SSWIN_CHECK(*total < ((int64_t)1 << 29), "%s: %lld groups are too many for one launch", who, (long long)*total);
    if (*total == 0) return 0;
    SSWIN_CHECK(tasks && tokens && bias, "%s: null pointer", who);
    SSWIN_CHECK(!mask || nmw > 0, "%s: mask without window count", who);
    return 0;
}

}  // namespace sswin

using namespace sswin;

extern "C" {

int sswin_window_attention_forward(int dtype, const int32_t* tasks, int64_t g_cap, const int64_t* bucket_counts,
                                   const int32_t* tokens, int64_t N, int H, int hd, const void* q_base,
                                   int64_t q_stride, int q_col0, const void* k_base, int64_t k_stride, int k_col0,
                                   const void* v_base, int64_t v_stride, int v_col0, float scale, const float* bias,
                                   int n, const int8_t* mask, int n_mask_windows, void* o_base, int64_t o_stride,
                                   int o_col0, float* lse, void* stream) {
    int64_t total = 0;
    if (check_common("window_attention_forward", dtype, tasks, g_cap, bucket_counts, tokens, N, H, hd, bias, n, mask,
                     n_mask_windows, &total))
        return 1;
    if (total == 0) return 0;
    SSWIN_CHECK(q_base && k_base && v_base && o_base && lse, "window_attention_forward: null pointer");
    if (check_tensor("window_attention_forward", "q", q_base, q_stride, q_col0, N, H, dtype) ||
        check_tensor("window_attention_forward", "k", k_base, k_stride, k_col0, N, H, dtype) ||
        check_tensor("window_attention_forward", "v", v_base, v_stride, v_col0, N, H, dtype) ||
        check_tensor("window_attention_forward", "o", o_base, o_stride, o_col0, N, H, dtype))
        return 1;
    const WAttnCommon a = make_common(tasks, g_cap, bucket_counts, tokens, N, H, n, scale, bias, mask, n_mask_windows);
    const TokenTensor32 q{q_base, q_stride, q_col0}, k{k_base, k_stride, k_col0}, v{v_base, v_stride, v_col0},
        o{o_base, o_stride, o_col0};
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case SSWIN_F32: return run_forward<float>(a, q, k, v, o, lse, s);
        case SSWIN_F16: return run_forward<__half>(a, q, k, v, o, lse, s);
        case SSWIN_BF16: return run_forward<__hip_bfloat16>(a, q, k, v, o, lse, s);
        default: return fail("window_attention_forward: unsupported token dtype %d", dtype);
    }
}

int sswin_window_attention_backward(int dtype, const int32_t* tasks, int64_t g_cap, const int64_t* bucket_counts,
                                    const int32_t* tokens, int64_t N, int H, int hd, const void* q_base,
                                    int64_t q_stride, int q_col0, const void* k_base, int64_t k_stride, int k_col0,
                                    const void* v_base, int64_t v_stride, int v_col0, float scale, const float* bias,
                                    int n, const int8_t* mask, int n_mask_windows, const void* o_base,
                                    int64_t o_stride, int o_col0, const void* do_base, int64_t do_stride,
                                    int do_col0, const float* lse, void* dq_base, int64_t dq_stride, int dq_col0,
                                    void* dk_base, int64_t dk_stride, int dk_col0, void* dv_base, int64_t dv_stride,
                                    int dv_col0, float* ds_out, int sides, void* stream) {
    int64_t total = 0;
    if (check_common("window_attention_backward", dtype, tasks, g_cap, bucket_counts, tokens, N, H, hd, bias, n, mask,
                     n_mask_windows, &total))
        return 1;
    if (total == 0) return 0;
    SSWIN_CHECK(sides == 1 || sides == 2 || sides == 3, "window_attention_backward: sides must be 1 (dQ), 2 (dK, dV) or 3 (all)");
    SSWIN_CHECK(q_base && k_base && v_base && o_base && do_base && lse, "window_attention_backward: null pointer");
    SSWIN_CHECK(!(sides & 1) || dq_base, "window_attention_backward: dq is null");
    SSWIN_CHECK(!(sides & 2) || (dk_base && dv_base), "window_attention_backward: dk or dv is null");
    {
        const char* who = "window_attention_backward";
        if (check_tensor(who, "q", q_base, q_stride, q_col0, N, H, dtype) ||
            check_tensor(who, "k", k_base, k_stride, k_col0, N, H, dtype) ||
            check_tensor(who, "v", v_base, v_stride, v_col0, N, H, dtype) ||
            check_tensor(who, "o", o_base, o_stride, o_col0, N, H, dtype) ||
            check_tensor(who, "do", do_base, do_stride, do_col0, N, H, dtype))
            return 1;
        if ((sides & 1) && check_tensor(who, "dq", dq_base, dq_stride, dq_col0, N, H, dtype)) return 1;
        if ((sides & 2) && (check_tensor(who, "dk", dk_base, dk_stride, dk_col0, N, H, dtype) ||
                            check_tensor(who, "dv", dv_base, dv_stride, dv_col0, N, H, dtype)))
            return 1;
    }
    const WAttnCommon a = make_common(tasks, g_cap, bucket_counts, tokens, N, H, n, scale, bias, mask, n_mask_windows);
    const TokenTensor32 q{q_base, q_stride, q_col0}, k{k_base, k_stride, k_col0}, v{v_base, v_stride, v_col0},
        o{o_base, o_stride, o_col0}, d_o{do_base, do_stride, do_col0}, dq{dq_base, dq_stride, dq_col0},
        dk{dk_base, dk_stride, dk_col0}, dv{dv_base, dv_stride, dv_col0};
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case SSWIN_F32: return run_backward<float>(a, q, k, v, o, d_o, lse, dq, dk, dv, ds_out, sides, s);
        case SSWIN_F16: return run_backward<__half>(a, q, k, v, o, d_o, lse, dq, dk, dv, ds_out, sides, s);
        case SSWIN_BF16: return run_backward<__hip_bfloat16>(a, q, k, v, o, d_o, lse, dq, dk, dv, ds_out, sides, s);
        default: return fail("window_attention_backward: unsupported token dtype %d", dtype);
    }
}

}  // extern "C"
