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

#include <stdlib.h>

#include "wattn_common.hpp"
#include "wattn_x16.hpp"

namespace sswin {

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
// rec: the task's own token record, rec0: the record of the group's first tile
__device__ __forceinline__ FwdIdx fwd_indices(const WAttnCommon& a, int64_t rec, int64_t rec0, int l32) {
    const int2 eq = token_entry(a, rec, l32), ek = token_entry(a, rec0, l32);
    FwdIdx x;
    x.vox_i = (uint32_t)eq.x;
    x.pos_i = eq.y;
    x.k0 = KIdx{(uint32_t)ek.x, ek.y};
    return x;
}

// One forward task on one wavefront.  `mid` runs once between the last key tile and the write-out (a hook for
// work that should overlap the write-out; the plain kernel passes nothing).
template <typename T, bool MASK, typename Mid>
__device__ __forceinline__ void fwd_task(const WAttnCommon& a, const GroupCtx& g, const int bi, const int64_t rec0,
                                         const FwdIdx& fi, float* tile, float* tile_x, uint32_t* tab_key, uint32_t* tab_alpha,
                                         const TokenTensor32& tq, const TokenTensor32& tk, const TokenTensor32& tv,
                                         const TokenTensor32& to, float* __restrict__ lse, Mid&& mid) {
    const int lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    const int c = g.c, h = g.h;
    const int nt = (c + 31) >> 5;
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
        const int2 e = token_entry(a, rec0 + t, l32);
        return KIdx{(uint32_t)e.x, e.y};
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
    int64_t d, rec;
    int bi;
    if (!locate(a, (int64_t)blockIdx.x * 4 + wave, d, bi, rec)) return;
    const int4 desc = a.tasks[d];                            // descriptor and token records travel together
    const FwdIdx fi = fwd_indices(a, rec, rec - bi, lane & 31);
    const GroupCtx g = decode_group(desc);
    if constexpr (std::is_same<T, float>::value) {
        if (g.c <= 16) {
            fwd_task_small<MASK>(a, g, fi, tiles[wave][0], tiles[wave][1], tabs[wave][0], tabs[wave][1], tq, tk, tv, to, lse);
            return;
        }
    }
    fwd_task<T, MASK>(a, g, bi, rec - bi, fi, tiles[wave][0], tiles[wave][1], tabs[wave][0], tabs[wave][1], tq, tk, tv, to, lse,
                      [] {});
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
    int64_t d, rec;
    int bi;
    if (!locate(a, task, d, bi, rec)) return;
    const PadTab tab_key = pad_tab(tile, 0), tab_D = pad_tab(tile, 1);
    // the descriptor, the queries' indices and those of the first key tile: one round trip
    const int4 desc = a.tasks[d];
    const int64_t rec0 = rec - bi;
    const int2 e_q = token_entry(a, rec, l32), e_k0 = token_entry(a, rec0, l32);
    const GroupCtx g = decode_group(desc);
    const int c = g.c, h = g.h;
    const int nt = (c + 31) >> 5;
    const int8_t* mrow = MASK ? a.mask + (int64_t)(g.w % a.nmw) * a.n : nullptr;
    const char* kbase = head_base<T>(tk, h);
    const char* vbase = head_base<T>(tv, h);
    const uint32_t kpitch = pitch_of<T>(tk), vpitch = pitch_of<T>(tv);

    const int i_q = bi * 32 + l32;
    const int i_c = i_q < c ? i_q : c - 1;
    const uint32_t vox_i = (uint32_t)e_q.x;
    const int pos_i = e_q.y;
    uint32_t vox_n = (uint32_t)e_k0.x;
    int pos_n = e_k0.y;
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
        if (t + 1 < nt) {                                    // indices of the next key tile, a tile ahead
            const int2 e = token_entry(a, rec0 + t + 1, l32);
            vox_n = (uint32_t)e.x;
            pos_n = e.y;
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
//              workgroup: each forms dS K for both query tiles, query tile 0 first, and puts the partial
//              result into its LDS exchange tile; after a workgroup barrier the wavefront that owns the
//              query tile adds the two parts.  S and dP of the group are then computed once instead of
//              twice (320 instead of 448 MFMA steps of 32x32x2 per group), and because both wavefronts
//              ask for the same query tile at the same time its rows leave memory once.
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
__device__ __forceinline__ void bwd_task_small(const WAttnCommon& a, const GroupCtx& g, const int2 entry, float* tile_q,
                                               float* tile_do,
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
    // token col of the group (the last one again behind it): key of this lane's column; `entry` is the record's
    // entry lane % 32
    const int t_c = col < c ? col : c - 1;
    const uint32_t vox = (uint32_t)__shfl(entry.x, col, 64);
    const int pos = __shfl(entry.y, col, 64);
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
    int64_t d, rec;
    int bj;
    if (!live || !locate(a, task, d, bj, rec)) {
        if (DQ == KV_PAIR)
            for (int k = 0; k < 4; ++k) __syncthreads();     // the barriers of a live pair (pair_dq, twice)
        return;
    }
    const PadTab tab_pos = pad_tab(tile_q, 0), tab_L = pad_tab(tile_q, 1), tab_D = pad_tab(tile_q, 2);
    // the descriptor, the keys' indices and those of the first query tile: one round trip
    const int t_first = 0;
    const int4 desc = a.tasks[d];
    const int64_t rec0 = rec - bj;
    const int2 e_k = token_entry(a, rec, l32), e_q0 = token_entry(a, rec0 + t_first, l32);
    const GroupCtx g = decode_group(desc);
    if constexpr (DQ == KV_SINGLE && std::is_same<T, float>::value) {
        if (g.c <= 16) {
            bwd_task_small<MASK>(a, g, e_k, tile_q, tile_do, tq, tk, tv, to, tdo, lse, tdq, tdk, tdv, ds_out);
            return;
        }
    }
    const int c = g.c, h = g.h;
    const int nt = (c + 31) >> 5;
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
    auto make_qidx = [&](const int t, const int2 e) {
        const int i = t * 32 + l32;
        const int i_c = i < c ? i : c - 1;
        QIdx q;
        q.vox = (uint32_t)e.x;
        q.pos = e.y;
        q.L2 = i < c ? lse_g[i_c] * LOG2E : INFINITY;
        return q;
    };
    auto load_qidx = [&](const int t) { return make_qidx(t, token_entry(a, rec0 + t, l32)); };
    // key side: lane l32 owns key bj*32 + l32
    const int j_k = bj * 32 + l32;
    const uint32_t vox_j = (uint32_t)e_k.x;
    const int pos_j = e_k.y;
    QIdx qcur = make_qidx(t_first, e_q0);
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
    // One query tile t against this task's keys.  What happens to dS K of the tile (dq_tag): 0 = not
    // formed, 1 = written out as dQ of a one-tile group, 2 = put into this wavefront's exchange tile (KV_PAIR).
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
    // KV_PAIR: the wavefront that owns query tile `own` adds the two partial products dS K of that tile, which both
    // wavefronts have put into their exchange tiles, and writes dQ.  Workgroup barriers before (both parts are there)
    // and after the reads (the exchange tiles may be written again).
    auto pair_dq = [&](const bool own) {
        __syncthreads();
        f32x16 dq = f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        if (own) {
            xch_add(xch, lane, dq);
            xch_add(xch_peer, lane, dq);
        }
        __syncthreads();
        if (own) {
#pragma unroll
            for (int r = 0; r < 16; ++r) dq[r] *= LN2;
            tile_put_acc(tile_do, l32, half, dq);
            __builtin_amdgcn_wave_barrier();
            tile_store_rows<T>(tile_do, const_cast<char*>(head_base<T>(tdq, h)), pitch_of<T>(tdq), vox_j, c - bj * 32, lane);
            __builtin_amdgcn_wave_barrier();
        }
    };
    if constexpr (DQ == KV_PAIR) {
        // Both wavefronts of the pair take query tile 0 first and tile 1 second, so their requests for a tile's rows
        // go out together and meet in the compute unit's cache: the rows leave memory once, not twice.
        const QIdx q1 = load_qidx(1);
        tile_pass(0, qcur, std::integral_constant<int, 2>{});
        request_rows(q1);
        pair_dq(bj == 0);
        tile_pass(1, q1, std::integral_constant<int, 2>{});
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
    if constexpr (DQ == KV_PAIR) pair_dq(bj == 1);
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
        const BwdSegments sg = make_segments(a);
        hipLaunchKernelGGL((wattn_bwd_all_kernel<T, MASK>), dim3((unsigned)sg.wgs), dim3(256), 0, s, a, sg, q, k, v, o, d_o, lse,
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

// Which kernels run a call.  fp32 tokens: the kernels of this file (fp32 matrix instructions, fp32 LDS tiles);
// 16-bit tokens: the 16-bit-operand kernels of window_attention_x16.hip.  SSWIN_WATTN=x16 or SSWIN_WATTN=fp32mfma in
// the environment forces one family for every type (fp32 tokens on the 16-bit operands are split into two fp16
// pieces); read at every call.
static bool legacy_kernels(int dtype) {
    const char* e = getenv("SSWIN_WATTN");
    if (e && e[0] == 'x') return false;
    if (e && e[0] == 'f') return true;
    return dtype == SSWIN_F32;
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
    a.recs = reinterpret_cast<const int2*>(tasks + 16 * g_cap);
    a.rec_first[0] = 0;
    for (int q = 0; q < 3; ++q) a.rec_first[q + 1] = a.rec_first[q] + counts[3 - q] / H * (4 - q);
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
    if (!legacy_kernels(dtype)) {
        x16::forward(dtype, a, q, k, v, o, lse, s);
        return launch_ok("window attention forward");
    }
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
    if (!legacy_kernels(dtype)) {
        x16::backward(dtype, a, q, k, v, o, d_o, lse, dq, dk, dv, ds_out, sides, s);
        return launch_ok("window attention backward");
    }
    switch (dtype) {
        case SSWIN_F32: return run_backward<float>(a, q, k, v, o, d_o, lse, dq, dk, dv, ds_out, sides, s);
        case SSWIN_F16: return run_backward<__half>(a, q, k, v, o, d_o, lse, dq, dk, dv, ds_out, sides, s);
        case SSWIN_BF16: return run_backward<__hip_bfloat16>(a, q, k, v, o, d_o, lse, dq, dk, dv, ds_out, sides, s);
        default: return fail("window_attention_backward: unsupported token dtype %d", dtype);
    }
}

}  // extern "C"
