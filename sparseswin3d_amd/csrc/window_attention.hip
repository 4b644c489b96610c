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
//   backward Q per (group, 32 queries): recomputes S^T, dP^T = V dO^T, dS = P (dP - D) with
//              D_i = dO_i . O_i, dQ = scale dS K.
//   backward KV per (group, 32 keys): recomputes S and dP = dO V^T in the other orientation,
//              dV = P^T dO, dK = scale dS^T Q; optionally stores dS for the bias gradient.
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
#include <math.h>

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

// the head's 16-channel half of one token row as an MFMA operand run
template <typename T>
__device__ __forceinline__ void load_slice(const TokenTensor32& t, int vox, int h, int half, float (&x)[16]) {
    const T* p = static_cast<const T*>(t.base) + (int64_t)vox * t.stride + t.col0 + h * 32 + half * 16;
    load_run16_full<T>(p, x);
}

template <typename T>
__device__ __forceinline__ const T* column_ptr(const TokenTensor32& t, int h, int l32) {
    return static_cast<const T*>(t.base) + t.col0 + h * 32 + l32;
}

// ------------------------------------------------------------------------------------------
// forward
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void wattn_fwd_kernel(WAttnCommon a, TokenTensor32 tq, TokenTensor32 tk,
                                                        TokenTensor32 tv, TokenTensor32 to,
                                                        float* __restrict__ lse) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    int64_t d;
    int bi;
    if (!locate(a, (int64_t)blockIdx.x * 4 + wave, d, bi)) return;
    const GroupCtx g = load_group(a.tasks, d);
    const int c = g.c, h = g.h;
    const int nt = (c + 31) >> 5;

    // query side: lane l32 owns query bi*32 + l32 (both halves), clamped to the last token
    const int i_q = bi * 32 + l32;
    const int i_c = i_q < c ? i_q : c - 1;
    const int vox_i = a.order[g.Tk + i_c];
    const int pos_i = a.tok_pos[g.Tk + i_c];
    const int8_t* mrow = a.mask ? a.mask + (int64_t)(g.w % a.nmw) * a.n : nullptr;
    const int reg_i = mrow ? mrow[pos_i] : 0;
    float qb[16];
    load_slice<T>(tq, vox_i, h, half, qb);
#pragma unroll
    for (int s = 0; s < 16; ++s) qb[s] *= a.scale;

    const float* brow = a.bias + ((int64_t)h * a.n + pos_i) * a.n;
    const T* vcol = column_ptr<T>(tv, h, l32);
    float m = 0.f;                                           // the operator's max(0, rowmax)
    float l = 0.f;                                           // this lane half's share of the row sum
    f32x16 o = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 1
    for (int t = 0; t < nt; ++t) {
        // S^T tile: rows = keys of tile t, columns = queries
        const int j = t * 32 + l32;
        const int j_c = j < c ? j : c - 1;
        const int vox_j = a.order[g.Tk + j_c];
        const int p = a.tok_pos[g.Tk + j_c];
        const int pj = p | ((mrow ? (int)mrow[p] : 0) << 8);
        f32x16 S = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        {
            float ka[16];
            load_slice<T>(tk, vox_j, h, half, ka);
#pragma unroll
            for (int s = 0; s < 16; ++s) S = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[s], qb[s], S, 0, 0, 0);
        }
        // V in B layout: lane (ch, half) reads V[key acc_row(r, half)][ch]; bias row entries
        float vb[16], bv[16];
        int pk[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int jl = acc_row(r, half);
            vb[r] = to_acc(vcol[(int64_t)__shfl(vox_j, jl, 64) * tv.stride]);
            pk[r] = __shfl(pj, jl, 64);
            bv[r] = brow[pk[r] & 0xff];
        }
        float mt = m;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float s = S[r] + bv[r];
            if (mrow && (pk[r] >> 8) != reg_i) s += -100.0f;
            s = t * 32 + acc_row(r, half) < c ? s : -INFINITY;
            S[r] = s;
            mt = fmaxf(mt, s);
        }
        mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
        if (t > 0) {                                         // rescale what earlier tiles accumulated
            const float alpha = expf(m - mt);
            l *= alpha;
#pragma unroll
            for (int r = 0; r < 16; ++r) o[r] *= __shfl(alpha, acc_row(r, half), 64);
        }
        m = mt;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float e = expf(S[r] - m);
            l += e;
            o = __builtin_amdgcn_mfma_f32_32x32x2f32(e, vb[r], o, 0, 0, 0);
        }
    }
    l += __shfl_xor(l, 32, 64);
    l += 1e-8f;
    if (half == 0 && i_q < c) lse[(int64_t)a.H * g.Tk + h * c + i_q] = m + logf(l);
    const float inv_l = 1.0f / l;
    T* ocol = const_cast<T*>(column_ptr<T>(to, h, l32));
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int il = acc_row(r, half);
        const int vox = __shfl(vox_i, il, 64);
        const float w = __shfl(inv_l, il, 64);
        if (bi * 32 + il < c) ocol[(int64_t)vox * to.stride] = from_acc<T>(o[r] * w);
    }
}

// ------------------------------------------------------------------------------------------
// backward, query side: dQ
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void wattn_bwd_q_kernel(WAttnCommon a, TokenTensor32 tq, TokenTensor32 tk,
                                                          TokenTensor32 tv, TokenTensor32 to, TokenTensor32 tdo,
                                                          const float* __restrict__ lse, TokenTensor32 tdq) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    int64_t d;
    int bi;
    if (!locate(a, (int64_t)blockIdx.x * 4 + wave, d, bi)) return;
    const GroupCtx g = load_group(a.tasks, d);
    const int c = g.c, h = g.h;
    const int nt = (c + 31) >> 5;

    const int i_q = bi * 32 + l32;
    const int i_c = i_q < c ? i_q : c - 1;
    const int vox_i = a.order[g.Tk + i_c];
    const int pos_i = a.tok_pos[g.Tk + i_c];
    const int8_t* mrow = a.mask ? a.mask + (int64_t)(g.w % a.nmw) * a.n : nullptr;
    const int reg_i = mrow ? mrow[pos_i] : 0;
    const float L = lse[(int64_t)a.H * g.Tk + h * c + i_c];
    float qb[16], dob[16];
    load_slice<T>(tq, vox_i, h, half, qb);
    load_slice<T>(tdo, vox_i, h, half, dob);
    float D = 0.f;
    {
        float ob[16];
        load_slice<T>(to, vox_i, h, half, ob);
#pragma unroll
        for (int s = 0; s < 16; ++s) D += dob[s] * ob[s];
    }
    D += __shfl_xor(D, 32, 64);
#pragma unroll
    for (int s = 0; s < 16; ++s) qb[s] *= a.scale;

    const float* brow = a.bias + ((int64_t)h * a.n + pos_i) * a.n;
    const T* kcol = column_ptr<T>(tk, h, l32);
    f32x16 dq = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 1
    for (int t = 0; t < nt; ++t) {
        const int j = t * 32 + l32;
        const int j_c = j < c ? j : c - 1;
        const int vox_j = a.order[g.Tk + j_c];
        const int p = a.tok_pos[g.Tk + j_c];
        const int pj = p | ((mrow ? (int)mrow[p] : 0) << 8);
        f32x16 St = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        f32x16 dPt = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        {
            float ka[16], va[16];
            load_slice<T>(tk, vox_j, h, half, ka);
            load_slice<T>(tv, vox_j, h, half, va);
#pragma unroll
            for (int s = 0; s < 16; ++s) St = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[s], qb[s], St, 0, 0, 0);
#pragma unroll
            for (int s = 0; s < 16; ++s) dPt = __builtin_amdgcn_mfma_f32_32x32x2f32(va[s], dob[s], dPt, 0, 0, 0);
        }
        int pk[16];
        float bv[16], kb[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int jl = acc_row(r, half);
            pk[r] = __shfl(pj, jl, 64);
            bv[r] = brow[pk[r] & 0xff];
            kb[r] = to_acc(kcol[(int64_t)__shfl(vox_j, jl, 64) * tk.stride]);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int jg = t * 32 + acc_row(r, half);
            float s = St[r] + bv[r];
            if (mrow && (pk[r] >> 8) != reg_i) s += -100.0f;
            const float pr = jg < c ? expf(s - L) : 0.f;
            const float ds = pr * (dPt[r] - D);
            dq = __builtin_amdgcn_mfma_f32_32x32x2f32(ds, kb[r], dq, 0, 0, 0);
        }
    }
    T* ocol = const_cast<T*>(column_ptr<T>(tdq, h, l32));
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int il = acc_row(r, half);
        const int vox = __shfl(vox_i, il, 64);
        if (bi * 32 + il < c) ocol[(int64_t)vox * tdq.stride] = from_acc<T>(dq[r] * a.scale);
    }
}

// ------------------------------------------------------------------------------------------
// backward, key side: dK, dV (and dS for the bias gradient)
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void wattn_bwd_kv_kernel(WAttnCommon a, TokenTensor32 tq, TokenTensor32 tk,
                                                           TokenTensor32 tv, TokenTensor32 to, TokenTensor32 tdo,
                                                           const float* __restrict__ lse, TokenTensor32 tdk,
                                                           TokenTensor32 tdv, float* __restrict__ ds_out) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    int64_t d;
    int bj;
    if (!locate(a, (int64_t)blockIdx.x * 4 + wave, d, bj)) return;
    const GroupCtx g = load_group(a.tasks, d);
    const int c = g.c, h = g.h;
    const int nt = (c + 31) >> 5;

    // key side: lane l32 owns key bj*32 + l32
    const int j_k = bj * 32 + l32;
    const int j_c = j_k < c ? j_k : c - 1;
    const int vox_j = a.order[g.Tk + j_c];
    const int pos_j = a.tok_pos[g.Tk + j_c];
    const int8_t* mrow = a.mask ? a.mask + (int64_t)(g.w % a.nmw) * a.n : nullptr;
    const int reg_j = mrow ? mrow[pos_j] : 0;
    float kb[16], vb[16];
    load_slice<T>(tk, vox_j, h, half, kb);
    load_slice<T>(tv, vox_j, h, half, vb);

    const float* bcol = a.bias + (int64_t)h * a.n * a.n + pos_j;
    const T* docol = column_ptr<T>(tdo, h, l32);
    const T* qcol = column_ptr<T>(tq, h, l32);
    f32x16 dk = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    f32x16 dv = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 1
    for (int t = 0; t < nt; ++t) {
        // query side of tile t: lane l32 owns query t*32 + l32
        const int i = t * 32 + l32;
        const int i_c = i < c ? i : c - 1;
        const int vox_i = a.order[g.Tk + i_c];
        const int p = a.tok_pos[g.Tk + i_c];
        const int pi = p | ((mrow ? (int)mrow[p] : 0) << 8);
        const float L_i = lse[(int64_t)a.H * g.Tk + h * c + i_c];
        f32x16 St = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        f32x16 dPt = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        float D_i = 0.f;
        {
            float qa[16], doa[16], oa[16];
            load_slice<T>(tq, vox_i, h, half, qa);
            load_slice<T>(tdo, vox_i, h, half, doa);
            load_slice<T>(to, vox_i, h, half, oa);
#pragma unroll
            for (int s = 0; s < 16; ++s) D_i += doa[s] * oa[s];
#pragma unroll
            for (int s = 0; s < 16; ++s)
                St = __builtin_amdgcn_mfma_f32_32x32x2f32(qa[s] * a.scale, kb[s], St, 0, 0, 0);
#pragma unroll
            for (int s = 0; s < 16; ++s) dPt = __builtin_amdgcn_mfma_f32_32x32x2f32(doa[s], vb[s], dPt, 0, 0, 0);
        }
        D_i += __shfl_xor(D_i, 32, 64);

        // the B-layout rows of dO and Q for the two products below
        float dob[16], qbr[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int64_t vox = __shfl(vox_i, acc_row(r, half), 64);
            dob[r] = to_acc(docol[vox * tdo.stride]);
            qbr[r] = to_acc(qcol[vox * tq.stride]);
        }
        // P and dS of the tile: rows = queries acc_row(r, half), column = this lane's key
        {
            int pk[16];
            float bv[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                pk[r] = __shfl(pi, acc_row(r, half), 64);
                bv[r] = bcol[(int64_t)(pk[r] & 0xff) * a.n];
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int il = acc_row(r, half);
                const int ig = t * 32 + il;
                const bool valid = ig < c && j_k < c;
                // cross-lane reads stay outside the predicated code: every lane must take part
                const float Lr = __shfl(L_i, il, 64), Dr = __shfl(D_i, il, 64);
                float s = St[r] + bv[r];
                if (mrow && (pk[r] >> 8) != reg_j) s += -100.0f;
                const float pr = valid ? expf(s - Lr) : 0.f;
                const float ds = pr * (dPt[r] - Dr);
                if (ds_out && valid) ds_out[(int64_t)g.sq + (int64_t)ig * c + j_k] = ds;
                dv = __builtin_amdgcn_mfma_f32_32x32x2f32(pr, dob[r], dv, 0, 0, 0);     // dV += P^T dO
                dk = __builtin_amdgcn_mfma_f32_32x32x2f32(ds, qbr[r], dk, 0, 0, 0);     // dK += dS^T Q
            }
        }
    }
    T* dkcol = const_cast<T*>(column_ptr<T>(tdk, h, l32));
    T* dvcol = const_cast<T*>(column_ptr<T>(tdv, h, l32));
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int jl = acc_row(r, half);
        const int vox = __shfl(vox_j, jl, 64);
        if (bj * 32 + jl < c) {
            dkcol[(int64_t)vox * tdk.stride] = from_acc<T>(dk[r] * a.scale);
            dvcol[(int64_t)vox * tdv.stride] = from_acc<T>(dv[r]);
        }
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
    hipLaunchKernelGGL((wattn_fwd_kernel<T>), dim3(blocks), dim3(256), 0, s, a, q, k, v, o, lse);
    return launch_ok("window attention forward");
}

template <typename T>
static int run_backward(const WAttnCommon& a, const TokenTensor32& q, const TokenTensor32& k, const TokenTensor32& v,
                        const TokenTensor32& o, const TokenTensor32& d_o, const float* lse, const TokenTensor32& dq,
                        const TokenTensor32& dk, const TokenTensor32& dv, float* ds_out, int sides, hipStream_t s) {
    const unsigned blocks = (unsigned)((a.first[4] + 3) / 4);
    if (sides & 1)
        hipLaunchKernelGGL((wattn_bwd_q_kernel<T>), dim3(blocks), dim3(256), 0, s, a, q, k, v, o, d_o, lse, dq);
    if (sides & 2)
        hipLaunchKernelGGL((wattn_bwd_kv_kernel<T>), dim3(blocks), dim3(256), 0, s, a, q, k, v, o, d_o, lse, dk, dv,
                           ds_out);
    return launch_ok("window attention backward");
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

static int check_common(const char* who, const int32_t* tasks, int64_t g_cap, const int64_t* counts,
                        const int32_t* tokens, int64_t N, int H, int hd, const float* bias, int n, const int8_t* mask,
                        int nmw, int64_t* total) {
    SSWIN_CHECK(hd == 32, "%s: head dimension %d is not supported (32 only)", who, hd);
    SSWIN_CHECK(N >= 0 && H > 0 && H < (1 << 23) && g_cap > 0, "%s: bad sizes", who);
    SSWIN_CHECK(n > 0 && n <= 128, "%s: windows of %d positions are not supported (128 at most)", who, n);
    SSWIN_CHECK(counts, "%s: bucket counts are null", who);
    *total = 0;
    for (int b = 0; b < WATTN_BUCKETS; ++b) {
        SSWIN_CHECK(counts[b] >= 0 && counts[b] <= g_cap, "%s: bucket %d holds %lld groups, capacity %lld", who, b,
                    (long long)counts[b], (long long)g_cap);
        *total += counts[b];
    }
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
    if (check_common("window_attention_forward", tasks, g_cap, bucket_counts, tokens, N, H, hd, bias, n, mask,
                     n_mask_windows, &total))
        return 1;
    if (total == 0) return 0;
    SSWIN_CHECK(q_base && k_base && v_base && o_base && lse, "window_attention_forward: null pointer");
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
    if (check_common("window_attention_backward", tasks, g_cap, bucket_counts, tokens, N, H, hd, bias, n, mask,
                     n_mask_windows, &total))
        return 1;
    if (total == 0) return 0;
    SSWIN_CHECK(sides >= 1 && sides <= 3, "window_attention_backward: sides must be 1 (dQ), 2 (dK, dV) or 3");
    SSWIN_CHECK(q_base && k_base && v_base && o_base && do_base && lse, "window_attention_backward: null pointer");
    SSWIN_CHECK(!(sides & 1) || dq_base, "window_attention_backward: dq is null");
    SSWIN_CHECK(!(sides & 2) || (dk_base && dv_base), "window_attention_backward: dk or dv is null");
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
