// Window-resident attention on 16-bit matrix-core operands (gfx950, wave64).
//
// Same tasks, same launches and the same results as window_attention.hip (reference: the composition of
// sparse_swin/swin3d_base.py:660-672 forward and :106-138, :177-188 backward, softmax semantics of
// ops.cu:128-194), but every product runs on v_mfma_f32_32x32x16_{f16,bf16}:
//
//   * fp16 / bf16 tokens: the token rows go to LDS as they are and are read back directly in the
//     instruction's operand layout; nothing is unpacked to fp32 or rounded again.
//   * fp32 tokens: a tile is scaled by a power of two so that its largest value lies in [2^14, 2^15) and
//     every value x is split into two fp16 pieces, h = rtz16(x) and l = rtz16(x - h), which together
//     carry 22 significant bits (the scaling keeps the pieces of all values down to 2^-18 of the
//     tile's largest out of the fp16 subnormals).  A product is h h + h l + l h, accumulated in fp32:
//     three 16-bit matrix instructions of 32 cycles per 16 reduction steps instead of eight fp32 ones
//     of 64 cycles, and - unlike v_mfma_f32_32x32x2_f32, which occupies the SIMD's vector ALU - they run
//     beside the vector instructions of the other wavefronts.  Error per product 2-3 10^-7 of
//     sum |a b|, the same as an fp32 FMA chain.  The powers of two are taken out again where the
//     accumulators are read (they commute with everything up to the exponential).
//
// Operand layouts (lane l: l32 = l % 32, hf = l / 32; a reduction "slot" is (chunk m, hf, s), s = 0..7):
//   R  a tile X[token][channel] with lane = token l32 and slot -> channel 16 m + 8 hf + s: one
//      16-byte LDS read per chunk and piece from a row-major 16-bit tile.
//   C  the accumulator layout of a 32 x 32 result: lane = column l32, register r = row acc_row(r, hf).
//      Registers 8 m + s of a lane, packed in pairs, ARE an operand with slot -> row acc_row(8 m + s, hf).
//   T  a tile X[token][channel] with lane = channel l32 and slot -> token acc_row(8 m + s, hf): the
//      operand of the products that reduce over tokens.  It is X in layout C, and X in layout R times an
//      identity operand is exactly that: the transposition is two matrix instructions per piece
//      (exact: every output is one input value times one) and no LDS traffic.  The same trick turns
//      dS^T (layout C, queries in the registers) into the operand of dQ = dS K.
//
// LDS per wavefront: two tiles of 32 rows x 36 dwords.  A row holds the h pieces of its 32 channels in
// dwords 0-15, the l pieces in dwords 16-31 (fp32 tokens only) and four table entries in dwords
// 32-35; the same memory stages fp32 accumulators (32 values per row) for the coalesced row stores.
#include "wattn_common.hpp"
#include "wattn_x16.hpp"

#ifndef X16_BWD_WAVES
#define X16_BWD_WAVES 3
#endif
#ifndef X16_FWD_WAVES
#define X16_FWD_WAVES 4
#endif

namespace sswin {
namespace x16 {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2_a __attribute__((ext_vector_type(2)));

template <typename T> struct Mode;
template <> struct Mode<float> {
    static constexpr int NP = 2;            // pieces per value
    static constexpr bool SPLIT = true;
    static constexpr bool BF = false;
    static constexpr int PSH = 14;          // attention probabilities are held as P 2^14
};
template <> struct Mode<__half> {
    static constexpr int NP = 1;
    static constexpr bool SPLIT = false;
    static constexpr bool BF = false;
    static constexpr int PSH = 0;
};
template <> struct Mode<__hip_bfloat16> {
    static constexpr int NP = 1;
    static constexpr bool SPLIT = false;
    static constexpr bool BF = true;
    static constexpr int PSH = 0;
};

template <typename T>
__device__ __forceinline__ f32x16 mfma16(const u32x4_a& a, const u32x4_a& b, const f32x16& c) {
    if constexpr (Mode<T>::BF)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

__device__ __forceinline__ GroupCtx decode_group(const int4& t) {
    GroupCtx g;
    g.Tk = __builtin_amdgcn_readfirstlane(t.x);
    g.c = __builtin_amdgcn_readfirstlane(t.y & 0xff);
    g.h = __builtin_amdgcn_readfirstlane(t.y >> 8);
    g.w = __builtin_amdgcn_readfirstlane(t.z);
    g.sq = __builtin_amdgcn_readfirstlane(t.w);
    return g;
}

__device__ __forceinline__ f32x16 zero16() { return f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}; }

// an operand of 32 reduction slots per lane: [chunk][piece] of eight packed 16-bit values
template <int NP>
struct Opnd {
    u32x4_a v[2][NP];
};

// acc += a . b over `chunks` chunks of 16 slots; split values: l h + h l + h h
template <typename T>
__device__ __forceinline__ f32x16 mma(const Opnd<Mode<T>::NP>& a, const Opnd<Mode<T>::NP>& b, f32x16 acc, int chunks = 2) {
    if constexpr (Mode<T>::SPLIT) {
        acc = mfma16<T>(a.v[0][1], b.v[0][0], acc);
        acc = mfma16<T>(a.v[0][0], b.v[0][1], acc);
    }
    acc = mfma16<T>(a.v[0][0], b.v[0][0], acc);
    if (chunks > 1) {
        if constexpr (Mode<T>::SPLIT) {
            acc = mfma16<T>(a.v[1][1], b.v[1][0], acc);
            acc = mfma16<T>(a.v[1][0], b.v[1][1], acc);
        }
        acc = mfma16<T>(a.v[1][0], b.v[1][0], acc);
    }
    return acc;
}

// two values -> one dword of the operand type.  pack_rt rounds (fp16: toward zero, one instruction
// for both; bf16: to nearest), pack_exact is for values known to be representable.
__device__ __forceinline__ uint32_t pkrtz(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
}
template <typename T>
__device__ __forceinline__ uint32_t pack_rt(float a, float b) {
    if constexpr (Mode<T>::BF) {
        const bf16x2 v = {(__bf16)a, (__bf16)b};
        return __builtin_bit_cast(uint32_t, v);
    } else {
        return pkrtz(a, b);
    }
}
template <typename T>
__device__ __forceinline__ uint32_t pack_exact(float a, float b) {
    if constexpr (Mode<T>::BF)
        return __builtin_amdgcn_perm(f2u(b), f2u(a), 0x07060302u);       // the upper halves of b and a
    else
        return pkrtz(a, b);
}
// y (already scaled) -> h = rtz16(y), l = rtz16(y - h), two values at a time
__device__ __forceinline__ void split2(float y0, float y1, uint32_t& h, uint32_t& l) {
    h = pkrtz(y0, y1);
    const f16x2 hv = __builtin_bit_cast(f16x2, h);
    l = pkrtz(y0 - (float)hv[0], y1 - (float)hv[1]);
}

__device__ __forceinline__ float pow2f(int e) { return u2f((uint32_t)(e + 127) << 23); }   // |e| <= 126
__device__ __forceinline__ float ldexp_fast(float x, int e) { return __builtin_amdgcn_ldexpf(x, e); }

// max(|a|, |b|, m) in one instruction (the library's fmaxf would quiet each operand first)
__device__ __forceinline__ float max3abs(float a, float b, float m) {
    float r;
    asm("v_max3_f32 %0, |%1|, |%2|, %3" : "=v"(r) : "v"(a), "v"(b), "v"(m));
    return r;
}
// Exponent sh of the power of two that brings the wavefront's largest |value| into [2^14, 2^15); 0 for a
// tile of zeros.  `m` is each lane's largest |value| (>= 0: such floats order like their bit patterns).
// Uniform result.
__device__ __forceinline__ int scale_exp(float m) {
    int b = (int)f2u(m);
    b = max(b, dpp_i32<0xB1>(b));
    b = max(b, dpp_i32<0x4E>(b));
    b = max(b, dpp_i32<0x141>(b));
    b = max(b, dpp_i32<0x140>(b));
    const int b0 = __builtin_amdgcn_readlane(b, 0), b1 = __builtin_amdgcn_readlane(b, 16);
    const int b2 = __builtin_amdgcn_readlane(b, 32), b3 = __builtin_amdgcn_readlane(b, 48);
    const int bm = max(max(b0, b1), max(b2, b3));
    const int E = bm >> 23;
    const int sh = 141 - E;
    return E == 0 ? 0 : (sh < -100 ? -100 : (sh > 100 ? 100 : sh));
}
__device__ __forceinline__ float amax_rows(const RowLoad<float>& r) {
    float m = 0.f;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        m = max3abs(u2f(r.v[v].x), u2f(r.v[v].y), m);
        m = max3abs(u2f(r.v[v].z), u2f(r.v[v].w), m);
    }
    return m;
}
template <typename T>
__device__ __forceinline__ int tile_exp(const RowLoad<T>& r) {
    if constexpr (Mode<T>::SPLIT) return scale_exp(amax_rows(r));
    return 0;
}

// token rows (coalesced pieces) -> 16-bit LDS tile; rows at or beyond `valid` are written as zeros.
// fp32: scaled by 2^sh and split.
template <typename T>
__device__ __forceinline__ void rows_to_tile16(float* tile, int lane, const RowLoad<T>& r, int sh, int valid) {
    uint32_t* t = reinterpret_cast<uint32_t*>(tile);
    if constexpr (Mode<T>::SPLIT) {
        const float f = pow2f(sh);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int R = v * 8 + lane / 8;
            uint32_t h0, l0, h1, l1;
            split2(u2f(r.v[v].x) * f, u2f(r.v[v].y) * f, h0, l0);
            split2(u2f(r.v[v].z) * f, u2f(r.v[v].w) * f, h1, l1);
            u32x2_a h = {h0, h1}, l = {l0, l1};
            if (R >= valid) h = l = u32x2_a{0, 0};
            *reinterpret_cast<u32x2_a*>(t + R * TILE_LD + (lane % 8) * 2) = h;
            *reinterpret_cast<u32x2_a*>(t + R * TILE_LD + 16 + (lane % 8) * 2) = l;
        }
    } else {
#pragma unroll
        for (int v = 0; v < 2; ++v) {
            const int R = v * 16 + lane / 4;
            u32x4_a x = r.v[v];
            if (R >= valid) x = u32x4_a{0, 0, 0, 0};
            *reinterpret_cast<u32x4_a*>(t + R * TILE_LD + (lane % 4) * 4) = x;
        }
    }
}
// layout R of a tile: lane = token l32, slot (m, hf, s) -> channel 16 m + 8 hf + s
template <typename T>
__device__ __forceinline__ Opnd<Mode<T>::NP> read_R(const float* tile, int l32, int hf) {
    const u32x4_a* p = reinterpret_cast<const u32x4_a*>(tile + l32 * TILE_LD + 4 * hf);
    Opnd<Mode<T>::NP> o;
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int pc = 0; pc < Mode<T>::NP; ++pc) o.v[m][pc] = p[4 * pc + 2 * m];
    return o;
}
// identity operands: KIND 0: slot -> 16 m + 8 hf + s (the channels of layout R), KIND 1: slot -> acc_row(8 m + s, hf)
template <typename T, int KIND>
__device__ __forceinline__ void make_ident(int l32, int hf, u32x4_a (&id)[2]) {
    constexpr uint32_t ONE = Mode<T>::BF ? 0x3f80u : 0x3c00u;
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int i0 = KIND == 0 ? 16 * m + 8 * hf + 2 * p : acc_row(8 * m + 2 * p, hf);
            id[m][p] = (i0 == l32 ? ONE : 0u) | (i0 + 1 == l32 ? ONE << 16 : 0u);      // acc_row(r + 1) = acc_row(r) + 1 for even r
        }
}
// accumulator (layout C) -> operand registers 8 m + s, values known to be representable
template <typename T>
__device__ __forceinline__ void pack_acc_exact(const f32x16& acc, u32x4_a& c0, u32x4_a& c1) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        c0[p] = pack_exact<T>(acc[2 * p], acc[2 * p + 1]);
        c1[p] = pack_exact<T>(acc[8 + 2 * p], acc[8 + 2 * p + 1]);
    }
}
// x (any operand, "rows" = its lanes) times the identity of the slot mapping it was built with: the same
// matrix with lanes and slots exchanged (slot -> acc_row of the former lane index)
template <typename T, int KIND>
__device__ __forceinline__ Opnd<Mode<T>::NP> transpose(const Opnd<Mode<T>::NP>& x, int l32, int hf) {
    u32x4_a id[2];
    make_ident<T, KIND>(l32, hf, id);
    Opnd<Mode<T>::NP> o;
#pragma unroll
    for (int pc = 0; pc < Mode<T>::NP; ++pc) {
        f32x16 acc = mfma16<T>(x.v[0][pc], id[0], zero16());
        acc = mfma16<T>(x.v[1][pc], id[1], acc);
        pack_acc_exact<T>(acc, o.v[0][pc], o.v[1][pc]);
    }
    return o;
}
// values in layout C (scaled by f) -> operand with slot -> row acc_row(8 m + s, hf)
template <typename T>
__device__ __forceinline__ Opnd<Mode<T>::NP> pack_C(const float (&x)[16], float f) {
    Opnd<Mode<T>::NP> o;
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const float y0 = x[8 * m + 2 * p] * f, y1 = x[8 * m + 2 * p + 1] * f;
            if constexpr (Mode<T>::SPLIT) {
                uint32_t hh, ll;
                split2(y0, y1, hh, ll);
                o.v[m][0][p] = hh;
                o.v[m][1][p] = ll;
            } else {
                o.v[m][0][p] = pack_rt<T>(y0, y1);
            }
        }
    return o;
}
// two neighbouring registers of layout C -> dword p of chunk m of an operand
template <typename T>
__device__ __forceinline__ void pack_pair(Opnd<Mode<T>::NP>& o, int m, int p, float y0, float y1) {
    if constexpr (Mode<T>::SPLIT) {
        uint32_t hh, ll;
        split2(y0, y1, hh, ll);
        o.v[m][0][p] = hh;
        o.v[m][1][p] = ll;
    } else {
        o.v[m][0][p] = pack_rt<T>(y0, y1);
    }
}
template <typename T>
__device__ __forceinline__ void clear_chunk(Opnd<Mode<T>::NP>& o, int m) {
#pragma unroll
    for (int pc = 0; pc < Mode<T>::NP; ++pc) o.v[m][pc] = u32x4_a{0, 0, 0, 0};
}
__device__ __forceinline__ float amax_acc(const f32x16& x, int n) {
    float m = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r += 2)
        if (r < n) m = max3abs(x[r], x[r + 1], m);
    return m;
}
// acc in units of 2^-from -> units of 2^-to
__device__ __forceinline__ void rescale(f32x16& acc, int from, int to) {
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = ldexp_fast(acc[r], to - from);
}
// table[row] = f * (x_row . y_row)
template <typename T>
__device__ __forceinline__ void rows_dot_to_table_scaled(const PadTab& tab, int lane, const RowLoad<T>& x, const RowLoad<T>& y, float f) {
    constexpr int CH = RowLoad<T>::CH, ROWS = RowLoad<T>::ROWS;
#pragma unroll
    for (int v = 0; v < RowLoad<T>::NI; ++v) {
        float d = chunk_dot<T>(x.v[v], y.v[v]);
        d += dpp_f32<0xB1>(d);
        d += dpp_f32<0x4E>(d);
        if (CH == 8) d += dpp_f32<0x141>(d);
        if (lane % CH == 0) tab.put(v * ROWS + lane / CH, f2u(d * f));
    }
}

// ------------------------------------------------------------------------------------------
// forward: one task = 32 queries of a group against all its keys.  S^T = K Q^T (keys in the registers,
// queries in the lanes), softmax in registers with online rescaling across key tiles, O = P V with P
// taken from the registers and V in layout T.
// ------------------------------------------------------------------------------------------
template <typename T, bool MASK>
__device__ __forceinline__ void fwd_task(const WAttnCommon& a, const GroupCtx& g, const int bi, const int64_t rec0,
                                         const int2 e_q, const int2 e_k0, float* tile, float* tile_x,
                                         const TokenTensor32& tq, const TokenTensor32& tk, const TokenTensor32& tv,
                                         const TokenTensor32& to, float* __restrict__ lse) {
    constexpr int PSH = Mode<T>::PSH;
    typedef Opnd<Mode<T>::NP> Op;
    const int lane = threadIdx.x & 63;
    const int hf = lane >> 5, l32 = lane & 31;
    const int c = g.c, h = g.h;
    const int nt = (c + 31) >> 5;
    const int8_t* mrow = MASK ? a.mask + (int64_t)(g.w % a.nmw) * a.n : nullptr;
    const char* kbase = head_base<T>(tk, h);
    const char* vbase = head_base<T>(tv, h);
    const uint32_t kpitch = pitch_of<T>(tk), vpitch = pitch_of<T>(tv);
    const PadTab tab_key = pad_tab(tile, 0), tab_alpha = pad_tab(tile, 1);

    const int i_q = bi * 32 + l32;
    const uint32_t vox_i = (uint32_t)e_q.x;
    const int pos_i = e_q.y;
    auto load_kidx = [&](const int t, uint32_t& vox, int& pos) {
        const int2 e = token_entry(a, rec0 + t, l32);
        vox = (uint32_t)e.x;
        pos = e.y;
    };
    uint32_t vox_j = (uint32_t)e_k0.x;
    int pos_j = e_k0.y;
    const int reg_i = MASK ? mrow[pos_i] : 0;
    const char* bias_h = reinterpret_cast<const char*>(a.bias + (int64_t)h * a.n * a.n);
    const uint32_t brow = (uint32_t)(pos_i * a.n) * 4u;
    RowLoad<T> rk, rv, rq;
    Op qR;
    int aQ = 0;
    uint32_t vox_n = vox_j;
    int pos_n = pos_j;

    float m = 0.f;                                           // the operator's max(0, rowmax), in units of log 2
    float l = 0.f;                                           // this lane half's share of the row sum, times 2^PSH
    f32x16 o = zero16();
    int xo = 0;                                              // o is in units of 2^-xo
#pragma unroll 1
    for (int t = 0; t < nt; ++t) {
        // Order of the requests of a tile: the key's mask region, the rows, then - while the rows travel - the
        // positions go through the LDS table and the 16 bias gathers go out; they are read after the score product.
        if (t > 0) {
            vox_j = vox_n;
            pos_j = pos_n;
        }
        const int reg_k = MASK ? mrow[pos_j] : 0;
        if (t == 0) rows_load<T>(head_base<T>(tq, h), pitch_of<T>(tq), vox_i, lane, rq);
        rows_load<T>(kbase, kpitch, vox_j, lane, rk);
        rows_load<T>(vbase, vpitch, vox_j, lane, rv);
        if (t + 1 < nt) load_kidx(t + 1, vox_n, pos_n);      // the indices of the next tile, a tile ahead
        __builtin_amdgcn_wave_barrier();
        table_put(tab_key, l32, (uint32_t)pos_j * 4u | (uint32_t)reg_k << 16);
        __builtin_amdgcn_wave_barrier();
        float bv[16];
        uint32_t differ = 0;                                  // bit r: regions of the query and the key differ
        {
            uint32_t pkr[16];
            table_get(tab_key, hf, pkr);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                bv[r] = *reinterpret_cast<const float*>(bias_h + (brow + (MASK ? (pkr[r] & 0xffffu) : pkr[r])));
                if (MASK) differ |= ((int)(pkr[r] >> 16) != reg_i ? 1u : 0u) << r;
            }
        }
        if (t == 0) {
            aQ = tile_exp<T>(rq);
            rows_to_tile16<T>(tile_x, lane, rq, aQ, 32);
            __builtin_amdgcn_wave_barrier();
            qR = read_R<T>(tile_x, l32, hf);
            __builtin_amdgcn_wave_barrier();
        }
        const int bK = tile_exp<T>(rk), cV = tile_exp<T>(rv);
        rows_to_tile16<T>(tile, lane, rk, bK, 32);
        rows_to_tile16<T>(tile_x, lane, rv, cV, 32);
        __builtin_amdgcn_wave_barrier();
        f32x16 S;
        {
            const Op kR = read_R<T>(tile, l32, hf);
            S = mma<T>(kR, qR, zero16());                    // S^T tile: rows = keys, columns = queries
        }
        const float c_s = ldexp_fast(a.scale, -(aQ + bK));
        const int kleft = c - t * 32;
        const int jlim = kleft - 4 * hf;                     // keys acc_row(r, 0) >= jlim are padding
        float mt = m;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float s = fmaf(S[r], c_s, bv[r]);
            if (MASK && (differ >> r & 1u)) s += -100.0f;
            s = (8 * (r >> 2) + (r & 3)) < jlim ? s * LOG2E : -INFINITY;
            S[r] = s;
            mt = fmaxf(mt, s);
        }
        mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
        const int nxo = PSH + cV;
        if (t > 0) {                                         // rescale what earlier tiles accumulated
            const float alpha = exp2_fast(m - mt);
            l *= alpha;
            __builtin_amdgcn_wave_barrier();
            table_put(tab_alpha, l32, f2u(ldexp_fast(alpha, nxo - xo)));
            __builtin_amdgcn_wave_barrier();
            uint32_t ar[16];
            table_get(tab_alpha, hf, ar);
#pragma unroll
            for (int r = 0; r < 16; ++r) o[r] *= u2f(ar[r]);
        }
        xo = nxo;
        m = mt;
        const float moff = m - (float)PSH;
        Op Pp;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
            const float p0 = exp2_fast(S[r] - moff), p1 = exp2_fast(S[r + 1] - moff);
            l += p0 + p1;
            pack_pair<T>(Pp, r >> 3, (r & 7) >> 1, p0, p1);
        }
        const Op vT = transpose<T, 0>(read_R<T>(tile_x, l32, hf), l32, hf);
        o = mma<T>(Pp, vT, o, kleft > 16 ? 2 : 1);
    }
    l += __shfl_xor(l, 32, 64);
    l = ldexp_fast(l, -PSH) + 1e-8f;
    if (hf == 0 && i_q < c) lse[(int64_t)a.H * g.Tk + h * c + i_q] = (m + __builtin_amdgcn_logf(l)) * LN2;
    // normalise (one factor per query row, through the table), accumulators -> LDS rows -> coalesced stores
    __builtin_amdgcn_wave_barrier();
    table_put(tab_alpha, l32, f2u(ldexp_fast(1.0f / l, -xo)));
    __builtin_amdgcn_wave_barrier();
    uint32_t ir[16];
    table_get(tab_alpha, hf, ir);
#pragma unroll
    for (int r = 0; r < 16; ++r) o[r] *= u2f(ir[r]);
    tile_put_acc(tile_x, l32, hf, o);
    __builtin_amdgcn_wave_barrier();
    tile_store_rows<T>(tile_x, const_cast<char*>(head_base<T>(to, h)), pitch_of<T>(to), vox_i, c - bi * 32, lane);
}

template <typename T, bool MASK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(X16_FWD_WAVES, X16_FWD_WAVES))) void wattn16_fwd_kernel(
    WAttnCommon a, TokenTensor32 tq, TokenTensor32 tk, TokenTensor32 tv, TokenTensor32 to, float* __restrict__ lse) {
    __shared__ __attribute__((aligned(16))) float tiles[4][2][TILE_WORDS];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int64_t d, rec;
    int bi;
    if (!locate(a, xcd_run_order(blockIdx.x) * 4 + wave, d, bi, rec)) return;
    // the descriptor, the queries' indices and those of the first key tile: one round trip
    const int4 desc = a.tasks[d];
    const int l32 = threadIdx.x & 31;
    const int2 e_q = token_entry(a, rec, l32), e_k0 = token_entry(a, rec - bi, l32);
    const GroupCtx g = decode_group(desc);
    fwd_task<T, MASK>(a, g, bi, rec - bi, e_q, e_k0, tiles[wave][0], tiles[wave][1], tq, tk, tv, to, lse);
}

// ------------------------------------------------------------------------------------------
// backward, query side (groups of three and four tiles): dQ of 32 queries.  S^T and dP^T with the keys
// in the registers; dS^T from the registers is the operand of dQ = dS K, K in layout T.
// ------------------------------------------------------------------------------------------
template <typename T, bool MASK>
__device__ __forceinline__ void bwd_q_task(const WAttnCommon& a, int64_t task, float* tile, float* tile_x,
                                           const TokenTensor32& tq, const TokenTensor32& tk, const TokenTensor32& tv,
                                           const TokenTensor32& to, const TokenTensor32& tdo,
                                           const float* __restrict__ lse, const TokenTensor32& tdq) {
    constexpr int PSH = Mode<T>::PSH;
    typedef Opnd<Mode<T>::NP> Op;
    const int lane = threadIdx.x & 63;
    const int hf = lane >> 5, l32 = lane & 31;
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
    const float Lm = lse[(int64_t)a.H * g.Tk + h * c + i_c] * LOG2E - (float)PSH;
    Op qR, doR;
    int aQ, eO;
    {
        RowLoad<T> rq, rdo, ro;
        rows_load<T>(head_base<T>(tq, h), pitch_of<T>(tq), vox_i, lane, rq);
        rows_load<T>(head_base<T>(tdo, h), pitch_of<T>(tdo), vox_i, lane, rdo);
        rows_load<T>(head_base<T>(to, h), pitch_of<T>(to), vox_i, lane, ro);
        aQ = tile_exp<T>(rq);
        eO = tile_exp<T>(rdo);
        rows_to_tile16<T>(tile_x, lane, rq, aQ, 32);
        rows_dot_to_table_scaled<T>(tab_D, lane, rdo, ro, pow2f(-PSH));       // D_i = dO_i . O_i, times 2^-PSH
        __builtin_amdgcn_wave_barrier();
        qR = read_R<T>(tile_x, l32, hf);
        __builtin_amdgcn_wave_barrier();
        rows_to_tile16<T>(tile_x, lane, rdo, eO, 32);
        __builtin_amdgcn_wave_barrier();
        doR = read_R<T>(tile_x, l32, hf);
    }
    const float D = u2f(tab_D.get(l32));
    const char* bias_h = reinterpret_cast<const char*>(a.bias + (int64_t)h * a.n * a.n);
    const uint32_t brow = (uint32_t)(pos_i * a.n) * 4u;

    f32x16 dq = zero16();
    int xq = 0;
    RowLoad<T> rk, rv;
    uint32_t vox_j = vox_n;                                  // indices of the current key tile, vox_n / pos_n: of the next
    int pos_j = pos_n;
#pragma unroll 1
    for (int t = 0; t < nt; ++t) {
        // Order of the requests of a tile: the key's mask region, the rows, the indices of the next tile; then -
        // while the rows travel - the positions go through the LDS table and the 16 bias gathers go out; they are
        // read after the two score products.
        const int reg_k = MASK ? mrow[pos_j] : 0;
        rows_load<T>(kbase, kpitch, vox_j, lane, rk);
        rows_load<T>(vbase, vpitch, vox_j, lane, rv);
        if (t + 1 < nt) {
            const int2 e = token_entry(a, rec0 + t + 1, l32);
            vox_n = (uint32_t)e.x;
            pos_n = e.y;
        }
        __builtin_amdgcn_wave_barrier();
        table_put(tab_key, l32, (uint32_t)pos_j * 4u | (uint32_t)reg_k << 16);
        __builtin_amdgcn_wave_barrier();
        float bv[16];
        uint32_t differ = 0;                                  // bit r: regions of the query and the key differ
        {
            uint32_t pkr[16];
            table_get(tab_key, hf, pkr);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                bv[r] = *reinterpret_cast<const float*>(bias_h + (brow + (MASK ? (pkr[r] & 0xffffu) : pkr[r])));
                if (MASK) differ |= ((int)(pkr[r] >> 16) != reg_i ? 1u : 0u) << r;
            }
        }
        const int bK = tile_exp<T>(rk), cV = tile_exp<T>(rv);
        const int kleft = c - t * 32;
        rows_to_tile16<T>(tile, lane, rk, bK, kleft);        // padding keys as zero rows: nothing of them reaches dQ
        rows_to_tile16<T>(tile_x, lane, rv, cV, 32);
        __builtin_amdgcn_wave_barrier();
        vox_j = vox_n;
        pos_j = pos_n;
        f32x16 St, dPt;
        {
            const Op kR = read_R<T>(tile, l32, hf);
            St = mma<T>(kR, qR, zero16());
        }
        {
            const Op vR = read_R<T>(tile_x, l32, hf);
            dPt = mma<T>(vR, doR, zero16());
        }
        const float c_s = ldexp_fast(a.scale, -(aQ + bK));
        const float c_p = ldexp_fast(1.0f, -(eO + cV + PSH));
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float s = fmaf(St[r], c_s, bv[r]);
            if (MASK && (differ >> r & 1u)) s += -100.0f;
            St[r] = exp2_fast(fmaf(s, LOG2E, -Lm));          // P 2^PSH (padding keys: finite, multiplied by zero rows of K)
            dPt[r] = fmaf(dPt[r], c_p, -D);                  // (dP - D) 2^-PSH
        }
        // |dS| <= max |dP - D|: the scale of the dS operand is taken from there, so dS is packed as it is formed
        const int eS = Mode<T>::SPLIT ? scale_exp(amax_acc(dPt, 16)) - PSH : 0;
        const float fS = pow2f(eS);
        Op dSp;
#pragma unroll
        for (int r = 0; r < 16; r += 2)
            pack_pair<T>(dSp, r >> 3, (r & 7) >> 1, St[r] * dPt[r] * fS, St[r + 1] * dPt[r + 1] * fS);
        const Op kT = transpose<T, 0>(read_R<T>(tile, l32, hf), l32, hf);
        const int nxq = eS + bK;
        if (Mode<T>::SPLIT && t > 0 && nxq != xq) rescale(dq, xq, nxq);
        xq = nxq;
        dq = mma<T>(dSp, kT, dq, kleft > 16 ? 2 : 1);
    }
    const float fq = ldexp_fast(a.scale, -xq);
#pragma unroll
    for (int r = 0; r < 16; ++r) dq[r] *= fq;
    __builtin_amdgcn_wave_barrier();
    tile_put_acc(tile_x, l32, hf, dq);
    __builtin_amdgcn_wave_barrier();
    tile_store_rows<T>(tile_x, const_cast<char*>(head_base<T>(tdq, h)), pitch_of<T>(tdq), vox_i, c - bi * 32, lane);
}

// ------------------------------------------------------------------------------------------
// backward, key side: dK, dV (and dS for the bias gradient) of 32 keys; S and dP with the queries in the
// registers, so P and dS are the operands of dV = P^T dO and dK = dS^T Q as they stand, dO and Q in
// layout T.  What a task does about dQ (the modes of window_attention.hip):
//   KV_ONLY    nothing (the group has query-side tasks of its own)
//   KV_SINGLE  a group of one tile: dS^T through the identity product is the operand of dQ = dS K
//   KV_PAIR    a group of two tiles, its two key-side tasks on neighbouring wavefronts of one workgroup:
//              each forms dS K for both query tiles and hands the part of the other wavefront's tile over
//              through an LDS exchange tile
// ------------------------------------------------------------------------------------------
enum { KV_ONLY = 0, KV_SINGLE = 1, KV_PAIR = 2 };

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

template <typename T, bool MASK, int DQ>
__device__ __forceinline__ void bwd_kv_task(const WAttnCommon& a, int64_t task, bool live, float* tile_q, float* tile_do,
                                            float* xch, const float* xch_peer,
                                            const TokenTensor32& tq, const TokenTensor32& tk, const TokenTensor32& tv,
                                            const TokenTensor32& to, const TokenTensor32& tdo,
                                            const float* __restrict__ lse, const TokenTensor32& tdk,
                                            const TokenTensor32& tdv, float* __restrict__ ds_out,
                                            const TokenTensor32& tdq) {
    constexpr int PSH = Mode<T>::PSH;
    constexpr bool SPLIT = Mode<T>::SPLIT;
    typedef Opnd<Mode<T>::NP> Op;
    const int lane = threadIdx.x & 63;
    const int hf = lane >> 5, l32 = lane & 31;
    int64_t d, rec;
    int bj;
    if (!live || !locate(a, task, d, bj, rec)) {
        if (DQ == KV_PAIR) __syncthreads();
        return;
    }
    const PadTab tab_pos = pad_tab(tile_q, 0), tab_L = pad_tab(tile_q, 1), tab_D = pad_tab(tile_q, 2);
    // the descriptor, the keys' indices and those of the first query tile: one round trip
    const int t_first = DQ == KV_PAIR ? 1 - bj : 0;           // KV_PAIR: the other wavefront's query tile first
    const int4 desc = a.tasks[d];
    const int64_t rec0 = rec - bj;
    const int2 e_k = token_entry(a, rec, l32), e_q0 = token_entry(a, rec0 + t_first, l32);
    const GroupCtx g = decode_group(desc);
    const int c = g.c, h = g.h;
    const int nt = (c + 31) >> 5;
    const int8_t* mrow = MASK ? a.mask + (int64_t)(g.w % a.nmw) * a.n : nullptr;
    const char* qbase = head_base<T>(tq, h);
    const char* obase = head_base<T>(to, h);
    const char* dobase = head_base<T>(tdo, h);
    const uint32_t qpitch = pitch_of<T>(tq), opitch = pitch_of<T>(to), dopitch = pitch_of<T>(tdo);
    const float* lse_g = lse + (int64_t)a.H * g.Tk + h * c;

    struct QIdx {
        uint32_t vox;        // voxel of query t*32 + l32 (clamped to the last token)
        int pos;
        float Lm;            // its log-sum-exp in units of log 2, minus PSH; +inf for padding queries: P and dS exactly zero
    };
    auto make_qidx = [&](const int t, const int2 e) {
        const int i = t * 32 + l32;
        const int i_c = i < c ? i : c - 1;
        QIdx q;
        q.vox = (uint32_t)e.x;
        q.pos = e.y;
        q.Lm = i < c ? lse_g[i_c] * LOG2E - (float)PSH : INFINITY;
        return q;
    };
    auto load_qidx = [&](const int t) { return make_qidx(t < nt ? t : nt - 1, token_entry(a, rec0 + (t < nt ? t : nt - 1), l32)); };
    // key side: lane l32 owns key bj*32 + l32
    const int j_k = bj * 32 + l32;
    const uint32_t vox_j = (uint32_t)e_k.x;
    const int pos_j = e_k.y;
    QIdx qcur = make_qidx(t_first, e_q0);
    const int reg_j = MASK ? mrow[pos_j] : 0;
    const int kleft = c - bj * 32;                            // keys of this task
    const char* bias_h = reinterpret_cast<const char*>(a.bias + (int64_t)h * a.n * a.n);
    const uint32_t bcol = (uint32_t)pos_j * 4u;
    float* ds_g = ds_out ? ds_out + g.sq + j_k : nullptr;

    // The requests of a query tile, in this order: the mask regions of its positions, its rows (request_rows);
    // then - while the rows travel - positions and log-sum-exps go through the LDS tables and the 16 bias
    // gathers go out (bias_ahead); they are read after the two score products of the tile.
    RowLoad<T> rq, rdo, ro;
    int reg_q = 0;
    float bv[16];
    uint32_t differ = 0;                                      // bit r: regions of row r and of the key differ
    constexpr bool ONCE = DQ == KV_SINGLE;                    // a group of one tile: nobody else reads these rows
    auto request_rows = [&](const QIdx& qi) {
        reg_q = MASK ? mrow[qi.pos] : 0;
        rows_load<T, ONCE>(qbase, qpitch, qi.vox, lane, rq);
        rows_load<T, ONCE>(dobase, dopitch, qi.vox, lane, rdo);
        rows_load<T, ONCE>(obase, opitch, qi.vox, lane, ro);
    };
    auto bias_ahead = [&](const QIdx& qi) {
        __builtin_amdgcn_wave_barrier();
        table_put(tab_pos, l32, (uint32_t)(qi.pos * a.n) * 4u | (uint32_t)reg_q << 16);   // byte offset of the bias row (< 2^16)
        table_put(tab_L, l32, f2u(qi.Lm));
        __builtin_amdgcn_wave_barrier();
        uint32_t pir[16];
        table_get(tab_pos, hf, pir);
        differ = 0;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            bv[r] = *reinterpret_cast<const float*>(bias_h + (bcol + (MASK ? (pir[r] & 0xffffu) : pir[r])));
            if (MASK) differ |= ((int)(pir[r] >> 16) != reg_j ? 1u : 0u) << r;
        }
    };
    Op kR, vR, kT_single;
    int bK, cV;
    {
        RowLoad<T> rk, rv;
        rows_load<T, ONCE>(head_base<T>(tk, h), pitch_of<T>(tk), vox_j, lane, rk);
        rows_load<T, ONCE>(head_base<T>(tv, h), pitch_of<T>(tv), vox_j, lane, rv);
        request_rows(qcur);
        bias_ahead(qcur);
        bK = tile_exp<T>(rk);
        cV = tile_exp<T>(rv);
        rows_to_tile16<T>(tile_q, lane, rk, bK, DQ == KV_ONLY ? 32 : kleft);   // padding keys as zero rows: nothing of them reaches dQ
        rows_to_tile16<T>(tile_do, lane, rv, cV, 32);
        __builtin_amdgcn_wave_barrier();
        kR = read_R<T>(tile_q, l32, hf);
        vR = read_R<T>(tile_do, l32, hf);
        if constexpr (DQ == KV_SINGLE) kT_single = transpose<T, 0>(kR, l32, hf);
    }

    f32x16 dk = zero16(), dv = zero16();
    int xk = 0, xv = 0;                                       // dk, dv are in units of 2^-xk, 2^-xv
    f32x16 dq_own;                                            // KV_PAIR: dS K of this wavefront's own query tile
    // One query tile t against this task's keys.  What happens to dS K of the tile (dq_tag): 0 = not
    // formed, 1 = written out as dQ of a one-tile group, 2 = handed to the other wavefront of the pair,
    // 3 = kept in dq_own.  rq, rdo, ro hold the rows of query tile t; its tables and bias values are on their way.
    auto tile_pass = [&](const int t, const bool first, auto dq_tag) {
        constexpr int DQ_USE = decltype(dq_tag)::value;
        const int aQ = tile_exp<T>(rq), eO = tile_exp<T>(rdo);
        __builtin_amdgcn_wave_barrier();
        rows_dot_to_table_scaled<T>(tab_D, lane, rdo, ro, pow2f(-PSH));      // D_i = dO_i . O_i, times 2^-PSH
        rows_to_tile16<T>(tile_q, lane, rq, aQ, 32);
        rows_to_tile16<T>(tile_do, lane, rdo, eO, 32);
        __builtin_amdgcn_wave_barrier();
        // S and dP of the tile: rows = queries acc_row(r, hf), column = this lane's key
        f32x16 St, dPt;
        {
            const Op qR = read_R<T>(tile_q, l32, hf);
            St = mma<T>(qR, kR, zero16());
        }
        {
            const Op doR = read_R<T>(tile_do, l32, hf);
            dPt = mma<T>(doR, vR, zero16());
        }
        const float c_s = ldexp_fast(a.scale, -(aQ + bK));
        const float c_p = ldexp_fast(1.0f, -(eO + cV + PSH));
        const int qleft = c - t * 32;                         // queries of this tile
        const int qchunks = qleft > 16 ? 2 : 1;               // queries 16.. of the tile are all padding: P = dS = 0
        float* ds_t = ds_g ? ds_g + (int64_t)(t * 32 + 4 * hf) * c : nullptr;
        const int ilim = qleft - 4 * hf;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (q == 2 && qchunks == 1) break;
            const u32x4_a Lq = tab_L.chunk(2 * q + hf), Dq = tab_D.chunk(2 * q + hf);
            const uint32_t Lr[4] = {Lq.x, Lq.y, Lq.z, Lq.w}, Dr[4] = {Dq.x, Dq.y, Dq.z, Dq.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int r = 4 * q + k;
                float s = fmaf(St[r], c_s, bv[r]);
                if (MASK && (differ >> r & 1u)) s += -100.0f;
                St[r] = exp2_fast(fmaf(s, LOG2E, -u2f(Lr[k])));               // P 2^PSH
                dPt[r] = fmaf(dPt[r], c_p, -u2f(Dr[k]));      // (dP - D) 2^-PSH
            }
        }
        // |dS| <= max |dP - D|: the scale of the dS operand is taken from there, so P and dS are packed as
        // they are formed
        const int eS = SPLIT ? scale_exp(amax_acc(dPt, 8 * qchunks)) - PSH : 0;
        const float fS = pow2f(eS);
        Op Pp, dSp;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
            if (r == 8 && qchunks == 1) {
                clear_chunk<T>(Pp, 1);
                clear_chunk<T>(dSp, 1);
                break;
            }
            const float ds0 = St[r] * dPt[r], ds1 = St[r + 1] * dPt[r + 1];          // dS
            const int row = 8 * (r >> 2) + (r & 3);
            if (ds_t && j_k < c) {
                if (row < ilim) ds_t[row * c] = ds0;
                if (row + 1 < ilim) ds_t[(row + 1) * c] = ds1;
            }
            pack_pair<T>(Pp, r >> 3, (r & 7) >> 1, St[r], St[r + 1]);
            pack_pair<T>(dSp, r >> 3, (r & 7) >> 1, ds0 * fS, ds1 * fS);
        }
        {   // dV += P^T dO
            const Op doT = transpose<T, 0>(read_R<T>(tile_do, l32, hf), l32, hf);
            const int nxv = PSH + eO;
            if (SPLIT && !first && nxv != xv) rescale(dv, xv, nxv);
            xv = nxv;
            dv = mma<T>(Pp, doT, dv, qchunks);
        }
        {   // dK += dS^T Q
            const Op qT = transpose<T, 0>(read_R<T>(tile_q, l32, hf), l32, hf);
            const int nxk = eS + aQ;
            if (SPLIT && !first && nxk != xk) rescale(dk, xk, nxk);
            xk = nxk;
            dk = mma<T>(dSp, qT, dk, qchunks);
        }
        if constexpr (DQ_USE != 0) {
            // dS^T (keys in the lanes, queries in the slots) -> queries in the lanes, keys in the slots;
            // dQ = scale dS K over this task's keys (zero rows of K stand for its padding keys)
            const Op dST = transpose<T, 1>(dSp, l32, hf);
            Op kT;
            if constexpr (DQ == KV_PAIR)
                kT = transpose<T, 0>(kR, l32, hf);           // two passes: kept as K in layout R, turned when needed
            else
                kT = kT_single;
            f32x16 dq = mma<T>(dST, kT, zero16(), kleft > 16 ? 2 : 1);
            const float fq = ldexp_fast(a.scale, -(eS + bK));
#pragma unroll
            for (int r = 0; r < 16; ++r) dq[r] *= fq;
            if constexpr (DQ_USE == 2) {
                xch_put(xch, lane, dq);
            } else if constexpr (DQ_USE == 3) {
                dq_own = dq;
            } else {
                __builtin_amdgcn_wave_barrier();
                tile_put_acc(tile_do, l32, hf, dq);
                __builtin_amdgcn_wave_barrier();
                tile_store_rows<T>(tile_do, const_cast<char*>(head_base<T>(tdq, h)), pitch_of<T>(tdq), vox_j, c, lane);
                __builtin_amdgcn_wave_barrier();
            }
        }
    };
    if constexpr (DQ == KV_PAIR) {
        // the other wavefront's query tile first, the own one last (its result stays in registers)
        const QIdx qown = load_qidx(bj);
        tile_pass(1 - bj, true, std::integral_constant<int, 2>{});
        request_rows(qown);
        bias_ahead(qown);
        tile_pass(bj, false, std::integral_constant<int, 3>{});
    } else if constexpr (DQ == KV_SINGLE) {
        tile_pass(0, true, std::integral_constant<int, 1>{});     // groups of one tile only
    } else {
        QIdx qnext = load_qidx(1);                            // indices a tile ahead
        tile_pass(0, true, std::integral_constant<int, 0>{});
#pragma unroll 1
        for (int t = 1; t < nt; ++t) {
            const QIdx qi = qnext;
            request_rows(qi);
            qnext = load_qidx(t + 1);
            bias_ahead(qi);
            tile_pass(t, false, std::integral_constant<int, 0>{});
        }
    }
    const float fk = ldexp_fast(a.scale, -xk), fv = ldexp_fast(1.0f, -xv);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        dk[r] *= fk;
        dv[r] *= fv;
    }
    __builtin_amdgcn_wave_barrier();
    tile_put_acc(tile_q, l32, hf, dk);
    tile_put_acc(tile_do, l32, hf, dv);
    __builtin_amdgcn_wave_barrier();
    tile_store_rows<T>(tile_q, const_cast<char*>(head_base<T>(tdk, h)), pitch_of<T>(tdk), vox_j, kleft, lane);
    tile_store_rows<T>(tile_do, const_cast<char*>(head_base<T>(tdv, h)), pitch_of<T>(tdv), vox_j, kleft, lane);
    if (DQ == KV_PAIR) {
        __syncthreads();                                     // both partial results of every pair are in LDS
        xch_add(xch_peer, lane, dq_own);
        tile_put_acc(tile_do, l32, hf, dq_own);
        __builtin_amdgcn_wave_barrier();
        tile_store_rows<T>(tile_do, const_cast<char*>(head_base<T>(tdq, h)), pitch_of<T>(tdq), vox_j, kleft, lane);
    }
}

template <typename T, bool MASK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void wattn16_bwd_q_kernel(
    WAttnCommon a, TokenTensor32 tq, TokenTensor32 tk, TokenTensor32 tv, TokenTensor32 to, TokenTensor32 tdo,
    const float* __restrict__ lse, TokenTensor32 tdq) {
    __shared__ __attribute__((aligned(16))) float tiles[4][2][TILE_WORDS];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    bwd_q_task<T, MASK>(a, xcd_run_order(blockIdx.x) * 4 + wave, tiles[wave][0], tiles[wave][1], tq, tk, tv, to, tdo, lse, tdq);
}

template <typename T, bool MASK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void wattn16_bwd_kv_kernel(
    WAttnCommon a, TokenTensor32 tq, TokenTensor32 tk, TokenTensor32 tv, TokenTensor32 to, TokenTensor32 tdo,
    const float* __restrict__ lse, TokenTensor32 tdk, TokenTensor32 tdv, float* __restrict__ ds_out) {
    __shared__ __attribute__((aligned(16))) float tiles[4][2][TILE_WORDS];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    bwd_kv_task<T, MASK, KV_ONLY>(a, xcd_run_order(blockIdx.x) * 4 + wave, true, tiles[wave][0], tiles[wave][1], nullptr, nullptr,
                                  tq, tk, tv, to, tdo, lse, tdk, tdv, ds_out, tdk);
}

// The whole backward in one launch (segments as described at BwdSegments).
template <typename T, bool MASK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(X16_BWD_WAVES, X16_BWD_WAVES))) void wattn16_bwd_all_kernel(
    WAttnCommon a, BwdSegments sg, TokenTensor32 tq, TokenTensor32 tk, TokenTensor32 tv, TokenTensor32 to,
    TokenTensor32 tdo, const float* __restrict__ lse, TokenTensor32 tdq, TokenTensor32 tdk, TokenTensor32 tdv,
    float* __restrict__ ds_out) {
    __shared__ __attribute__((aligned(16))) float tiles[4][2][TILE_WORDS];
    __shared__ __attribute__((aligned(16))) float xch[4][64 * 16];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t wg = xcd_run_order(blockIdx.x);
    if (wg >= sg.wgs) return;
    float* t0 = tiles[wave][0];
    float* t1 = tiles[wave][1];
    if (wg < sg.wg_pair) {
        // query side and key side of the larger groups side by side in the work order: both sides of a group, and
        // the heads of a window, run on one XCD at about the same time and share its L2
        const int64_t quad = wg >> 1;
        const int64_t task = quad * 4 + wave;
        if (task < sg.n_big) {
            if ((wg & 1) == 0)
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

template <typename T, bool MASK>
static void launch_backward(const WAttnCommon& a, const TokenTensor32& q, const TokenTensor32& k, const TokenTensor32& v,
                            const TokenTensor32& o, const TokenTensor32& d_o, const float* lse, const TokenTensor32& dq,
                            const TokenTensor32& dk, const TokenTensor32& dv, float* ds_out, int sides, hipStream_t s) {
    if (sides == 3) {
        const BwdSegments sg = make_segments(a, true);
        hipLaunchKernelGGL((wattn16_bwd_all_kernel<T, MASK>), dim3((unsigned)xcd_run_grid(sg.wgs)), dim3(256), 0, s, a, sg, q, k,
                           v, o, d_o, lse, dq, dk, dv, ds_out);
        return;
    }
    const unsigned blocks = (unsigned)xcd_run_grid((a.first[4] + 3) / 4);
    if (sides & 1)
        hipLaunchKernelGGL((wattn16_bwd_q_kernel<T, MASK>), dim3(blocks), dim3(256), 0, s, a, q, k, v, o, d_o, lse, dq);
    if (sides & 2)
        hipLaunchKernelGGL((wattn16_bwd_kv_kernel<T, MASK>), dim3(blocks), dim3(256), 0, s, a, q, k, v, o, d_o, lse, dk, dv,
                           ds_out);
}

template <typename T>
static void forward_t(const WAttnCommon& a, const TokenTensor32& q, const TokenTensor32& k, const TokenTensor32& v,
                      const TokenTensor32& o, float* lse, hipStream_t s) {
    const unsigned blocks = (unsigned)xcd_run_grid((a.first[4] + 3) / 4);
    if (a.mask)
        hipLaunchKernelGGL((wattn16_fwd_kernel<T, true>), dim3(blocks), dim3(256), 0, s, a, q, k, v, o, lse);
    else
        hipLaunchKernelGGL((wattn16_fwd_kernel<T, false>), dim3(blocks), dim3(256), 0, s, a, q, k, v, o, lse);
}
template <typename T>
static void backward_t(const WAttnCommon& a, const TokenTensor32& q, const TokenTensor32& k, const TokenTensor32& v,
                       const TokenTensor32& o, const TokenTensor32& d_o, const float* lse, const TokenTensor32& dq,
                       const TokenTensor32& dk, const TokenTensor32& dv, float* ds_out, int sides, hipStream_t s) {
    if (a.mask)
        launch_backward<T, true>(a, q, k, v, o, d_o, lse, dq, dk, dv, ds_out, sides, s);
    else
        launch_backward<T, false>(a, q, k, v, o, d_o, lse, dq, dk, dv, ds_out, sides, s);
}

void forward(int dtype, const WAttnCommon& a, const TokenTensor32& q, const TokenTensor32& k, const TokenTensor32& v,
             const TokenTensor32& o, float* lse, hipStream_t s) {
    switch (dtype) {
        case SSWIN_F32: forward_t<float>(a, q, k, v, o, lse, s); break;
        case SSWIN_F16: forward_t<__half>(a, q, k, v, o, lse, s); break;
        default: forward_t<__hip_bfloat16>(a, q, k, v, o, lse, s); break;
    }
}
void backward(int dtype, const WAttnCommon& a, const TokenTensor32& q, const TokenTensor32& k, const TokenTensor32& v,
              const TokenTensor32& o, const TokenTensor32& d_o, const float* lse, const TokenTensor32& dq,
              const TokenTensor32& dk, const TokenTensor32& dv, float* ds_out, int sides, hipStream_t s) {
    switch (dtype) {
        case SSWIN_F32: backward_t<float>(a, q, k, v, o, d_o, lse, dq, dk, dv, ds_out, sides, s); break;
        case SSWIN_F16: backward_t<__half>(a, q, k, v, o, d_o, lse, dq, dk, dv, ds_out, sides, s); break;
        default: backward_t<__hip_bfloat16>(a, q, k, v, o, d_o, lse, dq, dk, dv, ds_out, sides, s); break;
    }
}

}  // namespace x16
}  // namespace sswin
