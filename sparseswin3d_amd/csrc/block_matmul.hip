// Window-blocked dense products of the sparse attention path and their COO index emission.
//
// Every group g (one window, one head) owns dense row-major blocks inside the flat value
// arrays:  "mat" blocks of c*C values starting at row_start[g]*C and "sq" blocks of c*c values
// starting at sq_start[g].  Five products are needed (forward: Q.K^T, P.V; backward: the three
// gradient forms).  All of them are out[I x J] = sum_k A[i,k] * B'[k,j] with A row-major
// [I x K]; B is stored either k-major ([K x J]) or j-major ([J x K]):
//
//   mode      A            B                  out          I  J  K
//   QK        Q   mat      K^T mat, k-major   sq           c  c  C
//   PV        P   sq       V   mat, k-major   mat [c x C]  c  C  c
//   RC_CR     m1  mat      m2  mat, j-major   sq           c  c  C
//   RR_RC     m1  sq       m2  mat, j-major   mat [c x C]  c  C  c
//   CR_RR     m1  mat[Cxc] m2  sq,  j-major   mat [C x c]  C  c  c
//   TR_RC     m1^T, m1 sq  m2  mat, k-major   mat [c x C]  c  C  c     (A stored k-major: [K x I])
//   TC_RR     m1^T, m1 mat m2  sq,  k-major   mat [C x c]  C  c  c     (A stored k-major: [K x I])
// The last two are the second gradient of each product taken from the operands as the forward pass left them:
// TR_RC(P, dO) = RR_RC(P^T, (dO)^T stored [C x c]) and TC_RR(Q, dS) = CR_RR(Q^T, dS^T), without the transposed copies.
//
// Execution model (gfx950, wave64): the unit of work is one 32 x 32 output block of one group,
// computed by ONE wavefront with v_mfma_f32_32x32x2_f32.  Operands go from global memory
// straight into the MFMA lane layout — no LDS, no barriers, so wavefronts never wait for each
// other and small windows cost one short task each:
//   * lane l supplies A[i = l % 32][k] and B[k][j = l % 32]; within a 32-wide k chunk the MFMA
//     step s pairs k = s (lanes 0-31) with k = 16 + s (lanes 32-63).  The sum over k does not
//     care about that order, and it makes every row-contiguous operand a run of 16 consecutive
//     values per lane (four 16-byte loads), and every k-major operand one coalesced row per step.
//   * the accumulator of lane l holds column j = l % 32 of rows 8*(r/4) + 4*(l/32) + r%4,
//     r = 0..15, so each store instruction writes two contiguous row segments.
// A workgroup of four wavefronts takes four consecutive groups and deals their blocks round
// robin.  The work is HBM-bound (about 1.7 flop per byte); MFMA is used because it removes the
// LDS staging and the barriers, not because the arithmetic needs it.
#include <cstdlib>
#include <type_traits>

#include "mfma_block.hpp"
#include "sswin_common.hpp"

namespace sswin {

enum { MODE_QK = 0, MODE_PV = 1, MODE_RC_CR = 2, MODE_RR_RC = 3, MODE_CR_RR = 4, MODE_TR_RC = 5, MODE_TC_RR = 6 };

constexpr int GROUPS_PER_WG = 4;
constexpr int MAX_POS = 1024;          // largest window occupancy the simple kernel's LDS table holds

template <int MODE> __host__ __device__ constexpr bool b_is_kmajor() { return MODE == MODE_QK || MODE == MODE_PV || MODE >= MODE_TR_RC; }
template <int MODE> __host__ __device__ constexpr bool a_is_kmajor() { return MODE >= MODE_TR_RC; }
// shapes of the output block: I rows, J columns
template <int MODE> __host__ __device__ constexpr bool rows_are_channels() { return MODE == MODE_CR_RR || MODE == MODE_TC_RR; }
template <int MODE> __host__ __device__ constexpr bool cols_are_channels() { return MODE == MODE_PV || MODE == MODE_RR_RC || MODE == MODE_TR_RC; }

struct GroupDims {
    int I, J, K;
    int64_t a_off, b_off, o_off;
};

template <int MODE>
__device__ __forceinline__ GroupDims group_dims(int c, int C, int64_t rs, int64_t ss) {
    GroupDims d;
    const int64_t mat = rs * C;
    if (MODE == MODE_QK || MODE == MODE_RC_CR) { d.I = c; d.J = c; d.K = C; d.a_off = mat; d.b_off = mat; d.o_off = ss; }
    else if (cols_are_channels<MODE>()) { d.I = c; d.J = C; d.K = c; d.a_off = ss; d.b_off = mat; d.o_off = mat; }
    else { d.I = C; d.J = c; d.K = c; d.a_off = mat; d.b_off = ss; d.o_off = mat; }
    return d;
}

struct GroupTable {
    const int32_t* c;          // [G]
    const int32_t* row_start;  // [G] exclusive scan of c
    const int32_t* sq_start;   // [G] exclusive scan of c*c
    const int32_t* window;     // [G] or null
    const int32_t* head;       // [G] or null
};

#ifndef BP_WAVES
#define BP_WAVES 5
#endif
#ifndef BP_BUFFERED
#define BP_BUFFERED 1
#endif
#ifndef BP_WAVES_FWD
#define BP_WAVES_FWD 5
#endif
template <typename T, int MODE, bool EMIT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(EMIT ? 4 : MODE >= 2 ? BP_WAVES : BP_WAVES_FWD, EMIT ? 4 : MODE >= 2 ? BP_WAVES : BP_WAVES_FWD))) void block_product_mfma_kernel(const T* __restrict__ m1, const T* __restrict__ m2,
                                                                 GroupTable gt, int64_t G, int C,
                                                                 const int32_t* __restrict__ tok_pos,
                                                                 T* __restrict__ out, int32_t* __restrict__ out_idx,
                                                                 int64_t out_nnz) {
    // the wavefront's number as a scalar: everything that follows from it (its task, the group's size and offsets,
    // the operand bases) stays in scalar registers and the loads take a scalar base with a 32-bit lane offset
    // (measured on cfg2: 'q_k' 47.5 -> 44 us, 'qk_v' 41 -> 37, 'tr_rc' / 'tc_rr' 40 -> 35; the products whose operands
    // are both read along their rows lose by it, 'rr_rc' 41 -> 51 us, and keep the lane-held number)
    const int wave = (b_is_kmajor<MODE>() || a_is_kmajor<MODE>() || (BP_BUFFERED && !std::is_same<T, double>::value && !EMIT))
                         ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    const int64_t g0 = (int64_t)blockIdx.x * GROUPS_PER_WG;
    // values without index rows, task state in scalars: blocks addressed through buffer descriptors
    constexpr bool BUFFERED = BP_BUFFERED && !std::is_same<T, double>::value && !EMIT;

    // blocks of the workgroup's four groups
    // sizes and offsets of the four groups leave in one round of loads (the offsets do not wait for the sizes)
    int cq[GROUPS_PER_WG], nbj[GROUPS_PER_WG], first[GROUPS_PER_WG + 1], rsq[GROUPS_PER_WG], ssq[GROUPS_PER_WG];
    first[0] = 0;
#pragma unroll
    for (int q = 0; q < GROUPS_PER_WG; ++q) {
        const int64_t g = g0 + q;
        cq[q] = g < G ? gt.c[g] : 0;
        rsq[q] = g < G ? gt.row_start[g] : 0;
        ssq[q] = g < G ? gt.sq_start[g] : 0;
    }
#pragma unroll
    for (int q = 0; q < GROUPS_PER_WG; ++q) {
        const int c = cq[q];
        const int I = rows_are_channels<MODE>() ? C : c;
        const int J = cols_are_channels<MODE>() ? C : c;
        nbj[q] = (J + 31) >> 5;
        first[q + 1] = first[q] + (c > 0 ? ((I + 31) >> 5) * nbj[q] : 0);
    }
    const int total = first[GROUPS_PER_WG];

    // gridDim.y workgroups share the four groups' blocks (launches of large windows: a group of 227 tokens has 64 blocks)
    for (int t = wave + 4 * (int)blockIdx.y; t < total; t += 4 * (int)gridDim.y) {
        int q = 0;
#pragma unroll
        for (int qq = 1; qq < GROUPS_PER_WG; ++qq) q += (t >= first[qq]) ? 1 : 0;
        int c = cq[0], nj = nbj[0], f0 = first[0], rs_ = rsq[0], ss_ = ssq[0];
#pragma unroll
        for (int qq = 1; qq < GROUPS_PER_WG; ++qq)
            if (q == qq) { c = cq[qq]; nj = nbj[qq]; f0 = first[qq]; rs_ = rsq[qq]; ss_ = ssq[qq]; }
        const int64_t g = g0 + q;
        const int local = t - f0;
        const int bi = local / nj, bj = local - bi * nj;
        const int64_t rs = rs_, ss = ss_;
        const GroupDims d = group_dims<MODE>(c, C, rs, ss);
        const int i_a = bi * 32 + l32;           // operand row of A this lane feeds
        const int j_b = bj * 32 + l32;           // operand column of B this lane feeds

        // positions for the index rows; issued first so their latency hides behind the product
        int pos_i[16], pos_j = 0, win = 0, hd_ = 0;
        if (EMIT) {
            win = gt.window[g];
            hd_ = gt.head[g];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int i = bi * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                pos_i[r] = i < c ? tok_pos[(rs + i) * C] : 0;
            }
            if (MODE == MODE_QK) pos_j = j_b < c ? tok_pos[(rs + j_b) * C] : 0;
        }

        const T* A = m1 + d.a_off;
        const T* B = m2 + d.b_off;
        f32x16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        if constexpr (BUFFERED) {
            // every block through a buffer descriptor of exactly its size (buf_of and the loads of mfma_block.hpp)
            constexpr uint32_t OUTSIDE = BUF_OUTSIDE;
            constexpr uint32_t ES = (uint32_t)sizeof(T);               // 4 (float) or 2 (half, bfloat16)
            const __amdgpu_buffer_rsrc_t ra = buf_of(A, (uint32_t)(d.I * d.K) * ES);
            const __amdgpu_buffer_rsrc_t rb = buf_of(B, (uint32_t)(d.K * d.J) * ES);
            const __amdgpu_buffer_rsrc_t ro = buf_of(out + d.o_off, (uint32_t)(d.I * d.J) * ES);
            for (int kc = 0; kc < d.K; kc += 32) {
                const int chunk = d.K - kc < 32 ? d.K - kc : 32;
                const int kh = (chunk + 1) >> 1;
                const int left = half ? chunk - kh : kh;
                float a[16], b[16];
                if (a_is_kmajor<MODE>()) {
                    // element (kc + half * kh + s, i): rows of k behind the block's last one are outside by themselves
                    const uint32_t v0 = i_a < d.I ? (uint32_t)(half * kh * d.I + i_a) * ES : OUTSIDE;
#pragma unroll
                    for (int s = 0; s < 8; ++s) a[s] = buf_load1<T>(ra, v0 + (uint32_t)((kc + s) * d.I) * ES);
                    if (kh > 8) {
#pragma unroll
                        for (int s = 8; s < 16; ++s) a[s] = buf_load1<T>(ra, v0 + (uint32_t)((kc + s) * d.I) * ES);
                    }
                } else {
                    // a row per lane: 16 consecutive values of row i; values of k behind the row's end belong to the
                    // next row and are masked through their offsets
                    const uint32_t v0 = i_a < d.I ? (uint32_t)(i_a * d.K + kc + half * kh) * ES : OUTSIDE;
                    if (chunk == 32 && (ES == 4 || d.K % 8 == 0)) {      // 16-byte loads need rows that start at a multiple of 4 bytes
                        buf_load_run<T, 16>(ra, v0, a);
                    } else if (chunk == 16 && (ES == 4 || d.K % 8 == 0)) {
                        buf_load_run<T, 8>(ra, v0, a);
                    } else {
#pragma unroll
                        for (int s = 0; s < 16; ++s) a[s] = buf_load1<T>(ra, s < left ? v0 + ES * s : OUTSIDE);
                    }
                }
                if (b_is_kmajor<MODE>()) {
                    const uint32_t v0 = j_b < d.J ? (uint32_t)(half * kh * d.J + j_b) * ES : OUTSIDE;
#pragma unroll
                    for (int s = 0; s < 8; ++s) b[s] = buf_load1<T>(rb, v0 + (uint32_t)((kc + s) * d.J) * ES);
                    if (kh > 8) {
#pragma unroll
                        for (int s = 8; s < 16; ++s) b[s] = buf_load1<T>(rb, v0 + (uint32_t)((kc + s) * d.J) * ES);
                    }
                } else {
                    const uint32_t v0 = j_b < d.J ? (uint32_t)(j_b * d.K + kc + half * kh) * ES : OUTSIDE;
                    if (chunk == 32 && (ES == 4 || d.K % 8 == 0)) {
                        buf_load_run<T, 16>(rb, v0, b);
                    } else if (chunk == 16 && (ES == 4 || d.K % 8 == 0)) {
                        buf_load_run<T, 8>(rb, v0, b);
                    } else {
#pragma unroll
                        for (int s = 0; s < 16; ++s) b[s] = buf_load1<T>(rb, s < left ? v0 + ES * s : OUTSIDE);
                    }
                }
#pragma unroll
                for (int s = 0; s < 16; ++s)
                    if (s < kh) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[s], acc, 0, 0, 0);
            }
            const uint32_t o0 = j_b < d.J ? (uint32_t)((bi * 32 + 4 * half) * d.J + j_b) * ES : OUTSIDE;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float v = acc[r];                      // a scalar copy: a bit_cast of the vector element itself reads element 0
                buf_store1<T>(ro, o0 + (uint32_t)((8 * (r >> 2) + (r & 3)) * d.J) * ES, v);
            }
            continue;
        }
        for (int kc = 0; kc < d.K; kc += 32) {
            // the (at most 32) values of k of this round are split evenly between the two lane halves, so a
            // reduction over 16 channels takes eight matrix steps, not sixteen with one half feeding zeros
            const int chunk = d.K - kc < 32 ? d.K - kc : 32;
            const int kh = (chunk + 1) >> 1;                    // uniform: steps that carry data
            const int kb = kc + half * kh;
            const int left = half ? chunk - kh : kh;            // values of k of this lane half
            float a[16], b[16];
            // A k-major operand is read one row of k per step: element (kc + s) * width + (half * kh * width + column),
            // a scalar part plus a lane part.  Every lane loads from inside the block (offset clamped to its last
            // element) and drops what it has no use for: one select per value instead of a branch around each load.
            if (a_is_kmajor<MODE>()) {
                const unsigned lane_part = (unsigned)(half * kh * d.I + (i_a < d.I ? i_a : d.I - 1));
                const unsigned last = (unsigned)(d.K * d.I - 1);
                const bool iin = i_a < d.I;
#pragma unroll
                for (int s = 0; s < 16; ++s) {
                    const unsigned off = (unsigned)((kc + s) * d.I) + lane_part;
                    const float x = to_acc(A[off < last ? off : last]);
                    a[s] = (iin && s < left) ? x : 0.f;
                }
            } else {
                load_run16<T>(A + (int64_t)i_a * d.K + kb, i_a < d.I ? left : 0, a);
            }
            if (b_is_kmajor<MODE>()) {
                const unsigned lane_part = (unsigned)(half * kh * d.J + (j_b < d.J ? j_b : d.J - 1));
                const unsigned last = (unsigned)(d.K * d.J - 1);
                const bool jin = j_b < d.J;
#pragma unroll
                for (int s = 0; s < 16; ++s) {
                    const unsigned off = (unsigned)((kc + s) * d.J) + lane_part;
                    const float x = to_acc(B[off < last ? off : last]);
                    b[s] = (jin && s < left) ? x : 0.f;
                }
            } else {
                load_run16<T>(B + (int64_t)j_b * d.K + kb, j_b < d.J ? left : 0, b);
            }
#pragma unroll
            for (int s = 0; s < 16; ++s)
                if (s < kh) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[s], acc, 0, 0, 0);
        }

        if (j_b < d.J) {
            T* O = out + d.o_off + j_b;
            int32_t* X = EMIT ? out_idx + d.o_off + j_b : nullptr;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int i = bi * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                if (i < d.I) {
                    const int64_t off = (int64_t)i * d.J;
                    O[off] = from_acc<T>(acc[r]);
                    if (EMIT) {
                        X[off] = win;
                        X[off + out_nnz] = hd_;
                        X[off + 2 * out_nnz] = pos_i[r];
                        X[off + 3 * out_nnz] = MODE == MODE_QK ? pos_j : j_b;
                    }
                }
            }
        }
    }
}

// COO index rows for one group, written by NT threads of one workgroup (simple kernel only).
template <int NT, bool IS_QK>
__device__ __forceinline__ void emit_indices(int32_t* __restrict__ out_idx, int64_t out_nnz, int64_t base,
                                             int c, int C, int w, int h, const int* __restrict__ pos,
                                             int tid) {
    const int J = IS_QK ? c : C;
    const int count = c * J;
    int32_t* r0 = out_idx + base;
    for (int f = tid; f < count; f += NT) {
        const int i = f / J, j = f - i * J;
        r0[f] = w;
        r0[f + out_nnz] = h;
        r0[f + 2 * out_nnz] = pos[i];
        r0[f + 3 * out_nnz] = IS_QK ? pos[j] : j;
    }
}

// ------------------------------------------------------------------------------------------
// reference-shaped kernel for any value type (used for double): one workgroup per group,
// one output element per thread and step, operands read straight from global memory.
// ------------------------------------------------------------------------------------------
template <typename T, int MODE, bool EMIT>
__global__ __launch_bounds__(256) void block_product_simple_kernel(const T* __restrict__ m1,
                                                                   const T* __restrict__ m2, GroupTable gt,
                                                                   int64_t G, int C,
                                                                   const int32_t* __restrict__ tok_pos,
                                                                   T* __restrict__ out,
                                                                   int32_t* __restrict__ out_idx,
                                                                   int64_t out_nnz) {
    using AccT = typename acc_of<T>::type;
    __shared__ int pos_s[EMIT ? MAX_POS : 1];
    const int64_t g = blockIdx.x;
    if (g >= G) return;
    const int c = gt.c[g];
    const int64_t rs = gt.row_start[g], ss = gt.sq_start[g];
    const GroupDims d = group_dims<MODE>(c, C, rs, ss);
    const T* A = m1 + d.a_off;
    const T* B = m2 + d.b_off;
    T* O = out + d.o_off;
    const int count = d.I * d.J;
    for (int f = threadIdx.x; f < count; f += 256) {
        const int i = f / d.J, j = f - i * d.J;
        AccT sum = 0;
        for (int k = 0; k < d.K; ++k) {
            const AccT a = a_is_kmajor<MODE>() ? to_acc(A[(int64_t)k * d.I + i]) : to_acc(A[(int64_t)i * d.K + k]);
            const AccT b = b_is_kmajor<MODE>() ? to_acc(B[(int64_t)k * d.J + j]) : to_acc(B[(int64_t)j * d.K + k]);
            sum += a * b;
        }
        O[f] = from_acc<T>(sum);
    }
    if (EMIT) {
        for (int i = threadIdx.x; i < c; i += 256) pos_s[i] = tok_pos[(rs + i) * C];
        __syncthreads();
        emit_indices<256, MODE == MODE_QK>(out_idx, out_nnz, d.o_off, c, C, gt.window[g], gt.head[g], pos_s,
                                           threadIdx.x);
    }
}

// ------------------------------------------------------------------------------------------
// per-group transposes.  rc: [c x C] -> [C x c];  rr: [c x c] -> [c x c]^T.
// One wavefront per group.  A group's block is a few KB: it is read as one contiguous run into a
// wave-private LDS copy (odd pitch, so a column is spread over the banks) and written back as one
// contiguous run in transposed order, so both sides of the copy are coalesced.  Blocks that do not fit
// the LDS copy (more than TR_LDS_BYTES) go through it tile by tile.
// ------------------------------------------------------------------------------------------
constexpr int TR_LDS_BYTES = 6144;      // six workgroups per CU; 8192: rc 0.0207, rr 0.0353 ms on cfg2, 6144: 0.0195, 0.0345, 4096: 0.0225, 0.039

// f / d through a multiplication, exact for f * d < 2^32 (blocks here stay below 2^14 entries); d = 1 has no
// 32-bit multiplier and is marked by 0
__device__ __forceinline__ uint32_t div_magic(uint32_t d) { return d == 1 ? 0u : (uint32_t)((0x100000000ull + d - 1) / d); }
__device__ __forceinline__ int div_by(int f, uint32_t magic) { return magic ? (int)__umulhi((uint32_t)f, magic) : f; }

template <typename T, bool IS_RR>
__global__ __launch_bounds__(256) void block_transpose_kernel(const T* __restrict__ in, const int32_t* __restrict__ cs,
                                                              const int32_t* __restrict__ row_start,
                                                              const int32_t* __restrict__ sq_start, int64_t G,
                                                              int C, T* __restrict__ out) {
    __shared__ __attribute__((aligned(16))) char lds[GROUPS_PER_WG][TR_LDS_BYTES];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    T* t = reinterpret_cast<T*>(lds[wave]);
    constexpr int U = 8;                      // loads in flight per lane
    constexpr int cap = TR_LDS_BYTES / (int)sizeof(T);
    {
        const int64_t g = (int64_t)blockIdx.x * GROUPS_PER_WG + wave;
        if (g >= G) return;
        const int c = cs[g];
        const int64_t off = IS_RR ? (int64_t)sq_start[g] : (int64_t)row_start[g] * C;
        const int rows = c;                   // in is [rows x cols], out is [cols x rows]
        const int cols = IS_RR ? c : C;
        const T* src = in + off;
        T* dst = out + off;
        const uint32_t m_rows = div_magic((uint32_t)rows);
        const int pitch = cols | 1;
        if (rows * pitch <= cap) {
            const int count = rows * cols;
            const uint32_t m_cols = div_magic((uint32_t)cols);
            for (int f0 = lane; f0 < count; f0 += 64 * U) {
                T v[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int f = f0 + 64 * u;
                    v[u] = src[f < count ? f : count - 1];
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int f = f0 + 64 * u;
                    const int i = div_by(f, m_cols), j = f - i * cols;
                    if (f < count) t[i * pitch + j] = v[u];
                }
            }
            __builtin_amdgcn_wave_barrier();
            for (int f = lane; f < count; f += 64) {
                const int jo = div_by(f, m_rows), io = f - jo * rows;
                dst[f] = t[io * pitch + jo];
            }
            return;
        }
        // larger blocks: tiles of TS x TS values through the LDS copy (pitch TS + 1).  A tile is read as runs of
        // TS values of TS input rows and written as runs of TS values of TS output rows; the loads of the next
        // tile are issued before the current one passes through LDS (two register sets taken in turn: a copy
        // of loaded registers would wait for them).
        constexpr int TS = sizeof(T) <= 4 ? 32 : 16;
        constexpr int PER = TS * TS / 64;                     // values of a tile per lane
        static_assert((TS + 1) * TS * (int)sizeof(T) <= TR_LDS_BYTES, "a tile fits the LDS copy");
        const int tcols = (cols + TS - 1) / TS;
        const int tiles = ((rows + TS - 1) / TS) * tcols;
        auto fetch = [&](int tile, T (&v)[PER]) __attribute__((always_inline)) {
            const int bi = tile / tcols, bj = tile - bi * tcols;
#pragma unroll
            for (int u = 0; u < PER; ++u) {
                const int e = lane + 64 * u;
                const int gi = bi * TS + e / TS, gj = bj * TS + e % TS;
                const bool ok = gi < rows && gj < cols;
                v[u] = src[ok ? (int64_t)gi * cols + gj : 0];
            }
        };
        auto emit = [&](int tile, const T (&v)[PER]) __attribute__((always_inline)) {
            const int bi = tile / tcols, bj = tile - bi * tcols;
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int u = 0; u < PER; ++u) {
                const int e = lane + 64 * u;
                t[(e / TS) * (TS + 1) + e % TS] = v[u];
            }
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int u = 0; u < PER; ++u) {
                const int e = lane + 64 * u;
                const int orow = e / TS, ocol = e % TS;           // inside the output tile: row = input column
                const int gi = bj * TS + orow, gj = bi * TS + ocol;
                if (gi < cols && gj < rows) dst[(int64_t)gi * rows + gj] = t[ocol * (TS + 1) + orow];
            }
        };
        T va[PER], vb[PER];
        fetch(0, va);
        for (int tile = 0; tile < tiles; tile += 2) {
            if (tile + 1 < tiles) fetch(tile + 1, vb);
            emit(tile, va);
            if (tile + 1 >= tiles) break;
            if (tile + 2 < tiles) fetch(tile + 2, va);
            emit(tile + 1, vb);
        }
    }
}

// ------------------------------------------------------------------------------------------
// host dispatch
// ------------------------------------------------------------------------------------------
static bool force_simple() {
    static const bool v = [] {
        const char* e = getenv("SSWIN_FORCE_SIMPLE");
        return e && e[0] == '1';
    }();
    return v;
}

// COO index rows of a product, streamed by their own kernel: one wavefront per group, four
// consecutive entries per lane and 16-byte stores (a row of the index matrix is a pure function
// of the plan and the token positions, so the MFMA kernel does not have to carry it).
// rows: window, head, pos_i, and pos_j ('q_k', J = c) or the channel ('qk_v', J = C).
typedef int i32x4_u __attribute__((ext_vector_type(4), aligned(4)));

template <bool IS_QK>
__global__ __launch_bounds__(256) void emit_coo_kernel(GroupTable gt, int64_t G, int C,
                                                       const int32_t* __restrict__ tok_pos,
                                                       int32_t* __restrict__ out_idx, int64_t out_nnz) {
    __shared__ int pos_s[GROUPS_PER_WG][MAX_POS];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int64_t g = (int64_t)blockIdx.x * GROUPS_PER_WG + wave;
    if (g >= G) return;
    const int c = gt.c[g];
    const int64_t rs = gt.row_start[g];
    const int w = gt.window[g], h = gt.head[g];
    int* pos = pos_s[wave];
    for (int i = lane; i < c; i += 64) pos[i] = tok_pos[(rs + i) * C];
    __builtin_amdgcn_wave_barrier();
    const int J = IS_QK ? c : C;
    const int count = c * J;
    const int64_t base = IS_QK ? (int64_t)gt.sq_start[g] : rs * C;
    int32_t* r0 = out_idx + base;
    int32_t* r1 = r0 + out_nnz;
    int32_t* r2 = r1 + out_nnz;
    int32_t* r3 = r2 + out_nnz;
    const i32x4_u wv = {w, w, w, w}, hv = {h, h, h, h};
    for (int f = 4 * lane; f < count; f += 256) {
        int i = f / J, j = f - i * J;
        int pi[4], pj[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int ic = i < c ? i : c - 1;                 // entries past the end are not stored
            pi[k] = pos[ic];
            pj[k] = IS_QK ? pos[j] : j;
            if (++j == J) {
                j = 0;
                ++i;
            }
        }
        if (f + 3 < count) {
            *reinterpret_cast<i32x4_u*>(r0 + f) = wv;
            *reinterpret_cast<i32x4_u*>(r1 + f) = hv;
            *reinterpret_cast<i32x4_u*>(r2 + f) = i32x4_u{pi[0], pi[1], pi[2], pi[3]};
            *reinterpret_cast<i32x4_u*>(r3 + f) = i32x4_u{pj[0], pj[1], pj[2], pj[3]};
        } else {
            for (int k = 0; k < 4 && f + k < count; ++k) {
                r0[f + k] = w;
                r1[f + k] = h;
                r2[f + k] = pi[k];
                r3[f + k] = pj[k];
            }
        }
    }
}

template <int MODE>
static unsigned task_slices(int64_t G, int C, int64_t mat_nnz) {
    if (G <= 0 || C <= 0 || mat_nnz <= 0) return 1;
    const double mean_c = (double)mat_nnz / ((double)C * (double)G);
    return block_task_slices(mean_c, C, !(rows_are_channels<MODE>() || cols_are_channels<MODE>()), GROUPS_PER_WG);
}

template <typename T, int MODE, bool EMIT>
static int launch_product(const void* m1, const void* m2, const GroupTable& gt, int64_t G, int C, int64_t mat_nnz,
                          const int32_t* tok_pos, void* out, int32_t* out_idx, int64_t out_nnz,
                          hipStream_t s) {
    if (G == 0) return 0;
    bool tiled = false;
    if constexpr (!std::is_same<T, double>::value) {
        if (!force_simple()) {
            tiled = true;
            const unsigned blocks = (unsigned)((G + GROUPS_PER_WG - 1) / GROUPS_PER_WG);
            // 'q_k' writes its four index rows from a streaming kernel (measured faster than carrying
            // them through the MFMA kernel); 'qk_v' keeps them in the product kernel
            constexpr bool split = EMIT && MODE == MODE_QK;
            hipLaunchKernelGGL((block_product_mfma_kernel<T, MODE, EMIT && !split>), dim3(blocks, task_slices<MODE>(G, C, mat_nnz)), dim3(256), 0, s,
                               static_cast<const T*>(m1), static_cast<const T*>(m2), gt, G, C, tok_pos,
                               static_cast<T*>(out), out_idx, out_nnz);
            if (split)
                hipLaunchKernelGGL((emit_coo_kernel<true>), dim3(blocks), dim3(256), 0, s, gt, G, C, tok_pos, out_idx,
                                   out_nnz);
        }
    }
    if (!tiled) {
        hipLaunchKernelGGL((block_product_simple_kernel<T, MODE, EMIT>), dim3((unsigned)G), dim3(256), 0, s,
                           static_cast<const T*>(m1), static_cast<const T*>(m2), gt, G, C, tok_pos,
                           static_cast<T*>(out), out_idx, out_nnz);
    }
    return launch_ok("block product");
}

template <int MODE, bool EMIT>
static int dispatch_product(int dtype, const void* m1, const void* m2, const GroupTable& gt, int64_t G, int C,
                            int64_t mat_nnz, const int32_t* tok_pos, void* out, int32_t* out_idx, int64_t out_nnz,
                            hipStream_t s) {
    switch (dtype) {
        case SSWIN_F32: return launch_product<float, MODE, EMIT>(m1, m2, gt, G, C, mat_nnz, tok_pos, out, out_idx, out_nnz, s);
        case SSWIN_F16: return launch_product<__half, MODE, EMIT>(m1, m2, gt, G, C, mat_nnz, tok_pos, out, out_idx, out_nnz, s);
        case SSWIN_BF16: return launch_product<__hip_bfloat16, MODE, EMIT>(m1, m2, gt, G, C, mat_nnz, tok_pos, out, out_idx, out_nnz, s);
        case SSWIN_F64: return launch_product<double, MODE, EMIT>(m1, m2, gt, G, C, mat_nnz, tok_pos, out, out_idx, out_nnz, s);
        default: return fail("unsupported value dtype %d", dtype);
    }
}

template <typename T>
static int launch_transpose(int kind, const void* in, const int32_t* c, const int32_t* scans, int64_t G, int C,
                            void* out, hipStream_t s) {
    const unsigned blocks = (unsigned)((G + GROUPS_PER_WG - 1) / GROUPS_PER_WG);
    if (kind == SSWIN_TRANSPOSE_RR)
        hipLaunchKernelGGL((block_transpose_kernel<T, true>), dim3(blocks), dim3(256), 0, s,
                           static_cast<const T*>(in), c, scans, scans + G, G, C, static_cast<T*>(out));
    else
        hipLaunchKernelGGL((block_transpose_kernel<T, false>), dim3(blocks), dim3(256), 0, s,
                           static_cast<const T*>(in), c, scans, scans + G, G, C, static_cast<T*>(out));
    return launch_ok("block transpose");
}

}  // namespace sswin

using namespace sswin;

extern "C" {

int sswin_block_matmul(int kind, int dtype, const void* mat1_v, const void* mat2_v, const int32_t* tok_idx,
                       int64_t M, int C, const int32_t* plan, int64_t g_cap, int64_t G, int64_t c_max,
                       void* out_val, int32_t* out_idx, int64_t out_nnz, void* stream) {
    SSWIN_CHECK(kind == SSWIN_MUL_Q_K || kind == SSWIN_MUL_QK_V,
                "Invalid mul_type code %d. Expected 'q_k' or 'qk_v'.", kind);
    SSWIN_CHECK(C > 0 && M >= 0 && G >= 0 && G <= g_cap, "block_matmul: bad sizes");
    if (G == 0 || out_nnz == 0) return 0;
    SSWIN_CHECK(tok_idx && plan && (out_val || out_idx), "block_matmul: null pointer");
    SSWIN_CHECK(!out_val || (mat1_v && mat2_v), "block_matmul: null operand");
    SSWIN_CHECK(out_nnz < (int64_t)INT32_MAX, "block_matmul: output nnz does not fit int32 offsets");
    SSWIN_CHECK(c_max >= 1 && c_max <= MAX_POS,
                "block_matmul: largest group holds %lld tokens; supported range is [1, %d]", (long long)c_max, MAX_POS);
    GroupTable gt{plan, plan + g_cap, plan + 2 * g_cap, plan + 3 * g_cap, plan + 4 * g_cap};
    const int32_t* tok_pos = tok_idx + 2 * M;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (!out_val) {                                          // index rows only
        const unsigned blocks = (unsigned)((G + GROUPS_PER_WG - 1) / GROUPS_PER_WG);
        if (kind == SSWIN_MUL_Q_K)
            hipLaunchKernelGGL((emit_coo_kernel<true>), dim3(blocks), dim3(256), 0, s, gt, G, C, tok_pos, out_idx, out_nnz);
        else
            hipLaunchKernelGGL((emit_coo_kernel<false>), dim3(blocks), dim3(256), 0, s, gt, G, C, tok_pos, out_idx, out_nnz);
        return launch_ok("block product indices");
    }
    if (!out_idx) {                                          // values only
        if (kind == SSWIN_MUL_Q_K)
            return dispatch_product<MODE_QK, false>(dtype, mat1_v, mat2_v, gt, G, C, M, tok_pos, out_val, nullptr, out_nnz, s);
        return dispatch_product<MODE_PV, false>(dtype, mat1_v, mat2_v, gt, G, C, M, tok_pos, out_val, nullptr, out_nnz, s);
    }
    if (kind == SSWIN_MUL_Q_K)
        return dispatch_product<MODE_QK, true>(dtype, mat1_v, mat2_v, gt, G, C, M, tok_pos, out_val, out_idx, out_nnz, s);
    return dispatch_product<MODE_PV, true>(dtype, mat1_v, mat2_v, gt, G, C, M, tok_pos, out_val, out_idx, out_nnz, s);
}

int sswin_block_matmul_grad(int kind, int dtype, const void* m1, const void* m2, const int32_t* c,
                            const int32_t* scans, int64_t G, int C, int64_t mat_nnz, void* out, void* stream) {
    SSWIN_CHECK(kind >= SSWIN_GRAD_RC_CR && kind <= SSWIN_GRAD_TC_RR,
                "Invalid mul_type code %d. Expected 'rc_cr', 'rr_rc', 'cr_rr', 'tr_rc' or 'tc_rr'.", kind);
    SSWIN_CHECK(C > 0 && G >= 0 && mat_nnz >= 0, "block_matmul_grad: bad sizes");
    if (G == 0) return 0;
    SSWIN_CHECK(m1 && m2 && c && scans && out, "block_matmul_grad: null pointer");
    GroupTable gt{c, scans, scans + G, nullptr, nullptr};
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (kind) {
        case SSWIN_GRAD_RC_CR: return dispatch_product<MODE_RC_CR, false>(dtype, m1, m2, gt, G, C, mat_nnz, nullptr, out, nullptr, 0, s);
        case SSWIN_GRAD_RR_RC: return dispatch_product<MODE_RR_RC, false>(dtype, m1, m2, gt, G, C, mat_nnz, nullptr, out, nullptr, 0, s);
        case SSWIN_GRAD_CR_RR: return dispatch_product<MODE_CR_RR, false>(dtype, m1, m2, gt, G, C, mat_nnz, nullptr, out, nullptr, 0, s);
        case SSWIN_GRAD_TR_RC: return dispatch_product<MODE_TR_RC, false>(dtype, m1, m2, gt, G, C, mat_nnz, nullptr, out, nullptr, 0, s);
        default: return dispatch_product<MODE_TC_RR, false>(dtype, m1, m2, gt, G, C, mat_nnz, nullptr, out, nullptr, 0, s);
    }
}

int sswin_block_transpose(int kind, int dtype, const void* in, const int32_t* c, const int32_t* scans,
                          int64_t G, int C, void* out, void* stream) {
    SSWIN_CHECK(kind == SSWIN_TRANSPOSE_RC || kind == SSWIN_TRANSPOSE_RR,
                "Invalid mul_type code %d. Expected 'rc', or 'rr'.", kind);
    SSWIN_CHECK(C > 0 && G >= 0, "block_transpose: bad sizes");
    if (G == 0) return 0;
    SSWIN_CHECK(in && c && scans && out, "block_transpose: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case SSWIN_F32: return launch_transpose<float>(kind, in, c, scans, G, C, out, s);
        case SSWIN_F16: return launch_transpose<__half>(kind, in, c, scans, G, C, out, s);
        case SSWIN_BF16: return launch_transpose<__hip_bfloat16>(kind, in, c, scans, G, C, out, s);
        case SSWIN_F64: return launch_transpose<double>(kind, in, c, scans, G, C, out, s);
        default: return fail("unsupported value dtype %d", dtype);
    }
}

}  // extern "C"
