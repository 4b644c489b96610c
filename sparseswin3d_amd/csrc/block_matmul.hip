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
//
// Execution model (wave64, 256-thread workgroups, one workgroup per four consecutive groups):
//   * if all four groups have I, J, K <= 32, each wavefront multiplies one group on its own
//     (64 lanes = 8 x 8 register tiles of 4 x 4) — balanced work for the many small windows;
//   * otherwise the four groups are processed one after another by the whole workgroup with
//     fixed-size LDS blocks, so LDS use does not depend on the window occupancy.
// Operands are staged in LDS k-major (At[k][i], Bs[k][j]) so that the inner loop is two 16-byte
// LDS reads per 16 fused multiply-adds.  The work is HBM-bound (about 1.7 flop per byte).
#include <cstdlib>
#include <type_traits>

#include "sswin_common.hpp"

namespace sswin {

enum { MODE_QK = 0, MODE_PV = 1, MODE_RC_CR = 2, MODE_RR_RC = 3, MODE_CR_RR = 4 };

constexpr int KC = 32;                 // k extent of one LDS chunk
constexpr int GROUPS_PER_WG = 4;
constexpr int MAX_POS = 1024;          // largest supported window occupancy for index emission

typedef float f32x4_u __attribute__((ext_vector_type(4), aligned(4)));
typedef int i32x4_u __attribute__((ext_vector_type(4), aligned(4)));

template <int MODE> struct BlockShape;   // workgroup-path LDS block (IB x JB), IB*JB/16 == 256
template <> struct BlockShape<MODE_QK>    { static constexpr int IB = 64,  JB = 64;  };
template <> struct BlockShape<MODE_RC_CR> { static constexpr int IB = 64,  JB = 64;  };
template <> struct BlockShape<MODE_PV>    { static constexpr int IB = 128, JB = 32;  };
template <> struct BlockShape<MODE_RR_RC> { static constexpr int IB = 128, JB = 32;  };
template <> struct BlockShape<MODE_CR_RR> { static constexpr int IB = 32,  JB = 128; };

template <int MODE> __host__ __device__ constexpr bool b_is_kmajor() { return MODE == MODE_QK || MODE == MODE_PV; }

struct GroupDims {
    int I, J, K;
    int64_t a_off, b_off, o_off;
};

template <int MODE>
__device__ __forceinline__ GroupDims group_dims(int c, int C, int64_t rs, int64_t ss) {
    GroupDims d;
    const int64_t mat = rs * C;
    if (MODE == MODE_QK || MODE == MODE_RC_CR) { d.I = c; d.J = c; d.K = C; d.a_off = mat; d.b_off = mat; d.o_off = ss; }
    else if (MODE == MODE_PV || MODE == MODE_RR_RC) { d.I = c; d.J = C; d.K = c; d.a_off = ss; d.b_off = mat; d.o_off = mat; }
    else { d.I = C; d.J = c; d.K = c; d.a_off = mat; d.b_off = ss; d.o_off = mat; }
    return d;
}

// ------------------------------------------------------------------------------------------
// LDS staging.  NT threads (tid in [0, NT)) fill a chunk; out-of-range elements become zero so
// the multiply needs no bounds checks.
// ------------------------------------------------------------------------------------------
// source row-major [R x K] (k contiguous) -> dst[kk * P + rr], rr in [0, RB), kk in [0, KC)
template <int NT, int RB, typename T>
__device__ __forceinline__ void stage_transposed(const T* __restrict__ src, int R, int K, int r0, int k0,
                                                 float* __restrict__ dst, int tid) {
    constexpr int P = RB + 4;
#pragma unroll 4
    for (int f = tid; f < RB * KC; f += NT) {
        const int rr = f / KC, kk = f % KC;
        const int gr = r0 + rr, gk = k0 + kk;
        float v = 0.f;
        if (gr < R && gk < K) v = to_acc(src[(int64_t)gr * K + gk]);
        dst[kk * P + rr] = v;
    }
}

// source k-major [K x J] (j contiguous) -> dst[kk * P + jj], jj in [0, JB)
template <int NT, int JB, typename T>
__device__ __forceinline__ void stage_direct(const T* __restrict__ src, int K, int J, int k0, int j0,
                                             float* __restrict__ dst, int tid) {
    constexpr int P = JB + 4;
#pragma unroll 4
    for (int f = tid; f < JB * KC; f += NT) {
        const int kk = f / JB, jj = f % JB;
        const int gk = k0 + kk, gj = j0 + jj;
        float v = 0.f;
        if (gk < K && gj < J) v = to_acc(src[(int64_t)gk * J + gj]);
        dst[kk * P + jj] = v;
    }
}

template <int IB, int JB>
__device__ __forceinline__ void multiply_chunk(const float* __restrict__ At, const float* __restrict__ Bs,
                                               int ti, int tj, int kmax, float (&acc)[4][4]) {
    constexpr int IP = IB + 4, JP = JB + 4;
    const float* ap = At + 4 * ti;
    const float* bp = Bs + 4 * tj;
#pragma unroll 4
    for (int kk = 0; kk < kmax; ++kk) {
        const float4 a = *reinterpret_cast<const float4*>(ap + kk * IP);
        const float4 b = *reinterpret_cast<const float4*>(bp + kk * JP);
        const float av[4] = {a.x, a.y, a.z, a.w};
        const float bv[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int s = 0; s < 4; ++s) acc[r][s] = fmaf(av[r], bv[s], acc[r][s]);
    }
}

template <typename T>
__device__ __forceinline__ void store_tile(T* __restrict__ O, int I, int J, int i0, int j0,
                                           const float (&acc)[4][4]) {
    if (i0 >= I || j0 >= J) return;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int i = i0 + r;
        if (i >= I) break;
        T* p = O + (int64_t)i * J + j0;
        if (sizeof(T) == 4 && j0 + 3 < J) {
            f32x4_u v = {acc[r][0], acc[r][1], acc[r][2], acc[r][3]};
            *reinterpret_cast<f32x4_u*>(p) = v;
        } else {
#pragma unroll
            for (int s = 0; s < 4; ++s)
                if (j0 + s < J) p[s] = from_acc<T>(acc[r][s]);
        }
    }
}

// ------------------------------------------------------------------------------------------
// COO index emission for one group by NT threads.  Rows of out_idx are out_nnz apart.
//   QK: slot ss + i*c + j      -> (window, head, pos[i], pos[j])
//   PV: slot rs*C + i*C + ch   -> (window, head, pos[i], ch)
// ------------------------------------------------------------------------------------------
template <int NT, bool IS_QK>
__device__ __forceinline__ void emit_indices(int32_t* __restrict__ out_idx, int64_t out_nnz, int64_t base,
                                             int c, int C, int w, int h, const int* __restrict__ pos,
                                             int tid) {
    const int J = IS_QK ? c : C;
    const int count = c * J;
    int32_t* r0 = out_idx + base;
    int32_t* r1 = r0 + out_nnz;
    int32_t* r2 = r1 + out_nnz;
    int32_t* r3 = r2 + out_nnz;
    for (int f = tid * 4; f < count; f += NT * 4) {
        int i = f / J, j = f - i * J;
        int a[4], b[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int ii = i < c ? i : c - 1;              // clamp for the masked tail lanes
            a[q] = pos[ii];
            b[q] = IS_QK ? pos[j] : j;
            if (++j == J) { j = 0; ++i; }
        }
        if (f + 3 < count) {
            i32x4_u vw = {w, w, w, w}, vh = {h, h, h, h};
            i32x4_u va = {a[0], a[1], a[2], a[3]}, vb = {b[0], b[1], b[2], b[3]};
            *reinterpret_cast<i32x4_u*>(r0 + f) = vw;
            *reinterpret_cast<i32x4_u*>(r1 + f) = vh;
            *reinterpret_cast<i32x4_u*>(r2 + f) = va;
            *reinterpret_cast<i32x4_u*>(r3 + f) = vb;
        } else {
            for (int q = 0; q < 4 && f + q < count; ++q) {
                r0[f + q] = w; r1[f + q] = h; r2[f + q] = a[q]; r3[f + q] = b[q];
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// main kernel
// ------------------------------------------------------------------------------------------
struct GroupTable {
    const int32_t* c;          // [G]
    const int32_t* row_start;  // [G] exclusive scan of c
    const int32_t* sq_start;   // [G] exclusive scan of c*c
    const int32_t* window;     // [G] or null
    const int32_t* head;       // [G] or null
};

template <typename T, int MODE, bool EMIT>
__global__ __launch_bounds__(256) void block_product_kernel(const T* __restrict__ m1, const T* __restrict__ m2,
                                                            GroupTable gt, int64_t G, int C,
                                                            const int32_t* __restrict__ tok_pos,
                                                            T* __restrict__ out, int32_t* __restrict__ out_idx,
                                                            int64_t out_nnz) {
    using BS = BlockShape<MODE>;
    constexpr int WG_LDS = KC * (BS::IB + 4) + KC * (BS::JB + 4);
    constexpr int WAVE_LDS = 2 * KC * (32 + 4);
    constexpr int LDS_FLOATS = WG_LDS > 4 * WAVE_LDS ? WG_LDS : 4 * WAVE_LDS;
    __shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS];
    __shared__ int pos_s[EMIT ? MAX_POS : 1];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int64_t g0 = (int64_t)blockIdx.x * GROUPS_PER_WG;

    // this wave's own group (wave path) — also used to decide the path for the whole workgroup
    const int64_t gw = g0 + wave;
    const int cw = gw < G ? gt.c[gw] : 0;
    int cmax = 0;
#pragma unroll
    for (int q = 0; q < GROUPS_PER_WG; ++q) {
        const int64_t g = g0 + q;
        const int cq = g < G ? gt.c[g] : 0;
        cmax = cq > cmax ? cq : cmax;
    }
    const bool small = cmax <= 32 && C <= 32;

    if (small) {
        // ---------------- one group per wavefront ----------------
        float* At = lds + wave * WAVE_LDS;
        float* Bs = At + KC * 36;
        const bool active = cw > 0;
        GroupDims d = {0, 0, 0, 0, 0, 0};
        int64_t rs = 0, ss = 0;
        if (active) {
            rs = gt.row_start[gw];
            ss = gt.sq_start[gw];
            d = group_dims<MODE>(cw, C, rs, ss);
        }
        const T* A = m1 + d.a_off;
        const T* B = m2 + d.b_off;
        stage_transposed<64, 32, T>(A, d.I, d.K, 0, 0, At, lane);
        if (b_is_kmajor<MODE>()) stage_direct<64, 32, T>(B, d.K, d.J, 0, 0, Bs, lane);
        else stage_transposed<64, 32, T>(B, d.J, d.K, 0, 0, Bs, lane);
        if (EMIT && active && lane < cw) pos_s[wave * 32 + lane] = tok_pos[(rs + lane) * C];
        __syncthreads();
        float acc[4][4] = {};
        const int ti = lane >> 3, tj = lane & 7;
        multiply_chunk<32, 32>(At, Bs, ti, tj, d.K, acc);
        if (active) {
            store_tile<T>(out + d.o_off, d.I, d.J, 4 * ti, 4 * tj, acc);
            if (EMIT)
                emit_indices<64, MODE == MODE_QK>(out_idx, out_nnz, d.o_off, cw, C, gt.window[gw], gt.head[gw],
                                                  pos_s + wave * 32, lane);
        }
        return;
    }

    // ---------------- whole workgroup per group, groups one after another ----------------
    float* At = lds;
    float* Bs = lds + KC * (BS::IB + 4);
    constexpr int TJ = BS::JB / 4;
    const int ti = tid / TJ, tj = tid % TJ;
    for (int q = 0; q < GROUPS_PER_WG; ++q) {
        const int64_t g = g0 + q;
        if (g >= G) break;                                   // uniform across the workgroup
        const int c = gt.c[g];
        const int64_t rs = gt.row_start[g], ss = gt.sq_start[g];
        const GroupDims d = group_dims<MODE>(c, C, rs, ss);
        const T* A = m1 + d.a_off;
        const T* B = m2 + d.b_off;
        T* O = out + d.o_off;
        for (int ib = 0; ib < d.I; ib += BS::IB) {
            for (int jb = 0; jb < d.J; jb += BS::JB) {
                float acc[4][4] = {};
                for (int k0 = 0; k0 < d.K; k0 += KC) {
                    __syncthreads();                          // previous chunk fully consumed
                    stage_transposed<256, BS::IB, T>(A, d.I, d.K, ib, k0, At, tid);
                    if (b_is_kmajor<MODE>()) stage_direct<256, BS::JB, T>(B, d.K, d.J, k0, jb, Bs, tid);
                    else stage_transposed<256, BS::JB, T>(B, d.J, d.K, jb, k0, Bs, tid);
                    __syncthreads();
                    const int kmax = d.K - k0 < KC ? d.K - k0 : KC;
                    multiply_chunk<BS::IB, BS::JB>(At, Bs, ti, tj, kmax, acc);
                }
                store_tile<T>(O, d.I, d.J, ib + 4 * ti, jb + 4 * tj, acc);
            }
        }
        if (EMIT) {
            __syncthreads();                                  // pos_s of the previous group consumed
            for (int i = tid; i < c; i += 256) pos_s[i] = tok_pos[(rs + i) * C];
            __syncthreads();
            emit_indices<256, MODE == MODE_QK>(out_idx, out_nnz, d.o_off, c, C, gt.window[g], gt.head[g], pos_s,
                                               tid);
        }
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
            const AccT a = to_acc(A[(int64_t)i * d.K + k]);
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
// One workgroup per four groups; writes are contiguous, the strided reads stay inside the
// group's block (at most a few tens of KB) and are served from cache.
// ------------------------------------------------------------------------------------------
template <typename T, bool IS_RR>
__global__ __launch_bounds__(256) void block_transpose_kernel(const T* __restrict__ in, const int32_t* __restrict__ cs,
                                                              const int32_t* __restrict__ row_start,
                                                              const int32_t* __restrict__ sq_start, int64_t G,
                                                              int C, T* __restrict__ out) {
    const int64_t g0 = (int64_t)blockIdx.x * GROUPS_PER_WG;
    for (int q = 0; q < GROUPS_PER_WG; ++q) {
        const int64_t g = g0 + q;
        if (g >= G) return;
        const int c = cs[g];
        const int64_t off = IS_RR ? (int64_t)sq_start[g] : (int64_t)row_start[g] * C;
        const int rows_out = IS_RR ? c : C;       // out is [rows_out x c]
        const int ld_in = IS_RR ? c : C;          // in  is [c x ld_in]
        const int count = rows_out * c;
        const T* src = in + off;
        T* dst = out + off;
        for (int f = threadIdx.x; f < count; f += 256) {
            const int i = f / c, j = f - i * c;
            dst[f] = src[(int64_t)j * ld_in + i];
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

template <typename T, int MODE, bool EMIT>
static int launch_product(const void* m1, const void* m2, const GroupTable& gt, int64_t G, int C,
                          const int32_t* tok_pos, void* out, int32_t* out_idx, int64_t out_nnz,
                          hipStream_t s) {
    if (G == 0) return 0;
    bool tiled = false;
    if constexpr (!std::is_same<T, double>::value) {
        if (!force_simple()) {
            tiled = true;
            const unsigned blocks = (unsigned)((G + GROUPS_PER_WG - 1) / GROUPS_PER_WG);
            hipLaunchKernelGGL((block_product_kernel<T, MODE, EMIT>), dim3(blocks), dim3(256), 0, s,
                               static_cast<const T*>(m1), static_cast<const T*>(m2), gt, G, C, tok_pos,
                               static_cast<T*>(out), out_idx, out_nnz);
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
                            const int32_t* tok_pos, void* out, int32_t* out_idx, int64_t out_nnz,
                            hipStream_t s) {
    switch (dtype) {
        case SSWIN_F32: return launch_product<float, MODE, EMIT>(m1, m2, gt, G, C, tok_pos, out, out_idx, out_nnz, s);
        case SSWIN_F16: return launch_product<__half, MODE, EMIT>(m1, m2, gt, G, C, tok_pos, out, out_idx, out_nnz, s);
        case SSWIN_BF16: return launch_product<__hip_bfloat16, MODE, EMIT>(m1, m2, gt, G, C, tok_pos, out, out_idx, out_nnz, s);
        case SSWIN_F64: return launch_product<double, MODE, EMIT>(m1, m2, gt, G, C, tok_pos, out, out_idx, out_nnz, s);
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
    SSWIN_CHECK(mat1_v && mat2_v && tok_idx && plan && out_val && out_idx, "block_matmul: null pointer");
    SSWIN_CHECK(out_nnz < (int64_t)INT32_MAX, "block_matmul: output nnz does not fit int32 offsets");
    SSWIN_CHECK(c_max >= 1 && c_max <= MAX_POS,
                "block_matmul: largest group holds %lld tokens; supported range is [1, %d]", (long long)c_max, MAX_POS);
    GroupTable gt{plan, plan + g_cap, plan + 2 * g_cap, plan + 3 * g_cap, plan + 4 * g_cap};
    const int32_t* tok_pos = tok_idx + 2 * M;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (kind == SSWIN_MUL_Q_K)
        return dispatch_product<MODE_QK, true>(dtype, mat1_v, mat2_v, gt, G, C, tok_pos, out_val, out_idx, out_nnz, s);
    return dispatch_product<MODE_PV, true>(dtype, mat1_v, mat2_v, gt, G, C, tok_pos, out_val, out_idx, out_nnz, s);
}

int sswin_block_matmul_grad(int kind, int dtype, const void* m1, const void* m2, const int32_t* c,
                            const int32_t* scans, int64_t G, int C, void* out, void* stream) {
    SSWIN_CHECK(kind >= SSWIN_GRAD_RC_CR && kind <= SSWIN_GRAD_CR_RR,
                "Invalid mul_type code %d. Expected 'rc_cr', 'rr_rc' or 'cr_rr'.", kind);
    SSWIN_CHECK(C > 0 && G >= 0, "block_matmul_grad: bad sizes");
    if (G == 0) return 0;
    SSWIN_CHECK(m1 && m2 && c && scans && out, "block_matmul_grad: null pointer");
    GroupTable gt{c, scans, scans + G, nullptr, nullptr};
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (kind) {
        case SSWIN_GRAD_RC_CR: return dispatch_product<MODE_RC_CR, false>(dtype, m1, m2, gt, G, C, nullptr, out, nullptr, 0, s);
        case SSWIN_GRAD_RR_RC: return dispatch_product<MODE_RR_RC, false>(dtype, m1, m2, gt, G, C, nullptr, out, nullptr, 0, s);
        default: return dispatch_product<MODE_CR_RR, false>(dtype, m1, m2, gt, G, C, nullptr, out, nullptr, 0, s);
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
