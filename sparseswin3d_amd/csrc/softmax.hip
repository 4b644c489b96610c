// Sparse row softmax (forward and backward) over rows given as runs of equal consecutive ids.
//
// One workgroup owns a tile of SM_TILE consecutive non-zeros.  The tile's values and row ids are
// staged in LDS with coalesced loads; run starts are found with wave ballots and compacted into a
// start table; then each 16-lane DPP row of the workgroup walks over the rows that START inside
// the tile.  The row that is still open at the tile end is completed by reading on into the next
// tile(s); the row that was already open at the tile start belongs to an earlier workgroup.  Row
// maxima and sums are reduced with DPP cross-lane moves inside the 16-lane row: no atomics, no
// second pass over HBM, and results do not depend on scheduling.
//
// HBM traffic per non-zero: forward 4 (id) + 4 (value) read, 4 written; backward one more read.
#include "sswin_common.hpp"

namespace sswin {

constexpr int SM_THREADS = 256;
constexpr int SM_TILE = 2048;
constexpr int SM_ROUNDS = SM_TILE / SM_THREADS;   // 8 ballot rounds of 64 per wave
constexpr int VEC_PAD = 4;

__device__ __forceinline__ float exp_t(float x) { return expf(x); }
__device__ __forceinline__ double exp_t(double x) { return exp(x); }
__device__ __forceinline__ float max_t(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ double max_t(double a, double b) { return fmax(a, b); }

template <typename T, bool BWD>
__global__ __launch_bounds__(SM_THREADS) void softmax_rows_kernel(const int32_t* __restrict__ idx_row,
                                                                  const T* __restrict__ v,   // values (fwd) / y (bwd)
                                                                  const T* __restrict__ g,   // upstream grad (bwd)
                                                                  int64_t A, T* __restrict__ out) {
    __shared__ __attribute__((aligned(16))) T val_s[SM_TILE];
    __shared__ __attribute__((aligned(16))) T g_s[BWD ? SM_TILE : VEC_PAD];
    __shared__ int rid_s[SM_TILE + 1];      // rid_s[e + 1] = id of tile element e; rid_s[0] = predecessor
    __shared__ int start_s[SM_TILE + 1];
    __shared__ int wave_cnt_s[SM_THREADS / 64];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t tile_base = (int64_t)blockIdx.x * SM_TILE;
    const int tile_n = (int)((A - tile_base) < SM_TILE ? (A - tile_base) : SM_TILE);

    // 1. stage the tile: 16-byte loads for a whole tile (tile_base is a multiple of the tile and
    // the arrays are 16-byte aligned; the host checks), element loads for the last, partial tile
    constexpr int VEC = 16 / (int)sizeof(T);                 // values per 16 bytes
    typedef T vec_t __attribute__((ext_vector_type(VEC)));
    typedef int ivec_t __attribute__((ext_vector_type(4)));
    if (tile_n == SM_TILE) {
#pragma unroll
        for (int j = 0; j < SM_TILE / (SM_THREADS * VEC); ++j) {
            const int e = (j * SM_THREADS + tid) * VEC;
            *reinterpret_cast<vec_t*>(val_s + e) = *reinterpret_cast<const vec_t*>(v + tile_base + e);
            if (BWD) *reinterpret_cast<vec_t*>(g_s + e) = *reinterpret_cast<const vec_t*>(g + tile_base + e);
        }
#pragma unroll
        for (int j = 0; j < SM_TILE / (SM_THREADS * 4); ++j) {
            const int e = (j * SM_THREADS + tid) * 4;
            const ivec_t r = *reinterpret_cast<const ivec_t*>(idx_row + tile_base + e);
            rid_s[e + 1] = r.x; rid_s[e + 2] = r.y; rid_s[e + 3] = r.z; rid_s[e + 4] = r.w;
        }
    } else {
#pragma unroll
        for (int j = 0; j < SM_ROUNDS; ++j) {
            const int e = j * SM_THREADS + tid;
            if (e < tile_n) {
                val_s[e] = v[tile_base + e];
                rid_s[e + 1] = idx_row[tile_base + e];
                if (BWD) g_s[e] = g[tile_base + e];
            }
        }
    }
    if (tid == 0) rid_s[0] = tile_base > 0 ? idx_row[tile_base - 1] : idx_row[0] - 1;
    __syncthreads();

    // 2. run starts -> start_s[0 .. nrows), in element order
    int rnk[SM_ROUNDS];
    int wave_count = 0;
#pragma unroll
    for (int j = 0; j < SM_ROUNDS; ++j) {
        const int e = wave * (SM_TILE / 4) + j * 64 + lane;
        const bool flag = e < tile_n && rid_s[e + 1] != rid_s[e];
        const unsigned long long mask = __ballot(flag);
        const unsigned long long below = mask & ((1ull << lane) - 1ull);
        rnk[j] = flag ? wave_count + __popcll(below) : -1;
        wave_count += __popcll(mask);
    }
    if (lane == 0) wave_cnt_s[wave] = wave_count;
    __syncthreads();
    int wave_base = 0, nrows = 0;
#pragma unroll
    for (int w = 0; w < SM_THREADS / 64; ++w) {
        const int t = wave_cnt_s[w];
        if (w < wave) wave_base += t;
        nrows += t;
    }
#pragma unroll
    for (int j = 0; j < SM_ROUNDS; ++j)
        if (rnk[j] >= 0) start_s[wave_base + rnk[j]] = wave * (SM_TILE / 4) + j * 64 + lane;
    if (tid == 0) start_s[nrows] = tile_n;
    __syncthreads();

    // 3. rows that start in this tile, one per 16-lane row at a time
    const int sub = tid >> 4, l = tid & 15;
    const int64_t tile_end = tile_base + tile_n;
    for (int lr = sub; lr < nrows; lr += SM_THREADS / 16) {
        const int s = start_s[lr], e_end = start_s[lr + 1];
        // extension of the last row beyond the tile
        int64_t ext = 0;
        if (lr == nrows - 1 && tile_end < A) {
            const int id = rid_s[tile_n];
            while (true) {
                const int64_t p = tile_end + ext + l;
                const int in = (p < A && idx_row[p] == id) ? 1 : 0;
                const int n_in = row16_sum_i32(in);
                ext += n_in;
                if (n_in < 16) break;
            }
        }
        const int64_t ext_end = tile_end + ext;
        if (!BWD) {
            T m = 0;                                    // the row maximum starts from zero
            for (int e = s + l; e < e_end; e += 16) m = max_t(m, val_s[e]);
            for (int64_t p = tile_end + l; p < ext_end; p += 16) m = max_t(m, v[p]);
            m = row16_max(m);
            T sum = 0;
            for (int e = s + l; e < e_end; e += 16) {
                const T x = exp_t(val_s[e] - m);
                val_s[e] = x;
                sum += x;
            }
            for (int64_t p = tile_end + l; p < ext_end; p += 16) sum += exp_t(v[p] - m);
            sum = row16_sum(sum) + (T)1e-8;
            for (int e = s + l; e < e_end; e += 16) val_s[e] = val_s[e] / sum;
            for (int64_t p = tile_end + l; p < ext_end; p += 16) out[p] = exp_t(v[p] - m) / sum;
        } else {
            T dot = 0;
            for (int e = s + l; e < e_end; e += 16) dot += g_s[e] * val_s[e];
            for (int64_t p = tile_end + l; p < ext_end; p += 16) dot += g[p] * v[p];
            dot = row16_sum(dot);
            for (int e = s + l; e < e_end; e += 16) {
                const T y = val_s[e];
                val_s[e] = g_s[e] * y - y * dot;
            }
            for (int64_t p = tile_end + l; p < ext_end; p += 16) {
                const T y = v[p];
                out[p] = g[p] * y - y * dot;
            }
        }
    }
    // 4. the tile's results leave LDS with 16-byte stores.  Elements before the first row start
    // belong to a row of an earlier workgroup, which writes them itself.
    __syncthreads();
    if (nrows == 0) return;
    const int s0 = start_s[0];
#pragma unroll
    for (int j = 0; j < SM_TILE / (SM_THREADS * VEC); ++j) {
        const int e = (j * SM_THREADS + tid) * VEC;
        if (e >= s0 && e + VEC <= tile_n) {
            *reinterpret_cast<vec_t*>(out + tile_base + e) = *reinterpret_cast<const vec_t*>(val_s + e);
        } else {
#pragma unroll
            for (int k = 0; k < VEC; ++k)
                if (e + k >= s0 && e + k < tile_n) out[tile_base + e + k] = val_s[e + k];
        }
    }
}

template <typename T, bool BWD>
static int launch_softmax(const int32_t* idx_row, const void* v, const void* g, int64_t A, void* out,
                          hipStream_t s) {
    const unsigned blocks = (unsigned)((A + SM_TILE - 1) / SM_TILE);
    hipLaunchKernelGGL((softmax_rows_kernel<T, BWD>), dim3(blocks), dim3(SM_THREADS), 0, s, idx_row,
                       static_cast<const T*>(v), static_cast<const T*>(g), A, static_cast<T*>(out));
    return launch_ok(BWD ? "softmax backward" : "softmax forward");
}

// ------------------------------------------------------------------------------------------
// values + bias[head, pos_i, pos_j] (+ -100 where the mask regions of the two positions differ) for a
// [B, H, n, n] product in sorted order, group by group: what sp_add_rpb and sp_add_mask of
// sparse_swin/swin3d_base.py:557-581 compute through a linear index per entry and two gathers.  A group's
// row positions are the third index row at the first entry of each of its rows, its column positions the
// fourth index row along its first row: 2c index reads per group instead of 4c^2.  One wavefront per 32 rows of a group;
// the two roundings of the reference (after the bias, after the mask) are kept for 16-bit values.
// ------------------------------------------------------------------------------------------
constexpr int GBM_MAX_C = 512;
constexpr int GBM_ROWS = 32;                                 // attention rows of a group per wavefront
constexpr int GBM_U = 8;                                     // rows in flight per lane (4: 118 us, 8: 112, 16: 107 on 7^3 windows; 38, 38, 41 on 5^3)

// grid: x = four groups (one per wavefront), y = block of GBM_ROWS rows of the group.
// TABLE: `bias` is the relative position table [rows, H] itself and `code` the linear index of a position
// (bias of positions p, q = table[code[p] - code[q] + offset0]): the table is a few KB where the gathered [H, n, n]
// bias of 7^3 windows is 1.4 MB, so the gathers stay in the L1.
template <typename T, bool TABLE>
__global__ __launch_bounds__(256) void group_bias_mask_kernel(const T* __restrict__ val, const int32_t* __restrict__ row_pos,
                                                              const int32_t* __restrict__ cs, const int32_t* __restrict__ row_start,
                                                              const int32_t* __restrict__ sq_start,
                                                              const int32_t* __restrict__ window,
                                                              const int32_t* __restrict__ head, int64_t G, int n,
                                                              const float* __restrict__ bias, const int32_t* __restrict__ code,
                                                              int offset0, int H, const int8_t* __restrict__ mask,
                                                              int nmw, T* __restrict__ out) {
    using AccT = typename acc_of<T>::type;
    __shared__ int32_t pos_j[4][GBM_MAX_C];                  // position | region << 16 of the columns
    __shared__ int32_t pos_i[4][GBM_ROWS];                   // ... of this block's rows
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int64_t g = (int64_t)blockIdx.x * 4 + wave;
    if (g >= G) return;
    const int c = cs[g];
    const int i0 = blockIdx.y * GBM_ROWS;
    if (i0 >= c) return;
    const int rows = c - i0 < GBM_ROWS ? c - i0 : GBM_ROWS;
    const int h = head[g];
    const int64_t sq = sq_start[g];
    const int32_t* gpos = row_pos + row_start[g];            // window positions of the group's c tokens
    const int8_t* mrow = mask ? mask + (int64_t)(window[g] % nmw) * n : nullptr;
    int32_t* pj = pos_j[wave];
    int32_t* pi = pos_i[wave];
    // low half: the position (TABLE: its code), high half: its mask region
    for (int t = lane; t < c; t += 64) {
        const int b = gpos[t];
        pj[t] = (TABLE ? code[b] : b) | (mrow ? (int)mrow[b] << 16 : 0);
    }
    if (lane < rows) {
        const int a = gpos[i0 + lane];
        pi[lane] = (TABLE ? code[a] : a) | (mrow ? (int)mrow[a] << 16 : 0);
    }
    __builtin_amdgcn_wave_barrier();
    const float* bias_h = TABLE ? bias + h : bias + (int64_t)h * n * n;
    const T* src = val + sq + (int64_t)i0 * c;
    T* dst = out + sq + (int64_t)i0 * c;
    // Row by row, a lane keeps its column: the column's code and region are read once per chunk of columns, the
    // row's are one LDS broadcast, and no entry needs a division.  Rows of at most 32 entries go two to a wavefront.
    const int cw = c <= 32 ? 32 : 64;                        // lanes per row
    const int rstep = c <= 32 ? 2 : 1;                       // rows per step
    const int jl = lane & (cw - 1), rl = c <= 32 ? lane >> 5 : 0;
    for (int j0 = 0; j0 < c; j0 += cw) {
        const int j = j0 + jl;
        const bool jok = j < c;
        const int pbv = pj[jok ? j : 0];
        const int pb_lo = pbv & 0xffff, pb_hi = pbv >> 16;
        for (int i = rl; i < rows; i += GBM_U * rstep) {     // GBM_U steps in flight
            T v[GBM_U];
            int pa[GBM_U];
            float bb[GBM_U];
#pragma unroll
            for (int u = 0; u < GBM_U; ++u) {
                const int ii = i + u * rstep;
                const int ic = ii < rows ? ii : rows - 1;
                v[u] = src[jok ? ic * c + j : 0];
                pa[u] = pi[ic];
                bb[u] = TABLE ? bias_h[((pa[u] & 0xffff) - pb_lo + offset0) * H] : bias_h[(pa[u] & 0xffff) * n + pb_lo];
            }
#pragma unroll
            for (int u = 0; u < GBM_U; ++u) {
                const int ii = i + u * rstep;
                if (ii >= rows || !jok) continue;
                const T with_bias = from_acc<T>(to_acc(v[u]) + to_acc(from_acc<T>((AccT)bb[u])));
                dst[ii * c + j] = mrow ? from_acc<T>(to_acc(with_bias) + ((pa[u] >> 16) != pb_hi ? (AccT)-100 : (AccT)0)) : with_bias;
            }
        }
    }
}

}  // namespace sswin

using namespace sswin;

extern "C" {

int sswin_softmax_last_dim_forward(const int32_t* idx_row, const void* values, int dtype, int64_t A,
                                   void* out, void* stream) {
    SSWIN_CHECK(A >= 0, "softmax forward: negative length");
    if (A == 0) return 0;
    SSWIN_CHECK(idx_row && values && out, "softmax forward: null pointer");
    SSWIN_CHECK(((uintptr_t)idx_row | (uintptr_t)values | (uintptr_t)out) % 16 == 0, "softmax forward: arrays must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == SSWIN_F32) return launch_softmax<float, false>(idx_row, values, nullptr, A, out, s);
    if (dtype == SSWIN_F64) return launch_softmax<double, false>(idx_row, values, nullptr, A, out, s);
    return fail("softmax forward: values must be float32 or float64 (dtype code %d)", dtype);
}

int sswin_softmax_last_dim_backward(const int32_t* idx_row, const void* y, const void* grad, int dtype,
                                    int64_t A, void* out, void* stream) {
    SSWIN_CHECK(A >= 0, "softmax backward: negative length");
    if (A == 0) return 0;
    SSWIN_CHECK(idx_row && y && grad && out, "softmax backward: null pointer");
    SSWIN_CHECK(((uintptr_t)idx_row | (uintptr_t)y | (uintptr_t)grad | (uintptr_t)out) % 16 == 0,
                "softmax backward: arrays must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == SSWIN_F32) return launch_softmax<float, true>(idx_row, y, grad, A, out, s);
    if (dtype == SSWIN_F64) return launch_softmax<double, true>(idx_row, y, grad, A, out, s);
    return fail("softmax backward: values must be float32 or float64 (dtype code %d)", dtype);
}

static int launch_group_bias_mask(const char* who, bool table_form, int dtype, const void* values, const int32_t* row_pos,
                                  int64_t A, const int32_t* plan, int64_t g_cap, int64_t G, int c_max, int n, const float* bias,
                                  const int32_t* code, int offset0, int H, const int8_t* mask, int n_mask_windows, void* out,
                                  void* stream) {
    SSWIN_CHECK(A >= 0 && G >= 0 && G <= g_cap && n > 0 && n < (1 << 15), "%s: bad sizes", who);
    if (A == 0 || G == 0) return 0;
    SSWIN_CHECK(values && row_pos && plan && bias && out, "%s: null pointer", who);
    SSWIN_CHECK(c_max > 0 && c_max <= GBM_MAX_C, "%s: windows of %d tokens are not supported (%d at most)", who, c_max, GBM_MAX_C);
    SSWIN_CHECK(!mask || n_mask_windows > 0, "%s: mask without window count", who);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)((G + 3) / 4), (unsigned)((c_max + GBM_ROWS - 1) / GBM_ROWS));
    const int32_t *cs = plan, *rs = plan + g_cap, *sq = plan + 2 * g_cap, *win = plan + 3 * g_cap, *head = plan + 4 * g_cap;
#define SSWIN_GBM(T)                                                                                                   \
    do {                                                                                                               \
        if (table_form)                                                                                                \
            hipLaunchKernelGGL((group_bias_mask_kernel<T, true>), grid, dim3(256), 0, s, static_cast<const T*>(values), \
                               row_pos, cs, rs, sq, win, head, G, n, bias, code, offset0, H, mask,                     \
                               n_mask_windows, static_cast<T*>(out));                                                  \
        else                                                                                                           \
            hipLaunchKernelGGL((group_bias_mask_kernel<T, false>), grid, dim3(256), 0, s, static_cast<const T*>(values), \
                               row_pos, cs, rs, sq, win, head, G, n, bias, code, offset0, H, mask,                     \
                               n_mask_windows, static_cast<T*>(out));                                                  \
    } while (0)
    switch (dtype) {
        case SSWIN_F32: SSWIN_GBM(float); break;
        case SSWIN_F64: SSWIN_GBM(double); break;
        case SSWIN_F16: SSWIN_GBM(__half); break;
        case SSWIN_BF16: SSWIN_GBM(__hip_bfloat16); break;
        default: return fail("%s: unsupported value dtype %d", who, dtype);
    }
#undef SSWIN_GBM
    return launch_ok(who);
}

int sswin_group_add_bias_mask(int dtype, const void* values, const int32_t* row_pos, int64_t A, const int32_t* plan, int64_t g_cap,
                              int64_t G, int c_max, int n, const float* bias, const int8_t* mask, int n_mask_windows,
                              void* out, void* stream) {
    return launch_group_bias_mask("group_add_bias_mask", false, dtype, values, row_pos, A, plan, g_cap, G, c_max, n, bias, nullptr, 0,
                                  1, mask, n_mask_windows, out, stream);
}

int sswin_group_add_table_bias_mask(int dtype, const void* values, const int32_t* row_pos, int64_t A, const int32_t* plan,
                                    int64_t g_cap, int64_t G, int c_max, int n, const float* table, int table_rows, int H,
                                    const int32_t* code, int offset0, const int8_t* mask, int n_mask_windows, void* out,
                                    void* stream) {
    SSWIN_CHECK(table_rows > 0 && table_rows < (1 << 15) && H > 0 && (A == 0 || G == 0 || code),
                "group_add_table_bias_mask: bad table");
    return launch_group_bias_mask("group_add_table_bias_mask", true, dtype, values, row_pos, A, plan, g_cap, G, c_max, n, table, code,
                                  offset0, H, mask, n_mask_windows, out, stream);
}

}  // extern "C"
