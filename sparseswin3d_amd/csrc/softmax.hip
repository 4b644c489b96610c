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

}  // extern "C"
