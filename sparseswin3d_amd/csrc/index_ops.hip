// Integer index operators: flatten_indices, sort_indices, unique_consecutive_indices,
// return_inverse, qkv_sparse_indices.  All of them are HBM-bound integer work; the kernels
// are laid out for coalesced 64-lane accesses and use no floating point.
#include <cstring>
#include <mutex>
#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/iterator/counting_iterator.hpp>

#include "scan.hpp"
#include "sswin_common.hpp"

namespace sswin {

// thread-local error buffer lives here (one definition for the whole library)
char* error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}
int fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return 1;
}

// ------------------------------------------------------------------------------------------
// flatten_indices
// ------------------------------------------------------------------------------------------
struct Strides {
    uint32_t s[8];
};

template <int NDIM>
__global__ __launch_bounds__(256) void flatten_kernel(const int32_t* __restrict__ idx, int64_t M,
                                                      Strides st, int32_t* __restrict__ out) {
    // four consecutive columns per thread; vector path when the row pitch keeps 16-byte alignment
    const int64_t m4 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (m4 >= M) return;
    if ((M & 3) == 0 && m4 + 3 < M) {
        uint32_t h0 = 0, h1 = 0, h2 = 0, h3 = 0;
#pragma unroll
        for (int i = 0; i < NDIM; ++i) {
            const int4 v = *reinterpret_cast<const int4*>(idx + (int64_t)i * M + m4);
            h0 += (uint32_t)v.x * st.s[i];
            h1 += (uint32_t)v.y * st.s[i];
            h2 += (uint32_t)v.z * st.s[i];
            h3 += (uint32_t)v.w * st.s[i];
        }
        *reinterpret_cast<int4*>(out + m4) = make_int4((int)h0, (int)h1, (int)h2, (int)h3);
    } else {
        for (int64_t m = m4; m < M && m < m4 + 4; ++m) {
            uint32_t h = 0;
#pragma unroll
            for (int i = 0; i < NDIM; ++i) h += (uint32_t)idx[(int64_t)i * M + m] * st.s[i];
            out[m] = (int)h;
        }
    }
}

template <int NDIM>
static void launch_flatten(const int32_t* idx, int64_t M, const Strides& st, int32_t* out,
                           hipStream_t s) {
    const int64_t threads = (M + 3) / 4;
    hipLaunchKernelGGL(flatten_kernel<NDIM>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s,
                       idx, M, st, out);
}

// ------------------------------------------------------------------------------------------
// unique_consecutive_indices: inclusive scan of "differs from predecessor" flags
// ------------------------------------------------------------------------------------------
template <typename K>
struct RunFlagLoad {
    const K* x;
    __device__ int operator()(int64_t i) const { return (i > 0 && x[i] != x[i - 1]) ? 1 : 0; }
};
struct InclusiveStore {
    int32_t* out;
    __device__ void operator()(int64_t i, int ex, int item) const { out[i] = ex + item; }
};

// int32 keys: 16-byte loads and stores.  A tile is 256 threads x 4 rounds x 4 keys; round v of
// thread t covers keys (v*256 + t)*4 .. +3 of the tile, so every access is fully coalesced.  The
// four per-round counts of a thread are scanned at once, packed 16 bits apiece into an int64.
constexpr int UC_TILE = 4096;

__device__ __forceinline__ void uc_flags(const int32_t* __restrict__ x, int64_t M, int64_t tile0, int v, int4& key,
                                         int (&f)[4]) {
    const int lane = threadIdx.x & 63;
    const int64_t i0 = tile0 + ((int64_t)v * 256 + threadIdx.x) * 4;
    key = make_int4(0, 0, 0, 0);
    if (i0 + 3 < M) {
        key = *reinterpret_cast<const int4*>(x + i0);
    } else {
        if (i0 < M) key.x = x[i0];
        if (i0 + 1 < M) key.y = x[i0 + 1];
        if (i0 + 2 < M) key.z = x[i0 + 2];
    }
    int prev = __shfl_up(key.w, 1, 64);                       // last key of the left neighbour
    if (lane == 0) prev = (i0 > 0 && i0 < M) ? x[i0 - 1] : key.x;
    f[0] = (i0 > 0 && i0 < M && key.x != prev) ? 1 : 0;
    f[1] = (i0 + 1 < M && key.y != key.x) ? 1 : 0;
    f[2] = (i0 + 2 < M && key.z != key.y) ? 1 : 0;
    f[3] = (i0 + 3 < M && key.w != key.z) ? 1 : 0;
}

__global__ __launch_bounds__(256) void uc_reduce_kernel(const int32_t* __restrict__ x, int64_t M,
                                                        int32_t* __restrict__ tile_sums) {
    __shared__ int32_t lds[4];
    const int64_t tile0 = (int64_t)blockIdx.x * UC_TILE;
    int cnt = 0;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        int4 key;
        int f[4];
        uc_flags(x, M, tile0, v, key, f);
        cnt += f[0] + f[1] + f[2] + f[3];
    }
    int32_t total;
    (void)block_exclusive_scan<int32_t, 4>(cnt, lds, &total);
    if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

__global__ __launch_bounds__(256) void uc_scan_kernel(const int32_t* __restrict__ x, int64_t M,
                                                      const int32_t* __restrict__ tile_offs,
                                                      int32_t* __restrict__ out) {
    __shared__ int64_t lds[4];
    const int64_t tile0 = (int64_t)blockIdx.x * UC_TILE;
    int f[4][4];
    int64_t packed = 0;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        int4 key;
        uc_flags(x, M, tile0, v, key, f[v]);
        packed |= (int64_t)(f[v][0] + f[v][1] + f[v][2] + f[v][3]) << (16 * v);
    }
    int64_t total;
    const int64_t ex = block_exclusive_scan<int64_t, 4>(packed, lds, &total);
    int base = tile_offs[blockIdx.x];                          // flags before this tile
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        int r = base + (int)((ex >> (16 * v)) & 0xffff);      // flags before this thread's keys of round v
        const int64_t i0 = tile0 + ((int64_t)v * 256 + threadIdx.x) * 4;
        int4 o;
        r += f[v][0]; o.x = r;
        r += f[v][1]; o.y = r;
        r += f[v][2]; o.z = r;
        r += f[v][3]; o.w = r;
        if (i0 + 3 < M) {
            *reinterpret_cast<int4*>(out + i0) = o;
        } else {
            if (i0 < M) out[i0] = o.x;
            if (i0 + 1 < M) out[i0 + 1] = o.y;
            if (i0 + 2 < M) out[i0 + 2] = o.z;
        }
        base += (int)((total >> (16 * v)) & 0xffff);          // all flags of round v
    }
}

static int unique_consecutive_i32(const int32_t* keys, int64_t M, int32_t* out, int32_t* tile_sums, hipStream_t s) {
    if (M <= 0) return 0;
    const int64_t tiles = (M + UC_TILE - 1) / UC_TILE;
    hipLaunchKernelGGL(uc_reduce_kernel, dim3((unsigned)tiles), dim3(256), 0, s, keys, M, tile_sums);
    hipLaunchKernelGGL((scan_tile_sums_kernel<int32_t>), dim3(1), dim3(1024), 0, s, tile_sums, tiles, (int32_t*)nullptr);
    hipLaunchKernelGGL(uc_scan_kernel, dim3((unsigned)tiles), dim3(256), 0, s, keys, M, tile_sums, out);
    return launch_ok("unique_consecutive");
}

template <typename K>
static int unique_consecutive_t(const void* keys, int64_t M, int32_t* out, int32_t* tile_sums,
                                hipStream_t s) {
    RunFlagLoad<K> ld{static_cast<const K*>(keys)};
    InclusiveStore st{out};
    return device_exclusive_scan<int32_t>(ld, st, M, tile_sums, (int32_t*)nullptr, s, "unique_consecutive");
}

// ------------------------------------------------------------------------------------------
// presence bitmap helpers (return_inverse, qkv_sparse_indices)
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t* __restrict__ p, int64_t n, uint32_t v) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) p[i] = v;
}

// Values outside [0, limit) set no bit (the bitmap has `limit` bits): they are counted in *bad instead.
__global__ __launch_bounds__(256) void set_bits_kernel(const int32_t* __restrict__ x, int64_t M, int64_t limit,
                                                       uint32_t* __restrict__ bits, int32_t* __restrict__ bad) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < M) {
        const uint32_t v = (uint32_t)x[i];
        if ((int64_t)v < limit)
            atomicOr(&bits[v >> 5], 1u << (v & 31));
        else
            atomicAdd(bad, 1);
    }
}

// (window, pos) pairs -> bit window*n + pos; pairs outside [0,B) x [0,n) set no bit and are counted in *bad
__global__ __launch_bounds__(256) void set_bits_pairs_kernel(const int32_t* __restrict__ ind, int64_t N, int B,
                                                             int n, uint32_t* __restrict__ bits,
                                                             int32_t* __restrict__ bad) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < N) {
        const int2 wp = *reinterpret_cast<const int2*>(ind + 2 * i);
        if ((unsigned)wp.x < (unsigned)B && (unsigned)wp.y < (unsigned)n) {
            const uint64_t v = (uint64_t)(uint32_t)wp.x * (uint32_t)n + (uint32_t)wp.y;
            atomicOr(&bits[v >> 5], 1u << (v & 31));
        } else {
            atomicAdd(bad, 1);
        }
    }
}

struct PopcLoad {
    const uint32_t* bits;
    __device__ int operator()(int64_t i) const { return __popc(bits[i]); }
};
struct ExclusiveStore {
    int32_t* out;
    __device__ void operator()(int64_t i, int ex, int) const { out[i] = ex; }
};

__device__ __forceinline__ int rank_of_bit(const uint32_t* __restrict__ bits,
                                           const int32_t* __restrict__ word_prefix, uint64_t v) {
    const uint64_t w = v >> 5;
    const uint32_t below = bits[w] & ((1u << (v & 31)) - 1u);
    return word_prefix[w] + __popc(below);
}

__global__ __launch_bounds__(256) void rank_lookup_kernel(const int32_t* __restrict__ x, int64_t M, int64_t limit,
                                                          const uint32_t* __restrict__ bits,
                                                          const int32_t* __restrict__ word_prefix,
                                                          int32_t* __restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < M) {
        const uint32_t v = (uint32_t)x[i];
        out[i] = (int64_t)v < limit ? rank_of_bit(bits, word_prefix, v) : -1;    // out of range: counted by set_bits_kernel
    }
}

// max of int32 array into a single device int (one atomicMax per block)
__global__ __launch_bounds__(256) void max_i32_kernel(const int32_t* __restrict__ x, int64_t M,
                                                      int32_t* __restrict__ out) {
    __shared__ int lds[4];
    int m = INT32_MIN;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < M; i += (int64_t)gridDim.x * 256)
        m = max(m, x[i]);
    m = wave_max_i32(m);
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) atomicMax(out, max(max(lds[0], lds[1]), max(lds[2], lds[3])));
}

// ------------------------------------------------------------------------------------------
// qkv_sparse_indices
// ------------------------------------------------------------------------------------------
// Per voxel: rank r in (window, pos) order, and for rank r the source voxel, the rank T of the
// first token of its window and the token count c of its window.
// status: [0] pairs out of range, [1] distinct pairs (total of the bitmap scan).  The expansion kernels
// below run only if status[0] == 0 and status[1] == N: otherwise ranks would repeat or be missing and
// the destination slots computed from them would be arbitrary.
__device__ __forceinline__ bool pairs_valid(const int32_t* __restrict__ status, int64_t N) {
    return status[0] == 0 && (int64_t)status[1] == N;
}

__global__ __launch_bounds__(256) void voxel_rank_kernel(const int32_t* __restrict__ ind, int64_t N, int B, int n,
                                                         const uint32_t* __restrict__ bits,
                                                         const int32_t* __restrict__ word_prefix,
                                                         const int32_t* __restrict__ status,
                                                         int32_t* __restrict__ order,   // [N] voxel of rank r
                                                         int32_t* __restrict__ win_T,   // [N] by rank
                                                         int32_t* __restrict__ win_c) { // [N] by rank
    const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (v >= N || !pairs_valid(status, N)) return;
    const int2 wp = *reinterpret_cast<const int2*>(ind + 2 * v);
    (void)B;
    const uint64_t first = (uint64_t)(uint32_t)wp.x * (uint32_t)n;
    const int r = rank_of_bit(bits, word_prefix, first + (uint32_t)wp.y);
    const int T = rank_of_bit(bits, word_prefix, first);
    const int Tn = rank_of_bit(bits, word_prefix, first + (uint32_t)n);  // bitmap has a padding word
    order[r] = (int32_t)v;
    win_T[r] = T;
    win_c[r] = Tn - T;
}

// Element-level COO rows in input voxel order; four consecutive channels per thread.
// idx_qv rows: window, head, pos, channel.  idx_k rows: window, head, channel, pos.
__global__ __launch_bounds__(256) void expand_coo_kernel(const int32_t* __restrict__ ind, int64_t E,
                                                         int H, int hd, int32_t* __restrict__ idx_qv,
                                                         int32_t* __restrict__ idx_k) {
    const int64_t e = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (e >= E) return;
    const int D = H * hd;
    const int64_t v = e / D;
    const int local = (int)(e - v * D);
    const int h = local / hd, ch = local - h * hd;
    const int2 wp = *reinterpret_cast<const int2*>(ind + 2 * v);
    const int4 w4 = make_int4(wp.x, wp.x, wp.x, wp.x);
    const int4 h4 = make_int4(h, h, h, h);
    const int4 p4 = make_int4(wp.y, wp.y, wp.y, wp.y);
    const int4 c4 = make_int4(ch, ch + 1, ch + 2, ch + 3);
    *reinterpret_cast<int4*>(idx_qv + e) = w4;
    *reinterpret_cast<int4*>(idx_qv + E + e) = h4;
    *reinterpret_cast<int4*>(idx_qv + 2 * E + e) = p4;
    *reinterpret_cast<int4*>(idx_qv + 3 * E + e) = c4;
    *reinterpret_cast<int4*>(idx_k + e) = w4;
    *reinterpret_cast<int4*>(idx_k + E + e) = h4;
    *reinterpret_cast<int4*>(idx_k + 2 * E + e) = c4;
    *reinterpret_cast<int4*>(idx_k + 3 * E + e) = p4;
}

// sorted_qv: destination slot hd*(H*T + h*c + i) + ch holds source element v*D + h*hd + ch.
// One thread per (rank, head, channel quad): a 16-byte store, 128 contiguous bytes per hd=32 row.
__global__ __launch_bounds__(256) void sorted_qv_kernel(const int32_t* __restrict__ order,
                                                        const int32_t* __restrict__ win_T,
                                                        const int32_t* __restrict__ win_c,
                                                        const int32_t* __restrict__ status, int64_t N,
                                                        int H, int hd, int32_t* __restrict__ sorted_qv) {
    const int q = hd >> 2;                                  // channel quads per head
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t total = N * H * q;
    if (t >= total) return;
    if (!pairs_valid(status, N)) {                           // defined (all zero) output for a caller that checks later
        *reinterpret_cast<int4*>(sorted_qv + t * 4) = make_int4(0, 0, 0, 0);
        return;
    }
    const int cq = (int)(t % q);
    const int64_t rh = t / q;
    const int h = (int)(rh % H);
    const int64_t r = rh / H;
    const int T = win_T[r], c = win_c[r];
    const int i = (int)(r - T);
    const int64_t dst = (int64_t)hd * ((int64_t)H * T + (int64_t)h * c + i) + cq * 4;
    const int src = (int)((int64_t)order[r] * H * hd + h * hd + cq * 4);
    *reinterpret_cast<int4*>(sorted_qv + dst) = make_int4(src, src + 1, src + 2, src + 3);
}

// sorted_k: destination slot hd*(H*T + h*c) + ch*c + i.  Lanes run over consecutive ranks, so
// for a fixed (head, channel) a wave writes runs of c contiguous ints per window.
__global__ __launch_bounds__(256) void sorted_k_kernel(const int32_t* __restrict__ order,
                                                       const int32_t* __restrict__ win_T,
                                                       const int32_t* __restrict__ win_c,
                                                       const int32_t* __restrict__ status, int64_t N,
                                                       int H, int hd, int32_t* __restrict__ sorted_k) {
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (r >= N) return;
    if (!pairs_valid(status, N)) {
        int32_t* row = sorted_k + ((int64_t)blockIdx.y * N + r) * hd;
        for (int ch = 0; ch < hd; ++ch) row[ch] = 0;
        return;
    }
    const int T = win_T[r], c = win_c[r];
    const int i = (int)(r - T);
    const int h = blockIdx.y;
    const int64_t base = (int64_t)hd * ((int64_t)H * T + (int64_t)h * c) + i;
    const int src = (int)((int64_t)order[r] * H * hd + h * hd);
    for (int ch = 0; ch < hd; ++ch) sorted_k[base + (int64_t)ch * c] = src + ch;
}

// ------------------------------------------------------------------------------------------
// Values between voxel order and operand order.  A token tensor holds, for voxel v, the `hd` channels of head
// h at vox[v * stride + col0 + h * hd ...]; the sorted COO operands of qkv_sparse_cuda hold them at
//   Q, V (and any product with their structure):  hd * (H*T + h*c + i) + ch
//   K^T:                                           hd * (H*T + h*c) + ch * c + i
// for the voxel of rank T + i in a window of c tokens.  Both are permutations of the N*H*hd values, so the
// gradient of a copy in one direction is the copy in the other direction: no index_add, no atomics.
// ------------------------------------------------------------------------------------------
// One thread per (rank, head, piece of V bytes).  to_operand: voxel rows -> operand; else operand -> voxel rows.
template <typename V>
__global__ __launch_bounds__(256) void qv_order_copy_kernel(const int32_t* __restrict__ order, const int32_t* __restrict__ win_T,
                                                            const int32_t* __restrict__ win_c,
                                                            const int32_t* __restrict__ status, int64_t N, int H,
                                                            int pieces, char* __restrict__ vox, int64_t row_bytes,
                                                            int64_t col0_bytes, char* __restrict__ val, bool to_operand) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= N * H * pieces || !pairs_valid(status, N)) return;
    const int pc = (int)(t % pieces);
    const int64_t rh = t / pieces;
    const int h = (int)(rh % H);
    const int64_t r = rh / H;
    const int T = win_T[r], c = win_c[r];
    const int64_t row = (int64_t)H * T + (int64_t)h * c + (r - T);
    V* pv = reinterpret_cast<V*>(vox + (int64_t)order[r] * row_bytes + col0_bytes) + (int64_t)h * pieces + pc;
    V* po = reinterpret_cast<V*>(val) + row * pieces + pc;
    if (to_operand)
        *po = *pv;
    else
        *pv = *po;
}

// The same copy with every value multiplied by `scale` on the way (the `q * scale` of the attention module and, in the
// other direction, its gradient): one thread per (rank, head, piece of VEC values); the product is taken in the
// accumulation type of T and rounded once, as an elementwise multiply of the copied array would.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void qv_order_scale_kernel(const int32_t* __restrict__ order, const int32_t* __restrict__ win_T,
                                                             const int32_t* __restrict__ win_c,
                                                             const int32_t* __restrict__ status, int64_t N, int H,
                                                             int pieces, char* __restrict__ vox, int64_t row_bytes,
                                                             int64_t col0_bytes, char* __restrict__ val, bool to_operand,
                                                             typename acc_of<T>::type scale) {
    struct __attribute__((aligned(sizeof(T) * VEC))) Piece { T v[VEC]; };
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= N * H * pieces || !pairs_valid(status, N)) return;
    const int pc = (int)(t % pieces);
    const int64_t rh = t / pieces;
    const int h = (int)(rh % H);
    const int64_t r = rh / H;
    const int T0 = win_T[r], c = win_c[r];
    const int64_t row = (int64_t)H * T0 + (int64_t)h * c + (r - T0);
    Piece* pv = reinterpret_cast<Piece*>(vox + (int64_t)order[r] * row_bytes + col0_bytes) + (int64_t)h * pieces + pc;
    Piece* po = reinterpret_cast<Piece*>(val) + row * pieces + pc;
    Piece x = to_operand ? *pv : *po;
#pragma unroll
    for (int u = 0; u < VEC; ++u) x.v[u] = from_acc<T>(to_acc(x.v[u]) * scale);
    if (to_operand)
        *po = x;
    else
        *pv = x;
}

template <typename T>
static void launch_qv_scale(bool wide, const int32_t* order, const int32_t* win_T, const int32_t* win_c, const int32_t* status,
                            int64_t N, int H, int hd, char* v, int64_t row_bytes, int64_t col0_bytes, char* o, bool to_operand,
                            double scale, hipStream_t s) {
    constexpr int VEC = 16 / (int)sizeof(T);
    using A = typename acc_of<T>::type;
    if (wide) {
        const int pieces = hd / VEC;
        hipLaunchKernelGGL((qv_order_scale_kernel<T, VEC>), dim3((unsigned)((N * H * pieces + 255) / 256)), dim3(256), 0, s, order,
                           win_T, win_c, status, N, H, pieces, v, row_bytes, col0_bytes, o, to_operand, (A)scale);
    } else {
        hipLaunchKernelGGL((qv_order_scale_kernel<T, 1>), dim3((unsigned)((N * H * hd + 255) / 256)), dim3(256), 0, s, order,
                           win_T, win_c, status, N, H, hd, v, row_bytes, col0_bytes, o, to_operand, (A)scale);
    }
}

// One thread per rank and head (blockIdx.y), walking over the channels: for a fixed channel the lanes of a
// wavefront touch runs of c consecutive operand values per window; a lane's own voxel row stays in cache
// over the walk.
template <typename V>
__global__ __launch_bounds__(256) void k_order_copy_kernel(const int32_t* __restrict__ order, const int32_t* __restrict__ win_T,
                                                           const int32_t* __restrict__ win_c,
                                                           const int32_t* __restrict__ status, int64_t N, int H, int hd,
                                                           char* __restrict__ vox, int64_t row_bytes, int64_t col0_bytes,
                                                           char* __restrict__ val, bool to_operand) {
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (r >= N || !pairs_valid(status, N)) return;
    const int T = win_T[r], c = win_c[r];
    const int h = blockIdx.y;
    V* pv = reinterpret_cast<V*>(vox + (int64_t)order[r] * row_bytes + col0_bytes) + (int64_t)h * hd;
    V* po = reinterpret_cast<V*>(val) + (int64_t)hd * ((int64_t)H * T + (int64_t)h * c) + (r - T);
    if (to_operand) {
        for (int ch0 = 0; ch0 < hd; ch0 += 8) {
            V x[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (ch0 + u < hd) x[u] = pv[ch0 + u];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (ch0 + u < hd) po[(int64_t)(ch0 + u) * c] = x[u];
        }
    } else {
        for (int ch0 = 0; ch0 < hd; ch0 += 8) {
            V x[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (ch0 + u < hd) x[u] = po[(int64_t)(ch0 + u) * c];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (ch0 + u < hd) pv[ch0 + u] = x[u];
        }
    }
}

// The same through LDS for head slices of whole 16-byte pieces: a workgroup takes 64 consecutive ranks of one
// head (blockIdx.y); voxel rows are touched in whole slices (hd * sizeof(V) contiguous bytes, 16 per lane) and
// the operand in runs of consecutive ranks per channel, so both sides of the copy are coalesced.
template <typename V, int HD>
__global__ __launch_bounds__(256) void k_order_copy_lds_kernel(const int32_t* __restrict__ order, const int32_t* __restrict__ win_T,
                                                               const int32_t* __restrict__ win_c,
                                                               const int32_t* __restrict__ status, int64_t N, int H,
                                                               char* __restrict__ vox, int64_t row_bytes, int64_t col0_bytes,
                                                               char* __restrict__ val, bool to_operand) {
    constexpr int PER16 = 16 / (int)sizeof(V);               // values per 16-byte piece
    constexpr int PIECES = HD / PER16;                       // pieces per head slice
    constexpr int ROWS_PER_PASS = 256 / PIECES;
    __shared__ V tile[64][HD + 1];
    __shared__ int64_t s_base[64];                           // operand position of (rank, channel 0)
    __shared__ int32_t s_c[64];
    __shared__ int32_t s_vox[64];
    if (!pairs_valid(status, N)) return;
    const int64_t r0 = (int64_t)blockIdx.x * 64;
    const int h = blockIdx.y;
    const int tid = threadIdx.x;
    if (tid < 64) {
        const int64_t r = r0 + tid;
        if (r < N) {
            const int T = win_T[r], c = win_c[r];
            s_base[tid] = (int64_t)HD * ((int64_t)H * T + (int64_t)h * c) + (r - T);
            s_c[tid] = c;
            s_vox[tid] = order[r];
        } else {
            s_c[tid] = 0;
        }
    }
    __syncthreads();
    V* o = reinterpret_cast<V*>(val);
    const int lane_r = tid & 63, ch0 = tid >> 6;             // operand side: 64 ranks x 4 channels per pass
    const int piece = tid % PIECES, prow = tid / PIECES;     // voxel side: rows x 16-byte pieces
    if (to_operand) {
        for (int rr = prow; rr < 64; rr += ROWS_PER_PASS) {
            if (s_c[rr] == 0) continue;
            const int4 x = *reinterpret_cast<const int4*>(vox + (int64_t)s_vox[rr] * row_bytes + col0_bytes +
                                                          ((int64_t)h * HD + piece * PER16) * sizeof(V));
            const V* xv = reinterpret_cast<const V*>(&x);
#pragma unroll
            for (int u = 0; u < PER16; ++u) tile[rr][piece * PER16 + u] = xv[u];
        }
        __syncthreads();
        const int c = s_c[lane_r];
        if (c > 0) {
            const int64_t base = s_base[lane_r];
#pragma unroll 4
            for (int ch = ch0; ch < HD; ch += 4) o[base + (int64_t)ch * c] = tile[lane_r][ch];
        }
    } else {
        const int c = s_c[lane_r];
        if (c > 0) {
            const int64_t base = s_base[lane_r];
#pragma unroll 4
            for (int ch = ch0; ch < HD; ch += 4) tile[lane_r][ch] = o[base + (int64_t)ch * c];
        }
        __syncthreads();
        for (int rr = prow; rr < 64; rr += ROWS_PER_PASS) {
            if (s_c[rr] == 0) continue;
            int4 x;
            V* xv = reinterpret_cast<V*>(&x);
#pragma unroll
            for (int u = 0; u < PER16; ++u) xv[u] = tile[rr][piece * PER16 + u];
            *reinterpret_cast<int4*>(vox + (int64_t)s_vox[rr] * row_bytes + col0_bytes +
                                     ((int64_t)h * HD + piece * PER16) * sizeof(V)) = x;
        }
    }
}

// Q, K^T and V of one [N, 3, H, HD] token tensor in one launch (Q times `scale` on the way), or the three gradients back
// into it: the K^T copy above with the rows of Q and V of the same 64 ranks and head taken along.  A rank's Q / V slice
// is one contiguous run in the operand (HD values at HD * (H*T + h*c + i)), so it goes piece by piece without LDS.
template <typename T, int HD>
__global__ __launch_bounds__(256) void qkv_order_copy_kernel(const int32_t* __restrict__ order, const int32_t* __restrict__ win_T,
                                                             const int32_t* __restrict__ win_c,
                                                             const int32_t* __restrict__ status, int64_t N, int H,
                                                             char* __restrict__ vox, int64_t row_bytes, int64_t col0_bytes,
                                                             char* __restrict__ val_q, char* __restrict__ val_k,
                                                             char* __restrict__ val_v, bool to_operand, float scale) {
    constexpr int PER16 = 16 / (int)sizeof(T);
    constexpr int PIECES = HD / PER16;
    constexpr int ROWS_PER_PASS = 256 / PIECES;
    __shared__ T tile[64][HD + 1];
    __shared__ int64_t s_base[64];                           // operand position of (rank, channel 0) in K^T order
    __shared__ int64_t s_row[64];                            // the same in Q/V order
    __shared__ int32_t s_c[64];
    __shared__ int32_t s_vox[64];
    if (!pairs_valid(status, N)) return;
    const int64_t r0 = (int64_t)blockIdx.x * 64;
    const int h = blockIdx.y;
    const int tid = threadIdx.x;
    if (tid < 64) {
        const int64_t r = r0 + tid;
        if (r < N) {
            const int T0 = win_T[r], c = win_c[r];
            s_base[tid] = (int64_t)HD * ((int64_t)H * T0 + (int64_t)h * c) + (r - T0);
            s_row[tid] = (int64_t)HD * ((int64_t)H * T0 + (int64_t)h * c + (r - T0));
            s_c[tid] = c;
            s_vox[tid] = order[r];
        } else {
            s_c[tid] = 0;
        }
    }
    __syncthreads();
    T* ok = reinterpret_cast<T*>(val_k);
    const int lane_r = tid & 63, ch0 = tid >> 6;
    const int piece = tid % PIECES, prow = tid / PIECES;
    const int64_t head_bytes = (int64_t)H * HD * sizeof(T);  // Q, K, V slices of a voxel row lie this far apart
    const int64_t in_row = ((int64_t)h * HD + piece * PER16) * sizeof(T);
    if (to_operand) {
        for (int rr = prow; rr < 64; rr += ROWS_PER_PASS) {
            if (s_c[rr] == 0) continue;
            const char* src = vox + (int64_t)s_vox[rr] * row_bytes + col0_bytes + in_row;
            int4 xq = *reinterpret_cast<const int4*>(src);
            const int4 xk = *reinterpret_cast<const int4*>(src + head_bytes);
            const int4 xv = *reinterpret_cast<const int4*>(src + 2 * head_bytes);
            const T* kv = reinterpret_cast<const T*>(&xk);
#pragma unroll
            for (int u = 0; u < PER16; ++u) tile[rr][piece * PER16 + u] = kv[u];
            T* qv = reinterpret_cast<T*>(&xq);
#pragma unroll
            for (int u = 0; u < PER16; ++u) qv[u] = from_acc<T>(to_acc(qv[u]) * scale);
            const int64_t dst = (s_row[rr] + piece * PER16) * sizeof(T);
            *reinterpret_cast<int4*>(val_q + dst) = xq;
            *reinterpret_cast<int4*>(val_v + dst) = xv;
        }
        __syncthreads();
        const int c = s_c[lane_r];
        if (c > 0) {
            const int64_t base = s_base[lane_r];
#pragma unroll 4
            for (int ch = ch0; ch < HD; ch += 4) ok[base + (int64_t)ch * c] = tile[lane_r][ch];
        }
    } else {
        const int c = s_c[lane_r];
        if (c > 0) {
            const int64_t base = s_base[lane_r];
#pragma unroll 4
            for (int ch = ch0; ch < HD; ch += 4) tile[lane_r][ch] = ok[base + (int64_t)ch * c];
        }
        __syncthreads();
        for (int rr = prow; rr < 64; rr += ROWS_PER_PASS) {
            if (s_c[rr] == 0) continue;
            const int64_t from = (s_row[rr] + piece * PER16) * sizeof(T);
            int4 xq = *reinterpret_cast<const int4*>(val_q + from);
            const int4 xv = *reinterpret_cast<const int4*>(val_v + from);
            T* qv = reinterpret_cast<T*>(&xq);
#pragma unroll
            for (int u = 0; u < PER16; ++u) qv[u] = from_acc<T>(to_acc(qv[u]) * scale);
            int4 xk;
            T* kv = reinterpret_cast<T*>(&xk);
#pragma unroll
            for (int u = 0; u < PER16; ++u) kv[u] = tile[rr][piece * PER16 + u];
            char* dst = vox + (int64_t)s_vox[rr] * row_bytes + col0_bytes + in_row;
            *reinterpret_cast<int4*>(dst) = xq;
            *reinterpret_cast<int4*>(dst + head_bytes) = xk;
            *reinterpret_cast<int4*>(dst + 2 * head_bytes) = xv;
        }
    }
}

// Index matrices of the sorted operands written in place (what expand + sort + gather arrive at): idx_qv
// rows (window, head, pos, channel) at hd * (H*T + h*c + i) + ch; idx_k rows (window, head, channel, pos) at
// hd * (H*T + h*c) + ch * c + i.  idx_qv: one thread per (rank, head, channel quad), 16-byte stores.
__global__ __launch_bounds__(256) void sorted_coo_kernel(const int32_t* __restrict__ ind, const int32_t* __restrict__ order,
                                                         const int32_t* __restrict__ win_T, const int32_t* __restrict__ win_c,
                                                         const int32_t* __restrict__ status, int64_t N, int H, int hd,
                                                         int64_t E, int32_t* __restrict__ idx_qv) {
    const int q = hd >> 2;
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= N * H * q) return;
    if (!pairs_valid(status, N)) {                           // defined (all zero) indices for a caller that checks later
        for (int row = 0; row < 4; ++row) *reinterpret_cast<int4*>(idx_qv + row * E + 4 * t) = make_int4(0, 0, 0, 0);
        return;
    }
    const int cq = (int)(t % q);
    const int64_t rh = t / q;
    const int h = (int)(rh % H);
    const int64_t r = rh / H;
    const int T = win_T[r], c = win_c[r];
    const int i = (int)(r - T);
    const int2 wp = *reinterpret_cast<const int2*>(ind + 2 * (int64_t)order[r]);
    const int ch = 4 * cq;
    const int64_t e = (int64_t)hd * ((int64_t)H * T + (int64_t)h * c + i) + ch;
    *reinterpret_cast<int4*>(idx_qv + e) = make_int4(wp.x, wp.x, wp.x, wp.x);
    *reinterpret_cast<int4*>(idx_qv + E + e) = make_int4(h, h, h, h);
    *reinterpret_cast<int4*>(idx_qv + 2 * E + e) = make_int4(wp.y, wp.y, wp.y, wp.y);
    *reinterpret_cast<int4*>(idx_qv + 3 * E + e) = make_int4(ch, ch + 1, ch + 2, ch + 3);
}

// idx_k: one thread per rank and head (blockIdx.y), walking over the channels, so that the lanes of a wavefront
// write runs of consecutive positions
__global__ __launch_bounds__(256) void sorted_coo_k_kernel(const int32_t* __restrict__ ind, const int32_t* __restrict__ order,
                                                           const int32_t* __restrict__ win_T, const int32_t* __restrict__ win_c,
                                                           const int32_t* __restrict__ status, int64_t N, int H, int hd,
                                                           int64_t E, int32_t* __restrict__ idx_k) {
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (r >= N) return;
    const int h = blockIdx.y;
    if (!pairs_valid(status, N)) {                           // defined (all zero) indices for a caller that checks later
        for (int row = 0; row < 4; ++row)
            for (int ch = 0; ch < hd; ++ch) idx_k[row * E + ((int64_t)h * N + r) * hd + ch] = 0;
        return;
    }
    const int T = win_T[r], c = win_c[r];
    const int2 wp = *reinterpret_cast<const int2*>(ind + 2 * (int64_t)order[r]);
    const int64_t base = (int64_t)hd * ((int64_t)H * T + (int64_t)h * c) + (r - T);
#pragma unroll 4
    for (int ch = 0; ch < hd; ++ch) {
        const int64_t e = base + (int64_t)ch * c;
        idx_k[e] = wp.x;
        idx_k[E + e] = h;
        idx_k[2 * E + e] = ch;
        idx_k[3 * E + e] = wp.y;
    }
}

// four 16-byte pieces per thread, each instruction of a wavefront covering 1 KB of contiguous memory
__global__ __launch_bounds__(256) void calibration_copy_kernel(const int4* __restrict__ src, int4* __restrict__ dst, int64_t n16) {
    const int64_t base = (int64_t)blockIdx.x * 1024 + threadIdx.x;
    int4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
        if (base + 256 * u < n16) v[u] = src[base + 256 * u];
#pragma unroll
    for (int u = 0; u < 4; ++u)
        if (base + 256 * u < n16) dst[base + 256 * u] = v[u];
}

}  // namespace sswin

using namespace sswin;

// ==========================================================================================
// C ABI
// ==========================================================================================
extern "C" {

const char* sswin_last_error(void) { return error_buffer(); }
int sswin_abi_version(void) { return 29; }

int sswin_calibration_copy(void* dst, const void* src, int64_t bytes, void* stream) {
    SSWIN_CHECK(bytes >= 0 && bytes % 16 == 0, "calibration_copy: size must be a multiple of 16 bytes");
    if (bytes == 0) return 0;
    SSWIN_CHECK(dst && src && ((uintptr_t)dst % 16) == 0 && ((uintptr_t)src % 16) == 0,
                "calibration_copy: pointers must be 16-byte aligned device addresses");
    const int64_t n16 = bytes / 16;
    const int64_t blocks = (n16 + 256 * 4 - 1) / (256 * 4);
    SSWIN_CHECK(blocks < ((int64_t)1 << 31), "calibration_copy: too large");
    hipLaunchKernelGGL(calibration_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const int4*>(src), static_cast<int4*>(dst), n16);
    return launch_ok("calibration_copy");
}

int sswin_flatten_indices(const int32_t* idx, int ndim, int64_t M, const int32_t* sizes, int32_t* out,
                          void* stream) {
    SSWIN_CHECK(ndim >= 1 && ndim <= 8, "flatten_indices: ndim %d not in [1, 8]", ndim);
    SSWIN_CHECK(M >= 0, "flatten_indices: negative column count");
    if (M == 0) return 0;
    SSWIN_CHECK(idx && out && sizes, "flatten_indices: null pointer");
    Strides st;
    st.s[ndim - 1] = 1u;
    for (int i = ndim - 2; i >= 0; --i) st.s[i] = st.s[i + 1] * (uint32_t)sizes[i + 1];
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (ndim) {
        case 1: launch_flatten<1>(idx, M, st, out, s); break;
        case 2: launch_flatten<2>(idx, M, st, out, s); break;
        case 3: launch_flatten<3>(idx, M, st, out, s); break;
        case 4: launch_flatten<4>(idx, M, st, out, s); break;
        case 5: launch_flatten<5>(idx, M, st, out, s); break;
        case 6: launch_flatten<6>(idx, M, st, out, s); break;
        case 7: launch_flatten<7>(idx, M, st, out, s); break;
        default: launch_flatten<8>(idx, M, st, out, s); break;
    }
    return launch_ok("flatten_indices");
}

// ---- sort_indices ---------------------------------------------------------------------------
size_t sswin_sort_indices_workspace_bytes(int64_t M) {
    if (M <= 0) return 256;
    size_t tmp = 0;
    rocprim::radix_sort_pairs(nullptr, tmp, (const int32_t*)nullptr, (int32_t*)nullptr,
                              rocprim::counting_iterator<int32_t>(0), (int32_t*)nullptr, (size_t)M, 0, 32,
                              (hipStream_t)0);
    return align_up(tmp, 256) + align_up((size_t)M * sizeof(int32_t), 256) + 256;
}

int sswin_sort_indices(const int32_t* keys, int64_t M, int32_t* perm_out, void* ws, size_t ws_bytes,
                       void* stream) {
    SSWIN_CHECK(M >= 0 && M < (int64_t)INT32_MAX, "sort_indices: element count %lld out of range", (long long)M);
    if (M == 0) return 0;
    SSWIN_CHECK(keys && perm_out && ws, "sort_indices: null pointer");
    SSWIN_CHECK(ws_bytes >= sswin_sort_indices_workspace_bytes(M), "sort_indices: workspace too small");
    Carver cv(ws, ws_bytes);
    int32_t* keys_sorted = cv.take<int32_t>((size_t)M);
    size_t tmp = 0;
    rocprim::radix_sort_pairs(nullptr, tmp, keys, keys_sorted, rocprim::counting_iterator<int32_t>(0),
                              perm_out, (size_t)M, 0, 32, (hipStream_t)0);
    void* tmp_ptr = cv.take<char>(tmp);
    SSWIN_CHECK(cv.ok(), "sort_indices: workspace too small");
    SSWIN_HIP(rocprim::radix_sort_pairs(tmp_ptr, tmp, keys, keys_sorted,
                                        rocprim::counting_iterator<int32_t>(0), perm_out, (size_t)M, 0, 32,
                                        static_cast<hipStream_t>(stream)));
    return 0;
}

// ---- unique_consecutive_indices ---------------------------------------------------------------
size_t sswin_unique_consecutive_workspace_bytes(int64_t M) {
    return align_up((size_t)(scan_num_tiles(M > 0 ? M : 1)) * sizeof(int32_t), 256) + 256;
}

// tile_sums: device int32 [scan_num_tiles(M)]
static int unique_consecutive_run(const void* keys, int key_dtype, int64_t M, int32_t* out, int32_t* tile_sums,
                                  hipStream_t s) {
    switch (key_dtype) {
        case SSWIN_I32:
            if (((uintptr_t)keys % 16) == 0 && ((uintptr_t)out % 16) == 0)
                return unique_consecutive_i32(static_cast<const int32_t*>(keys), M, out, tile_sums, s);
            return unique_consecutive_t<int32_t>(keys, M, out, tile_sums, s);
        case SSWIN_I64: return unique_consecutive_t<int64_t>(keys, M, out, tile_sums, s);
        case SSWIN_I16: return unique_consecutive_t<int16_t>(keys, M, out, tile_sums, s);
        case SSWIN_I8: return unique_consecutive_t<int8_t>(keys, M, out, tile_sums, s);
        case SSWIN_U8: return unique_consecutive_t<uint8_t>(keys, M, out, tile_sums, s);
        default: return fail("unique_consecutive_indices: unsupported key dtype %d", key_dtype);
    }
}

int sswin_unique_consecutive_indices(const void* keys, int key_dtype, int64_t M, int32_t* out, void* ws,
                                     size_t ws_bytes, void* stream) {
    SSWIN_CHECK(M >= 0, "unique_consecutive_indices: negative length");
    if (M == 0) return 0;
    SSWIN_CHECK(keys && out && ws, "unique_consecutive_indices: null pointer");
    SSWIN_CHECK(ws_bytes >= sswin_unique_consecutive_workspace_bytes(M),
                "unique_consecutive_indices: workspace too small");
    Carver cv(ws, ws_bytes);
    int32_t* tile_sums = cv.take<int32_t>((size_t)scan_num_tiles(M));
    return unique_consecutive_run(keys, key_dtype, M, out, tile_sums, static_cast<hipStream_t>(stream));
}

// ---- unique_consecutive_indices for callers that cannot allocate ---------------------------------
// The tile sums of the scan live in a file-scope device array instead of a caller workspace.  In host
// code the array's name is only a handle for hipGetSymbolAddress: the device address is looked up
// once per device and that pointer is what the kernels receive.
constexpr int64_t UC_STATIC_TILES = 65536;                                   // 256 KiB per device
constexpr int64_t UC_STATIC_MAX_M = UC_STATIC_TILES * SCAN_TILE;             // 134 217 728 keys
static __device__ __align__(256) int32_t uc_static_scratch[UC_STATIC_TILES];

constexpr int UC_MAX_DEVICES = 64;
static int32_t* uc_static_ptr[UC_MAX_DEVICES] = {nullptr};
static std::mutex uc_static_mutex;

// device address of this device's copy of the array (looked up on the first call per device)
static int uc_static_address(int32_t** out) {
    int dev = -1;
    SSWIN_HIP(hipGetDevice(&dev));
    SSWIN_CHECK(dev >= 0 && dev < UC_MAX_DEVICES, "unique_consecutive_indices_static: device %d out of range", dev);
    std::lock_guard<std::mutex> lock(uc_static_mutex);
    if (!uc_static_ptr[dev]) {
        void* p = nullptr;
        SSWIN_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(uc_static_scratch)));
        SSWIN_CHECK(p, "unique_consecutive_indices_static: the scratch array has no device address");
        uc_static_ptr[dev] = static_cast<int32_t*>(p);
    }
    *out = uc_static_ptr[dev];
    return 0;
}

static_assert(UC_STATIC_MAX_M == SSWIN_UNIQUE_CONSECUTIVE_STATIC_MAX, "header and library disagree on the limit");

int sswin_unique_consecutive_indices_static(const void* keys, int key_dtype, int64_t M, int32_t* out, void* stream) {
    SSWIN_CHECK(M >= 0, "unique_consecutive_indices_static: negative length");
    SSWIN_CHECK(M <= UC_STATIC_MAX_M,
                "unique_consecutive_indices_static: %lld keys exceed the built-in scratch (%lld keys at most); "
                "use sswin_unique_consecutive_indices with a workspace",
                (long long)M, (long long)UC_STATIC_MAX_M);
    if (M == 0) return 0;
    SSWIN_CHECK(keys && out, "unique_consecutive_indices_static: null pointer");
    int32_t* tile_sums = nullptr;
    if (uc_static_address(&tile_sums)) return 1;
    // every tile sum the scan reads is written by the reduce launch of the same call, so nothing
    // has to be cleared between calls
    return unique_consecutive_run(keys, key_dtype, M, out, tile_sums, static_cast<hipStream_t>(stream));
}

// ---- return_inverse ---------------------------------------------------------------------------
static size_t bitmap_words(int64_t nbits) { return (size_t)((nbits + 31) / 32) + 1; }  // +1 padding word

size_t sswin_return_inverse_workspace_bytes(int64_t M, int64_t maxnum_bound) {
    (void)M;
    if (maxnum_bound < 1) maxnum_bound = 1;
    const size_t words = bitmap_words(maxnum_bound);
    return align_up(words * 4, 256) * 2 + align_up((size_t)scan_num_tiles((int64_t)words) * 4, 256) + 1024;
}

int sswin_return_inverse(const int32_t* x, int64_t M, int64_t maxnum, int32_t* out, int64_t* count_out,
                         void* ws, size_t ws_bytes, void* stream) {
    SSWIN_CHECK(M >= 0, "return_inverse: negative length");
    if (M == 0) {
        if (count_out) *count_out = 0;
        return 0;
    }
    SSWIN_CHECK(x && out && ws, "return_inverse: null pointer");
    SSWIN_CHECK(maxnum >= -1, "return_inverse: maxnum %lld invalid", (long long)maxnum);
    SSWIN_CHECK(maxnum != -1 || count_out, "return_inverse: maxnum = -1 needs count_out (synchronous call)");
    hipStream_t s = static_cast<hipStream_t>(stream);
    Carver cv(ws, ws_bytes);
    int32_t* total_dev = cv.take<int32_t>(3);   // [0] distinct count, [1] max, [2] values outside [0, maxnum)
    SSWIN_CHECK(cv.ok(), "return_inverse: workspace too small");
    if (maxnum == -1) {
        int32_t* max_dev = total_dev + 1;
        hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(256), 0, s, reinterpret_cast<uint32_t*>(max_dev),
                           (int64_t)1, (uint32_t)INT32_MIN);
        const unsigned blocks = (unsigned)std::min<int64_t>((M + 255) / 256, 2048);
        hipLaunchKernelGGL(max_i32_kernel, dim3(blocks), dim3(256), 0, s, x, M, max_dev);
        int32_t mx = 0;
        SSWIN_HIP(hipMemcpyAsync(&mx, max_dev, sizeof(int32_t), hipMemcpyDeviceToHost, s));
        SSWIN_HIP(hipStreamSynchronize(s));
        SSWIN_CHECK(mx >= 0, "return_inverse: all values negative");
        maxnum = (int64_t)mx + 1;
    }
    const size_t words = bitmap_words(maxnum);
    uint32_t* bits = cv.take<uint32_t>(words);
    int32_t* word_prefix = cv.take<int32_t>(words);
    int32_t* tile_sums = cv.take<int32_t>((size_t)scan_num_tiles((int64_t)words));
    SSWIN_CHECK(cv.ok(), "return_inverse: workspace too small for maxnum %lld", (long long)maxnum);
    const unsigned fill_blocks = (unsigned)std::min<size_t>((words + 255) / 256, 4096);
    hipLaunchKernelGGL(fill_u32_kernel, dim3(fill_blocks), dim3(256), 0, s, bits, (int64_t)words, 0u);
    hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(256), 0, s, reinterpret_cast<uint32_t*>(total_dev + 2), (int64_t)1, 0u);
    hipLaunchKernelGGL(set_bits_kernel, dim3((unsigned)((M + 255) / 256)), dim3(256), 0, s, x, M, maxnum, bits,
                       total_dev + 2);
    PopcLoad ld{bits};
    ExclusiveStore st{word_prefix};
    if (device_exclusive_scan<int32_t>(ld, st, (int64_t)words, tile_sums, total_dev, s, "return_inverse scan")) return 1;
    hipLaunchKernelGGL(rank_lookup_kernel, dim3((unsigned)((M + 255) / 256)), dim3(256), 0, s, x, M, maxnum, bits,
                       word_prefix, out);
    if (launch_ok("return_inverse")) return 1;
    if (count_out) {
        int32_t back[3] = {0, 0, 0};
        SSWIN_HIP(hipMemcpyAsync(back, total_dev, sizeof(back), hipMemcpyDeviceToHost, s));
        SSWIN_HIP(hipStreamSynchronize(s));
        SSWIN_CHECK(back[2] == 0, "return_inverse: %d values lie outside [0, %lld)", back[2], (long long)maxnum);
        *count_out = back[0];
    }
    return 0;
}

// ---- qkv_sparse_indices -----------------------------------------------------------------------
size_t sswin_qkv_sparse_indices_workspace_bytes(int64_t N, int B, int n) {
    const size_t words = bitmap_words((int64_t)B * n + n);
    return align_up(words * 4, 256) * 2 + align_up((size_t)scan_num_tiles((int64_t)words) * 4, 256) +
           3 * align_up((size_t)(N > 0 ? N : 1) * 4, 256) + 256 + 1024;
}

// ranks of the voxels in (window, pos) order: order / win_T / win_c by rank, status = {pairs out of range,
// distinct pairs}; all carved from `ws`
struct VoxelRanks {
    int32_t *order, *win_T, *win_c, *status;
};
// (`map` != NULL: in a caller's array [3N + 2] instead)
static int build_voxel_ranks(const char* who, const int32_t* indices, int64_t N, int B, int n, void* ws, size_t ws_bytes,
                             int32_t* map, VoxelRanks* out, hipStream_t s) {
    Carver cv(ws, ws_bytes);
    const size_t words = bitmap_words((int64_t)B * n + n);
    uint32_t* bits = cv.take<uint32_t>(words);
    int32_t* word_prefix = cv.take<int32_t>(words);
    int32_t* tile_sums = cv.take<int32_t>((size_t)scan_num_tiles((int64_t)words));
    out->order = map ? map : cv.take<int32_t>((size_t)N);
    out->win_T = map ? map + N : cv.take<int32_t>((size_t)N);
    out->win_c = map ? map + 2 * N : cv.take<int32_t>((size_t)N);
    out->status = map ? map + 3 * N : cv.take<int32_t>(2);
    SSWIN_CHECK(cv.ok(), "%s: workspace too small", who);
    const unsigned fill_blocks = (unsigned)std::min<size_t>((words + 255) / 256, 4096);
    hipLaunchKernelGGL(fill_u32_kernel, dim3(fill_blocks), dim3(256), 0, s, bits, (int64_t)words, 0u);
    hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(256), 0, s, reinterpret_cast<uint32_t*>(out->status), (int64_t)2, 0u);
    const unsigned nb = (unsigned)((N + 255) / 256);
    hipLaunchKernelGGL(set_bits_pairs_kernel, dim3(nb), dim3(256), 0, s, indices, N, B, n, bits, out->status);
    PopcLoad ld{bits};
    ExclusiveStore st{word_prefix};
    if (device_exclusive_scan<int32_t>(ld, st, (int64_t)words, tile_sums, out->status + 1, s, who)) return 1;
    hipLaunchKernelGGL(voxel_rank_kernel, dim3(nb), dim3(256), 0, s, indices, N, B, n, bits, word_prefix, out->status,
                       out->order, out->win_T, out->win_c);
    return 0;
}

static int report_pairs(const char* who, const int32_t* status, int64_t N, int validate, int32_t* status_out, hipStream_t s) {
    if (status_out) {                                        // the caller checks later: {out of range, distinct pairs}
        SSWIN_HIP(hipMemcpyAsync(status_out, status, 2 * sizeof(int32_t), hipMemcpyDeviceToHost, s));
    }
    if (validate) {
        int32_t back[2] = {0, 0};
        SSWIN_HIP(hipMemcpyAsync(back, status, sizeof(back), hipMemcpyDeviceToHost, s));
        SSWIN_HIP(hipStreamSynchronize(s));
        SSWIN_CHECK(back[0] == 0, "%s: %d voxel indices lie outside [0, batch_size) x [0, spatial_dim)", who, back[0]);
        SSWIN_CHECK(back[1] == N, "%s: (window, pos) pairs must be distinct: %lld voxels share a pair with another", who,
                    (long long)(N - back[1]));
    }
    return 0;
}

int sswin_qkv_sparse_indices(const int32_t* indices, int64_t N, int B, int n, int H, int hd,
                             int32_t* idx_qv, int32_t* sorted_qv, int32_t* idx_k, int32_t* sorted_k,
                             void* ws, size_t ws_bytes, int validate, int32_t* status_out, void* stream) {
    SSWIN_CHECK(N >= 0 && B > 0 && n > 0 && H > 0 && hd > 0, "qkv_sparse_indices: bad sizes");
    SSWIN_CHECK(hd % 4 == 0, "qkv_sparse_indices: head dim %d must be a multiple of 4", hd);
    const int64_t E = N * H * hd;
    SSWIN_CHECK(E < (int64_t)INT32_MAX, "qkv_sparse_indices: N*H*hd = %lld does not fit int32", (long long)E);
    SSWIN_CHECK((int64_t)B * n + n < ((int64_t)1 << 36), "qkv_sparse_indices: B*n too large");
    if (N == 0) return 0;
    SSWIN_CHECK(indices && idx_qv && sorted_qv && idx_k && sorted_k && ws, "qkv_sparse_indices: null pointer");
    SSWIN_CHECK(ws_bytes >= sswin_qkv_sparse_indices_workspace_bytes(N, B, n),
                "qkv_sparse_indices: workspace too small");
    hipStream_t s = static_cast<hipStream_t>(stream);
    VoxelRanks vr;
    if (build_voxel_ranks("qkv_sparse_indices", indices, N, B, n, ws, ws_bytes, nullptr, &vr, s)) return 1;
    const unsigned nb = (unsigned)((N + 255) / 256);
    hipLaunchKernelGGL(expand_coo_kernel, dim3((unsigned)((E / 4 + 255) / 256)), dim3(256), 0, s, indices, E, H,
                       hd, idx_qv, idx_k);
    const int64_t qv_threads = N * H * (hd / 4);
    hipLaunchKernelGGL(sorted_qv_kernel, dim3((unsigned)((qv_threads + 255) / 256)), dim3(256), 0, s, vr.order,
                       vr.win_T, vr.win_c, vr.status, N, H, hd, sorted_qv);
    hipLaunchKernelGGL(sorted_k_kernel, dim3(nb, (unsigned)H), dim3(256), 0, s, vr.order, vr.win_T, vr.win_c, vr.status, N, H,
                       hd, sorted_k);
    if (launch_ok("qkv_sparse_indices")) return 1;
    return report_pairs("qkv_sparse_indices", vr.status, N, validate, status_out, s);
}

// ---- sorted operands without the permutations ---------------------------------------------------
size_t sswin_operand_map_workspace_bytes(int64_t N, int B, int n) { return sswin_qkv_sparse_indices_workspace_bytes(N, B, n); }

int sswin_operand_map(const int32_t* indices, int64_t N, int B, int n, int32_t* map, void* ws, size_t ws_bytes,
                      int validate, int32_t* status_out, void* stream) {
    SSWIN_CHECK(N >= 0 && B > 0 && n > 0, "operand_map: bad sizes");
    SSWIN_CHECK((int64_t)B * n + n < ((int64_t)1 << 36), "operand_map: B*n too large");
    if (N == 0) return 0;
    SSWIN_CHECK(indices && map && ws, "operand_map: null pointer");
    SSWIN_CHECK(N < (int64_t)INT32_MAX / 4, "operand_map: too many voxels");
    SSWIN_CHECK(ws_bytes >= sswin_operand_map_workspace_bytes(N, B, n), "operand_map: workspace too small");
    hipStream_t s = static_cast<hipStream_t>(stream);
    VoxelRanks vr;
    if (build_voxel_ranks("operand_map", indices, N, B, n, ws, ws_bytes, map, &vr, s)) return 1;
    if (launch_ok("operand_map")) return 1;
    return report_pairs("operand_map", vr.status, N, validate, status_out, s);
}

static int value_bytes(int dtype) { return dtype == SSWIN_F64 ? 8 : dtype == SSWIN_F32 ? 4 : 2; }

int sswin_operand_copy(int dtype, int layout, int to_operand, void* vox, int64_t vox_stride, int vox_col0, void* val,
                       const int32_t* map, int64_t N, int H, int hd, double scale, void* stream) {
    SSWIN_CHECK(dtype >= SSWIN_F32 && dtype <= SSWIN_F64, "operand_copy: unsupported value dtype %d", dtype);
    SSWIN_CHECK(layout == 0 || layout == 1, "operand_copy: layout must be 0 (Q, V) or 1 (K^T)");
    SSWIN_CHECK(scale == 1.0 || layout == 0, "operand_copy: only the Q/V order takes a scale");
    SSWIN_CHECK(N >= 0 && H > 0 && hd > 0 && vox_col0 >= 0 && vox_stride >= (int64_t)vox_col0 + (int64_t)H * hd,
                "operand_copy: bad sizes");
    if (N == 0) return 0;
    SSWIN_CHECK(vox && val && map, "operand_copy: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int esz = value_bytes(dtype);
    const int32_t *order = map, *win_T = map + N, *win_c = map + 2 * N, *status = map + 3 * N;
    const int64_t row_bytes = vox_stride * esz, col0_bytes = (int64_t)vox_col0 * esz;
    char* v = static_cast<char*>(vox);
    char* o = static_cast<char*>(val);
    if (layout == 0) {
        const int head_bytes = hd * esz;
        const bool wide = head_bytes % 16 == 0 && row_bytes % 16 == 0 && col0_bytes % 16 == 0 && ((uintptr_t)vox % 16) == 0 &&
                          ((uintptr_t)val % 16) == 0;
        if (scale != 1.0) {
            const bool up = to_operand != 0;
            switch (dtype) {
                case SSWIN_F32: launch_qv_scale<float>(wide, order, win_T, win_c, status, N, H, hd, v, row_bytes, col0_bytes, o, up, scale, s); break;
                case SSWIN_F16: launch_qv_scale<__half>(wide, order, win_T, win_c, status, N, H, hd, v, row_bytes, col0_bytes, o, up, scale, s); break;
                case SSWIN_BF16: launch_qv_scale<__hip_bfloat16>(wide, order, win_T, win_c, status, N, H, hd, v, row_bytes, col0_bytes, o, up, scale, s); break;
                default: launch_qv_scale<double>(wide, order, win_T, win_c, status, N, H, hd, v, row_bytes, col0_bytes, o, up, scale, s); break;
            }
            return launch_ok("operand_copy");
        }
        const int pieces = wide ? head_bytes / 16 : hd;
        const int64_t threads = N * H * pieces;
        const dim3 grid((unsigned)((threads + 255) / 256));
        if (wide)
            hipLaunchKernelGGL(qv_order_copy_kernel<int4>, grid, dim3(256), 0, s, order, win_T, win_c, status, N, H, pieces, v,
                               row_bytes, col0_bytes, o, to_operand != 0);
        else if (esz == 8)
            hipLaunchKernelGGL(qv_order_copy_kernel<int64_t>, grid, dim3(256), 0, s, order, win_T, win_c, status, N, H, pieces, v,
                               row_bytes, col0_bytes, o, to_operand != 0);
        else if (esz == 4)
            hipLaunchKernelGGL(qv_order_copy_kernel<int32_t>, grid, dim3(256), 0, s, order, win_T, win_c, status, N, H, pieces, v,
                               row_bytes, col0_bytes, o, to_operand != 0);
        else
            hipLaunchKernelGGL(qv_order_copy_kernel<int16_t>, grid, dim3(256), 0, s, order, win_T, win_c, status, N, H, pieces, v,
                               row_bytes, col0_bytes, o, to_operand != 0);
    } else {
        const bool wide = row_bytes % 16 == 0 && col0_bytes % 16 == 0 && ((uintptr_t)vox % 16) == 0 && (hd * esz) % 16 == 0;
        const dim3 grid64((unsigned)((N + 63) / 64), (unsigned)H);
#define SSWIN_K_LDS(V, HD)                                                                                              \
    hipLaunchKernelGGL((k_order_copy_lds_kernel<V, HD>), grid64, dim3(256), 0, s, order, win_T, win_c, status, N, H, v,   \
                       row_bytes, col0_bytes, o, to_operand != 0)
        if (wide && esz == 4 && hd == 32) {
            SSWIN_K_LDS(int32_t, 32);
            return launch_ok("operand_copy");
        }
        if (wide && esz == 4 && hd == 16) {
            SSWIN_K_LDS(int32_t, 16);
            return launch_ok("operand_copy");
        }
        if (wide && esz == 2 && hd == 32) {
            SSWIN_K_LDS(int16_t, 32);
            return launch_ok("operand_copy");
        }
        if (wide && esz == 2 && hd == 16) {
            SSWIN_K_LDS(int16_t, 16);
            return launch_ok("operand_copy");
        }
#undef SSWIN_K_LDS
        const dim3 grid((unsigned)((N + 255) / 256), (unsigned)H);
        if (esz == 8)
            hipLaunchKernelGGL(k_order_copy_kernel<int64_t>, grid, dim3(256), 0, s, order, win_T, win_c, status, N, H, hd, v,
                               row_bytes, col0_bytes, o, to_operand != 0);
        else if (esz == 4)
            hipLaunchKernelGGL(k_order_copy_kernel<int32_t>, grid, dim3(256), 0, s, order, win_T, win_c, status, N, H, hd, v,
                               row_bytes, col0_bytes, o, to_operand != 0);
        else
            hipLaunchKernelGGL(k_order_copy_kernel<int16_t>, grid, dim3(256), 0, s, order, win_T, win_c, status, N, H, hd, v,
                               row_bytes, col0_bytes, o, to_operand != 0);
    }
    return launch_ok("operand_copy");
}

int sswin_operand_copy_qkv(int dtype, int to_operand, void* vox, int64_t vox_stride, int vox_col0, void* val_q, void* val_k,
                           void* val_v, const int32_t* map, int64_t N, int H, int hd, double q_scale, void* stream) {
    SSWIN_CHECK(dtype >= SSWIN_F32 && dtype <= SSWIN_F64, "operand_copy_qkv: unsupported value dtype %d", dtype);
    SSWIN_CHECK(N >= 0 && H > 0 && hd > 0 && vox_col0 >= 0 && vox_stride >= (int64_t)vox_col0 + 3 * (int64_t)H * hd,
                "operand_copy_qkv: bad sizes");
    if (N == 0) return 0;
    SSWIN_CHECK(vox && val_q && val_k && val_v && map, "operand_copy_qkv: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int esz = value_bytes(dtype);
    const int64_t row_bytes = vox_stride * esz, col0_bytes = (int64_t)vox_col0 * esz;
    const bool wide = dtype != SSWIN_F64 && (hd == 32 || hd == 16) && row_bytes % 16 == 0 && col0_bytes % 16 == 0 &&
                      ((int64_t)H * hd * esz) % 16 == 0 && ((uintptr_t)vox % 16) == 0 && ((uintptr_t)val_q % 16) == 0 &&
                      ((uintptr_t)val_v % 16) == 0;
    if (!wide) {                                             // any other shape: the three copies one by one
        const int D = H * hd;
        if (sswin_operand_copy(dtype, 0, to_operand, vox, vox_stride, vox_col0, val_q, map, N, H, hd, q_scale, stream)) return 1;
        if (sswin_operand_copy(dtype, 1, to_operand, vox, vox_stride, vox_col0 + D, val_k, map, N, H, hd, 1.0, stream)) return 1;
        return sswin_operand_copy(dtype, 0, to_operand, vox, vox_stride, vox_col0 + 2 * D, val_v, map, N, H, hd, 1.0, stream);
    }
    const int32_t *order = map, *win_T = map + N, *win_c = map + 2 * N, *status = map + 3 * N;
    const dim3 grid((unsigned)((N + 63) / 64), (unsigned)H);
#define SSWIN_QKV(T, HD)                                                                                                  \
    hipLaunchKernelGGL((qkv_order_copy_kernel<T, HD>), grid, dim3(256), 0, s, order, win_T, win_c, status, N, H,            \
                       static_cast<char*>(vox), row_bytes, col0_bytes, static_cast<char*>(val_q), static_cast<char*>(val_k), \
                       static_cast<char*>(val_v), to_operand != 0, (float)q_scale)
    if (dtype == SSWIN_F32 && hd == 32) SSWIN_QKV(float, 32);
    else if (dtype == SSWIN_F32) SSWIN_QKV(float, 16);
    else if (dtype == SSWIN_F16 && hd == 32) SSWIN_QKV(__half, 32);
    else if (dtype == SSWIN_F16) SSWIN_QKV(__half, 16);
    else if (hd == 32) SSWIN_QKV(__hip_bfloat16, 32);
    else SSWIN_QKV(__hip_bfloat16, 16);
#undef SSWIN_QKV
    return launch_ok("operand_copy_qkv");
}

int sswin_sorted_coo_indices(const int32_t* indices, const int32_t* map, int64_t N, int H, int hd, int32_t* idx_qv,
                             int32_t* idx_k, void* stream) {
    SSWIN_CHECK(N >= 0 && H > 0 && hd > 0 && hd % 4 == 0, "sorted_coo_indices: bad sizes (head dim a multiple of 4)");
    const int64_t E = N * H * hd;
    SSWIN_CHECK(E < (int64_t)INT32_MAX, "sorted_coo_indices: N*H*hd = %lld does not fit int32", (long long)E);
    if (N == 0) return 0;
    SSWIN_CHECK(indices && map && (idx_qv || idx_k), "sorted_coo_indices: null pointer");
    SSWIN_CHECK((!idx_qv || ((uintptr_t)idx_qv % 16) == 0) && (!idx_k || ((uintptr_t)idx_k % 16) == 0),
                "sorted_coo_indices: index matrices must be 16-byte aligned");
    const int64_t threads = N * H * (hd / 4);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (idx_qv)
        hipLaunchKernelGGL(sorted_coo_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, indices, map, map + N,
                           map + 2 * N, map + 3 * N, N, H, hd, E, idx_qv);
    if (idx_k)
        hipLaunchKernelGGL(sorted_coo_k_kernel, dim3((unsigned)((N + 255) / 256), (unsigned)H), dim3(256), 0, s, indices, map,
                           map + N, map + 2 * N, map + 3 * N, N, H, hd, E, idx_k);
    return launch_ok("sorted_coo_indices");
}

}  // extern "C"
