// Device-wide exclusive scan of integer items produced by a functor, in three launches:
//   1. tile_reduce:    one block per tile of SCAN_TILE items -> tile_sums[tile]
//   2. scan_tile_sums: a single block scans tile_sums in place (exclusive), writes the total
//   3. tile_scan:      one block per tile recomputes its items and hands every item its
//                      exclusive prefix through a store functor
// Reduce-then-scan is used instead of a single-pass chained scan on purpose: no block ever
// waits on another block, so forward progress never depends on the hardware scheduler.
//
// The value type V is int32_t, or int64_t when two 31-bit sums are scanned at once packed as
// (high << 32) | low.
#pragma once

#include "sswin_common.hpp"

namespace sswin {

constexpr int SCAN_THREADS = 256;
constexpr int SCAN_ITEMS = 8;
constexpr int SCAN_TILE = SCAN_THREADS * SCAN_ITEMS;

inline int64_t scan_num_tiles(int64_t n) { return (n + SCAN_TILE - 1) / SCAN_TILE; }

template <typename V>
__device__ __forceinline__ V wave_inclusive_scan(V v) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        V t = __shfl_up(v, d, 64);
        if (lane >= d) v += t;
    }
    return v;
}

// Exclusive scan over a block of NWAVES*64 threads; `lds` holds NWAVES values.
// Contains two __syncthreads(), so every thread of the block must call it.
template <typename V, int NWAVES>
__device__ __forceinline__ V block_exclusive_scan(V v, V* lds, V* total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    V inc = wave_inclusive_scan<V>(v);
    if (lane == 63) lds[wave] = inc;
    __syncthreads();
    V base = 0, sum = 0;
#pragma unroll
    for (int w = 0; w < NWAVES; ++w) {
        V t = lds[w];
        if (w < wave) base += t;
        sum += t;
    }
    __syncthreads();
    *total = sum;
    return base + inc - v;
}

template <typename V, class Load>
__global__ __launch_bounds__(SCAN_THREADS) void tile_reduce_kernel(Load load, int64_t n,
                                                                  V* __restrict__ tile_sums) {
    __shared__ V lds[SCAN_THREADS / 64];
    const int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
    V s = 0;
#pragma unroll
    for (int j = 0; j < SCAN_ITEMS; ++j) {
        int64_t i = base + j;
        if (i < n) s += load(i);
    }
    V total;
    (void)block_exclusive_scan<V, SCAN_THREADS / 64>(s, lds, &total);
    if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// Single block of 1024 threads; exclusive scan in place; total_out[0] = grand total.
template <typename V>
__global__ __launch_bounds__(1024) void scan_tile_sums_kernel(V* __restrict__ sums, int64_t ntiles,
                                                              V* __restrict__ total_out) {
    __shared__ V lds[16];
    __shared__ V carry_s;
    if (threadIdx.x == 0) carry_s = 0;
    __syncthreads();
    for (int64_t start = 0; start < ntiles; start += 1024) {
        int64_t i = start + threadIdx.x;
        V v = (i < ntiles) ? sums[i] : (V)0;
        V total;
        V ex = block_exclusive_scan<V, 16>(v, lds, &total);
        V carry = carry_s;
        if (i < ntiles) sums[i] = carry + ex;
        __syncthreads();
        if (threadIdx.x == 0) carry_s = carry + total;
        __syncthreads();
    }
    if (threadIdx.x == 0 && total_out) total_out[0] = carry_s;
}

template <typename V, class Load, class Store>
__global__ __launch_bounds__(SCAN_THREADS) void tile_scan_kernel(Load load, Store store, int64_t n,
                                                                const V* __restrict__ tile_offs) {
    __shared__ V lds[SCAN_THREADS / 64];
    const int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
    V item[SCAN_ITEMS];
    V s = 0;
#pragma unroll
    for (int j = 0; j < SCAN_ITEMS; ++j) {
        int64_t i = base + j;
        item[j] = (i < n) ? load(i) : (V)0;
        s += item[j];
    }
    V total;
    V ex = block_exclusive_scan<V, SCAN_THREADS / 64>(s, lds, &total) + tile_offs[blockIdx.x];
#pragma unroll
    for (int j = 0; j < SCAN_ITEMS; ++j) {
        int64_t i = base + j;
        if (i < n) store(i, ex, item[j]);
        ex += item[j];
    }
}

// Host driver.  tile_sums: device V [scan_num_tiles(n)]; total_dev: device V* or null.
template <typename V, class Load, class Store>
int device_exclusive_scan(Load load, Store store, int64_t n, V* tile_sums, V* total_dev,
                          hipStream_t stream, const char* what) {
    if (n <= 0) return 0;
    const int64_t tiles = scan_num_tiles(n);
    hipLaunchKernelGGL((tile_reduce_kernel<V, Load>), dim3((unsigned)tiles), dim3(SCAN_THREADS), 0, stream,
                       load, n, tile_sums);
    hipLaunchKernelGGL((scan_tile_sums_kernel<V>), dim3(1), dim3(1024), 0, stream, tile_sums, tiles,
                       total_dev);
    hipLaunchKernelGGL((tile_scan_kernel<V, Load, Store>), dim3((unsigned)tiles), dim3(SCAN_THREADS), 0,
                       stream, load, store, n, tile_sums);
    return launch_ok(what);
}

}  // namespace sswin
