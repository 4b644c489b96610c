// Per-group offsets of the window-blocked products ("plan").
//
// A coalesced 4-D COO operand [B, H, n, inner] with a dense last dimension is a sequence of
// token rows (one per `inner` consecutive columns), sorted by (window, head, pos).  A group is
// a run of token rows with equal (window, head).
//
// plan_tile_kernel works on tiles of PLAN_TILE token rows: the (window, head) keys of the tile
// are staged in LDS, run heads are found with wave ballots and compacted into a start table,
// and the token count of a group is the distance to the next head (one look-ahead past the
// tile end for the last head of the tile).  Pass 1 reduces (number of heads, sum of c*c) per
// tile, a single block scans the tile sums, pass 2 repeats the tile work and writes the plan.
#include "scan.hpp"
#include "sswin_common.hpp"

namespace sswin {

constexpr int PLAN_THREADS = 256;
constexpr int PLAN_TILE = 2048;
constexpr int PLAN_ROUNDS = PLAN_TILE / PLAN_THREADS;

template <bool WRITE>
__global__ __launch_bounds__(PLAN_THREADS) void plan_tile_kernel(const int32_t* __restrict__ i0,
                                                                const int32_t* __restrict__ i1, int64_t R,
                                                                int inner, int64_t* __restrict__ tile_sums,
                                                                int32_t* __restrict__ plan, int64_t g_cap,
                                                                int32_t* __restrict__ cmax_out) {
    __shared__ int kw[PLAN_TILE + 1], kh[PLAN_TILE + 1];     // slot e + 1 = key of tile row e; slot 0 = predecessor
    __shared__ int start_s[PLAN_TILE + 1];
    __shared__ int wave_cnt_s[PLAN_THREADS / 64];
    __shared__ long long scan_lds[PLAN_THREADS / 64];
    __shared__ int next_head_s;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t tile_base = (int64_t)blockIdx.x * PLAN_TILE;
    const int tile_n = (int)((R - tile_base) < PLAN_TILE ? (R - tile_base) : PLAN_TILE);

#pragma unroll
    for (int j = 0; j < PLAN_ROUNDS; ++j) {
        const int e = j * PLAN_THREADS + tid;
        if (e < tile_n) {
            const int64_t col = (tile_base + e) * inner;
            kw[e + 1] = i0[col];
            kh[e + 1] = i1[col];
        }
    }
    if (tid == 0) {
        if (tile_base > 0) {
            kw[0] = i0[(tile_base - 1) * inner];
            kh[0] = i1[(tile_base - 1) * inner];
        } else {
            kw[0] = ~i0[0];                                  // anything different from row 0
            kh[0] = 0;
        }
    }
    __syncthreads();

    // heads, compacted in row order
    int rnk[PLAN_ROUNDS];
    int wave_count = 0;
#pragma unroll
    for (int j = 0; j < PLAN_ROUNDS; ++j) {
        const int e = wave * (PLAN_TILE / 4) + j * 64 + lane;
        const bool flag = e < tile_n && (kw[e + 1] != kw[e] || kh[e + 1] != kh[e]);
        const unsigned long long mask = __ballot(flag);
        rnk[j] = flag ? wave_count + __popcll(mask & ((1ull << lane) - 1ull)) : -1;
        wave_count += __popcll(mask);
    }
    if (lane == 0) wave_cnt_s[wave] = wave_count;
    __syncthreads();
    int wave_base = 0, nheads = 0;
#pragma unroll
    for (int w = 0; w < PLAN_THREADS / 64; ++w) {
        const int t = wave_cnt_s[w];
        if (w < wave) wave_base += t;
        nheads += t;
    }
#pragma unroll
    for (int j = 0; j < PLAN_ROUNDS; ++j)
        if (rnk[j] >= 0) start_s[wave_base + rnk[j]] = wave * (PLAN_TILE / 4) + j * 64 + lane;

    // first head after the tile: first row whose key differs from the tile's last key
    if (wave == 0 && nheads > 0) {
        const int lw = kw[tile_n], lh = kh[tile_n];
        int64_t p = tile_base + tile_n;
        int64_t found = R;
        while (p < R) {
            const int64_t r = p + lane;
            bool differs = false;
            if (r < R) {
                const int64_t col = r * inner;
                differs = i0[col] != lw || i1[col] != lh;
            }
            const unsigned long long mask = __ballot(differs);
            if (mask) {
                found = p + (__ffsll((long long)mask) - 1);
                break;
            }
            p += 64;
        }
        if (lane == 0) next_head_s = (int)(found - tile_base);
    }
    __syncthreads();
    if (tid == 0 && nheads > 0) start_s[nheads] = next_head_s;
    __syncthreads();

    // per-thread heads k = tid * PLAN_ROUNDS .. (blocked, so that a block scan gives prefixes in order)
    long long sq_local = 0;
    int cvals[PLAN_ROUNDS];
    int cmx = 0;
#pragma unroll
    for (int j = 0; j < PLAN_ROUNDS; ++j) {
        const int k = tid * PLAN_ROUNDS + j;
        int c = 0;
        if (k < nheads) c = start_s[k + 1] - start_s[k];
        cvals[j] = c;
        sq_local += (long long)c * c;
        cmx = c > cmx ? c : cmx;
    }
    long long sq_total;
    long long sq_prefix = block_exclusive_scan<long long, PLAN_THREADS / 64>(sq_local, scan_lds, &sq_total);
    if (!WRITE) {
        if (tid == 0) tile_sums[blockIdx.x] = (long long)nheads | (sq_total << 32);
        return;
    }
    const long long off = tile_sums[blockIdx.x];             // exclusive prefix over tiles (packed)
    const int64_t g_base = off & 0xffffffffll;
    long long sq = (off >> 32) + sq_prefix;
#pragma unroll
    for (int j = 0; j < PLAN_ROUNDS; ++j) {
        const int k = tid * PLAN_ROUNDS + j;
        if (k < nheads) {
            const int64_t g = g_base + k;
            if (g < g_cap) {
                const int e = start_s[k];
                plan[g] = cvals[j];
                plan[g_cap + g] = (int32_t)(tile_base + e);
                plan[2 * g_cap + g] = (int32_t)sq;
                plan[3 * g_cap + g] = kw[e + 1];
                plan[4 * g_cap + g] = kh[e + 1];
            }
            sq += (long long)cvals[j] * cvals[j];
        }
    }
    cmx = wave_max_i32(cmx);
    if (lane == 0 && cmx > 0) atomicMax(cmax_out, cmx);
}

__global__ void zero_i32_kernel(int32_t* p, int n) {
    if ((int)threadIdx.x < n) p[threadIdx.x] = 0;
}

// scans of a given c[]: item = c | c*c << 32
struct CountLoad {
    const int32_t* c;
    __device__ int64_t operator()(int64_t g) const {
        const int64_t v = c[g];
        return v | ((v * v) << 32);
    }
};
struct CountStore {
    int32_t* scans;
    int64_t G;
    __device__ void operator()(int64_t g, int64_t ex, int64_t) const {
        scans[g] = (int32_t)(ex & 0xffffffffll);
        scans[G + g] = (int32_t)(ex >> 32);
    }
};

// ------------------------------------------------------------------------------------------
// Order of a coalesced [B, H, n, C] operand (dense last dimension) after permute (0, 2, 1, 3).
// The reference re-hashes the permuted indices and sorts all of them (sparse_swin/swin3d_base.py:47-59).
// When every head of a window holds the same positions - what an attention output does - the
// sorted order follows from the plan: row i of head number r of a window that starts at row R0
// and has Hw heads of c rows each goes to row R0 + i*Hw + r.  One wavefront per group writes its
// rows' entries and checks the premise (equal counts, equal positions as the window's first head);
// a group that fails it is counted in *bad and writes nothing.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void permute_heads_kernel(const int32_t* __restrict__ pos_row, const int32_t* __restrict__ plan,
                                                            int64_t g_cap, int64_t G, int C, int32_t* __restrict__ perm,
                                                            int32_t* __restrict__ bad) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t g = (int64_t)blockIdx.x * 4 + wave;
    if (g >= G) return;
    const int32_t* win = plan + 3 * g_cap;
    const int c = plan[g], rs = plan[g_cap + g], w = win[g];
    int64_t g0 = g, g1 = g;                                   // the window's groups are g0 .. g1
    while (g0 > 0 && win[g0 - 1] == w) --g0;
    while (g1 + 1 < G && win[g1 + 1] == w) ++g1;
    const int heads = (int)(g1 - g0 + 1), r = (int)(g - g0);
    const int rs0 = plan[g_cap + g0];
    bool ok = plan[g0] == c && rs == rs0 + r * c;
    // the tensor must be coalesced for the derived order to be the sorted one: (window, head) keys ascend from group
    // to group and positions ascend inside a group (a tensor that is not goes through the sort, as in the reference)
    if (g > 0) {
        const int32_t* head = plan + 4 * g_cap;
        ok = ok && (win[g - 1] < w || (win[g - 1] == w && head[g - 1] < head[g]));
    }
    if (ok)
        for (int i = lane; i < c; i += 64) {
            const int p = pos_row[(int64_t)(rs + i) * C];
            if (r > 0) ok = ok && p == pos_row[(int64_t)(rs0 + i) * C];
            if (i > 0) ok = ok && p > pos_row[(int64_t)(rs + i - 1) * C];
        }
    if (!__all(ok)) {
        if (lane == 0) atomicAdd(bad, 1);
        return;
    }
    const int q = C >> 2;                                     // 16-byte pieces per row
    for (int t = lane; t < c * q; t += 64) {
        const int i = t / q, cq = t - i * q;
        const int src = (rs + i) * C + 4 * cq;
        const int64_t dst = (int64_t)(rs0 + i * heads + r) * C + 4 * cq;
        *reinterpret_cast<int4*>(perm + dst) = make_int4(src, src + 1, src + 2, src + 3);
    }
}

// ------------------------------------------------------------------------------------------
// Row ids of a [B, H, n, n] product in sorted COO order: entry sq_start[g] + i*c + j belongs to attention row
// row_start[g] + i.  The reference hashes the first three index rows and runs unique_consecutive over the
// hash (sparse_swin/swin3d_base.py:140-150); every attention row of every group is non-empty, so the
// running id is the row number.  One wavefront per group.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void rows_from_counts_kernel(const int32_t* __restrict__ cs, const int32_t* __restrict__ row_start,
                                                               const int32_t* __restrict__ sq_start, int64_t G,
                                                               int32_t* __restrict__ rows) {
    const int64_t g = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (g >= G) return;
    const int lane = threadIdx.x & 63;
    const int c = cs[g], rs = row_start[g];
    int32_t* out = rows + sq_start[g];
    const int count = c * c;
    const float inv = 1.0f / (float)c;
    // gridDim.y wavefronts share a group's entries: one wavefront alone would write the 51 529 entries of a
    // 227-token window in 805 rounds
    for (int f = lane + 64 * (int)blockIdx.y; f < count; f += 64 * (int)gridDim.y) {
        int i = (int)((float)f * inv);                        // f / c up to one, corrected below (f < 2^24)
        i -= i * c > f ? 1 : 0;
        i += (i + 1) * c <= f ? 1 : 0;
        out[f] = rs + i;
    }
}

// position (third index row) of every attention row of a [B, H, n, n] product: out[row_start[g] + i] = the index at
// the first entry of row i of group g
__global__ __launch_bounds__(256) void group_row_positions_kernel(const int32_t* __restrict__ idx_pi, const int32_t* __restrict__ cs,
                                                                  const int32_t* __restrict__ row_start,
                                                                  const int32_t* __restrict__ sq_start, int64_t G,
                                                                  int32_t* __restrict__ out) {
    const int64_t g = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (g >= G) return;
    const int c = cs[g];
    const int64_t sq = sq_start[g];
    for (int i = threadIdx.x & 63; i < c; i += 64) out[row_start[g] + i] = idx_pi[sq + (int64_t)i * c];
}

}  // namespace sswin

using namespace sswin;

extern "C" {

int sswin_permute_heads_order(const int32_t* idx, int64_t M, int C, const int32_t* plan, int64_t g_cap, int64_t G,
                              int32_t* perm_out, int32_t* bad_groups, void* stream) {
    SSWIN_CHECK(C > 0 && C % 4 == 0 && M >= 0 && M % C == 0, "permute_heads_order: bad sizes");
    SSWIN_CHECK(M < (int64_t)INT32_MAX, "permute_heads_order: too many entries for int32 positions");
    SSWIN_CHECK(G >= 0 && G <= g_cap, "permute_heads_order: bad group count");
    SSWIN_CHECK(bad_groups, "permute_heads_order: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(zero_i32_kernel, dim3(1), dim3(64), 0, s, bad_groups, 1);
    if (G == 0 || M == 0) return launch_ok("permute_heads_order");
    SSWIN_CHECK(idx && plan && perm_out, "permute_heads_order: null pointer");
    SSWIN_CHECK(((uintptr_t)perm_out % 16) == 0, "permute_heads_order: perm_out is not 16-byte aligned");
    hipLaunchKernelGGL(permute_heads_kernel, dim3((unsigned)((G + 3) / 4)), dim3(256), 0, s, idx + 2 * M, plan, g_cap, G, C,
                       perm_out, bad_groups);
    return launch_ok("permute_heads_order");
}

size_t sswin_plan_workspace_bytes(int64_t M, int inner) {
    const int64_t R = inner > 0 ? M / inner : 0;
    const int64_t tiles = (R + PLAN_TILE - 1) / PLAN_TILE;
    return align_up((size_t)(tiles > 0 ? tiles : 1) * sizeof(int64_t), 256) + 1024;
}

int sswin_plan_from_indices(const int32_t* idx, int64_t M, int inner, int32_t* plan, int64_t g_cap,
                            int64_t* totals_out, void* ws, size_t ws_bytes, void* stream) {
    SSWIN_CHECK(inner > 0 && M >= 0 && M % inner == 0,
                "plan: nnz %lld is not a multiple of the dense inner extent %d", (long long)M, inner);
    SSWIN_CHECK(totals_out, "plan: totals_out is null");
    const int64_t R = M / inner;
    totals_out[0] = totals_out[1] = totals_out[2] = totals_out[3] = 0;
    if (R == 0) return 0;
    SSWIN_CHECK(idx && plan && ws, "plan: null pointer");
    SSWIN_CHECK(g_cap > 0, "plan: g_cap must be positive");
    SSWIN_CHECK(ws_bytes >= sswin_plan_workspace_bytes(M, inner), "plan: workspace too small");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t tiles = (R + PLAN_TILE - 1) / PLAN_TILE;
    Carver cv(ws, ws_bytes);
    int64_t* total_dev = cv.take<int64_t>(2);           // [0] packed total, [1] low word: c_max
    int64_t* tile_sums = cv.take<int64_t>((size_t)tiles);
    SSWIN_CHECK(cv.ok(), "plan: workspace too small");
    int32_t* cmax = reinterpret_cast<int32_t*>(total_dev + 1);
    hipLaunchKernelGGL(zero_i32_kernel, dim3(1), dim3(64), 0, s, cmax, 2);
    hipLaunchKernelGGL(plan_tile_kernel<false>, dim3((unsigned)tiles), dim3(PLAN_THREADS), 0, s, idx, idx + M, R,
                       inner, tile_sums, plan, g_cap, cmax);
    hipLaunchKernelGGL((scan_tile_sums_kernel<int64_t>), dim3(1), dim3(1024), 0, s, tile_sums, tiles, total_dev);
    hipLaunchKernelGGL(plan_tile_kernel<true>, dim3((unsigned)tiles), dim3(PLAN_THREADS), 0, s, idx, idx + M, R,
                       inner, tile_sums, plan, g_cap, cmax);
    if (launch_ok("plan")) return 1;
    int64_t host[2] = {0, 0};
    SSWIN_HIP(hipMemcpyAsync(host, total_dev, sizeof(host), hipMemcpyDeviceToHost, s));
    SSWIN_HIP(hipStreamSynchronize(s));
    SSWIN_CHECK(host[0] >= 0, "plan: the product has 2^31 or more non-zeros, which int32 offsets cannot address");
    const int64_t G = host[0] & 0xffffffffll;
    totals_out[0] = G;
    totals_out[1] = R;
    totals_out[2] = host[0] >> 32;
    totals_out[3] = (int32_t)(host[1] & 0xffffffffll);
    SSWIN_CHECK(G <= g_cap, "plan: %lld groups exceed the plan capacity %lld", (long long)G, (long long)g_cap);
    return 0;
}

int sswin_softmax_rows_from_counts(const int32_t* c, const int32_t* scans, int64_t G, int64_t A, int32_t* rows_out,
                                   void* stream) {
    SSWIN_CHECK(G >= 0 && A >= 0, "softmax_rows_from_counts: negative size");
    if (G == 0 || A == 0) return 0;
    SSWIN_CHECK(c && scans && rows_out, "softmax_rows_from_counts: null pointer");
    // wavefronts per group from the mean number of entries of a group: about 256 entries (four rounds) per wavefront
    // measured best (windows of 5^3: 14.9 -> 12.4 us, of 7^3: 45.6 -> 24.2 us; 128 and 512 entries: 14.3 / 13.4 us
    // and 24.5 / 25.0 us)
    const int64_t per = 256;
    const int64_t y = (A / G + per / 2) / per;
    hipLaunchKernelGGL(rows_from_counts_kernel, dim3((unsigned)((G + 3) / 4), (unsigned)(y < 1 ? 1 : (y > 16 ? 16 : y))), dim3(256), 0,
                       static_cast<hipStream_t>(stream), c, scans, scans + G, G, rows_out);
    return launch_ok("softmax_rows_from_counts");
}

int sswin_group_row_positions(const int32_t* idx, int64_t A, const int32_t* plan, int64_t g_cap, int64_t G, int32_t* out,
                              void* stream) {
    SSWIN_CHECK(A >= 0 && G >= 0 && G <= g_cap, "group_row_positions: bad sizes");
    if (G == 0 || A == 0) return 0;
    SSWIN_CHECK(idx && plan && out, "group_row_positions: null pointer");
    hipLaunchKernelGGL(group_row_positions_kernel, dim3((unsigned)((G + 3) / 4)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       idx + 2 * A, plan, plan + g_cap, plan + 2 * g_cap, G, out);
    return launch_ok("group_row_positions");
}

size_t sswin_scan_counts_workspace_bytes(int64_t G) {
    return align_up((size_t)scan_num_tiles(G > 0 ? G : 1) * sizeof(int64_t), 256) + 256;
}

int sswin_scan_counts(const int32_t* c, int64_t G, int32_t* scans, void* ws, size_t ws_bytes, void* stream) {
    SSWIN_CHECK(G >= 0, "scan_counts: negative group count");
    if (G == 0) return 0;
    SSWIN_CHECK(c && scans && ws, "scan_counts: null pointer");
    SSWIN_CHECK(ws_bytes >= sswin_scan_counts_workspace_bytes(G), "scan_counts: workspace too small");
    Carver cv(ws, ws_bytes);
    int64_t* tile_sums = cv.take<int64_t>((size_t)scan_num_tiles(G));
    CountLoad ld{c};
    CountStore st{scans, G};
    return device_exclusive_scan<int64_t>(ld, st, G, tile_sums, (int64_t*)nullptr,
                                          static_cast<hipStream_t>(stream), "scan_counts");
}

}  // extern "C"
