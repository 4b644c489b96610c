// Per-group offsets of the window-blocked products ("plan").
//
// A coalesced 4-D COO operand [B, H, n, inner] with a dense last dimension is a sequence of
// token rows (one per `inner` consecutive columns), sorted by (window, head, pos).  A group is
// a run of token rows with equal (window, head).  One packed scan yields, per group, its index
// and the exclusive sum of c*c; the head row of a group is its exclusive sum of c.
#include "scan.hpp"
#include "sswin_common.hpp"

namespace sswin {

struct RowKeys {
    const int32_t* i0;   // idx row 0 (window)
    const int32_t* i1;   // idx row 1 (head)
    int64_t R;           // token rows
    int inner;
    __device__ bool same(int64_t a, int64_t b) const {
        return i0[a * inner] == i0[b * inner] && i1[a * inner] == i1[b * inner];
    }
    __device__ bool is_head(int64_t r) const { return r == 0 || !same(r, r - 1); }
    // number of token rows of the group starting at r (rows are sorted, so the group is the
    // maximal run of rows equal to r): gallop, then bisect.
    __device__ int64_t run_length(int64_t r) const {
        int64_t lo = r, step = 1;            // lo: last row known equal
        int64_t hi = R;                      // hi: first row known different (or R)
        while (true) {
            int64_t p = lo + step;
            if (p >= R) break;
            if (same(r, p)) { lo = p; step <<= 1; } else { hi = p; break; }
        }
        while (hi - lo > 1) {
            int64_t mid = lo + (hi - lo) / 2;
            if (same(r, mid)) lo = mid; else hi = mid;
        }
        return hi - r;
    }
};

// item = 1 | c*c << 32 at group heads, else 0
struct PlanLoad {
    RowKeys k;
    __device__ int64_t operator()(int64_t r) const {
        if (!k.is_head(r)) return 0;
        const int64_t c = k.run_length(r);
        return (int64_t)1 | ((c * c) << 32);
    }
};

struct PlanStore {
    RowKeys k;
    int32_t* plan;
    int64_t g_cap;
    int32_t* cmax;
    __device__ void operator()(int64_t r, int64_t ex, int64_t item) const {
        if (item == 0) return;
        const int64_t g = ex & 0xffffffffll;
        if (g >= g_cap) return;
        // c*c is a perfect square below 2^31: the double square root is exact
        const int c = (int)(sqrt((double)(item >> 32)) + 0.5);
        plan[g] = c;
        plan[g_cap + g] = (int32_t)r;
        plan[2 * g_cap + g] = (int32_t)(ex >> 32);
        plan[3 * g_cap + g] = k.i0[r * k.inner];
        plan[4 * g_cap + g] = k.i1[r * k.inner];
        if (c > *cmax) atomicMax(cmax, c);
    }
};

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

}  // namespace sswin

using namespace sswin;

extern "C" {

size_t sswin_plan_workspace_bytes(int64_t M, int inner) {
    const int64_t R = inner > 0 ? M / inner : 0;
    return align_up((size_t)scan_num_tiles(R > 0 ? R : 1) * sizeof(int64_t), 256) + 1024;
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
    Carver cv(ws, ws_bytes);
    int64_t* total_dev = cv.take<int64_t>(2);           // [0] packed total, [1] low word: c_max
    int64_t* tile_sums = cv.take<int64_t>((size_t)scan_num_tiles(R));
    SSWIN_CHECK(cv.ok(), "plan: workspace too small");
    int32_t* cmax = reinterpret_cast<int32_t*>(total_dev + 1);
    hipLaunchKernelGGL(zero_i32_kernel, dim3(1), dim3(64), 0, s, cmax, 2);
    RowKeys k{idx, idx + M, R, inner};
    PlanLoad ld{k};
    PlanStore st{k, plan, g_cap, cmax};
    if (device_exclusive_scan<int64_t>(ld, st, R, tile_sums, total_dev, s, "plan scan")) return 1;
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
