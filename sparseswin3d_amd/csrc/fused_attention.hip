// Fused window-attention path used inside WindowAttentionSparse.
//
// The reference assembles Q, K^T and V as sorted COO copies of the dense qkv tensor
// (sparse_swin/swin3d_base.py:483-498), multiplies them, adds bias and mask with index_select
// passes (:557-581), and un-sorts the result with a permute + return_inverse + index_select
// (:673-675).  Here the MFMA block products read token rows straight from the dense tensors
// through the token order, so none of those copies exist:
//
//   token plan   (window, pos) voxel indices -> token order, per-group table          (sswin_token_plan)
//   tokens -> sq S = (scale*Q) K^T + bias + mask   or   dP = dO V^T                    (fused_sq_kernel)
//   sq -> tokens O = P V, dV = P^T dO, dQ = scale * dS K, dK = scale * dS^T Q        (fused_tok_kernel)
//   bias grad    d_rpb[h, p_i, p_j] += dS                                             (rpb_grad_kernel)
//
// "sq" arrays are fp32 arrays of all [c x c] blocks in group order (group = window, head);
// token tensors are [N, row_stride] arrays addressed as row order[T_k + i], column col0 + h*hd + ch.
// The softmax between the two products is the ordinary sparse row softmax; its row ids are a
// by-product of the first kernel.
#include <type_traits>
#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "mfma_block.hpp"
#include "scan.hpp"
#include "sswin_common.hpp"

#ifndef FUSED_TOK_WAVES
#define FUSED_TOK_WAVES 5
#endif
#ifndef FUSED_SQ_PLAIN_WAVES
#define FUSED_SQ_PLAIN_WAVES 4
#endif

namespace sswin {

constexpr int FUSED_GROUPS_PER_WG = 4;

// ------------------------------------------------------------------------------------------
// token plan
//
// Five phases, no sort:
//   1. clear the presence bitmap (W = ceil(n/32) words per window slot) and the counters
//   2. one atomicOr per voxel (indices outside [0,B) x [0,n) are counted and skipped)
//   3. per block of 256 window slots: sums of (tokens, tokens^2, non-empty windows, windows per
//      tile-count bucket) and the largest window
//   4. per block: prefix of the earlier blocks' sums, scan inside the block; every non-empty
//      window learns the rank T of its first token, its rank k among the non-empty windows, the
//      sum of c*c before it and its rank inside its bucket, and writes its H plan rows and task
//      descriptors (no atomics: one counter per bucket, bumped once per wavefront from eight XCDs,
//      made this phase 13 us instead of 5)
//   5. per voxel: rank = T(window) + number of occupied positions below its own
// Reduce-then-scan (3, 4) instead of a chained scan: no block waits for another block.  One launch
// per phase.  (All five phases in one cooperative launch with grid-wide barriers in between were
// measured: a barrier across the eight XCDs costs about 8 us, write-back and invalidation of the
// per-XCD L2 included, against 3 to 5 us for a launch boundary.)
// ------------------------------------------------------------------------------------------
constexpr int TP_BLOCK = 256;

// counters (int32) behind the two 64-bit totals: five buckets, c_max, indices out of range
constexpr int TPC_CMAX = 5, TPC_RANGE = 6;

struct TokenPlanArgs {
    const int32_t* ind;      // [N, 2] (window, pos)
    int64_t N;
    int B, n, W, H;
    uint32_t* bits;          // [B * W]
    int32_t* win_T;          // [B]
    int64_t* partial_a;      // [4 * blocks]
    int32_t* partial_b;      // [blocks]
    int64_t* totals;         // [8]: windows, sum c | sum c*c << 32, then twelve int32 counters
    int32_t* plan;
    int64_t g_cap;
    int4* tasks;
    int2* recs;              // token records behind the descriptors (or null): [rec_cap][32] {voxel, pos}
    int64_t rec_cap;
    int32_t* win_rec;        // [B] bucket << 28 | rank of the window inside its bucket, -1 without records
    int32_t* tokens;         // [5 * N]
    int blocks;              // ceil(B / window slots per block) of the launch the plan goes into
    int order_only;          // tokens holds its first row only (voxel of rank r)
};

__device__ __forceinline__ int32_t* tp_counters(const TokenPlanArgs& a) { return reinterpret_cast<int32_t*>(a.totals + 2); }

// gtid / gthreads: this thread's index and the number of threads that share the phase
__device__ __forceinline__ void tp_phase_clear(const TokenPlanArgs& a, int64_t gtid, int64_t gthreads) {
    const int64_t words = (int64_t)a.B * a.W;
    for (int64_t i = gtid; i < words; i += gthreads) a.bits[i] = 0u;
    if (gtid < 8) a.totals[gtid] = 0;
}

__device__ __forceinline__ void tp_phase_set_bits(const TokenPlanArgs& a, int64_t gtid, int64_t gthreads) {
    for (int64_t i = gtid; i < a.N; i += gthreads) {
        const int2 wp = *reinterpret_cast<const int2*>(a.ind + 2 * i);
        if ((unsigned)wp.x < (unsigned)a.B && (unsigned)wp.y < (unsigned)a.n)
            atomicOr(&a.bits[(int64_t)wp.x * a.W + (wp.y >> 5)], 1u << (wp.y & 31));
        else
            atomicAdd(&tp_counters(a)[TPC_RANGE], 1);
    }
}

__device__ __forceinline__ int tp_window_count(const uint32_t* bits, int64_t w, int W) {
    int c = 0;
    if (W == 4) {
        const uint4 v = *reinterpret_cast<const uint4*>(bits + w * 4);
        c = __popc(v.x) + __popc(v.y) + __popc(v.z) + __popc(v.w);
    } else {
        for (int k = 0; k < W; ++k) c += __popc(bits[w * W + k]);
    }
    return c;
}

constexpr int TP_SUMS = 4;      // running sums of the plan, two 32-bit fields each

struct TpShared {
    int64_t a[TP_BLOCK / 64];
    int64_t base[TP_SUMS];
    int32_t m[TP_BLOCK / 64];
    int32_t base_m;
};

// What a window slot adds to the four running sums (each an int64 holding two 32-bit fields):
//   sum c, sum c*c
//   windows of one tile, of two tiles
//   windows of three tiles, of four tiles
//   windows of more than four tiles, non-empty windows
__device__ __forceinline__ int tp_bucket(int64_t c) { return c > 0 ? min(((int)c - 1) >> 5, 4) : -1; }
__device__ __forceinline__ void tp_items(int64_t c, int64_t (&item)[TP_SUMS]) {
    const int b = tp_bucket(c);
    item[0] = c | ((c * c) << 32);
    item[1] = b == 0 ? 1 : (b == 1 ? (int64_t)1 << 32 : 0);
    item[2] = b == 2 ? 1 : (b == 3 ? (int64_t)1 << 32 : 0);
    item[3] = (b == 4 ? 1 : 0) | (c > 0 ? (int64_t)1 << 32 : 0);
}
// windows of bucket b counted in the sums s
__device__ __forceinline__ int64_t tp_bucket_count(const int64_t (&s)[TP_SUMS], int b) {
    const int64_t word = s[1 + (b >> 1)];
    return (b & 1) ? word >> 32 : word & 0xffffffffll;
}
__device__ __forceinline__ int tp_block_max(int v, TpShared& sh) {
    const int wm = wave_max_i32(v);
    if ((threadIdx.x & 63) == 0) sh.m[threadIdx.x >> 6] = wm;
    __syncthreads();
    int m = 0;
#pragma unroll
    for (int w = 0; w < TP_BLOCK / 64; ++w) m = max(m, sh.m[w]);
    __syncthreads();
    return m;
}

// A thread of the per-block phases owns ITEMS consecutive window slots, a block TP_BLOCK * ITEMS of them.  Plans
// with millions of window slots, nearly all of them empty (the 2 x 2 x 2 cells of a stride-2 merge), take ITEMS = 4:
// the cost of these phases is the block-wide scans (ten per block), so four slots per thread cut it four times and
// the number of blocks, whose partial sums every later block adds up, with it.  (Measured instead and dropped:
// blocks of 1 024 threads, windows phase 158 us against 35; a single-workgroup scan of the partial sums between
// the two phases, 56 us for 12 288 blocks; eight slots per thread, windows phase 25 us against 22.)
constexpr int TP_ITEMS_WIDE = 4;
constexpr int64_t TP_WIDE_FROM = 1 << 16;     // window slots from which a plan's launches take ITEMS = 4

// block sums: partial_a[TP_SUMS * blk + k] = the sums over the block's window slots, partial_b[blk] = largest c
template <int ITEMS>
__device__ __forceinline__ void tp_phase_block_sums(const TokenPlanArgs& a, int blk, TpShared& sh) {
    const int64_t w0 = ((int64_t)blk * TP_BLOCK + threadIdx.x) * ITEMS;
    int64_t sum[TP_SUMS] = {0, 0, 0, 0}, total[TP_SUMS];
    int cmax = 0;
#pragma unroll
    for (int u = 0; u < ITEMS; ++u) {
        const int64_t c = w0 + u < a.B ? tp_window_count(a.bits, w0 + u, a.W) : 0;
        int64_t item[TP_SUMS];
        tp_items(c, item);
#pragma unroll
        for (int k = 0; k < TP_SUMS; ++k) sum[k] += item[k];
        cmax = max(cmax, (int)c);
    }
#pragma unroll
    for (int k = 0; k < TP_SUMS; ++k) (void)block_exclusive_scan<int64_t, TP_BLOCK / 64>(sum[k], sh.a, &total[k]);
    const int cm = tp_block_max(cmax, sh);
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < TP_SUMS; ++k) a.partial_a[TP_SUMS * blk + k] = total[k];
        a.partial_b[blk] = cm;
    }
}

// Groups are bucketed by their number of 32-token tiles (bucket b: 32*b < c <= 32*(b+1), b = 0..3;
// counters[4] counts larger groups, which get no descriptor).  Descriptor = {T, c | head << 8,
// window, sq_start}.  A window's slot inside its bucket is its rank among the bucket's windows in
// window order (prefix of the earlier blocks' counts + scan inside the block): no atomics, and the same
// descriptor order on every run.
template <int ITEMS>
__device__ __forceinline__ void tp_phase_windows(const TokenPlanArgs& a, int blk, TpShared& sh) {
    const int H = a.H;
    const int64_t g_cap = a.g_cap;
    int32_t* counters = tp_counters(a);
    // this thread's bitmap words are requested first: the loads overlap the prefix below
    const int64_t w0 = ((int64_t)blk * TP_BLOCK + threadIdx.x) * ITEMS;
    int64_t c[ITEMS];
    int cmax = 0;
#pragma unroll
    for (int u = 0; u < ITEMS; ++u) {
        c[u] = w0 + u < a.B ? tp_window_count(a.bits, w0 + u, a.W) : 0;
        cmax = max(cmax, (int)c[u]);
    }
    // prefix of the earlier blocks
    int64_t p[TP_SUMS] = {0, 0, 0, 0};
    int pm = 0;
    for (int64_t i = threadIdx.x; i < blk; i += TP_BLOCK) {
#pragma unroll
        for (int k = 0; k < TP_SUMS; ++k) p[k] += a.partial_a[TP_SUMS * i + k];
        pm = max(pm, a.partial_b[i]);
    }
    int64_t total[TP_SUMS];
#pragma unroll
    for (int k = 0; k < TP_SUMS; ++k) (void)block_exclusive_scan<int64_t, TP_BLOCK / 64>(p[k], sh.a, &total[k]);
    const int bm = tp_block_max(max(pm, cmax), sh);              // largest c up to and including this block
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < TP_SUMS; ++k) sh.base[k] = total[k];
    }
    __syncthreads();
    // running sums in front of this thread's first slot: scan of the threads' sums, then slot by slot
    int64_t sum[TP_SUMS] = {0, 0, 0, 0}, e[TP_SUMS];
#pragma unroll
    for (int u = 0; u < ITEMS; ++u) {
        int64_t item[TP_SUMS];
        tp_items(c[u], item);
#pragma unroll
        for (int k = 0; k < TP_SUMS; ++k) sum[k] += item[k];
    }
#pragma unroll
    for (int k = 0; k < TP_SUMS; ++k)
        e[k] = block_exclusive_scan<int64_t, TP_BLOCK / 64>(sum[k], sh.a, &total[k]) + sh.base[k];
    if (blk == a.blocks - 1 && threadIdx.x == 0) {
        int64_t all[TP_SUMS];
#pragma unroll
        for (int q = 0; q < TP_SUMS; ++q) all[q] = sh.base[q] + total[q];
        a.totals[0] = all[3] >> 32;                              // non-empty windows
        a.totals[1] = all[0];                                    // sum c | sum c*c << 32
#pragma unroll
        for (int b = 0; b < 5; ++b) counters[b] = (int32_t)(tp_bucket_count(all, b) * H);
        counters[TPC_CMAX] = bm;
    }
#pragma unroll
    for (int u = 0; u < ITEMS; ++u) {
        const int64_t w = w0 + u, cu = c[u];
        const int32_t k = (int32_t)(e[3] >> 32);                 // non-empty windows before this one
        const int32_t T = (int32_t)(e[0] & 0xffffffffll);
        const int64_t q2 = e[0] >> 32;
        if (w < a.B) a.win_T[w] = T;

        const bool live = cu > 0 && ((int64_t)k + 1) * H <= g_cap;
        if (live) {
            for (int h = 0; h < H; ++h) {
                const int64_t g = (int64_t)k * H + h;
                a.plan[g] = (int32_t)cu;
                a.plan[g_cap + g] = T;
                a.plan[2 * g_cap + g] = (int32_t)(q2 * H + (int64_t)h * cu * cu);
                a.plan[3 * g_cap + g] = (int32_t)w;
                a.plan[4 * g_cap + g] = h;
            }
        }
        const int b = tp_bucket(cu);
        int32_t wrec = -1;
        if (a.tasks != nullptr && live && b < 4) {
            const int64_t slot = tp_bucket_count(e, b) * H;
            if (slot + H <= g_cap) {
                for (int h = 0; h < H; ++h)
                    a.tasks[(int64_t)b * g_cap + slot + h] =
                        make_int4(T, (int)cu | (h << 8), (int)w, (int32_t)(q2 * H + (int64_t)h * cu * cu));
                wrec = (int32_t)((b << 28) | (int32_t)tp_bucket_count(e, b));
            }
        }
        if (a.recs != nullptr && w < a.B) a.win_rec[w] = wrec;
        if (ITEMS > 1) {                                         // on to the thread's next slot
            int64_t item[TP_SUMS];
            tp_items(cu, item);
#pragma unroll
            for (int q = 0; q < TP_SUMS; ++q) e[q] += item[q];
        }
    }
}

// per voxel -> entries by token rank: source voxel, first rank and size of its window, pos, window
__device__ __forceinline__ void tp_phase_rank(const TokenPlanArgs& a, int64_t gtid, int64_t gthreads) {
    const int W = a.W;
    const int64_t N = a.N;
    int32_t* order = a.tokens;
    int32_t* tok_T = a.tokens + N;
    int32_t* tok_c = a.tokens + 2 * N;
    int32_t* tok_pos = a.tokens + 3 * N;
    int32_t* tok_win = a.tokens + 4 * N;
    for (int64_t v = gtid; v < N; v += gthreads) {
        const int2 wp = *reinterpret_cast<const int2*>(a.ind + 2 * v);
        if ((unsigned)wp.x >= (unsigned)a.B || (unsigned)wp.y >= (unsigned)a.n) continue;   // counted in phase 2
        const int T = a.win_T[wp.x];
        const int word = wp.y >> 5;
        const uint32_t below_mask = (1u << (wp.y & 31)) - 1u;
        int below = 0, c = 0;
        if (W == 4) {
            const uint4 q = *reinterpret_cast<const uint4*>(a.bits + (int64_t)wp.x * 4);
            const uint32_t b[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int pc = __popc(b[k]);
                c += pc;
                below += k < word ? pc : (k == word ? __popc(b[k] & below_mask) : 0);
            }
        } else {
            for (int k = 0; k < W; ++k) {
                const uint32_t x = a.bits[(int64_t)wp.x * W + k];
                const int pc = __popc(x);
                c += pc;
                below += k < word ? pc : (k == word ? __popc(x & below_mask) : 0);
            }
        }
        const int r = T + below;
        if (r < N) {                                            // duplicates cannot push a rank past the end, but stay inside anyway
            order[r] = (int32_t)v;
            if (a.order_only) continue;
            tok_T[r] = T;
            tok_c[r] = c;
            tok_pos[r] = wp.y;
            tok_win[r] = wp.x;
        }
        if (a.recs != nullptr) {
            // Token records of the window-resident kernels: one record of 32 {voxel, pos} entries per (window, tile
            // of 32 tokens), at the position of the tile's task inside its bucket, so that a task finds its tokens
            // from its own number, in the same round trip as its group descriptor.  The entries behind the last
            // token of a window repeat that token (what the kernels feed their padding rows with).
            const int32_t wr = a.win_rec[wp.x];
            if (wr >= 0) {
                const int b = wr >> 28, nt = b + 1;
                const int32_t* counters = tp_counters(a);
                int64_t first = 0;                               // records of the buckets of more tiles come first
                for (int bb = 3; bb > b; --bb) first += (int64_t)(counters[bb] / a.H) * (bb + 1);
                const int64_t rec = first + (int64_t)(wr & 0x0fffffff) * nt + (below >> 5);
                if (rec < a.rec_cap && below < c) {
                    const int2 entry = make_int2((int)v, wp.y);
                    a.recs[rec * 32 + (below & 31)] = entry;
                    if (below == c - 1)
                        for (int k = (below & 31) + 1; k < 32; ++k) a.recs[rec * 32 + k] = entry;
                }
            }
        }
    }
}

// ---- the five launches ----
// Each launch works on up to TP_MAX_BATCH independent plans at once (blockIdx.y picks the plan): the phases of
// one plan are a few microseconds each and mostly launch boundary, so the plans of the blocks of a stage share
// their launches.  The grid's x extent is the largest any plan of the batch needs; the per-voxel and per-word
// phases walk their plan with a grid stride, the per-block phases leave when the plan has fewer blocks.
constexpr int TP_MAX_BATCH = 4;
struct TokenPlanBatch {
    TokenPlanArgs p[TP_MAX_BATCH];
};

__global__ __launch_bounds__(256) void tp_clear_kernel(TokenPlanBatch b) {
    tp_phase_clear(b.p[blockIdx.y], (int64_t)blockIdx.x * 256 + threadIdx.x, (int64_t)gridDim.x * 256);
}
__global__ __launch_bounds__(256) void tp_set_bits_kernel(TokenPlanBatch b) {
    tp_phase_set_bits(b.p[blockIdx.y], (int64_t)blockIdx.x * 256 + threadIdx.x, (int64_t)gridDim.x * 256);
}
template <int ITEMS>
__global__ __launch_bounds__(TP_BLOCK) void tp_block_sums_kernel(TokenPlanBatch b) {
    __shared__ TpShared sh;
    const TokenPlanArgs& a = b.p[blockIdx.y];
    if ((int)blockIdx.x < a.blocks) tp_phase_block_sums<ITEMS>(a, blockIdx.x, sh);
}
template <int ITEMS>
__global__ __launch_bounds__(TP_BLOCK) void tp_windows_kernel(TokenPlanBatch b) {
    __shared__ TpShared sh;
    const TokenPlanArgs& a = b.p[blockIdx.y];
    if ((int)blockIdx.x < a.blocks) tp_phase_windows<ITEMS>(a, blockIdx.x, sh);
}
__global__ __launch_bounds__(256) void tp_rank_kernel(TokenPlanBatch b) {
    tp_phase_rank(b.p[blockIdx.y], (int64_t)blockIdx.x * 256 + threadIdx.x, (int64_t)gridDim.x * 256);
}

// ------------------------------------------------------------------------------------------
// group table of the fused kernels
// ------------------------------------------------------------------------------------------
struct FusedGroups {
    const int32_t* c;        // tokens of the group's window
    const int32_t* T;        // rank of the window's first token
    const int32_t* sq;       // start of the group's [c x c] block in sq arrays
    const int32_t* window;
    const int32_t* head;
    int64_t G;
};

struct TokenTensor {         // rows addressed by voxel, columns col0 + h*hd + ch
    const void* base;
    int64_t stride;
    int col0;
};

// work distribution: four consecutive groups per workgroup, their 32-row x 32-column blocks dealt
// round robin to the four wavefronts of the gridDim.y workgroups that share them.  Lane q < 4 of every wavefront
// holds the fields of group g0 + q (one load per field for all four groups, and nothing waits for a second round);
// a task reads its group's fields from that lane into scalar registers.
struct GroupLanes {
    int c, T, sq, h, w;
};
template <bool WINDOW>
__device__ __forceinline__ GroupLanes load_groups(const FusedGroups& gt, int64_t g0, int lane) {
    const int64_t g = g0 + (lane & (FUSED_GROUPS_PER_WG - 1));
    const bool in = g < gt.G;
    GroupLanes f;
    f.c = in ? gt.c[g] : 0;
    f.T = in ? gt.T[g] : 0;
    f.sq = in ? gt.sq[g] : 0;
    f.h = in ? gt.head[g] : 0;
    f.w = WINDOW && in ? gt.window[g] : 0;
    return f;
}

// blocks of a group of c tokens: [c x c] results (square) or [c x hd]
__device__ __forceinline__ int blocks_across(int c, bool square, int hd) { return square ? (c + 31) >> 5 : (hd + 31) >> 5; }

struct TaskSet {
    int first[FUSED_GROUPS_PER_WG + 1];     // first[q]: blocks of the groups in front of group q (scalars)
};
__device__ __forceinline__ TaskSet make_tasks(const GroupLanes& f, bool square, int hd) {
    TaskSet t;
    t.first[0] = 0;
#pragma unroll
    for (int q = 0; q < FUSED_GROUPS_PER_WG; ++q) {
        const int c = __builtin_amdgcn_readlane(f.c, q);
        t.first[q + 1] = t.first[q] + ((c + 31) >> 5) * blocks_across(c, square, hd);
    }
    return t;
}

// a task belongs to the whole wavefront: its parameters are scalars
struct Task {
    int c, bi, bj, T, sq, h, w;
};
__device__ __forceinline__ Task locate_task(const TaskSet& ts, const GroupLanes& f, int t, bool square, int hd) {
    int q = 0, f0 = 0;
#pragma unroll
    for (int qq = 1; qq < FUSED_GROUPS_PER_WG; ++qq) {
        const bool behind = t >= ts.first[qq];
        q += behind ? 1 : 0;
        f0 = behind ? ts.first[qq] : f0;
    }
    Task k;
    k.c = __builtin_amdgcn_readlane(f.c, q);
    k.T = __builtin_amdgcn_readlane(f.T, q);
    k.sq = __builtin_amdgcn_readlane(f.sq, q);
    k.h = __builtin_amdgcn_readlane(f.h, q);
    k.w = __builtin_amdgcn_readlane(f.w, q);
    const int nj = blocks_across(k.c, square, hd), local = t - f0;
    k.bi = local / nj;
    k.bj = local - k.bi * nj;
    return k;
}

// Token rows through a buffer descriptor over the whole tensor, shifted to the head's first channel: element
// (voxel v, channel ch of head h) is at byte offset v * stride * sizeof(T) + ch * sizeof(T).  `span` = bytes of the
// whole [N, stride] tensor (at most 2^31: the launcher checks).
template <typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t head_rows(const TokenTensor& t, int h, int hd, uint32_t span) {
    const uint32_t shift = (uint32_t)(t.col0 + h * hd) * (uint32_t)sizeof(T);
    return buf_of(static_cast<const T*>(t.base) + t.col0 + h * hd, span - shift);
}

// ------------------------------------------------------------------------------------------
// tokens x tokens -> sq :  out[i, j] = sum_ch A[token i, ch] * B[token j, ch]   (K = hd)
//   EPI = SQ_SCORES: S = scale*acc + bias[h, pos_i, pos_j] + (mask region differs ? -100 : 0), row ids
//   EPI = SQ_PLAIN : plain product (dP = dO V^T)
//   EPI = SQ_SCORE_GRAD: dS = P (dO V^T - D) with D_i = dO_i . O_i (= sum_j P_ij dP_ij, since O = P V): the softmax
//         backward (ops.cu:169-194) as the epilogue of the product, so dP never reaches memory and no softmax
//         launch follows.  A = dO, B = V, tc = O (rows like A's), `bias` = P (the sq array of the forward pass).
// Rows of tokens behind the window's last one are read as zeros and their results dropped by the bounds checks
// of the buffer descriptors (mfma_block.hpp).
// ------------------------------------------------------------------------------------------
enum { SQ_PLAIN = 0, SQ_SCORES = 1, SQ_SCORE_GRAD = 2 };

template <typename T, int EPI>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(EPI == SQ_PLAIN ? FUSED_SQ_PLAIN_WAVES : 4, EPI == SQ_PLAIN ? FUSED_SQ_PLAIN_WAVES : 4))) void fused_sq_kernel(FusedGroups gt, const int32_t* __restrict__ order,
                                                       const int32_t* __restrict__ tok_pos, int H, int hd,
                                                       TokenTensor ta, TokenTensor tb, TokenTensor tc, uint32_t a_span, uint32_t b_span,
                                                       uint32_t c_span, float scale_a,
                                                       const float* __restrict__ bias, int n,
                                                       const int8_t* __restrict__ mask, int n_mask_windows,
                                                       float* __restrict__ out, int32_t* __restrict__ row_ids) {
    constexpr uint32_t ES = (uint32_t)sizeof(T);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    const int64_t g0 = (int64_t)blockIdx.x * FUSED_GROUPS_PER_WG;
    const GroupLanes gl = load_groups<EPI == SQ_SCORES>(gt, g0, lane);
    const TaskSet ts = make_tasks(gl, true, hd);
    const int total = ts.first[FUSED_GROUPS_PER_WG];
    const uint32_t a_pitch = (uint32_t)ta.stride * ES, b_pitch = (uint32_t)tb.stride * ES, c_pitch = (uint32_t)tc.stride * ES;

    for (int t = wave + 4 * (int)blockIdx.y; t < total; t += 4 * (int)gridDim.y) {   // gridDim.y workgroups share the groups' blocks
        const Task k = locate_task(ts, gl, t, true, hd);
        const int c = k.c, Tk = k.T, h = k.h, bi = k.bi, bj = k.bj;
        const int i_a = bi * 32 + l32, j_b = bj * 32 + l32;
        const bool a_in = i_a < c, b_in = j_b < c;
        const int32_t* ord = order + Tk;
        const int vox_i = ord[a_in ? i_a : c - 1], vox_j = ord[b_in ? j_b : c - 1];
        // epilogue inputs: one load per lane (row token, column token); the 16 rows a lane stores
        // are fetched from the row lanes with cross-lane reads in the epilogue
        int pos_a = 0, pos_j = 0, m_a = 0, m_j = 0;
        if (EPI == SQ_SCORES) {
            pos_a = tok_pos[Tk + (a_in ? i_a : c - 1)];
            pos_j = tok_pos[Tk + (b_in ? j_b : c - 1)];
            if (mask) {
                const int8_t* mrow = mask + (int64_t)(k.w % n_mask_windows) * n;
                m_a = mrow[pos_a];
                m_j = mrow[pos_j];
            }
        }
        const __amdgpu_buffer_rsrc_t ra = head_rows<T>(ta, h, hd, a_span), rb = head_rows<T>(tb, h, hd, b_span);
        const uint32_t row_a = a_in ? (uint32_t)vox_i * a_pitch : BUF_OUTSIDE;
        const uint32_t row_b = b_in ? (uint32_t)vox_j * b_pitch : BUF_OUTSIDE;
        // entry (i, j) of the block at byte offset (i * c + j) * 4: rows behind the last one are outside by themselves
        const uint32_t o0 = b_in ? (uint32_t)((bi * 32 + 4 * half) * c + j_b) * 4u : BUF_OUTSIDE;
        // score gradient: D collects dO_i . O_i over this lane's channels
        float d_part = 0.f;
        __amdgpu_buffer_rsrc_t rc = ra;
        uint32_t row_c = BUF_OUTSIDE;
        if (EPI == SQ_SCORE_GRAD) {
            rc = head_rows<T>(tc, h, hd, c_span);
            row_c = a_in ? (uint32_t)vox_i * c_pitch : BUF_OUTSIDE;
        }

        // scores: the bias values of the 16 rows a lane stores are gathered here, beside the row loads (behind the matrix
        // steps they were one more memory round trip per task); position and mask region of a row come from its row
        // lane in one cross-lane read
        float bv[16];
        int m_i[16];
        if (EPI == SQ_SCORES) {
            const float* brow = bias + (int64_t)h * n * n + pos_j;
            const int pm_a = pos_a | (m_a << 16);                   // positions stay below 2^15, regions below 2^7
#pragma unroll
            for (int r = 0; r < 16; ++r) {                          // all lanes take part in the cross-lane reads
                const int pm = __shfl(pm_a, acc_row(r, half), 64);
                bv[r] = brow[(pm & 0xffff) * n];
                m_i[r] = pm >> 16;
            }
        }

        f32x16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        for (int kc = 0; kc < hd; kc += 32) {
            // the channels of a chunk are split evenly between the two lane halves: a head of 16 channels takes
            // eight matrix steps, not sixteen with one half feeding zeros
            const int chunk = hd - kc < 32 ? hd - kc : 32;
            const int kh = (chunk + 1) >> 1;
            const int left = half ? chunk - kh : kh;
            const uint32_t ch0 = (uint32_t)(kc + half * kh) * ES;
            float a[16], b[16];
            if (chunk == 32) {
                buf_load_run<T, 16>(ra, row_a + ch0, a);
                buf_load_run<T, 16>(rb, row_b + ch0, b);
            } else if (chunk == 16) {
                buf_load_run<T, 8>(ra, row_a + ch0, a);
                buf_load_run<T, 8>(rb, row_b + ch0, b);
            } else {
#pragma unroll
                for (int s = 0; s < 16; ++s) {
                    a[s] = buf_load1<T>(ra, s < left ? row_a + ch0 + ES * s : BUF_OUTSIDE);
                    b[s] = buf_load1<T>(rb, s < left ? row_b + ch0 + ES * s : BUF_OUTSIDE);
                }
            }
            if (EPI == SQ_SCORE_GRAD) {
                float o[16];
                if (chunk == 32) {
                    buf_load_run<T, 16>(rc, row_c + ch0, o);
                } else if (chunk == 16) {
                    buf_load_run<T, 8>(rc, row_c + ch0, o);
                } else {
#pragma unroll
                    for (int s = 0; s < 16; ++s) o[s] = buf_load1<T>(rc, s < left ? row_c + ch0 + ES * s : BUF_OUTSIDE);
                }
#pragma unroll
                for (int s = 0; s < 16; ++s)
                    if (s < kh) d_part = fmaf(a[s], o[s], d_part);
            }
            if (scale_a != 1.0f) {
#pragma unroll
                for (int s = 0; s < 16; ++s) a[s] *= scale_a;
            }
#pragma unroll
            for (int s = 0; s < 16; ++s)
                if (s < kh) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[s], acc, 0, 0, 0);
        }

        if constexpr (EPI == SQ_SCORE_GRAD) {
            // the block of P (requested behind the matrix steps: sixteen more registers in flight beside the operands
            // would spill); D of row i_a: the two lane halves hold the two halves of its channels
            const __amdgpu_buffer_rsrc_t rp = buf_of(bias + k.sq, (uint32_t)(c * c) * 4u);
            float pv[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) pv[r] = buf_load1<float>(rp, o0 + (uint32_t)((8 * (r >> 2) + (r & 3)) * c) * 4u);
            const float d_row = d_part + __shfl_xor(d_part, 32, 64);
            const __amdgpu_buffer_rsrc_t ro = buf_of(out + k.sq, (uint32_t)(c * c) * 4u);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float d_r = __shfl(d_row, acc_row(r, half), 64);
                const float v = acc[r];
                buf_store1<float>(ro, o0 + (uint32_t)((8 * (r >> 2) + (r & 3)) * c) * 4u, pv[r] * (v - d_r));
            }
        } else {
            const __amdgpu_buffer_rsrc_t ro = buf_of(out + k.sq, (uint32_t)(c * c) * 4u);
            const __amdgpu_buffer_rsrc_t rr = buf_of(row_ids ? row_ids + k.sq : nullptr, row_ids ? (uint32_t)(c * c) * 4u : 0u);
            const int rid0 = H * Tk + h * c + bi * 32 + 4 * half;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = 8 * (r >> 2) + (r & 3);             // + 4 * half: the row of the block
                float v = acc[r];
                if (EPI) {
                    v += bv[r];
                    if (mask && m_i[r] != m_j) v += -100.0f;
                    if (row_ids) __builtin_amdgcn_raw_buffer_store_b32((uint32_t)(rid0 + row), rr, o0 + (uint32_t)(row * c) * 4u, 0, 0);
                }
                buf_store1<float>(ro, o0 + (uint32_t)(row * c) * 4u, v);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// sq x tokens -> tokens :  out[token i, ch] = scale * sum_k A(i, k) * B[token k, ch]   (K = c)
//   A_KMAJOR = false: A(i, k) = sq[i*c + k]   (O = P V, dQ = dS K)
//   A_KMAJOR = true : A(i, k) = sq[k*c + i]   (dV = P^T dO, dK = dS^T Q)
// ------------------------------------------------------------------------------------------
template <typename T, bool A_KMAJOR>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(FUSED_TOK_WAVES, FUSED_TOK_WAVES))) void fused_tok_kernel(FusedGroups gt, const int32_t* __restrict__ order, int hd,
                                                        const float* __restrict__ sq, TokenTensor tb,
                                                        TokenTensor to, uint32_t b_span, uint32_t o_span, float scale_out) {
    constexpr uint32_t ES = (uint32_t)sizeof(T);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    const int64_t g0 = (int64_t)blockIdx.x * FUSED_GROUPS_PER_WG;
    const GroupLanes gl = load_groups<false>(gt, g0, lane);
    const TaskSet ts = make_tasks(gl, false, hd);
    const int total = ts.first[FUSED_GROUPS_PER_WG];
    const uint32_t b_pitch = (uint32_t)tb.stride * ES, o_pitch = (uint32_t)to.stride * ES;

    for (int t = wave + 4 * (int)blockIdx.y; t < total; t += 4 * (int)gridDim.y) {   // gridDim.y workgroups share the groups' blocks
        const Task k = locate_task(ts, gl, t, false, hd);
        const int c = k.c, Tk = k.T, h = k.h, bi = k.bi, bj = k.bj;
        const int i_a = bi * 32 + l32, j_b = bj * 32 + l32;
        const bool a_in = i_a < c, b_in = j_b < hd;
        const int32_t* ord = order + Tk;
        // voxel of this lane's row token (the 16 rows a lane stores are fetched with cross-lane reads) and the
        // voxels of the first 32 reduction tokens
        const int vox_a = ord[a_in ? i_a : c - 1];
        int ord_l = ord[l32 < c ? l32 : c - 1];
        const __amdgpu_buffer_rsrc_t rs = buf_of(sq + k.sq, (uint32_t)(c * c) * 4u);
        const __amdgpu_buffer_rsrc_t rb = head_rows<T>(tb, h, hd, b_span), ro = head_rows<T>(to, h, hd, o_span);
        const uint32_t col = (uint32_t)j_b * ES;

        f32x16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        for (int kc = 0; kc < c; kc += 32) {
            const int chunk = c - kc < 32 ? c - kc : 32;
            const int kh = (chunk + 1) >> 1;                        // reduction tokens per lane half (uniform)
            const int left = half ? chunk - kh : kh;
            // voxels of the next chunk's tokens: requested now, so that its rows do not wait for them
            const int ord_cur = ord_l;
            if (kc + 32 < c) ord_l = ord[kc + 32 + l32 < c ? kc + 32 + l32 : c - 1];
            float a[16], b[16];
            // B: row of token kc + half * kh + s, this lane's channel
            auto b_load = [&](const int s) __attribute__((always_inline)) {
                const int vox = __shfl(ord_cur, half * kh + s, 64);
                b[s] = buf_load1<T>(rb, (b_in && s < left) ? (uint32_t)vox * b_pitch + col : BUF_OUTSIDE);
            };
#pragma unroll
            for (int s = 0; s < 8; ++s) b_load(s);
            if (kh > 8) {
#pragma unroll
                for (int s = 8; s < 16; ++s) b_load(s);
            }
            if (!A_KMAJOR) {
                // a row per lane: values of k behind the row's end belong to the next row and are masked through their offsets
                const uint32_t v0 = a_in ? (uint32_t)(i_a * c + kc + half * kh) * 4u : BUF_OUTSIDE;
                if (chunk == 32) {
                    buf_load_run<float, 16>(rs, v0, a);
                } else {
#pragma unroll
                    for (int s = 0; s < 16; ++s) a[s] = buf_load1<float>(rs, s < left ? v0 + 4u * s : BUF_OUTSIDE);
                }
            } else {
                // element (kc + half * kh + s, i): rows of k behind the block's last one are outside by themselves
                const uint32_t v0 = a_in ? (uint32_t)(half * kh * c + i_a) * 4u : BUF_OUTSIDE;
#pragma unroll
                for (int s = 0; s < 8; ++s) a[s] = buf_load1<float>(rs, v0 + (uint32_t)((kc + s) * c) * 4u);
                if (kh > 8) {
#pragma unroll
                    for (int s = 8; s < 16; ++s) a[s] = buf_load1<float>(rs, v0 + (uint32_t)((kc + s) * c) * 4u);
                }
            }
#pragma unroll
            for (int s = 0; s < 16; ++s)
                if (s < kh) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[s], acc, 0, 0, 0);
        }

#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int il = acc_row(r, half);
            const int vox = __shfl(vox_a, il, 64);
            const float v = acc[r] * scale_out;
            buf_store1<T>(ro, (b_in && bi * 32 + il < c) ? (uint32_t)vox * o_pitch + col : BUF_OUTSIDE, v);
        }
    }
}

// ------------------------------------------------------------------------------------------
// sq -> sq: the sparse row softmax of the operator set (ops.cu:128-194: m = max(0, row maximum),
// y = exp(x - m) / (sum + 1e-8); backward gx = y (g - sum_j g_j y_j)) over the rows of the groups' [c x c] blocks.
// The rows are known from the group table, so no row ids are written by the score product or read here (4 of the
// 12 / 16 bytes per entry of the id-driven kernel).  A task = 32 rows of a group; LPR lanes share a row (16, 32 or
// all 64, the smallest that holds the row in at most six values per lane), so a wavefront works on 4, 2 or 1 rows
// at a time and reduces with DPP moves inside 16 lanes plus one or two cross-lane reads.  In place (out == the
// input, or == grad in the backward) is fine: a wavefront reads the values of a row before it writes any of them.
// ------------------------------------------------------------------------------------------
template <int LPR>
__device__ __forceinline__ float seg_sum(float v) {
    v = row16_sum(v);
    if (LPR >= 32) v += __shfl_xor(v, 16, 64);
    if (LPR >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}
// B steps of a task are requested together (a step alone would wait for its loads before the next one asks for its own)
template <int LPR>
__device__ __forceinline__ int seg_max_i32(int v) {
    v = max(v, dpp_i32<0xB1>(v));
    v = max(v, dpp_i32<0x4E>(v));
    v = max(v, dpp_i32<0x141>(v));
    v = max(v, dpp_i32<0x140>(v));
    if (LPR >= 32) v = max(v, __shfl_xor(v, 16, 64));
    if (LPR >= 64) v = max(v, __shfl_xor(v, 32, 64));
    return v;
}

template <bool BWD, int LPR, int U, int B>
__device__ __forceinline__ void group_softmax_rows(const __amdgpu_buffer_rsrc_t& rx, const __amdgpu_buffer_rsrc_t& rg,
                                                   const __amdgpu_buffer_rsrc_t& ro, int c, int row0, int rows, int lane) {
    constexpr int RPS = 64 / LPR;                              // rows per step
    const int j0 = lane & (LPR - 1), rl = lane / LPR;
    for (int r0 = 0; r0 < rows; r0 += RPS * B) {
        float x[B][U], g[B][U];
        uint32_t off[B][U];
#pragma unroll
        for (int b = 0; b < B; ++b) {
            const int r = r0 + b * RPS + rl;
            const uint32_t base = (uint32_t)((row0 + r) * c) * 4u;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int j = j0 + LPR * u;
                off[b][u] = (j < c && r < rows) ? base + 4u * (uint32_t)j : BUF_OUTSIDE;
                x[b][u] = buf_load1<float>(rx, off[b][u]);
                if (BWD) g[b][u] = buf_load1<float>(rg, off[b][u]);
            }
        }
#pragma unroll
        for (int b = 0; b < B; ++b) {
            if (!BWD) {
                // m = max(0, row maximum): values below zero do not matter, and the bit patterns of floats from zero
                // upwards are ordered like integers, so the maximum is taken over max(bits, 0) with integer
                // instructions (a negative float is a negative integer; loads outside the row gave zero)
                int mb = 0;
#pragma unroll
                for (int u = 0; u < U; ++u) mb = max(mb, __builtin_bit_cast(int, x[b][u]));
                const float m = __builtin_bit_cast(float, seg_max_i32<LPR>(mb));
                float sum = 0.f;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    x[b][u] = off[b][u] != BUF_OUTSIDE ? __builtin_amdgcn_exp2f((x[b][u] - m) * 1.44269504088896f) : 0.f;   // x - m <= 0: no range problem
                    sum += x[b][u];
                }
                const float inv = __builtin_amdgcn_rcpf(seg_sum<LPR>(sum) + 1e-8f);   // 1 ulp: inside the tolerance of a product of two roundings
#pragma unroll
                for (int u = 0; u < U; ++u) buf_store1<float>(ro, off[b][u], x[b][u] * inv);
            } else {
                float dot = 0.f;
#pragma unroll
                for (int u = 0; u < U; ++u) dot += x[b][u] * g[b][u];   // loads outside the row are zero
                dot = seg_sum<LPR>(dot);
#pragma unroll
                for (int u = 0; u < U; ++u) buf_store1<float>(ro, off[b][u], x[b][u] * (g[b][u] - dot));
            }
        }
    }
}

template <bool BWD>
__global__ __launch_bounds__(256) void group_softmax_kernel(FusedGroups gt, const float* __restrict__ xs,
                                                            const float* __restrict__ gs, float* __restrict__ out) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int64_t g0 = (int64_t)blockIdx.x * FUSED_GROUPS_PER_WG;
    const GroupLanes gl = load_groups<false>(gt, g0, lane);
    const TaskSet ts = make_tasks(gl, false, 1);                // one task per 32 rows of a group
    const int total = ts.first[FUSED_GROUPS_PER_WG];
    for (int t = wave + 4 * (int)blockIdx.y; t < total; t += 4 * (int)gridDim.y) {
        const Task k = locate_task(ts, gl, t, false, 1);
        const int c = k.c, row0 = k.bi * 32;
        const int rows = c - row0 < 32 ? c - row0 : 32;
        const uint32_t bytes = (uint32_t)(c * c) * 4u;
        const __amdgpu_buffer_rsrc_t rx = buf_of(xs + k.sq, bytes), rg = buf_of(BWD ? gs + k.sq : xs + k.sq, bytes);
        const __amdgpu_buffer_rsrc_t ro = buf_of(out + k.sq, bytes);
        if (c <= 16) group_softmax_rows<BWD, 16, 1, 8>(rx, rg, ro, c, row0, rows, lane);
        else if (c <= 32) group_softmax_rows<BWD, 32, 1, 16>(rx, rg, ro, c, row0, rows, lane);
        else if (c <= 128) group_softmax_rows<BWD, 64, 2, 8>(rx, rg, ro, c, row0, rows, lane);
        else group_softmax_rows<BWD, 64, 6, 2>(rx, rg, ro, c, row0, rows, lane);
    }
}

// ------------------------------------------------------------------------------------------
// The same two products with 64-bit addresses, for token tensors that a buffer descriptor cannot cover (more than
// 2^31 bytes, or 16-bit rows that do not start at a multiple of four bytes).
// tokens x tokens -> sq :  out[i, j] = sum_ch A[token i, ch] * B[token j, ch]   (K = hd)
//   EPI = true : S = scale*acc + bias[h, pos_i, pos_j] + (mask region differs ? -100 : 0), row ids
//   EPI = false: plain product (dP = dO V^T)
// ------------------------------------------------------------------------------------------
template <typename T, bool EPI>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void fused_sq_wide_kernel(FusedGroups gt, const int32_t* __restrict__ order,
                                                       const int32_t* __restrict__ tok_pos, int H, int hd,
                                                       TokenTensor ta, TokenTensor tb, float scale_a,
                                                       const float* __restrict__ bias, int n,
                                                       const int8_t* __restrict__ mask, int n_mask_windows,
                                                       float* __restrict__ out, int32_t* __restrict__ row_ids) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    const int64_t g0 = (int64_t)blockIdx.x * FUSED_GROUPS_PER_WG;
    const GroupLanes gl = load_groups<EPI>(gt, g0, lane);
    const TaskSet ts = make_tasks(gl, true, hd);
    const int total = ts.first[FUSED_GROUPS_PER_WG];
    const T* A = static_cast<const T*>(ta.base);
    const T* B = static_cast<const T*>(tb.base);

    for (int t = wave + 4 * (int)blockIdx.y; t < total; t += 4 * (int)gridDim.y) {   // gridDim.y workgroups share the groups' blocks
        const Task k = locate_task(ts, gl, t, true, hd);
        const int c = k.c, bi = k.bi, bj = k.bj, Tk = k.T, h = k.h;
        const int64_t sq0 = k.sq;
        const int i_a = bi * 32 + l32, j_b = bj * 32 + l32;
        const bool a_in = i_a < c, b_in = j_b < c;
        // rows past the end of the window are clamped to its last token: their products are finite
        // garbage that is never stored, and no load needs a predicate
        const int i_c = a_in ? i_a : c - 1, j_c = b_in ? j_b : c - 1;
        const T* pa = A + (int64_t)order[Tk + i_c] * ta.stride + ta.col0 + h * hd;
        const T* pb = B + (int64_t)order[Tk + j_c] * tb.stride + tb.col0 + h * hd;

        // epilogue inputs: one load per lane (row token, column token); the 16 rows a lane stores
        // are fetched from the row lanes with cross-lane reads in the epilogue
        int pos_a = 0, pos_j = 0, m_a = 0, m_j = 0;
        if (EPI) {
            pos_a = tok_pos[Tk + i_c];
            pos_j = tok_pos[Tk + j_c];
            if (mask) {
                const int8_t* mrow = mask + (int64_t)(k.w % n_mask_windows) * n;
                m_a = mrow[pos_a];
                m_j = mrow[pos_j];
            }
        }

        f32x16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        for (int kc = 0; kc < hd; kc += 32) {
            const int kb = kc + half * 16;
            float a[16], b[16];
            if (kc + 32 <= hd) {                                   // full chunk (uniform)
                load_run16_full<T>(pa + kb, a);
                load_run16_full<T>(pb + kb, b);
                if (scale_a != 1.0f) {
#pragma unroll
                    for (int s = 0; s < 16; ++s) a[s] *= scale_a;
                }
#pragma unroll
                for (int s = 0; s < 16; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[s], acc, 0, 0, 0);
            } else {
                // the channels left are split evenly between the two lane halves: a head of 16 channels takes eight
                // matrix steps, not sixteen with one half feeding zeros
                const int chunk = hd - kc;
                const int kh = (chunk + 1) >> 1;
                const int left = half ? chunk - kh : kh;
                load_run16<T>(pa + kc + half * kh, left, a);
                load_run16<T>(pb + kc + half * kh, left, b);
                if (scale_a != 1.0f) {
#pragma unroll
                    for (int s = 0; s < 16; ++s) a[s] *= scale_a;
                }
#pragma unroll
                for (int s = 0; s < 16; ++s)
                    if (s < kh) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[s], acc, 0, 0, 0);
            }
        }

        {
            float* O = out + sq0 + j_b;
            const float* brow = EPI ? bias + (int64_t)h * n * n + pos_j : nullptr;
            const int rid0 = H * Tk + h * c;
            // bias values of the 16 rows are gathered before any of them is used, so that the
            // gather latencies overlap instead of adding up
            float bv[16];
            int m_i[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                bv[r] = 0.f;
                m_i[r] = 0;
                if (EPI) {                                          // all lanes take part in the shuffles
                    const int il = acc_row(r, half);
                    bv[r] = brow[__shfl(pos_a, il, 64) * n];
                    if (mask) m_i[r] = __shfl(m_a, il, 64);
                }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int i = bi * 32 + acc_row(r, half);
                if (b_in && i < c) {
                    float v = acc[r];
                    if (EPI) {
                        v += bv[r];
                        if (mask && m_i[r] != m_j) v += -100.0f;
                        if (row_ids) row_ids[sq0 + (int64_t)i * c + j_b] = rid0 + i;
                    }
                    O[(int64_t)i * c] = v;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// sq x tokens -> tokens :  out[token i, ch] = scale * sum_k A(i, k) * B[token k, ch]   (K = c)
//   A_KMAJOR = false: A(i, k) = sq[i*c + k]   (O = P V, dQ = dS K)
//   A_KMAJOR = true : A(i, k) = sq[k*c + i]   (dV = P^T dO, dK = dS^T Q)
// ------------------------------------------------------------------------------------------
template <typename T, bool A_KMAJOR>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void fused_tok_wide_kernel(FusedGroups gt, const int32_t* __restrict__ order, int hd,
                                                        const float* __restrict__ sq, TokenTensor tb,
                                                        TokenTensor to, float scale_out) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    const int64_t g0 = (int64_t)blockIdx.x * FUSED_GROUPS_PER_WG;
    const GroupLanes gl = load_groups<false>(gt, g0, lane);
    const TaskSet ts = make_tasks(gl, false, hd);
    const int total = ts.first[FUSED_GROUPS_PER_WG];
    const T* B = static_cast<const T*>(tb.base);
    T* O = static_cast<T*>(const_cast<void*>(to.base));

    for (int t = wave + 4 * (int)blockIdx.y; t < total; t += 4 * (int)gridDim.y) {   // gridDim.y workgroups share the groups' blocks
        // the block of the attention matrix is addressed by a scalar base plus 32-bit lane offsets (c <= 32767, so
        // c * c * 4 fits)
        const Task k = locate_task(ts, gl, t, false, hd);
        const int c = k.c, bi = k.bi, bj = k.bj, Tk = k.T, h = k.h;
        const float* S = sq + k.sq;
        const int i_a = bi * 32 + l32, j_b = bj * 32 + l32;
        const bool a_in = i_a < c, b_in = j_b < hd;
        const int i_c = a_in ? i_a : c - 1, j_c = b_in ? j_b : hd - 1;     // clamped: loads need no predicate

        // voxel of this lane's row token; the 16 rows a lane stores are fetched with cross-lane reads
        const int vox_a = a_in ? order[Tk + i_a] : -1;
        const T* bcol = B + tb.col0 + h * hd + j_c;

        f32x16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        for (int kc = 0; kc < c; kc += 32) {
            const int kb = kc + half * 16;
            // voxels of the 32 tokens of this k chunk: one coalesced load, then cross-lane reads
            const int kt = kc + l32;
            const int ord_l = order[Tk + (kt < c ? kt : c - 1)];
            float a[16], b[16];
#pragma unroll
            for (int s = 0; s < 16; ++s) {
                const int vox = __shfl(ord_l, half * 16 + s, 64);
                b[s] = to_acc(bcol[(int64_t)vox * tb.stride]);
            }
            if (kc + 32 <= c) {                                    // full chunk (uniform)
                if (!A_KMAJOR) {
                    load_run16_full<float>(S + (uint32_t)(i_c * c + kb), a);
                } else {
                    const uint32_t o0 = (uint32_t)(kb * c + i_c);
#pragma unroll
                    for (int s = 0; s < 16; ++s) a[s] = S[o0 + (uint32_t)(s * c)];
                }
#pragma unroll
                for (int s = 0; s < 16; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[s], acc, 0, 0, 0);
            } else {
                const int left = c - kb;                           // k values left for this lane half
#pragma unroll
                for (int s = 0; s < 16; ++s) {
                    const int k = kb + s < c ? kb + s : c - 1;
                    const float v = S[A_KMAJOR ? (uint32_t)(k * c + i_c) : (uint32_t)(i_c * c + k)];
                    a[s] = s < left ? v : 0.f;                     // zero A kills the clamped B rows
                }
                const int steps = c - kc;
#pragma unroll
                for (int s = 0; s < 16; ++s)
                    if (s < steps) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[s], acc, 0, 0, 0);
            }
        }

        {
            const int col = to.col0 + h * hd + j_b;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int vox = __shfl(vox_a, acc_row(r, half), 64);
                if (b_in && vox >= 0) O[(int64_t)vox * to.stride + col] = from_acc<T>(acc[r] * scale_out);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// gradient of the relative position bias: d_rpb[h, pos_i, pos_j] = sum of dS over all windows.
// Stage 1, grid (slices, H): a workgroup of 16 wavefronts walks its share of the windows and
// accumulates into an LDS copy of one head's [n x n] table.  All wavefronts look at the same
// window; wavefront r owns the table rows [r*RB, (r+1)*RB), i.e. the rows of dS whose token
// position falls into that range (a contiguous run of rows, positions being sorted inside a
// window).  Table rows are therefore private to a wavefront: plain LDS read-add-write, no
// atomics, and a fixed summation order.  The next window's header and positions are fetched
// while the current one is processed.  Stage 2 sums the per-slice tables in slice order.
// ------------------------------------------------------------------------------------------
constexpr int RPB_THREADS = 1024;

struct RpbWindow {
    int c, Tk, pos0, pos1;
    int64_t sq;
};

__device__ __forceinline__ RpbWindow rpb_fetch(const FusedGroups& gt, const int32_t* __restrict__ tok_pos,
                                               int64_t k, int64_t windows, int H, int h, int lane) {
    RpbWindow w{0, 0, 0, 0, 0};
    if (k < windows) {
        const int64_t g = k * H + h;
        w.c = gt.c[g];
        w.Tk = gt.T[g];
        w.sq = gt.sq[g];
        w.pos0 = lane < w.c ? tok_pos[w.Tk + lane] : -1;
        w.pos1 = 64 + lane < w.c ? tok_pos[w.Tk + 64 + lane] : -1;
    }
    return w;
}

__global__ __launch_bounds__(RPB_THREADS) void rpb_grad_partial_kernel(FusedGroups gt,
                                                                       const int32_t* __restrict__ tok_pos, int H,
                                                                       int n, const float* __restrict__ ds,
                                                                       float* __restrict__ partial) {
    extern __shared__ float table[];
    const int h = blockIdx.y;
    const int nn = n * n;
    constexpr int WAVES = RPB_THREADS / 64;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int rb = (n + WAVES - 1) / WAVES;
    const int lo = wave * rb, hi = lo + rb;                        // table rows owned by this wavefront
    for (int e = threadIdx.x; e < nn; e += RPB_THREADS) table[e] = 0.f;
    __syncthreads();
    const int64_t windows = gt.G / H;
    RpbWindow next = rpb_fetch(gt, tok_pos, blockIdx.x, windows, H, h, lane);
    for (int64_t k = blockIdx.x; k < windows; k += gridDim.x) {
        const RpbWindow w = next;
        next = rpb_fetch(gt, tok_pos, k + gridDim.x, windows, H, h, lane);
        const int c = w.c;
        // rows of this window whose position lies in [lo, hi): a contiguous run i_lo .. i_lo+cnt-1
        const unsigned long long m0 = __ballot(w.pos0 >= lo && w.pos0 < hi);
        const unsigned long long m1 = __ballot(w.pos1 >= lo && w.pos1 < hi);
        const int cnt = __popcll(m0) + __popcll(m1);
        if (cnt == 0) continue;                                     // wave-uniform
        const int i_lo = m0 ? __ffsll((long long)m0) - 1 : 64 + __ffsll((long long)m1) - 1;
        const int count = cnt * c;                                  // contiguous values of dS
        const float* S = ds + w.sq + (int64_t)i_lo * c;
        const uint32_t magic = (uint32_t)((0x100000000ull + (uint32_t)c - 1) / (uint32_t)c);
        for (int f0 = 0; f0 < count; f0 += 64 * 4) {
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int f = f0 + u * 64 + lane;
                v[u] = f < count ? S[f] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int f = f0 + u * 64 + lane;
                const int fc = f < count ? f : 0;
                const int il = (int)__umulhi((uint32_t)fc, magic);
                const int j = fc - il * c;
                const int i = i_lo + il;
                const int pi0 = __shfl(w.pos0, i & 63, 64), pi1 = __shfl(w.pos1, i & 63, 64);
                const int pj0 = __shfl(w.pos0, j & 63, 64), pj1 = __shfl(w.pos1, j & 63, 64);
                const int pi = i < 64 ? pi0 : pi1, pj = j < 64 ? pj0 : pj1;
                if (f < count) table[pi * n + pj] += v[u];
            }
        }
    }
    __syncthreads();
    float* dst = partial + ((int64_t)blockIdx.x * H + h) * nn;
    for (int e = threadIdx.x; e < nn; e += RPB_THREADS) dst[e] = table[e];
}

__global__ __launch_bounds__(256) void rpb_grad_reduce_kernel(const float* __restrict__ partial, int slices,
                                                              int64_t table_elems, float* __restrict__ d_rpb) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= table_elems) return;
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
    int s = 0;
    for (; s + 4 <= slices; s += 4) {
#pragma unroll
        for (int u = 0; u < 4; ++u) sum[u] += partial[(int64_t)(s + u) * table_elems + e];
    }
    for (; s < slices; ++s) sum[0] += partial[(int64_t)s * table_elems + e];
    d_rpb[e] += (sum[0] + sum[1]) + (sum[2] + sum[3]);
}

// ------------------------------------------------------------------------------------------
// Gradient of the relative position bias *table*: d_table[rel(p_i, p_j), h] = sum of dS over all
// windows, where rel(p_i, p_j) = code[p_i] - code[p_j] + offset0 (the index arithmetic of
// sparse_swin/swin3d_base.py:630-647 is linear in the two positions).  A table has (2w-1)^3 rows
// (729 for 5^3 windows), so every wavefront keeps a private copy of one head's column in LDS:
// wavefront (h, s) walks its slice of the windows in plan order, reads the [c x c] blocks of dS
// row by row: the entries of one row of dS go to different table rows, so a half wavefront adds a
// row chunk with plain read-add-write, and the two halves work on alternate rows with a copy of
// the column each (ds_add_f32 instead: 0.15 ms against 0.04 on 12 M entries, the LDS adds one lane at a
// time).  Partial columns are summed in slice order by rpb_table_reduce_kernel.
// ------------------------------------------------------------------------------------------
// bias[h][p][q] = table[code[p] - code[q] + offset0][h]: the gather of swin3d_base.py:644-647 and its
// permute(2, 0, 1) in one pass (entries whose table row is out of range read as zero).
__global__ __launch_bounds__(256) void rpb_gather_kernel(const float* __restrict__ table, int rows, int H,
                                                         const int32_t* __restrict__ code, int offset0, int n,
                                                         float* __restrict__ bias) {
    const int e = blockIdx.x * 256 + threadIdx.x;
    if (e >= n * n) return;
    const int p = e / n, q = e - p * n;
    const unsigned r = (unsigned)(code[p] - code[q] + offset0);
    for (int h = 0; h < H; ++h) bias[(int64_t)h * n * n + e] = r < (unsigned)rows ? table[(int64_t)r * H + h] : 0.f;
}

constexpr int RPBT_MAX_ROWS = 4096;

// f(integral_constant<U>) for U = U0 .. U1 - 1 while it returns true
template <int U0, int U1, typename F>
__device__ __forceinline__ void static_steps(F&& f) {
    if constexpr (U0 < U1) {
        if (f(std::integral_constant<int, U0>())) static_steps<U0 + 1, U1>(f);
    }
}
constexpr int RPBT_U = 16;                                      // steps of a batch: one per lane of a DPP row
// dynamic LDS: [wave 4][half 2][rows_pad] floats, then the [n] codes of the window positions
//
// A step adds one row of a chunk of 32 columns per half wavefront: the entries of a row go to different table
// rows, and the halves (rows i and i + 1) add into separate copies of the table, so plain read-add-write is
// enough and the sums have a fixed order.  RPBT_U steps (2 RPBT_U rows of one chunk) make a batch.  All loads of a
// batch (its entries of dS, the positions of its rows and columns) follow from the window's header, so a
// cursor runs two batches ahead of the adds and the batches wait in three register slots taken in turn (a
// slot is never copied: a copy would wait for its loads).
//
// Which batches a wavefront adds (BY_TASKS):
//   false: from the group table.  A slice of wavefronts takes every wslices-th window and deals the batches of its
//          windows among its rsplit members (each member walks over all windows of the slice).
//   true:  from the task descriptors of a token plan, which list the groups by their number of 32-token tiles
//          (fused TokenPlan, windows of at most 128 tokens).  The batches of a head, numbered bucket by bucket (16, 9,
//          4 or 1 per group), are cut into Q runs of equal length, one per wavefront of the head (consecutive
//          batches: neighbouring blocks of dS, and the same descriptor for the batches of a group), so every
//          wavefront adds the same number of batches (the slices of the group table differ by the sizes of the windows
//          that fall to them: 1.6 x between the fullest slice and the mean on a room of 112 000 voxels), and nothing
//          is walked: lane l decodes the l-th batch of the wavefront's run and loads its descriptor.
struct BatchList {
    const int4* tasks;       // [4][g_cap] descriptors {T, c | head << 8, window, sq}, bucket b = groups of b + 1 tiles
    int64_t g_cap;
    int first[4];            // batches of a head in front of bucket b (buckets in the order 3, 2, 1, 0)
    int total;               // batches of a head
};

template <bool BY_TASKS>
__global__ __launch_bounds__(256) void rpb_table_partial_kernel(FusedGroups gt, BatchList bl, const int32_t* __restrict__ tok_pos,
                                                                int H, const int32_t* __restrict__ code, int n,
                                                                int offset0, int rows, int rows_pad,
                                                                const float* __restrict__ ds, int64_t windows,
                                                                int wslices, int rsplit, float* __restrict__ partial) {
    extern __shared__ __attribute__((aligned(16))) float rpbt_lds[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int half = lane >> 5, l32 = lane & 31;
    int32_t* code_lds = reinterpret_cast<int32_t*>(rpbt_lds + 8 * rows_pad);
    for (int e = threadIdx.x; e < n; e += 256) code_lds[e] = code[e];
    __syncthreads();
    const int64_t p = (int64_t)blockIdx.x * 4 + wave;           // wavefront id = h * slices + sl
    const int slices = wslices * rsplit;                        // a multiple of four: the wavefronts of a workgroup share a head
    if (p >= (int64_t)slices * H) return;                       // (the whole workgroup then)
    const int h = (int)(p / slices);
    const int64_t sl = p % slices;
    const int64_t ws = sl % wslices;                            // windows ws, ws + wslices, ...
    const int rs = (int)(sl / wslices);                         // which of the rsplit wavefronts of this window slice
    float* tables = rpbt_lds + wave * 2 * rows_pad;
    float* mine = tables + half * rows_pad;
    for (int e = l32; e < rows; e += 32) mine[e] = 0.f;

    // A slice takes every wslices-th window (crowded windows are neighbours in plan order, so dealing them out
    // evens the load); the batches of its windows are dealt to the rsplit wavefronts of the slice.
    // The headers of 64 windows of the slice at a time sit in the lanes (lane l: the l-th of them).
    int hw_c = 0, hw_T = 0, hw_sq = 0, hw_ch = 0, hw_ib = 0;
    const int per_wave = BY_TASKS ? (bl.total + slices - 1) / slices : 0;   // a wavefront's run of consecutive batches
    auto load_headers = [&](int m_first) __attribute__((always_inline)) {
        hw_c = 0;
        if constexpr (BY_TASKS) {
            // batch number sl * per_wave + m_first + lane of head h -> bucket, group inside it, chunk and row block
            const int64_t f64 = sl * per_wave + m_first + lane;
            if (m_first + lane < per_wave && f64 < bl.total) {
                const int f = (int)f64;
                int b = 3, r = f - bl.first[3];
                if (f >= bl.first[2]) { b = 2; r = f - bl.first[2]; }
                if (f >= bl.first[1]) { b = 1; r = f - bl.first[1]; }
                if (f >= bl.first[0]) { b = 0; r = f - bl.first[0]; }
                const int nb = b + 1, per = nb * nb;
                const int gi = r / per, rem = r - gi * per;
                const int4 d = bl.tasks[(int64_t)b * bl.g_cap + (int64_t)gi * H + h];
                hw_T = d.x;
                hw_c = d.y & 0xff;
                hw_sq = d.w;
                hw_ib = (rem / nb) * 32;
                hw_ch = rem - (rem / nb) * nb;
            }
        } else {
            const int64_t k = ws + ((int64_t)m_first + lane) * wslices;
            if (k < windows) {
                const int64_t g = k * H + h;
                hw_c = gt.c[g];
                hw_T = gt.T[g];
                hw_sq = gt.sq[g];
            }
        }
    };
    constexpr int BR = 2 * RPBT_U;                              // rows of a batch
    struct Cursor {
        int m, m0, rot, c, T, sq, ch, ib;
        bool valid;
    };
    // The batches of a window, numbered chunk by chunk inside a block of BR rows, then block by block, are dealt to
    // the rsplit wavefronts of the slice: this one takes the numbers rot, rot + rsplit, ...; rot moves on by one
    // with every window.  A count of chunks beyond the window's chunks carries into the row blocks.
    auto carry = [&](Cursor cur) __attribute__((always_inline)) -> Cursor {
        const int nch = (cur.c + 31) >> 5;
        if (nch <= 1) {
            cur.ib += BR * cur.ch;
            cur.ch = 0;
        } else {
            while (cur.ch >= nch) {
                cur.ch -= nch;
                cur.ib += BR;
            }
        }
        return cur;
    };
    // first batch of window cur.m and after among the 64 windows whose headers are loaded, or none.  (Loading
    // headers here, inside the pipeline, would put a wait for all loads in flight on every path.)
    auto seek = [&](Cursor cur) __attribute__((always_inline)) -> Cursor {
        if constexpr (BY_TASKS) {
            // the batch of lane cur.m - cur.m0, or none (a lane without a batch holds c = 0)
            const int at = cur.m - cur.m0;
            const int c_at = at < 64 ? __builtin_amdgcn_readlane(hw_c, at & 63) : 0;
            if (c_at == 0) return Cursor{cur.m, cur.m0, 0, 1, 0, 0, 0, 0, false};
            return Cursor{cur.m, cur.m0, 0, c_at, __builtin_amdgcn_readlane(hw_T, at & 63), __builtin_amdgcn_readlane(hw_sq, at & 63),
                          __builtin_amdgcn_readlane(hw_ch, at & 63), __builtin_amdgcn_readlane(hw_ib, at & 63), true};
        }
        for (;;) {
            if (cur.m - cur.m0 == 64)                           // a batch nobody adds, at a safe address
                return Cursor{cur.m, cur.m0, cur.rot, 1, 0, 0, 0, 0, false};
            cur.c = __builtin_amdgcn_readlane(hw_c, cur.m - cur.m0);
            cur.ch = cur.rot;
            cur.ib = 0;
            cur = carry(cur);
            if (cur.ib < cur.c) {
                cur.T = __builtin_amdgcn_readlane(hw_T, cur.m - cur.m0);
                cur.sq = __builtin_amdgcn_readlane(hw_sq, cur.m - cur.m0);
                return cur;
            }
            ++cur.m;
            cur.rot = cur.rot + 1 == rsplit ? 0 : cur.rot + 1;
        }
    };
    auto advance = [&](Cursor cur) __attribute__((always_inline)) -> Cursor {
        if (!cur.valid) return cur;
        if constexpr (BY_TASKS) {
            ++cur.m;
            return seek(cur);
        }
        cur.ch += rsplit;
        cur = carry(cur);
        if (cur.ib < cur.c) return cur;
        ++cur.m;
        cur.rot = cur.rot + 1 == rsplit ? 0 : cur.rot + 1;
        return seek(cur);
    };
    struct Slot {
        float v[RPBT_U];
        int pj, pi;         // positions of this lane's column and of row ib + 2 (lane & 15) + half
        int c, ch, ib;
        bool valid;
    };
    const uint32_t table_off = (uint32_t)((wave * 2 + half) * rows_pad) * 4u;   // byte offset of this half's table
    const uint32_t trash_rel = (uint32_t)(rows_pad - 32 + l32) * 4u;            // a spare row per lane: rows_pad >= rows + 32
    auto issue = [&](Slot& s, const Cursor& cur) __attribute__((always_inline)) {
        // the loads are issued in any case: the waits of the other slots count on them
        s.valid = cur.valid;
        const uint32_t c = (uint32_t)cur.c;
        s.c = cur.c;
        s.ch = cur.ch;
        s.ib = cur.ib;
        const uint32_t j = (uint32_t)(cur.ch * 32 + l32);
        const uint32_t jc = j < c ? j : 0u;
        const float* src = ds + cur.sq;
        const uint32_t last = (c - 1u) * c + jc;
        const uint32_t first = (uint32_t)(cur.ib + half) * c + jc;
        // unconditional loads, rows beyond the window clamped to its last row and dropped later
#pragma unroll
        for (int u = 0; u < RPBT_U; ++u) {
            const uint32_t off = first + (uint32_t)(2 * u) * c;
            s.v[u] = src[off < last ? off : last];
        }
        const uint32_t ir = (uint32_t)(cur.ib + 2 * (lane & 15) + half);
        s.pj = tok_pos[(uint32_t)cur.T + jc];
        s.pi = tok_pos[(uint32_t)cur.T + (ir < c ? ir : c - 1u)];
    };
    // Step u of a batch: rows ib + 2u (first half of the wavefront) and ib + 2u + 1 (second half).  Lane l holds
    // the code of row ib + 2 (l & 15) + half, times four, so one DPP broadcast inside each 16 lanes (lane u
    // of them) hands every lane the code of its half's row.  Dead rows and columns carry codes that put the byte
    // offset beyond the table, as a table row below zero does: those entries land in a spare row, without a branch.
    auto consume = [&](const Slot& s) __attribute__((always_inline)) {
        const int c = s.c;
        const bool jlive = s.ch * 32 + l32 < c;
        const bool rlive = s.ib + 2 * (lane & 15) + half < c;
        const int cjb = jlive ? (code_lds[s.pj] - offset0) * 4 : -(1 << 30);
        const int crow4 = rlive ? code_lds[s.pi] * 4 : (1 << 30);
        static_steps<0, RPBT_U>([&](auto uc) __attribute__((always_inline)) {
            constexpr int u = decltype(uc)::value;
            if (s.ib + 2 * u >= c) return false;
            const int ci4 = __builtin_amdgcn_update_dpp(0, crow4, 0x150 + u, 0xf, 0xf, false);   // row_newbcast:u
            const uint32_t rel = (uint32_t)(ci4 - cjb);          // table row times four; negative or dead: huge
            const uint32_t off = (rel < trash_rel ? rel : trash_rel) + table_off;
            float* dst = reinterpret_cast<float*>(reinterpret_cast<char*>(rpbt_lds) + off);
            *dst += s.v[u];
            return true;
        });
    };
    int rot = rs;
    for (int m0 = 0; BY_TASKS ? m0 < per_wave && sl * per_wave + m0 < bl.total : ws + (int64_t)m0 * wslices < windows; m0 += 64) {
        load_headers(m0);
        Cursor cur = seek(Cursor{m0, m0, rot, 1, 0, 0, 0, 0, true});
        Slot sa, sb, sc;
        issue(sa, cur);
        cur = advance(cur);
        issue(sb, cur);
        cur = advance(cur);
        for (;;) {
            if (!sa.valid) break;
            issue(sc, cur);
            cur = advance(cur);
            consume(sa);
            if (!sb.valid) break;
            issue(sa, cur);
            cur = advance(cur);
            consume(sb);
            if (!sc.valid) break;
            issue(sb, cur);
            cur = advance(cur);
            consume(sc);
        }
        rot = cur.rot;
    }
    // the eight tables of the workgroup (four wavefronts, two halves each) are one head's: summed here in a fixed
    // order, so a quarter of the partial tables reaches memory and the reduction
    __syncthreads();
    float* out = partial + ((int64_t)h * (slices / 4) + sl / 4) * rows;
    for (int e = threadIdx.x; e < rows; e += 256) {
        float total = 0.f;
#pragma unroll
        for (int t = 0; t < 8; ++t) total += rpbt_lds[t * rows_pad + e];
        out[e] = total;
    }
}

// d_table[row, h] = sum over slices of partial[h][slice][row].  One workgroup per 16 table rows
// of one head: thread (q, r) adds the slices q, q+64, ... of row r (short chains, four loads in
// flight each), then the 64 chain sums of a row are added in the order of q: a fixed order.
__global__ __launch_bounds__(1024) void rpb_table_reduce_kernel(const float* __restrict__ partial, int slices, int rows,
                                                                int H, float* __restrict__ d_table) {
    __shared__ float part[64][17];
    const int r = threadIdx.x & 15, q = threadIdx.x >> 4;
    const int h = blockIdx.y;
    const int row = blockIdx.x * 16 + r;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (row < rows) {
        const float* src = partial + (int64_t)h * slices * rows + row;
        int s = q;
        for (; s + 192 < slices; s += 256) {
            s0 += src[(int64_t)s * rows];
            s1 += src[(int64_t)(s + 64) * rows];
            s2 += src[(int64_t)(s + 128) * rows];
            s3 += src[(int64_t)(s + 192) * rows];
        }
        for (; s < slices; s += 64) s0 += src[(int64_t)s * rows];
    }
    part[q][r] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (q == 0 && row < rows) {
        float total = 0.f;
#pragma unroll
        for (int k = 0; k < 64; ++k) total += part[k][r];
        d_table[(int64_t)row * H + h] = total;
    }
}

// Whether the rows of a token tensor can go through a buffer descriptor: the tensor spans at most 2^31 bytes and, for
// 16-bit values, every head's row slice starts at a multiple of four bytes (what the 16-byte loads need).
// SSWIN_FUSED_WIDE=1 in the environment sends everything to the kernels with 64-bit addresses.
template <typename T>
static bool rows_fit_descriptor(const TokenTensor& t, int64_t N, int hd, uint32_t* span) {
    const int64_t bytes = N * t.stride * (int64_t)sizeof(T);
    *span = (uint32_t)bytes;
    if (bytes > ((int64_t)1 << 31) || t.stride <= 0) return false;
    if (sizeof(T) == 2 && (((uintptr_t)t.base & 3) || (t.stride & 1) || (t.col0 & 1) || (hd & 1))) return false;
    const char* e = getenv("SSWIN_FUSED_WIDE");
    return !(e && e[0] == '1');
}

// epi: SQ_PLAIN, SQ_SCORES or SQ_SCORE_GRAD (then tc = O rows and bias = P).  *fused_done says whether the epilogue
// ran inside the product (always for the first two; the score gradient only on the descriptor kernel: otherwise
// the plain product is written and the caller runs the softmax backward over it).
template <typename T>
static int launch_sq(int epi, const FusedGroups& gt, int64_t N, double mean_c, const int32_t* order, const int32_t* tok_pos, int H, int hd,
                     const TokenTensor& ta, const TokenTensor& tb, const TokenTensor& tc, float scale_a, const float* bias, int n,
                     const int8_t* mask, int nmw, float* out, int32_t* row_ids, hipStream_t s, bool* fused_done) {
    const dim3 grid((unsigned)((gt.G + FUSED_GROUPS_PER_WG - 1) / FUSED_GROUPS_PER_WG),
                    block_task_slices(mean_c, hd, true, FUSED_GROUPS_PER_WG));
    uint32_t a_span, b_span, c_span = 0;
    const bool fit_a = rows_fit_descriptor<T>(ta, N, hd, &a_span), fit_b = rows_fit_descriptor<T>(tb, N, hd, &b_span);
    const bool fit_c = epi != SQ_SCORE_GRAD || rows_fit_descriptor<T>(tc, N, hd, &c_span);
    if (fused_done) *fused_done = true;
    if (fit_a && fit_b && fit_c) {
        if (epi == SQ_SCORES)
            hipLaunchKernelGGL((fused_sq_kernel<T, SQ_SCORES>), grid, dim3(256), 0, s, gt, order, tok_pos, H, hd, ta,
                               tb, tc, a_span, b_span, c_span, scale_a, bias, n, mask, nmw, out, row_ids);
        else if (epi == SQ_SCORE_GRAD)
            hipLaunchKernelGGL((fused_sq_kernel<T, SQ_SCORE_GRAD>), grid, dim3(256), 0, s, gt, order, tok_pos, H, hd, ta,
                               tb, tc, a_span, b_span, c_span, scale_a, bias, n, mask, nmw, out, row_ids);
        else
            hipLaunchKernelGGL((fused_sq_kernel<T, SQ_PLAIN>), grid, dim3(256), 0, s, gt, order, tok_pos, H, hd, ta,
                               tb, tc, a_span, b_span, c_span, scale_a, bias, n, mask, nmw, out, row_ids);
    } else if (epi == SQ_SCORES) {
        hipLaunchKernelGGL((fused_sq_wide_kernel<T, true>), grid, dim3(256), 0, s, gt, order, tok_pos, H, hd, ta,
                           tb, scale_a, bias, n, mask, nmw, out, row_ids);
    } else {
        if (fused_done) *fused_done = epi != SQ_SCORE_GRAD;
        hipLaunchKernelGGL((fused_sq_wide_kernel<T, false>), grid, dim3(256), 0, s, gt, order, tok_pos, H, hd, ta,
                           tb, scale_a, nullptr, n, nullptr, 0, out, nullptr);
    }
    return launch_ok("fused tokens->sq product");
}

template <typename T>
static int launch_tok(bool a_kmajor, const FusedGroups& gt, int64_t N, double mean_c, const int32_t* order, int hd, const float* sq,
                      const TokenTensor& tb, const TokenTensor& to, float scale_out, hipStream_t s) {
    const dim3 grid((unsigned)((gt.G + FUSED_GROUPS_PER_WG - 1) / FUSED_GROUPS_PER_WG),
                    block_task_slices(mean_c, hd, false, FUSED_GROUPS_PER_WG));
    uint32_t b_span, o_span;
    const bool fit_b = rows_fit_descriptor<T>(tb, N, hd, &b_span), fit_o = rows_fit_descriptor<T>(to, N, hd, &o_span);
    if (fit_b && fit_o) {
        if (a_kmajor)
            hipLaunchKernelGGL((fused_tok_kernel<T, true>), grid, dim3(256), 0, s, gt, order, hd, sq, tb, to, b_span,
                               o_span, scale_out);
        else
            hipLaunchKernelGGL((fused_tok_kernel<T, false>), grid, dim3(256), 0, s, gt, order, hd, sq, tb, to, b_span,
                               o_span, scale_out);
    } else if (a_kmajor) {
        hipLaunchKernelGGL((fused_tok_wide_kernel<T, true>), grid, dim3(256), 0, s, gt, order, hd, sq, tb, to,
                           scale_out);
    } else {
        hipLaunchKernelGGL((fused_tok_wide_kernel<T, false>), grid, dim3(256), 0, s, gt, order, hd, sq, tb, to,
                           scale_out);
    }
    return launch_ok("fused sq->tokens product");
}

static FusedGroups groups_of(const int32_t* plan, int64_t g_cap, int64_t G) {
    return FusedGroups{plan, plan + g_cap, plan + 2 * g_cap, plan + 3 * g_cap, plan + 4 * g_cap, G};
}

}  // namespace sswin

using namespace sswin;

extern "C" {

static int tp_words_per_window(int n) { return (n + 31) / 32; }
static int64_t tp_blocks(int B) { return ((int64_t)B + TP_BLOCK - 1) / TP_BLOCK; }

size_t sswin_token_plan_workspace_bytes(int64_t N, int B, int n) {
    (void)N;
    const size_t words = (size_t)B * tp_words_per_window(n);
    const size_t blocks = (size_t)tp_blocks(B);
    return align_up(words * 4, 256) + 2 * align_up((size_t)B * 4, 256) + align_up(blocks * 32, 256) +
           align_up(blocks * 4, 256) + 1024;
}

// `tasks` holds the group descriptors [4][g_cap] (int4) and, behind them, the token records [rec_cap][32] (int2)
static int64_t tp_rec_cap(int64_t N, int64_t g_cap, int H) { return N / 32 + g_cap / H + 4; }
size_t sswin_token_plan_task_ints(int64_t N, int64_t g_cap, int H) {
    if (N < 0 || g_cap <= 0 || H <= 0) return 0;
    return (size_t)(16 * g_cap + 64 * tp_rec_cap(N, g_cap, H));
}

// Checks one plan's arguments and carves its workspace; `a` is ready to launch afterwards.
static int token_plan_args(const int32_t* indices, int64_t N, int B, int n, int H, int32_t* tokens, int32_t* plan,
                           int64_t g_cap, int32_t* tasks, int64_t* totals_out, void* ws, size_t ws_bytes, int flags,
                           TokenPlanArgs& a) {
    SSWIN_CHECK((flags & ~SSWIN_PLAN_ORDER_ONLY) == 0, "token_plan: unknown flags %d", flags);
    a.order_only = (flags & SSWIN_PLAN_ORDER_ONLY) ? 1 : 0;
    SSWIN_CHECK(N > 0 && B > 0 && n > 0 && H > 0 && H < 256, "token_plan: bad sizes");
    SSWIN_CHECK(indices && tokens && plan && ws && totals_out, "token_plan: null pointer");
    SSWIN_CHECK(N < (int64_t)INT32_MAX, "token_plan: too many voxels");
    SSWIN_CHECK(g_cap > 0, "token_plan: g_cap must be positive");
    SSWIN_CHECK(ws_bytes >= sswin_token_plan_workspace_bytes(N, B, n), "token_plan: workspace too small");
    Carver cv(ws, ws_bytes);
    a.ind = indices;
    a.N = N;
    a.B = B;
    a.n = n;
    a.W = tp_words_per_window(n);
    a.H = H;
    const size_t words = (size_t)B * a.W;
    const int64_t blocks = tp_blocks(B);
    a.blocks = (int)blocks;
    a.totals = cv.take<int64_t>(8);       // [0] windows, [1] sum c | sum c*c << 32, [2..7] counters
    a.bits = cv.take<uint32_t>(words);
    a.win_T = cv.take<int32_t>((size_t)B);
    a.win_rec = cv.take<int32_t>((size_t)B);
    a.partial_a = cv.take<int64_t>(4 * (size_t)blocks);
    a.partial_b = cv.take<int32_t>((size_t)blocks);
    SSWIN_CHECK(cv.ok(), "token_plan: workspace too small");
    a.plan = plan;
    a.g_cap = g_cap;
    a.tasks = reinterpret_cast<int4*>(tasks);
    a.recs = tasks && !a.order_only ? reinterpret_cast<int2*>(tasks + 16 * g_cap) : nullptr;
    a.rec_cap = tp_rec_cap(N, g_cap, H);
    a.tokens = tokens;
    return 0;
}

// The five launches for `count` plans (1..TP_MAX_BATCH) and the copies of their raw totals to the host.
static int token_plan_launch(const TokenPlanArgs* args, int64_t* const* totals_out, int count, hipStream_t s) {
    TokenPlanBatch b;
    size_t words = 0;
    int64_t voxels = 0;
    int blocks = 0;
    for (int k = 0; k < TP_MAX_BATCH; ++k) {
        b.p[k] = args[k < count ? k : 0];  // unused slots repeat the first plan; no block ever reads them
        if (k >= count) continue;
        words = std::max(words, (size_t)args[k].B * args[k].W);
        voxels = std::max(voxels, args[k].N);
        blocks = std::max(blocks, args[k].blocks);
    }
    // all plans of a launch share the slots per thread: four as soon as one of them has that many window slots
    int64_t slots = 0;
    for (int k = 0; k < count; ++k) slots = std::max<int64_t>(slots, args[k].B);
    const int items = slots >= TP_WIDE_FROM ? TP_ITEMS_WIDE : 1;
    blocks = 0;
    for (int k = 0; k < TP_MAX_BATCH; ++k) {
        b.p[k].blocks = (int)(((int64_t)b.p[k].B + TP_BLOCK * items - 1) / (TP_BLOCK * items));
        if (k < count) blocks = std::max(blocks, b.p[k].blocks);
    }
    const unsigned y = (unsigned)count;
    const unsigned clear_blocks = (unsigned)std::min<size_t>((words + 255) / 256, 2048);
    const unsigned nb = (unsigned)std::min<int64_t>((voxels + 255) / 256, 1 << 20);
    hipLaunchKernelGGL(tp_clear_kernel, dim3(clear_blocks, y), dim3(256), 0, s, b);
    hipLaunchKernelGGL(tp_set_bits_kernel, dim3(nb, y), dim3(256), 0, s, b);
    if (items == TP_ITEMS_WIDE) {
        hipLaunchKernelGGL(tp_block_sums_kernel<TP_ITEMS_WIDE>, dim3((unsigned)blocks, y), dim3(TP_BLOCK), 0, s, b);
        hipLaunchKernelGGL(tp_windows_kernel<TP_ITEMS_WIDE>, dim3((unsigned)blocks, y), dim3(TP_BLOCK), 0, s, b);
    } else {
        hipLaunchKernelGGL(tp_block_sums_kernel<1>, dim3((unsigned)blocks, y), dim3(TP_BLOCK), 0, s, b);
        hipLaunchKernelGGL(tp_windows_kernel<1>, dim3((unsigned)blocks, y), dim3(TP_BLOCK), 0, s, b);
    }
    hipLaunchKernelGGL(tp_rank_kernel, dim3(nb, y), dim3(256), 0, s, b);
    if (launch_ok("token plan")) return 1;
    // raw totals: the caller decodes them with sswin_token_plan_totals once the copies have landed
    for (int k = 0; k < count; ++k)
        SSWIN_HIP(hipMemcpyAsync(totals_out[k], args[k].totals, 8 * sizeof(int64_t), hipMemcpyDeviceToHost, s));
    return 0;
}

int sswin_token_plan(const int32_t* indices, int64_t N, int B, int n, int H, int32_t* tokens,
                     int32_t* plan, int64_t g_cap, int32_t* tasks, int64_t* totals_out, void* ws,
                     size_t ws_bytes, int synchronize, void* stream) {
    SSWIN_CHECK(N >= 0 && B > 0 && n > 0 && H > 0 && H < 256, "token_plan: bad sizes");
    SSWIN_CHECK(totals_out, "token_plan: totals_out is null");
    for (int i = 0; i < 9; ++i) totals_out[i] = 0;
    if (N == 0) return 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    TokenPlanArgs a;
    if (token_plan_args(indices, N, B, n, H, tokens, plan, g_cap, tasks, totals_out, ws, ws_bytes, 0, a)) return 1;
    totals_out[8] = N;                     // read back by sswin_token_plan_totals (the copy fills [0..7])
    if (token_plan_launch(&a, &totals_out, 1, s)) return 1;
    if (!synchronize) return 0;
    SSWIN_HIP(hipStreamSynchronize(s));
    return sswin_token_plan_totals(totals_out, H, g_cap);
}

int sswin_token_plan_batch(const sswin_token_plan_desc* descs, int count, void* stream) {
    SSWIN_CHECK(count >= 0 && count <= TP_MAX_BATCH, "token_plan_batch: between 0 and %d plans per call", TP_MAX_BATCH);
    SSWIN_CHECK(count == 0 || descs, "token_plan_batch: descs is null");
    TokenPlanArgs args[TP_MAX_BATCH];
    int64_t* totals[TP_MAX_BATCH];
    int live = 0;
    for (int k = 0; k < count; ++k) {
        const sswin_token_plan_desc& d = descs[k];
        SSWIN_CHECK(d.N >= 0 && d.B > 0 && d.n > 0 && d.H > 0 && d.H < 256, "token_plan_batch: bad sizes in plan %d", k);
        SSWIN_CHECK(d.totals_out, "token_plan_batch: totals_out of plan %d is null", k);
        for (int i = 0; i < 9; ++i) d.totals_out[i] = 0;
        if (d.N == 0) continue;            // an empty plan: all totals zero, nothing to launch
        if (token_plan_args(d.indices, d.N, d.B, d.n, d.H, d.tokens, d.plan, d.g_cap, d.tasks, d.totals_out, d.ws,
                            d.ws_bytes, d.flags, args[live]))
            return 1;
        d.totals_out[8] = d.N;
        totals[live++] = d.totals_out;
    }
    if (live == 0) return 0;
    return token_plan_launch(args, totals, live, static_cast<hipStream_t>(stream));
}

int sswin_token_plan_totals(int64_t* totals, int H, int64_t g_cap) {
    SSWIN_CHECK(totals && H > 0, "token_plan_totals: bad arguments");
    int64_t raw[9];
    memcpy(raw, totals, sizeof(raw));
    int32_t counters[12];
    memcpy(counters, raw + 2, sizeof(counters));
    const int64_t windows = raw[0];
    const int64_t s2 = raw[1] >> 32;
    const int64_t distinct = raw[1] & 0xffffffffll;
    const int64_t N = raw[8];
    SSWIN_CHECK(counters[TPC_RANGE] == 0,
                "token_plan: %d voxel indices lie outside [0, batch_size) x [0, positions per window)", counters[TPC_RANGE]);
    SSWIN_CHECK(distinct == N, "token_plan: (window, pos) pairs must be distinct: %lld voxels share a pair with another",
                (long long)(N - distinct));
    SSWIN_CHECK(raw[1] >= 0 && s2 * H < (int64_t)INT32_MAX,
                "token_plan: the attention matrix has 2^31 or more non-zeros, which int32 offsets cannot address");
    SSWIN_CHECK(windows * H <= g_cap, "token_plan: %lld groups exceed the plan capacity %lld",
                (long long)(windows * H), (long long)g_cap);
    totals[0] = windows * H;
    totals[1] = windows;
    totals[2] = s2 * H;
    totals[3] = counters[TPC_CMAX];
    for (int b = 0; b < 5; ++b) totals[4 + b] = counters[b];
    return 0;
}

int sswin_fused_tokens_to_sq(int dtype, int epilogue, const int32_t* plan, int64_t g_cap, int64_t G,
                             const int32_t* tokens, int64_t N, int H, int hd, const void* a_base,
                             int64_t a_stride, int a_col0, const void* b_base, int64_t b_stride, int b_col0,
                             float scale_a, const float* bias, int n, const int8_t* mask, int n_mask_windows,
                             float* out, int32_t* row_ids, void* stream) {
    SSWIN_CHECK(G >= 0 && G <= g_cap && N >= 0 && H > 0 && hd > 0, "fused_tokens_to_sq: bad sizes");
    if (G == 0) return 0;
    SSWIN_CHECK(plan && tokens && a_base && b_base && out, "fused_tokens_to_sq: null pointer");
    SSWIN_CHECK(!epilogue || (bias && n > 0), "fused_tokens_to_sq: the epilogue needs the bias table");
    SSWIN_CHECK(!mask || n_mask_windows > 0, "fused_tokens_to_sq: mask without window count");
    const FusedGroups gt = groups_of(plan, g_cap, G);
    const TokenTensor ta{a_base, a_stride, a_col0}, tb{b_base, b_stride, b_col0};
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int32_t* order = tokens;
    const int32_t* tok_pos = tokens + 3 * N;
    const double mean_c = (double)N * H / (double)G;          // every voxel is a token of one window, in each of its H groups
    switch (dtype) {
        case SSWIN_F32: return launch_sq<float>(epilogue ? SQ_SCORES : SQ_PLAIN, gt, N, mean_c, order, tok_pos, H, hd, ta, tb, ta, scale_a, bias, n, mask, n_mask_windows, out, row_ids, s, nullptr);
        case SSWIN_F16: return launch_sq<__half>(epilogue ? SQ_SCORES : SQ_PLAIN, gt, N, mean_c, order, tok_pos, H, hd, ta, tb, ta, scale_a, bias, n, mask, n_mask_windows, out, row_ids, s, nullptr);
        case SSWIN_BF16: return launch_sq<__hip_bfloat16>(epilogue ? SQ_SCORES : SQ_PLAIN, gt, N, mean_c, order, tok_pos, H, hd, ta, tb, ta, scale_a, bias, n, mask, n_mask_windows, out, row_ids, s, nullptr);
        default: return fail("fused_tokens_to_sq: unsupported token dtype %d", dtype);
    }
}

int sswin_fused_sq_to_tokens(int dtype, int a_kmajor, const int32_t* plan, int64_t g_cap, int64_t G,
                             const int32_t* tokens, int64_t N, int H, int hd, const float* sq, const void* b_base,
                             int64_t b_stride, int b_col0, void* o_base, int64_t o_stride, int o_col0,
                             float scale_out, void* stream) {
    SSWIN_CHECK(G >= 0 && G <= g_cap && N >= 0 && H > 0 && hd > 0, "fused_sq_to_tokens: bad sizes");
    if (G == 0) return 0;
    SSWIN_CHECK(plan && tokens && sq && b_base && o_base, "fused_sq_to_tokens: null pointer");
    const FusedGroups gt = groups_of(plan, g_cap, G);
    const TokenTensor tb{b_base, b_stride, b_col0}, to{o_base, o_stride, o_col0};
    hipStream_t s = static_cast<hipStream_t>(stream);
    const double mean_c = (double)N * H / (double)G;
    switch (dtype) {
        case SSWIN_F32: return launch_tok<float>(a_kmajor, gt, N, mean_c, tokens, hd, sq, tb, to, scale_out, s);
        case SSWIN_F16: return launch_tok<__half>(a_kmajor, gt, N, mean_c, tokens, hd, sq, tb, to, scale_out, s);
        case SSWIN_BF16: return launch_tok<__hip_bfloat16>(a_kmajor, gt, N, mean_c, tokens, hd, sq, tb, to, scale_out, s);
        default: return fail("fused_sq_to_tokens: unsupported token dtype %d", dtype);
    }
}

int sswin_group_softmax(int backward, const int32_t* plan, int64_t g_cap, int64_t G, int64_t N, int H, int c_max,
                        const float* x_or_y, const float* grad, float* out, void* stream) {
    SSWIN_CHECK(G >= 0 && G <= g_cap && N >= 0 && H > 0, "group_softmax: bad sizes");
    if (G == 0) return 0;
    SSWIN_CHECK(plan && x_or_y && out && (!backward || grad), "group_softmax: null pointer");
    SSWIN_CHECK(c_max > 0 && c_max <= 384, "group_softmax: windows of %d tokens are not supported (384 at most)", c_max);
    const FusedGroups gt = groups_of(plan, g_cap, G);
    const dim3 grid((unsigned)((G + FUSED_GROUPS_PER_WG - 1) / FUSED_GROUPS_PER_WG),
                    block_task_slices((double)N * H / (double)G, 1, false, FUSED_GROUPS_PER_WG));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (backward)
        hipLaunchKernelGGL((group_softmax_kernel<true>), grid, dim3(256), 0, s, gt, x_or_y, grad, out);
    else
        hipLaunchKernelGGL((group_softmax_kernel<false>), grid, dim3(256), 0, s, gt, x_or_y, grad, out);
    return launch_ok("group softmax");
}

int sswin_fused_score_grad(int dtype, const int32_t* plan, int64_t g_cap, int64_t G, const int32_t* tokens, int64_t N,
                           int H, int hd, int c_max, const void* do_base, int64_t do_stride, int do_col0,
                           const void* v_base, int64_t v_stride, int v_col0, const void* o_base, int64_t o_stride,
                           int o_col0, const float* p, float* ds, void* stream) {
    SSWIN_CHECK(G >= 0 && G <= g_cap && N >= 0 && H > 0 && hd > 0, "fused_score_grad: bad sizes");
    if (G == 0) return 0;
    SSWIN_CHECK(plan && tokens && do_base && v_base && o_base && p && ds, "fused_score_grad: null pointer");
    SSWIN_CHECK(c_max > 0 && c_max <= 384, "fused_score_grad: windows of %d tokens are not supported (384 at most)", c_max);
    const FusedGroups gt = groups_of(plan, g_cap, G);
    const TokenTensor ta{do_base, do_stride, do_col0}, tb{v_base, v_stride, v_col0}, tc{o_base, o_stride, o_col0};
    hipStream_t s = static_cast<hipStream_t>(stream);
    const double mean_c = (double)N * H / (double)G;
    bool done = false;
    int rc;
    switch (dtype) {
        case SSWIN_F32: rc = launch_sq<float>(SQ_SCORE_GRAD, gt, N, mean_c, tokens, tokens + 3 * N, H, hd, ta, tb, tc, 1.0f, p, 0, nullptr, 0, ds, nullptr, s, &done); break;
        case SSWIN_F16: rc = launch_sq<__half>(SQ_SCORE_GRAD, gt, N, mean_c, tokens, tokens + 3 * N, H, hd, ta, tb, tc, 1.0f, p, 0, nullptr, 0, ds, nullptr, s, &done); break;
        case SSWIN_BF16: rc = launch_sq<__hip_bfloat16>(SQ_SCORE_GRAD, gt, N, mean_c, tokens, tokens + 3 * N, H, hd, ta, tb, tc, 1.0f, p, 0, nullptr, 0, ds, nullptr, s, &done); break;
        default: return fail("fused_score_grad: unsupported token dtype %d", dtype);
    }
    if (rc != 0 || done) return rc;
    // token tensors beyond the reach of a buffer descriptor: ds holds dP now, the softmax backward runs over it in place
    return sswin_group_softmax(1, plan, g_cap, G, N, H, c_max, p, ds, ds, stream);
}

static int bias_grad_slices(int64_t windows, int H) {
    // about two 1024-thread workgroups per CU over all heads, at least eight windows per slice
    const int64_t want = std::max<int64_t>(1, 512 / std::max(H, 1));
    const int64_t useful = std::max<int64_t>(1, (windows + 7) / 8);
    return (int)std::min<int64_t>(want, useful);
}

size_t sswin_fused_bias_grad_workspace_bytes(int64_t G, int H, int n) {
    const int64_t windows = H > 0 ? G / H : 0;
    return (size_t)bias_grad_slices(windows, H) * H * n * n * sizeof(float) + 256;
}

int sswin_fused_bias_grad(const int32_t* plan, int64_t g_cap, int64_t G, const int32_t* tokens, int64_t N,
                          int H, int n, const float* ds, float* d_bias, void* ws, size_t ws_bytes,
                          void* stream) {
    SSWIN_CHECK(G >= 0 && G <= g_cap && H > 0 && n > 0, "fused_bias_grad: bad sizes");
    if (G == 0) return 0;
    SSWIN_CHECK(plan && tokens && ds && d_bias && ws, "fused_bias_grad: null pointer");
    SSWIN_CHECK((size_t)n * n * sizeof(float) <= 64 * 1024 && n <= 128,
                "fused_bias_grad: a window of %d positions needs a %zu-byte LDS table (limit 64 KiB, 128 positions)",
                n, (size_t)n * n * sizeof(float));
    SSWIN_CHECK(ws_bytes >= sswin_fused_bias_grad_workspace_bytes(G, H, n), "fused_bias_grad: workspace too small");
    const FusedGroups gt = groups_of(plan, g_cap, G);
    const int slices = bias_grad_slices(G / H, H);
    hipStream_t s = static_cast<hipStream_t>(stream);
    float* partial = static_cast<float*>(ws);
    hipLaunchKernelGGL(rpb_grad_partial_kernel, dim3((unsigned)slices, (unsigned)H), dim3(RPB_THREADS),
                       (size_t)n * n * sizeof(float), s, gt, tokens + 3 * N, H, n, ds, partial);
    const int64_t elems = (int64_t)H * n * n;
    hipLaunchKernelGGL(rpb_grad_reduce_kernel, dim3((unsigned)((elems + 255) / 256)), dim3(256), 0, s, partial, slices,
                       elems, d_bias);
    return launch_ok("fused bias gradient");
}

// slices = window slices x wavefronts per window slice.  About 3072 wavefronts (three per SIMD: what a
// wavefront waits for is its own chain of LDS read-add-writes, so a few of them share a SIMD well), eight per
// window slice: the batches of a crowded window (up to 3 x 3 of them for 89 tokens) spread over all eight.
// Measured on cfg2 (the two launches): 2048 wavefronts / 4 per slice 0.038 ms, 3072 / 8 0.036, 4096 / 8 0.040.
// A table of more than 1 664 rows (windows of 7^3 positions: 2 197) leaves room for two workgroups per compute unit
// only, a larger one for one: the launch then holds 2 048 or 1 024 wavefronts, so that all of them are resident at once
// (3 072 wavefronts on two workgroups per unit ran as one full round and a half-empty second one).
static size_t table_grad_lds(int table_rows, int n) {
    const int rows_pad = (table_rows + 31) / 32 * 32 + 32;  // 32 spare rows
    return (size_t)8 * rows_pad * sizeof(float) + (size_t)n * sizeof(int32_t);
}
static void table_grad_slices(int64_t windows, int H, int table_rows, int* wslices, int* rsplit) {
    constexpr int64_t PER_SLICE = 8;
    const int64_t resident = std::max<int64_t>(1, std::min<int64_t>(3, (int64_t)(160 * 1024) / (int64_t)table_grad_lds(table_rows, 384)));
    const int64_t WAVES = 1024 * resident;
    const int64_t want = std::max<int64_t>(1, WAVES / (std::max(H, 1) * PER_SLICE));
    *wslices = (int)std::min<int64_t>(want, std::max<int64_t>(1, windows));
    *rsplit = (int)PER_SLICE;
}

size_t sswin_bias_table_grad_workspace_bytes(int64_t G, int H, int table_rows) {
    const int64_t windows = H > 0 ? G / H : 0;
    int wslices, rsplit;
    table_grad_slices(windows, H, table_rows, &wslices, &rsplit);
    return (size_t)wslices * rsplit * H * table_rows * sizeof(float) + 256;
}

// the two launches of the table gradient; bl == nullptr: batches from the group table
static int launch_table_grad(const FusedGroups& gt, const BatchList* bl, int64_t G, const int32_t* tokens, int64_t N, int H, int n,
                             const int32_t* code, int offset0, int table_rows, const float* ds, float* d_table, void* ws,
                             size_t ws_bytes, hipStream_t s) {
    SSWIN_CHECK(ws_bytes >= sswin_bias_table_grad_workspace_bytes(G, H, table_rows), "bias_table_grad: workspace too small");
    const int64_t windows = G / H;
    int wslices, rsplit;
    table_grad_slices(windows, H, table_rows, &wslices, &rsplit);
    if (bl) {
        // dealt batches: a wavefront should have about six of them before it is worth its table (small inputs: 22 000
        // voxels 18.5 -> 15 us with half the wavefronts; more wavefronts than the walking kernel's never paid)
        const int per_head = (int)std::max<int64_t>(32, std::min<int64_t>((int64_t)wslices * rsplit, bl->total / 6));
        wslices = (per_head + 3) / 4 * 4;                          // whole workgroups per head
        rsplit = 1;
    }
    const int slices = wslices * rsplit;
    float* partial = static_cast<float*>(ws);
    const int64_t waves = (int64_t)slices * H;
    const int rows_pad = (table_rows + 31) / 32 * 32 + 32;  // 32 spare rows
    const size_t lds = table_grad_lds(table_rows, n);
    SSWIN_CHECK(lds <= 160 * 1024, "bias_table_grad: a table of %d rows needs %zu bytes of LDS (160 KB at most)", table_rows, lds);
    if (lds > 64 * 1024) {
        // more than the default 64 KB of dynamic LDS: asked for with every such launch (cheap, and correct for any
        // number of host threads and devices)
        const void* fn = bl ? reinterpret_cast<const void*>(rpb_table_partial_kernel<true>)
                            : reinterpret_cast<const void*>(rpb_table_partial_kernel<false>);
        const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        SSWIN_CHECK(e == hipSuccess, "bias_table_grad: the request for %zu bytes of LDS per workgroup was refused: %s", lds,
                    hipGetErrorString(e));
    }
    const dim3 grid((unsigned)((waves + 3) / 4));
    if (bl)
        hipLaunchKernelGGL(rpb_table_partial_kernel<true>, grid, dim3(256), lds, s, gt, *bl, tokens + 3 * N, H,
                           code, n, offset0, table_rows, rows_pad, ds, windows, wslices, rsplit, partial);
    else
        hipLaunchKernelGGL(rpb_table_partial_kernel<false>, grid, dim3(256), lds, s, gt, BatchList{}, tokens + 3 * N, H,
                           code, n, offset0, table_rows, rows_pad, ds, windows, wslices, rsplit, partial);
    hipLaunchKernelGGL(rpb_table_reduce_kernel, dim3((unsigned)((table_rows + 15) / 16), (unsigned)H), dim3(1024), 0, s,
                       partial, slices / 4, table_rows, H, d_table);
    return launch_ok("bias table gradient");
}

int sswin_bias_table_grad(const int32_t* plan, int64_t g_cap, int64_t G, const int32_t* tokens, int64_t N, int H,
                          int n, const int32_t* code, int offset0, int table_rows, const float* ds, float* d_table,
                          void* ws, size_t ws_bytes, void* stream) {
    SSWIN_CHECK(G >= 0 && G <= g_cap && H > 0 && n > 0, "bias_table_grad: bad sizes");
    SSWIN_CHECK(n <= 384, "bias_table_grad: windows of %d positions are not supported (384 at most)", n);
    SSWIN_CHECK(table_rows > 0 && table_rows <= RPBT_MAX_ROWS, "bias_table_grad: a table of %d rows is not supported (%d at most)",
                table_rows, RPBT_MAX_ROWS);
    SSWIN_CHECK(d_table, "bias_table_grad: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (G == 0) {
        zero_fill(d_table, (int64_t)table_rows * H, s);
        return launch_ok("bias_table_grad");
    }
    SSWIN_CHECK(plan && tokens && code && ds && ws, "bias_table_grad: null pointer");
    return launch_table_grad(groups_of(plan, g_cap, G), nullptr, G, tokens, N, H, n, code, offset0, table_rows, ds, d_table, ws,
                             ws_bytes, s);
}

int sswin_bias_table_grad_tasks(const int32_t* tasks, int64_t g_cap, const int64_t* bucket_counts, int64_t G,
                                const int32_t* tokens, int64_t N, int H, int n, const int32_t* code, int offset0,
                                int table_rows, const float* ds, float* d_table, void* ws, size_t ws_bytes, void* stream) {
    SSWIN_CHECK(G >= 0 && G <= g_cap && H > 0 && n > 0 && n <= 128, "bias_table_grad_tasks: bad sizes");
    SSWIN_CHECK(table_rows > 0 && table_rows <= RPBT_MAX_ROWS, "bias_table_grad_tasks: a table of %d rows is not supported (%d at most)",
                table_rows, RPBT_MAX_ROWS);
    SSWIN_CHECK(d_table && bucket_counts, "bias_table_grad_tasks: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (G == 0) {
        zero_fill(d_table, (int64_t)table_rows * H, s);
        return launch_ok("bias_table_grad_tasks");
    }
    SSWIN_CHECK(tasks && tokens && code && ds && ws, "bias_table_grad_tasks: null pointer");
    int64_t groups = 0;
    for (int b = 0; b < 4; ++b) {
        SSWIN_CHECK(bucket_counts[b] >= 0 && bucket_counts[b] % H == 0, "bias_table_grad_tasks: bucket %d holds %lld groups, not a multiple of the %d heads",
                    b, (long long)bucket_counts[b], H);
        groups += bucket_counts[b];
    }
    SSWIN_CHECK(groups == G, "bias_table_grad_tasks: the buckets hold %lld groups, the plan %lld (windows of more than 128 tokens have no descriptor)",
                (long long)groups, (long long)G);
    BatchList bl;
    bl.tasks = reinterpret_cast<const int4*>(tasks);
    bl.g_cap = g_cap;
    int64_t at = 0;
    for (int b = 3; b >= 0; --b) {
        bl.first[b] = (int)at;
        at += bucket_counts[b] / H * (b + 1) * (b + 1);
    }
    SSWIN_CHECK(at < ((int64_t)1 << 31), "bias_table_grad_tasks: too many batches");
    bl.total = (int)at;
    // the group table is not read on this path: only its size G matters
    const FusedGroups gt{nullptr, nullptr, nullptr, nullptr, nullptr, G};
    return launch_table_grad(gt, &bl, G, tokens, N, H, n, code, offset0, table_rows, ds, d_table, ws, ws_bytes, s);
}

int sswin_bias_from_table(const float* table, int table_rows, int H, const int32_t* code, int offset0, int n, float* bias,
                          void* stream) {
    SSWIN_CHECK(table_rows > 0 && H > 0 && n > 0 && n <= 4096, "bias_from_table: bad sizes");
    SSWIN_CHECK(table && code && bias, "bias_from_table: null pointer");
    hipLaunchKernelGGL(rpb_gather_kernel, dim3((unsigned)((n * n + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       table, table_rows, H, code, offset0, n, bias);
    return launch_ok("bias_from_table");
}

}  // extern "C"
