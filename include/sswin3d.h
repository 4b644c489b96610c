/*
 * sswin3d — C ABI of the MI355X (gfx950) sparse window-attention operator library.
 *
 * Plain pointers and sizes only: every pointer marked "device" is a HIP device address,
 * every other pointer is host memory.  `stream` is a hipStream_t passed as void*.
 * No function allocates or frees device memory: scratch space is passed in by the caller
 * (`ws`, `ws_bytes`, sized by the matching *_workspace_bytes query).  All kernels are
 * enqueued on `stream`; functions that return a size to the host (documented below)
 * synchronise that stream once, everything else is asynchronous.
 *
 * Return value: 0 on success, non-zero on error; sswin_last_error() then holds a message
 * (thread-local).  Errors are argument errors detected on the host before any launch.
 *
 * Each entry point replaces one operator of the reference's pybind module `custom_ops`
 * (sparse_swin/ops.cpp:7-18, declarations sparse_swin/ops.h:4-50); the citation beside
 * each declaration is the reference function it stands in for.
 */
#ifndef SSWIN3D_H
#define SSWIN3D_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* value dtypes */
enum { SSWIN_F32 = 0, SSWIN_F16 = 1, SSWIN_BF16 = 2, SSWIN_F64 = 3 };
/* key dtypes of sswin_unique_consecutive_indices */
enum { SSWIN_I32 = 0, SSWIN_I64 = 1, SSWIN_I16 = 2, SSWIN_I8 = 3, SSWIN_U8 = 4 };
/* block product kinds */
enum { SSWIN_MUL_Q_K = 0, SSWIN_MUL_QK_V = 1 };
enum { SSWIN_GRAD_RC_CR = 0, SSWIN_GRAD_RR_RC = 1, SSWIN_GRAD_CR_RR = 2, SSWIN_GRAD_TR_RC = 3, SSWIN_GRAD_TC_RR = 4 };
enum { SSWIN_TRANSPOSE_RC = 0, SSWIN_TRANSPOSE_RR = 1 };

const char* sswin_last_error(void);
/* library ABI version, bumped on any signature change */
int sswin_abi_version(void);

/* A plain copy of `bytes` bytes (a multiple of 16; src, dst: device, 16-byte aligned, not overlapping): every
 * byte is read once and written once.  It has no counterpart in the reference: a profiling run launches it
 * beside the kernels it measures, and what the memory counters read for this known traffic gives their unit. */
int sswin_calibration_copy(void* dst, const void* src, int64_t bytes, void* stream);

/* ---- index operators -------------------------------------------------------------- */

/* flatten_indices (sparse_swin/ops.cu:232-273, ops.h:38): wrapping int32 row-major hash of a
 * contiguous [ndim, M] int32 index matrix; strides come from sizes[1:]. ndim <= 8.
 * idx, out: device.  sizes: host, ndim entries. */
int sswin_flatten_indices(const int32_t* idx, int ndim, int64_t M, const int32_t* sizes,
                          int32_t* out, void* stream);

/* sort_indices (sparse_swin/ops.cu:276-289, ops.h:39): stable ascending argsort of signed
 * int32 keys.  keys, perm_out, ws: device. */
size_t sswin_sort_indices_workspace_bytes(int64_t M);
int sswin_sort_indices(const int32_t* keys, int64_t M, int32_t* perm_out, void* ws,
                       size_t ws_bytes, void* stream);

/* unique_consecutive_indices (sparse_swin/ops.cu:32-103, ops.h:41): 0-based rank of the run
 * of equal consecutive keys each element belongs to.  keys, out, ws: device. */
size_t sswin_unique_consecutive_workspace_bytes(int64_t M);
int sswin_unique_consecutive_indices(const void* keys, int key_dtype, int64_t M, int32_t* out,
                                     void* ws, size_t ws_bytes, void* stream);

/* The same operator for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference:
 * it is sswin_unique_consecutive_indices with the scan's tile sums kept in a 256 KiB device array
 * built into the library (one copy per GPU, held until the process ends) instead of a caller
 * workspace.  The caller still passes keys and out.  M may not exceed
 * SSWIN_UNIQUE_CONSECUTIVE_STATIC_MAX keys (error otherwise).  Calls no hipMalloc / hipFree.
 * All calls on one GPU share that array: calls that overlap on one GPU (two streams, two threads)
 * race; nothing has to be cleared between calls.  Asynchronous. */
#define SSWIN_UNIQUE_CONSECUTIVE_STATIC_MAX 134217728LL
int sswin_unique_consecutive_indices_static(const void* keys, int key_dtype, int64_t M, int32_t* out,
                                            void* stream);

/* return_inverse (sparse_swin/ops.cu:718-730, ops.h:40): rank of x[i] among the distinct
 * values of x, and the number of distinct values.  maxnum = -1 means max(x)+1 (costs one
 * extra stream synchronisation).  Values of x must lie in [0, maxnum): others set no bit, get
 * rank -1, and are reported as an error when count_out is delivered.
 * x, out, ws: device.  count_out: host.  Synchronises `stream` to deliver count_out;
 * pass count_out = NULL to stay asynchronous (only possible with maxnum >= 0).
 * workspace query: pass the same maxnum you will pass to the call, or, for maxnum = -1,
 * an upper bound of max(x)+1. */
size_t sswin_return_inverse_workspace_bytes(int64_t M, int64_t maxnum_bound);
int sswin_return_inverse(const int32_t* x, int64_t M, int64_t maxnum, int32_t* out,
                         int64_t* count_out, void* ws, size_t ws_bytes, void* stream);

/* qkv_sparse_indices (sparse_swin/ops.cu:206-227, 293-335, ops.h:23-28): from [N,2]
 * (window, pos) voxel indices build the element-level COO indices of Q/V ([4,E], rows
 * window, head, pos, channel) and of K^T ([4,E], rows window, head, channel, pos) in input
 * voxel order, and the permutations that sort their row-major hashes (shapes
 * {B,H,n,hd} and {B,H,hd,n}).  E = N*H*hd.  (window, pos) pairs must be distinct,
 * window in [0,B), pos in [0,n).  The ordering is that of the exact (non-wrapping) hash.
 * Pairs outside that range, or a pair that occurs twice, never turn into a device address: the
 * kernels that would use them fill sorted_qv / sorted_k with zeros instead.  validate != 0 waits for the
 * stream and reports such input as an error; validate == 0 stays asynchronous, and status_out (pinned host
 * int32 [2], or NULL) then receives {pairs out of range, distinct pairs} once the stream has run: the input
 * was valid iff status_out[0] == 0 and status_out[1] == N.
 * All array arguments: device. */
size_t sswin_qkv_sparse_indices_workspace_bytes(int64_t N, int B, int n);
int sswin_qkv_sparse_indices(const int32_t* indices, int64_t N, int B, int n, int H, int hd,
                             int32_t* idx_qv, int32_t* sorted_qv, int32_t* idx_k,
                             int32_t* sorted_k, void* ws, size_t ws_bytes, int validate, int32_t* status_out,
                             void* stream);

/* ---- sorted operands without the permutations ------------------------------------------------
 * qkv_sparse_cuda (sparse_swin/swin3d_base.py:483-498) gathers the index matrices and the values of
 * Q, K^T, V through the two permutations of qkv_sparse_indices, and autograd sends the gradients back
 * through index_add; the tail of WindowAttention.forward (:672-675) un-sorts the output through another
 * hash, sort and gather.  All of these are fixed permutations of the N*H*hd values, known from the rank
 * of every voxel in (window, pos) order.  The three calls below produce the same tensors directly.
 *
 * sswin_operand_map: map (device int32 [3N + 2]) = voxel of rank r, rank T of the first token of its window,
 *   tokens c of its window (each [N], by rank), then {pairs out of range, distinct pairs}.  validate /
 *   status_out as in sswin_qkv_sparse_indices; with invalid pairs the calls below copy nothing.
 * sswin_operand_copy: layout 0 (Q, V, attention output): val[hd*(H*T + h*c + i) + ch], layout 1 (K^T):
 *   val[hd*(H*T + h*c) + ch*c + i]  <->  vox[voxel * vox_stride + vox_col0 + h*hd + ch] (strides in values);
 *   to_operand != 0 copies voxel rows into the operand, 0 copies the operand into voxel rows.  Each direction is
 *   the gradient of the other.  dtype: any value dtype.  scale != 1 (layout 0 only): every copied value is multiplied
 *   by it on the way, in the accumulation type of dtype and rounded once (the `q * self.scale` of
 *   sparse_swin/swin3d_base.py:660 and, with to_operand == 0, its gradient) instead of a pass of its own.
 * sswin_sorted_coo_indices: the [4, E] index matrices of Q/V and of K^T in sorted order (either may be NULL),
 *   equal to idx.index_select(1, sorted) of sswin_qkv_sparse_indices.
 * All asynchronous unless validate != 0. */
size_t sswin_operand_map_workspace_bytes(int64_t N, int B, int n);
int sswin_operand_map(const int32_t* indices, int64_t N, int B, int n, int32_t* map, void* ws, size_t ws_bytes,
                      int validate, int32_t* status_out, void* stream);
int sswin_operand_copy(int dtype, int layout, int to_operand, void* vox, int64_t vox_stride, int vox_col0, void* val,
                       const int32_t* map, int64_t N, int H, int hd, double scale, void* stream);
/* The three copies of one attention call in one launch: vox is a [N, 3, H, hd] projection output (Q, K, V slices of a
 * voxel row H*hd values apart, Q at vox_col0); Q goes to / comes from val_q in Q/V order times q_scale, K val_k in K^T
 * order, V val_v in Q/V order (the gathers of sparse_swin/swin3d_base.py:492-498 and `q * self.scale`, :660; with
 * to_operand == 0 their gradients). */
int sswin_operand_copy_qkv(int dtype, int to_operand, void* vox, int64_t vox_stride, int vox_col0, void* val_q, void* val_k,
                           void* val_v, const int32_t* map, int64_t N, int H, int hd, double q_scale, void* stream);
int sswin_sorted_coo_indices(const int32_t* indices, const int32_t* map, int64_t N, int H, int hd, int32_t* idx_qv,
                             int32_t* idx_k, void* stream);

/* ---- per-group offsets ("plan") ----------------------------------------------------- */

/* Group structure of a coalesced 4-D COO operand whose last dimension is dense
 * (sparse_swin/ops.cu:781-784, 836-841, 870-876: bincount_, the three cumsums and the
 * .item() totals).  A group is a non-empty (index0, index1) = (window, head) pair;
 * groups appear in ascending order.  `idx` is the [4, M] int32 index matrix of Q (for
 * 'q_k') or V (for 'qk_v'); `inner` is its dense last-dimension extent (head dim), so
 * that M / inner token rows exist.
 *
 * plan (device, int32, capacity 5 * g_cap entries, g_cap >= number of groups; M/inner is
 * always enough) receives five rows of g_cap entries each:
 *   row 0  c[g]           tokens of group g                  (the reference's `_c`)
 *   row 1  row_start[g]   exclusive scan of c                (`idx_starts`)
 *   row 2  sq_start[g]    exclusive scan of c*c              (`pos_starts`)
 *   row 3  window[g]      index0 of the group
 *   row 4  head[g]        index1 of the group
 * totals_out (host, 4 x int64): {G, sum c, sum c*c, max c}.  Synchronises `stream`. */
size_t sswin_plan_workspace_bytes(int64_t M, int inner);
int sswin_plan_from_indices(const int32_t* idx, int64_t M, int inner, int32_t* plan,
                            int64_t g_cap, int64_t* totals_out, void* ws, size_t ws_bytes,
                            void* stream);

/* The order SparseTensor.permute((0, 2, 1, 3)) of sparse_swin/swin3d_base.py:47-59 arrives at by hashing the
 * permuted indices and sorting them, for a coalesced [B, H, n, C] operand whose heads hold the same
 * positions in every window (an attention output): perm_out[k] = position in the operand of the k-th
 * entry of the permuted, sorted operand.  idx: its [4, M] indices; plan / g_cap / G: from
 * sswin_plan_from_indices(idx, M, C).  C a multiple of 4; perm_out (device int32 [M]) 16-byte aligned.
 * bad_groups (device int32 [1]) receives the number of groups that do not fit the premise (different
 * counts or positions than the first head of their window); those groups write nothing, and the caller
 * falls back to flatten_indices + sort_indices when it is not zero.  Asynchronous. */
int sswin_permute_heads_order(const int32_t* idx, int64_t M, int C, const int32_t* plan, int64_t g_cap,
                              int64_t G, int32_t* perm_out, int32_t* bad_groups, void* stream);

/* Row ids of the sparse softmax for a [B, H, n, n] product in sorted order: rows_out[sq_start[g] + i*c + j] =
 * row_start[g] + i.  Equal to unique_consecutive_indices(flatten_indices(idx[:3])) of that product
 * (sparse_swin/swin3d_base.py:140-150), without reading its index matrix.  c: device int32 [G] (windows of fewer than
 * 4096 tokens), scans: device int32 [2*G] as sswin_scan_counts writes them, rows_out: device int32 [A], A = sum c*c
 * (a host number; the launch is sized from the mean group A / G).  Asynchronous. */
int sswin_softmax_rows_from_counts(const int32_t* c, const int32_t* scans, int64_t G, int64_t A, int32_t* rows_out,
                                   void* stream);

/* values + bias[head, pos_i, pos_j], and -100 more where the mask regions of the two positions differ, for a
 * [B, H, n, n] 'q_k' product in sorted order (sp_add_rpb and sp_add_mask, sparse_swin/swin3d_base.py:557-581), from the
 * product's plan (as sswin_plan_from_indices writes it) instead of a linear index per entry.  values / out: [A] of
 * `dtype`; row_pos: device int32 [sum c], the window position of every token row in group order (from
 * sswin_group_row_positions on the product's indices, or every C-th entry of row 2 of the Q operand's indices: the
 * product's own index matrix is not read); bias: fp32 [H, n, n]
 * (rounded to `dtype` before the addition, as the reference's dense bias is); mask: int8 [n_mask_windows, n] region ids
 * or NULL; c_max: largest group (at most 512 tokens).  Asynchronous. */
int sswin_group_add_bias_mask(int dtype, const void* values, const int32_t* row_pos, int64_t A, const int32_t* plan, int64_t g_cap,
                              int64_t G, int c_max, int n, const float* bias, const int8_t* mask, int n_mask_windows,
                              void* out, void* stream);

/* The same with the bias taken from the relative position table itself: bias of positions p, q =
 * table[code[p] - code[q] + offset0][head] (the gather of sparse_swin/swin3d_base.py:644-647 folded in; table: fp32
 * [table_rows, H], code: device int32 [n], both as sswin_bias_from_table takes them; codes and table rows below 2^15).
 * The table is a few KB where the gathered bias of 7^3 windows is 1.4 MB.  Asynchronous. */
int sswin_group_add_table_bias_mask(int dtype, const void* values, const int32_t* row_pos, int64_t A, const int32_t* plan,
                                    int64_t g_cap, int64_t G, int c_max, int n, const float* table, int table_rows, int H,
                                    const int32_t* code, int offset0, const int8_t* mask, int n_mask_windows, void* out,
                                    void* stream);

/* Window position of every attention row of a [B, H, n, n] product in sorted order: out[row_start[g] + i] = idx[2] at
 * the first entry of row i of group g (plan as sswin_plan_from_indices writes it; out: device int32 [sum c]).  With
 * this array in place of the token positions and the plan's row_start in place of the windows' first ranks,
 * sswin_bias_table_grad takes the gradient of such a product's values (tokens = out, N = 0).  Asynchronous. */
int sswin_group_row_positions(const int32_t* idx, int64_t A, const int32_t* plan, int64_t g_cap, int64_t G, int32_t* out,
                              void* stream);

/* Same three scans from a given `_c` (what the reference recomputes inside every
 * matmul_grad / qkv_transpose call, sparse_swin/ops.cu:681, 697, 965-968, 986-989,
 * 1007-1010).  c: device int32 [G].  scans: device int32 [2*G]: row 0 = exclusive scan of c,
 * row 1 = exclusive scan of c*c.  Asynchronous. */
size_t sswin_scan_counts_workspace_bytes(int64_t G);
int sswin_scan_counts(const int32_t* c, int64_t G, int32_t* scans, void* ws, size_t ws_bytes,
                      void* stream);

/* ---- block products ------------------------------------------------------------------ */

/* matmul_cuda_naive (sparse_swin/ops.cu:344-418, 788-943, 1034-1088, ops.h:4-12).
 *  kind = SSWIN_MUL_Q_K : mat1 = Q values [sum c*C] (per group row-major [c x C]),
 *                         mat2 = K^T values, per group row-major [C x c];
 *                         out_val [sum c*c], out_idx [4, sum c*c] = (window, head, pos_i, pos_j)
 *  kind = SSWIN_MUL_QK_V: mat1 = P values [sum c*c] (per group row-major [c x c]),
 *                         mat2 = V values, per group row-major [c x C];
 *                         out_val [sum c*C], out_idx [4, sum c*C] = (window, head, pos_i, channel)
 * `plan`/`g_cap`/`G`/`c_max` come from sswin_plan_from_indices on `tok_idx`, the [4, M] index matrix
 * of the operand that carries the token rows (Q for q_k, V for qk_v), M = sum c*C; its row 2
 * provides pos.  out_idx == NULL: values only (a caller that composes the operators and never reads the product's
 * index matrix saves its 16 bytes per entry); out_val == NULL: index rows only (mat1_v, mat2_v and dtype are then
 * ignored), so the two halves can be asked for at different times.  All array arguments: device.  Asynchronous. */
int sswin_block_matmul(int kind, int dtype, const void* mat1_v, const void* mat2_v,
                       const int32_t* tok_idx, int64_t M, int C, const int32_t* plan,
                       int64_t g_cap, int64_t G, int64_t c_max, void* out_val,
                       int32_t* out_idx, int64_t out_nnz, void* stream);

/* matmul_grad_cuda_naive (sparse_swin/ops.cu:422-515, 945-1031, 1092-1114, ops.h:15-21):
 * value-only block products; both operands are read along their rows.
 *  SSWIN_GRAD_RC_CR: out[c x c] = m1[c x C] . m2[c x C]^T
 *  SSWIN_GRAD_RR_RC: out[c x C] = m1[c x c] . m2[C x c]^T
 *  SSWIN_GRAD_CR_RR: out[C x c] = m1[C x c] . m2[c x c]^T
 * Two more kinds have no operator of their own in the reference: they are what its Python backward
 * (sparse_swin/swin3d_base.py:121-134) composes from two qkv_transpose calls and one of the products above, read
 * from the untransposed operands instead (the transposed copies are never written):
 *  SSWIN_GRAD_TR_RC: out[c x C] = m1[c x c]^T . m2[c x C]     = RR_RC(transpose_rr(m1), transpose_rc(m2))
 *  SSWIN_GRAD_TC_RR: out[C x c] = m1[c x C]^T . m2[c x c]     = CR_RR(transpose_rc(m1), transpose_rr(m2))
 * c: device int32 [G]; scans: device, from sswin_scan_counts; mat_nnz: number of values of the [c x C] operand or
 * result (sum of c*C over the groups, a host number: the numel of that tensor), from which the launch is sized for
 * the mean group.  Asynchronous. */
int sswin_block_matmul_grad(int kind, int dtype, const void* m1, const void* m2,
                            const int32_t* c, const int32_t* scans, int64_t G, int C,
                            int64_t mat_nnz, void* out, void* stream);

/* qkv_transpose (sparse_swin/ops.cu:518-557, 663-715, 1117-1132, ops.h:30-35):
 *  SSWIN_TRANSPOSE_RC: per group [c x C] -> [C x c];  SSWIN_TRANSPOSE_RR: [c x c] -> transposed.
 * Asynchronous. */
int sswin_block_transpose(int kind, int dtype, const void* in, const int32_t* c,
                          const int32_t* scans, int64_t G, int C, void* out, void* stream);

/* ---- sparse row softmax ---------------------------------------------------------------- */

/* softmax_last_dim_forward (sparse_swin/ops.cu:107-167, ops.h:43-45): rows are runs of equal
 * consecutive ids in idx_row (sorted).  y = exp(v - max(0, rowmax)) / (rowsum + 1e-8).
 * dtype SSWIN_F32 or SSWIN_F64.  Deterministic (no atomics).  Asynchronous. */
int sswin_softmax_last_dim_forward(const int32_t* idx_row, const void* values, int dtype,
                                   int64_t A, void* out, void* stream);

/* softmax_last_dim_backward (sparse_swin/ops.cu:169-194, ops.h:47-50):
 * gx = g*y - y * sum_row(g*y).  Asynchronous. */
int sswin_softmax_last_dim_backward(const int32_t* idx_row, const void* y, const void* grad,
                                    int dtype, int64_t A, void* out, void* stream);

/* ---- fused window attention (replaces Python glue of the reference, no operator of ops.h) ---- */

/* Token plan: what sparse_swin/swin3d_base.py:483-498 (qkv_sparse_cuda: index expansion, two
 * sorts, five gathers) and :673-675 (permute, return_inverse, un-sort gather) establish by
 * sorting, derived once from the [N,2] (window, pos) voxel indices without any sort.
 * tokens (device int32 [5*N]): five rows of N entries indexed by token rank r (rank in
 *   (window, pos) order): voxel of rank r; rank of the first token of its window; tokens of its
 *   window; pos; window.
 * plan (device int32 [5*g_cap]): rows c, T (rank of the window's first token), sq_start
 *   (exclusive scan of c*c over groups), window, head — groups ordered (window, head).
 * tasks (device int32, sswin_token_plan_task_ints(N, g_cap, H) entries, or NULL): group descriptors
 *   [4][g_cap][4] {T, c | head << 8, window, sq_start} bucketed by ceil(c/32) = 1..4 for
 *   sswin_window_attention_* (a window's H descriptors side by side, windows of a bucket in window
 *   order), followed by the token records [N/32 + g_cap/H + 4][32][2]: one record {voxel, pos} x 32 per
 *   (window, tile of 32 tokens), bucket of four tiles first, inside a bucket by window, then tile;
 *   entries behind a window's last token repeat it.  A task of the attention kernels finds its
 *   descriptor and its tokens from its own number alone (one memory round trip instead of two).
 * totals_out (host, 9 x int64): {groups G, non-empty windows, sum over groups of c*c, max c,
 *   groups in bucket 1..4, groups with c > 128 (no descriptor)}; the last five are 0 without tasks.
 * (window, pos) pairs must be distinct, window in [0,B), pos in [0,n): indices outside that range
 * are skipped on the device (nothing is written through them) and reported as an error when the
 * totals are decoded, and so are pairs that occur twice.
 * synchronize != 0: waits for `stream` and decodes the totals.  synchronize == 0: only enqueues
 * the work and a copy of the raw totals into totals_out (pinned host memory); once the caller
 * has waited for the stream, sswin_token_plan_totals(totals_out, H, g_cap) decodes them in place
 * and performs the checks (range, distinctness, capacity). */
size_t sswin_token_plan_workspace_bytes(int64_t N, int B, int n);
size_t sswin_token_plan_task_ints(int64_t N, int64_t g_cap, int H);
int sswin_token_plan(const int32_t* indices, int64_t N, int B, int n, int H, int32_t* tokens,
                     int32_t* plan, int64_t g_cap, int32_t* tasks, int64_t* totals_out, void* ws,
                     size_t ws_bytes, int synchronize, void* stream);
int sswin_token_plan_totals(int64_t* totals, int H, int64_t g_cap);

/* Up to four token plans in one set of launches: the regular and the shifted block of a stage
 * (sparse_swin/swin3d_base.py:889-905 runs them one after the other, each with its own
 * coalesce / sort chain, ops.cu:781-784, 836-841) partition the same voxels differently, and one plan
 * is a few microseconds of work per launch.  Every descriptor holds the arguments of one
 * sswin_token_plan call with synchronize == 0 and gives the same results; plans with N == 0 are
 * skipped (totals all zero).  After waiting for `stream`, decode each totals_out with
 * sswin_token_plan_totals.  Rejects count > 4.
 * flags: SSWIN_PLAN_ORDER_ONLY writes only the first row of `tokens` (voxel of rank r; `tokens` may then hold N
 * entries): what the stride-2 merge reads (sswin_pool_windows), four scattered stores per voxel fewer. */
#define SSWIN_PLAN_ORDER_ONLY 1
typedef struct sswin_token_plan_desc {
    const int32_t* indices;
    int64_t N;
    int32_t B, n, H, flags;
    int32_t* tokens;
    int32_t* plan;
    int64_t g_cap;
    int32_t* tasks;
    int64_t* totals_out;
    void* ws;
    size_t ws_bytes;
} sswin_token_plan_desc;
int sswin_token_plan_batch(const sswin_token_plan_desc* descs, int count, void* stream);

/* Token tensors are dense [N, stride] arrays of `dtype`; element (voxel v, head h, channel ch) is
 * base[v*stride + col0 + h*hd + ch].  "sq" arrays are fp32 arrays of all [c x c] blocks; a window holds at most
 * 16 384 tokens (a block is addressed with 32-bit byte offsets below 2^31).
 *
 * tokens x tokens -> sq: out[g][i][j] = sum_ch (scale_a * A[token i, ch]) * B[token j, ch].
 * With epilogue != 0 (the product S = Q K^T of swin3d_base.py:660-668): adds
 * bias[h, pos_i, pos_j] (fp32 [H,n,n], :557-566) and, if mask != NULL (int8 [n_mask_windows, n]
 * region ids, :569-581), -100 where the regions of the two tokens differ; row_ids (optional)
 * receives the softmax row id H*T + h*c + i of every element.  Asynchronous. */
int sswin_fused_tokens_to_sq(int dtype, int epilogue, const int32_t* plan, int64_t g_cap, int64_t G,
                             const int32_t* tokens, int64_t N, int H, int hd, const void* a_base,
                             int64_t a_stride, int a_col0, const void* b_base, int64_t b_stride,
                             int b_col0, float scale_a, const float* bias, int n, const int8_t* mask,
                             int n_mask_windows, float* out, int32_t* row_ids, void* stream);

/* sq x tokens -> tokens: out[token i, ch] = scale_out * sum_k A(i,k) * B[token k, ch] with
 * A(i,k) = sq[g][i][k] (a_kmajor = 0: O = P V, dQ = dS K) or sq[g][k][i] (a_kmajor = 1:
 * dV = P^T dO, dK = dS^T Q).  Every (voxel, head, channel) of the output is written once.
 * Replaces 'qk_v' + permute + un-sort (swin3d_base.py:672-675) and the backward products with
 * their transposes (:119-134).  Asynchronous. */
int sswin_fused_sq_to_tokens(int dtype, int a_kmajor, const int32_t* plan, int64_t g_cap, int64_t G,
                             const int32_t* tokens, int64_t N, int H, int hd, const float* sq,
                             const void* b_base, int64_t b_stride, int b_col0, void* o_base,
                             int64_t o_stride, int o_col0, float scale_out, void* stream);

/* Gradient of the scores from the gradient of the attention output, in one launch:
 *   ds[g][i][j] = p[g][i][j] * (sum_ch dO[token i, ch] * V[token j, ch] - D_i),   D_i = sum_ch dO[token i, ch] * O[token i, ch],
 * which is the product dP = dO V^T (swin3d_base.py:119-134) followed by the softmax backward (ops.cu:169-194):
 * sum_j p_ij dP_ij = dO_i . O_i because O = P V, so dP is never written.  dO, V, O: token tensors as above; p: the
 * attention matrix of the forward pass, ds: fp32 sq arrays.  c_max <= 384.  Token tensors that a 32-bit offset cannot
 * cover run the product and sswin_group_softmax one after the other instead.  Asynchronous. */
int sswin_fused_score_grad(int dtype, const int32_t* plan, int64_t g_cap, int64_t G, const int32_t* tokens,
                           int64_t N, int H, int hd, int c_max, const void* do_base, int64_t do_stride,
                           int do_col0, const void* v_base, int64_t v_stride, int v_col0, const void* o_base,
                           int64_t o_stride, int o_col0, const float* p, float* ds, void* stream);

/* The sparse row softmax over the rows of the groups' [c x c] blocks, forward (backward == 0: out = softmax of
 * x_or_y, grad ignored) or backward (out = y (g - sum_j g_j y_j) with y = x_or_y, g = grad).  The arithmetic of
 * softmax_last_dim_forward / _backward (sparse_swin/ops.cu:128-194: zero-initialised maximum, + 1e-8 in the
 * denominator); the rows come from the group table instead of a row id per entry (swin3d_base.py:140-150 builds those
 * ids with flatten_indices + unique_consecutive).  fp32 sq arrays; out may be x_or_y or grad (in place).  N, H: voxels
 * and heads of the plan (the launch is sized from the mean group N*H/G); c_max <= 384.  Asynchronous. */
int sswin_group_softmax(int backward, const int32_t* plan, int64_t g_cap, int64_t G, int64_t N, int H,
                        int c_max, const float* x_or_y, const float* grad, float* out, void* stream);

/* d_bias[h, pos_i, pos_j] += ds over all windows (the backward of swin3d_base.py:557-566, which
 * autograd performs as an index_add).  d_bias: fp32 [H,n,n], accumulated into (zero it first).
 * n*n*4 bytes must fit 64 KiB of LDS.  No atomics: every table row is owned by one wavefront
 * and partial tables are summed in a fixed order, so the result is reproducible.  Asynchronous. */
size_t sswin_fused_bias_grad_workspace_bytes(int64_t G, int H, int n);
int sswin_fused_bias_grad(const int32_t* plan, int64_t g_cap, int64_t G, const int32_t* tokens,
                          int64_t N, int H, int n, const float* ds, float* d_bias, void* ws,
                          size_t ws_bytes, void* stream);

/* bias[H,n,n] (fp32) from the relative position bias table [table_rows, H] (fp32):
 * bias[h][p][q] = table[code[p] - code[q] + offset0][h], the gather and permute of
 * swin3d_base.py:644-647 in one launch (code as for sswin_bias_table_grad).  Asynchronous. */
int sswin_bias_from_table(const float* table, int table_rows, int H, const int32_t* code, int offset0,
                          int n, float* bias, void* stream);

/* Gradient of the relative position bias table itself (swin3d_base.py:624-652 gathers the
 * [H,n,n] bias from a [(2w-1)^3, H] table by relative_position_index; autograd scatters back with
 * an index_add).  The index is linear in the two positions: rel(p_i,p_j) = code[p_i] - code[p_j]
 * + offset0 (code: device int32 [n]).  d_table (fp32 [table_rows, H]) is overwritten.
 * table_rows <= 4096, n <= 384 (up to 160 KB of LDS for the largest tables).  No atomics, fixed summation order.  Asynchronous (the G == 0 case records a memset: do not capture it). */
size_t sswin_bias_table_grad_workspace_bytes(int64_t G, int H, int table_rows);
int sswin_bias_table_grad(const int32_t* plan, int64_t g_cap, int64_t G, const int32_t* tokens,
                          int64_t N, int H, int n, const int32_t* code, int offset0, int table_rows,
                          const float* ds, float* d_table, void* ws, size_t ws_bytes, void* stream);

/* The same gradient with the batches taken from the task descriptors of a token plan (`tasks`, `bucket_counts`: what
 * sswin_window_attention_forward takes) instead of its group table: the descriptors list the groups by their number
 * of 32-token tiles, so the 32 x 32 batches of dS can be dealt to the wavefronts evenly.  For plans whose windows all
 * hold at most 128 tokens (the sum of bucket_counts equals G); same workspace, same result up to the order of the
 * fp32 sums (fixed from run to run).  No counterpart in the reference (autograd's index_add, swin3d_base.py:557-566). */
int sswin_bias_table_grad_tasks(const int32_t* tasks, int64_t g_cap, const int64_t* bucket_counts, int64_t G,
                                const int32_t* tokens, int64_t N, int H, int n, const int32_t* code,
                                int offset0, int table_rows, const float* ds, float* d_table, void* ws,
                                size_t ws_bytes, void* stream);

/* Column sums (fp32) of a dense [N, P] matrix of `dtype` (fp32 / fp16 / bf16; P a multiple of 4,
 * rows contiguous): the bias gradient of the qkv / proj nn.Linear (swin3d_base.py:606-610;
 * autograd's grad_out.sum(0)).  Fixed summation order.  Asynchronous (N == 0 records a memset). */
size_t sswin_column_sum_workspace_bytes(int64_t N, int P);
int sswin_column_sum(const void* x, int dtype, int64_t N, int P, float* out, void* ws,
                     size_t ws_bytes, void* stream);

/* y[N,P] = x[N,K] w[P,K]^T + bias[P] (bias may be NULL) for dense fp32 row-major arrays: the forward
 * of the qkv and proj nn.Linear (swin3d_base.py:606-610, applied at :658 and :676).  K a multiple of
 * 16 up to 192 or of 96 up to 768; P a multiple of 96 (sswin_tall_linear_supported tells).  Runs on the bf16 matrix
 * cores with every fp32 operand split exactly into three bf16 pieces and the six largest piece
 * products summed in fp32: results agree with an fp32 GEMM to its own rounding level.  x and w
 * 16-byte aligned.  Asynchronous, no workspace. */
int sswin_tall_linear_supported(int P, int K);
int sswin_tall_linear_forward(const float* x, int64_t N, int K, const float* w, const float* bias,
                              int P, float* y, void* stream);

/* dx[N,K] = dy[N,P] w[P,K]: input gradient of the same layers (autograd of nn.Linear,
 * swin3d_base.py:606-610).  fp32, P and K multiples of 96 (sswin_tall_linear_input_grad_supported
 * tells); same split-operand arithmetic as the forward.  dy 16-byte aligned.  Asynchronous. */
int sswin_tall_linear_input_grad_supported(int P, int K);
int sswin_tall_linear_input_grad(const float* dy, int64_t N, int P, const float* w, int K, float* dx,
                                 void* stream);

/* dw[P,K] = dy[N,P]^T x[N,K] and, when db is not NULL, db[P] = column sums of dy: weight and bias
 * gradient of the same layers (autograd of nn.Linear, swin3d_base.py:606-610).  fp32, P a multiple
 * of 96, K = 32, 64, 96 or a multiple of 96 up to 768, taken in passes of 96 columns of x (the
 * workspace size is 0 for anything else).  Same split-operand
 * arithmetic as the forward; partial sums per workgroup are added in a fixed order, so the result
 * is the same on every run.  dw, db and ws 16-byte aligned.  Asynchronous. */
size_t sswin_tall_linear_weight_grad_workspace_bytes(int64_t N, int P, int K);
int sswin_tall_linear_weight_grad(const float* dy, const float* x, int64_t N, int P, int K, float* dw,
                                  float* db, void* ws, size_t ws_bytes, void* stream);

/* ---- window-resident attention (whole forward / backward of the attention core) ---------- */

/* Forward of sparse_swin/swin3d_base.py:660-672 for every (window, head) group in one pass:
 * O = softmax((scale*Q) K^T + bias + mask) V with the operator's softmax semantics
 * (ops.cu:128-167: max(0,rowmax), sum + 1e-8).  The attention matrix stays in registers.
 * tasks / bucket_counts (host, 4 x int64) come from sswin_token_plan; q, k, v, o are token
 * tensors as above with hd = 32; lse (fp32 [H*N]) receives m + log(sum) of attention row
 * H*T + h*c + i (the row id of the sparse softmax).  Windows of at most 128 tokens.  Asynchronous. */
int sswin_window_attention_forward(int dtype, const int32_t* tasks, int64_t g_cap,
                                   const int64_t* bucket_counts, const int32_t* tokens, int64_t N,
                                   int H, int hd, const void* q_base, int64_t q_stride, int q_col0,
                                   const void* k_base, int64_t k_stride, int k_col0,
                                   const void* v_base, int64_t v_stride, int v_col0, float scale,
                                   const float* bias, int n, const int8_t* mask, int n_mask_windows,
                                   void* o_base, int64_t o_stride, int o_col0, float* lse,
                                   void* stream);

/* Backward of the same (swin3d_base.py:106-138 and :177-188 composed): from O, dO and lse,
 * recomputes P per tile and writes dQ = scale dS K, dK = scale dS^T Q, dV = P^T dO with
 * dS = P (dP - rowsum(dO o O)).  ds_out (fp32 "sq" array in plan order, or NULL) receives dS
 * for the bias gradient.  sides: 1 = dQ only (query-side kernel), 2 = dK and dV (and dS) only
 * (key-side kernel), 3 = all in one launch: the key-side tasks then also produce dQ of the groups of
 * at most 64 tokens (one tile: from the dS already in registers; two tiles: the two key-side tasks of a
 * group exchange their partial dS K through LDS) and only the larger groups have query-side tasks.
 * Asynchronous. */
int sswin_window_attention_backward(int dtype, const int32_t* tasks, int64_t g_cap,
                                    const int64_t* bucket_counts, const int32_t* tokens, int64_t N,
                                    int H, int hd, const void* q_base, int64_t q_stride, int q_col0,
                                    const void* k_base, int64_t k_stride, int k_col0,
                                    const void* v_base, int64_t v_stride, int v_col0, float scale,
                                    const float* bias, int n, const int8_t* mask, int n_mask_windows,
                                    const void* o_base, int64_t o_stride, int o_col0,
                                    const void* do_base, int64_t do_stride, int do_col0,
                                    const float* lse, void* dq_base, int64_t dq_stride, int dq_col0,
                                    void* dk_base, int64_t dk_stride, int dk_col0, void* dv_base,
                                    int64_t dv_stride, int dv_col0, float* ds_out, int sides,
                                    void* stream);

/* ---- voxel grid glue of a stage (callers of the attention: block and stage level) ---------- */

/* (batch, d, h, w) voxel coordinates -> (window slot, position inside the window) of the grid
 * shifted cyclically by -shift: pad_sparse_tensor + roll_sparse_tensor + window_partition_sparse
 * (sparse_swin/swin3d_base.py:501-554, 336-372) in one pass.  coords: device int32 [N,4]
 * (16-byte aligned); dims: host int32[3] padded extents (multiples of window); window, shift: host
 * int32[3], 0 <= shift < extent; indices: device int32 [N,2].  window slot =
 * ((batch*nd + wz)*nh + wy)*nw + wx.  With window = {2,2,2} and no shift the result is (merged
 * voxel, child slot) of the floor(coord/2) down-sampling between stages.  Asynchronous. */
int sswin_window_indices(const int32_t* coords, int64_t N, int batch_size, const int32_t* dims,
                         const int32_t* window, const int32_t* shift, int32_t* indices,
                         void* stream);

/* Region ids of the shifted-window attention mask, int8 [windows per batch item, positions]:
 * compute_mask (swin3d_base.py:416-452: 27 slice assignments into a dense volume, then
 * window_partition) evaluated per element.  A shift of 0 along an axis gives region 2 on that
 * axis, as the reference's slices do.  Asynchronous. */
int sswin_shift_mask(const int32_t* dims, const int32_t* window, const int32_t* shift, int8_t* mask,
                     void* stream);

/* (batch, wz, wy, wx) of the M non-empty windows of a token plan made with H = 1, in plan order
 * (ascending window slot): the output coordinates of the stride-2 down-sampling
 * (swin3d_base.py:950-976, spconv SparseConv3d kernel 2 stride 2: out = floor(coord/2), deduped).
 * coords_out: device int32 [M,4], 16-byte aligned.  Asynchronous. */
int sswin_window_coords(const int32_t* plan, int64_t g_cap, int64_t M, const int32_t* dims,
                        const int32_t* window, int32_t* coords_out, void* stream);

/* Rows of the voxels of each non-empty window reduced to one row, in (window, position) order and
 * therefore in a fixed order without atomics: dst[m] = sum (mean != 0: average) of src[voxel] over
 * the voxels of window m (plan / tokens from sswin_token_plan with H = 1).  backward != 0 is the
 * gradient: src = [M, C] gradient of the pooled rows, dst[voxel] = src[m] (/ count).  C a multiple of
 * 4; src, dst dense rows of `dtype` with the given strides.  Stands where the reference uses the
 * strided sparse convolution between stages (swin3d_base.py:950-976).  Asynchronous. */
int sswin_pool_windows(int dtype, int backward, int mean, const int32_t* plan, int64_t g_cap,
                       int64_t M, const int32_t* tokens, int64_t N, const void* src,
                       int64_t src_stride, int C, void* dst, int64_t dst_stride, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SSWIN3D_H */
