/*
 * CPU oracle for the sparse window-attention operator set.  TEST INFRASTRUCTURE ONLY:
 * it is the checker for the HIP library, never the thing that is shipped or measured
 * as the product.  Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of
 * bench.py may load it.
 *
 * Every function restates, in plain scalar C, the algorithm of one operator of the
 * reference (citations are relative to the reference checkout, file:line).  The
 * restatement deliberately keeps the reference's *general* formulation (hash every COO
 * column, rank the hashes, transpose the right-hand operand through a CSR->CSC
 * re-ordering, run the block kernels, gather the keys back) instead of the closed forms
 * the HIP library uses, so that a parity test compares two independent derivations.
 *
 * What pins each function (see tests/test_oracle_pins.py):
 *   flatten_indices            numpy.ravel_multi_index in wrapping int32
 *   sort_indices               numpy.argsort(kind="stable")
 *   unique_consecutive_indices torch.unique_consecutive(return_inverse=True)
 *   return_inverse             numpy.unique(return_inverse=True)
 *   qkv_sparse_indices         numpy.lexsort over brute-force 4-tuples + closed forms
 *   matmul q_k / qk_v          dense [B,H,n,n] brute force with numpy.einsum, coalesced COO
 *   matmul_grad, qkv_transpose numpy per-group matmul / .T
 *   softmax fwd/bwd            scipy.special.softmax per row, closed-form Jacobian, fp64
 * The reference itself holds no tests, golden vectors or fixtures for this path, so
 * nothing of the reference's own pins these; "parity unpinned by reference fixtures"
 * applies to every function, and the pins above are what replaces them.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

/* ------------------------------------------------------------------------------------ */
/* flatten_indices: wrapping int32 row-major hash.  sparse_swin/ops.cu:232-273          */
/* strides come from sizes[1:]; sizes[0] never enters (ops.cu:237-245).                 */
/* ------------------------------------------------------------------------------------ */
void orc_flatten_indices(const int32_t* idx, int ndim, int64_t M, const int32_t* sizes,
                         int32_t* out) {
    uint32_t stride[16];
    stride[ndim - 1] = 1u;
    for (int i = ndim - 2; i >= 0; --i) stride[i] = stride[i + 1] * (uint32_t)sizes[i + 1];
    for (int64_t m = 0; m < M; ++m) {
        uint32_t h = 0;
        for (int i = 0; i < ndim; ++i) h += (uint32_t)idx[(int64_t)i * M + m] * stride[i];
        out[m] = (int32_t)h;
    }
}

/* ------------------------------------------------------------------------------------ */
/* sort_indices: argsort ascending of signed int32 keys; radix sort is stable, so equal  */
/* keys keep input order.  sparse_swin/ops.cu:276-289                                    */
/* ------------------------------------------------------------------------------------ */
static void merge_sort_perm(const int32_t* keys, int32_t* perm, int32_t* tmp, int64_t n) {
    for (int64_t w = 1; w < n; w *= 2) {
        for (int64_t lo = 0; lo < n; lo += 2 * w) {
            int64_t mid = lo + w < n ? lo + w : n, hi = lo + 2 * w < n ? lo + 2 * w : n;
            int64_t a = lo, b = mid, o = lo;
            while (a < mid && b < hi) tmp[o++] = (keys[perm[b]] < keys[perm[a]]) ? perm[b++] : perm[a++];
            while (a < mid) tmp[o++] = perm[a++];
            while (b < hi) tmp[o++] = perm[b++];
        }
        memcpy(perm, tmp, (size_t)n * sizeof(int32_t));
    }
}

void orc_sort_indices(const int32_t* keys, int64_t M, int32_t* perm) {
    int32_t* tmp = (int32_t*)malloc((size_t)(M > 0 ? M : 1) * sizeof(int32_t));
    for (int64_t i = 0; i < M; ++i) perm[i] = (int32_t)i;
    merge_sort_perm(keys, perm, tmp, M);
    free(tmp);
}

/* ------------------------------------------------------------------------------------ */
/* unique_consecutive_indices: rank of the run each element belongs to                   */
/* (adjacent_difference with not_equal, first forced to 0, inclusive scan).              */
/* sparse_swin/ops.cu:36-57, 60-103                                                      */
/* ------------------------------------------------------------------------------------ */
void orc_unique_consecutive_i32(const int32_t* x, int64_t M, int32_t* out) {
    int32_t r = 0;
    for (int64_t i = 0; i < M; ++i) {
        if (i > 0 && x[i] != x[i - 1]) ++r;
        out[i] = r;
    }
}
void orc_unique_consecutive_i64(const int64_t* x, int64_t M, int32_t* out) {
    int32_t r = 0;
    for (int64_t i = 0; i < M; ++i) {
        if (i > 0 && x[i] != x[i - 1]) ++r;
        out[i] = r;
    }
}

/* ------------------------------------------------------------------------------------ */
/* return_inverse: presence table of size maxnum (max+1 when maxnum == -1), rank of each  */
/* present value among the present values, number of distinct values.                    */
/* sparse_swin/ops.cu:718-730                                                            */
/* ------------------------------------------------------------------------------------ */
int64_t orc_return_inverse(const int32_t* x, int64_t M, int64_t maxnum, int32_t* out) {
    if (M == 0) return 0;
    if (maxnum == -1) {
        int32_t mx = x[0];
        for (int64_t i = 1; i < M; ++i) if (x[i] > mx) mx = x[i];
        maxnum = (int64_t)mx + 1;
    }
    uint8_t* present = (uint8_t*)calloc((size_t)maxnum, 1);
    int32_t* rank = (int32_t*)malloc((size_t)maxnum * sizeof(int32_t));
    for (int64_t i = 0; i < M; ++i) present[x[i]] = 1;
    int64_t c = 0;
    for (int64_t v = 0; v < maxnum; ++v) if (present[v]) rank[v] = (int32_t)c++;
    for (int64_t i = 0; i < M; ++i) out[i] = rank[x[i]];
    free(present);
    free(rank);
    return c;
}

/* ------------------------------------------------------------------------------------ */
/* qkv_sparse_indices: expand [N,2] (window,pos) to element-level COO for Q/V and for K^T */
/* (rows 2 and 3 swapped), hash both with {B,H,n,hd} / {B,H,hd,n}, argsort the hashes.    */
/* sparse_swin/ops.cu:206-227 (expand), 293-335 (host)                                    */
/* ------------------------------------------------------------------------------------ */
void orc_qkv_sparse_indices(const int32_t* indices, int64_t N, int B, int n, int H, int hd,
                            int32_t* idx_qv, int32_t* sorted_qv, int32_t* idx_k,
                            int32_t* sorted_k) {
    int64_t E = N * H * hd;
    for (int64_t e = 0; e < E; ++e) {
        int64_t v = e / ((int64_t)H * hd);
        int32_t local = (int32_t)(e % ((int64_t)H * hd));
        int32_t h = local / hd, ch = local % hd;
        int32_t w = indices[2 * v], p = indices[2 * v + 1];
        idx_qv[0 * E + e] = w;  idx_qv[1 * E + e] = h;  idx_qv[2 * E + e] = p;   idx_qv[3 * E + e] = ch;
        idx_k[0 * E + e] = w;   idx_k[1 * E + e] = h;   idx_k[2 * E + e] = ch;   idx_k[3 * E + e] = p;
    }
    int32_t* flat = (int32_t*)malloc((size_t)(E > 0 ? E : 1) * sizeof(int32_t));
    int32_t s_qv[4] = {B, H, n, hd}, s_k[4] = {B, H, hd, n};
    orc_flatten_indices(idx_qv, 4, E, s_qv, flat);
    orc_sort_indices(flat, E, sorted_qv);
    orc_flatten_indices(idx_k, 4, E, s_k, flat);
    orc_sort_indices(flat, E, sorted_k);
    free(flat);
}

/* ------------------------------------------------------------------------------------ */
/* helpers for the block matmul                                                          */
/* ------------------------------------------------------------------------------------ */
/* reshape_sparse: 2-D row/col hashes of a 4-D COO.  sparse_swin/ops.cu:732-779          */
static void reshape_rows_cols(const int32_t* idx, int64_t M, const int32_t* shape,
                              int32_t* row, int32_t* col) {
    uint32_t x2 = (uint32_t)shape[1], x3 = (uint32_t)shape[2], x4 = (uint32_t)shape[3];
    for (int64_t m = 0; m < M; ++m) {
        uint32_t i0 = (uint32_t)idx[m], i1 = (uint32_t)idx[M + m], i2 = (uint32_t)idx[2 * M + m],
                 i3 = (uint32_t)idx[3 * M + m];
        row[m] = (int32_t)(i0 * x2 * x3 + i1 * x3 + i2);
        col[m] = (int32_t)(i0 * x2 * x4 + i1 * x4 + i3);
    }
}

/* bincount_ then drop zeros (ops.cu:781-784) of a[0], a[step], a[2*step] ...            */
static int32_t* nonzero_bincount_strided(const int32_t* a, int64_t M, int64_t step, int64_t* G) {
    int64_t cnt = M / step;
    int32_t mx = -1;
    for (int64_t i = 0; i < cnt; ++i) if (a[i * step] > mx) mx = a[i * step];
    int32_t* bins = (int32_t*)calloc((size_t)mx + 2, sizeof(int32_t));
    for (int64_t i = 0; i < cnt; ++i) bins[a[i * step]]++;
    int64_t g = 0;
    for (int64_t v = 0; v <= mx; ++v) if (bins[v]) g++;
    int32_t* c = (int32_t*)malloc((size_t)(g > 0 ? g : 1) * sizeof(int32_t));
    g = 0;
    for (int64_t v = 0; v <= mx; ++v) if (bins[v]) c[g++] = bins[v];
    free(bins);
    *G = g;
    return c;
}

static int32_t* excl_scan_mul(const int32_t* c, int64_t G, int mode, int32_t C) {
    /* mode 0: c, 1: c*c, 2: c*C ; int32 cumsum as in ops.cu:838-840 */
    int32_t* s = (int32_t*)malloc((size_t)(G > 0 ? G : 1) * sizeof(int32_t));
    uint32_t acc = 0;
    for (int64_t g = 0; g < G; ++g) {
        s[g] = (int32_t)acc;
        uint32_t v = (uint32_t)c[g];
        acc += mode == 0 ? v : (mode == 1 ? v * v : v * (uint32_t)C);
    }
    return s;
}

typedef struct {
    int64_t G;
    int64_t nnz;
    int32_t* idx;     /* [4, nnz] */
    void* val;        /* [nnz]    */
    int32_t* c;       /* [G]      */
} orc_matmul_result;

void orc_free_result(orc_matmul_result* r) {
    free(r->idx); free(r->val); free(r->c);
    r->idx = NULL; r->val = NULL; r->c = NULL;
}

/* CSR -> CSC value re-ordering of mat2 (ops.cu:803-829): entries ordered by (col rank, row).  *
 * rows arrive sorted, so a stable sort by column hash is exactly that order.                    */
static int32_t* transpose_order(const int32_t* col2, int64_t M2) {
    int32_t* perm = (int32_t*)malloc((size_t)(M2 > 0 ? M2 : 1) * sizeof(int32_t));
    orc_sort_indices(col2, M2, perm);
    return perm;
}

#define DEFINE_MATMUL(NAME, T)                                                                     \
int NAME(const T* m1v, const int32_t* m1i, int64_t M1, const int32_t* shape1,                      \
         const T* m2v, const int32_t* m2i, int64_t M2, const int32_t* shape2,                      \
         int is_qk_v, orc_matmul_result* res) {                                                    \
    int32_t *r1 = malloc((size_t)(M1 + 1) * 4), *c1 = malloc((size_t)(M1 + 1) * 4);                \
    int32_t *r2 = malloc((size_t)(M2 + 1) * 4), *c2 = malloc((size_t)(M2 + 1) * 4);                \
    reshape_rows_cols(m1i, M1, shape1, r1, c1);                                                    \
    reshape_rows_cols(m2i, M2, shape2, r2, c2);                                                    \
    /* transposed values of mat2 (csrt_values_b) */                                                \
    int32_t* tperm = transpose_order(c2, M2);                                                      \
    T* m2t = (T*)malloc((size_t)(M2 + 1) * sizeof(T));                                             \
    for (int64_t m = 0; m < M2; ++m) m2t[m] = m2v[tperm[m]];                                       \
    /* key_rows = unique_consecutive(mat1 rows) (ops.cu:813) */                                    \
    int32_t* key_rows = (int32_t*)malloc((size_t)(M1 + 1) * 4);                                    \
    int64_t n_rows = 0;                                                                            \
    for (int64_t m = 0; m < M1; ++m) if (m == 0 || r1[m] != r1[m - 1]) key_rows[n_rows++] = r1[m]; \
    int32_t* key_cols; int64_t n_cols;                                                             \
    if (!is_qk_v) { key_cols = key_rows; n_cols = n_rows; }                                        \
    else { /* sorted unique of mat2 col hashes (at::_unique on the GPU sorts, ops.cu:818) */        \
        key_cols = (int32_t*)malloc((size_t)(M2 + 1) * 4); n_cols = 0;                             \
        for (int64_t m = 0; m < M2; ++m) {                                                         \
            int32_t v = c2[tperm[m]];                                                              \
            if (n_cols == 0 || key_cols[n_cols - 1] != v) key_cols[n_cols++] = v;                  \
        }                                                                                          \
    }                                                                                              \
    int32_t C; int64_t G; int32_t* c;                                                              \
    if (!is_qk_v) { C = shape1[3]; c = nonzero_bincount_strided(c1, M1, C, &G); }                  \
    else          { C = shape2[3]; c = nonzero_bincount_strided(c2, M2, C, &G); }                  \
    int32_t* idx_starts = excl_scan_mul(c, G, 0, C);                                               \
    int32_t* sq_starts  = excl_scan_mul(c, G, 1, C);                                               \
    int32_t* mat_starts = excl_scan_mul(c, G, 2, C);                                               \
    int64_t total = 0;                                                                             \
    for (int64_t g = 0; g < G; ++g) total += is_qk_v ? (int64_t)c[g] * C : (int64_t)c[g] * c[g];   \
    int32_t* rows = (int32_t*)malloc((size_t)(total + 1) * 4);                                     \
    int32_t* cols = (int32_t*)malloc((size_t)(total + 1) * 4);                                     \
    T* val = (T*)malloc((size_t)(total + 1) * sizeof(T));                                          \
    for (int64_t g = 0; g < G; ++g) {                                                              \
        int32_t rc = c[g], start = idx_starts[g];                                                  \
        if (!is_qk_v) { /* indices_kernel_q_k, ops.cu:344-378 */                                   \
            int64_t ps = sq_starts[g], pm = mat_starts[g];                                         \
            for (int i = 0; i < rc; ++i) for (int j = 0; j < rc; ++j) {                            \
                int64_t pos = ps + (int64_t)i * rc + j;                                            \
                cols[pos] = j + start; rows[pos] = i + start;                                      \
                T sum = 0;                                                                         \
                for (int k = 0; k < C; ++k) sum += m1v[pm + (int64_t)i * C + k] * m2t[pm + (int64_t)j * C + k]; \
                val[pos] = sum;                                                                    \
            }                                                                                      \
        } else { /* indices_kernel_qk_v, ops.cu:381-418 */                                         \
            int64_t ps = mat_starts[g], p1 = sq_starts[g], p2 = mat_starts[g];                     \
            for (int i = 0; i < rc; ++i) for (int j = 0; j < C; ++j) {                             \
                int64_t pos = ps + (int64_t)i * C + j;                                             \
                cols[pos] = j + (int32_t)(g * C); rows[pos] = i + start;                           \
                T sum = 0;                                                                         \
                for (int k = 0; k < rc; ++k) sum += m1v[p1 + (int64_t)i * rc + k] * m2t[p2 + (int64_t)j * rc + k]; \
                val[pos] = sum;                                                                    \
            }                                                                                      \
        }                                                                                          \
    }                                                                                              \
    /* key gather + 4-D rebuild, ops.cu:909-942 */                                                 \
    int32_t x2 = shape1[1], x3 = shape1[2], x4 = shape2[3];                                        \
    int32_t* oi = (int32_t*)malloc((size_t)(4 * total + 1) * 4);                                   \
    int bad = 0;                                                                                   \
    for (int64_t p = 0; p < total; ++p) {                                                          \
        if (rows[p] >= n_rows || cols[p] >= n_cols) { bad = 1; break; }                            \
        int32_t row = key_rows[rows[p]], col = key_cols[cols[p]];                                  \
        int32_t rem = row % (x2 * x3);                                                             \
        oi[p] = row / (x2 * x3); oi[total + p] = rem / x3; oi[2 * total + p] = rem % x3;           \
        oi[3 * total + p] = col % x4;                                                              \
    }                                                                                              \
    res->G = G; res->nnz = total; res->idx = oi; res->val = val; res->c = c;                       \
    if (is_qk_v) free(key_cols);                                                                   \
    free(key_rows); free(r1); free(c1); free(r2); free(c2); free(tperm); free(m2t);                \
    free(idx_starts); free(sq_starts); free(mat_starts); free(rows); free(cols);                   \
    return bad;                                                                                    \
}

DEFINE_MATMUL(orc_matmul_f32, float)
DEFINE_MATMUL(orc_matmul_f64, double)

/* ------------------------------------------------------------------------------------ */
/* matmul_grad: value-only block products, both operands read along their rows.          */
/* rc_cr ops.cu:422-451, rr_rc :454-483, cr_rr :486-515; host :945-1031                   */
/* mode 0 rc_cr: out[c x c] = m1[c x C] . m2[c x C]^T                                     */
/* mode 1 rr_rc: out[c x C] = m1[c x c] . m2[C x c]^T                                     */
/* mode 2 cr_rr: out[C x c] = m1[C x c] . m2[c x c]^T                                     */
/* ------------------------------------------------------------------------------------ */
#define DEFINE_GRAD(NAME, T)                                                                       \
void NAME(const T* m1, const T* m2, const int32_t* c, int64_t G, int32_t C, int mode, T* out) {    \
    int64_t o = 0, a = 0, b = 0;                                                                   \
    for (int64_t g = 0; g < G; ++g) {                                                              \
        int64_t rc = c[g];                                                                         \
        int64_t I = mode == 2 ? C : rc, J = mode == 0 ? rc : (mode == 1 ? C : rc);                 \
        int64_t K = mode == 0 ? C : rc;                                                            \
        for (int64_t i = 0; i < I; ++i) for (int64_t j = 0; j < J; ++j) {                          \
            T sum = 0;                                                                             \
            for (int64_t k = 0; k < K; ++k) sum += m1[a + i * K + k] * m2[b + j * K + k];          \
            out[o + i * J + j] = sum;                                                              \
        }                                                                                          \
        o += I * J; a += I * K; b += J * K;                                                        \
    }                                                                                              \
}
DEFINE_GRAD(orc_matmul_grad_f32, float)
DEFINE_GRAD(orc_matmul_grad_f64, double)

/* ------------------------------------------------------------------------------------ */
/* qkv_transpose: per-group transposes.  rc: [c x C] -> [C x c] (ops.cu:518-536);          */
/* rr: [c x c] -> transposed (ops.cu:539-557); host :663-715                              */
/* ------------------------------------------------------------------------------------ */
#define DEFINE_TRANSPOSE(NAME, T)                                                                  \
void NAME(const T* m, const int32_t* c, int64_t G, int32_t C, int is_rr, T* out) {                 \
    int64_t p = 0;                                                                                 \
    for (int64_t g = 0; g < G; ++g) {                                                              \
        int64_t rc = c[g];                                                                         \
        if (!is_rr) {                                                                              \
            for (int64_t i = 0; i < C; ++i) for (int64_t j = 0; j < rc; ++j)                       \
                out[p + i * rc + j] = m[p + i + j * C];                                            \
            p += rc * C;                                                                           \
        } else {                                                                                   \
            for (int64_t i = 0; i < rc; ++i) for (int64_t j = 0; j < rc; ++j)                      \
                out[p + i * rc + j] = m[p + i + j * rc];                                           \
            p += rc * rc;                                                                          \
        }                                                                                          \
    }                                                                                              \
}
DEFINE_TRANSPOSE(orc_qkv_transpose_f32, float)
DEFINE_TRANSPOSE(orc_qkv_transpose_f64, double)

/* ------------------------------------------------------------------------------------ */
/* softmax over rows given as sorted dense row ids.                                      */
/* forward  ops.cu:128-167: row max starts from a ZERO-initialised buffer (:137), so the   */
/*          subtracted value is max(0, max_row v); the row sum gets +1e-8 (:164).          */
/* backward ops.cu:169-194: g*y - y * sum_row(g*y)                                         */
/* ------------------------------------------------------------------------------------ */
#define DEFINE_SOFTMAX(FWD, BWD, T, EXPF)                                                          \
void FWD(const int32_t* row, const T* v, int64_t A, T* out) {                                      \
    int64_t s = 0;                                                                                 \
    while (s < A) {                                                                                \
        int64_t e = s; T mx = 0;                                                                   \
        while (e < A && row[e] == row[s]) { if (v[e] > mx) mx = v[e]; ++e; }                       \
        T sum = 0;                                                                                 \
        for (int64_t i = s; i < e; ++i) { out[i] = EXPF(v[i] - mx); sum += out[i]; }               \
        sum += (T)1e-8;                                                                            \
        for (int64_t i = s; i < e; ++i) out[i] = out[i] / sum;                                     \
        s = e;                                                                                     \
    }                                                                                              \
}                                                                                                  \
void BWD(const int32_t* row, const T* y, const T* g, int64_t A, T* out) {                          \
    int64_t s = 0;                                                                                 \
    while (s < A) {                                                                                \
        int64_t e = s; T dot = 0;                                                                  \
        while (e < A && row[e] == row[s]) { dot += g[e] * y[e]; ++e; }                             \
        for (int64_t i = s; i < e; ++i) out[i] = g[i] * y[i] - y[i] * dot;                         \
        s = e;                                                                                     \
    }                                                                                              \
}
DEFINE_SOFTMAX(orc_softmax_fwd_f32, orc_softmax_bwd_f32, float, expf)
DEFINE_SOFTMAX(orc_softmax_fwd_f64, orc_softmax_bwd_f64, double, exp)
