// pybind11 module with the ten operators of the reference's extension module `custom_ops`
// (sparse_swin/ops.cpp:7-18, declarations sparse_swin/ops.h:4-50): same Python names, same positional
// signatures, at::Tensor in and out.  Every function is a thin layer over the C ABI of libsswin3d.so
// (include/sswin3d.h): it checks its arguments as the reference's entry points do (ops.cu:1034-1132),
// allocates outputs and scratch through the caching allocator, and launches on the current HIP stream.
// Unlike sparseswin3d_amd/custom_ops.py it keeps no plan cache between calls: like the reference, each
// matmul_grad / qkv_transpose call derives its offsets from `_c` again.
//
// Built by sparseswin3d_amd/build.py with hipcc (no translation pass, HIP-native torch headers).
#include <torch/extension.h>

// PyTorch on ROCm labels GPU tensors "cuda": guards and streams for them are the *MasqueradingAsCUDA ones
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <string>
#include <tuple>
#include <vector>

#include "../../include/sswin3d.h"

namespace {

void* current_stream(const at::Tensor& t) { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream(); }

#define SSWIN_OK(expr) TORCH_CHECK((expr) == 0, sswin_last_error())

int value_code(const at::Tensor& t) {
    switch (t.scalar_type()) {
        case at::kFloat: return SSWIN_F32;
        case at::kHalf: return SSWIN_F16;
        case at::kBFloat16: return SSWIN_BF16;
        case at::kDouble: return SSWIN_F64;
        default: TORCH_CHECK(false, "unsupported value dtype ", t.scalar_type());
    }
}

void on_gpu(const at::Tensor& t, const char* what) {
    TORCH_CHECK(t.is_cuda(), what, ": the operators run on the GPU only; there is no CPU fallback");
}

at::Tensor scratch(size_t bytes, const at::Tensor& like) {
    return at::empty({(int64_t)(bytes ? bytes : 1)}, like.options().dtype(at::kByte));
}

int product_kind(const std::string& s) {
    if (s == "q_k") return SSWIN_MUL_Q_K;
    if (s == "qk_v") return SSWIN_MUL_QK_V;
    TORCH_CHECK(false, "Invalid mul_type: ", s, ". Expected 'q_k' or 'qk_v'.");
}
int grad_kind(const std::string& s) {
    if (s == "rc_cr") return SSWIN_GRAD_RC_CR;
    if (s == "rr_rc") return SSWIN_GRAD_RR_RC;
    if (s == "cr_rr") return SSWIN_GRAD_CR_RR;
    TORCH_CHECK(false, "Invalid mul_type: ", s, ". Expected 'rc_cr', 'rr_rc' or 'cr_rr'.");
}
int transpose_kind(const std::string& s) {
    if (s == "rc") return SSWIN_TRANSPOSE_RC;
    if (s == "rr") return SSWIN_TRANSPOSE_RR;
    TORCH_CHECK(false, "Invalid mul_type: ", s, ". Expected 'rc', or 'rr'.");
}

// exclusive scans of c and c*c for the value-only operators
at::Tensor scans_of(const at::Tensor& c, void* stream) {
    const int64_t G = c.numel();
    at::Tensor scans = at::empty({2 * std::max<int64_t>(G, 1)}, c.options());
    const size_t bytes = sswin_scan_counts_workspace_bytes(G);
    at::Tensor ws = scratch(bytes, c);
    SSWIN_OK(sswin_scan_counts(c.data_ptr<int32_t>(), G, scans.data_ptr<int32_t>(), ws.data_ptr(), bytes, stream));
    return scans;
}

}  // namespace

// ops.h:4-12, ops.cu:1034-1088
std::tuple<at::Tensor, at::Tensor, std::vector<int32_t>, at::Tensor> matmul_cuda_naive(
    const at::Tensor& mat1_v, const at::Tensor& mat1_idx, const std::vector<int32_t>& mat1_shape,
    const at::Tensor& mat2_v, const at::Tensor& mat2_idx, const std::vector<int32_t>& mat2_shape, std::string mul_type) {
    TORCH_CHECK(mat1_idx.dim() == 2, "Expected mat1_idx.dim() == 2 to be true, but got false.");
    TORCH_CHECK(mat2_idx.dim() == 2, "Expected mat2_idx.dim() == 2 to be true, but got false.");
    TORCH_CHECK(mat1_v.dim() == 1, "Expected mat1_v.dim() == 1 to be true, but got false.");
    TORCH_CHECK(mat2_v.dim() == 1, "Expected mat2_v.dim() == 1 to be true, but got false.");
    const int kind = product_kind(mul_type);
    TORCH_CHECK(mat1_v.scalar_type() == mat2_v.scalar_type(), "mat1 dtype ", mat1_v.scalar_type(),
                " does not match mat2 dtype ", mat2_v.scalar_type());
    TORCH_CHECK(mat1_idx.scalar_type() == mat2_idx.scalar_type(), "mat1 dtype ", mat1_idx.scalar_type(),
                " does not match mat2 dtype ", mat2_idx.scalar_type());
    TORCH_CHECK(mat1_idx.scalar_type() == at::kInt, "mat1 dtype is not int32, but ", mat1_idx.scalar_type());
    TORCH_CHECK(mat1_shape.size() == 4 && mat2_shape.size() == 4 && mat1_shape[0] == mat2_shape[0] &&
                    mat1_shape[1] == mat2_shape[1] && mat1_shape[3] == mat2_shape[2],
                "Invalid shapes: mat1_shape ", mat1_shape, " and mat2_shape ", mat2_shape,
                ". Expected sizes: 4. Expected mat1_shape[0] == mat2_shape[0], mat1_shape[1] == mat2_shape[1], "
                "mat1_shape[3] == mat2_shape[2].");
    on_gpu(mat1_v, "matmul_cuda_naive");
    TORCH_CHECK(mat1_idx.size(0) == 4 && mat2_idx.size(0) == 4, "index matrices must have 4 rows");
    TORCH_CHECK(mat1_idx.size(1) == mat1_v.numel() && mat2_idx.size(1) == mat2_v.numel(), "index and value counts differ");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(mat1_v.device());
    void* stream = current_stream(mat1_v);
    const at::Tensor v1 = mat1_v.contiguous(), v2 = mat2_v.contiguous();
    const at::Tensor i1 = mat1_idx.contiguous(), i2 = mat2_idx.contiguous();
    const at::Tensor& tok = kind == SSWIN_MUL_Q_K ? i1 : i2;       // the operand that carries the token rows
    const int inner = kind == SSWIN_MUL_Q_K ? mat1_shape[3] : mat2_shape[3];
    const int64_t M = tok.size(1);
    std::vector<int32_t> out_shape = {mat1_shape[0], mat1_shape[1], mat1_shape[2], mat2_shape[3]};
    if (M == 0)
        return {at::empty({4, 0}, i1.options()), at::empty({0}, v1.options()), out_shape, at::empty({0}, i1.options())};
    TORCH_CHECK(M % inner == 0, "operand nnz ", M, " is not a multiple of its dense last dimension ", inner);
    const int64_t g_cap = std::max<int64_t>(1, std::min<int64_t>(M / inner, (int64_t)mat1_shape[0] * mat1_shape[1]));
    at::Tensor plan = at::empty({5 * g_cap}, i1.options());
    int64_t totals[4] = {0, 0, 0, 0};
    {
        const size_t bytes = sswin_plan_workspace_bytes(M, inner);
        at::Tensor ws = scratch(bytes, i1);
        SSWIN_OK(sswin_plan_from_indices(tok.data_ptr<int32_t>(), M, inner, plan.data_ptr<int32_t>(), g_cap, totals,
                                         ws.data_ptr(), bytes, stream));
    }
    const int64_t G = totals[0], sum_c2 = totals[2], c_max = totals[3];
    int64_t nnz;
    if (kind == SSWIN_MUL_Q_K) {
        TORCH_CHECK(v2.numel() == M, "'q_k': mat2 holds ", v2.numel(), " values, expected ", M);
        nnz = sum_c2;
    } else {
        TORCH_CHECK(v1.numel() == sum_c2, "'qk_v': mat1 holds ", v1.numel(), " values, expected sum of c*c = ", sum_c2);
        nnz = M;
    }
    at::Tensor out_idx = at::empty({4, nnz}, i1.options());
    at::Tensor out_val = at::empty({nnz}, v1.options());
    SSWIN_OK(sswin_block_matmul(kind, value_code(v1), v1.data_ptr(), v2.data_ptr(), tok.data_ptr<int32_t>(), M, inner,
                                plan.data_ptr<int32_t>(), g_cap, G, c_max, out_val.data_ptr(),
                                out_idx.data_ptr<int32_t>(), nnz, stream));
    return {out_idx, out_val, out_shape, plan.slice(0, 0, G)};
}

// ops.h:15-21, ops.cu:1092-1114
at::Tensor matmul_grad_cuda_naive(const at::Tensor& mat1_v, const at::Tensor& mat2_v, const at::Tensor& _c, int32_t& C,
                                  std::string& mul_type) {
    const int kind = grad_kind(mul_type);
    TORCH_CHECK(mat1_v.scalar_type() == mat2_v.scalar_type(), "mat1 dtype ", mat1_v.scalar_type(),
                " does not match mat2 dtype ", mat2_v.scalar_type());
    TORCH_CHECK(_c.scalar_type() == at::kInt, "_c must be int32");
    on_gpu(mat1_v, "matmul_grad_cuda_naive");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(mat1_v.device());
    void* stream = current_stream(mat1_v);
    const at::Tensor v1 = mat1_v.contiguous(), v2 = mat2_v.contiguous(), c = _c.contiguous();
    const int64_t G = c.numel();
    const at::Tensor scans = scans_of(c, stream);
    // output size: 'rc_cr' -> sum c*c (= numel of the [c x c] operand it pairs with), the others -> sum c*C
    int64_t out_n;
    if (kind == SSWIN_GRAD_RC_CR) {
        TORCH_CHECK(C > 0 && v1.numel() % C == 0 && v1.numel() == v2.numel(), "'rc_cr': operands must hold sum(c)*C values each");
        // sum of c*c = last exclusive scan entry + last c squared: one read-back, as ops.cu:965-968 has
        out_n = G ? (scans[2 * G - 1] + c[G - 1] * c[G - 1]).item<int64_t>() : 0;
    } else {
        out_n = kind == SSWIN_GRAD_RR_RC ? v2.numel() : v1.numel();
    }
    at::Tensor out = at::empty({out_n}, v1.options());
    SSWIN_OK(sswin_block_matmul_grad(kind, value_code(v1), v1.data_ptr(), v2.data_ptr(), c.data_ptr<int32_t>(),
                                     scans.data_ptr<int32_t>(), G, C, kind == SSWIN_GRAD_RC_CR ? v1.numel() : out_n,
                                     out.data_ptr(), stream));
    return out;
}

// ops.h:23-28, ops.cu:293-335
std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor> qkv_sparse_indices(const at::Tensor indices, int& batch_size,
                                                                              int& spatial_dim, int& num_heads, int& c) {
    TORCH_CHECK(indices.dim() == 2 && indices.size(1) == 2, "qkv_sparse_indices: indices must be [N, 2]");
    TORCH_CHECK(indices.scalar_type() == at::kInt, "qkv_sparse_indices: indices must be int32");
    on_gpu(indices, "qkv_sparse_indices");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(indices.device());
    const at::Tensor ind = indices.contiguous();
    const int64_t N = ind.size(0), E = N * num_heads * c;
    at::Tensor idx_qv = at::empty({4, E}, ind.options()), idx_k = at::empty({4, E}, ind.options());
    at::Tensor sorted_qv = at::empty({E}, ind.options()), sorted_k = at::empty({E}, ind.options());
    const size_t bytes = sswin_qkv_sparse_indices_workspace_bytes(N, batch_size, spatial_dim);
    at::Tensor ws = scratch(bytes, ind);
    SSWIN_OK(sswin_qkv_sparse_indices(ind.data_ptr<int32_t>(), N, batch_size, spatial_dim, num_heads, c,
                                      idx_qv.data_ptr<int32_t>(), sorted_qv.data_ptr<int32_t>(), idx_k.data_ptr<int32_t>(),
                                      sorted_k.data_ptr<int32_t>(), ws.data_ptr(), bytes, /*validate=*/1, nullptr,
                                      current_stream(ind)));
    return {idx_qv, sorted_qv, idx_k, sorted_k};
}

// ops.h:30-35, ops.cu:1117-1132
at::Tensor qkv_transpose(const at::Tensor& mat1_v, const at::Tensor& _c, int32_t& C, std::string& mul_type) {
    const int kind = transpose_kind(mul_type);
    TORCH_CHECK(_c.scalar_type() == at::kInt, "_c must be int32");
    on_gpu(mat1_v, "qkv_transpose");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(mat1_v.device());
    void* stream = current_stream(mat1_v);
    const at::Tensor v = mat1_v.contiguous(), c = _c.contiguous();
    const at::Tensor scans = scans_of(c, stream);
    at::Tensor out = at::empty_like(v);
    SSWIN_OK(sswin_block_transpose(kind, value_code(v), v.data_ptr(), c.data_ptr<int32_t>(), scans.data_ptr<int32_t>(),
                                   c.numel(), C, out.data_ptr(), stream));
    return out;
}

// ops.h:38, ops.cu:232-273
at::Tensor flatten_indices_impl(const at::Tensor& indices, const std::vector<int>& sizes) {
    TORCH_CHECK(indices.dim() == 2 && indices.scalar_type() == at::kInt, "flatten_indices: indices must be int32 [ndim, M]");
    TORCH_CHECK((int64_t)sizes.size() == indices.size(0), "flatten_indices: sizes has ", sizes.size(), " entries for ",
                indices.size(0), " index rows");
    on_gpu(indices, "flatten_indices");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(indices.device());
    const at::Tensor ind = indices.contiguous();
    at::Tensor out = at::empty({ind.size(1)}, ind.options());
    std::vector<int32_t> sz(sizes.begin(), sizes.end());
    SSWIN_OK(sswin_flatten_indices(ind.data_ptr<int32_t>(), (int)ind.size(0), ind.size(1), sz.data(), out.data_ptr<int32_t>(),
                                   current_stream(ind)));
    return out;
}

// ops.h:39, ops.cu:276-289
at::Tensor sort_indices_impl(const at::Tensor& flattened_indices) {
    TORCH_CHECK(flattened_indices.scalar_type() == at::kInt, "sort_indices: keys must be int32");
    on_gpu(flattened_indices, "sort_indices");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(flattened_indices.device());
    const at::Tensor keys = flattened_indices.contiguous().view(-1);
    at::Tensor out = at::empty_like(keys);
    const size_t bytes = sswin_sort_indices_workspace_bytes(keys.numel());
    at::Tensor ws = scratch(bytes, keys);
    SSWIN_OK(sswin_sort_indices(keys.data_ptr<int32_t>(), keys.numel(), out.data_ptr<int32_t>(), ws.data_ptr(), bytes,
                                current_stream(keys)));
    return out;
}

// ops.h:40, ops.cu:718-730
std::tuple<at::Tensor, int64_t> return_inverse_impl(const at::Tensor& x, int64_t maxnum) {
    TORCH_CHECK(x.scalar_type() == at::kInt, "return_inverse: x must be int32");
    on_gpu(x, "return_inverse");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    const at::Tensor xc = x.contiguous().view(-1);
    at::Tensor out = at::empty_like(xc);
    if (xc.numel() == 0) return {out, 0};
    int64_t bound = maxnum;
    if (maxnum == -1) {                                      // the table size is data dependent: one read-back, as ops.cu:721
        bound = xc.max().item<int64_t>() + 1;
        TORCH_CHECK(bound >= 1, "return_inverse: all values negative");
        maxnum = bound;
    }
    const size_t bytes = sswin_return_inverse_workspace_bytes(xc.numel(), bound);
    at::Tensor ws = scratch(bytes, xc);
    int64_t count = 0;
    SSWIN_OK(sswin_return_inverse(xc.data_ptr<int32_t>(), xc.numel(), maxnum, out.data_ptr<int32_t>(), &count, ws.data_ptr(),
                                  bytes, current_stream(xc)));
    return {out, count};
}

// ops.h:41, ops.cu:32-103
at::Tensor unique_consecutive_indices(const at::Tensor& nums) {
    TORCH_CHECK(nums.dim() == 1, "unique_consecutive_indices: expected a 1-D tensor");
    int code;
    switch (nums.scalar_type()) {
        case at::kInt: code = SSWIN_I32; break;
        case at::kLong: code = SSWIN_I64; break;
        case at::kShort: code = SSWIN_I16; break;
        case at::kChar: code = SSWIN_I8; break;
        case at::kByte: code = SSWIN_U8; break;
        default: TORCH_CHECK(false, "unique_consecutive_indices: unsupported dtype ", nums.scalar_type());
    }
    on_gpu(nums, "unique_consecutive_indices");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(nums.device());
    const at::Tensor keys = nums.contiguous();
    at::Tensor out = at::empty({keys.numel()}, keys.options().dtype(at::kInt));
    const size_t bytes = sswin_unique_consecutive_workspace_bytes(keys.numel());
    at::Tensor ws = scratch(bytes, keys);
    SSWIN_OK(sswin_unique_consecutive_indices(keys.data_ptr(), code, keys.numel(), out.data_ptr<int32_t>(), ws.data_ptr(), bytes,
                                              current_stream(keys)));
    return out;
}

namespace {
bool is_16bit(const at::Tensor& t) { return t.scalar_type() == at::kHalf || t.scalar_type() == at::kBFloat16; }
void check_softmax(const at::Tensor& indices, const at::Tensor& values, const char* who) {
    TORCH_CHECK(indices.scalar_type() == at::kInt, who, ": row ids must be int32");
    TORCH_CHECK(values.scalar_type() == at::kFloat || values.scalar_type() == at::kDouble || is_16bit(values), who,
                ": values must be fp32, fp64, fp16 or bf16");
    TORCH_CHECK(indices.numel() == values.numel(), who, ": ", indices.numel(), " row ids for ", values.numel(), " values");
    on_gpu(values, who);
}
}  // namespace

// ops.h:43-45, ops.cu:128-167.  16-bit values (the reference dispatches AT_DISPATCH_FLOATING_TYPES_AND_HALF, ops.cu:140)
// are computed in fp32 and rounded once at the end.
at::Tensor softmax_last_dim_forward(const at::Tensor& indices, const at::Tensor& values) {
    check_softmax(indices, values, "softmax_last_dim_forward");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(values.device());
    const at::Tensor rows = indices.contiguous();
    const at::Tensor v = is_16bit(values) ? values.to(at::kFloat).contiguous() : values.contiguous();
    at::Tensor out = at::empty_like(v);
    SSWIN_OK(sswin_softmax_last_dim_forward(rows.data_ptr<int32_t>(), v.data_ptr(), value_code(v), v.numel(), out.data_ptr(),
                                            current_stream(v)));
    return is_16bit(values) ? out.to(values.scalar_type()) : out;
}

// ops.h:47-50, ops.cu:169-194
at::Tensor softmax_last_dim_backward(const at::Tensor& indices, const at::Tensor& values, const at::Tensor& grad_values) {
    check_softmax(indices, values, "softmax_last_dim_backward");
    TORCH_CHECK(grad_values.scalar_type() == values.scalar_type() && grad_values.numel() == values.numel(),
                "softmax_last_dim_backward: gradient and output differ in dtype or size");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(values.device());
    const bool narrow = is_16bit(values);
    const at::Tensor rows = indices.contiguous();
    const at::Tensor y = narrow ? values.to(at::kFloat).contiguous() : values.contiguous();
    const at::Tensor g = narrow ? grad_values.to(at::kFloat).contiguous() : grad_values.contiguous();
    at::Tensor out = at::empty_like(y);
    SSWIN_OK(sswin_softmax_last_dim_backward(rows.data_ptr<int32_t>(), y.data_ptr(), g.data_ptr(), value_code(y), y.numel(),
                                             out.data_ptr(), current_stream(y)));
    return narrow ? out.to(values.scalar_type()) : out;
}

// the ten names of the reference's module (ops.cpp:7-18), positional arguments as in ops.h
PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("matmul_cuda_naive", &matmul_cuda_naive,
          "(mat1_v, mat1_idx, mat1_shape, mat2_v, mat2_idx, mat2_shape, mul_type 'q_k'|'qk_v') -> (idx, val, shape, group sizes): "
          "window-blocked COO product on the matrix cores");
    m.def("matmul_grad_cuda_naive", &matmul_grad_cuda_naive,
          "(mat1_v, mat2_v, group sizes, C, mul_type 'rc_cr'|'rr_rc'|'cr_rr') -> values of the gradient product");
    m.def("qkv_sparse_indices", &qkv_sparse_indices,
          "(indices [N,2], batch_size, spatial_dim, num_heads, c) -> (Q/V index matrix, its sort order, K^T index matrix, its "
          "sort order), from a presence bitmap instead of a sort");
    m.def("flatten_indices", &flatten_indices_impl, "(indices [ndim,M], sizes) -> row-major int32 key per column");
    m.def("sort_indices", &sort_indices_impl, "(keys) -> stable ascending argsort, int32");
    m.def("return_inverse", &return_inverse_impl, "(keys, maxnum) -> (rank of every key among the distinct keys, their number)");
    m.def("unique_consecutive_indices", &unique_consecutive_indices, "(keys) -> 0-based rank of the run each key belongs to");
    m.def("softmax_last_dim_forward", &softmax_last_dim_forward,
          "(row ids, values) -> exp(v - max(0, rowmax)) / (rowsum + 1e-8) per row");
    m.def("softmax_last_dim_backward", &softmax_last_dim_backward, "(row ids, softmax output, gradient) -> y (g - sum_row g y)");
    m.def("qkv_transpose", &qkv_transpose, "(values, group sizes, C, 'rc'|'rr') -> every group's block transposed");
}
