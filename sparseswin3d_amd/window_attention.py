"""Sparse window attention on top of the HIP operator module.

Host-side mirror of the attention part of the reference's ``sparse_swin/swin3d_base.py``
(same public names, argument meaning and error behaviour), written against
:mod:`sparseswin3d_amd.custom_ops`:

* :class:`SparseTensor` — 4-D COO container with int32 indices            (ref ``:29-65``)
* :func:`spspmm_block_naive` / ``_spspmm_block_naive``                      (ref ``:68-158``)
* :func:`softmax_last_dim` / ``_softmax_last_dim``                          (ref ``:161-197``)
* :func:`qkv_sparse_cuda`, :func:`sp_add_rpb`, :func:`sp_add_mask`          (ref ``:483-498, 557-581``)
* :class:`WindowAttentionSparse`                                            (ref ``:589-677``)

The input of :class:`WindowAttentionSparse` is any object with the attributes ``features``
[N, D], ``indices`` int32 [N, 2] = (window, pos), ``spatial_shape`` = (tokens per window,),
``batch_size`` = number of window slots, and ``replace_feature(new)`` — a
``spconv.SparseConvTensor`` after window partition, or :class:`SparseVoxelTensor` below.
"""
from __future__ import annotations

import contextlib
import copy
import math
import warnings
from typing import Sequence

import torch
import torch.nn as nn
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from . import _lib
from . import custom_ops as ops


class SparseVoxelTensor:
    """Minimal stand-in for ``spconv.SparseConvTensor`` (features + integer voxel indices).

    spconv has no ROCm build in this environment; real spconv tensors work too because only
    these five members are used.
    """

    def __init__(self, features, indices, spatial_shape, batch_size):
        self.features = features
        self.indices = indices
        self.spatial_shape = tuple(spatial_shape) if not isinstance(spatial_shape, tuple) else spatial_shape
        self.batch_size = batch_size

    def replace_feature(self, new_features):
        out = copy.copy(self)
        out.features = new_features
        return out


def replace_feature(out, new_features):
    return out.replace_feature(new_features)


class _LazyIndices:
    """The [4, nnz] index matrix of a block product, written by the library the first time somebody reads it.  The
    matrix is a function of the token operand's indices alone, and a composition of the operators that goes from
    product to product by the group sizes never reads it (16 bytes per entry, 164 MB for the attention of 100 000
    voxels)."""

    def __init__(self, fn):
        self.fn, self.value = fn, None

    def get(self):
        if self.value is None:
            self.value, self.fn = self.fn(), None
        return self.value


class SparseTensor:
    """4-D COO tensor: ``indices`` int32 [4, nnz], ``values`` [nnz], ``shape`` list of 4."""

    def __init__(self, indices, values, shape, group_counts=None, row_positions=None):
        if not isinstance(indices, _LazyIndices):
            assert indices.shape[0] == 4, "Invalid shape"
            assert indices.ndim == 2, "Invalid shape"
        assert values.ndim == 1, "Invalid shape"
        assert len(shape) == 4, "Invalid shape"
        self._idx = indices
        self.values = values
        self.shape = shape
        # tokens per (window, head) group when the tensor is a 'q_k' product (or shares its index matrix):
        # lets softmax_last_dim number the attention rows without hashing the index matrix
        self.group_counts = group_counts
        # window position of every token row in group order (int32 [sum c]) when the tensor is a 'q_k' product:
        # what the bias and mask kernels need of the index matrix
        self.row_positions = row_positions

    @property
    def indices(self):
        if isinstance(self._idx, _LazyIndices):
            self._idx = self._idx.get()
        return self._idx

    @indices.setter
    def indices(self, value):
        self._idx = value

    def index_source(self):
        """The index matrix, or the object that will produce it: what a tensor with the same structure is built from
        without forcing the matrix into existence."""
        if isinstance(self._idx, _LazyIndices) and self._idx.value is not None:
            self._idx = self._idx.value
        return self._idx

    def __repr__(self):
        return f"SparseTensor(indices={self.indices}, values={self.values}, shape={self.shape})"

    def _sorted_order(self, indices, shape):
        # the row-major hash is int32 (sparse_swin/ops.cu:264): beyond 2^31 it wraps and the sorted order is
        # undefined, in the reference as well; refuse instead of returning a mis-ordered tensor
        cells = 1
        for extent in shape:
            cells *= int(extent)
        if cells > 2 ** 31:
            raise RuntimeError(f"SparseTensor of shape {list(shape)}: its {cells} cells do not fit the int32 hash "
                               "that orders the entries (coalesce / permute); split the batch")
        return ops.sort_indices(ops.flatten_indices(indices, shape))

    def coalesce(self):
        order = self._sorted_order(self.indices, self.shape)
        return SparseTensor(self.indices.index_select(1, order), self.values.index_select(0, order), self.shape)

    def permute(self, dims):
        if len(dims) != len(self.shape):
            raise ValueError(
                f"The length of dims {dims} must match the number of dimensions in shape {self.shape}.")
        if sorted(dims) != list(range(len(self.shape))):
            raise ValueError(f"dims {dims} must be a permutation of the dimensions [0, {len(self.shape) - 1}].")
        new_shape = [self.shape[d] for d in dims]
        new_indices = self.indices[list(dims), :]
        order = None
        if tuple(dims) == (0, 2, 1, 3) and self.indices.is_cuda:
            # an attention output: every head of a window holds the same rows, so the sorted order of the
            # permuted indices follows from the group structure (checked on the device); no hash, no sort
            order = ops.permute_heads_order(self.indices, self.shape)
        if order is None:
            order = self._sorted_order(new_indices, new_shape)
        return SparseTensor(new_indices.index_select(1, order), self.values.index_select(0, order), new_shape)

    def __mul__(self, other):
        if isinstance(other, (int, float)):
            return SparseTensor(self.index_source(), self.values * other, self.shape, self.group_counts,
                                self.row_positions)
        raise NotImplementedError


# ------------------------------------------------------------------------------------------
# block products with autograd
# ------------------------------------------------------------------------------------------
_MUL_TYPES = ("q_k", "qk_v")


def _check_mul_type(mul_type):
    if mul_type not in _MUL_TYPES:
        raise ValueError(f"Invalid value for 'mul': {mul_type}. Must be 'q_k' or 'qk_v'.")


# The reference's backward of a block product (swin3d_base.py:121-134) transposes both operands of the second gradient
# with ``qkv_transpose`` and multiplies the copies.  True: do the same (four transposed copies per attention); False
# (default): the product reads the operands as they are (``ops.matmul_grad_untransposed``, same sums in the same order).
TRANSPOSED_COPIES = False


class _spspmm_block_naive(Function):
    """Window-blocked sparse x sparse product; gradients flow to both value arrays."""

    @staticmethod
    def forward(ctx, mat1_v, mat1_idx, mat1_shape, mat2_v, mat2_idx, mat2_shape, mul_type, want_indices=True):
        _check_mul_type(mul_type)
        mat3_idx, mat3_v, mat3_shape, counts = ops.block_product(
            mat1_v, mat1_idx, mat1_shape, mat2_v, mat2_idx, mat2_shape, mul_type, indices=want_indices)
        ctx.save_for_backward(mat2_v, mat1_v, counts)
        ctx.mul_type = mul_type
        ctx.inner = mat1_shape[-1] if mul_type == "q_k" else mat2_shape[-1]
        ctx.mark_non_differentiable(*(t for t in (mat3_idx, counts) if t is not None))
        # without this autograd hands backward a zero tensor for every output that has no gradient, the [4, nnz]
        # index matrix included (a 360 MB fill for 7^3 windows)
        ctx.set_materialize_grads(False)
        return mat3_idx, mat3_v, mat3_shape, counts

    @staticmethod
    @once_differentiable
    def backward(ctx, _grad_idx, grad_v, _grad_shape, _grad_counts):
        if grad_v is None:
            return None, None, None, None, None, None, None, None
        grad_v = grad_v.contiguous()
        mat2_v, mat1_v, counts = ctx.saved_tensors
        inner = ctx.inner
        if ctx.mul_type == "q_k":
            # S = Q K:  dQ = dS K^T (K^T is stored [C x c], so it is read along its rows);
            #           dK^T = Q^T dS, assembled from the two transposed operands.
            grad_mat1 = ops.matmul_grad_cuda_naive(grad_v, mat2_v, counts, inner, "rr_rc")
            if TRANSPOSED_COPIES:
                mat1_t = ops.qkv_transpose(mat1_v, counts, inner, "rc")
                grad_t = ops.qkv_transpose(grad_v, counts, inner, "rr")
                grad_mat2 = ops.matmul_grad_cuda_naive(mat1_t, grad_t, counts, inner, "cr_rr")
            else:
                grad_mat2 = ops.matmul_grad_untransposed(mat1_v, grad_v, counts, inner, "tc_rr")
        else:
            # O = P V:  dP = dO V^T;  dV = P^T dO.
            grad_mat1 = ops.matmul_grad_cuda_naive(grad_v, mat2_v, counts, inner, "rc_cr")
            if TRANSPOSED_COPIES:
                mat1_t = ops.qkv_transpose(mat1_v, counts, inner, "rr")
                grad_t = ops.qkv_transpose(grad_v, counts, inner, "rc")
                grad_mat2 = ops.matmul_grad_cuda_naive(mat1_t, grad_t, counts, inner, "rr_rc")
            else:
                grad_mat2 = ops.matmul_grad_untransposed(mat1_v, grad_v, counts, inner, "tr_rc")
        return grad_mat1, None, None, grad_mat2, None, None, None, None


def spspmm_block_naive(mat1: SparseTensor, mat2: SparseTensor, mul_type="q_k") -> SparseTensor:
    """Window-blocked product of two sparse tensors.  On the GPU the result's index matrix is written when it is
    first read (``result.indices``): the products, the bias / mask pass and the softmax of the attention go by the
    group sizes and never ask for it."""
    _check_mul_type(mul_type)
    # only the operand with the token rows (Q for 'q_k', V for 'qk_v') is read for its indices; the other one's may
    # still be unwritten and stay so
    idx1 = mat1.indices if mul_type == "q_k" else _written_indices(mat1)
    idx2 = mat2.indices if mul_type == "qk_v" else _written_indices(mat2)
    lazy = mat1.values.is_cuda
    idx, val, shape, counts = _spspmm_block_naive.apply(mat1.values, idx1, mat1.shape, mat2.values, idx2, mat2.shape,
                                                        mul_type, not lazy)
    if lazy:
        s1, s2 = list(mat1.shape), list(mat2.shape)
        idx = _LazyIndices(lambda: ops.block_product(None, idx1, s1, None, idx2, s2, mul_type, values=False)[0])
    if mul_type != "q_k":
        return SparseTensor(idx, val, shape)
    inner = int(mat1.shape[-1])
    return SparseTensor(idx, val, shape, counts, idx1[2, ::inner].contiguous() if lazy else None)


def _written_indices(mat: SparseTensor):
    src = mat.index_source()
    return None if isinstance(src, _LazyIndices) else src


# ------------------------------------------------------------------------------------------
# softmax over the last dimension of a COO tensor
# ------------------------------------------------------------------------------------------
class _softmax_last_dim(Function):
    @staticmethod
    def forward(ctx, mat_v, mat_idx, mat_shape, group_counts=None):
        if group_counts is not None:
            # a 'q_k' product: its attention rows are numbered from the group sizes (same ids, no hash of the indices)
            rows = ops.softmax_rows_from_counts(group_counts, mat_v.numel())
        else:
            rows = ops.unique_consecutive_indices(ops.flatten_indices(mat_idx, mat_shape))
        out = ops.softmax_last_dim_forward(rows, mat_v)
        ctx.save_for_backward(out, rows)
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_mat):
        out, rows = ctx.saved_tensors
        return ops.softmax_last_dim_backward(rows, out, grad_mat.contiguous()), None, None, None


def softmax_last_dim(mat: SparseTensor) -> SparseTensor:
    dtype = mat.values.dtype
    out = _softmax_last_dim.apply(mat.values.float(), None if mat.group_counts is not None else mat.indices[:3],
                                  mat.shape[:-1], mat.group_counts)
    return SparseTensor(mat.index_source(), out.to(dtype), mat.shape, mat.group_counts, mat.row_positions)


# ------------------------------------------------------------------------------------------
# glue around the operators
# ------------------------------------------------------------------------------------------
class _SortedOperandValues(Function):
    """Values of Q, K^T, V in sorted operand order from ``qkv`` [N, 3, H, hd].  The reference gathers them
    through the permutations of ``qkv_sparse_indices`` (swin3d_base.py:483-498) and autograd returns the
    gradients through ``index_add``; the same permutations applied directly, in both directions."""

    @staticmethod
    def forward(ctx, qkv, omap, q_scale=1.0):
        n_vox, _, num_heads, c = qkv.shape
        flat = qkv.contiguous().view(n_vox, 3 * num_heads * c)
        out = [torch.empty(n_vox * num_heads * c, dtype=qkv.dtype, device=qkv.device) for _ in range(3)]
        # one launch for the three; Q takes its factor on the way (the module's `q * self.scale`, swin3d_base.py:660)
        ops.operand_copy_qkv(flat, *out, omap, num_heads, c, True, q_scale)
        ctx.save_for_backward(omap)
        ctx.shape = qkv.shape
        ctx.q_scale = q_scale
        return tuple(out)

    @staticmethod
    @once_differentiable
    def backward(ctx, d_q, d_k, d_v):
        (omap,) = ctx.saved_tensors
        n_vox, _, num_heads, c = ctx.shape
        d_qkv = torch.empty(ctx.shape, dtype=d_q.dtype, device=d_q.device)
        flat = d_qkv.view(n_vox, 3 * num_heads * c)
        ops.operand_copy_qkv(flat, d_q.contiguous(), d_k.contiguous(), d_v.contiguous(), omap, num_heads, c, False, ctx.q_scale)
        return d_qkv, None, None


class _OperandToVoxels(Function):
    """Values of a [B, H, n, hd] product in Q/V order -> token rows [N, H*hd] in voxel order: what
    ``permute((0, 2, 1, 3))``, ``return_inverse`` and ``index_select`` arrive at in the reference
    (swin3d_base.py:672-675)."""

    @staticmethod
    def forward(ctx, val, omap, num_heads, c):
        n_vox = (omap.numel() - 2) // 3
        out = torch.empty(n_vox, num_heads * c, dtype=val.dtype, device=val.device)
        ops.operand_copy(out, 0, val.contiguous(), omap, num_heads, c, 0, False)
        ctx.save_for_backward(omap)
        ctx.heads = (num_heads, c)
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        (omap,) = ctx.saved_tensors
        num_heads, c = ctx.heads
        grad = grad.contiguous()
        d_val = torch.empty(grad.numel(), dtype=grad.dtype, device=grad.device)
        ops.operand_copy(grad, 0, d_val, omap, num_heads, c, 0, True)
        return d_val, None, None, None


def qkv_sparse_cuda(qkv: torch.Tensor, indices: torch.Tensor, batch_size: int, spatial_shape, plan=None, q_scale=1.0):
    """Sorted COO operands Q [B,H,n,hd], K^T [B,H,hd,n], V [B,H,n,hd] from ``qkv`` [N,3,H,hd]
    (reference swin3d_base.py:483-498: same tensors; the index matrices and values are written in sorted
    order directly instead of being expanded, hashed, sorted and gathered).  The returned tensors carry
    ``operand_map``, which :class:`_OperandToVoxels` takes to bring a product back to voxel order.
    ``q_scale``: Q's values come out multiplied by it (``q * q_scale`` without a pass of its own)."""
    num_heads, c = qkv.shape[2:]
    n = spatial_shape
    if plan is not None:
        # a token plan of these indices made earlier (possibly still in flight, possibly shared with other modules)
        plan.finish()
        omap = torch.cat([plan.tokens[:3 * plan.N], _valid_status(plan.N, indices.device)])
    elif qkv.is_cuda and indices.shape[0] > 0 and indices.dtype == torch.int32 and num_heads < 256:
        # One token plan gives both what the operands need (voxel, first rank and size of its window by rank: the
        # operand map) and what the block products need (sizes and offsets of the (window, head) groups), so neither
        # the operand map's own ranking nor the products' pass over the [4, E] index matrix runs.  Invalid
        # (window, pos) pairs raise here.
        from . import fused
        plan = fused.TokenPlan(indices, batch_size, n, num_heads, tasks=False)
        omap = torch.cat([plan.tokens[:3 * plan.N], _valid_status(plan.N, indices.device)])
    else:
        omap = ops.operand_map(indices, batch_size, n)
    # the index matrix of K^T is read by nobody in the attention (the 'q_k' product takes its structure from Q):
    # it is written when it is first asked for
    idx_qv, _ = ops.sorted_coo_indices(indices, omap, num_heads, c, k=False)
    idx_k = _LazyIndices(lambda: ops.sorted_coo_indices(indices, omap, num_heads, c, qv=False)[1])
    if plan is not None and plan.G > 0:
        # group table of the products: the token plan's, with the row offset of a group in place of the first rank
        # of its window (row_start = H * T + head * c)
        table = plan.plan.clone().view(5, plan.g_cap)
        table[1].mul_(num_heads).addcmul_(table[4], table[0])
        ops.register_index_plan(idx_qv, c, table.view(-1), plan.g_cap, plan.G, num_heads * plan.N, plan.A, plan.c_max)
    q_val, k_val, v_val = _SortedOperandValues.apply(qkv, omap, float(q_scale))
    q = SparseTensor(idx_qv, q_val, [batch_size, num_heads, n, c])
    k_t = SparseTensor(idx_k, k_val, [batch_size, num_heads, c, n])
    v = SparseTensor(idx_qv, v_val, [batch_size, num_heads, n, c])
    q.operand_map = k_t.operand_map = v.operand_map = omap
    return q, k_t, v


_STATUS_OK = {}


def _valid_status(n_vox: int, device):
    """The validity pair {pairs out of range = 0, distinct pairs = N} that ends an operand map."""
    key = (device, n_vox)
    if key not in _STATUS_OK:
        if len(_STATUS_OK) > 64:
            _STATUS_OK.clear()
        _STATUS_OK[key] = torch.tensor([0, n_vox], dtype=torch.int32, device=device)
    return _STATUS_OK[key]


def sp_add_rpb(sparse: SparseTensor, dense: torch.Tensor) -> SparseTensor:
    """``values += dense[head, pos_i, pos_j]`` for a dense bias [H, n, n]."""
    i = sparse.indices
    flat = i[1] * (dense.shape[1] * dense.shape[2]) + i[2] * dense.shape[2] + i[3]
    return SparseTensor(i, sparse.values + dense.reshape(-1).index_select(0, flat), sparse.shape, sparse.group_counts)


def sp_add_mask(sparse: SparseTensor, dense: torch.Tensor) -> SparseTensor:
    """Shifted-window mask: ``-100`` where the region ids [nW, n] of the two tokens differ."""
    i = sparse.indices
    row = (i[0] % dense.shape[0]) * dense.shape[1]
    flat = dense.reshape(-1)
    differ = flat.index_select(0, row + i[3]) != flat.index_select(0, row + i[2])
    return SparseTensor(i, sparse.values + differ.to(sparse.values.dtype) * -100.0, sparse.shape, sparse.group_counts)


class _GroupBiasMask(Function):
    """``sp_add_mask(sp_add_rpb(attn, bias), mask)`` for a 'q_k' product whose bias comes from a relative position
    table with a linear index: one pass over the values forward (positions read per group, not per entry), the table
    gradient summed in a fixed order backward (the reference's composition goes through a linear index per entry, two
    gathers, and an ``index_add`` into the dense bias)."""

    @staticmethod
    def forward(ctx, values, table, row_pos, gp, n, mask, table_index, token_plan=None):
        # row_pos: window position of every token row in group order (int32 [sum c]); token_plan: the TokenPlan the
        # product's group table was taken from, if any (its task descriptors let the backward deal the work evenly)
        idx = row_pos
        num_heads = table.shape[1]
        table32 = table.detach().to(torch.float32).contiguous()
        ctx.save_for_backward(idx)
        ctx.meta = (gp, n, table_index, table.shape[0], num_heads, table.dtype)
        ctx.token_plan = token_plan
        if table.shape[0] < (1 << 15):
            # the kernel reads the table itself (a few KB; the gathered [H, n, n] bias of 7^3 windows is 1.4 MB)
            return ops.group_add_table_bias_mask(values, idx, gp, n, table32, table_index.code, table_index.offset0, mask)
        from . import _lib
        import ctypes as C
        bias32 = torch.empty((num_heads, n, n), dtype=torch.float32, device=values.device)
        with _lib.on_device(values.device):
            _lib.check(_lib.load().sswin_bias_from_table(
                C.c_void_p(table32.data_ptr()), table32.shape[0], num_heads, C.c_void_p(table_index.code.data_ptr()),
                table_index.offset0, n, C.c_void_p(bias32.data_ptr()),
                _lib.stream_handle(values.device)))
        return ops.group_add_bias_mask(values, idx, gp, n, bias32, mask)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        (idx,) = ctx.saved_tensors
        gp, n, table_index, table_rows, num_heads, table_dtype = ctx.meta
        d_table = None
        if ctx.needs_input_grad[1]:
            from . import fused
            tp = ctx.token_plan
            if tp is not None and tp.H == num_heads and tp.A == grad.numel():
                # the values of the product lie in the plan's group order: the fused path's table gradient applies
                # as it is (batches dealt from the task descriptors where every window has one)
                d_table = fused._bias_gradient(tp, num_heads, grad.float().contiguous(), (table_dtype, (table_rows, num_heads)),
                                               table_index)
            else:
                d_table = ops.group_bias_table_grad(grad.float(), idx, gp, num_heads, n, table_index.code,
                                                    table_index.offset0, table_rows).to(table_dtype)
        return grad, d_table, None, None, None, None, None, None


def sp_add_table_bias_and_mask(sparse: SparseTensor, table: torch.Tensor, table_index, mask, token_plan=None) -> SparseTensor:
    """``sp_add_rpb`` with the bias gathered from ``table`` [rows, H], then ``sp_add_mask``, in one pass (a 'q_k'
    product with its group sizes attached, int8 mask or None); None if the input is not of that kind."""
    if sparse.group_counts is None or table_index is None or (mask is not None and mask.dtype != torch.int8):
        return None
    gp = ops.group_plan(sparse.group_counts)
    n = sparse.shape[2]
    if gp is None or gp.c_max > 512 or n > 384:
        return None
    row_pos = sparse.row_positions if sparse.row_positions is not None else ops.group_row_positions(sparse.indices, gp)
    out = _GroupBiasMask.apply(sparse.values, table, row_pos, gp, n, mask, table_index, token_plan)
    return SparseTensor(sparse.index_source(), out, sparse.shape, sparse.group_counts, row_pos)


def trunc_normal_(tensor, mean=0.0, std=1.0, a=-2.0, b=2.0):
    """Truncated-normal initialisation (inverse-CDF sampling, clamp to [a, b])."""
    if std <= 0:
        raise ValueError("the standard deviation should be greater than zero.")
    if a >= b:
        raise ValueError("minimum cutoff value (a) should be smaller than maximum cutoff value (b).")

    def cdf(x):
        return 0.5 * (1.0 + math.erf(x / math.sqrt(2.0)))

    with torch.no_grad():
        lo, hi = cdf((a - mean) / std), cdf((b - mean) / std)
        tensor.uniform_(2 * lo - 1, 2 * hi - 1).erfinv_().mul_(std * math.sqrt(2.0)).add_(mean)
        return tensor.clamp_(min=a, max=b)


@contextlib.contextmanager
def _rocblas_gemm():
    """Run the enclosed matrix products on rocBLAS.  On [10^5 x 96] x [96 x 96..288] shapes its
    kernels take 25 / 28 / 46 us (proj forward, input gradient, weight gradient at N = 107 500)
    where the hipBLASLt heuristics pick tiles that take 40 / 40 / 220 us."""
    prev = torch.backends.cuda.preferred_blas_library()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        torch.backends.cuda.preferred_blas_library("cublas")
    try:
        yield
    finally:
        torch.backends.cuda.preferred_blas_library(prev)


_SUM_DTYPE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _column_sum(t: torch.Tensor) -> torch.Tensor:
    """``t.sum(0)`` of a tall [N, P] matrix on the GPU through the library's two-stage kernel (sums
    in fp32, fixed order; about twice as fast as the generic reduction on [10^5 x 288])."""
    p = t.shape[1] if t.dim() == 2 else 0
    if not (t.is_cuda and t.dtype in _SUM_DTYPE and t.dim() == 2 and p % 4 == 0 and t.shape[0] > 0):
        return t.sum(0)
    import ctypes as C
    from . import _lib
    lib = _lib.load()
    t = t.contiguous()
    with _lib.on_device(t.device):
        out = torch.empty(p, dtype=torch.float32, device=t.device)
        nbytes = lib.sswin_column_sum_workspace_bytes(t.shape[0], p)
        ws = torch.empty(int(nbytes), dtype=torch.uint8, device=t.device)
        _lib.check(lib.sswin_column_sum(C.c_void_p(t.data_ptr()), _SUM_DTYPE[t.dtype], t.shape[0], p,
                                        C.c_void_p(out.data_ptr()), C.c_void_p(ws.data_ptr()), nbytes,
                                        _lib.stream_handle(t.device)))
    return out.to(t.dtype)


def _split_linear_forward(x: torch.Tensor, weight: torch.Tensor, bias):
    """``x @ W^T + b`` through the library's matrix-core kernel for fp32 (operands split into bf16
    pieces, fp32 accuracy), or None when the shape or dtype is outside what that kernel takes."""
    if not (x.is_cuda and x.dtype == torch.float32 and weight.dtype == torch.float32 and x.dim() == 2
            and x.shape[0] > 0 and (bias is None or bias.dtype == torch.float32)):
        return None
    import ctypes as C
    from . import _lib
    lib = _lib.load()
    n, k = x.shape
    p = weight.shape[0]
    if not lib.sswin_tall_linear_supported(p, k) or (k > 192 and n < 20000):   # few rows, many channels: the library wins
        return None
    x = x.contiguous()
    weight = weight.contiguous()
    if x.data_ptr() % 16:
        x = x.clone()
    if weight.data_ptr() % 16:
        weight = weight.clone()
    with _lib.on_device(x.device):
        y = torch.empty(n, p, dtype=torch.float32, device=x.device)
        b = bias.contiguous() if bias is not None else None
        _lib.check(lib.sswin_tall_linear_forward(C.c_void_p(x.data_ptr()), n, k, C.c_void_p(weight.data_ptr()),
                                                 C.c_void_p(b.data_ptr() if b is not None else None), p,
                                                 C.c_void_p(y.data_ptr()),
                                                 _lib.stream_handle(x.device)))
    return y


def _split_linear_input_grad(grad_out: torch.Tensor, weight: torch.Tensor):
    """``grad_out @ W`` through the library's matrix-core kernels for fp32, where they beat the library
    GEMM (see the row thresholds below), else None."""
    if not (grad_out.is_cuda and grad_out.dtype == torch.float32 and weight.dtype == torch.float32
            and grad_out.dim() == 2 and grad_out.shape[0] > 0):
        return None
    import ctypes as C
    from . import _lib
    lib = _lib.load()
    n, p = grad_out.shape
    k = weight.shape[1]
    # measured against rocBLAS on an MI355X: the 96-column kernel wins from 32 rows on, the kernel that keeps
    # all of W on the CU (192..288 columns) from about 16 000 rows, the chunked one from about 60 000
    enough_rows = n >= 32 if p == 96 else n >= 16000 if p <= 288 else n >= 60000
    if p < 96 or (96 < p < 192) or not enough_rows or not lib.sswin_tall_linear_input_grad_supported(p, k):
        return None
    weight = weight.contiguous()
    if grad_out.data_ptr() % 16:
        grad_out = grad_out.clone()
    with _lib.on_device(grad_out.device):
        dx = torch.empty(n, k, dtype=torch.float32, device=grad_out.device)
        _lib.check(lib.sswin_tall_linear_input_grad(C.c_void_p(grad_out.data_ptr()), n, p, C.c_void_p(weight.data_ptr()), k,
                                                    C.c_void_p(dx.data_ptr()),
                                                    _lib.stream_handle(grad_out.device)))
    return dx


def _split_linear_weight_grad(grad_out: torch.Tensor, x: torch.Tensor, want_bias: bool):
    """``(grad_out^T @ x, grad_out.sum(0))`` through the library's matrix-core kernel for fp32 (one
    pass over both operands, partial sums added in a fixed order), or ``(None, None)`` when the shape
    or dtype is outside what that kernel takes."""
    if not (x.is_cuda and x.dtype == torch.float32 and grad_out.dtype == torch.float32 and x.dim() == 2
            and grad_out.dim() == 2 and x.shape[0] > 0):
        return None, None
    import ctypes as C
    from . import _lib
    lib = _lib.load()
    n, k = x.shape
    p = grad_out.shape[1]
    if k > 96 and n < 16000:                     # passes of 96 columns over few rows: the library wins
        return None, None
    nbytes = int(lib.sswin_tall_linear_weight_grad_workspace_bytes(n, p, k))
    if nbytes == 0:
        return None, None
    x = x.contiguous()
    with _lib.on_device(x.device):
        dw = torch.empty(p, k, dtype=torch.float32, device=x.device)
        db = torch.empty(p, dtype=torch.float32, device=x.device) if want_bias else None
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        _lib.check(lib.sswin_tall_linear_weight_grad(C.c_void_p(grad_out.data_ptr()), C.c_void_p(x.data_ptr()), n, p, k,
                                                     C.c_void_p(dw.data_ptr()),
                                                     C.c_void_p(db.data_ptr() if db is not None else None),
                                                     C.c_void_p(ws.data_ptr()), nbytes,
                                                     _lib.stream_handle(x.device)))
    return dw, db


class _TallLinear(Function):
    """``x @ W^T + b`` for a very tall ``x`` [N, in] (N = number of voxels).  The fp32 forward runs on
    the bf16 matrix cores with exactly split operands where the shape allows, and so do the weight
    and bias gradient and the input gradient of wide layers; everything else is a library GEMM, routed
    to the BLAS backend that handles tall-skinny shapes best (see :func:`_rocblas_gemm`)."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        y = _split_linear_forward(x, weight, bias)
        if y is not None:
            return y
        with _rocblas_gemm():
            return torch.nn.functional.linear(x, weight, bias)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out):
        x, weight = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        grad_x = grad_w = grad_b = None
        want_b = ctx.has_bias and ctx.needs_input_grad[2]
        if ctx.needs_input_grad[1]:
            grad_w, grad_b = _split_linear_weight_grad(grad_out, x, want_b)
        if ctx.needs_input_grad[0]:
            grad_x = _split_linear_input_grad(grad_out, weight)
        # a forward that ran under autocast hands back a 16-bit gradient for fp32 x and W: the library
        # products then run in the gradient's type, as autocast itself would run them
        with _rocblas_gemm():
            if ctx.needs_input_grad[0] and grad_x is None:
                grad_x = (grad_out @ weight.to(grad_out.dtype)).to(x.dtype)
            if ctx.needs_input_grad[1] and grad_w is None:
                grad_w = (grad_out.t() @ x.to(grad_out.dtype)).to(weight.dtype)
        if want_b and grad_b is None:
            grad_b = _column_sum(grad_out).to(weight.dtype)
        return grad_x, grad_w, grad_b


def tall_linear(x, layer: nn.Linear):
    """Apply an ``nn.Linear`` to a tall 2-D input with the split-reduction weight gradient."""
    if x.dim() == 2 and x.is_cuda and not torch.is_autocast_enabled(x.device.type):
        return _TallLinear.apply(x, layer.weight, layer.bias)
    return layer(x)                                  # CPU tensors, and autocast regions (the split kernels are fp32 only)


class _BiasTableGather(Function):
    """``table.index_select(0, index)`` whose backward adds the rows of each table entry in a
    fixed order (``bins[t]`` lists the positions of ``index`` equal to ``t``, padded with
    ``len(index)``), so the table gradient is the same bit pattern on every run; an
    index_add with atomics is not."""

    @staticmethod
    def forward(ctx, table, index, bins):
        ctx.save_for_backward(bins)
        return table.index_select(0, index)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        (bins,) = ctx.saved_tensors
        padded = torch.cat([grad, grad.new_zeros(1, grad.shape[1])], 0)
        rows = padded.index_select(0, bins.reshape(-1)).reshape(bins.shape[0], bins.shape[1], -1)
        return rows.sum(1), None, None


def _index_bins(index: torch.Tensor, table_rows: int) -> torch.Tensor:
    """[table_rows, m] positions of ``index`` per table row, padded with ``len(index)``."""
    order = torch.argsort(index, stable=True)
    counts = torch.bincount(index, minlength=table_rows)
    starts = torch.cumsum(counts, 0) - counts
    m = max(int(counts.max()), 1)
    slot = torch.arange(m, device=index.device)[None, :]
    take = (starts[:, None] + slot).clamp_(max=max(len(index) - 1, 0))
    bins = order[take] if len(index) else take
    return torch.where(slot < counts[:, None], bins, torch.full_like(bins, len(index)))


def relative_position_index_3d(window_size: Sequence[int]) -> torch.Tensor:
    """[n, n] index into the (2w-1)^3 relative position bias table for a 3-D window."""
    wd, wh, ww = window_size
    coords = torch.stack(torch.meshgrid(torch.arange(wd), torch.arange(wh), torch.arange(ww), indexing="ij"))
    flat = coords.flatten(1)                                   # [3, n]
    rel = (flat[:, :, None] - flat[:, None, :]).permute(1, 2, 0).contiguous()
    rel[..., 0] += wd - 1
    rel[..., 1] += wh - 1
    rel[..., 2] += ww - 1
    rel[..., 0] *= (2 * wh - 1) * (2 * ww - 1)
    rel[..., 1] *= 2 * ww - 1
    return rel.sum(-1)


class WindowAttentionSparse(nn.Module):
    """Window multi-head self attention with relative position bias on sparse windows.

    ``fused`` (class or instance attribute, default True) selects the fused HIP path of
    :mod:`sparseswin3d_amd.fused` wherever it is supported (windows up to 384 positions with a relative
    position table, 7^3 included; measured faster than the operator path there too: 1.05 against 1.19 ms per
    module call on a room of 112 000 voxels, 3 heads of 16 channels); with ``fused = False`` the forward pass is
    the operator-by-operator composition of the reference.  ``resident`` picks between the two
    fused variants: True = window-resident kernels (attention matrix kept in registers, heads
    of 32 channels only), False = block products with the attention matrix in HBM, None =
    resident whenever it applies.  All paths give the same result.
    """

    fused = True
    resident = None

    def __init__(self, dim: int, num_heads: int, window_size: Sequence[int], qkv_bias: bool = False,
                 attn_drop: float = 0.0, proj_drop: float = 0.0) -> None:
        super().__init__()
        self.dim = dim
        self.window_size = window_size
        self.num_heads = num_heads
        self.scale = (dim // num_heads) ** -0.5
        if len(window_size) != 3:
            raise ValueError("window_size must have three entries")
        table = (2 * window_size[0] - 1) * (2 * window_size[1] - 1) * (2 * window_size[2] - 1)
        self.relative_position_bias_table = nn.Parameter(torch.zeros(table, num_heads))
        self.register_buffer("relative_position_index", relative_position_index_3d(window_size))
        self.qkv = nn.Linear(dim, dim * 3, bias=qkv_bias)
        self.attn_drop = nn.Dropout(attn_drop)      # constructed for state-dict parity; not applied
        self.proj = nn.Linear(dim, dim)
        self.proj_drop = nn.Dropout(proj_drop)
        trunc_normal_(self.relative_position_bias_table, std=0.02)
        self._bias_bins = {}        # (n, device) -> (index, bins) of the deterministic bias gather

    def _table_index(self, n: int):
        """BiasTableIndex of the first n positions on the table's device (cached), or None."""
        from . import fused
        table = self.relative_position_bias_table
        key = ("table", n, table.device)
        if key not in self._bias_bins:
            self._bias_bins[key] = fused.BiasTableIndex.build(self.relative_position_index[:n, :n], table.shape[0])
        return self._bias_bins[key]

    def relative_position_bias(self, n: int, dtype) -> torch.Tensor:
        table = self.relative_position_bias_table
        cached = self._bias_bins.get((n, table.device))
        if cached is None:
            index = self.relative_position_index[:n, :n].reshape(-1)
            cached = self._bias_bins[(n, table.device)] = (index, _index_bins(index, table.shape[0]))
        bias = _BiasTableGather.apply(table, *cached).reshape(n, n, -1)
        return bias.permute(2, 0, 1).contiguous().to(dtype)

    def prefetch_plan(self, x):
        """Enqueue the token plan of ``x``'s window indices now and keep it in ``x.plan_cache`` (created if
        missing), so that its totals have reached the host by the time :meth:`forward` asks for them.
        Returns the plan, or None for inputs that are not on the GPU.  :func:`prefetch_plans` does the same for
        several blocks with shared launches."""
        return prefetch_plans([(self, x)])[0]

    def forward(self, x, mask):
        n = x.spatial_shape[0]
        b = x.batch_size
        c = x.features.shape[-1]
        plan = None
        from . import fused
        if _takes_token_plan(self, x):
            # the token plan is enqueued first; the projection below runs while its totals travel.
            # A stage hands the same window indices to several blocks: they share one plan.
            cache = getattr(x, "plan_cache", None)
            plan = cache.get(self.num_heads) if cache is not None else None
            if plan is None:
                plan = fused.TokenPlan(x.indices, b, n, self.num_heads, defer=True)
                if cache is not None:
                    cache[self.num_heads] = plan
        qkv = tall_linear(x.features, self.qkv).reshape(-1, 3, self.num_heads, c // self.num_heads)
        table_index = self._table_index(n) if plan is not None and self.fused else None
        if plan is not None and self.fused and fused.supports(x.features, n, table_index is not None):
            resident = fused.supports_resident(qkv, n) if self.resident is None else self.resident
            if table_index is not None:
                out = fused.fused_window_attention(qkv, self.relative_position_bias_table, x.indices, mask, b, n,
                                                   self.scale, resident, plan, table_index)
            else:
                out = fused.fused_window_attention(qkv, self.relative_position_bias(n, torch.float32), x.indices,
                                                   mask, b, n, self.scale, resident, plan)
            x = replace_feature(x, out)
            return replace_feature(x, self.proj_drop(tall_linear(x.features, self.proj)))
        q, k_t, v = qkv_sparse_cuda(qkv, x.indices, b, n, plan, q_scale=self.scale)         # q = q * self.scale
        attn = spspmm_block_naive(q, k_t, "q_k")
        biased = sp_add_table_bias_and_mask(attn, self.relative_position_bias_table, self._table_index(n), mask, plan)
        if biased is not None:
            attn = biased
        else:
            attn = sp_add_rpb(attn, self.relative_position_bias(n, attn.values.dtype))
            if mask is not None:
                attn = sp_add_mask(attn, mask)
        attn = softmax_last_dim(attn)
        out = spspmm_block_naive(attn, v, "qk_v")
        omap = getattr(v, "operand_map", None)
        if omap is not None:
            # the product has V's structure: one copy takes its values from operand order to voxel rows
            x = replace_feature(x, _OperandToVoxels.apply(out.values, omap, self.num_heads, c // self.num_heads))
        else:
            out = out.permute((0, 2, 1, 3))                                  # (window, pos, head, ch)
            # the keys are below b * n: passing that bound spares return_inverse its search for the maximum
            unsort = ops.return_inverse(ops.flatten_indices(x.indices.T.contiguous(), [b, n]), b * n)[0]
            x = replace_feature(x, out.values.reshape(x.features.shape).index_select(0, unsort))
        return replace_feature(x, self.proj_drop(tall_linear(x.features, self.proj)))


def _takes_token_plan(attn, x) -> bool:
    """Every path of the module starts from a token plan of the window indices (the window-resident and fused
    kernels walk it, the operator path takes its operand map and group table from it) when these are int32 on the
    GPU."""
    return x.features.is_cuda and x.indices.is_cuda and x.indices.dtype == torch.int32 and x.indices.shape[0] > 0 \
        and attn.num_heads < 256


def prefetch_plans(pairs, extra=()):
    """Token plans for several ``(WindowAttentionSparse, window view)`` pairs, enqueued now by shared launches and
    kept in each view's ``plan_cache``: a stage calls this for all its blocks before the first one runs, so the
    plans' totals have reached the host by the time the blocks ask for them, and the regular and the shifted
    partition cost one set of launches instead of two.  Returns one plan per pair (None for inputs that are not on
    the GPU); pairs that share a view and a head count share a plan.  ``extra``:
    argument tuples of further ``TokenPlan``s (the stride-2 merge of the stage) built in the same launches;
    their plans follow the pairs' in the returned list."""
    from . import fused
    extra = list(extra)
    out, missing = [None] * len(pairs), {}
    for k, (attn, x) in enumerate(pairs):
        n = x.spatial_shape[0]
        if not _takes_token_plan(attn, x):
            continue
        cache = getattr(x, "plan_cache", None)
        if cache is None:
            cache = x.plan_cache = {}
        plan = cache.get(attn.num_heads)
        if plan is not None:
            out[k] = plan
        else:
            missing.setdefault((id(cache), attn.num_heads), (cache, x, n, attn.num_heads, []))[4].append(k)
    todo = list(missing.values())
    plans = fused.TokenPlan.batch([(x.indices, x.batch_size, n, heads) for _, x, n, heads, _ in todo] + extra)
    for (cache, _, _, heads, ks), plan in zip(todo, plans):
        cache[heads] = plan
        for k in ks:
            out[k] = plan
    return out + plans[len(todo):]
