"""Drop-in replacement of the reference's ``custom_ops`` extension module.

Same ten operator names, positional signatures, return types and error behaviour as the
pybind module built from ``sparse_swin/ops.cpp:7-18`` / ``sparse_swin/ops.h:4-50`` of the
reference.  Every operator runs hand-written HIP kernels from ``libsswin3d.so`` on the
current HIP stream of the tensors' device; torch is used only to allocate outputs and
scratch space and to hand over device pointers and the stream.  There is no CPU fallback:
tensors that are not on a GPU, or a missing library, raise ``RuntimeError``.

Use in the reference's ``swin3d_base.py`` by replacing its JIT ``load(...)`` call with
``from sparseswin3d_amd import custom_ops as ops``.
"""
from __future__ import annotations

import ctypes as C
import weakref
from collections import OrderedDict

import torch

from . import _lib

_DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2, torch.float64: 3}
_KEY_CODE = {torch.int32: 0, torch.int64: 1, torch.int16: 2, torch.int8: 3, torch.uint8: 4}
_MUL = {"q_k": 0, "qk_v": 1}
_GRAD = {"rc_cr": 0, "rr_rc": 1, "cr_rr": 2}
_TRANSPOSE = {"rc": 0, "rr": 1}


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _dev(*tensors):
    d = tensors[0].device
    _check(d.type == "cuda", "sparseswin3d_amd.custom_ops runs on the GPU only; got a tensor on "
                             f"'{d}'. There is no CPU fallback.")
    for t in tensors[1:]:
        _check(t.device == d, f"tensors on different devices: {d} and {t.device}")
    return d


def _stream(device):
    return _lib.stream_handle(device)


def _ptr(t):
    return C.c_void_p(t.data_ptr())


def _ws(nbytes, device):
    return torch.empty(int(nbytes), dtype=torch.uint8, device=device)


def _host_i32(values):
    arr = (C.c_int32 * len(values))(*[int(v) for v in values])
    return arr


# --------------------------------------------------------------------------------------- #
# index operators
# --------------------------------------------------------------------------------------- #
def flatten_indices(indices, sizes):
    """Wrapping int32 row-major hash of ``indices[:len(sizes)]`` (reference ops.cu:232-273)."""
    lib = _lib.load()
    d = _dev(indices)
    _check(indices.dim() == 2, "flatten_indices: indices must be 2-D [ndim, nnz]")
    _check(indices.dtype == torch.int32, f"flatten_indices: indices must be int32, got {indices.dtype}")
    ndim = len(sizes)
    _check(1 <= ndim <= indices.shape[0], "flatten_indices: len(sizes) exceeds the number of index rows")
    indices = indices.contiguous()
    m = indices.shape[1]
    out = torch.empty(m, dtype=torch.int32, device=d)
    with _lib.on_device(d):
        _lib.check(lib.sswin_flatten_indices(_ptr(indices), ndim, m, _host_i32(sizes), _ptr(out), _stream(d)))
    return out


def sort_indices(flattened_indices):
    """Stable ascending argsort of int32 keys, int32 result (reference ops.cu:276-289)."""
    lib = _lib.load()
    d = _dev(flattened_indices)
    _check(flattened_indices.dtype == torch.int32, "sort_indices: keys must be int32")
    keys = flattened_indices.contiguous().view(-1)
    m = keys.numel()
    out = torch.empty(m, dtype=torch.int32, device=d)
    nbytes = lib.sswin_sort_indices_workspace_bytes(m)
    ws = _ws(nbytes, d)
    with _lib.on_device(d):
        _lib.check(lib.sswin_sort_indices(_ptr(keys), m, _ptr(out), _ptr(ws), nbytes, _stream(d)))
    return out


def unique_consecutive_indices(nums):
    """Rank of the run of equal consecutive values each element belongs to (ops.cu:32-103)."""
    lib = _lib.load()
    d = _dev(nums)
    _check(nums.dim() == 1, "unique_consecutive_indices: expected a 1-D tensor")
    _check(nums.dtype in _KEY_CODE, f"unique_consecutive_indices: unsupported dtype {nums.dtype}")
    nums = nums.contiguous()
    m = nums.numel()
    out = torch.empty(m, dtype=torch.int32, device=d)
    nbytes = lib.sswin_unique_consecutive_workspace_bytes(m)
    ws = _ws(nbytes, d)
    with _lib.on_device(d):
        _lib.check(lib.sswin_unique_consecutive_indices(_ptr(nums), _KEY_CODE[nums.dtype], m, _ptr(out),
                                                        _ptr(ws), nbytes, _stream(d)))
    return out


def return_inverse(x, maxnum=-1):
    """``(rank of x[i] among the distinct values, number of distinct values)`` (ops.cu:718-730)."""
    lib = _lib.load()
    d = _dev(x)
    _check(x.dtype == torch.int32, "return_inverse: x must be int32")
    x = x.contiguous().view(-1)
    m = x.numel()
    out = torch.empty(m, dtype=torch.int32, device=d)
    if m == 0:
        return out, 0
    maxnum = int(maxnum)
    bound = maxnum
    if maxnum == -1:
        # the table size is data dependent: one read-back here, as in the reference (ops.cu:721)
        bound = int(x.max().item()) + 1
        _check(bound >= 1, "return_inverse: all values negative")
        maxnum = bound
    nbytes = lib.sswin_return_inverse_workspace_bytes(m, bound)
    ws = _ws(nbytes, d)
    count = C.c_int64(0)
    with _lib.on_device(d):
        _lib.check(lib.sswin_return_inverse(_ptr(x), m, maxnum, _ptr(out), C.byref(count), _ptr(ws), nbytes,
                                            _stream(d)))
        _check_pending()
    return out, int(count.value)


# ------------------------------------------------------------------------------------------
# Sorted operands without the permutations (helpers of qkv_sparse_cuda and of the module's tail; not
# operators of the reference's module)
# ------------------------------------------------------------------------------------------
def operand_map(indices, batch_size, spatial_dim):
    """Rank of every voxel in (window, pos) order as an int32 tensor [3N + 2] (voxel of rank r, first rank
    and size of its window, then the validity pair); input for :func:`operand_copy` and
    :func:`sorted_coo_indices`.  Invalid (window, pos) pairs (out of range, repeated) are skipped on the device and
    reported by the next operator of this module that waits for the stream (:func:`_check_pending`)."""
    lib = _lib.load()
    d = _dev(indices)
    _check(indices.dim() == 2 and indices.shape[1] == 2, "operand_map: indices must be [N, 2]")
    _check(indices.dtype == torch.int32, "operand_map: indices must be int32")
    indices = indices.contiguous()
    n_vox = indices.shape[0]
    out = torch.empty(3 * n_vox + 2, dtype=torch.int32, device=d)
    nbytes = lib.sswin_operand_map_workspace_bytes(n_vox, int(batch_size), int(spatial_dim))
    ws = _ws(nbytes, d)
    status = torch.zeros(2, dtype=torch.int32, pin_memory=True)
    with _lib.on_device(d):
        _check_pending()
        _lib.check(lib.sswin_operand_map(_ptr(indices), n_vox, int(batch_size), int(spatial_dim), _ptr(out), _ptr(ws),
                                         nbytes, 0, C.c_void_p(status.data_ptr()), _stream(d)))
        if n_vox > 0:
            event = torch.cuda.Event()
            event.record(torch.cuda.current_stream(d))
            _pending.append((event, status, n_vox))
    return out


def operand_copy(vox, col0, val, omap, num_heads, c, layout, to_operand, scale=1.0):
    """Copy between a token tensor ``vox`` [N, stride] (columns ``col0 + h*c + ch``) and a sorted operand's
    value array ``val`` [N*H*c]: layout 0 = Q/V order, 1 = K^T order; ``to_operand`` gives the direction.
    ``scale`` (Q/V order only): the values are multiplied by it on the way."""
    lib = _lib.load()
    d = _dev(vox, val, omap)
    _check(vox.dim() == 2 and vox.stride(1) == 1 and val.is_contiguous() and vox.dtype == val.dtype,
           "operand_copy: vox must be [N, stride] with unit column stride and val contiguous of the same dtype")
    _check(vox.dtype in _DTYPE_CODE, f"unsupported value dtype {vox.dtype}")
    n_vox = vox.shape[0]
    _check(omap.numel() == 3 * n_vox + 2 and val.numel() == n_vox * num_heads * c, "operand_copy: sizes do not match")
    with _lib.on_device(d):
        _lib.check(lib.sswin_operand_copy(_DTYPE_CODE[vox.dtype], int(layout), 1 if to_operand else 0, _ptr(vox),
                                          vox.stride(0), int(col0), _ptr(val), _ptr(omap), n_vox, int(num_heads), int(c),
                                          float(scale), _stream(d)))


def operand_copy_qkv(vox, val_q, val_k, val_v, omap, num_heads, c, to_operand, q_scale=1.0):
    """The three operand copies of one attention call in one launch: ``vox`` [N, 3*H*c] (a projection output, Q | K | V)
    to or from ``val_q`` (Q/V order, times ``q_scale``), ``val_k`` (K^T order), ``val_v`` (Q/V order)."""
    lib = _lib.load()
    d = _dev(vox, val_q, val_k, val_v, omap)
    n_vox = vox.shape[0]
    _check(vox.dim() == 2 and vox.stride(1) == 1 and vox.shape[1] == 3 * num_heads * c, "operand_copy_qkv: vox must be [N, 3*H*c]")
    _check(vox.dtype in _DTYPE_CODE, f"unsupported value dtype {vox.dtype}")
    for val in (val_q, val_k, val_v):
        _check(val.is_contiguous() and val.dtype == vox.dtype and val.numel() == n_vox * num_heads * c,
               "operand_copy_qkv: operands must be contiguous [N*H*c] arrays of vox's dtype")
    _check(omap.numel() == 3 * n_vox + 2, "operand_copy_qkv: sizes do not match")
    with _lib.on_device(d):
        _lib.check(lib.sswin_operand_copy_qkv(_DTYPE_CODE[vox.dtype], 1 if to_operand else 0, _ptr(vox), vox.stride(0), 0,
                                              _ptr(val_q), _ptr(val_k), _ptr(val_v), _ptr(omap), n_vox, int(num_heads), int(c),
                                              float(q_scale), _stream(d)))


def sorted_coo_indices(indices, omap, num_heads, c, qv=True, k=True):
    """The sorted [4, E] index matrices of Q/V and of K^T (``idx.index_select(1, order)`` of
    :func:`qkv_sparse_indices`), written directly.  ``qv=False`` / ``k=False``: None in place of that matrix."""
    lib = _lib.load()
    d = _dev(indices, omap)
    indices = indices.contiguous()
    n_vox = indices.shape[0]
    e = n_vox * num_heads * c
    idx_qv = torch.empty((4, e), dtype=torch.int32, device=d) if qv else None
    idx_k = torch.empty((4, e), dtype=torch.int32, device=d) if k else None
    if qv or k:
        with _lib.on_device(d):
            _lib.check(lib.sswin_sorted_coo_indices(_ptr(indices), _ptr(omap), n_vox, int(num_heads), int(c),
                                                    _ptr(idx_qv) if qv else None, _ptr(idx_k) if k else None, _stream(d)))
    return idx_qv, idx_k


# Input checks of :func:`operand_map` whose verdict is still on its way from the GPU: (event, pinned status,
# voxel count).  An operator that has just waited for the stream anyway looks at them (:func:`_check_pending`).
_pending = []


def _check_pending(wait=False):
    """Raise for a deferred :func:`operand_map` check whose status has arrived (all of them after
    ``wait=True`` or after the caller has synchronised the stream)."""
    keep = []
    bad = None
    for event, status, n_vox in _pending:
        if not (wait or event.query()):
            keep.append((event, status, n_vox))
            continue
        event.synchronize()
        out_of_range, distinct = int(status[0]), int(status[1])
        if out_of_range:
            bad = (f"operand_map: {out_of_range} voxel indices lie outside [0, batch_size) x [0, spatial_dim)")
        elif distinct != n_vox:
            bad = (f"operand_map: (window, pos) pairs must be distinct: {n_vox - distinct} voxels share a "
                   "pair with another")
    _pending[:] = keep
    if bad:
        raise RuntimeError(bad)


def qkv_sparse_indices(indices, batch_size, spatial_dim, num_heads, c):
    """Element-level COO indices of Q/V and K^T plus their sorting permutations (ops.cu:293-335)."""
    lib = _lib.load()
    d = _dev(indices)
    _check(indices.dim() == 2 and indices.shape[1] == 2, "qkv_sparse_indices: indices must be [N, 2]")
    _check(indices.dtype == torch.int32, "qkv_sparse_indices: indices must be int32")
    indices = indices.contiguous()
    n_vox = indices.shape[0]
    e = n_vox * num_heads * c
    idx_qv = torch.empty((4, e), dtype=torch.int32, device=d)
    idx_k = torch.empty((4, e), dtype=torch.int32, device=d)
    sorted_qv = torch.empty(e, dtype=torch.int32, device=d)
    sorted_k = torch.empty(e, dtype=torch.int32, device=d)
    nbytes = lib.sswin_qkv_sparse_indices_workspace_bytes(n_vox, int(batch_size), int(spatial_dim))
    ws = _ws(nbytes, d)
    # Indices the kernels cannot address (out of range, repeated pairs) are reported as an error by this call (it
    # waits for the stream); the two permutations of such input are all zero, so nothing reads out of bounds.
    with _lib.on_device(d):
        _check_pending()
        _lib.check(lib.sswin_qkv_sparse_indices(_ptr(indices), n_vox, int(batch_size), int(spatial_dim),
                                                int(num_heads), int(c), _ptr(idx_qv), _ptr(sorted_qv),
                                                _ptr(idx_k), _ptr(sorted_k), _ptr(ws), nbytes, 1, None, _stream(d)))
    return idx_qv, sorted_qv, idx_k, sorted_k


# --------------------------------------------------------------------------------------- #
# per-group offsets: a small cache so that the eight backward calls that receive the `_c`
# tensor returned by matmul_cuda_naive do not rescan it.
# --------------------------------------------------------------------------------------- #
class _PlanCache:
    """Maps the storage address of a `_c` tensor handed out by :func:`matmul_cuda_naive` to
    its scans.  Entries hold a reference to the plan tensor, so the address cannot be reused
    while an entry is alive; the version counter guards against in-place edits."""

    def __init__(self, capacity=32):
        self.capacity = capacity
        self.entries = OrderedDict()
        self.scans = {}                              # key -> contiguous [2 * G] scans of a plan with g_cap > G

    def put(self, c_view, plan, g_cap, totals):
        key = (c_view.device.index, c_view.data_ptr(), c_view.numel())
        self.entries[key] = (plan, g_cap, totals, c_view._version)
        self.scans.pop(key, None)
        self.entries.move_to_end(key)
        while len(self.entries) > self.capacity:
            self.scans.pop(self.entries.popitem(last=False)[0], None)

    def packed_scans(self, c, hit):
        """The two scan rows of a cached plan side by side (the layout the kernels take), packed once per plan."""
        key = (c.device.index, c.data_ptr(), c.numel())
        packed = self.scans.get(key)
        if packed is None:
            plan, g_cap = hit[0], hit[1]
            rows = plan.view(5, g_cap)
            g = c.numel()
            packed = self.scans[key] = torch.stack([rows[1, :g], rows[2, :g]]).reshape(-1)
        return packed

    def get(self, c):
        key = (c.device.index, c.data_ptr(), c.numel())
        hit = self.entries.get(key)
        if hit is None or hit[3] != c._version or c.dtype != torch.int32 or not c.is_contiguous():
            return None
        self.entries.move_to_end(key)
        return hit

    def clear(self):
        self.entries.clear()
        self.scans.clear()


_plan_cache = _PlanCache()


class _IndexPlanCache:
    """Plans keyed by the index matrix they were derived from.  'q_k' and 'qk_v' of one forward
    pass receive the same sorted Q/V index tensor, so the second call skips the plan kernels and
    their host synchronisation.  An entry holds only a weak reference to the index tensor: it is
    valid while that tensor is alive (its address cannot have been handed to another tensor) and
    unchanged (version counter), and it does not keep the [4, E] matrix in memory.  A plan enters the
    cache only after the host has waited for the stream that built it (the totals are read back), so a
    hit from another stream reads finished data."""

    def __init__(self, capacity=8):
        self.capacity = capacity
        self.entries = OrderedDict()

    @staticmethod
    def _key(idx, inner):
        return (idx.device.index, idx.data_ptr(), idx.shape[1], inner)

    def get(self, idx, inner):
        key = self._key(idx, inner)
        hit = self.entries.get(key)
        if hit is None:
            return None
        alive = hit[0]()
        if alive is None or alive._version != hit[1]:
            del self.entries[key]
            return None
        return hit[2:]

    def put(self, idx, inner, plan, g_cap, totals):
        self.entries[self._key(idx, inner)] = (weakref.ref(idx), idx._version, plan, g_cap, totals)
        while len(self.entries) > self.capacity:
            self.entries.popitem(last=False)

    def clear(self):
        self.entries.clear()


_index_plan_cache = _IndexPlanCache()


def register_index_plan(idx, inner, plan, g_cap, groups, rows, nnz_sq, c_max):
    """Tell the block products the plan of a sorted [4, M] index matrix ``idx`` (dense last dimension ``inner``) that
    the caller has derived by other means: ``plan`` int32 [5 * g_cap] = rows c, row_start, sq_start, window, head of
    the ``groups`` (window, head) groups, ``rows`` = sum of c, ``nnz_sq`` = sum of c*c, ``c_max`` = largest c.  The
    stream that wrote ``plan`` must have been waited for.  The products of ``idx`` then skip the pass over it."""
    _index_plan_cache.put(idx, int(inner), plan, int(g_cap), (int(groups), int(rows), int(nnz_sq), int(c_max)))


def clear_caches():
    """Drop cached plans (and the tensors they keep alive)."""
    _plan_cache.clear()
    _index_plan_cache.clear()
    _pending.clear()


def _scans_for(c, lib, d):
    """Return ``(scans [2,G] int32 rows: excl-scan c, excl-scan c*c; sum_c2 or None)``."""
    hit = _plan_cache.get(c)
    g = c.numel()
    if hit is not None:
        plan, g_cap, totals, _ = hit
        rows = plan.view(5, g_cap)
        if g_cap == g:
            return rows[1:3].reshape(-1), totals[2]
        return _plan_cache.packed_scans(c, hit), totals[2]
    scans = torch.empty(2 * max(g, 1), dtype=torch.int32, device=d)
    nbytes = lib.sswin_scan_counts_workspace_bytes(g)
    ws = _ws(nbytes, d)
    _lib.check(lib.sswin_scan_counts(_ptr(c), g, _ptr(scans), _ptr(ws), nbytes, _stream(d)))
    return scans, None


# --------------------------------------------------------------------------------------- #
# block products
# --------------------------------------------------------------------------------------- #
def matmul_cuda_naive(mat1_v, mat1_idx, mat1_shape, mat2_v, mat2_idx, mat2_shape, mul_type):
    """Window-blocked sparse product ``'q_k'`` or ``'qk_v'`` (reference ops.cu:788-943, 1034-1088).

    Returns ``(indices int32 [4, nnz], values [nnz], shape list[4], _c int32 [G])``.
    """
    _check(mat1_idx.dim() == 2, "Expected mat1_idx.dim() == 2 to be true, but got false.")
    _check(mat2_idx.dim() == 2, "Expected mat2_idx.dim() == 2 to be true, but got false.")
    return block_product(mat1_v, mat1_idx, mat1_shape, mat2_v, mat2_idx, mat2_shape, mul_type)


def block_product(mat1_v, mat1_idx, mat1_shape, mat2_v, mat2_idx, mat2_shape, mul_type, values=True, indices=True):
    """:func:`matmul_cuda_naive` with either half of the result optional: ``indices=False`` returns None in place of
    the product's [4, nnz] index matrix (a composition of the operators that never reads it saves its 16 bytes per
    entry), ``values=False`` returns None in place of the values (then the value arrays may be None), so that the
    index matrix can be produced later, when somebody asks for it.  The index matrix of the operand that carries no
    token rows (``mat2_idx`` of 'q_k', ``mat1_idx`` of 'qk_v') may be None: the product reads nothing from it."""
    lib = _lib.load()
    _check(mul_type in _MUL, f"Invalid mul_type: {mul_type}. Expected 'q_k' or 'qk_v'.")
    _check(values or indices, "block_product: nothing asked for")
    kind = _MUL[mul_type]
    tok_idx, other_idx = (mat1_idx, mat2_idx) if kind == 0 else (mat2_idx, mat1_idx)
    _check(tok_idx is not None and tok_idx.dim() == 2, "the operand with the token rows needs its [4, M] index matrix")
    if values:
        _check(mat1_v.dim() == 1, "Expected mat1_v.dim() == 1 to be true, but got false.")
        _check(mat2_v.dim() == 1, "Expected mat2_v.dim() == 1 to be true, but got false.")
        _check(mat1_v.dtype == mat2_v.dtype, f"mat1 dtype {mat1_v.dtype} does not match mat2 dtype {mat2_v.dtype}")
        _check(mat1_v.dtype in _DTYPE_CODE, f"unsupported value dtype {mat1_v.dtype}")
    if other_idx is not None:
        _check(mat1_idx.dtype == mat2_idx.dtype,
               f"mat1 dtype {mat1_idx.dtype} does not match mat2 dtype {mat2_idx.dtype}")
    _check(tok_idx.dtype == torch.int32, f"mat1 dtype is not int32, but {tok_idx.dtype}")
    s1, s2 = [int(v) for v in mat1_shape], [int(v) for v in mat2_shape]
    _check(len(s1) == 4 and len(s2) == 4 and s1[0] == s2[0] and s1[1] == s2[1] and s1[3] == s2[2],
           f"Invalid shapes: mat1_shape {s1} and mat2_shape {s2}. Expected sizes: 4. Expected "
           "mat1_shape[0] == mat2_shape[0], mat1_shape[1] == mat2_shape[1], mat1_shape[3] == mat2_shape[2].")
    d = _dev(*(t for t in (mat1_v, mat1_idx, mat2_v, mat2_idx) if t is not None))
    _check(tok_idx.shape[0] == 4 and (other_idx is None or other_idx.shape[0] == 4), "index matrices must have 4 rows")
    if values:
        for v, i in ((mat1_v, mat1_idx), (mat2_v, mat2_idx)):
            _check(i is None or i.shape[1] == v.numel(), "index and value counts differ")
        mat1_v, mat2_v = mat1_v.contiguous(), mat2_v.contiguous()
    tok_idx = tok_idx.contiguous()
    value_dtype = mat1_v.dtype if values else torch.float32

    inner = s1[3] if kind == 0 else s2[3]
    m = tok_idx.shape[1]
    out_shape = [s1[0], s1[1], s1[2], s2[3]]
    if m == 0:
        return (torch.empty((4, 0), dtype=torch.int32, device=d) if indices else None,
                torch.empty(0, dtype=value_dtype, device=d) if values else None,
                out_shape, torch.empty(0, dtype=torch.int32, device=d))
    _check(m % inner == 0, f"operand nnz {m} is not a multiple of its dense last dimension {inner}")
    rows = m // inner
    stream = _stream(d)
    with _lib.on_device(d):
        plan, g_cap, (g, sum_c, sum_c2, c_max) = _plan_of(tok_idx, inner, s1[0] * s1[1], lib, d)
        if kind == 0:
            _check(not values or mat2_v.numel() == m, f"'q_k': mat2 holds {mat2_v.numel() if values else 0} values, expected {m}")
            nnz = sum_c2
        else:
            _check(not values or mat1_v.numel() == sum_c2,
                   f"'qk_v': mat1 holds {mat1_v.numel() if values else 0} values, expected sum of c*c = {sum_c2}")
            nnz = m
        out_idx = torch.empty((4, nnz), dtype=torch.int32, device=d) if indices else None
        out_val = torch.empty(nnz, dtype=value_dtype, device=d) if values else None
        _lib.check(lib.sswin_block_matmul(kind, _DTYPE_CODE[value_dtype], _ptr(mat1_v) if values else None,
                                          _ptr(mat2_v) if values else None, _ptr(tok_idx), m, inner, _ptr(plan), g_cap, g,
                                          c_max, _ptr(out_val) if values else None, _ptr(out_idx) if indices else None,
                                          nnz, stream))
    c_view = plan[:g]
    _plan_cache.put(c_view, plan, g_cap, (g, sum_c, sum_c2, c_max))
    if kind == 1 and indices:
        # the product has the group structure of V (same windows, heads, rows and dense extent): a later
        # permute of it finds the plan without another pass over its indices
        _index_plan_cache.put(out_idx, inner, plan, g_cap, (g, sum_c, sum_c2, c_max))
    return out_idx, out_val, out_shape, c_view


def _plan_of(idx, inner, batch_heads, lib, d):
    """Plan of a coalesced [4, M] index matrix with dense last dimension ``inner`` (cached)."""
    cached = _index_plan_cache.get(idx, inner)
    if cached is not None:
        return cached
    m = idx.shape[1]
    g_cap = max(1, min(m // inner, batch_heads))
    plan = torch.empty(5 * g_cap, dtype=torch.int32, device=d)
    totals = (C.c_int64 * 4)()
    nbytes = lib.sswin_plan_workspace_bytes(m, inner)
    ws = _ws(nbytes, d)
    _lib.check(lib.sswin_plan_from_indices(_ptr(idx), m, inner, _ptr(plan), g_cap, totals, _ptr(ws), nbytes, _stream(d)))
    _check_pending()                                  # the stream has just been waited for
    out = (plan, g_cap, tuple(int(totals[i]) for i in range(4)))
    _index_plan_cache.put(idx, inner, *out)
    return out


def permute_heads_order(indices, shape):
    """Order of a coalesced [B, H, n, C] COO operand after ``permute((0, 2, 1, 3))`` (what
    ``sort_indices(flatten_indices(indices[[0, 2, 1, 3]], ...))`` returns), derived from the group
    structure without a sort; ``None`` if the heads of some window do not hold the same positions
    (the caller then sorts).  Not an operator of the reference's module: a helper of
    :meth:`SparseTensor.permute`."""
    lib = _lib.load()
    d = _dev(indices)
    inner = int(shape[3])
    m = indices.shape[1]
    if indices.dtype != torch.int32 or inner % 4 or m == 0 or m % inner or not indices.is_contiguous():
        return None
    with _lib.on_device(d):
        plan, g_cap, (g, _, _, _) = _plan_of(indices, inner, int(shape[0]) * int(shape[1]), lib, d)
        order = torch.empty(m, dtype=torch.int32, device=d)
        bad = torch.empty(1, dtype=torch.int32, device=d)
        _lib.check(lib.sswin_permute_heads_order(_ptr(indices), m, inner, _ptr(plan), g_cap, g, _ptr(order), _ptr(bad),
                                                 _stream(d)))
        if int(bad.item()) != 0:
            return None
        _check_pending()
    return order


def softmax_rows_from_counts(_c, nnz):
    """Row ids of the sparse softmax over a 'q_k' product with group sizes ``_c`` and ``nnz`` entries: what
    ``unique_consecutive_indices(flatten_indices(idx[:3], shape[:3]))`` returns for it, from the group sizes alone.
    Not an operator of the reference's module: a helper of :func:`softmax_last_dim`."""
    lib = _lib.load()
    d = _dev(_c)
    _check(_c.dtype == torch.int32 and _c.dim() == 1, "_c must be int32 [G]")
    c = _c.contiguous()
    rows = torch.empty(int(nnz), dtype=torch.int32, device=d)
    with _lib.on_device(d):
        scans, sum_c2 = _scans_for(c, lib, d)
        _check(sum_c2 is None or sum_c2 == nnz, f"softmax_rows_from_counts: {nnz} entries, the groups hold {sum_c2}")
        _lib.check(lib.sswin_softmax_rows_from_counts(_ptr(c), _ptr(scans), c.numel(), int(nnz), _ptr(rows), _stream(d)))
    return rows


class GroupPlan:
    """The plan behind a ``_c`` that :func:`matmul_cuda_naive` returned (group sizes, offsets, windows, heads), held
    by reference so that a backward pass finds it however many plans have been made since."""

    def __init__(self, plan, g_cap, groups, rows, c_max):
        self.plan, self.g_cap, self.groups, self.rows, self.c_max = plan, g_cap, groups, rows, c_max


def group_plan(_c):
    """:class:`GroupPlan` of a ``_c`` from :func:`matmul_cuda_naive`, or None if the plan is no longer cached."""
    hit = _plan_cache.get(_c)
    if hit is None:
        return None
    plan, g_cap, totals, _ = hit
    return GroupPlan(plan, g_cap, int(totals[0]), int(totals[1]), int(totals[3]))


def group_row_positions(idx, gp):
    """Window position of every attention row of a 'q_k' product with indices ``idx`` [4, A] and :class:`GroupPlan`
    ``gp``, in group order: int32 [sum c].  (Every ``C``-th entry of row 2 of the Q operand's index matrix holds the
    same numbers.)"""
    lib = _lib.load()
    d = _dev(idx)
    _check(idx.dtype == torch.int32 and idx.dim() == 2 and idx.shape[0] == 4, "group_row_positions: idx must be int32 [4, A]")
    idx = idx.contiguous()
    rows = torch.empty(max(gp.rows, 1), dtype=torch.int32, device=d)
    with _lib.on_device(d):
        _lib.check(lib.sswin_group_row_positions(_ptr(idx), idx.shape[1], _ptr(gp.plan), gp.g_cap, gp.groups, _ptr(rows),
                                                 _stream(d)))
    return rows


def group_add_bias_mask(values, row_pos, gp, n, bias32, mask):
    """``values + bias[head, pos_i, pos_j]`` (and ``-100`` where the int8 mask regions of the two positions differ) for a
    'q_k' product with row positions ``row_pos`` (:func:`group_row_positions`) and :class:`GroupPlan` ``gp``:
    sp_add_rpb followed by sp_add_mask."""
    lib = _lib.load()
    d = _dev(values, row_pos, bias32)
    _check(values.dtype in _DTYPE_CODE and bias32.dtype == torch.float32 and row_pos.dtype == torch.int32, "group_add_bias_mask: dtypes")
    _check(row_pos.dim() == 1 and row_pos.numel() >= gp.rows, "group_add_bias_mask: one position per token row")
    _check(mask is None or mask.dtype == torch.int8, "group_add_bias_mask: the mask must hold int8 region ids")
    values, idx, bias32 = values.contiguous(), row_pos.contiguous(), bias32.contiguous()
    mask = None if mask is None else mask.contiguous()
    out = torch.empty_like(values)
    with _lib.on_device(d):
        _lib.check(lib.sswin_group_add_bias_mask(_DTYPE_CODE[values.dtype], _ptr(values), _ptr(idx), values.numel(), _ptr(gp.plan),
                                                 gp.g_cap, gp.groups, gp.c_max, int(n), _ptr(bias32),
                                                 _ptr(mask) if mask is not None else None,
                                                 0 if mask is None else mask.shape[0], _ptr(out), _stream(d)))
    return out


def group_add_table_bias_mask(values, row_pos, gp, n, table32, code, offset0, mask):
    """:func:`group_add_bias_mask` with the bias taken from the relative position table ``table32`` [rows, H] itself:
    bias of positions p, q = ``table32[code[p] - code[q] + offset0, head]``."""
    lib = _lib.load()
    d = _dev(values, row_pos, table32, code)
    _check(values.dtype in _DTYPE_CODE and table32.dtype == torch.float32 and row_pos.dtype == torch.int32 and code.dtype == torch.int32,
           "group_add_table_bias_mask: dtypes")
    _check(row_pos.dim() == 1 and row_pos.numel() >= gp.rows, "group_add_table_bias_mask: one position per token row")
    _check(mask is None or mask.dtype == torch.int8, "group_add_table_bias_mask: the mask must hold int8 region ids")
    _check(table32.dim() == 2 and code.numel() >= n, "group_add_table_bias_mask: table [rows, H] and one code per position")
    values, idx, table32, code = values.contiguous(), row_pos.contiguous(), table32.contiguous(), code.contiguous()
    mask = None if mask is None else mask.contiguous()
    out = torch.empty_like(values)
    with _lib.on_device(d):
        _lib.check(lib.sswin_group_add_table_bias_mask(
            _DTYPE_CODE[values.dtype], _ptr(values), _ptr(idx), values.numel(), _ptr(gp.plan), gp.g_cap, gp.groups, gp.c_max, int(n),
            _ptr(table32), table32.shape[0], table32.shape[1], _ptr(code), int(offset0),
            _ptr(mask) if mask is not None else None, 0 if mask is None else mask.shape[0], _ptr(out), _stream(d)))
    return out


def group_bias_table_grad(grad_values, row_pos, gp, num_heads, n, code, offset0, table_rows):
    """Gradient of the relative position bias table [table_rows, H] from the gradient of a 'q_k' product's values
    (fp32) and its row positions (:func:`group_row_positions`), summed in a fixed order."""
    lib = _lib.load()
    d = _dev(grad_values, row_pos)
    _check(grad_values.dtype == torch.float32, "group_bias_table_grad: the gradient must be float32")
    _check(row_pos.dtype == torch.int32 and row_pos.dim() == 1 and row_pos.numel() >= gp.rows,
           "group_bias_table_grad: one int32 position per token row")
    grad_values, rows = grad_values.contiguous(), row_pos.contiguous()
    d_table = torch.empty((table_rows, num_heads), dtype=torch.float32, device=d)
    with _lib.on_device(d):
        nbytes = lib.sswin_bias_table_grad_workspace_bytes(gp.groups, int(num_heads), int(table_rows))
        ws = _ws(nbytes, d)
        _lib.check(lib.sswin_bias_table_grad(_ptr(gp.plan), gp.g_cap, gp.groups, _ptr(rows), 0, int(num_heads), int(n), _ptr(code),
                                             int(offset0), int(table_rows), _ptr(grad_values), _ptr(d_table), _ptr(ws), nbytes,
                                             _stream(d)))
    return d_table


def matmul_grad_cuda_naive(mat1_v, mat2_v, _c, C_, mul_type):
    """Value-only block products of the backward pass (reference ops.cu:945-1031, 1092-1114)."""
    lib = _lib.load()
    _check(mul_type in _GRAD, f"Invalid mul_type: {mul_type}. Expected 'rc_cr', 'rr_rc' or 'cr_rr'.")
    _check(mat1_v.dtype == mat2_v.dtype, f"mat1 dtype {mat1_v.dtype} does not match mat2 dtype {mat2_v.dtype}")
    _check(mat1_v.dtype in _DTYPE_CODE, f"unsupported value dtype {mat1_v.dtype}")
    _check(_c.dtype == torch.int32, "_c must be int32")
    d = _dev(mat1_v, mat2_v, _c)
    mat1_v, mat2_v, _c = mat1_v.contiguous(), mat2_v.contiguous(), _c.contiguous()
    g, C_ = _c.numel(), int(C_)
    kind = _GRAD[mul_type]
    with _lib.on_device(d):
        scans, sum_c2 = _scans_for(_c, lib, d)
        if kind == 0:
            if sum_c2 is None:      # output size is data dependent: one read-back (reference ops.cu:968)
                sum_c2 = int((_c.to(torch.int64) ** 2).sum().item())
            total = sum_c2
            _check(mat1_v.numel() == mat2_v.numel(), "'rc_cr': operands must have equal sizes")
        elif kind == 1:
            total = mat2_v.numel()
        else:
            total = mat1_v.numel()
        out = torch.empty(total, dtype=mat1_v.dtype, device=d)
        if g > 0 and total > 0:
            _lib.check(lib.sswin_block_matmul_grad(kind, _DTYPE_CODE[mat1_v.dtype], _ptr(mat1_v), _ptr(mat2_v),
                                                   _ptr(_c), _ptr(scans), g, C_,
                                                   mat1_v.numel() if kind == 0 else total, _ptr(out), _stream(d)))
    return out


_GRAD_UNTRANSPOSED = {"tr_rc": 3, "tc_rr": 4}


def matmul_grad_untransposed(mat1_v, mat2_v, _c, C_, mul_type):
    """The second gradient of a block product from the operands as the forward pass left them (no counterpart among
    the reference's operators; its Python backward, swin3d_base.py:121-134, transposes both operands first):
    ``'tr_rc'``: out [c x C] = mat1[c x c]^T . mat2[c x C], equal to
    ``matmul_grad_cuda_naive(qkv_transpose(mat1, 'rr'), qkv_transpose(mat2, 'rc'), 'rr_rc')``;
    ``'tc_rr'``: out [C x c] = mat1[c x C]^T . mat2[c x c], equal to
    ``matmul_grad_cuda_naive(qkv_transpose(mat1, 'rc'), qkv_transpose(mat2, 'rr'), 'cr_rr')``."""
    lib = _lib.load()
    _check(mul_type in _GRAD_UNTRANSPOSED, f"Invalid mul_type: {mul_type}. Expected 'tr_rc' or 'tc_rr'.")
    _check(mat1_v.dtype == mat2_v.dtype, f"mat1 dtype {mat1_v.dtype} does not match mat2 dtype {mat2_v.dtype}")
    _check(mat1_v.dtype in _DTYPE_CODE, f"unsupported value dtype {mat1_v.dtype}")
    _check(_c.dtype == torch.int32, "_c must be int32")
    d = _dev(mat1_v, mat2_v, _c)
    mat1_v, mat2_v, _c = mat1_v.contiguous(), mat2_v.contiguous(), _c.contiguous()
    g = _c.numel()
    kind = _GRAD_UNTRANSPOSED[mul_type]
    out = torch.empty_like(mat2_v if kind == 3 else mat1_v)
    with _lib.on_device(d):
        scans, _ = _scans_for(_c, lib, d)
        if g > 0 and out.numel() > 0:
            _lib.check(lib.sswin_block_matmul_grad(kind, _DTYPE_CODE[mat1_v.dtype], _ptr(mat1_v), _ptr(mat2_v),
                                                   _ptr(_c), _ptr(scans), g, int(C_), out.numel(), _ptr(out),
                                                   _stream(d)))
    return out


def qkv_transpose(mat1_v, _c, C_, mul_type):
    """Per-group transposes ``'rc'`` / ``'rr'`` (reference ops.cu:663-715, 1117-1132)."""
    lib = _lib.load()
    _check(mul_type in _TRANSPOSE, f"Invalid mul_type: {mul_type}. Expected 'rc', or 'rr'.")
    _check(mat1_v.dtype in _DTYPE_CODE, f"unsupported value dtype {mat1_v.dtype}")
    _check(_c.dtype == torch.int32, "_c must be int32")
    d = _dev(mat1_v, _c)
    mat1_v, _c = mat1_v.contiguous(), _c.contiguous()
    g = _c.numel()
    out = torch.empty_like(mat1_v)
    with _lib.on_device(d):
        scans, _ = _scans_for(_c, lib, d)
        if g > 0 and mat1_v.numel() > 0:
            _lib.check(lib.sswin_block_transpose(_TRANSPOSE[mul_type], _DTYPE_CODE[mat1_v.dtype], _ptr(mat1_v),
                                                 _ptr(_c), _ptr(scans), g, int(C_), _ptr(out), _stream(d)))
    return out


# --------------------------------------------------------------------------------------- #
# sparse row softmax
# --------------------------------------------------------------------------------------- #
def _softmax_args(indices, *vals):
    d = _dev(indices, *vals)
    _check(indices.dtype == torch.int32, "softmax: row ids must be int32")
    _check(all(v.dim() == 1 and v.numel() == indices.numel() for v in vals), "softmax: size mismatch")
    dtype = vals[0].dtype
    _check(all(v.dtype == dtype for v in vals), "softmax: dtype mismatch")
    _check(dtype in (torch.float32, torch.float64, torch.float16, torch.bfloat16),
           f"softmax: unsupported dtype {dtype}")
    work = dtype if dtype in (torch.float32, torch.float64) else torch.float32
    def aligned(t):
        # the kernels move 16 bytes at a time: a view that starts inside an allocation is copied
        t = t.contiguous()
        return t if t.data_ptr() % 16 == 0 else t.clone()
    return d, dtype, work, aligned(indices), [aligned(v.to(work)) for v in vals]


def softmax_last_dim_forward(indices, values):
    """``exp(v - max(0, rowmax)) / (rowsum + 1e-8)`` over sorted row ids (reference ops.cu:128-167)."""
    lib = _lib.load()
    d, dtype, work, indices, (values,) = _softmax_args(indices, values)
    out = torch.empty_like(values)
    with _lib.on_device(d):
        _lib.check(lib.sswin_softmax_last_dim_forward(_ptr(indices), _ptr(values), _DTYPE_CODE[work],
                                                      values.numel(), _ptr(out), _stream(d)))
    return out.to(dtype)


def softmax_last_dim_backward(indices, values, grad_values):
    """``g*y - y*sum_row(g*y)`` (reference ops.cu:169-194)."""
    lib = _lib.load()
    d, dtype, work, indices, (values, grad_values) = _softmax_args(indices, values, grad_values)
    out = torch.empty_like(values)
    with _lib.on_device(d):
        _lib.check(lib.sswin_softmax_last_dim_backward(_ptr(indices), _ptr(values), _ptr(grad_values),
                                                       _DTYPE_CODE[work], values.numel(), _ptr(out), _stream(d)))
    return out.to(dtype)
