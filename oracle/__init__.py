"""CPU oracle for the sparse window-attention operators — TEST INFRASTRUCTURE ONLY.

Loads ``liboracle.so`` (built from ``sswin_oracle.c`` by ``oracle/Makefile``) and exposes
the reference's ten operator names on numpy arrays.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this
package; the product (``sparseswin3d_amd``) never does.

Parity status: the reference ships no tests or golden vectors for this path, so every
function here is pinned by library routines, closed forms and brute force instead
(``tests/test_oracle_pins.py``); see the header of ``sswin_oracle.c`` for the list.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (seconds)."""
    src = os.path.join(_HERE, "sswin_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


class _Result(C.Structure):
    _fields_ = [("G", C.c_int64), ("nnz", C.c_int64), ("idx", C.POINTER(C.c_int32)),
                ("val", C.c_void_p), ("c", C.POINTER(C.c_int32))]


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_return_inverse.restype = C.c_int64
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


# --------------------------------------------------------------------------- #
def flatten_indices(indices, sizes):
    indices = _i32(indices)
    ndim, m = indices.shape
    assert ndim == len(sizes)
    out = np.empty(m, np.int32)
    lib().orc_flatten_indices(_p(indices), C.c_int(ndim), C.c_int64(m), _p(_i32(sizes)), _p(out))
    return out


def sort_indices(flat):
    flat = _i32(flat)
    out = np.empty(flat.shape[0], np.int32)
    lib().orc_sort_indices(_p(flat), C.c_int64(flat.shape[0]), _p(out))
    return out


def unique_consecutive_indices(nums):
    nums = np.ascontiguousarray(nums)
    out = np.empty(nums.shape[0], np.int32)
    if nums.dtype == np.int64:
        lib().orc_unique_consecutive_i64(_p(nums), C.c_int64(nums.shape[0]), _p(out))
    else:
        nums = _i32(nums)
        lib().orc_unique_consecutive_i32(_p(nums), C.c_int64(nums.shape[0]), _p(out))
    return out


def return_inverse(x, maxnum=-1):
    x = _i32(x)
    out = np.empty(x.shape[0], np.int32)
    cnt = lib().orc_return_inverse(_p(x), C.c_int64(x.shape[0]), C.c_int64(maxnum), _p(out))
    return out, int(cnt)


def qkv_sparse_indices(indices, batch_size, spatial_dim, num_heads, c):
    indices = _i32(indices)
    n = indices.shape[0]
    e = n * num_heads * c
    idx_qv = np.empty((4, e), np.int32)
    idx_k = np.empty((4, e), np.int32)
    s_qv = np.empty(e, np.int32)
    s_k = np.empty(e, np.int32)
    lib().orc_qkv_sparse_indices(_p(indices), C.c_int64(n), C.c_int(batch_size), C.c_int(spatial_dim),
                                 C.c_int(num_heads), C.c_int(c), _p(idx_qv), _p(s_qv), _p(idx_k), _p(s_k))
    return idx_qv, s_qv, idx_k, s_k


def _fp(a):
    a = np.ascontiguousarray(a)
    if a.dtype not in (np.float32, np.float64):
        a = a.astype(np.float32)
    return a


def matmul_cuda_naive(mat1_v, mat1_idx, mat1_shape, mat2_v, mat2_idx, mat2_shape, mul_type):
    if mul_type not in ("q_k", "qk_v"):
        raise RuntimeError(f"Invalid mul_type: {mul_type}. Expected 'q_k' or 'qk_v'.")
    mat1_v, mat2_v = _fp(mat1_v), _fp(mat2_v)
    assert mat1_v.dtype == mat2_v.dtype
    mat1_idx, mat2_idx = _i32(mat1_idx), _i32(mat2_idx)
    fn = lib().orc_matmul_f32 if mat1_v.dtype == np.float32 else lib().orc_matmul_f64
    res = _Result()
    bad = fn(_p(mat1_v), _p(mat1_idx), C.c_int64(mat1_idx.shape[1]), _p(_i32(mat1_shape)),
             _p(mat2_v), _p(mat2_idx), C.c_int64(mat2_idx.shape[1]), _p(_i32(mat2_shape)),
             C.c_int(1 if mul_type == "qk_v" else 0), C.byref(res))
    try:
        if bad:
            raise RuntimeError("oracle matmul: operands do not have matching block structure")
        nnz, g = res.nnz, res.G
        idx = np.ctypeslib.as_array(res.idx, shape=(4 * max(nnz, 1),))[: 4 * nnz].reshape(4, nnz).copy()
        vbuf = (C.c_char * (max(nnz, 1) * mat1_v.itemsize)).from_address(res.val)
        val = np.frombuffer(vbuf, dtype=mat1_v.dtype)[:nnz].copy()
        cc = np.ctypeslib.as_array(res.c, shape=(max(g, 1),))[:g].copy()
    finally:
        lib().orc_free_result(C.byref(res))
    shape = [int(mat1_shape[0]), int(mat1_shape[1]), int(mat1_shape[2]), int(mat2_shape[3])]
    return idx, val, shape, cc


_GRAD_MODE = {"rc_cr": 0, "rr_rc": 1, "cr_rr": 2}


def matmul_grad_cuda_naive(mat1_v, mat2_v, _c, C_, mul_type):
    if mul_type not in _GRAD_MODE:
        raise RuntimeError(f"Invalid mul_type: {mul_type}. Expected 'rc_cr', 'rr_rc' or 'cr_rr'.")
    mat1_v, mat2_v = _fp(mat1_v), _fp(mat2_v)
    _c = _i32(_c)
    c64 = _c.astype(np.int64)
    total = int((c64 * c64).sum()) if mul_type == "rc_cr" else int((c64 * C_).sum())
    out = np.empty(total, mat1_v.dtype)
    fn = lib().orc_matmul_grad_f32 if mat1_v.dtype == np.float32 else lib().orc_matmul_grad_f64
    fn(_p(mat1_v), _p(mat2_v), _p(_c), C.c_int64(len(_c)), C.c_int32(C_), C.c_int(_GRAD_MODE[mul_type]), _p(out))
    return out


def qkv_transpose(mat1_v, _c, C_, mul_type):
    if mul_type not in ("rc", "rr"):
        raise RuntimeError(f"Invalid mul_type: {mul_type}. Expected 'rc', or 'rr'.")
    mat1_v = _fp(mat1_v)
    _c = _i32(_c)
    out = np.empty_like(mat1_v)
    fn = lib().orc_qkv_transpose_f32 if mat1_v.dtype == np.float32 else lib().orc_qkv_transpose_f64
    fn(_p(mat1_v), _p(_c), C.c_int64(len(_c)), C.c_int32(C_), C.c_int(1 if mul_type == "rr" else 0), _p(out))
    return out


def softmax_last_dim_forward(indices, values):
    indices, values = _i32(indices), _fp(values)
    out = np.empty_like(values)
    fn = lib().orc_softmax_fwd_f32 if values.dtype == np.float32 else lib().orc_softmax_fwd_f64
    fn(_p(indices), _p(values), C.c_int64(len(values)), _p(out))
    return out


def softmax_last_dim_backward(indices, values, grad_values):
    indices, values, grad_values = _i32(indices), _fp(values), _fp(grad_values)
    assert values.dtype == grad_values.dtype
    out = np.empty_like(values)
    fn = lib().orc_softmax_bwd_f32 if values.dtype == np.float32 else lib().orc_softmax_bwd_f64
    fn(_p(indices), _p(values), _p(grad_values), C.c_int64(len(values)), _p(out))
    return out
