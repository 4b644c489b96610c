"""The entry point that allocates nothing: ``sswin_unique_consecutive_indices_static`` against
``sswin_unique_consecutive_indices`` (reference operator sparse_swin/ops.cu:32-103), through the C ABI.

Bit-exact int32 ranks; two calls in a row on the same GPU, the second with a smaller input (the
built-in scratch keeps the first call's contents), then the size limit's error path."""
import ctypes as C

import numpy as np
import pytest
import torch

from sparseswin3d_amd import _lib

pytestmark = pytest.mark.gpu

I32, I64 = 0, 1


def _runs(rng, m, mean_run):
    """sorted keys with runs of random length"""
    return np.repeat(np.arange(m), rng.integers(1, 2 * mean_run, size=m))[:m]


def _both(lib, keys_np, code):
    dev = torch.device("cuda:0")
    keys = torch.from_numpy(keys_np).to(dev)
    m = keys.numel()
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    want = torch.full((m,), -1, dtype=torch.int32, device=dev)
    nbytes = lib.sswin_unique_consecutive_workspace_bytes(m)
    ws = torch.empty(int(nbytes), dtype=torch.uint8, device=dev)
    _lib.check(lib.sswin_unique_consecutive_indices(C.c_void_p(keys.data_ptr()), code, m, C.c_void_p(want.data_ptr()),
                                                    C.c_void_p(ws.data_ptr()), nbytes, stream))
    got = torch.full((m,), -2, dtype=torch.int32, device=dev)
    # a first call may load the code object; the second one must leave the device's free memory as it was (the
    # driver's own count: an allocation inside the library would show there, not in PyTorch's allocator)
    _lib.check(lib.sswin_unique_consecutive_indices_static(C.c_void_p(keys.data_ptr()), code, m,
                                                           C.c_void_p(got.data_ptr()), stream))
    torch.cuda.synchronize()
    got.fill_(-2)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(dev)[0]
    before = torch.cuda.memory_allocated(dev)
    _lib.check(lib.sswin_unique_consecutive_indices_static(C.c_void_p(keys.data_ptr()), code, m,
                                                           C.c_void_p(got.data_ptr()), stream))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    return got.cpu().numpy(), want.cpu().numpy()


def test_static_scratch_matches_workspace_entry_point_twice(oracle):
    lib = _lib.load()
    rng = np.random.default_rng(7)
    big = _runs(rng, 1_000_003, 9).astype(np.int32)          # 245 tiles of 4096 keys, ragged tail
    got, want = _both(lib, big, I32)
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(got, oracle.unique_consecutive_indices(big))
    small = _runs(rng, 5_001, 3).astype(np.int32)             # second call, smaller: stale tile sums behind it
    got, want = _both(lib, small, I32)
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(got, oracle.unique_consecutive_indices(small))
    wide = _runs(rng, 70_001, 5).astype(np.int64)             # the generic (2048-key tile) kernels
    got, want = _both(lib, wide, I64)
    np.testing.assert_array_equal(got, want)


def test_static_scratch_rejects_oversize_and_null():
    lib = _lib.load()
    rc = lib.sswin_unique_consecutive_indices_static(None, I32, 134217728 + 1, None, None)
    assert rc != 0 and b"exceed the built-in scratch" in lib.sswin_last_error()
    rc = lib.sswin_unique_consecutive_indices_static(None, I32, 10, None, None)
    assert rc != 0 and b"null pointer" in lib.sswin_last_error()
    assert lib.sswin_unique_consecutive_indices_static(None, I32, 0, None, None) == 0
