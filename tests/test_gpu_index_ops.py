"""GPU parity of the integer index operators against the CPU oracle: bit-exact."""
import numpy as np
import pytest
import torch

from helpers import ragged_window_indices, random_window_indices

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.fixture(scope="module")
def ops():
    from sparseswin3d_amd import custom_ops
    return custom_ops


@pytest.mark.parametrize("ndim,m", [(2, 1), (2, 1000), (3, 4096), (3, 12345), (4, 40000), (4, 7), (4, 4)])
def test_flatten_indices(ops, oracle, ndim, m):
    rng = np.random.default_rng(ndim * 1000 + m)
    sizes = [int(s) for s in rng.integers(3, 200, size=ndim)]
    idx = np.stack([rng.integers(0, s, size=m) for s in sizes]).astype(np.int32)
    out = ops.flatten_indices(dev(idx), sizes).cpu().numpy()
    assert out.dtype == np.int32
    np.testing.assert_array_equal(out, oracle.flatten_indices(idx, sizes))


def test_flatten_indices_wraps_like_int32(ops, oracle):
    # sizes whose product exceeds 2^31: the hash wraps, identically on both sides
    sizes = [70000, 24, 125, 768]
    rng = np.random.default_rng(7)
    idx = np.stack([rng.integers(0, s, size=5000) for s in sizes]).astype(np.int32)
    out = ops.flatten_indices(dev(idx), sizes).cpu().numpy()
    ref = oracle.flatten_indices(idx, sizes)
    assert (ref < 0).any()
    np.testing.assert_array_equal(out, ref)


def test_flatten_indices_row_subset(ops, oracle):
    # softmax path: first three rows of a [4, nnz] matrix with a 3-entry size list
    rng = np.random.default_rng(3)
    idx = rng.integers(0, 50, size=(4, 999)).astype(np.int32)
    out = ops.flatten_indices(dev(idx)[:3], [60, 50, 50]).cpu().numpy()
    np.testing.assert_array_equal(out, oracle.flatten_indices(idx[:3], [60, 50, 50]))


@pytest.mark.parametrize("m", [0, 1, 2, 255, 4097, 300_000])
def test_sort_indices(ops, oracle, m):
    rng = np.random.default_rng(m)
    keys = rng.integers(-50, 5000, size=m).astype(np.int32)      # duplicates and negatives
    out = ops.sort_indices(dev(keys)).cpu().numpy()
    assert out.dtype == np.int32
    np.testing.assert_array_equal(out, oracle.sort_indices(keys))   # stable order


def test_sort_indices_full_range(ops, oracle):
    rng = np.random.default_rng(11)
    keys = rng.integers(-2**31, 2**31 - 1, size=100_000).astype(np.int32)
    np.testing.assert_array_equal(ops.sort_indices(dev(keys)).cpu().numpy(), oracle.sort_indices(keys))


@pytest.mark.parametrize("m,dtype", [(1, np.int32), (2, np.int32), (3, np.int32), (5, np.int32), (2048, np.int32),
                                     (2049, np.int32), (4095, np.int32), (4096, np.int32), (4097, np.int32),
                                     (100_003, np.int32), (1_000_001, np.int32), (50_000, np.int64)])
def test_unique_consecutive_indices(ops, oracle, m, dtype):
    rng = np.random.default_rng(m)
    x = np.cumsum(rng.random(m) < 0.3).astype(dtype)            # sorted with runs
    out = ops.unique_consecutive_indices(dev(x)).cpu().numpy()
    assert out.dtype == np.int32
    np.testing.assert_array_equal(out, oracle.unique_consecutive_indices(x))


def test_unique_consecutive_unaligned_view(ops, oracle):
    """A view that starts 4 bytes into an allocation takes the generic (unvectorised) kernel."""
    rng = np.random.default_rng(3)
    x = np.cumsum(rng.random(10_001) < 0.5).astype(np.int32)
    t = dev(x)[1:]
    np.testing.assert_array_equal(ops.unique_consecutive_indices(t).cpu().numpy(),
                                  oracle.unique_consecutive_indices(x[1:]))


def test_unique_consecutive_unsorted_runs(ops, oracle):
    x = np.array([5, 5, 2, 2, 2, 5, 9, 9, 1], np.int32)
    np.testing.assert_array_equal(ops.unique_consecutive_indices(dev(x)).cpu().numpy(),
                                  oracle.unique_consecutive_indices(x))


@pytest.mark.parametrize("m,hi,maxnum", [(1, 1, -1), (1000, 5000, -1), (1000, 5000, 6000),
                                         (200_000, 3_000_000, -1), (50_000, 300, -1)])
def test_return_inverse(ops, oracle, m, hi, maxnum):
    rng = np.random.default_rng(m + hi)
    x = rng.integers(0, hi, size=m).astype(np.int32)
    out, cnt = ops.return_inverse(dev(x), maxnum)
    ref, ref_cnt = oracle.return_inverse(x, maxnum)
    assert cnt == ref_cnt
    np.testing.assert_array_equal(out.cpu().numpy(), ref)


@pytest.mark.parametrize("B,n,H,hd,N", [(6, 8, 2, 4, 17), (40, 125, 3, 32, 900), (1, 125, 1, 32, 125),
                                        (300, 27, 6, 32, 2000), (7, 343, 2, 16, 600)])
def test_qkv_sparse_indices(ops, oracle, B, n, H, hd, N):
    rng = np.random.default_rng(B * n + N)
    ind = random_window_indices(rng, B, n, N)
    got = ops.qkv_sparse_indices(dev(ind), B, n, H, hd)
    ref = oracle.qkv_sparse_indices(ind, B, n, H, hd)
    for name, g, r in zip(("idx_qv", "sorted_qv", "idx_k", "sorted_k"), got, ref):
        assert g.dtype == torch.int32
        np.testing.assert_array_equal(g.cpu().numpy(), r, err_msg=name)


def test_qkv_sparse_indices_ragged_and_last_slot(ops, oracle):
    # occupancies 1..125, empty windows in between, and the very last window slot occupied
    rng = np.random.default_rng(5)
    counts = [1, 0, 125, 2, 0, 0, 33, 64, 5, 17, 1, 1, 100]
    ind = ragged_window_indices(rng, counts, 125)
    B = len(counts)
    got = ops.qkv_sparse_indices(dev(ind), B, 125, 3, 32)
    ref = oracle.qkv_sparse_indices(ind, B, 125, 3, 32)
    for g, r in zip(got, ref):
        np.testing.assert_array_equal(g.cpu().numpy(), r)


def test_index_ops_report_indices_they_cannot_address(ops):
    """A window id >= batch_size, a position >= n, a negative entry, a repeated (window, pos) pair, or a value
    >= maxnum never becomes a device address: the kernels skip it and the operator raises."""
    rng = np.random.default_rng(11)
    B, n, H, hd = 30, 125, 3, 32
    good = random_window_indices(rng, B, n, 700)
    for bad_row, what in (([B, 0], "outside"), ([0, n], "outside"), ([-3, 5], "outside"), ([4, -1], "outside"),
                          (list(good[5]), "distinct")):
        ind = np.concatenate([good[:300], np.array([bad_row], np.int32), good[300:]])
        with pytest.raises(RuntimeError, match=what):
            ops.qkv_sparse_indices(dev(ind), B, n, H, hd)
    x = rng.integers(0, 500, size=2000).astype(np.int32)
    x[77] = 500
    with pytest.raises(RuntimeError, match="outside"):
        ops.return_inverse(dev(x), 500)
    x[77] = -2
    with pytest.raises(RuntimeError, match="outside"):
        ops.return_inverse(dev(x), 500)
    # qkv_sparse_cuda builds its operands from a token plan, which reports the same faults
    from sparseswin3d_amd.window_attention import qkv_sparse_cuda
    ind = np.concatenate([good[:300], good[5:6], good[300:]])
    qkv = torch.randn(len(ind), 3, H, hd, device="cuda")
    with pytest.raises(RuntimeError, match="distinct"):
        qkv_sparse_cuda(qkv, dev(ind), B, n)
    # the operand map on its own defers the check: the next operator that waits for the stream raises
    omap = ops.operand_map(dev(ind), B, n)
    ops.sorted_coo_indices(dev(ind), omap, H, hd)
    with pytest.raises(RuntimeError, match="distinct"):
        ops.return_inverse(dev(x.clip(0, 499)), 500)
    ops.clear_caches()
    got = ops.qkv_sparse_indices(dev(good), B, n, H, hd)            # and the library still works afterwards
    assert got[1].numel() == 700 * H * hd


def test_ops_reject_cpu_tensors(ops):
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.flatten_indices(torch.zeros((2, 4), dtype=torch.int32), [3, 3])


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 1e-5), (torch.float16, 1e-5)])
@pytest.mark.parametrize("N,P", [(1, 96), (7, 288), (1000, 96), (107500, 288), (4099, 4), (5000, 1024), (8200, 2304),
                                 (300, 1100)])
def test_column_sum(N, P, dtype, tol):
    """Bias gradient of the projections: column sums of a tall matrix in fp32, fixed order."""
    import ctypes as C
    from sparseswin3d_amd import _lib
    lib = _lib.load()
    g = torch.Generator().manual_seed(N + P)
    x = torch.randn(N, P, generator=g).to(dtype)
    xd = x.cuda()
    out = torch.full((P,), float("nan"), device="cuda")
    nbytes = lib.sswin_column_sum_workspace_bytes(N, P)
    ws = torch.empty(int(nbytes), dtype=torch.uint8, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    for _ in range(2):
        _lib.check(lib.sswin_column_sum(C.c_void_p(xd.data_ptr()), code, N, P, C.c_void_p(out.data_ptr()),
                                        C.c_void_p(ws.data_ptr()), nbytes, stream))
    ref = x.double().sum(0).numpy()                      # the rounded inputs, summed exactly
    got = out.cpu().numpy().astype(np.float64)
    scale = np.abs(x.double()).sum(0).numpy() / max(N, 1) ** 0.5
    assert np.all(np.abs(got - ref) <= tol * (np.abs(ref) + scale + 1e-6))
