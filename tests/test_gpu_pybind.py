"""The pybind11 build of the operator module (``sparseswin3d_amd.custom_ops_pybind``: the ten names of the
reference's ``PYBIND11_MODULE``, sparse_swin/ops.cpp:7-18, with ``at::Tensor`` arguments as in
sparse_swin/ops.h:4-50).  Every name is called through it and checked against the CPU oracle to the same
bar as the ctypes module (integers bit-exact, fp32 values within rel 1e-5 of the fp64 oracle), and
against the ctypes module bit for bit (both drive the same kernels)."""
import numpy as np
import pytest
import torch

from helpers import softmax_bwd_mag, close, product_mag, qkv_operands, ragged_window_indices

pytestmark = pytest.mark.gpu

COUNTS = [1, 40, 2, 125, 0, 0, 17, 32, 90, 3, 33, 64]
N_POS, H, HD = 125, 3, 32


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t if dtype is None else t.to(dtype)


def host(t):
    return t.detach().to(torch.float64).cpu().numpy() if t.is_floating_point() else t.cpu().numpy()


@pytest.fixture(scope="module")
def mods():
    from sparseswin3d_amd import custom_ops, custom_ops_pybind
    return custom_ops_pybind, custom_ops


@pytest.fixture(scope="module")
def case(oracle):
    rng = np.random.default_rng(20)
    ind = ragged_window_indices(rng, COUNTS, N_POS)
    d = qkv_operands(oracle, ind, len(COUNTS), N_POS, H, HD, rng, dtype=np.float32)
    d["ind"] = ind
    return d


def same(a, b):
    assert a.dtype == b.dtype and a.shape == b.shape
    assert torch.equal(a, b)


def test_index_operators(mods, oracle, case):
    pb, ct = mods
    B = len(COUNTS)
    ind = dev(case["ind"])
    got = pb.qkv_sparse_indices(ind, B, N_POS, H, HD)
    want = oracle.qkv_sparse_indices(case["ind"], B, N_POS, H, HD)
    for g, w, c in zip(got, want, ct.qkv_sparse_indices(ind, B, N_POS, H, HD)):
        np.testing.assert_array_equal(host(g), w)
        same(g, c)
    perm = np.ascontiguousarray(case["qi"][[0, 2, 1, 3]])
    sizes = [B, N_POS, H, HD]
    flat = pb.flatten_indices(dev(perm), sizes)
    r_flat = oracle.flatten_indices(perm, sizes)
    np.testing.assert_array_equal(host(flat), r_flat)
    order = pb.sort_indices(flat)
    np.testing.assert_array_equal(host(order), oracle.sort_indices(r_flat))
    same(order, ct.sort_indices(flat))
    keys = oracle.flatten_indices(np.ascontiguousarray(case["ind"].T), [B, N_POS])
    for maxnum in (-1, B * N_POS):
        inv, count = pb.return_inverse(dev(keys), maxnum)
        r_inv, r_count = oracle.return_inverse(keys, maxnum)
        np.testing.assert_array_equal(host(inv), r_inv)
        assert count == r_count == ct.return_inverse(dev(keys), maxnum)[1]
    runs = np.repeat(np.arange(50), np.random.default_rng(3).integers(1, 9, 50)).astype(np.int32)
    for dt in (np.int32, np.int64, np.uint8):
        np.testing.assert_array_equal(host(pb.unique_consecutive_indices(dev(runs.astype(dt)))),
                                      oracle.unique_consecutive_indices(runs.astype(dt)))


def test_products_softmax_gradients_transposes(mods, oracle, case):
    pb, ct = mods
    d = case
    q, kt, v = dev(d["q"]), dev(d["kt"]), dev(d["v"])
    qi, ki = dev(d["qi"]), dev(d["ki"])
    s_idx, s_val, s_shape, c = pb.matmul_cuda_naive(q, qi, d["q_shape"], kt, ki, d["k_shape"], "q_k")
    r_idx, r_val, r_shape, r_c = oracle.matmul_cuda_naive(host(q), d["qi"], d["q_shape"], host(kt), d["ki"], d["k_shape"], "q_k")
    assert list(s_shape) == r_shape
    np.testing.assert_array_equal(host(s_idx), r_idx)
    np.testing.assert_array_equal(host(c), r_c)
    close(host(s_val), r_val, 1e-5, "q_k",
          mag=product_mag(oracle, "matmul_cuda_naive", host(q), d["qi"], d["q_shape"], host(kt), d["ki"], d["k_shape"], "q_k"))
    c_idx, c_val, _, c_c = ct.matmul_cuda_naive(q, qi, d["q_shape"], kt, ki, d["k_shape"], "q_k")
    same(s_idx, c_idx), same(s_val, c_val), same(c, c_c)

    rows = pb.unique_consecutive_indices(pb.flatten_indices(s_idx[:3].contiguous(), list(s_shape[:3])))
    r_rows = oracle.unique_consecutive_indices(oracle.flatten_indices(r_idx[:3], r_shape[:3]))
    np.testing.assert_array_equal(host(rows), r_rows)
    p = pb.softmax_last_dim_forward(rows, s_val)
    close(host(p), oracle.softmax_last_dim_forward(r_rows, host(s_val)), 1e-5, "softmax forward", seg=r_rows)
    same(p, ct.softmax_last_dim_forward(rows, s_val))
    gp = dev(np.random.default_rng(5).standard_normal(p.numel()), torch.float32)
    gs = pb.softmax_last_dim_backward(rows, p, gp)
    close(host(gs), oracle.softmax_last_dim_backward(r_rows, host(p), host(gp)), 1e-5, "softmax backward",
          mag=softmax_bwd_mag(r_rows, host(p), host(gp)))
    same(gs, ct.softmax_last_dim_backward(rows, p, gp))

    o_idx, o_val, o_shape, c2 = pb.matmul_cuda_naive(p, s_idx, list(s_shape), v, qi, d["q_shape"], "qk_v")
    ro_idx, ro_val, ro_shape, ro_c = oracle.matmul_cuda_naive(host(p), r_idx, r_shape, host(v), d["qi"], d["q_shape"], "qk_v")
    assert list(o_shape) == ro_shape
    np.testing.assert_array_equal(host(o_idx), ro_idx)
    np.testing.assert_array_equal(host(c2), ro_c)
    close(host(o_val), ro_val, 1e-5, "qk_v",
          mag=product_mag(oracle, "matmul_cuda_naive", host(p), r_idx, r_shape, host(v), d["qi"], d["q_shape"], "qk_v"))

    g_o = dev(np.random.default_rng(6).standard_normal(o_val.numel()), torch.float32)
    for kind, a, b in (("rc_cr", g_o, v), ("rr_rc", gs, kt), ("cr_rr", q, gs)):
        out = pb.matmul_grad_cuda_naive(a, b, c, HD, kind)
        close(host(out), oracle.matmul_grad_cuda_naive(host(a), host(b), r_c, HD, kind), 1e-5, kind,
              mag=product_mag(oracle, "matmul_grad_cuda_naive", host(a), host(b), r_c, HD, kind))
        same(out, ct.matmul_grad_cuda_naive(a, b, c, HD, kind))
    for kind, a in (("rc", v), ("rr", p)):
        out = pb.qkv_transpose(a, c, HD, kind)
        np.testing.assert_array_equal(host(out), oracle.qkv_transpose(host(a), r_c, HD, kind))
        same(out, ct.qkv_transpose(a, c, HD, kind))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_softmax_takes_16_bit_values(mods, oracle, dtype):
    """The reference dispatches its softmax over the floating types and half (ops.cu:140, 155, 183): 16-bit values are
    computed in fp32 and rounded once, the same as the ctypes module."""
    pb, ct = mods
    rng = np.random.default_rng(8)
    rows_np = np.repeat(np.arange(40), rng.integers(1, 60, 40)).astype(np.int32)
    rows = dev(rows_np)
    v = dev(rng.standard_normal(len(rows_np)) * 2.0, dtype)
    g = dev(rng.standard_normal(len(rows_np)), dtype)
    y = pb.softmax_last_dim_forward(rows, v)
    assert y.dtype == dtype
    close(host(y), oracle.softmax_last_dim_forward(rows_np, host(v)), 2e-2, f"softmax forward {dtype}", seg=rows_np)
    same(y, ct.softmax_last_dim_forward(rows, v))
    gx = pb.softmax_last_dim_backward(rows, y, g)
    assert gx.dtype == dtype
    close(host(gx), oracle.softmax_last_dim_backward(rows_np, host(y), host(g)), 2e-2, f"softmax backward {dtype}",
          mag=softmax_bwd_mag(rows_np, host(y), host(g)))
    same(gx, ct.softmax_last_dim_backward(rows, y, g))


def test_error_behaviour(mods):
    pb, _ = mods
    e_idx = torch.empty(4, 0, dtype=torch.int32, device="cuda")
    e_val = torch.empty(0, device="cuda")
    with pytest.raises(RuntimeError, match="Invalid mul_type"):
        pb.matmul_cuda_naive(e_val, e_idx, [1, 1, 8, 4], e_val, e_idx, [1, 1, 4, 8], "k_q")
    with pytest.raises(RuntimeError, match="Invalid shapes"):
        pb.matmul_cuda_naive(e_val, e_idx, [1, 1, 8, 4], e_val, e_idx, [1, 2, 4, 8], "q_k")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        pb.softmax_last_dim_forward(torch.zeros(3, dtype=torch.int32), torch.zeros(3))
    idx, val, shape, c = pb.matmul_cuda_naive(e_val, e_idx, [4, 2, 125, 32], e_val, e_idx, [4, 2, 32, 125], "q_k")
    assert idx.shape == (4, 0) and val.numel() == 0 and c.numel() == 0 and list(shape) == [4, 2, 125, 125]
