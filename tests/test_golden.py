"""Committed golden vectors (tests/golden/tiny_ops.npz): the oracle must reproduce them on the CPU,
the HIP operators on the GPU.  Integer results bit-exact; values within rel 1e-12 (oracle, fp64)
and rel 1e-5 (HIP, fp32)."""
import os

import numpy as np
import pytest

from helpers import softmax_bwd_mag, close, product_mag

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tiny_ops.npz")


@pytest.fixture(scope="module")
def gold():
    return dict(np.load(GOLD))


def _operands(g):
    B, n, H, hd = (int(g[k]) for k in ("B", "n", "H", "hd"))
    qi = np.ascontiguousarray(g["idx_qv"][:, g["sorted_qv"]])
    ki = np.ascontiguousarray(g["idx_k"][:, g["sorted_k"]])
    q = g["qkv"][:, 0].reshape(-1)[g["sorted_qv"]]
    kt = g["qkv"][:, 1].reshape(-1)[g["sorted_k"]]
    v = g["qkv"][:, 2].reshape(-1)[g["sorted_qv"]]
    return B, n, H, hd, qi, ki, q, kt, v


def test_oracle_reproduces_golden(oracle, gold):
    g = gold
    B, n, H, hd, qi, ki, q, kt, v = _operands(g)
    iqv, sqv, ik, sk = oracle.qkv_sparse_indices(g["ind"], B, n, H, hd)
    for a, b in ((iqv, "idx_qv"), (sqv, "sorted_qv"), (ik, "idx_k"), (sk, "sorted_k")):
        np.testing.assert_array_equal(a, g[b])
    s_idx, s_val, _, c = oracle.matmul_cuda_naive(q, qi, [B, H, n, hd], kt, ki, [B, H, hd, n], "q_k")
    np.testing.assert_array_equal(s_idx, g["s_idx"])
    np.testing.assert_array_equal(c, g["c"])
    np.testing.assert_array_equal(c, [1, 1, 2, 2, 5, 5])
    close(s_val, g["s_val"], 1e-12, "oracle q_k", seg="all")
    rows = oracle.unique_consecutive_indices(oracle.flatten_indices(s_idx[:3], [B, H, n]))
    np.testing.assert_array_equal(rows, g["rows"])
    close(oracle.softmax_last_dim_forward(rows, s_val), g["p"], 1e-12, "oracle softmax", seg=rows)
    o_idx, o_val, _, _ = oracle.matmul_cuda_naive(g["p"], s_idx, [B, H, n, n], v, qi, [B, H, n, hd], "qk_v")
    np.testing.assert_array_equal(o_idx, g["o_idx"])
    close(o_val, g["o_val"], 1e-12, "oracle qk_v", seg="all")
    close(oracle.softmax_last_dim_backward(rows, g["p"], g["d_p"]), g["d_s"], 1e-12, "oracle softmax backward",
          mag=softmax_bwd_mag(rows, g["p"], g["d_p"]))
    out, cnt = oracle.return_inverse(g["tok"], -1)
    np.testing.assert_array_equal(out, g["unsort"])
    assert cnt == int(g["n_unique"]) == len(g["ind"])


@pytest.mark.gpu
def test_hip_operators_reproduce_golden(oracle, gold):
    import torch
    from sparseswin3d_amd import custom_ops as ops
    g = gold
    B, n, H, hd, qi, ki, q, kt, v = _operands(g)
    dev = lambda a, dt=None: (torch.from_numpy(np.ascontiguousarray(a)).cuda() if dt is None
                              else torch.from_numpy(np.ascontiguousarray(a)).cuda().to(dt))
    f32 = torch.float32
    got = ops.qkv_sparse_indices(dev(g["ind"]), B, n, H, hd)
    for a, b in zip(got, ("idx_qv", "sorted_qv", "idx_k", "sorted_k")):
        np.testing.assert_array_equal(a.cpu().numpy(), g[b])
    s_idx, s_val, s_shape, c = ops.matmul_cuda_naive(dev(q, f32), dev(qi), [B, H, n, hd], dev(kt, f32), dev(ki),
                                                     [B, H, hd, n], "q_k")
    np.testing.assert_array_equal(s_idx.cpu().numpy(), g["s_idx"])
    np.testing.assert_array_equal(c.cpu().numpy(), g["c"])
    f64 = lambda a: np.asarray(a, dtype=np.float32).astype(np.float64)       # what the GPU operators are fed
    qs, ks = [B, H, n, hd], [B, H, hd, n]
    close(s_val.cpu().numpy(), g["s_val"], 1e-5, "q_k", mag=product_mag(oracle, "matmul_cuda_naive", f64(q), qi, qs, f64(kt), ki, ks, "q_k"))
    flat = ops.flatten_indices(s_idx[:3], s_shape[:3])
    np.testing.assert_array_equal(flat.cpu().numpy(), g["flat"])
    rows = ops.unique_consecutive_indices(flat)
    np.testing.assert_array_equal(rows.cpu().numpy(), g["rows"])
    p = ops.softmax_last_dim_forward(rows, dev(g["s_val"], f32))
    close(p.cpu().numpy(), g["p"], 1e-5, "softmax", seg=g["rows"])
    o_idx, o_val, _, _ = ops.matmul_cuda_naive(dev(g["p"], f32), s_idx, s_shape, dev(v, f32), dev(qi), [B, H, n, hd], "qk_v")
    np.testing.assert_array_equal(o_idx.cpu().numpy(), g["o_idx"])
    close(o_val.cpu().numpy(), g["o_val"], 1e-5, "qk_v",
          mag=product_mag(oracle, "matmul_cuda_naive", f64(g["p"]), g["s_idx"], [B, H, n, n], f64(v), qi, qs, "qk_v"))
    d_p = ops.matmul_grad_cuda_naive(dev(g["g_o"], f32), dev(v, f32), c, hd, "rc_cr")
    cc = g["c"]
    gmag = lambda a, b, kind: product_mag(oracle, "matmul_grad_cuda_naive", f64(a), f64(b), cc, hd, kind)
    close(d_p.cpu().numpy(), g["d_p"], 1e-5, "dP", mag=gmag(g["g_o"], v, "rc_cr"))
    d_v = ops.matmul_grad_cuda_naive(ops.qkv_transpose(dev(g["p"], f32), c, hd, "rr"),
                                     ops.qkv_transpose(dev(g["g_o"], f32), c, hd, "rc"), c, hd, "rr_rc")
    close(d_v.cpu().numpy(), g["d_v"], 1e-5, "dV",
          mag=gmag(oracle.qkv_transpose(f64(g["p"]), cc, hd, "rr"), oracle.qkv_transpose(f64(g["g_o"]), cc, hd, "rc"), "rr_rc"))
    d_s = ops.softmax_last_dim_backward(rows, dev(g["p"], f32), dev(g["d_p"], f32))
    close(d_s.cpu().numpy(), g["d_s"], 1e-5, "dS", mag=softmax_bwd_mag(g["rows"], f64(g["p"]), f64(g["d_p"])))
    d_q = ops.matmul_grad_cuda_naive(dev(g["d_s"], f32), dev(kt, f32), c, hd, "rr_rc")
    close(d_q.cpu().numpy(), g["d_q"], 1e-5, "dQ", mag=gmag(g["d_s"], kt, "rr_rc"))
    d_kt = ops.matmul_grad_cuda_naive(ops.qkv_transpose(dev(q, f32), c, hd, "rc"),
                                      ops.qkv_transpose(dev(g["d_s"], f32), c, hd, "rr"), c, hd, "cr_rr")
    close(d_kt.cpu().numpy(), g["d_kt"], 1e-5, "dK^T",
          mag=gmag(oracle.qkv_transpose(f64(q), cc, hd, "rc"), oracle.qkv_transpose(f64(g["d_s"]), cc, hd, "rr"), "cr_rr"))
    unsort, cnt = ops.return_inverse(ops.flatten_indices(dev(np.ascontiguousarray(g["ind"].T)), [B, n]), -1)
    np.testing.assert_array_equal(unsort.cpu().numpy(), g["unsort"])
    assert cnt == int(g["n_unique"])
