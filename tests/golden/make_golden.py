"""Writes tests/golden/tiny_ops.npz: inputs and expected outputs of every operator on a tiny
case (3 windows holding 1, 2 and 5 tokens, 2 heads, head dim 4, 8 positions per window).

The expected values come from this repository's own CPU oracle after it has been pinned
(tests/test_oracle_pins.py); the reference holds no fixtures for this path.  The file exists so
that a change of the oracle or of the kernels shows up as a diff against committed numbers.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

import oracle  # noqa: E402
from helpers import qkv_operands, ragged_window_indices  # noqa: E402


def main():
    rng = np.random.default_rng(2024)
    counts, n, H, hd = [1, 2, 0, 5], 8, 2, 4
    B = len(counts)
    ind = ragged_window_indices(rng, counts, n)
    d = qkv_operands(oracle, ind, B, n, H, hd, rng, dtype=np.float64)
    s_idx, s_val, s_shape, c = oracle.matmul_cuda_naive(d["q"], d["qi"], d["q_shape"], d["kt"], d["ki"], d["k_shape"], "q_k")
    flat = oracle.flatten_indices(s_idx[:3], s_shape[:3])
    rows = oracle.unique_consecutive_indices(flat)
    p = oracle.softmax_last_dim_forward(rows, s_val)
    o_idx, o_val, o_shape, _ = oracle.matmul_cuda_naive(p, s_idx, s_shape, d["v"], d["qi"], d["q_shape"], "qk_v")
    g_o = rng.standard_normal(len(o_val))
    d_p = oracle.matmul_grad_cuda_naive(g_o, d["v"], c, hd, "rc_cr")
    d_v = oracle.matmul_grad_cuda_naive(oracle.qkv_transpose(p, c, hd, "rr"), oracle.qkv_transpose(g_o, c, hd, "rc"), c, hd, "rr_rc")
    d_s = oracle.softmax_last_dim_backward(rows, p, d_p)
    d_q = oracle.matmul_grad_cuda_naive(d_s, d["kt"], c, hd, "rr_rc")
    d_kt = oracle.matmul_grad_cuda_naive(oracle.qkv_transpose(d["q"], c, hd, "rc"), oracle.qkv_transpose(d_s, c, hd, "rr"), c, hd, "cr_rr")
    tok = oracle.flatten_indices(np.ascontiguousarray(ind.T), [B, n])
    unsort, n_unique = oracle.return_inverse(tok, -1)
    np.savez(os.path.join(HERE, "tiny_ops.npz"), ind=ind, B=B, n=n, H=H, hd=hd, qkv=d["qkv"],
             idx_qv=d["idx_qv"], idx_k=d["idx_k"], sorted_qv=d["sorted_qv"], sorted_k=d["sorted_k"],
             s_idx=s_idx, s_val=s_val, c=c, flat=flat, rows=rows, p=p, o_idx=o_idx, o_val=o_val, g_o=g_o,
             d_p=d_p, d_v=d_v, d_s=d_s, d_q=d_q, d_kt=d_kt, tok=tok, unsort=unsort, n_unique=n_unique)
    print("wrote tiny_ops.npz:", len(ind), "voxels,", len(s_val), "attention non-zeros")


if __name__ == "__main__":
    main()
