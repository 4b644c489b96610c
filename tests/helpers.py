"""Shared input builders for the parity tests (numpy side)."""
from __future__ import annotations

import numpy as np


def random_window_indices(rng, n_windows_slots, n, n_tokens):
    """Distinct (window, pos) pairs in random order, int32 [N, 2]."""
    keys = rng.choice(n_windows_slots * n, size=n_tokens, replace=False)
    return np.stack([keys // n, keys % n], 1).astype(np.int32)


def ragged_window_indices(rng, counts, n, slot_stride=1):
    """One window per entry of ``counts`` (tokens per window, 0 allowed), window ids spaced by
    ``slot_stride``; positions are a random subset of [0, n).  Random voxel order."""
    rows = []
    for k, c in enumerate(counts):
        pos = np.sort(rng.choice(n, size=c, replace=False))
        rows.append(np.stack([np.full(c, k * slot_stride), pos], 1))
    ind = np.concatenate(rows, 0).astype(np.int32)
    return ind[rng.permutation(len(ind))]


def qkv_operands(orc, ind, B, n, H, hd, rng, dtype=np.float32, scale=1.0):
    """Q, K^T, V COO operands exactly as qkv_sparse_cuda assembles them
    (reference sparse_swin/swin3d_base.py:483-498), built with the oracle."""
    N = len(ind)
    qkv = (rng.standard_normal((N, 3, H, hd)) * scale).astype(dtype)
    iqv, sqv, ik, sk = orc.qkv_sparse_indices(ind, B, n, H, hd)
    qi = np.ascontiguousarray(iqv[:, sqv])
    ki = np.ascontiguousarray(ik[:, sk])
    q = qkv[:, 0].reshape(-1)[sqv]
    kt = qkv[:, 1].reshape(-1)[sk]
    v = qkv[:, 2].reshape(-1)[sqv]
    return dict(qkv=qkv, q=q, kt=kt, v=v, qi=qi, ki=ki, q_shape=[B, H, n, hd], k_shape=[B, H, hd, n],
                sorted_qv=sqv, sorted_k=sk, idx_qv=iqv, idx_k=ik)


def close(out, ref, rtol, what=""):
    """|out - ref| <= rtol * (|ref| + max|ref|): relative to the element, with an absolute
    floor tied to the array's scale so that cancellation near zero does not count."""
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert out.shape == ref.shape, f"{what}: shape {out.shape} vs {ref.shape}"
    if ref.size == 0:
        return
    scale = np.abs(ref).max()
    err = np.abs(out - ref)
    bound = rtol * (np.abs(ref) + scale)
    worst = np.argmax(err - bound)
    assert (err <= bound).all(), (f"{what}: worst element {worst}: out={out.flat[worst]!r} "
                                  f"ref={ref.flat[worst]!r} err={err.flat[worst]:.3e} bound={bound.flat[worst]:.3e}")


PATHS = ["resident", "fused", "operators"]


def set_path(attn, path):
    """Select the implementation behind WindowAttentionSparse.forward: "resident" = window-resident
    kernels, "fused" = block products with the attention matrix in memory, "operators" = the
    operator-by-operator composition of the reference."""
    attn.fused = path != "operators"
    attn.resident = {"resident": True, "fused": False, "operators": None}[path]
