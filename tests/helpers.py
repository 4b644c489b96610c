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


# every values check of a session: (what, worst |err| / bound, worst pure relative error over the elements that carry
# at least a thousandth of their own scale); conftest prints the tightest ones at the end of the run
CHECK_LOG = []


def close(out, ref, rtol, what="", mag=None, seg=None):
    """Values check with a bound that follows the conditioning of each element:

        |out - ref| <= rtol * scale_of_the_element

    ``mag``  the element's condition magnitude, e.g. sum_k |a_ik * b_kj| for a product (computed by
             running the same fp64 oracle on the absolute values of the operands): a result that has
             lost a low-order term of its sum fails, cancellation inside the sum does not;
    ``seg``  segment ids of a flat array (the softmax row of every entry): scale = |ref| + the largest
             |ref| of the element's own segment;
    neither: arrays with two or more axes use their rows (last axis) as segments: a token's own output
             row, an output channel's own weight row.  A flat array needs ``mag`` or ``seg``
             (``seg="all"`` = one segment, for small homogeneous vectors such as a bias gradient).
    """
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert out.shape == ref.shape, f"{what}: shape {out.shape} vs {ref.shape}"
    if ref.size == 0:
        return
    aref = np.abs(ref)
    if mag is not None:
        scale = np.maximum(np.abs(np.asarray(mag, dtype=np.float64)).reshape(ref.shape), aref)
    elif isinstance(seg, str):
        assert seg == "all"
        scale = aref + aref.max()
    elif seg is not None:
        seg = np.asarray(seg).reshape(-1)
        top = np.zeros(int(seg.max()) + 1)
        np.maximum.at(top, seg, aref.reshape(-1))
        scale = aref + top[seg].reshape(ref.shape)
    else:
        assert ref.ndim >= 2, f"{what}: a flat array needs mag= or seg="
        scale = aref + aref.max(axis=-1, keepdims=True)
    err = np.abs(out - ref)
    bound = rtol * scale
    with np.errstate(divide="ignore", invalid="ignore"):
        ratio = np.where(bound > 0, err / bound, np.where(err > 0, np.inf, 0.0))
        carrying = aref >= 1e-3 * scale
        rel = float((err[carrying] / aref[carrying]).max()) if carrying.any() else 0.0
    worst = int(np.argmax(ratio))
    CHECK_LOG.append((what, float(ratio.flat[worst]), rel, rtol))
    print(f"[values] {what}: worst |err|/bound {ratio.flat[worst]:.3f}, worst relative error {rel:.2e} (rtol {rtol:g})")
    assert ratio.flat[worst] <= 1.0, (f"{what}: worst element {worst}: out={out.flat[worst]!r} "
                                      f"ref={ref.flat[worst]!r} err={err.flat[worst]:.3e} bound={bound.flat[worst]:.3e}")


def product_mag(orc, fn, *args):
    """The oracle's product ``fn`` on the absolute values of its floating-point operands: sum_k |a_ik| |b_kj| per
    output element, the quantity a relative tolerance of a sum refers to."""
    conv = [np.abs(a) if isinstance(a, np.ndarray) and a.dtype.kind == "f" else a for a in args]
    res = getattr(orc, fn)(*conv)
    return res[1] if isinstance(res, tuple) else res


class BiasGradMagnitude:
    """sum |dS| over the attention entries that share a row of the relative position bias table: the magnitude the
    table gradient (a sum of dS over those entries) is conditioned by.  ``probe`` goes to the CPU path."""

    def __init__(self, heads, n):
        import torch
        self.probe = {"abs_ds": torch.zeros(heads, n, n, dtype=torch.float64)}

    def table(self, relative_position_index, table_rows):
        import torch
        a = self.probe["abs_ds"]
        H, n, _ = a.shape
        mag = torch.zeros(table_rows, H, dtype=torch.float64)
        mag.index_add_(0, relative_position_index[:n, :n].reshape(-1).long().cpu(), a.permute(1, 2, 0).reshape(-1, H))
        return mag.numpy()


PATHS = ["resident", "fused", "operators"]


def set_path(attn, path):
    """Select the implementation behind WindowAttentionSparse.forward: "resident" = window-resident
    kernels, "fused" = block products with the attention matrix in memory, "operators" = the
    operator-by-operator composition of the reference."""
    attn.fused = path != "operators"
    attn.resident = {"resident": True, "fused": False, "operators": None}[path]
