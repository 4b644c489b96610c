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


# every values check of a session: (what, worst |err| / bound, worst pure relative error |err| / |ref| over the elements
# that are at least a tenth of their own scale); conftest prints the tightest ones at the end of the run
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
    bound = rtol * scale + 1e-30                             # fp32 results below about 1e-38 underflow
    with np.errstate(divide="ignore", invalid="ignore"):
        ratio = np.where(bound > 0, err / bound, np.where(err > 0, np.inf, 0.0))
        carrying = (aref >= 0.1 * scale) & (aref > 0)        # elements of the size of their own scale
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


def softmax_bwd_mag(rows, y, g):
    """Condition magnitude of the softmax gradient gx_i = y_i (g_i - sum_j g_j y_j): y_i (|g_i| + sum_j |g_j| y_j).
    The two terms cancel where a row is dominated by one entry, so |gx_i| itself says nothing about the rounding
    error to expect."""
    rows = np.asarray(rows).reshape(-1)
    y = np.abs(np.asarray(y, dtype=np.float64))
    g = np.abs(np.asarray(g, dtype=np.float64))
    s = np.bincount(rows, weights=g * y)
    return y * (g + s[rows])


def score_grad_mag(P, dO, V, O):
    """Condition magnitude of dS = P (dP - D), dP = dO V^T, D_i = dO_i . O_i, for one (window, head):
    P (|dO| |V|^T + |dO| . |O|).  P [c, c], dO, V, O [c, hd] (torch, fp64)."""
    return P * (dO.abs() @ V.abs().t() + (dO.abs() * O.abs()).sum(-1, keepdim=True))


class BiasGradMagnitude:
    """What the gradient of a relative position bias entry is conditioned by: the sum of score_grad_mag over the
    attention entries that read it.  ``probe`` goes to the CPU path, which fills it."""

    def __init__(self, heads, n):
        self.probe = {}
        self.heads, self.n = heads, n

    def dense(self):
        """[H, n, n]"""
        import torch
        pr = self.probe
        H = self.heads
        P, V = pr["P"].double(), pr["V"].double()
        N = V.shape[0]
        O, dO = pr["O"].double().reshape(N, H, -1), pr["dO"].double().reshape(N, H, -1)
        mags = []
        t0 = e0 = 0
        for c in pr["sizes"]:
            for h in range(H):
                Pw = P[e0:e0 + c * c].reshape(c, c)
                mags.append(score_grad_mag(Pw, dO[t0:t0 + c, h], V[t0:t0 + c, h], O[t0:t0 + c, h]).reshape(-1))
                e0 += c * c
            t0 += c
        out = torch.zeros(H * self.n * self.n, dtype=torch.float64).index_add_(0, pr["cells"], torch.cat(mags))
        return out.reshape(H, self.n, self.n)

    def table(self, relative_position_index, table_rows):
        import torch
        a = self.dense()
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
