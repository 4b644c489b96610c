"""PyTorch-CPU restatement of the sparse window-attention path — TEST INFRASTRUCTURE ONLY.

This is the path the reference's README describes as its slow baseline: one ``torch.mm`` per
(window, head) for Q.K^T and for attn.V (``README.md:29-30``) and the scatter-based softmax
(``README.md:66-75``, ``sparse_swin/swin3d_base.py:455-480``), with the backward pass left to
``torch.autograd``.  It is used (a) as the end-to-end checker of ``WindowAttentionSparse``
(forward values and gradients) and (b) as the timed ``cpu_baseline`` of ``bench.py``.
The product never imports it.

Two softmax flavours exist because the reference itself has two:
  "ops"    exp(v - max(0, rowmax)) / (rowsum + 1e-8)   — the operator (ops.cu:128-167)
  "readme" exp(v - rowmax) / rowsum                    — the README / softmax_last_dim_
They differ by at most 1e-8 relative unless a whole row is below about -87.
"""
from __future__ import annotations

import math

import numpy as np
import torch


def sparse_softmax_readme(vals: torch.Tensor, idx_row: torch.Tensor, n_rows: int) -> torch.Tensor:
    """README.md:66-75 verbatim in behaviour: scatter amax, exp, scatter add, divide."""
    src_max = torch.zeros(n_rows, dtype=vals.dtype)
    src_max = src_max.scatter_reduce(0, idx_row, vals, reduce="amax", include_self=False)
    out = (vals - src_max.index_select(0, idx_row)).exp()
    out_sum = torch.zeros(n_rows, dtype=out.dtype).scatter_add(0, idx_row, out)
    return out / out_sum.index_select(0, idx_row)


def sparse_softmax_ops(vals: torch.Tensor, idx_row: torch.Tensor, n_rows: int) -> torch.Tensor:
    """The operator's variant: maximum taken against a zero-initialised buffer, sum + 1e-8."""
    src_max = torch.zeros(n_rows, dtype=vals.dtype)
    src_max = src_max.scatter_reduce(0, idx_row, vals, reduce="amax", include_self=True)
    out = (vals - src_max.index_select(0, idx_row)).exp()
    out_sum = torch.zeros(n_rows, dtype=out.dtype).scatter_add(0, idx_row, out) + 1e-8
    return out / out_sum.index_select(0, idx_row)


def window_order(win_idx: np.ndarray, n: int):
    """Token order (window, pos), per-window token counts of the non-empty windows."""
    key = win_idx[:, 0].astype(np.int64) * n + win_idx[:, 1]
    perm = np.argsort(key, kind="stable")
    wins, counts = np.unique(win_idx[perm, 0], return_counts=True)
    return perm, wins, counts


def window_attention_cpu(features: torch.Tensor, win_idx: np.ndarray, n: int, num_heads: int,
                         qkv_w, qkv_b, proj_w, proj_b, rpb: torch.Tensor, mask: np.ndarray | None,
                         softmax: str = "ops", probe: dict | None = None) -> torch.Tensor:
    """Forward of the attention module on the CPU; differentiable w.r.t. every tensor input.

    features [N, D]; win_idx int32 [N, 2] = (window, pos); rpb [H, n, n] (already gathered from
    the bias table); mask int8 [nW, n] region ids or None.  Returns [N, D] in input voxel order.
    ``probe``: an empty dict; it receives what the conditioning of the score gradient dS = P (dP - D),
    dP = dO V^T, D = dO . O, is made of: ``P`` (the attention values), ``cells`` (index (head, pos_i, pos_j) of every
    entry in an [H, n, n] array), ``sizes`` (tokens per window), ``V`` and ``O`` in window order and, during the
    backward pass, ``dO`` (the gradient that reaches O).
    """
    N, D = features.shape
    H, hd = num_heads, D // num_heads
    scale = hd ** -0.5
    qkv = torch.nn.functional.linear(features, qkv_w, qkv_b).reshape(N, 3, H, hd)
    perm, wins, counts = window_order(win_idx, n)
    perm_t = torch.from_numpy(perm)
    q = qkv[:, 0].index_select(0, perm_t) * scale
    k = qkv[:, 1].index_select(0, perm_t)
    v = qkv[:, 2].index_select(0, perm_t)
    pos = torch.from_numpy(win_idx[perm, 1].astype(np.int64))
    mask_t = None if mask is None else torch.from_numpy(np.asarray(mask)).to(torch.int64)

    # one split per operand: its backward is a single concatenation, whereas slicing
    # q[start:start+c] per window would make autograd build a full-size zero tensor per slice
    sizes = [int(c) for c in counts]
    q_w, k_w, v_w = q.split(sizes), k.split(sizes), v.split(sizes)

    scores, row_ids, cells = [], [], []
    start = 0
    row_base = 0
    for k_win, (w, c) in enumerate(zip(wins, counts)):
        c = int(c)
        p = pos[start:start + c]
        if mask_t is not None:
            region = mask_t[int(w) % mask_t.shape[0]].index_select(0, p)
            penalty = (region[None, :] != region[:, None]).to(features.dtype) * -100.0
        for h in range(H):
            s = torch.mm(q_w[k_win][:, h], k_w[k_win][:, h].t())
            s = s + rpb[h].index_select(0, p).index_select(1, p)
            if mask_t is not None:
                s = s + penalty
            if probe is not None:
                cells.append(((h * n + p[:, None]) * n + p[None, :]).reshape(-1))
            scores.append(s.reshape(-1))
            row_ids.append(torch.arange(row_base, row_base + c).repeat_interleave(c))
            row_base += c
        start += c
    vals = torch.cat(scores)
    idx_row = torch.cat(row_ids)
    sm = sparse_softmax_ops if softmax == "ops" else sparse_softmax_readme
    attn = sm(vals, idx_row, row_base)
    if probe is not None:
        probe.update(P=attn.detach(), cells=torch.cat(cells), sizes=sizes, V=v.detach())

    outs = []
    blocks = attn.split([c * c for c in sizes for _ in range(H)])
    for k_win, c in enumerate(sizes):
        per_head = [torch.mm(blocks[k_win * H + h].reshape(c, c), v_w[k_win][:, h]) for h in range(H)]
        outs.append(torch.stack(per_head, 1).reshape(c, D))      # (token, head, channel)
    out_sorted = torch.cat(outs, 0)
    if probe is not None:
        probe["O"] = out_sorted.detach()
        if out_sorted.requires_grad:
            out_sorted.register_hook(lambda g: probe.__setitem__("dO", g.detach()))
    inv = np.empty_like(perm)
    inv[perm] = np.arange(N)
    out = out_sorted.index_select(0, torch.from_numpy(inv))
    return torch.nn.functional.linear(out, proj_w, proj_b)


def dense_window_attention_reference(features, win_idx, n, num_heads, qkv_w, qkv_b, proj_w, proj_b,
                                     rpb, mask):
    """Textbook dense Swin window attention (zero-padded windows + key padding mask via -inf),
    used only to pin :func:`window_attention_cpu` itself: softmax(QK^T*scale + bias + mask) V."""
    N, D = features.shape
    H, hd = num_heads, D // num_heads
    qkv = torch.nn.functional.linear(features, qkv_w, qkv_b).reshape(N, 3, H, hd)
    wins = np.unique(win_idx[:, 0])
    slot = {int(w): i for i, w in enumerate(wins)}
    W = len(wins)
    dense = torch.zeros(W, n, 3, H, hd, dtype=features.dtype)
    present = torch.zeros(W, n, dtype=torch.bool)
    wi = torch.tensor([slot[int(w)] for w in win_idx[:, 0]])
    pi = torch.from_numpy(win_idx[:, 1].astype(np.int64))
    dense = dense.index_put((wi, pi), qkv)
    present[wi, pi] = True
    q = dense[:, :, 0].permute(0, 2, 1, 3) * hd ** -0.5
    k = dense[:, :, 1].permute(0, 2, 1, 3)
    v = dense[:, :, 2].permute(0, 2, 1, 3)
    s = q @ k.transpose(-1, -2) + rpb[None]
    if mask is not None:
        m = torch.from_numpy(np.asarray(mask)).to(torch.int64)[torch.from_numpy(wins.astype(np.int64)) % mask.shape[0]]
        s = s + ((m[:, None, :] != m[:, :, None]).to(features.dtype) * -100.0)[:, None]
    s = s.masked_fill(~present[:, None, None, :], -math.inf)
    p = torch.softmax(s, -1)
    o = (p @ v).permute(0, 2, 1, 3).reshape(W, n, D)
    return torch.nn.functional.linear(o[wi, pi], proj_w, proj_b)
