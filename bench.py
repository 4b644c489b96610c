#!/usr/bin/env python3
"""Benchmark of the sparse window-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--kernels-json PATH]

Workload (``config.workload``): the stage-1 block pair of the synthetic ScanNet-like room —
``WindowAttentionSparse`` with the regular 5^3 windows, then with the windows shifted by 2,
dim 96, 3 heads, fp32, forward + backward, about 100k voxels.  One step = forward of both
attention modules chained, then backward from N(0,1) upstream gradients.  Inputs (features,
window indices, mask, upstream gradients, weights) are resident in HBM before timing.

``value`` = tokens/s = (attention calls per step x voxels) / step time.

The JSON line also carries
  roofline      the kernel that takes the largest share of a step, timed alone with HIP events
                on the stream it is launched on; achieved = algorithmic bytes / duration
  cpu_baseline  the PyTorch-CPU path (per-window torch.mm + scatter softmax + autograd) timed
                on the host cores on a bounded sample of the same workload
A per-kernel table goes to stderr and, with --kernels-json, to a file.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

# HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE) for the kernels
# below on this workload; None = not measured.  Source summaries live in profiles/.
MEASURED_TRAFFIC_BYTES = {
    # profiles/wattn_kernels_cfg2_pmc.txt and profiles/fused_tok_kernel_cfg2_pmc.txt:
    # FETCH_SIZE x 2.0 KiB + WRITE_SIZE x 1.0 KiB per launch
    "resident forward": 174.2e6,
    "resident backward (dQ,dK,dV,dS)": 490.7e6,
    "resident backward dQ, all groups": 258.0e6,
    "resident backward dK,dV,dS only": 344.5e6,
    "fused dV=P^T dO": 128.1e6,
    "fused dK=dS^T Q": 128.1e6,      # same kernel instantiation and operand shapes as dV
    "fused O=PV": 135.4e6,
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# ------------------------------------------------------------------------------------------
def build_workload(device, name="cfg2"):
    from sparseswin3d_amd import synth
    from sparseswin3d_amd.window_attention import WindowAttentionSparse
    w = {"cfg1": synth.config1, "cfg2": synth.config2, "cfg3": synth.config3, "cfg4": synth.config4}[name]()
    dtype = torch.bfloat16 if w.dtype == "bf16" else torch.float32
    ws = w.window
    shift = tuple(s // 2 for s in ws)
    torch.manual_seed(2)
    N = len(w.coords4)
    blocks = []
    pshape = synth.padded_shape(w.spatial_shape, ws)
    mask = torch.from_numpy(synth.shift_region_mask(pshape, ws, shift)).to(device)
    for sh in ((0, 0, 0), shift):
        idx, nw, n = synth.window_indices(w.coords4, w.spatial_shape, ws, sh)
        st = synth.scene_stats(idx, nw * w.batch_size)
        attn = WindowAttentionSparse(w.dim, w.heads, ws, qkv_bias=True).to(device)
        torch.nn.init.xavier_uniform_(attn.qkv.weight)
        attn = attn.to(dtype)
        blocks.append(dict(attn=attn, idx=torch.from_numpy(idx).to(device), idx_np=idx, slots=nw * w.batch_size,
                           n=n, mask=mask if any(sh) else None, stats=st.describe(w.heads), shift=sh))
    feats = torch.randn(N, w.dim, device=device).to(dtype)
    upstream = torch.randn(N, w.dim, device=device).to(dtype)
    return dict(name=w.name, dtype=dtype, N=N, dim=w.dim, heads=w.heads, blocks=blocks, feats=feats, upstream=upstream,
                mask_np=mask.cpu().numpy(), coords4=torch.from_numpy(w.coords4).to(device),
                spatial_shape=tuple(w.spatial_shape), batch_size=w.batch_size, window=tuple(ws), shift=shift,
                padded=tuple(pshape))


def run_step(wl):
    from sparseswin3d_amd.window_attention import SparseVoxelTensor
    for blk in wl["blocks"]:                                  # as a training step does: fresh gradients
        blk["attn"].zero_grad(set_to_none=True)
    x = wl["feats"].detach().requires_grad_(True)
    h = x
    for b in wl["blocks"]:
        t = SparseVoxelTensor(h, b["idx"], (b["n"],), b["slots"])
        h = b["attn"](t, b["mask"]).features
    h.backward(wl["upstream"])
    return x.grad


# ------------------------------------------------------------------------------------------
def event_time_ms(fn, reps, warmup=2):
    for _ in range(warmup):
        fn()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / reps


def kernel_table(wl, reps=20, only=None):
    """Time every operator's kernels alone on the first block's tensors (regular windows)."""
    from sparseswin3d_amd import _lib, custom_ops as ops
    from sparseswin3d_amd.window_attention import qkv_sparse_cuda
    lib = _lib.load()
    b = wl["blocks"][0]
    H, D = wl["heads"], wl["dim"]
    hd = D // H
    N = wl["N"]
    dev = wl["feats"].device
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ptr = lambda t: C.c_void_p(t.data_ptr())

    qkv = torch.randn(N, 3, H, hd, device=dev)
    q, kt, v = qkv_sparse_cuda(qkv, b["idx"], b["slots"], b["n"])
    s_idx, s_val, s_shape, c = ops.matmul_cuda_naive(q.values, q.indices, q.shape, kt.values, kt.indices, kt.shape, "q_k")
    flat = ops.flatten_indices(s_idx[:3], s_shape[:3])
    rows = ops.unique_consecutive_indices(flat)
    p_val = ops.softmax_last_dim_forward(rows, s_val)
    o_idx, o_val, o_shape, c2 = ops.matmul_cuda_naive(p_val, s_idx, s_shape, v.values, v.indices, v.shape, "qk_v")
    E, A, G = q.values.numel(), s_val.numel(), c.numel()
    s = 4

    # plan once, then the product kernels alone
    m = E
    g_cap = max(1, min(m // hd, b["slots"] * H))
    plan = torch.empty(5 * g_cap, dtype=torch.int32, device=dev)
    totals = (C.c_int64 * 4)()
    nb = lib.sswin_plan_workspace_bytes(m, hd)
    ws = torch.empty(nb, dtype=torch.uint8, device=dev)
    _lib.check(lib.sswin_plan_from_indices(ptr(q.indices), m, hd, ptr(plan), g_cap, totals, ptr(ws), nb, stream))
    c_max = int(totals[3])
    scans = torch.stack([plan.view(5, g_cap)[1, :G], plan.view(5, g_cap)[2, :G]]).reshape(-1).contiguous()
    cc = plan[:G].contiguous()
    out_s = torch.empty(A, device=dev)
    out_si = torch.empty((4, A), dtype=torch.int32, device=dev)
    out_o = torch.empty(E, device=dev)
    out_oi = torch.empty((4, E), dtype=torch.int32, device=dev)
    g_s = torch.randn(A, device=dev)
    g_o = torch.randn(E, device=dev)

    def mm(kind, a, bb, tok, ov, oi, nnz):
        return lambda: _lib.check(lib.sswin_block_matmul(kind, 0, ptr(a), ptr(bb), ptr(tok), m, hd, ptr(plan), g_cap, G,
                                                         c_max, ptr(ov), ptr(oi), nnz, stream))

    def grad(kind, a, bb, out):
        return lambda: _lib.check(lib.sswin_block_matmul_grad(kind, 0, ptr(a), ptr(bb), ptr(cc), ptr(scans), G, hd,
                                                              ptr(out), stream))

    def tr(kind, a, out):
        return lambda: _lib.check(lib.sswin_block_transpose(kind, 0, ptr(a), ptr(cc), ptr(scans), G, hd, ptr(out), stream))

    tmp_e, tmp_a = torch.empty(E, device=dev), torch.empty(A, device=dev)
    idxT = b["idx"].T.contiguous()
    flat_tok = ops.flatten_indices(idxT, [b["slots"], b["n"]])
    perm_idx = o_idx[[0, 2, 1, 3], :].contiguous()
    flat_perm = ops.flatten_indices(perm_idx, [o_shape[0], o_shape[2], o_shape[1], o_shape[3]])

    entries = [
        # name, callable, algorithmic bytes, calls per attention fwd+bwd
        ("qkv_sparse_indices", lambda: ops.qkv_sparse_indices(b["idx"], b["slots"], b["n"], H, hd, _defer_check=True), 8 * N + 40 * E, 1),
        ("plan_from_indices", lambda: _lib.check(lib.sswin_plan_from_indices(ptr(q.indices), m, hd, ptr(plan), g_cap, totals, ptr(ws), nb, stream)), 0, 2),
        ("block_matmul q_k", mm(0, q.values, kt.values, q.indices, out_s, out_si, A), 2 * s * E + (s + 16) * A + 4 * G, 1),
        ("flatten_indices [3,A]", lambda: ops.flatten_indices(s_idx[:3], s_shape[:3]), 16 * A, 1),
        ("unique_consecutive_indices [A]", lambda: ops.unique_consecutive_indices(flat), 8 * A, 1),
        ("softmax_last_dim_forward", lambda: ops.softmax_last_dim_forward(rows, s_val), 12 * A, 1),
        ("block_matmul qk_v", mm(1, p_val, v.values, v.indices, out_o, out_oi, E), s * A + s * E + (s + 16) * E + 4 * G, 1),
        ("permute order from the group structure [E]", lambda: ops.permute_heads_order(o_idx, o_shape), 0, 1),
        ("flatten_indices [4,E] (generic permute)", lambda: ops.flatten_indices(perm_idx, [o_shape[0], o_shape[2], o_shape[1], o_shape[3]]), 0, 0),
        ("sort_indices [E] (generic permute)", lambda: ops.sort_indices(flat_perm), 0, 0),
        ("return_inverse [N]", lambda: ops.return_inverse(flat_tok, b["slots"] * b["n"]), 0, 1),
        ("softmax_last_dim_backward", lambda: ops.softmax_last_dim_backward(rows, p_val, g_s), 16 * A, 1),
        ("grad rc_cr", grad(0, g_o, v.values, tmp_a), 2 * s * E + s * A, 1),
        ("grad rr_rc", grad(1, g_s, kt.values, tmp_e), s * A + 2 * s * E, 2),
        ("grad cr_rr", grad(2, q.values, g_s, tmp_e), s * A + 2 * s * E, 1),
        ("transpose rc", tr(0, q.values, tmp_e), 2 * s * E, 2),
        ("transpose rr", tr(1, g_s, tmp_a), 2 * s * A, 2),
    ]
    # ---- the fused path (what WindowAttentionSparse.forward runs by default) ----
    from sparseswin3d_amd import fused as F
    tp = F.TokenPlan(b["idx"], b["slots"], b["n"], H)
    qkv_c = qkv.contiguous()
    bias = torch.randn(H, b["n"], b["n"], device=dev)
    mask = wl["blocks"][1]["mask"]
    s_f = torch.empty(tp.A, device=dev)
    rows_f = torch.empty(tp.A, dtype=torch.int32, device=dev)
    out_f = torch.empty(N, D, device=dev)
    dqkv = torch.empty_like(qkv_c)
    dbias = torch.zeros(H, b["n"], b["n"], device=dev)
    dt = torch.float32
    bg_bytes = lib.sswin_fused_bias_grad_workspace_bytes(tp.G, H, b["n"])
    bg_ws = torch.empty(int(bg_bytes), dtype=torch.uint8, device=dev)
    f_entries = [
        ("fused token_plan", lambda: F.TokenPlan(b["idx"], b["slots"], b["n"], H), 28 * N + 20 * tp.G, 1),
        ("fused S=QK^T+bias+mask", lambda: F._tokens_to_sq(tp, dt, True, qkv_c, 3 * D, 0, qkv_c, 3 * D, D, hd, 0.17, bias, mask, s_f, rows_f), 8 * E + 8 * A, 1),
        ("fused softmax fwd", lambda: ops.softmax_last_dim_forward(rows_f, s_f), 12 * A, 1),
        ("fused O=PV", lambda: F._sq_to_tokens(tp, dt, False, p_val, qkv_c, 3 * D, 2 * D, out_f, D, 0, hd, 1.0), 4 * A + 8 * E, 1),
        ("fused dP=dO V^T", lambda: F._tokens_to_sq(tp, dt, False, out_f, D, 0, qkv_c, 3 * D, 2 * D, hd, 1.0, None, None, s_f, None), 8 * E + 4 * A, 1),
        ("fused dV=P^T dO", lambda: F._sq_to_tokens(tp, dt, True, p_val, out_f, D, 0, dqkv, 3 * D, 2 * D, hd, 1.0), 4 * A + 8 * E, 1),
        ("fused softmax bwd", lambda: ops.softmax_last_dim_backward(rows_f, p_val, g_s), 16 * A, 1),
        ("fused dQ=dS K", lambda: F._sq_to_tokens(tp, dt, False, g_s, qkv_c, 3 * D, D, dqkv, 3 * D, 0, hd, 0.17), 4 * A + 8 * E, 1),
        ("fused dK=dS^T Q", lambda: F._sq_to_tokens(tp, dt, True, g_s, qkv_c, 3 * D, 0, dqkv, 3 * D, D, hd, 0.17), 4 * A + 8 * E, 1),
        ("fused bias grad", lambda: _lib.check(lib.sswin_fused_bias_grad(ptr(tp.plan), tp.g_cap, tp.G, ptr(tp.tokens), tp.N, H, b["n"], ptr(g_s), ptr(dbias), ptr(bg_ws), bg_bytes, stream)), 4 * A, 1),
    ]

    # ---- the window-resident kernels (what the step runs for heads of 32 channels) ----
    lse = torch.empty(H * N, device=dev)
    mask_p, nmw = ptr(mask), (0 if mask is None else mask.shape[0])
    qa = (ptr(qkv_c), 3 * D, 0, ptr(qkv_c), 3 * D, D, ptr(qkv_c), 3 * D, 2 * D)
    da = (ptr(dqkv), 3 * D, 0, ptr(dqkv), 3 * D, D, ptr(dqkv), 3 * D, 2 * D)
    up_r = torch.randn(N, D, device=dev)

    def r_fwd():
        _lib.check(lib.sswin_window_attention_forward(0, ptr(tp.tasks), tp.g_cap, tp.bucket_counts, ptr(tp.tokens), N, H,
                                                      hd, *qa, C.c_float(0.17), ptr(bias), b["n"], mask_p, nmw,
                                                      ptr(out_f), D, 0, ptr(lse), stream))

    # The step asks for all gradients at once (sides = 3): one launch in which groups of at most
    # 64 tokens get dQ from their key-side tasks and only the larger groups have query-side tasks.
    # The parts are timed alone for comparison: restricted bucket counts = the query-side kernel on
    # the groups of more than 32 tokens, 1 / 2 = the per-side kernels.
    bc = [int(x) for x in tp.bucket_counts]
    cg = tp.plan[:tp.G].to(torch.int64)                                  # plan row 0: tokens of each group
    rows1, rowsL = int(cg[cg <= 32].sum()), int(cg[cg > 32].sum())       # token-head rows of small / large groups
    only_large = [0, bc[1], bc[2], bc[3]]

    def r_bwd(sides, counts=None):
        counts = tp.bucket_counts if counts is None else (C.c_int64 * 4)(*counts)
        return lambda: _lib.check(lib.sswin_window_attention_backward(
            0, ptr(tp.tasks), tp.g_cap, counts, ptr(tp.tokens), N, H, hd, *qa, C.c_float(0.17), ptr(bias),
            b["n"], mask_p, nmw, ptr(out_f), D, 0, ptr(up_r), D, 0, ptr(lse), *da, ptr(s_f), sides, stream))

    from sparseswin3d_amd.window_attention import relative_position_index_3d
    ti = F.BiasTableIndex.build(relative_position_index_3d(wl["blocks"][0]["attn"].window_size).to(dev), 729)
    d_table = torch.empty(729, H, device=dev)
    tg_bytes = lib.sswin_bias_table_grad_workspace_bytes(tp.G, H, 729)
    tg_ws = torch.empty(int(tg_bytes), dtype=torch.uint8, device=dev)

    def r_table_grad():
        _lib.check(lib.sswin_bias_table_grad(ptr(tp.plan), tp.g_cap, tp.G, ptr(tp.tokens), tp.N, H, b["n"], ptr(ti.code),
                                             ti.offset0, 729, ptr(s_f), ptr(d_table), ptr(tg_ws), tg_bytes, stream))

    r_fwd()                                       # lse and out_f must hold a real forward for the backward timings
    r_entries = [
        ("resident token_plan", lambda: F.TokenPlan(b["idx"], b["slots"], b["n"], H), 28 * N + 36 * tp.G, 1),
        ("resident forward", r_fwd, 16 * E + 4 * H * N, 1),
        ("resident backward (dQ,dK,dV,dS)", r_bwd(3), 32 * E + 4 * A + 4 * H * N, 1),
        ("resident backward dQ, groups > 32 tokens", r_bwd(1, only_large), (24 * hd + 4) * rowsL, 0),
        ("resident backward dQ, all groups", r_bwd(1), 24 * E + 4 * H * N, 0),
        ("resident backward dK,dV,dS only", r_bwd(2), 28 * E + 4 * A + 4 * H * N, 0),
        ("resident bias table grad", r_table_grad, 4 * A, 1),
        ("resident bias grad [H,n,n]", lambda: _lib.check(lib.sswin_fused_bias_grad(ptr(tp.plan), tp.g_cap, tp.G, ptr(tp.tokens), tp.N, H, b["n"], ptr(s_f), ptr(dbias), ptr(bg_ws), bg_bytes, stream)), 4 * A, 0),
    ]

    def measure(items, path):
        rows_ = []
        for name, fn, nbytes, calls in items:
            ms = event_time_ms(fn, reps)
            gbps = nbytes / ms / 1e6 if nbytes else None
            rows_.append(dict(kernel=name, path=path, ms=ms, algorithmic_bytes=nbytes, calls=calls,
                              achieved_gbps=gbps, frac=(gbps / HBM_PEAK_GBPS) if gbps else None))
        return rows_

    if only is not None:
        # profiling mode: run the named kernels (substring match) `reps` times each, plus a plain
        # device-to-device copy of known size that calibrates the FETCH_SIZE / WRITE_SIZE counters
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        picked = [e for e in r_entries + f_entries + entries + projection_entries(wl) if only in e[0]]
        for name, fn, nbytes, calls in picked:
            log(f"profiling {name}: {reps} launches, algorithmic bytes {nbytes}")
            for _ in range(reps):
                fn()
        for _ in range(reps):
            dst.copy_(src)
        torch.cuda.synchronize()
        log(f"calibration copy: {reps} launches of {src.numel() * 4} bytes read and written")
        return [], dict(N=N, E=E, A=A, G=G, c_max=c_max)
    table = measure(r_entries, "resident") + measure(f_entries, "fused") + measure(entries, "operators")
    table += measure(stage_entries(wl), "stage")
    table += measure(projection_entries(wl), "projections")
    return table, dict(N=N, E=E, A=A, G=G, c_max=c_max)


def stage_entries(wl):
    """Index glue of a stage (block and stage level callers of the attention): the kernels, and
    the tensor-op chains of the reference's formulation they replace (calls = 0)."""
    from sparseswin3d_amd import layers
    from sparseswin3d_amd.window_attention import SparseVoxelTensor
    N, D = wl["N"], wl["dim"]
    c4, ws, sh, pd = wl["coords4"], wl["window"], wl["shift"], wl["padded"]
    n = ws[0] * ws[1] * ws[2]
    windows = (pd[0] // ws[0]) * (pd[1] // ws[1]) * (pd[2] // ws[2])
    x = SparseVoxelTensor(wl["feats"].float(), c4, wl["spatial_shape"], wl["batch_size"])
    plan, coords, _ = layers.downsample_plan(x, 2)
    M = plan.windows

    def torch_partition():
        t = SparseVoxelTensor(x.features, c4, pd, wl["batch_size"])
        t = layers.roll_sparse_tensor(t, tuple(-s for s in sh), (1, 2, 3))
        return layers.window_partition_sparse(t, ws)

    def torch_pool():
        inv = torch.repeat_interleave(torch.arange(M, device=c4.device), plan.plan[:M].long())
        out = torch.zeros(M, D, device=c4.device).index_add_(0, inv, x.features[plan.tokens[:N].long()])
        return out / plan.plan[:M, None]

    return [
        ("stage window indices (pad+roll+partition)", lambda: layers.sparse_window_indices(c4, wl["batch_size"], pd, ws, sh), 24 * N, 1),
        ("stage shift mask", lambda: layers.compute_mask(list(pd), list(ws), list(sh), c4.device), windows * n, 1),
        ("stage merge plan (2x2x2 cells, coords)", lambda: layers.downsample_plan(x, 2), 16 * N + 20 * N + 16 * M, 1),
        ("stage merge mean pool", lambda: layers._PoolWindows.apply(x.features, plan, True), 4 * D * (N + M), 1),
        ("torch roll + partition (reference form)", torch_partition, 24 * N, 0),
        ("torch index_add mean pool", torch_pool, 4 * D * (N + M), 0),
    ]


def projection_entries(wl):
    """The qkv and proj nn.Linear of one attention call (fp32 on the bf16 matrix cores with split
    operands), and the library GEMMs they replace (calls = 0)."""
    from sparseswin3d_amd import window_attention as wa
    N, D = wl["N"], wl["dim"]
    dev = wl["feats"].device
    x = torch.randn(N, D, device=dev)
    entries = []
    for name, P in (("qkv", 3 * D), ("proj", D)):
        w = torch.randn(P, D, device=dev) * 0.1
        b = torch.randn(P, device=dev)
        dy = torch.randn(N, P, device=dev)
        io = 4 * N * (D + P)
        entries += [
            (f"{name} forward", (lambda w=w, b=b: wa._split_linear_forward(x, w, b)), io + 4 * P * D, 1),
            (f"{name} weight+bias gradient", (lambda dy=dy: wa._split_linear_weight_grad(dy, x, True)), io + 4 * P * D, 1),
        ]
        def lib_dx(dy=dy, w=w):
            with wa._rocblas_gemm():
                return dy @ w

        entries.append((f"{name} input gradient", (lambda dy=dy, w=w: wa._split_linear_input_grad(dy, w)), io + 4 * P * D, 1))

        def lib_fwd(w=w, b=b):
            with wa._rocblas_gemm():
                return torch.nn.functional.linear(x, w, b)

        def lib_wgrad(dy=dy):
            with wa._rocblas_gemm():
                return dy.t() @ x, wa._column_sum(dy)

        entries += [(f"{name} forward, library GEMM", lib_fwd, io + 4 * P * D, 0),
                    (f"{name} weight+bias gradient, library GEMM + column sums", lib_wgrad, io + 4 * P * D, 0)]
        entries.append((f"{name} input gradient, library GEMM", lib_dx, io + 4 * P * D, 0))
    return entries


# ------------------------------------------------------------------------------------------
def cpu_baseline(wl, target_tokens=None, budget_s=15.0, max_repeats=3):
    """README path on the host cores, forward + backward, on block 0 (regular windows).

    Bounded sample: the whole first attention call of the workload (or its first
    `target_tokens` voxels in window order, whole windows), timed repeatedly for about
    `budget_s` seconds after a warm-up on a small prefix."""
    from oracle import cpu_path
    b = wl["blocks"][0]
    idx = b["idx_np"]
    order = np.argsort(idx[:, 0], kind="stable")
    take = order[:target_tokens or len(order)]
    # keep whole windows only
    last_win = idx[take[-1], 0]
    take = order[idx[order, 0] <= last_win]
    sub_idx = idx[take]
    attn = b["attn"]
    p = {k: v.detach().float().cpu() for k, v in attn.state_dict().items()}
    n = b["n"]
    feats = wl["feats"][torch.from_numpy(take).to(wl["feats"].device)].cpu().requires_grad_(True)
    up = wl["upstream"][torch.from_numpy(take).to(wl["feats"].device)].cpu()
    table = p["relative_position_bias_table"].clone().requires_grad_(True)
    qw = p["qkv.weight"].clone().requires_grad_(True)
    pw = p["proj.weight"].clone().requires_grad_(True)
    rel = attn.relative_position_index.cpu()[:n, :n].reshape(-1)

    def once(f, ix, u):
        rpb = table[rel].reshape(n, n, -1).permute(2, 0, 1)
        out = cpu_path.window_attention_cpu(f, ix, n, attn.num_heads, qw, p.get("qkv.bias"), pw,
                                            p["proj.bias"], rpb, None, softmax="readme")
        out.backward(u)

    warm = idx[order[:4000], 0].max()
    wsel = idx[take, 0] < warm
    once(feats[wsel].detach().requires_grad_(True), sub_idx[wsel], up[wsel])     # warm-up
    repeats, t0 = 0, time.perf_counter()
    while repeats < max_repeats and (repeats == 0 or time.perf_counter() - t0 < budget_s):
        once(feats, sub_idx, up)
        repeats += 1
        log(f"cpu baseline pass {repeats}: {time.perf_counter() - t0:.1f} s elapsed")
    dt = (time.perf_counter() - t0) / repeats
    return dict(value=len(take) / dt, unit="tokens/s", cores=torch.get_num_threads(), kind="port",
                sample=f"one WindowAttentionSparse fwd+bwd (regular windows) on the first {len(take)} voxels "
                       f"({len(np.unique(sub_idx[:, 0]))} windows) of the workload, {dt:.1f} s per pass x {repeats}, "
                       f"host has {os.cpu_count()} logical cpus")


# ------------------------------------------------------------------------------------------
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg2", choices=["cfg1", "cfg2", "cfg3", "cfg4"],
                    help="cfg2 is the benchmark; the others report the step time only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel table")
    ap.add_argument("--kernels-json", default=None)
    ap.add_argument("--profile-kernel", default=None, metavar="NAME",
                    help="run only the kernels whose table name contains NAME (for rocprofv3) and exit")
    ap.add_argument("--profile-reps", type=int, default=5)
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (windows are independent; sharding is "
                 "described in DESIGN.md); rerun with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no HIP GPU visible")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    wl = build_workload(device, args.workload)
    if args.workload != "cfg2":
        args.no_cpu = args.no_kernels = True
    log(f"workload {wl['name']}: N={wl['N']}, blocks: " + "; ".join(str(b["stats"]) for b in wl["blocks"]))
    if args.profile_kernel is not None:
        kernel_table(wl, reps=args.profile_reps, only=args.profile_kernel)
        return

    for _ in range(args.warmup):
        run_step(wl)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_step(wl)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    calls = len(wl["blocks"])
    value = calls * wl["N"] / (dt / args.steps)

    # the attention launches inside real steps: HIP events on the launch stream around each
    # library call (a few extra steps after the timed region, so the events do not perturb `value`)
    from sparseswin3d_amd import fused
    fused.launch_timer = []
    for _ in range(max(3, min(10, args.steps))):
        run_step(wl)
    torch.cuda.synchronize()
    in_step = {}
    for name, start, stop in fused.launch_timer:
        in_step.setdefault(name, []).append(start.elapsed_time(stop))
    fused.launch_timer = None
    in_step = {k: sum(v) / len(v) for k, v in in_step.items()}
    log("attention launches inside a step (HIP events, mean over both blocks): " +
        ", ".join(f"{k} {v:.4f} ms" for k, v in in_step.items()))

    roofline = None
    sizes = {}
    if not args.no_kernels:
        table, sizes = kernel_table(wl)
        log(f"{'kernel':36s} {'ms':>9s} {'calls':>5s} {'alg MB':>9s} {'GB/s':>9s} {'% HBM':>7s}")
        summary = {}
        titles = {"stage": "-- index glue of one stage (window indices, mask, stride-2 merge) --",
                  "projections": "-- qkv and proj layers of one attention call (dense [N, C] GEMMs) --"}
        scope = {"stage": "once per stage", "projections": "one attention fwd+bwd"}
        for path in ("resident", "fused", "operators", "stage", "projections"):
            rows_ = [r for r in table if r["path"] == path]
            log(titles.get(path, f"-- {path} path, one attention forward+backward --"))
            for r in rows_:
                log(f"{r['kernel']:36s} {r['ms']:9.4f} {r['calls']:5d} {r['algorithmic_bytes'] / 1e6:9.1f} "
                    f"{(r['achieved_gbps'] or 0):9.1f} {100 * (r['frac'] or 0):7.2f}")
            ms_ = sum(r["ms"] * r["calls"] for r in rows_)
            alg = sum(r["algorithmic_bytes"] * r["calls"] for r in rows_)
            summary[path] = dict(ms=round(ms_, 4), algorithmic_bytes=alg,
                                 frac=round(alg / ms_ / 1e6 / HBM_PEAK_GBPS, 4))
            log(f"{path} kernels, {scope.get(path, 'one attention fwd+bwd')}: {ms_:.3f} ms for {alg / 1e6:.1f} MB algorithmic "
                f"= {alg / ms_ / 1e6:.1f} GB/s = {100 * alg / ms_ / 1e6 / HBM_PEAK_GBPS:.2f}% of HBM peak")
        # the step runs the window-resident path: its slowest kernel is the dominant one
        # (the token plan is a sequence of small launches, not a kernel)
        dom = max((r for r in table if r["path"] == "resident" and "token_plan" not in r["kernel"]),
                  key=lambda r: r["ms"] * r["calls"])
        # its duration inside the step (events above) is what the roofline entry uses; the same
        # launch repeated back to back on its own (the table) runs 10-20 % slower
        step_ms = in_step.get("window_attention_backward") if "backward (dQ,dK,dV,dS)" in dom["kernel"] else None
        ms = step_ms or dom["ms"]
        gbps = dom["algorithmic_bytes"] / ms / 1e6
        roofline = dict(bound="hbm", kernel=dom["kernel"], achieved=round(gbps, 1),
                        peak=HBM_PEAK_GBPS, unit="GB/s", frac=round(gbps / HBM_PEAK_GBPS, 4),
                        traffic=MEASURED_TRAFFIC_BYTES.get(dom["kernel"]),
                        algorithmic_bytes=dom["algorithmic_bytes"], ms=round(ms, 4),
                        ms_alone=round(dom["ms"], 4), timed="inside the step" if step_ms else "alone",
                        path_summaries=summary)
        if args.kernels_json:
            with open(args.kernels_json, "w") as f:
                json.dump(dict(sizes=sizes, kernels=table), f, indent=1)

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(wl)
        log(f"cpu baseline: {cpu}")

    line = {
        "metric": "window-attn tokens/s fwd+bwd on 1 MI355X", "value": value, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if wl["dtype"] == torch.bfloat16 else "f32", "data": "synthetic",
        "config": {"workload": f"{wl['name']}: block pair (regular 5^3 windows, then shifted by 2) of "
                               f"WindowAttentionSparse, dim {wl['dim']}, {wl['heads']} heads, forward+backward",
                   "voxels": wl["N"], "attention_calls_per_step": calls, **sizes},
        "roofline": roofline, "cpu_baseline": cpu,
    }
    if cpu:
        line["speedup_vs_cpu"] = value / cpu["value"]
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
