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

CALIBRATION_BYTES = 256 * 1024 * 1024      # size of the plain copy a profiling run launches beside the kernels
MFMA_PEAK_TFLOPS = {"f32": 157.3, "bf16": 2500.0, "f16": 2500.0}      # dense, MI355X
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")


def source_digest(rel_paths):
    """sha256 over the named source files: a traffic figure is valid for the sources it was measured on."""
    import hashlib
    h = hashlib.sha256()
    for rel in sorted(rel_paths):
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` on `workload` as rocprofv3 --pmc measured them (FETCH_SIZE, WRITE_SIZE,
    scaled by a calibration copy; written by --pmc-summary into profiles/traffic.json), or None with the
    reason: not measured, or measured on other kernel sources than the ones in the tree."""
    try:
        with open(TRAFFIC_JSON) as f:
            rec = json.load(f).get(workload, {}).get(kernel)
    except FileNotFoundError:
        rec = None
    if rec is None:
        return None, "not measured"
    if source_digest(rec["sources"]) != rec["digest"]:
        return None, f"stale: {', '.join(rec['sources'])} changed since {rec['summary']} was taken"
    return rec["bytes"], rec["summary"]


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# ------------------------------------------------------------------------------------------
def build_workload(device, name="cfg2"):
    from sparseswin3d_amd import synth
    from sparseswin3d_amd.window_attention import WindowAttentionSparse
    w = {"cfg1": synth.config1, "cfg2": synth.config2, "cfg3": synth.config3, "cfg4": synth.config4,
         "ref7": synth.config_ref7}[name]()
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
    from sparseswin3d_amd.window_attention import SparseVoxelTensor, prefetch_plans, replace_feature
    for blk in wl["blocks"]:                                  # as a training step does: fresh gradients
        blk["attn"].zero_grad(set_to_none=True)
    x = wl["feats"].detach().requires_grad_(True)
    # as a stage does: the token plans of all its blocks are enqueued before the first block runs (they need the
    # window indices only) and share their launches, so the totals of the later ones are on the host when their
    # block asks
    views = [SparseVoxelTensor(x, b["idx"], (b["n"],), b["slots"]) for b in wl["blocks"]]
    prefetch_plans([(b["attn"], t) for b, t in zip(wl["blocks"], views)])
    h = x
    for b, t in zip(wl["blocks"], views):
        h = b["attn"](replace_feature(t, h), b["mask"]).features
    h.backward(wl["upstream"])
    return x.grad


def build_encoder(device):
    """Configuration 5: four rooms in one batch, four attention stages (dims 96 / 192 / 384 / 768, heads of 32
    channels, windows 5^3 shifted by 2), bf16, forward only; floor(coord / 2) with mean pooling and channel doubling
    between the stages."""
    from sparseswin3d_amd import synth
    from sparseswin3d_amd.window_attention import WindowAttentionSparse
    w, _ = synth.config5_rooms()
    torch.manual_seed(5)
    stages = []
    for dim, heads in zip((96, 192, 384, 768), (3, 6, 12, 24)):
        attn = WindowAttentionSparse(dim, heads, (5, 5, 5), qkv_bias=True).to(device)
        torch.nn.init.xavier_uniform_(attn.qkv.weight)
        stages.append(attn.to(torch.bfloat16))
    return dict(name=w.name, dtype=torch.bfloat16, N=len(w.coords4), stages=stages, batch_size=w.batch_size,
                coords4=torch.from_numpy(w.coords4).to(device), spatial_shape=tuple(w.spatial_shape),
                feats=torch.randn(len(w.coords4), 96, device=device).to(torch.bfloat16))


def run_encoder(wl):
    """One forward pass of the four stages: per stage the window indices and the shift mask from the voxel grid
    kernels, the attention, then the stride-2 merge.  Returns the voxel count of every stage."""
    from sparseswin3d_amd import layers
    from sparseswin3d_amd.window_attention import SparseVoxelTensor, prefetch_plans
    ws, sh = (5, 5, 5), (2, 2, 2)
    coords, shape, feats = wl["coords4"], wl["spatial_shape"], wl["feats"]
    counts = []
    with torch.no_grad():
        for k, attn in enumerate(wl["stages"]):
            counts.append(coords.shape[0])
            dims = [-(-e // w_) * w_ for e, w_ in zip(shape, ws)]
            idx = layers.sparse_window_indices(coords, wl["batch_size"], dims, ws, sh)
            mask = layers.compute_mask(list(dims), list(ws), list(sh), coords.device)
            slots = wl["batch_size"] * (dims[0] // 5) * (dims[1] // 5) * (dims[2] // 5)
            view = SparseVoxelTensor(feats, idx, (125,), slots)
            last = k == len(wl["stages"]) - 1
            # as BasicLayer does: the plan of the attention and the plan of the merge behind it share their launches
            x = SparseVoxelTensor(feats, coords, shape, wl["batch_size"])
            merge_plan = prefetch_plans([(attn, view)], [] if last else [layers.downsample_plan_request(x, 2)])[1:]
            out = attn(view, mask).features
            if last:
                break
            plan, coords, shape = layers.downsample_plan(x, 2, merge_plan[0])
            pooled = layers._PoolWindows.apply(out, plan, True)
            feats = torch.cat([pooled, pooled], 1)
    return counts


def bench_encoder(device, args):
    """`--workload cfg5`: the forward pass of the four-stage encoder, timed as a whole."""
    from sparseswin3d_amd import _lib
    wl = build_encoder(device)
    counts = run_encoder(wl)
    log(f"workload {wl['name']}: voxels per stage {counts}")
    for _ in range(args.warmup):
        run_encoder(wl)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_encoder(wl)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    _lib.launch_timer, _lib.launch_timer_only = [], {"sswin_window_attention_forward"}
    for _ in range(5):
        run_encoder(wl)
    torch.cuda.synchronize()
    per_stage = [[] for _ in wl["stages"]]
    fw = [(a, b) for name, _, a, b in _lib.launch_timer if name == "sswin_window_attention_forward"]
    _lib.launch_timer = _lib.launch_timer_only = None
    for i, (a, b) in enumerate(fw):
        per_stage[i % len(per_stage)].append(a.elapsed_time(b))
    stage_ms = [sum(v) / len(v) for v in per_stage]
    log("attention forward launch per stage (HIP events inside the pass): " + ", ".join(f"{m:.4f} ms" for m in stage_ms))
    # the first stage's launch is the longest: q, k, v read and o written once (2 bytes each), lse written
    dims, heads = (96, 192, 384, 768), (3, 6, 12, 24)
    k = max(range(len(stage_ms)), key=lambda i: stage_ms[i])
    alg = 4 * 2 * counts[k] * dims[k] + 4 * heads[k] * counts[k]
    gbps = alg / stage_ms[k] / 1e6
    roofline = dict(bound="hbm", kernel=f"resident forward, stage {k + 1}", achieved=round(gbps, 1), peak=HBM_PEAK_GBPS,
                    unit="GB/s", frac=round(gbps / HBM_PEAK_GBPS, 4), traffic=None,
                    traffic_source="no counter run for this workload", algorithmic_bytes=alg, ms=round(stage_ms[k], 4),
                    timed="inside the pass", stage_forward_ms=[round(m, 4) for m in stage_ms])
    line = {
        "metric": "window-attn tokens/s fwd+bwd on 1 MI355X", "value": sum(counts) / dt, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{wl['name']}: four rooms in one batch, four attention stages (dims 96/192/384/768, "
                               "heads of 32 channels, windows 5^3 shifted by 2) with stride-2 merges in between, "
                               "FORWARD ONLY as the configuration says; value = attention tokens of all stages per second",
                   "voxels_per_stage": counts},
        "roofline": roofline, "cpu_baseline": None,
    }
    print(json.dumps(line), flush=True)


# ------------------------------------------------------------------------------------------
_QUEUE_FILL = []


def event_time_ms(fn, reps, warmup=2, queue_ahead=False):
    """Mean GPU time of `fn` between two HIP events over `reps` calls.  `queue_ahead`: about a millisecond of plain
    copies is enqueued in front of the first event, so the host has all `reps` calls in the queue before the GPU
    reaches them; without it a call shorter than its own enqueue cost (about 20 us from Python) is timed at that
    cost."""
    for _ in range(warmup):
        fn()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    if queue_ahead:
        if not _QUEUE_FILL:
            _QUEUE_FILL.extend(torch.empty(CALIBRATION_BYTES // 4, dtype=torch.int32, device="cuda") for _ in range(2))
        for _ in range(max(2, reps * 2 // 5)):                # 0.1 ms each: 40 us per call to come
            _QUEUE_FILL[1].copy_(_QUEUE_FILL[0])
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / reps


DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}

# table name of a kernel -> (substring of its symbol in a rocprofv3 trace, source files it is built from)
KERNEL_SYMBOLS = {
    # fp32 tokens run the kernels of window_attention.hip (wattn_*), 16-bit tokens those of window_attention_x16.hip (wattn16_*)
    "resident forward": ("_fwd_kernel", ["sparseswin3d_amd/csrc/window_attention.hip", "sparseswin3d_amd/csrc/window_attention_x16.hip",
                                         "sparseswin3d_amd/csrc/wattn_common.hpp"]),
    "resident backward (dQ,dK,dV,dS)": ("_bwd_all_kernel", ["sparseswin3d_amd/csrc/window_attention.hip",
                                                            "sparseswin3d_amd/csrc/window_attention_x16.hip",
                                                            "sparseswin3d_amd/csrc/wattn_common.hpp"]),
    "block_matmul q_k, values": ("block_product_mfma_kernel<float, 0", ["sparseswin3d_amd/csrc/block_matmul.hip", "sparseswin3d_amd/csrc/mfma_block.hpp"]),
    "block_matmul qk_v, values": ("block_product_mfma_kernel<float, 1, false", ["sparseswin3d_amd/csrc/block_matmul.hip", "sparseswin3d_amd/csrc/mfma_block.hpp"]),
    "block_matmul qk_v (values + index matrix)": ("block_product_mfma_kernel<float, 1, true", ["sparseswin3d_amd/csrc/block_matmul.hip", "sparseswin3d_amd/csrc/mfma_block.hpp"]),
    "grad rc_cr": ("block_product_mfma_kernel<float, 2", ["sparseswin3d_amd/csrc/block_matmul.hip", "sparseswin3d_amd/csrc/mfma_block.hpp"]),
    "grad rr_rc": ("block_product_mfma_kernel<float, 3", ["sparseswin3d_amd/csrc/block_matmul.hip", "sparseswin3d_amd/csrc/mfma_block.hpp"]),
    "grad cr_rr": ("block_product_mfma_kernel<float, 4", ["sparseswin3d_amd/csrc/block_matmul.hip", "sparseswin3d_amd/csrc/mfma_block.hpp"]),
    "grad tr_rc (dV = P^T dO)": ("block_product_mfma_kernel<float, 5", ["sparseswin3d_amd/csrc/block_matmul.hip", "sparseswin3d_amd/csrc/mfma_block.hpp"]),
    "grad tc_rr (dK^T = Q^T dS)": ("block_product_mfma_kernel<float, 6", ["sparseswin3d_amd/csrc/block_matmul.hip", "sparseswin3d_amd/csrc/mfma_block.hpp"]),
    "operand_copy_qkv": ("qkv_order_copy_kernel", ["sparseswin3d_amd/csrc/index_ops.hip"]),
    "bias + mask add, one pass [A]": ("group_bias_mask_kernel", ["sparseswin3d_amd/csrc/softmax.hip"]),
    "transpose rc": ("block_transpose_kernel<float, false", ["sparseswin3d_amd/csrc/block_matmul.hip"]),
    "transpose rr": ("block_transpose_kernel<float, true", ["sparseswin3d_amd/csrc/block_matmul.hip"]),
    "softmax_last_dim_forward": ("softmax_rows_kernel<float, false", ["sparseswin3d_amd/csrc/softmax.hip"]),
    "softmax_last_dim_backward": ("softmax_rows_kernel<float, true", ["sparseswin3d_amd/csrc/softmax.hip"]),
    "resident bias table grad": ("rpb_table_partial_kernel", ["sparseswin3d_amd/csrc/fused_attention.hip"]),
    "fused S=QK^T+bias+mask": ("fused_sq_kernel<float, 1", ["sparseswin3d_amd/csrc/fused_attention.hip", "sparseswin3d_amd/csrc/mfma_block.hpp"]),
    "fused dS=P(dO V^T - dO.O)": ("fused_sq_kernel<float, 2", ["sparseswin3d_amd/csrc/fused_attention.hip", "sparseswin3d_amd/csrc/mfma_block.hpp"]),
    "fused dV=P^T dO": ("fused_tok_kernel<float, true", ["sparseswin3d_amd/csrc/fused_attention.hip", "sparseswin3d_amd/csrc/mfma_block.hpp"]),
    "fused O=PV": ("fused_tok_kernel<float, false", ["sparseswin3d_amd/csrc/fused_attention.hip", "sparseswin3d_amd/csrc/mfma_block.hpp"]),
    "fused softmax fwd (rows from the group table)": ("group_softmax_kernel<false", ["sparseswin3d_amd/csrc/fused_attention.hip"]),
}


# operator-path table row -> (library entry point, leading integer arguments or None for any) of the launch it times
OPERATOR_LAUNCHES = {
    "token plan, one of a stage's two (operand map + group table)": ("sswin_token_plan", None),
    "sorted_coo_indices [4,E], Q/V": ("sswin_sorted_coo_indices", None),
    "operand_copy_qkv, voxel rows -> Q*scale, K^T, V": ("sswin_operand_copy_qkv", (0, 1)),
    "operand_copy_qkv, gradients -> voxel rows": ("sswin_operand_copy_qkv", (0, 0)),
    "operand_copy Q/V order, operand -> voxel rows": ("sswin_operand_copy", (0, 0, 0)),
    "operand_copy Q/V order, voxel rows -> operand": ("sswin_operand_copy", (0, 0, 1)),
    "block_matmul q_k, values": ("sswin_block_matmul", (0, 0)),
    "bias + mask add, one pass [A]": ("sswin_group_add_table_bias_mask", None),
    "bias table gradient (batches from the token plan)": ("sswin_bias_table_grad_tasks", None),
    "bias table gradient from the product's groups": ("sswin_bias_table_grad", None),
    "softmax rows from the group sizes [A]": ("sswin_softmax_rows_from_counts", None),
    "softmax_last_dim_forward": ("sswin_softmax_last_dim_forward", None),
    "block_matmul qk_v, values": ("sswin_block_matmul", (1, 0)),
    "softmax_last_dim_backward": ("sswin_softmax_last_dim_backward", None),
    "grad rc_cr": ("sswin_block_matmul_grad", (0, 0)),
    "grad rr_rc": ("sswin_block_matmul_grad", (1, 0)),
    "grad tr_rc (dV = P^T dO)": ("sswin_block_matmul_grad", (3, 0)),
    "grad tc_rr (dK^T = Q^T dS)": ("sswin_block_matmul_grad", (4, 0)),
}


def operators_in_module(wl, reps=5):
    """Every library launch of one attention module call (forward + backward, regular windows) on the operator path,
    timed where it runs: HIP events around each launch on its stream.  Returns {(entry point, leading integer
    arguments): (mean ms, launches per call)}."""
    from sparseswin3d_amd import _lib
    from sparseswin3d_amd.window_attention import SparseVoxelTensor
    b = wl["blocks"][0]
    attn = b["attn"]
    keep = (attn.fused, attn.resident)
    attn.fused, attn.resident = False, None

    def once():
        attn.zero_grad(set_to_none=True)
        x = wl["feats"].detach().requires_grad_(True)
        attn(SparseVoxelTensor(x, b["idx"], (b["n"],), b["slots"]), None).features.backward(wl["upstream"])

    for _ in range(3):
        once()
    torch.cuda.synchronize()
    _lib.launch_timer = []
    for _ in range(reps):
        once()
    torch.cuda.synchronize()
    acc = {}
    for name, ints, start, stop in _lib.launch_timer:
        acc.setdefault((name, ints), []).append(start.elapsed_time(stop))
    _lib.launch_timer = None
    attn.fused, attn.resident = keep
    return {k: (sum(v) / len(v), len(v) / reps) for k, v in acc.items()}


def kernel_table(wl, reps=20, only=None):
    """Time every operator's kernels alone on the first block's tensors (regular windows).  The operator
    and fused paths are timed for fp32 tokens only; the window-resident kernels in the workload's dtype."""
    from sparseswin3d_amd import _lib, custom_ops as ops, fused as F
    from sparseswin3d_amd.window_attention import qkv_sparse_cuda, relative_position_index_3d
    lib = _lib.load()
    b = wl["blocks"][0]
    H, D = wl["heads"], wl["dim"]
    hd = D // H
    N = wl["N"]
    dev = wl["feats"].device
    tdt = wl["dtype"]
    code = DTYPE_CODE[tdt]
    es = 2 if code else 4                                    # bytes per token value
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ptr = lambda t: C.c_void_p(t.data_ptr() if t is not None else 0)
    mask = wl["blocks"][1]["mask"]
    qkv = torch.randn(N, 3, H, hd, device=dev)
    tp = F.TokenPlan(b["idx"], b["slots"], b["n"], H)
    E, A, G = N * D, int(tp.A), int(tp.G)

    def staged_plan():
        # the plans of the regular and the shifted partition in one set of launches, totals not waited for
        F.TokenPlan.batch([(bb["idx"], bb["slots"], bb["n"], H) for bb in wl["blocks"][:2]])
    staged_plan.per_call_share = 1.0 / len(wl["blocks"][:2])
    sizes = dict(N=N, E=E, A=A, G=G, c_max=int(tp.c_max) if hasattr(tp, "c_max") else None)
    entries, f_entries = [], []

    if code == 0:
        q, kt, v = qkv_sparse_cuda(qkv, b["idx"], b["slots"], b["n"])
        s_idx, s_val, s_shape, c = ops.matmul_cuda_naive(q.values, q.indices, q.shape, kt.values, kt.indices, kt.shape, "q_k")
        flat = ops.flatten_indices(s_idx[:3], s_shape[:3])
        rows = ops.unique_consecutive_indices(flat)
        p_val = ops.softmax_last_dim_forward(rows, s_val)
        o_idx, o_val, o_shape, c2 = ops.matmul_cuda_naive(p_val, s_idx, s_shape, v.values, v.indices, v.shape, "qk_v")
        assert (E, A, G) == (q.values.numel(), s_val.numel(), c.numel())
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
        sizes["c_max"] = c_max
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
                                                                  E, ptr(out), stream))

        def tr(kind, a, out):
            return lambda: _lib.check(lib.sswin_block_transpose(kind, 0, ptr(a), ptr(cc), ptr(scans), G, hd, ptr(out), stream))

        tmp_e, tmp_a = torch.empty(E, device=dev), torch.empty(A, device=dev)
        idxT = b["idx"].T.contiguous()
        flat_tok = ops.flatten_indices(idxT, [b["slots"], b["n"]])
        perm_idx = o_idx[[0, 2, 1, 3], :].contiguous()
        flat_perm = ops.flatten_indices(perm_idx, [o_shape[0], o_shape[2], o_shape[1], o_shape[3]])

        # operands straight from the voxel ranks (what qkv_sparse_cuda and the module's tail run)
        omap = ops.operand_map(b["idx"], b["slots"], b["n"])
        feat_rows = torch.randn(N, D, device=dev)
        qkv_rows = qkv.view(N, 3 * D)
        val_e, val_e2, val_e3 = (torch.empty(E, device=dev) for _ in range(3))
        qkv_rows_out = torch.empty_like(qkv_rows)

        gp = ops.group_plan(c)
        row_pos = ops.group_row_positions(s_idx, gp)
        bias_d = torch.randn(H, b["n"], b["n"], device=dev)
        n_table_o = int(wl["blocks"][0]["attn"].relative_position_bias_table.shape[0])
        table_o = wl["blocks"][0]["attn"].relative_position_bias_table.detach().float().contiguous()
        ti_o = F.BiasTableIndex.build(relative_position_index_3d(wl["blocks"][0]["attn"].window_size).to(dev), n_table_o)
        dealt_o = tp.tasks is not None and b["n"] <= 128 and sum(tp.bucket_counts) == tp.G   # every window has a task descriptor

        entries = [
            # name, callable, algorithmic bytes, calls per attention fwd+bwd of the module (0: not on the module's path)
            # the module takes the operand map and the products' group table from one token plan
            ("token plan, one of a stage's two (operand map + group table)", staged_plan, 28 * N + 20 * G, 1),
            ("token_plan built and waited for on its own", lambda: F.TokenPlan(b["idx"], b["slots"], b["n"], H, tasks=False), 28 * N + 20 * G, 0),
            ("operand_map [N] (on its own)", lambda: ops.operand_map(b["idx"], b["slots"], b["n"]), 20 * N, 0),
            # the module asks for the Q/V matrix only; K^T's and the products' index matrices are written when somebody
            # reads them (rows with 0 calls below: what the reference's operators always write)
            ("sorted_coo_indices [4,E], Q/V", lambda: ops.sorted_coo_indices(b["idx"], omap, H, hd, k=False), 16 * E + 20 * N, 1),
            ("sorted_coo_indices [4,E] x 2 (with K^T's)", lambda: ops.sorted_coo_indices(b["idx"], omap, H, hd), 32 * E + 20 * N, 0),
            # the module copies Q (times the attention scale), K^T and V in one launch each way, and the attention output
            # to voxel rows (and its gradient back) with one Q/V-order copy each
            ("operand_copy_qkv, voxel rows -> Q*scale, K^T, V", lambda: ops.operand_copy_qkv(qkv_rows, val_e, val_e2, val_e3, omap, H, hd, True, 0.17), 6 * s * E, 1),
            ("operand_copy_qkv, gradients -> voxel rows", lambda: ops.operand_copy_qkv(qkv_rows_out, val_e, val_e2, val_e3, omap, H, hd, False, 0.17), 6 * s * E, 1),
            ("operand_copy Q/V order, operand -> voxel rows", lambda: ops.operand_copy(feat_rows, 0, val_e, omap, H, hd, 0, False), 2 * s * E, 1),
            ("operand_copy Q/V order, voxel rows -> operand", lambda: ops.operand_copy(qkv_rows, 2 * D, val_e, omap, H, hd, 0, True), 2 * s * E, 1),
            ("operand_copy K^T order", lambda: ops.operand_copy(qkv_rows, D, val_e, omap, H, hd, 1, True), 2 * s * E, 0),
            ("qkv_sparse_indices (reference operator)", lambda: ops.qkv_sparse_indices(b["idx"], b["slots"], b["n"], H, hd), 8 * N + 40 * E, 0),
            ("plan_from_indices (group table from a [4,E] index matrix)", lambda: _lib.check(lib.sswin_plan_from_indices(ptr(q.indices), m, hd, ptr(plan), g_cap, totals, ptr(ws), nb, stream)), 0, 0),
            ("block_matmul q_k, values", mm(0, q.values, kt.values, q.indices, out_s, None, A), 2 * s * E + s * A + 4 * G, 1),
            ("block_matmul q_k (values + index matrix)", mm(0, q.values, kt.values, q.indices, out_s, out_si, A), 2 * s * E + (s + 16) * A + 4 * G, 0),
            ("bias + mask add, one pass [A]", lambda: ops.group_add_table_bias_mask(s_val, row_pos, gp, b["n"], table_o, ti_o.code, ti_o.offset0, mask), 2 * s * A + 8 * G, 1),
            ("bias + mask add from a gathered [H,n,n] bias", lambda: ops.group_add_bias_mask(s_val, row_pos, gp, b["n"], bias_d, mask), 2 * s * A + 8 * G, 0),
            # what the module's backward calls: with a token plan at hand the batches are dealt from its descriptors
            ("bias table gradient (batches from the token plan)", lambda: F._bias_gradient(tp, H, g_s, (torch.float32, (n_table_o, H)), ti_o), 4 * A, int(dealt_o)),
            ("bias table gradient from the product's groups", lambda: ops.group_bias_table_grad(g_s, row_pos, gp, H, b["n"], ti_o.code, ti_o.offset0, n_table_o), 4 * A, int(not dealt_o)),
            ("softmax rows from the group sizes [A]", lambda: ops.softmax_rows_from_counts(c, A), 4 * A + 12 * G, 1),
            ("flatten_indices [3,A] (generic softmax rows)", lambda: ops.flatten_indices(s_idx[:3], s_shape[:3]), 16 * A, 0),
            ("unique_consecutive_indices [A] (generic softmax rows)", lambda: ops.unique_consecutive_indices(flat), 8 * A, 0),
            ("softmax_last_dim_forward", lambda: ops.softmax_last_dim_forward(rows, s_val), 12 * A, 1),
            ("block_matmul qk_v, values", mm(1, p_val, v.values, v.indices, out_o, None, E), s * A + 2 * s * E + 4 * G, 1),
            ("block_matmul qk_v (values + index matrix)", mm(1, p_val, v.values, v.indices, out_o, out_oi, E), s * A + s * E + (s + 16) * E + 4 * G, 0),
            ("permute order from the group structure [E]", lambda: ops.permute_heads_order(o_idx, o_shape), 0, 0),
            ("flatten_indices [4,E] (generic permute)", lambda: ops.flatten_indices(perm_idx, [o_shape[0], o_shape[2], o_shape[1], o_shape[3]]), 0, 0),
            ("sort_indices [E] (generic permute)", lambda: ops.sort_indices(flat_perm), 0, 0),
            ("return_inverse [N]", lambda: ops.return_inverse(flat_tok, b["slots"] * b["n"]), 0, 0),
            ("softmax_last_dim_backward", lambda: ops.softmax_last_dim_backward(rows, p_val, g_s), 16 * A, 1),
            ("grad rc_cr", grad(0, g_o, v.values, tmp_a), 2 * s * E + s * A, 1),
            ("grad rr_rc", grad(1, g_s, kt.values, tmp_e), s * A + 2 * s * E, 1),
            # the second gradient of each product reads the operands as the forward pass left them; the reference's
            # composition (two transposed copies, then cr_rr / rr_rc) is what the rows with 0 calls time
            ("grad tr_rc (dV = P^T dO)", grad(3, p_val, g_o, tmp_e), s * A + 2 * s * E, 1),
            ("grad tc_rr (dK^T = Q^T dS)", grad(4, q.values, g_s, tmp_e), s * A + 2 * s * E, 1),
            ("grad cr_rr", grad(2, q.values, g_s, tmp_e), s * A + 2 * s * E, 0),
            ("transpose rc", tr(0, q.values, tmp_e), 2 * s * E, 0),
            ("transpose rr", tr(1, g_s, tmp_a), 2 * s * A, 0),
        ]
        # ---- the fused path (S and P in memory; what the module runs for heads that are not 32 wide) ----
        qkv_c = qkv.contiguous()
        bias = torch.randn(H, b["n"], b["n"], device=dev)
        s_f = torch.empty(tp.A, device=dev)
        p_f = torch.empty(tp.A, device=dev)
        out_f = torch.empty(N, D, device=dev)
        dqkv = torch.empty_like(qkv_c)
        dbias = torch.zeros(H, b["n"], b["n"], device=dev)
        dt = torch.float32
        bg_bytes = lib.sswin_fused_bias_grad_workspace_bytes(tp.G, H, b["n"])
        bg_ws = torch.empty(int(bg_bytes), dtype=torch.uint8, device=dev)
        f_entries = [
            ("fused token plan, one of a stage's two", staged_plan, 28 * N + 20 * tp.G, 1),
            ("fused S=QK^T+bias+mask", lambda: F._tokens_to_sq(tp, dt, True, qkv_c, 3 * D, 0, qkv_c, 3 * D, D, hd, 0.17, bias, mask, s_f, None), 8 * E + 4 * A, 1),
            ("fused softmax fwd (rows from the group table)", lambda: F._group_softmax(tp, False, s_f, None, p_f), 8 * A, 1),
            ("fused O=PV", lambda: F._sq_to_tokens(tp, dt, False, p_val, qkv_c, 3 * D, 2 * D, out_f, D, 0, hd, 1.0), 4 * A + 8 * E, 1),
            ("fused dS=P(dO V^T - dO.O)", lambda: F._score_grad(tp, dt, out_f, D, 0, qkv_c, 3 * D, 2 * D, out_f, D, 0, hd, p_val, s_f), 12 * E + 8 * A, 1),
            ("fused dP=dO V^T (the product alone)", lambda: F._tokens_to_sq(tp, dt, False, out_f, D, 0, qkv_c, 3 * D, 2 * D, hd, 1.0, None, None, s_f, None), 8 * E + 4 * A, 0),
            ("fused dV=P^T dO", lambda: F._sq_to_tokens(tp, dt, True, p_val, out_f, D, 0, dqkv, 3 * D, 2 * D, hd, 1.0), 4 * A + 8 * E, 1),
            ("fused softmax bwd (rows from the group table; alone)", lambda: F._group_softmax(tp, True, p_val, g_s, p_f), 12 * A, 0),
            ("fused dQ=dS K", lambda: F._sq_to_tokens(tp, dt, False, g_s, qkv_c, 3 * D, D, dqkv, 3 * D, 0, hd, 0.17), 4 * A + 8 * E, 1),
            ("fused dK=dS^T Q", lambda: F._sq_to_tokens(tp, dt, True, g_s, qkv_c, 3 * D, 0, dqkv, 3 * D, D, hd, 0.17), 4 * A + 8 * E, 1),
            ("fused bias table grad", lambda: F._bias_gradient(tp, H, g_s, (torch.float32, (n_table, H)), ti), 4 * A, 1),
            ("fused bias grad [H,n,n]", lambda: _lib.check(lib.sswin_fused_bias_grad(ptr(tp.plan), tp.g_cap, tp.G, ptr(tp.tokens), tp.N, H, b["n"], ptr(g_s), ptr(dbias), ptr(bg_ws), bg_bytes, stream)), 4 * A, 0),
        ]

        if b["n"] > 128:                                    # the dense-bias gradient takes windows of at most 128 positions
            f_entries = [e for e in f_entries if e[0] != "fused bias grad [H,n,n]"]

    # ---- the window-resident kernels (what the step runs for heads of 32 channels), in the workload's dtype ----
    qkv_r = qkv.reshape(N, 3 * D).to(tdt).contiguous()
    bias_r = torch.randn(H, b["n"], b["n"], device=dev)
    out_r = torch.empty(N, D, device=dev, dtype=tdt)
    dqkv_r = torch.empty_like(qkv_r)
    ds_r = torch.empty(A, device=dev)
    lse = torch.empty(H * N, device=dev)
    mask_p, nmw = ptr(mask), (0 if mask is None else mask.shape[0])
    qa = (ptr(qkv_r), 3 * D, 0, ptr(qkv_r), 3 * D, D, ptr(qkv_r), 3 * D, 2 * D)
    da = (ptr(dqkv_r), 3 * D, 0, ptr(dqkv_r), 3 * D, D, ptr(dqkv_r), 3 * D, 2 * D)
    up_r = torch.randn(N, D, device=dev).to(tdt)
    Er = es * E // 4                                         # E in units of four bytes of token values

    def r_fwd():
        _lib.check(lib.sswin_window_attention_forward(code, ptr(tp.tasks), tp.g_cap, tp.bucket_counts, ptr(tp.tokens), N, H,
                                                      hd, *qa, C.c_float(0.17), ptr(bias_r), b["n"], mask_p, nmw,
                                                      ptr(out_r), D, 0, ptr(lse), stream))

    # The step asks for all gradients at once (sides = 3): one launch in which groups of at most
    # 64 tokens get dQ from their key-side tasks and only the larger groups have query-side tasks.
    # The parts are timed alone for comparison: restricted bucket counts = the query-side kernel on
    # the groups of more than 32 tokens, 1 / 2 = the per-side kernels.
    bc = [int(x) for x in tp.bucket_counts]
    cg = tp.plan[:tp.G].to(torch.int64)                                  # plan row 0: tokens of each group
    rowsL = int(cg[cg > 32].sum())                                       # token-head rows of the large groups
    only_large = [0, bc[1], bc[2], bc[3]]

    def r_bwd(sides, counts=None):
        counts = tp.bucket_counts if counts is None else (C.c_int64 * 4)(*counts)
        return lambda: _lib.check(lib.sswin_window_attention_backward(
            code, ptr(tp.tasks), tp.g_cap, counts, ptr(tp.tokens), N, H, hd, *qa, C.c_float(0.17), ptr(bias_r),
            b["n"], mask_p, nmw, ptr(out_r), D, 0, ptr(up_r), D, 0, ptr(lse), *da, ptr(ds_r), sides, stream))

    n_table = int(wl["blocks"][0]["attn"].relative_position_bias_table.shape[0])
    ti = F.BiasTableIndex.build(relative_position_index_3d(wl["blocks"][0]["attn"].window_size).to(dev), n_table)
    d_table = torch.empty(n_table, H, device=dev)
    tg_bytes = lib.sswin_bias_table_grad_workspace_bytes(tp.G, H, n_table)
    tg_ws = torch.empty(int(tg_bytes), dtype=torch.uint8, device=dev)

    def r_table_grad_groups():
        _lib.check(lib.sswin_bias_table_grad(ptr(tp.plan), tp.g_cap, tp.G, ptr(tp.tokens), tp.N, H, b["n"], ptr(ti.code),
                                             ti.offset0, n_table, ptr(ds_r), ptr(d_table), ptr(tg_ws), tg_bytes, stream))

    # what the module calls when every window holds at most 128 tokens: the batches dealt from the task descriptors
    by_tasks = tp.tasks is not None and b["n"] <= 128 and sum(tp.bucket_counts) == tp.G

    def r_table_grad():
        if not by_tasks:
            return r_table_grad_groups()
        _lib.check(lib.sswin_bias_table_grad_tasks(ptr(tp.tasks), tp.g_cap, tp.bucket_counts, tp.G, ptr(tp.tokens), tp.N, H, b["n"],
                                                   ptr(ti.code), ti.offset0, n_table, ptr(ds_r), ptr(d_table), ptr(tg_ws), tg_bytes,
                                                   stream))

    resident_ok = hd == 32 and int(tp.c_max) <= 128       # otherwise the module runs the fused path
    if resident_ok:
        r_fwd()                                   # lse and out_r must hold a real forward for the backward timings
    # flops of a launch: 2 c^2 hd per product and group = 2 A hd per product (two in the forward, five in the backward)
    r_entries = [
        # what a stage (and the step) does: the plans of its two partitions from shared launches, nobody waiting for
        # the totals; the row is half the GPU time of the two plans
        ("resident token plan, one of a stage's two", staged_plan, 28 * N + 36 * tp.G, 1),
        ("token_plan built and waited for on its own", lambda: F.TokenPlan(b["idx"], b["slots"], b["n"], H), 28 * N + 36 * tp.G, 0),
        ("resident forward", r_fwd, 16 * Er + 4 * H * N, 1, 4 * A * hd),
        ("resident backward (dQ,dK,dV,dS)", r_bwd(3), 32 * Er + 4 * A + 4 * H * N, 1, 10 * A * hd),
        ("resident backward dQ, groups > 32 tokens", r_bwd(1, only_large), (24 * es // 4 * hd + 4) * rowsL, 0),
        ("resident backward dQ, all groups", r_bwd(1), 24 * Er + 4 * H * N, 0),
        ("resident backward dK,dV,dS only", r_bwd(2), 28 * Er + 4 * A + 4 * H * N, 0),
        ("resident bias table grad", r_table_grad, 4 * A, 1),
        ("bias table grad, batches from the group table", r_table_grad_groups, 4 * A, 0),
    ]
    if code == 0:
        r_entries.append(("resident bias grad [H,n,n]", lambda: _lib.check(lib.sswin_fused_bias_grad(
            ptr(tp.plan), tp.g_cap, tp.G, ptr(tp.tokens), tp.N, H, b["n"], ptr(ds_r), ptr(dbias), ptr(bg_ws), bg_bytes, stream)), 4 * A, 0))
    if not resident_ok:
        r_entries = r_entries[:2]

    def measure(items, path):
        rows_ = []
        for name, fn, nbytes, calls, *flops in items:
            ms = event_time_ms(fn, reps, queue_ahead=True) * getattr(fn, "per_call_share", 1.0)
            gbps = nbytes / ms / 1e6 if nbytes else None
            rows_.append(dict(kernel=name, path=path, ms=ms, algorithmic_bytes=nbytes, calls=calls,
                              achieved_gbps=gbps, frac=(gbps / HBM_PEAK_GBPS) if gbps else None,
                              flops=flops[0] if flops else None))
        return rows_

    if only is not None:
        # profiling mode: run the named kernels (substring match) `reps` times each, plus a plain
        # device-to-device copy of known size that calibrates the FETCH_SIZE / WRITE_SIZE counters
        src = torch.empty(CALIBRATION_BYTES // 4, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        names = [o for o in only.split(",") if o]
        picked = [e for e in r_entries + f_entries + entries + (projection_entries(wl) if code == 0 else [])
                  if any(o in e[0] for o in names)]
        for name, fn, nbytes, calls, *_ in picked:
            log(f"profiling {name}: {reps} launches, algorithmic bytes {nbytes}")
            for _ in range(reps):
                fn()
        for _ in range(reps):
            _lib.check(lib.sswin_calibration_copy(ptr(dst), ptr(src), CALIBRATION_BYTES, stream))
        torch.cuda.synchronize()
        log(f"calibration copy: {reps} launches of {CALIBRATION_BYTES} bytes read and written")
        return [], sizes
    table = measure(r_entries, "resident")
    if code == 0:
        op_rows = measure(entries, "operators")
        # the same launches inside a module call: what the path's summary is made of
        timed = operators_in_module(wl)
        seen = set()
        for row in op_rows:
            fn, ints = OPERATOR_LAUNCHES.get(row["kernel"], (None, None))
            hits = [(k, v) for k, v in timed.items() if k[0] == fn and (ints is None or k[1] == ints)]
            if hits and row["calls"]:
                seen.update(k for k, _ in hits)
                launches = sum(v[1] for _, v in hits)
                row["ms_in_module"] = sum(v[0] * v[1] for _, v in hits) / launches
                row["calls"] = int(round(launches))
        stray = {k: v for k, v in timed.items() if k not in seen and "tall_linear" not in k[0] and "column_sum" not in k[0]}
        for (fn, ints), (ms, launches) in stray.items():        # a launch of the call that no table row stands for
            op_rows.append(dict(kernel=f"{fn}{ints} (in the module call only)", path="operators", ms=ms, ms_in_module=ms,
                                algorithmic_bytes=0, calls=int(round(launches)), achieved_gbps=None, frac=None, flops=None))
        table += measure(f_entries, "fused") + op_rows
        table += measure(stage_entries(wl), "stage")
        table += measure(projection_entries(wl), "projections")
    return table, sizes


def module_times(wl, reps=10):
    """One attention module call, forward + backward (projections and torch glue included), on each of the
    three paths: HIP events around the whole call, regular windows."""
    from sparseswin3d_amd.window_attention import SparseVoxelTensor
    if wl["dtype"] != torch.float32:
        return {}
    b = wl["blocks"][0]
    attn = b["attn"]
    keep = (attn.fused, attn.resident)

    def once():
        attn.zero_grad(set_to_none=True)
        x = wl["feats"].detach().requires_grad_(True)
        out = attn(SparseVoxelTensor(x, b["idx"], (b["n"],), b["slots"]), None).features
        out.backward(wl["upstream"])

    out = {}
    hd = wl["dim"] // wl["heads"]
    for name, fused_, resident in (("resident", True, True), ("fused", True, False), ("operators", False, None)):
        if name == "resident" and (hd != 32 or b["stats"]["c_max"] > 128):
            continue                                          # the resident kernels do not take this shape
        attn.fused, attn.resident = fused_, resident
        out[name] = round(event_time_ms(once, reps), 4)
    attn.fused, attn.resident = keep
    return out


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

    def fresh_mask():
        layers._MASKS.clear()
        return layers.compute_mask(list(pd), list(ws), list(sh), c4.device)

    return [
        ("stage window indices (pad+roll+partition)", lambda: layers.sparse_window_indices(c4, wl["batch_size"], pd, ws, sh), 24 * N, 1),
        ("stage shift mask (first pass of a stage; kept per shape afterwards)", fresh_mask, windows * n, 1),
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
        # what the module runs: this library's kernels where they take the shape (calls = 1), else the library GEMM
        own_f = wa._split_linear_forward(x, w, b) is not None
        own_w = wa._split_linear_weight_grad(dy, x, True)[0] is not None
        own_x = wa._split_linear_input_grad(dy, w) is not None
        if own_f:
            entries.append((f"{name} forward", (lambda w=w, b=b: wa._split_linear_forward(x, w, b)), io + 4 * P * D, 1))
        if own_w:
            entries.append((f"{name} weight+bias gradient", (lambda dy=dy: wa._split_linear_weight_grad(dy, x, True)), io + 4 * P * D, 1))
        def lib_dx(dy=dy, w=w):
            with wa._rocblas_gemm():
                return dy @ w

        if own_x:
            entries.append((f"{name} input gradient", (lambda dy=dy, w=w: wa._split_linear_input_grad(dy, w)), io + 4 * P * D, 1))

        def lib_fwd(w=w, b=b):
            with wa._rocblas_gemm():
                return torch.nn.functional.linear(x, w, b)

        def lib_wgrad(dy=dy):
            with wa._rocblas_gemm():
                return dy.t() @ x, wa._column_sum(dy)

        entries += [(f"{name} forward, library GEMM", lib_fwd, io + 4 * P * D, 0 if own_f else 1),
                    (f"{name} weight+bias gradient, library GEMM + column sums", lib_wgrad, io + 4 * P * D, 0 if own_w else 1)]
        entries.append((f"{name} input gradient, library GEMM", lib_dx, io + 4 * P * D, 0 if own_x else 1))
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
def pmc_summary(dirs, out_name, workload, command, only=None):
    """Turn the csv output of rocprofv3 --pmc runs of ``bench.py --profile-kernel`` (one run per counter set,
    each written with ``--output-format csv -d DIR``) into a text summary ``profiles/<out_name>.txt`` and
    into ``profiles/traffic.json`` (HBM bytes per launch of every kernel of KERNEL_SYMBOLS found in the runs).
    FETCH_SIZE and WRITE_SIZE are scaled by what they read for the calibration copy of CALIBRATION_BYTES."""
    import collections
    import csv
    import glob
    acc = collections.defaultdict(list)
    for d in dirs:
        for path in glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True):
            for r in csv.DictReader(open(path)):
                acc[(r["Kernel_Name"], r["Counter_Name"])].append(float(r["Counter_Value"]))
    if not acc:
        sys.exit(f"no *counter_collection.csv under {dirs}")
    mean = {k: sum(v) / len(v) for k, v in acc.items()}
    kernels = sorted({k for k, _ in mean if k.startswith(("void sswin::", "sswin::"))})
    cal = next((k for k in kernels if "calibration_copy_kernel" in k), None)
    wanted = only or [sym for sym, _ in KERNEL_SYMBOLS.values()]
    kernels = [k for k in kernels if k == cal or any(w in k for w in wanted)]
    unit = {}
    if cal:
        for cname in ("FETCH_SIZE", "WRITE_SIZE"):
            if (cal, cname) in mean:
                unit[cname] = CALIBRATION_BYTES / mean[(cal, cname)]
    lines = [f"rocprofv3 --pmc counters, workload {workload}, means per dispatch over the launches of each run.",
             "Commands (one rocprofv3 run per counter set; --pmc cannot split a set over passes):"]
    lines += [f"  {c}" for c in command]
    lines.append(f"Calibration: sswin::calibration_copy_kernel copies {CALIBRATION_BYTES} bytes (read once, written once): " +
                 ", ".join(f"{c} reads {mean[(cal, c)]:.1f} -> {unit[c]:.1f} bytes per count" for c in unit))
    lines.append("")
    try:
        with open(TRAFFIC_JSON) as f:
            traffic = json.load(f)
    except FileNotFoundError:
        traffic = {}
    for k in kernels:
        if k == cal:
            continue
        cs = {c: v for (kk, c), v in mean.items() if kk == k}
        lines.append(k if len(k) < 110 else k[:110] + " ...")
        nb = None
        if "FETCH_SIZE" in cs and "WRITE_SIZE" in cs and len(unit) == 2:
            rd, wr = cs["FETCH_SIZE"] * unit["FETCH_SIZE"], cs["WRITE_SIZE"] * unit["WRITE_SIZE"]
            nb = rd + wr
            lines.append(f"    HBM traffic per launch: read {rd / 1e6:.1f} MB + written {wr / 1e6:.1f} MB = {nb / 1e6:.1f} MB")
        raw = [f"{c}={cs[c]:.0f}" for c in sorted(cs)]
        for i in range(0, len(raw), 5):                         # the counters themselves, five to a line
            lines.append("    " + "  ".join(raw[i:i + 5]))
        if "SQ_WAVES" in cs and "SQ_INSTS_VALU" in cs:
            w = cs["SQ_WAVES"]
            lines.append(f"    per wave: {cs['SQ_INSTS_VALU'] / w:.0f} VALU, {cs.get('SQ_INSTS_MFMA', 0) / w:.1f} MFMA, "
                         f"{cs.get('SQ_INSTS_LDS', 0) / w:.0f} LDS, {cs.get('SQ_INSTS_VMEM_RD', 0) / w:.1f} loads, "
                         f"{cs.get('SQ_INSTS_VMEM_WR', 0) / w:.1f} stores, {cs.get('SQ_INSTS_SALU', 0) / w:.0f} SALU instructions")
        if "SQ_VALU_MFMA_BUSY_CYCLES" in cs and "SQ_BUSY_CYCLES" in cs and "GRBM_GUI_ACTIVE" in cs:
            # MFMA busy cycles are summed over the SIMDs; 256 CUs x 4 SIMDs; GRBM_GUI_ACTIVE is summed over 8 XCDs
            busy = cs["SQ_VALU_MFMA_BUSY_CYCLES"] / 1024
            active = cs["GRBM_GUI_ACTIVE"] / 8
            lines.append(f"    matrix cores busy {busy:.0f} cycles per SIMD of {active:.0f} GPU-active cycles = {100 * busy / active:.1f} %")
        if "SQ_WAIT_INST_ANY" in cs and "SQ_WAVE_CYCLES" in cs:
            lines.append(f"    waves waiting for an instruction's operands or issue: {100 * cs['SQ_WAIT_INST_ANY'] / cs['SQ_WAVE_CYCLES']:.1f} % of wave cycles")
        if "SQ_LDS_BANK_CONFLICT" in cs and "SQ_ACTIVE_INST_LDS" in cs and cs["SQ_ACTIVE_INST_LDS"]:
            # conflicts are counted in cycles, active time in units of four cycles
            lines.append(f"    LDS bank conflict cycles / LDS active cycles: {100 * cs['SQ_LDS_BANK_CONFLICT'] / (4 * cs['SQ_ACTIVE_INST_LDS']):.1f} %")
        lines.append("")
        if nb is not None:
            for name, (sym, srcs) in KERNEL_SYMBOLS.items():
                if sym in k:
                    traffic.setdefault(workload, {})[name] = dict(bytes=round(nb), summary=f"profiles/{out_name}.txt",
                                                                  kernel=k[:120], sources=srcs, digest=source_digest(srcs))
    # figures taken on other sources than the tree's are dropped
    for w in list(traffic):
        for name in list(traffic[w]):
            rec = traffic[w][name]
            if source_digest(rec["sources"]) != rec["digest"]:
                del traffic[w][name]
    out = os.path.join(ROOT, "profiles", out_name + ".txt")
    with open(out, "w") as f:
        f.write("\n".join(lines))
    with open(TRAFFIC_JSON, "w") as f:
        json.dump(traffic, f, indent=1, sort_keys=True)
    print("\n".join(lines))


def trace_summary(dirs, out_name, command):
    """Turn the ``*kernel_stats.csv`` of ``rocprofv3 --kernel-trace --stats`` runs of this script (one directory
    per workload, named ..._<workload>) into the text summary ``profiles/<out_name>.txt``: time per step and
    kernel.  The step count is read off the backward launch (one per attention call, two calls per step); a trace
    without backward launches is the forward pass of the four-stage encoder (four forward launches per pass)."""
    import csv
    import glob
    lines = ["rocprofv3 kernel traces of the benchmark step (step = regular + shifted block pair, forward + backward; "
             "cfg5: one forward pass of the four-stage encoder).",
             "Commands (from the repository root, TMPDIR=/tmp):"]
    lines += [f"  {c}" for c in command]
    lines.append("Durations in microseconds; kernels shorter than 1 us per step are left out of the tables.")
    for d in dirs:
        paths = glob.glob(os.path.join(d, "**", "*kernel_stats.csv"), recursive=True)
        if not paths:
            sys.exit(f"no *kernel_stats.csv under {d}")
        rows = list(csv.DictReader(open(paths[0])))
        # one backward launch per attention call: the resident kernels' or, on the fused path, the score gradient's
        bwd = sum(int(r["Calls"]) for r in rows if "_bwd_all_kernel" in r["Name"]) or \
            sum(int(r["Calls"]) for r in rows if "fused_sq_kernel<" in r["Name"] and ", 2>" in r["Name"])
        steps = max(bwd // 2, 1)
        if bwd == 0:                                 # the forward-only encoder: four attention launches per pass
            steps = max(sum(int(r["Calls"]) for r in rows if "_fwd_kernel<" in r["Name"] and "wattn" in r["Name"]) // 4, 1)
        tot = sum(float(r["TotalDurationNs"]) for r in rows)
        groups = {"library GEMMs (Cijk_*)": 0.0, "kernels of this library (sswin::*)": 0.0, "PyTorch element-wise / copies": 0.0}
        lines += ["", f"{os.path.basename(d.rstrip('/'))}: {steps} steps, GPU kernel time {tot / 1e3 / steps:.1f} us per step "
                      f"over {sum(int(r['Calls']) for r in rows) / steps:.0f} dispatches",
                  " calls/step   us/step    avg us      %  kernel"]
        for r in sorted(rows, key=lambda r: -float(r["TotalDurationNs"])):
            t, name = float(r["TotalDurationNs"]), r["Name"]
            key = ("library GEMMs (Cijk_*)" if name.startswith("Cijk") else
                   "kernels of this library (sswin::*)" if "sswin::" in name else "PyTorch element-wise / copies")
            groups[key] += t
            if t / 1e3 / steps < 1.0:
                continue
            short = name.replace("void ", "")
            if "sswin::" in short:
                short = short.split("(")[0]
            lines.append(f"{int(r['Calls']) / steps:11.1f}  {t / 1e3 / steps:8.1f}  {float(r['AverageNs']) / 1e3:8.1f}  "
                         f"{100 * t / tot:5.2f}  {short[:100]}")
        lines.append("per step: " + ", ".join(f"{k} {v / 1e3 / steps:.0f} us" for k, v in groups.items()))
    out = os.path.join(ROOT, "profiles", out_name + ".txt")
    with open(out, "w") as f:
        f.write("\n".join(lines) + "\n")
    print("\n".join(lines))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg2", choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "ref7"],
                    help="cfg2 is the benchmark (the configuration the metric is quoted on); cfg1, cfg3 and cfg4 are "
                         "reported the same way, without the CPU leg; cfg5 is the forward pass of the four-stage encoder; "
                         "ref7 is the room of cfg2 in the reference's own setting (window 7, 3 heads of 16 channels), which "
                         "runs on the fused path")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel table")
    ap.add_argument("--kernels-json", default=None)
    ap.add_argument("--profile-kernel", default=None, metavar="NAME",
                    help="run only the kernels whose table name contains NAME (several: comma separated; for rocprofv3) and exit")
    ap.add_argument("--profile-reps", type=int, default=5)
    ap.add_argument("--pmc-summary", nargs="+", default=None, metavar="DIR",
                    help="no GPU work: summarise the rocprofv3 --pmc csv output under these directories into "
                         "profiles/<--pmc-name>.txt and profiles/traffic.json")
    ap.add_argument("--trace-summary", nargs="+", default=None, metavar="DIR",
                    help="no GPU work: summarise the kernel_stats.csv of rocprofv3 --kernel-trace --stats runs of this "
                         "script into profiles/<--pmc-name>.txt")
    ap.add_argument("--pmc-name", default=None)
    ap.add_argument("--pmc-kernels", nargs="+", default=None, metavar="SUBSTR",
                    help="kernel symbols to keep in the summary (default: those of KERNEL_SYMBOLS)")
    ap.add_argument("--pmc-command", action="append", default=[], help="command line(s) quoted in the summary")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (windows are independent attention problems, so the path "
                 "would shard by window ranges with no exchange); rerun with --gpus 1")
    if args.trace_summary:
        trace_summary(args.trace_summary, args.pmc_name or "bench_step_kernel_trace", args.pmc_command)
        return
    if args.pmc_summary:
        from sparseswin3d_amd import synth
        name = {"cfg1": synth.config1, "cfg2": synth.config2, "cfg3": synth.config3, "cfg4": synth.config4,
                "ref7": synth.config_ref7}[args.workload]().name
        pmc_summary(args.pmc_summary, args.pmc_name or f"pmc_{args.workload}", name, args.pmc_command, args.pmc_kernels)
        return
    if not torch.cuda.is_available():
        sys.exit("bench.py: no HIP GPU visible")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.workload == "cfg5":
        bench_encoder(device, args)
        return
    wl = build_workload(device, args.workload)
    if args.workload != "cfg2":
        args.no_cpu = True
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
    from sparseswin3d_amd import _lib
    _lib.launch_timer = []
    _lib.launch_timer_only = {"sswin_window_attention_forward", "sswin_window_attention_backward"}
    for _ in range(max(3, min(10, args.steps))):
        run_step(wl)
    torch.cuda.synchronize()
    in_step = {}
    for name, _, start, stop in _lib.launch_timer:
        in_step.setdefault(name.replace("sswin_", ""), []).append(start.elapsed_time(stop))
    _lib.launch_timer = _lib.launch_timer_only = None
    in_step = {k: sum(v) / len(v) for k, v in in_step.items()}
    log("attention launches inside a step (HIP events, mean over both blocks): " +
        ", ".join(f"{k} {v:.4f} ms" for k, v in in_step.items()))

    roofline = None
    sizes = {}
    dtype_name = {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16"}[wl["dtype"]]
    if not args.no_kernels:
        table, sizes = kernel_table(wl)
        log(f"{'kernel':36s} {'ms':>9s} {'calls':>5s} {'alg MB':>9s} {'GB/s':>9s} {'% HBM':>7s}")
        summary = {}
        titles = {"stage": "-- index glue of one stage (window indices, mask, stride-2 merge) --",
                  "projections": "-- qkv and proj layers of one attention call (dense [N, C] GEMMs) --"}
        scope = {"stage": "once per stage", "projections": "one attention fwd+bwd"}
        for path in ("resident", "fused", "operators", "stage", "projections"):
            rows_ = [r for r in table if r["path"] == path]
            if not rows_:
                continue
            log(titles.get(path, f"-- {path} path, one attention forward+backward --"))
            for r in rows_:
                inm = r.get("ms_in_module")
                log(f"{r['kernel']:36s} {r['ms']:9.4f} {r['calls']:5d} {r['algorithmic_bytes'] / 1e6:9.1f} "
                    f"{(r['achieved_gbps'] or 0):9.1f} {100 * (r['frac'] or 0):7.2f}" +
                    (f"   in the module call {inm:.4f} ms = {100 * r['algorithmic_bytes'] / inm / 1e6 / HBM_PEAK_GBPS:.2f} %" if inm else ""))
            # the operator path is summed from the durations inside a module call (events around every launch of
            # the call), the other paths from the launches timed alone
            ms_ = sum(r.get("ms_in_module", r["ms"]) * r["calls"] for r in rows_)
            alg = sum(r["algorithmic_bytes"] * r["calls"] for r in rows_)
            summary[path] = dict(ms=round(ms_, 4), algorithmic_bytes=alg,
                                 frac=round(alg / ms_ / 1e6 / HBM_PEAK_GBPS, 4))
            if path == "operators":
                alone = sum(r["ms"] * r["calls"] for r in rows_)
                summary[path].update(timed="inside a module call", ms_alone=round(alone, 4),
                                     frac_alone=round(alg / alone / 1e6 / HBM_PEAK_GBPS, 4))
            log(f"{path} kernels, {scope.get(path, 'one attention fwd+bwd')}: {ms_:.3f} ms for {alg / 1e6:.1f} MB algorithmic "
                f"= {alg / ms_ / 1e6:.1f} GB/s = {100 * alg / ms_ / 1e6 / HBM_PEAK_GBPS:.2f}% of HBM peak")
        # the step runs the window-resident path: its slowest kernel is the dominant one
        # (the token plan is a sequence of small launches, not a kernel)
        # the path the step runs (the module's own choice): resident where its kernels apply, else fused
        run_path = "resident" if any(r["kernel"] == "resident forward" for r in table) else "fused"
        dom = max((r for r in table if r["path"] == run_path and "token plan" not in r["kernel"] and "token_plan" not in r["kernel"]),
                  key=lambda r: r.get("ms_in_module", r["ms"]) * r["calls"])
        # its duration inside the step (events above) is what the roofline entry uses; the same
        # launch repeated back to back on its own (the table) runs 10-20 % slower
        step_ms = in_step.get("window_attention_backward") if "backward (dQ,dK,dV,dS)" in dom["kernel"] else None
        ms = step_ms or dom.get("ms_in_module") or dom["ms"]
        gbps = dom["algorithmic_bytes"] / ms / 1e6
        traffic, traffic_note = measured_traffic(wl["name"], dom["kernel"])
        roofline = dict(bound="hbm", kernel=dom["kernel"], achieved=round(gbps, 1),
                        peak=HBM_PEAK_GBPS, unit="GB/s", frac=round(gbps / HBM_PEAK_GBPS, 4),
                        traffic=traffic, traffic_source=traffic_note,
                        algorithmic_bytes=dom["algorithmic_bytes"], ms=round(ms, 4),
                        ms_alone=round(dom["ms"], 4), path=run_path,
                        timed="inside the step" if step_ms else "inside a module call" if dom.get("ms_in_module") else "alone")
        if dom.get("flops"):
            # the same launch against the matrix-core roof of the type its products run in
            tflops = dom["flops"] / ms / 1e9
            roofline["mfma"] = dict(achieved=round(tflops, 2), peak=MFMA_PEAK_TFLOPS[dtype_name], unit="TFLOP/s",
                                    frac=round(tflops / MFMA_PEAK_TFLOPS[dtype_name], 4), flops=dom["flops"],
                                    note="algorithmic flops: 2 c^2 hd per product and group, padding of the 32-token tiles not counted")
        # the sparse softmax on its own (forward and backward), as the operator path runs it
        for key, row_name in (("softmax_fwd", "softmax_last_dim_forward"), ("softmax_bwd", "softmax_last_dim_backward")):
            row = next((r for r in table if r["kernel"] == row_name and r["path"] == "operators"), None)
            if row:
                t_bytes, t_note = measured_traffic(wl["name"], row_name)
                ms_ = row.get("ms_in_module", row["ms"])
                roofline[key] = dict(kernel=row_name, ms=round(ms_, 4), ms_alone=round(row["ms"], 4),
                                     algorithmic_bytes=row["algorithmic_bytes"],
                                     achieved=round(row["algorithmic_bytes"] / ms_ / 1e6, 1), unit="GB/s",
                                     frac=round(row["algorithmic_bytes"] / ms_ / 1e6 / HBM_PEAK_GBPS, 4),
                                     traffic=t_bytes, traffic_source=t_note,
                                     timed="inside a module call" if "ms_in_module" in row else "alone")
        roofline["path_summaries"] = summary
        roofline["module_call_ms"] = module_times(wl)
        log(f"one module call forward+backward by path (ms, projections and glue included): {roofline['module_call_ms']}")
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
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype_name, "data": "synthetic",
        "config": {"workload": f"{wl['name']}: block pair (regular {wl['window'][0]}^3 windows, then shifted by "
                               f"{wl['shift'][0]}) of WindowAttentionSparse, dim {wl['dim']}, {wl['heads']} heads, forward+backward",
                   "voxels": wl["N"], "attention_calls_per_step": calls, **sizes},
        "roofline": roofline, "cpu_baseline": cpu,
    }
    if cpu:
        line["speedup_vs_cpu"] = value / cpu["value"]
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
