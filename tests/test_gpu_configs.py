"""Parity at the full sizes of the five benchmark configurations (synth.config1 … config5_rooms).

Two kinds of check per configuration:
  * the operator chain (qkv_sparse_indices → q_k → flatten/unique_consecutive → softmax → qk_v and
    the backward operators) on the GPU against the scalar C oracle on the same seeded inputs:
    every index, offset and permutation bit-exact, values within the stated tolerance;
  * the attention module (fused path and operator path) against the PyTorch-CPU path in fp64,
    plus size-independent properties (row sums of the attention, linearity of the backward in
    the upstream gradient, invariance to the order of the voxels).

Tolerances: fp32 rel 1e-5, bf16 rel 2e-2, measured per element against its condition magnitude: sum_k |a_ik b_kj|
for products, the element's own softmax row, a token's own row of the module outputs, sum |dS| for the bias table
gradient (helpers.close)."""
import numpy as np
import pytest
import torch

from helpers import softmax_bwd_mag, PATHS, BiasGradMagnitude, close, product_mag, qkv_operands, set_path

pytestmark = pytest.mark.gpu


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t if dtype is None else t.to(dtype)


def host(t):
    return t.detach().to(torch.float64).cpu().numpy() if t.is_floating_point() else t.cpu().numpy()


@pytest.fixture(scope="module")
def ops():
    from sparseswin3d_amd import custom_ops
    return custom_ops


def _workload(name):
    from sparseswin3d_amd import synth
    if name == "cfg5":
        return synth.config5_rooms()[0]
    return getattr(synth, {"cfg1": "config1", "cfg2": "config2", "cfg3": "config3", "cfg4": "config4"}[name])()


def _windows(w, shift):
    from sparseswin3d_amd import synth
    idx, nw, n = synth.window_indices(w.coords4, w.spatial_shape, w.window, shift)
    mask = synth.shift_region_mask(synth.padded_shape(w.spatial_shape, w.window), w.window, (2, 2, 2)) if any(shift) else None
    return idx, nw * w.batch_size, n, mask


# ------------------------------------------------------------------------------------------
# operator chain against the C oracle, full size
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("cfg,shift,dtype", [("cfg1", (0, 0, 0), torch.float32), ("cfg2", (2, 2, 2), torch.float32),
                                             ("cfg3", (2, 2, 2), torch.float32), ("cfg4", (0, 0, 0), torch.bfloat16)],
                         ids=["cfg1", "cfg2", "cfg3", "cfg4-bf16"])
def test_operator_chain_full_size(ops, oracle, cfg, shift, dtype):
    w = _workload(cfg)
    idx, B, n, _ = _windows(w, shift)
    H, hd = w.heads, w.dim // w.heads
    rtol = 1e-5 if dtype == torch.float32 else 2e-2
    rng = np.random.default_rng(7)
    d = qkv_operands(oracle, idx, B, n, H, hd, rng, dtype=np.float32, scale=0.5 if cfg == "cfg4" else 1.0)

    # I1: element-level COO of Q/V and K^T, both permutations
    got = ops.qkv_sparse_indices(dev(idx), B, n, H, hd)
    for g, r, what in zip(got, (d["idx_qv"], d["sorted_qv"], d["idx_k"], d["sorted_k"]),
                          ("_indices_qv", "sorted_qv", "_indices_k", "sorted_k")):
        assert g.dtype == torch.int32
        np.testing.assert_array_equal(host(g), r, err_msg=what)
    del got

    # M1: S = Q K, COO indices and group counts
    q, kt, v = (dev(d[k], dtype) for k in ("q", "kt", "v"))
    qi, ki = dev(d["qi"]), dev(d["ki"])
    s_idx, s_val, s_shape, c = ops.matmul_cuda_naive(q, qi, d["q_shape"], kt, ki, d["k_shape"], "q_k")
    q64, kt64, v64 = host(q), host(kt), host(v)
    r_idx, r_val, r_shape, r_c = oracle.matmul_cuda_naive(q64, d["qi"], d["q_shape"], kt64, d["ki"], d["k_shape"], "q_k")
    assert s_shape == r_shape
    np.testing.assert_array_equal(host(c), r_c)
    np.testing.assert_array_equal(host(s_idx), r_idx)
    close(host(s_val), r_val, rtol, "q_k values",
          mag=product_mag(oracle, "matmul_cuda_naive", q64, d["qi"], d["q_shape"], kt64, d["ki"], d["k_shape"], "q_k"))

    # I2 + I4: softmax row ids
    rows = ops.unique_consecutive_indices(ops.flatten_indices(s_idx[:3].contiguous(), s_shape[:3]))
    r_rows = oracle.unique_consecutive_indices(oracle.flatten_indices(r_idx[:3], r_shape[:3]))
    np.testing.assert_array_equal(host(rows), r_rows)

    # S1 / S2 (always fp32, as the reference's wrapper casts; the oracle runs them in fp64)
    s32 = dev(r_val, torch.float32)
    p = ops.softmax_last_dim_forward(rows, s32)
    r_p = oracle.softmax_last_dim_forward(r_rows, host(s32))
    close(host(p), r_p, 1e-5, "softmax forward", seg=r_rows)
    # every attention row sums to se / (se + 1e-8), se = sum of exp(v - max(0, rowmax)): 1 up to 1e-8 unless a
    # whole row is far below zero (a window of one token with a negative score)
    sums = np.bincount(r_rows, weights=host(p))
    row_max = np.full(r_rows[-1] + 1, -np.inf)
    np.maximum.at(row_max, r_rows, host(s32))
    se = np.bincount(r_rows, weights=np.exp(host(s32) - np.maximum(row_max, 0.0)[r_rows]))
    assert np.all(np.abs(sums - se / (se + 1e-8)) < 1e-5)
    assert np.all(np.abs(sums[row_max >= 0] - 1.0) < 1e-5)
    gp = dev(rng.standard_normal(len(r_val)), torch.float32)
    gs = ops.softmax_last_dim_backward(rows, p, gp)
    close(host(gs), oracle.softmax_last_dim_backward(r_rows, host(p), host(gp)), 1e-5, "softmax backward",
          mag=softmax_bwd_mag(r_rows, host(p), host(gp)))
    zero = np.bincount(r_rows, weights=host(gs))
    assert np.all(np.abs(zero) < 1e-4 * max(1.0, np.abs(host(gs)).max()))   # softmax gradient rows sum to 0

    # M2: O = P V
    pd = p.to(dtype)
    o_idx, o_val, o_shape, c2 = ops.matmul_cuda_naive(pd, s_idx, s_shape, v, qi, d["q_shape"], "qk_v")
    ro_idx, ro_val, ro_shape, ro_c = oracle.matmul_cuda_naive(host(pd), r_idx, r_shape, v64, d["qi"], d["q_shape"], "qk_v")
    assert o_shape == ro_shape
    np.testing.assert_array_equal(host(c2), ro_c)
    np.testing.assert_array_equal(host(o_idx), ro_idx)
    close(host(o_val), ro_val, rtol, "qk_v values",
          mag=product_mag(oracle, "matmul_cuda_naive", host(pd), r_idx, r_shape, v64, d["qi"], d["q_shape"], "qk_v"))
    del o_idx, ro_idx, s_idx, r_idx

    # M3 / M4: the three gradient products and the two transposes
    go = dev(rng.standard_normal(len(ro_val)), dtype)
    for kind, a, b in (("rc_cr", go, kt), ("rr_rc", pd, go), ("cr_rr", kt, pd)):
        out = ops.matmul_grad_cuda_naive(a, b, c, hd, kind)
        close(host(out), oracle.matmul_grad_cuda_naive(host(a), host(b), r_c, hd, kind), rtol, kind,
              mag=product_mag(oracle, "matmul_grad_cuda_naive", host(a), host(b), r_c, hd, kind))
    np.testing.assert_array_equal(host(ops.qkv_transpose(v, c, hd, "rc")), oracle.qkv_transpose(v64, r_c, hd, "rc"))
    np.testing.assert_array_equal(host(ops.qkv_transpose(pd, c, hd, "rr")), oracle.qkv_transpose(host(pd), r_c, hd, "rr"))

    # T1 + I3 + I5: the un-sort at the end of the module (permute, then rank by window*n+pos)
    flat = ops.flatten_indices(qi, d["q_shape"])
    np.testing.assert_array_equal(host(flat), oracle.flatten_indices(d["qi"], d["q_shape"]))
    key = dev((idx[:, 0].astype(np.int64) * n + idx[:, 1]).astype(np.int32))
    inv, count = ops.return_inverse(key, B * n)
    r_inv, r_count = oracle.return_inverse(host(key), B * n)
    assert count == r_count == len(idx)
    np.testing.assert_array_equal(host(inv), r_inv)
    scrambled = dev(rng.permutation(len(idx) * 7).astype(np.int32)[: len(idx)])
    np.testing.assert_array_equal(host(ops.sort_indices(scrambled)), oracle.sort_indices(host(scrambled)))


# ------------------------------------------------------------------------------------------
# the module against the PyTorch-CPU path, full size
# ------------------------------------------------------------------------------------------
def _attention(dim, heads, dtype, seed=0):
    from sparseswin3d_amd.window_attention import WindowAttentionSparse
    torch.manual_seed(seed)
    a = WindowAttentionSparse(dim, heads, (5, 5, 5), qkv_bias=True)
    with torch.no_grad():
        torch.nn.init.xavier_uniform_(a.qkv.weight)
        a.relative_position_bias_table.normal_(0, 0.5)
    return a.cuda().to(dtype)


def _cpu(attn, feats64, idx, n, mask):
    from oracle import cpu_path
    p = {k: v.detach().double().cpu() for k, v in attn.state_dict().items()}
    leaves = {k: p[k].clone().requires_grad_(True) for k in
              ("qkv.weight", "qkv.bias", "proj.weight", "proj.bias", "relative_position_bias_table")}
    table = leaves["relative_position_bias_table"]
    rpb = table[p["relative_position_index"][:n, :n].reshape(-1).long()].reshape(n, n, -1).permute(2, 0, 1)
    mag = BiasGradMagnitude(attn.num_heads, n)
    out = cpu_path.window_attention_cpu(feats64, idx, n, attn.num_heads, leaves["qkv.weight"], leaves["qkv.bias"],
                                        leaves["proj.weight"], leaves["proj.bias"], rpb, mask, "ops", probe=mag.probe)
    leaves["table_mag"] = lambda: mag.table(p["relative_position_index"], table.shape[0])     # after backward
    return out, leaves


def _gpu(attn, feats, idx, B, n, mask, upstream=None):
    from sparseswin3d_amd.window_attention import SparseVoxelTensor
    attn.zero_grad()
    f = feats.cuda().requires_grad_(upstream is not None)
    m = None if mask is None else torch.from_numpy(mask).cuda()
    out = attn(SparseVoxelTensor(f, torch.from_numpy(idx).cuda(), (n,), B), m).features
    if upstream is not None:
        out.backward(upstream.cuda())
    return out.detach(), f.grad


@pytest.mark.parametrize("path", PATHS)
def test_cfg1_forward_against_cpu_path(path):
    """Configuration 1: one forward, regular windows, fp32, ~22k voxels."""
    w = _workload("cfg1")
    idx, B, n, _ = _windows(w, (0, 0, 0))
    attn = _attention(w.dim, w.heads, torch.float32)
    set_path(attn, path)
    torch.manual_seed(1)
    feats = torch.randn(len(idx), w.dim)
    out, _ = _gpu(attn, feats, idx, B, n, None)
    with torch.no_grad():
        ref, _ = _cpu(attn, feats.double(), idx, n, None)
    close(host(out), ref.numpy(), 1e-5, "cfg1 forward")


@pytest.mark.parametrize("cfg,path,shift", [("cfg2", "resident", 2), ("cfg2", "fused", 2), ("cfg2", "operators", 2),
                                            ("cfg2", "resident", 0), ("cfg3", "resident", 2), ("cfg3", "fused", 2),
                                            ("cfg3", "operators", 2)])
def test_forward_backward_against_cpu_path(cfg, path, shift):
    """Configurations 2 (both blocks of the pair: regular windows, then shifted windows with the region mask) and 3
    (shifted): fp32 forward + backward with N(0,1) upstream gradients, at full size."""
    w = _workload(cfg)
    idx, B, n, mask = _windows(w, (shift, shift, shift))
    attn = _attention(w.dim, w.heads, torch.float32)
    set_path(attn, path)
    torch.manual_seed(2)
    feats = torch.randn(len(idx), w.dim)
    up = torch.randn(len(idx), w.dim)
    out, gf = _gpu(attn, feats, idx, B, n, mask, up)
    f64 = feats.double().requires_grad_(True)
    ref, leaves = _cpu(attn, f64, idx, n, mask)
    ref.backward(up.double())
    close(host(out), ref.detach().numpy(), 1e-5, "forward")
    close(host(gf), f64.grad.numpy(), 1e-5, "d features")
    close(host(attn.qkv.weight.grad), leaves["qkv.weight"].grad.numpy(), 1e-5, "d qkv.weight")
    close(host(attn.qkv.bias.grad), leaves["qkv.bias"].grad.numpy(), 1e-5, "d qkv.bias", seg="all")
    close(host(attn.proj.weight.grad), leaves["proj.weight"].grad.numpy(), 1e-5, "d proj.weight")
    close(host(attn.relative_position_bias_table.grad), leaves["relative_position_bias_table"].grad.numpy(), 1e-5,
          "d bias table", mag=leaves["table_mag"]())


@pytest.mark.parametrize("path", PATHS)
def test_cfg4_bf16_dense_windows_against_cpu_fp64(path):
    """Configuration 4: ~8k voxels in windows of 100-125 tokens, dim 768, 24 heads, bf16."""
    w = _workload("cfg4")
    idx, B, n, mask = _windows(w, (2, 2, 2))
    attn = _attention(w.dim, w.heads, torch.bfloat16)
    set_path(attn, path)
    torch.manual_seed(3)
    feats = (torch.randn(len(idx), w.dim) * 0.5).to(torch.bfloat16)
    up = torch.randn(len(idx), w.dim).to(torch.bfloat16)
    out, gf = _gpu(attn, feats, idx, B, n, mask, up)
    f64 = feats.double().requires_grad_(True)
    ref, leaves = _cpu(attn, f64, idx, n, mask)
    ref.backward(up.double())
    close(host(out), ref.detach().numpy(), 2e-2, "forward")
    close(host(gf), f64.grad.numpy(), 2e-2, "d features")
    close(host(attn.relative_position_bias_table.grad), leaves["relative_position_bias_table"].grad.numpy(), 2e-2,
          "d bias table", mag=leaves["table_mag"]())


def test_cfg5_four_stage_encoder_bf16_forward():
    """Configuration 5: four rooms in one batch (~430k voxels), four attention stages of dims
    96/192/384/768, shift 2, bf16, forward only; floor(coord/2) + mean pooling between stages.
    Each stage's attention is checked against the fp64 CPU path fed with the same stage input.

    Stage 1 has 216 320 window slots: slots*125*96 exceeds 2^31, where the reference's int32
    row-major hash (ops.cu:264) wraps and its own ordering is undefined; all three paths of the module
    order by the exact (window, pos) rank, so every stage runs on all of them."""
    from sparseswin3d_amd import synth
    w = _workload("cfg5")
    coords = w.coords4
    shape = w.spatial_shape
    torch.manual_seed(5)
    feats = torch.randn(len(coords), 96).to(torch.bfloat16)
    dims, heads = (96, 192, 384, 768), (3, 6, 12, 24)
    for stage, (dim, H) in enumerate(zip(dims, heads)):
        idx, nw, n = synth.window_indices(coords, shape, (5, 5, 5), (2, 2, 2))
        B = nw * w.batch_size
        mask = synth.shift_region_mask(synth.padded_shape(shape, (5, 5, 5)), (5, 5, 5), (2, 2, 2))
        # the same indices and mask from the grid kernels, at the stage's full size
        from sparseswin3d_amd.layers import compute_mask, sparse_window_indices
        pdims = synth.padded_shape(shape, (5, 5, 5))
        np.testing.assert_array_equal(
            sparse_window_indices(torch.from_numpy(coords).cuda(), w.batch_size, pdims, (5, 5, 5), (2, 2, 2)).cpu().numpy(), idx)
        np.testing.assert_array_equal(compute_mask(list(pdims), [5, 5, 5], [2, 2, 2], "cuda").cpu().numpy(), mask)
        attn = _attention(dim, H, torch.bfloat16, seed=10 + stage)
        set_path(attn, "resident")
        out, _ = _gpu(attn, feats, idx, B, n, mask)
        with torch.no_grad():
            ref, _ = _cpu(attn, feats.double(), idx, n, mask)
        close(host(out), ref.numpy(), 2e-2, f"stage {stage + 1} resident")
        set_path(attn, "fused")
        out_f, _ = _gpu(attn, feats, idx, B, n, mask)
        close(host(out_f), ref.numpy(), 2e-2, f"stage {stage + 1} fused")
        # stage 1 has B * n * dim above 2^31: the module's operator path orders by voxel rank, not by the int32 hash
        set_path(attn, "operators")
        out_ops, _ = _gpu(attn, feats, idx, B, n, mask)
        close(host(out_ops), ref.numpy(), 2e-2, f"stage {stage + 1} operators")
        if stage == 3:
            break
        # between stages: merge voxels by floor(coord/2), average their features, widen channels;
        # the merge runs on the GPU (window indices of 2x2x2 cells -> token plan -> pooling kernel)
        # and is checked against the CPU restatement at full size
        from oracle import grid as og
        from sparseswin3d_amd.layers import _PoolWindows, downsample_plan
        from sparseswin3d_amd.window_attention import SparseVoxelTensor
        xs = SparseVoxelTensor(out.float(), torch.from_numpy(coords).cuda(), shape, w.batch_size)
        plan, new_coords_d, new_shape = downsample_plan(xs, 2)
        pooled = _PoolWindows.apply(xs.features, plan, True)
        ref_coords, ref_pooled, _ = og.downsample(coords, out.float().cpu().numpy())
        new_coords = new_coords_d.cpu().numpy()
        np.testing.assert_array_equal(new_coords, ref_coords)
        np.testing.assert_allclose(pooled.cpu().numpy(), ref_pooled, rtol=1e-5, atol=1e-6)
        assert tuple(new_shape) == tuple((s_ + 1) // 2 for s_ in shape)
        feats = torch.cat([pooled, pooled], 1).to(torch.bfloat16).cpu()       # dim -> 2*dim
        coords = new_coords
        shape = tuple((s + 1) // 2 for s in shape)


# ------------------------------------------------------------------------------------------
# size-independent properties at the benchmark size (configuration 2)
# ------------------------------------------------------------------------------------------
def test_cfg2_properties_voxel_order_and_linearity():
    w = _workload("cfg2")
    idx, B, n, mask = _windows(w, (2, 2, 2))
    attn = _attention(w.dim, w.heads, torch.float32)
    torch.manual_seed(4)
    N = len(idx)
    feats = torch.randn(N, w.dim)
    up1, up2 = torch.randn(N, w.dim), torch.randn(N, w.dim)
    out, g1 = _gpu(attn, feats, idx, B, n, mask, up1)
    tg1 = attn.relative_position_bias_table.grad.clone()
    # (a) the result does not depend on the order in which the voxels are listed
    perm = np.random.default_rng(0).permutation(N)
    out_p, g1_p = _gpu(attn, feats[perm], idx[perm], B, n, mask, up1[perm])
    close(host(out_p), host(out)[perm], 1e-5, "permuted voxels: forward")
    close(host(g1_p), host(g1)[perm], 1e-5, "permuted voxels: backward")
    # (b) the backward pass is linear in the upstream gradient
    _, g2 = _gpu(attn, feats, idx, B, n, mask, up2)
    tg2 = attn.relative_position_bias_table.grad.clone()
    _, g12 = _gpu(attn, feats, idx, B, n, mask, 2.0 * up1 - 3.0 * up2)
    close(host(g12), 2.0 * host(g1) - 3.0 * host(g2), 2e-5, "linearity d features")
    close(host(attn.relative_position_bias_table.grad), 2.0 * host(tg1) - 3.0 * host(tg2), 2e-5, "linearity d bias")
    # (c) both paths agree and the fused path is deterministic run to run
    out2, _ = _gpu(attn, feats, idx, B, n, mask, up1)
    assert torch.equal(out2, out)
    assert torch.equal(attn.relative_position_bias_table.grad, tg1)      # fixed-order table gradient
    for path in ("fused", "operators"):
        set_path(attn, path)
        out_o, g_o = _gpu(attn, feats, idx, B, n, mask, up1)
        close(host(out_o), host(out), 1e-5, f"{path} path forward")
        close(host(g_o), host(g1), 1e-5, f"{path} path backward")
