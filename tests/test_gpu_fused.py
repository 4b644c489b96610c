"""The fused window-attention path: token plan bit-exact against closed forms, module results
equal to the operator-by-operator path and to the CPU path (fp32 rel 1e-5, 16-bit rel 2e-2)."""
import numpy as np
import pytest
import torch

from helpers import close, ragged_window_indices, random_window_indices

pytestmark = pytest.mark.gpu


def _closed_form_plan(ind, n, H):
    key = ind[:, 0].astype(np.int64) * n + ind[:, 1]
    order = np.argsort(key, kind="stable")
    wins, first, counts = np.unique(ind[order, 0], return_index=True, return_counts=True)
    T = np.repeat(first, counts)
    c = np.repeat(counts, counts)
    q2 = np.concatenate([[0], np.cumsum(counts.astype(np.int64) ** 2)[:-1]])
    g_c = np.repeat(counts, H)
    g_T = np.repeat(first, H)
    g_h = np.tile(np.arange(H), len(wins))
    g_sq = np.repeat(q2, H) * H + g_h * np.repeat(counts.astype(np.int64) ** 2, H)
    g_w = np.repeat(wins, H)
    tokens = np.stack([order, T, c, ind[order, 1], ind[order, 0]])
    return tokens, np.stack([g_c, g_T, g_sq, g_w, g_h]), int((counts.astype(np.int64) ** 2).sum()) * H, int(counts.max())


@pytest.mark.parametrize("case", ["random", "ragged", "single", "big"])
def test_token_plan_closed_forms(case):
    from sparseswin3d_amd.fused import TokenPlan
    rng = np.random.default_rng(len(case))
    if case == "random":
        B, n, H = 50, 125, 3
        ind = random_window_indices(rng, B, n, 1500)
    elif case == "ragged":
        counts = [1, 0, 125, 2, 0, 0, 33, 64, 5, 17, 1, 1, 100]
        B, n, H = len(counts), 125, 6
        ind = ragged_window_indices(rng, counts, n)
    elif case == "single":
        B, n, H = 4, 27, 1
        ind = np.array([[3, 26]], np.int32)
    else:
        B, n, H = 20000, 125, 3
        ind = random_window_indices(rng, B, n, 120000)
    tp = TokenPlan(torch.from_numpy(ind).cuda(), B, n, H)
    tokens, plan, A, c_max = _closed_form_plan(ind, n, H)
    assert (tp.G, tp.A, tp.c_max) == (plan.shape[1], A, c_max)
    np.testing.assert_array_equal(tp.tokens.view(5, -1).cpu().numpy(), tokens)
    np.testing.assert_array_equal(tp.plan.view(5, -1)[:, :tp.G].cpu().numpy(), plan)


def _modules(dim, heads, dtype):
    from sparseswin3d_amd.window_attention import WindowAttentionSparse
    torch.manual_seed(0)
    a = WindowAttentionSparse(dim, heads, (5, 5, 5), qkv_bias=True).cuda().to(dtype)
    with torch.no_grad():
        a.relative_position_bias_table.normal_(0, 0.5)
    return a


@pytest.mark.parametrize("shift", [(0, 0, 0), (2, 2, 2)])
def test_fused_equals_operator_path(shift):
    from sparseswin3d_amd import synth
    from sparseswin3d_amd.window_attention import SparseVoxelTensor
    c4, _ = synth.with_batch([synth.box_surfaces_scene(seed=21, grid=(45, 45, 45), n_boxes=4)])
    idx, nw, n = synth.window_indices(c4, (45, 45, 45), (5, 5, 5), shift)
    mask = torch.from_numpy(synth.shift_region_mask((45, 45, 45), (5, 5, 5), (2, 2, 2))).cuda() if any(shift) else None
    attn = _modules(96, 3, torch.float32)
    feats = torch.randn(len(idx), 96, device="cuda")
    up = torch.randn(len(idx), 96, device="cuda")
    res = {}
    for fused in (True, False):
        attn.fused = fused
        attn.zero_grad()
        f = feats.clone().requires_grad_(True)
        out = attn(SparseVoxelTensor(f, torch.from_numpy(idx).cuda(), (n,), nw), mask).features
        out.backward(up)
        res[fused] = [t.detach().cpu().numpy() for t in
                      (out, f.grad, attn.qkv.weight.grad, attn.relative_position_bias_table.grad)]
    for a, b, what in zip(res[True], res[False], ("out", "d feats", "d qkv.w", "d bias table")):
        close(a, b, 1e-5, what)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_16bit_against_cpu_fp64(dtype):
    from oracle import cpu_path
    from sparseswin3d_amd import synth
    from sparseswin3d_amd.window_attention import SparseVoxelTensor
    c4, _ = synth.with_batch([synth.filled_blob_scene(seed=4, grid=(10, 10, 10), fill=0.9)])
    idx, nw, n = synth.window_indices(c4, (10, 10, 10), (5, 5, 5), (2, 2, 2))
    mask_np = synth.shift_region_mask((10, 10, 10), (5, 5, 5), (2, 2, 2))
    attn = _modules(64, 2, dtype)
    feats = (torch.randn(len(idx), 64) * 0.5).to(dtype)
    x = SparseVoxelTensor(feats.cuda(), torch.from_numpy(idx).cuda(), (n,), nw)
    out = attn(x, torch.from_numpy(mask_np).cuda()).features
    p = {k: v.detach().double().cpu() for k, v in attn.state_dict().items()}
    rpb = p["relative_position_bias_table"][p["relative_position_index"].reshape(-1).long()].reshape(n, n, -1).permute(2, 0, 1)
    ref = cpu_path.window_attention_cpu(feats.double(), idx, n, 2, p["qkv.weight"], p["qkv.bias"], p["proj.weight"],
                                        p["proj.bias"], rpb, mask_np)
    close(out.detach().double().cpu().numpy(), ref.numpy(), 2e-2, f"fused {dtype}")
