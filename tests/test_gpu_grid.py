"""GPU parity of the voxel-grid glue of a stage (window indices, shift mask, stride-2 merge) against
the step-by-step CPU restatement in oracle/grid.py: integers bit-exact, pooled features 1e-6 (fp32)."""
import numpy as np
import pytest
import torch

from helpers import close

pytestmark = pytest.mark.gpu


def _coords(rng, batch, grid, count):
    c = np.stack([rng.integers(0, batch, count)] + [rng.integers(0, g, count) for g in grid], 1)
    c = np.unique(c, axis=0).astype(np.int32)
    return c[rng.permutation(len(c))]


@pytest.mark.parametrize("grid,ws,ss,batch", [((33, 28, 17), (5, 5, 5), (2, 2, 2), 2), ((33, 28, 17), (5, 5, 5), (0, 0, 0), 2),
                                              ((12, 9, 7), (4, 3, 7), (2, 1, 0), 3), ((5, 5, 5), (5, 5, 5), (0, 0, 0), 1),
                                              ((64, 64, 30), (7, 7, 7), (3, 3, 3), 1), ((2, 2, 2), (2, 2, 2), (0, 0, 0), 4)])
def test_window_indices(grid, ws, ss, batch):
    from oracle import grid as og
    from sparseswin3d_amd.layers import sparse_window_indices
    rng = np.random.default_rng(sum(grid) + batch)
    c4 = _coords(rng, batch, grid, 5000)
    ref, nw, n = og.window_indices(c4, grid, ws, ss)
    dims = [-(-g // w) * w for g, w in zip(grid, ws)]
    got = sparse_window_indices(torch.from_numpy(c4).cuda(), batch, dims, ws, ss)
    assert got.dtype == torch.int32
    np.testing.assert_array_equal(got.cpu().numpy(), ref)
    assert int(got[:, 0].max()) < batch * nw and int(got[:, 1].max()) < n


def test_window_indices_empty_and_errors():
    from sparseswin3d_amd.layers import sparse_window_indices
    empty = torch.zeros((0, 4), dtype=torch.int32, device="cuda")
    assert sparse_window_indices(empty, 1, [5, 5, 5], (5, 5, 5)).shape == (0, 2)
    one = torch.zeros((1, 4), dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="multiple of the window"):
        sparse_window_indices(one, 1, [6, 5, 5], (5, 5, 5))
    with pytest.raises(RuntimeError, match="shift"):
        sparse_window_indices(one, 1, [5, 5, 5], (5, 5, 5), (5, 0, 0))
    with pytest.raises(RuntimeError, match="GPU only"):
        sparse_window_indices(one.cpu(), 1, [5, 5, 5], (5, 5, 5))


@pytest.mark.parametrize("dims,ws,ss", [((35, 30, 20), (5, 5, 5), (2, 2, 2)), ((6, 8, 4), (3, 4, 2), (1, 2, 1)),
                                        ((5, 10, 5), (5, 5, 5), (0, 2, 0)), ((4, 4, 4), (2, 2, 2), (0, 0, 0)),
                                        ((260, 260, 100), (5, 5, 5), (2, 2, 2))])
def test_shift_mask(dims, ws, ss):
    from oracle import grid as og
    from sparseswin3d_amd.layers import compute_mask
    got = compute_mask(list(dims), list(ws), list(ss), "cuda")
    assert got.dtype == torch.int8
    np.testing.assert_array_equal(got.cpu().numpy(), og.shift_mask(dims, ws, ss))


def test_window_indices_full_size_room():
    """The 107 500-voxel room of the benchmark: shifted window indices, bit for bit."""
    from oracle import grid as og
    from sparseswin3d_amd import synth
    from sparseswin3d_amd.layers import sparse_window_indices
    w = synth.config2()
    ref, nw, n = og.window_indices(w.coords4, w.spatial_shape, (5, 5, 5), (2, 2, 2))
    dims = synth.padded_shape(w.spatial_shape, (5, 5, 5))
    got = sparse_window_indices(torch.from_numpy(w.coords4).cuda(), w.batch_size, dims, (5, 5, 5), (2, 2, 2))
    np.testing.assert_array_equal(got.cpu().numpy(), ref)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.bfloat16, 1e-2), (torch.float16, 2e-3)])
@pytest.mark.parametrize("grid,batch", [((33, 28, 17), 2), ((2, 2, 2), 3), ((7, 1, 40), 1)])
def test_downsample_pool_forward_backward(grid, batch, dtype, tol):
    from oracle import grid as og
    from sparseswin3d_amd.layers import _PoolWindows, downsample_plan
    from sparseswin3d_amd.window_attention import SparseVoxelTensor
    rng = np.random.default_rng(grid[0] * 7 + batch)
    c4 = _coords(rng, batch, grid, 4000)
    f = rng.standard_normal((len(c4), 24)).astype(np.float32)
    feats = torch.from_numpy(f).to(dtype).cuda().requires_grad_(True)
    x = SparseVoxelTensor(feats, torch.from_numpy(c4).cuda(), grid, batch)
    plan, coords, shape = downsample_plan(x, 2)
    ref_coords, ref_pooled, inverse = og.downsample(c4, feats.detach().float().cpu().numpy())
    np.testing.assert_array_equal(coords.cpu().numpy(), ref_coords)          # ascending (batch, d, h, w)
    assert list(shape) == [(g + 1) // 2 for g in grid]
    pooled = _PoolWindows.apply(feats, plan, True)
    close(pooled.detach().float().cpu().numpy(), ref_pooled, tol, "mean pool")
    g = rng.standard_normal(ref_pooled.shape).astype(np.float32)
    gd = torch.from_numpy(g).to(dtype).cuda()
    pooled.backward(gd)
    cnt = np.bincount(inverse, minlength=len(ref_coords))
    close(feats.grad.float().cpu().numpy(), (gd.float().cpu().numpy() / cnt[:, None])[inverse], tol, "mean pool gradient")
    summed = _PoolWindows.apply(feats.detach(), plan, False)
    _, ref_sum, _ = og.downsample(c4, feats.detach().float().cpu().numpy(), mean=False)
    close(summed.float().cpu().numpy(), ref_sum, tol, "sum pool")


def test_stage_with_downsample_and_shared_plans(monkeypatch):
    """BasicLayer(depth=4, downsample): the four blocks need two token plans (regular, shifted),
    and the merged stage output matches the CPU restatement built from the same weights."""
    import copy
    from oracle import cpu_path, grid as og
    from sparseswin3d_amd import fused, synth
    from sparseswin3d_amd.layers import BasicLayer, PoolDownsample
    from sparseswin3d_amd.window_attention import SparseVoxelTensor
    made = []
    real = fused.TokenPlan

    class Counting(real):
        def _allocate(self, indices, batch_size, n, num_heads, tasks, order_only=False):
            made.append(tasks)
            assert order_only == (not tasks)             # the merge's plan is the one that keeps the voxel order only
            super()._allocate(indices, batch_size, n, num_heads, tasks, order_only)

    monkeypatch.setattr(fused, "TokenPlan", Counting)
    torch.manual_seed(3)
    rng = np.random.default_rng(3)
    grid, batch = (21, 18, 11), 2
    c4 = _coords(rng, batch, grid, 3000)
    layer = BasicLayer(dim=96, depth=4, num_heads=3, window_size=(5, 5, 5), drop_path=0.0, qkv_bias=True,
                       downsample=PoolDownsample).cuda()
    feats = torch.randn(len(c4), 96)
    y = layer(SparseVoxelTensor(feats.cuda(), torch.from_numpy(c4).cuda(), grid, batch))
    assert made == [True, True, False]           # regular windows, shifted windows, the 2x2x2 merge

    mask_np = og.shift_mask(synth.padded_shape(grid, (5, 5, 5)), (5, 5, 5), (2, 2, 2))
    h = feats.double()
    with torch.no_grad():
        for i, blk in enumerate(layer.blocks):
            b = copy.deepcopy(blk).cpu().double()
            shift = (0, 0, 0) if i % 2 == 0 else (2, 2, 2)
            win_idx, nw, n = og.window_indices(c4, grid, (5, 5, 5), shift)
            a = b.attn
            rpb = a.relative_position_bias_table[a.relative_position_index[:n, :n].reshape(-1)].reshape(n, n, -1).permute(2, 0, 1)
            t = cpu_path.window_attention_cpu(b.norm1(h), win_idx, n, a.num_heads, a.qkv.weight, a.qkv.bias,
                                              a.proj.weight, a.proj.bias, rpb, mask_np if any(shift) else None)
            h = h + t
            h = h + b.mlp(b.norm2(h))
        ref_coords, pooled, _ = og.downsample(c4, h.numpy())
        d = copy.deepcopy(layer.downsample).cpu().double()
        ref = d.reduction(d.norm(torch.from_numpy(pooled)))
    np.testing.assert_array_equal(y.indices.cpu().numpy(), ref_coords)
    assert list(y.spatial_shape) == [(g + 1) // 2 for g in grid] and y.features.shape[1] == 192
    close(y.features.detach().cpu().numpy(), ref.numpy(), 1e-4, "stage output after four blocks and the merge")


def test_shift_masks_are_kept_per_shape():
    """compute_mask returns the stored mask for shapes it has seen on this stream, a new one for others, and keeps
    at most eight."""
    from sparseswin3d_amd import layers
    layers._MASKS.clear()
    a = layers.compute_mask([10, 10, 10], [5, 5, 5], [2, 2, 2], "cuda")
    assert layers.compute_mask([10, 10, 10], [5, 5, 5], [2, 2, 2], torch.device("cuda", 0)) is a
    b = layers.compute_mask([10, 10, 15], [5, 5, 5], [2, 2, 2], "cuda")
    assert b is not a and b.shape == (12, 125) and a.shape == (8, 125)
    c = layers.compute_mask([10, 10, 10], [5, 5, 5], [2, 0, 2], "cuda")
    assert c is not a and not torch.equal(c, a)
    for k in range(9):
        layers.compute_mask([5, 5, 5 * (k + 1)], [5, 5, 5], [2, 2, 2], "cuda")
    assert len(layers._MASKS) == 8
    again = layers.compute_mask([10, 10, 10], [5, 5, 5], [2, 2, 2], "cuda")        # dropped meanwhile: built anew
    assert again is not a and torch.equal(again, a)
