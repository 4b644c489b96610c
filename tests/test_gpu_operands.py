"""Sorted operands written directly (sswin_operand_map / sswin_operand_copy / sswin_sorted_coo_indices) against
the reference's composition through the permutations of qkv_sparse_indices (swin3d_base.py:483-498, 672-675),
restated with the CPU oracle.  Index matrices and values are permutations of the inputs: everything is compared
bit for bit, gradients included."""
import numpy as np
import pytest
import torch

from helpers import ragged_window_indices

pytestmark = pytest.mark.gpu

COUNTS = [1, 40, 2, 125, 0, 0, 17, 32, 90, 3, 33, 64, 0, 5]


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("H,hd", [(3, 32), (2, 16), (1, 64), (5, 8), (2, 12)])
def test_qkv_sparse_cuda_equals_the_gathers_through_the_permutations(oracle, H, hd, dtype):
    from sparseswin3d_amd.window_attention import qkv_sparse_cuda
    rng = np.random.default_rng(H * 100 + hd)
    n = 125
    ind = ragged_window_indices(rng, COUNTS, n)
    N, B = len(ind), len(COUNTS)
    qkv = torch.randn(N, 3, H, hd, dtype=torch.float64).to(dtype)
    qkv_d = qkv.cuda().requires_grad_(True)
    q, k_t, v = qkv_sparse_cuda(qkv_d, dev(ind), B, n)
    iqv, sqv, ik, sk = oracle.qkv_sparse_indices(ind, B, n, H, hd)
    assert q.shape == [B, H, n, hd] and k_t.shape == [B, H, hd, n] and v.shape == [B, H, n, hd]
    np.testing.assert_array_equal(q.indices.cpu().numpy(), iqv[:, sqv])
    np.testing.assert_array_equal(v.indices.cpu().numpy(), iqv[:, sqv])
    np.testing.assert_array_equal(k_t.indices.cpu().numpy(), ik[:, sk])
    sqv_t, sk_t = torch.from_numpy(sqv).long(), torch.from_numpy(sk).long()
    want = (qkv[:, 0].reshape(-1)[sqv_t], qkv[:, 1].reshape(-1)[sk_t], qkv[:, 2].reshape(-1)[sqv_t])
    for got, ref in zip((q, k_t, v), want):
        assert got.values.dtype == dtype and torch.equal(got.values.detach().cpu(), ref)
    # gradients: the inverse permutations (what index_add of the gathers gives, without the additions)
    ups = [torch.randn(N * H * hd, dtype=torch.float64).to(dtype) for _ in range(3)]
    torch.autograd.backward([q.values, k_t.values, v.values], [u.cuda() for u in ups])
    parts = [torch.zeros(N * H * hd, dtype=dtype) for _ in range(3)]
    for part, order, up in zip(parts, (sqv_t, sk_t, sqv_t), ups):
        part[order] = up
    ref_grad = torch.stack([p.reshape(N, H * hd) for p in parts], 1)
    assert torch.equal(qkv_d.grad.cpu().reshape(N, 3, H * hd), ref_grad)


@pytest.mark.parametrize("H,hd", [(3, 32), (2, 16)])
def test_operand_to_voxels_equals_permute_and_unsort(oracle, H, hd):
    """The tail of WindowAttention.forward (reference swin3d_base.py:672-675): permute((0, 2, 1, 3)), hash of the voxel
    indices, return_inverse, index_select - against the single copy, forward and backward."""
    from sparseswin3d_amd import custom_ops as ops
    from sparseswin3d_amd.window_attention import SparseTensor, _OperandToVoxels, qkv_sparse_cuda
    rng = np.random.default_rng(7 + hd)
    n = 125
    ind = ragged_window_indices(rng, COUNTS, n)
    N, B = len(ind), len(COUNTS)
    ind_d = dev(ind)
    _, _, v = qkv_sparse_cuda(torch.randn(N, 3, H, hd, device="cuda"), ind_d, B, n)
    val = torch.randn(N * H * hd, device="cuda", requires_grad=True)
    fast = _OperandToVoxels.apply(val, v.operand_map, H, hd)
    out = SparseTensor(v.indices, val, [B, H, n, hd]).permute((0, 2, 1, 3))
    unsort = ops.return_inverse(ops.flatten_indices(ind_d.T.contiguous(), [B, n]), B * n)[0]
    slow = out.values.reshape(N, H * hd).index_select(0, unsort)
    assert torch.equal(fast, slow)
    up = torch.randn(N, H * hd, device="cuda")
    (g_fast,) = torch.autograd.grad(fast, val, up)
    (g_slow,) = torch.autograd.grad(slow, val, up)
    assert torch.equal(g_fast, g_slow)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64])
@pytest.mark.parametrize("hd", [32, 6])
def test_copy_with_a_factor_equals_copy_then_multiply(dtype, hd):
    """``operand_copy(..., scale)`` in both directions: the module's ``q * self.scale`` (swin3d_base.py:660) and its
    gradient, folded into the copies; bit-equal to the copy followed by the tensor multiply."""
    from sparseswin3d_amd import custom_ops as ops
    rng = np.random.default_rng(11)
    ind = ragged_window_indices(rng, [4, 0, 27, 9, 1], 27)
    N, H = len(ind), 3
    scale = hd ** -0.5
    omap = ops.operand_map(dev(ind), 5, 27)
    vox = torch.randn(N, 3 * H * hd, device="cuda", dtype=dtype)
    plain = torch.empty(N * H * hd, device="cuda", dtype=dtype)
    scaled = torch.empty_like(plain)
    ops.operand_copy(vox, H * hd, plain, omap, H, hd, 0, True)
    ops.operand_copy(vox, H * hd, scaled, omap, H, hd, 0, True, scale)
    assert torch.equal(scaled, plain * scale)
    back, back_scaled = torch.zeros_like(vox), torch.zeros_like(vox)
    ops.operand_copy(back, 0, plain, omap, H, hd, 0, False)
    ops.operand_copy(back_scaled, 0, plain, omap, H, hd, 0, False, scale)
    assert torch.equal(back_scaled, back * scale)
    with pytest.raises(RuntimeError, match="only the Q/V order takes a scale"):
        ops.operand_copy(vox, H * hd, scaled, omap, H, hd, 1, True, scale)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64])
@pytest.mark.parametrize("hd", [32, 16, 6])
def test_three_copies_in_one_launch(dtype, hd):
    """``operand_copy_qkv`` against the three single copies it stands for, in both directions, bit for bit."""
    from sparseswin3d_amd import custom_ops as ops
    rng = np.random.default_rng(12)
    counts = [4, 0, 27, 9, 1] + [int(x) for x in rng.integers(0, 28, 40)]
    ind = ragged_window_indices(rng, counts, 27)
    N, H = len(ind), 3
    D = H * hd
    scale = hd ** -0.5
    omap = ops.operand_map(dev(ind), len(counts), 27)
    vox = torch.randn(N, 3 * D, device="cuda", dtype=dtype)
    one = [torch.empty(N * D, device="cuda", dtype=dtype) for _ in range(3)]
    three = [torch.empty_like(t) for t in one]
    ops.operand_copy_qkv(vox, *one, omap, H, hd, True, scale)
    for slot, layout in enumerate((0, 1, 0)):
        ops.operand_copy(vox, slot * D, three[slot], omap, H, hd, layout, True, scale if slot == 0 else 1.0)
        assert torch.equal(one[slot], three[slot]), slot
    back_one, back_three = torch.zeros_like(vox), torch.zeros_like(vox)
    ops.operand_copy_qkv(back_one, *one, omap, H, hd, False, scale)
    for slot, layout in enumerate((0, 1, 0)):
        ops.operand_copy(back_three, slot * D, one[slot], omap, H, hd, layout, False, scale if slot == 0 else 1.0)
    assert torch.equal(back_one, back_three)


def test_strided_token_tensor_and_empty_input():
    from sparseswin3d_amd import custom_ops as ops
    rng = np.random.default_rng(3)
    ind = ragged_window_indices(rng, [4, 0, 9], 27)
    N, H, hd = len(ind), 2, 8
    omap = ops.operand_map(dev(ind), 3, 27)
    wide = torch.randn(N, 5 * H * hd, device="cuda")
    val = torch.empty(N * H * hd, device="cuda")
    ops.operand_copy(wide, 2 * H * hd, val, omap, H, hd, 0, True)             # columns [2D, 3D) of a wider row
    back = torch.zeros_like(wide)
    ops.operand_copy(back, 2 * H * hd, val, omap, H, hd, 0, False)
    assert torch.equal(back[:, 2 * H * hd:3 * H * hd], wide[:, 2 * H * hd:3 * H * hd]) and back[:, :2 * H * hd].abs().sum() == 0
    e_map = ops.operand_map(torch.empty(0, 2, dtype=torch.int32, device="cuda"), 3, 27)
    assert e_map.numel() == 2
