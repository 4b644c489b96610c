"""Host-side logic that needs no GPU: which dense layers the projection kernels take, and that the
layers they do not take fall through to ``nn.Linear`` unchanged."""
import torch


def test_tall_linear_on_cpu_is_the_plain_layer():
    from sparseswin3d_amd.window_attention import tall_linear
    torch.manual_seed(0)
    layer = torch.nn.Linear(96, 288)
    x = torch.randn(50, 96, requires_grad=True)
    y = tall_linear(x, layer)
    ref = layer(x)
    assert torch.equal(y, ref)
    y.sum().backward()
    assert x.grad is not None and layer.weight.grad is not None


def test_mlp_on_cpu_matches_its_definition():
    """linear, activation, dropout, linear, dropout (the block's feed-forward part)."""
    from sparseswin3d_amd.layers import MLP
    torch.manual_seed(1)
    mlp = MLP(32, 128).eval()
    x = torch.randn(7, 32)
    ref = mlp.linear2(torch.nn.functional.gelu(mlp.linear1(x)))
    assert torch.allclose(mlp(x), ref)
    x3 = torch.randn(2, 5, 32)                      # not 2-D: nn.Linear itself
    assert mlp(x3).shape == (2, 5, 32)


def test_split_linear_helpers_decline_what_the_kernels_do_not_take():
    """CPU tensors, 16-bit tensors and empty inputs are left to the library path (None), without loading
    the HIP library."""
    from sparseswin3d_amd import window_attention as wa
    x = torch.randn(40, 96)
    w = torch.randn(288, 96)
    assert wa._split_linear_forward(x, w, None) is None
    assert wa._split_linear_input_grad(torch.randn(40, 288), w) is None
    assert wa._split_linear_weight_grad(torch.randn(40, 288), x, True) == (None, None)


def test_tall_linear_function_under_autocast_backward_does_not_mix_dtypes():
    """fp32 x and W, forward under autocast on a shape the split kernels do not take (48 -> 144, the
    reference's shipped feature_size with enable_amp): the library fallback returns a 16-bit result, and
    the backward, which runs outside autocast, must still multiply operands of one type."""
    from sparseswin3d_amd.window_attention import _TallLinear
    torch.manual_seed(2)
    layer = torch.nn.Linear(48, 144)
    x = torch.randn(33, 48, requires_grad=True)
    with torch.autocast("cpu", dtype=torch.bfloat16):
        y = _TallLinear.apply(x, layer.weight, layer.bias)
    assert y.dtype == torch.bfloat16
    y.float().sum().backward()
    assert x.grad.dtype == torch.float32 and layer.weight.grad.dtype == torch.float32
    ref_x = torch.ones(33, 144) @ layer.weight.detach()
    assert torch.allclose(x.grad, ref_x, rtol=2e-2, atol=2e-2)
    assert torch.allclose(layer.bias.grad, torch.full((144,), 33.0), rtol=1e-2)


def test_tall_linear_leaves_autocast_regions_to_the_layer():
    from sparseswin3d_amd.window_attention import tall_linear
    layer = torch.nn.Linear(48, 144)
    x = torch.randn(9, 48)
    with torch.autocast("cpu", dtype=torch.bfloat16):
        assert tall_linear(x, layer).dtype == torch.bfloat16


def test_sparse_tensor_refuses_shapes_beyond_the_int32_hash():
    # the reference's row-major hash (sparse_swin/ops.cu:264) is int32; past 2^31 cells the order of
    # coalesce / permute is undefined there, here it is an error raised before any kernel runs
    import pytest
    from sparseswin3d_amd.window_attention import SparseTensor
    idx = torch.zeros(4, 2, dtype=torch.int32)
    t = SparseTensor(idx, torch.zeros(2), [216320, 125, 3, 32])
    with pytest.raises(RuntimeError, match="int32 hash"):
        t.coalesce()
    with pytest.raises(RuntimeError, match="int32 hash"):
        t.permute((0, 2, 1, 3))


def test_sparse_tensor_index_matrix_on_demand():
    """A SparseTensor built around a producer of its index matrix calls it once, the first time ``indices`` is read;
    tensors derived from it share the produced matrix; ``index_source`` hands the producer on without calling it."""
    import torch
    from sparseswin3d_amd.window_attention import SparseTensor, _LazyIndices
    calls = []
    matrix = torch.arange(12, dtype=torch.int32).reshape(4, 3)

    def produce():
        calls.append(1)
        return matrix

    t = SparseTensor(_LazyIndices(produce), torch.ones(3), [1, 1, 3, 3], group_counts=torch.tensor([3]),
                     row_positions=torch.tensor([0, 1, 2]))
    scaled = t * 2.0
    assert not calls and isinstance(t.index_source(), _LazyIndices) and scaled.index_source() is t.index_source()
    assert scaled.group_counts is t.group_counts and scaled.row_positions is t.row_positions
    assert t.indices is matrix and calls == [1]
    assert scaled.indices is matrix and t.indices is matrix and calls == [1]
    assert t.index_source() is matrix
    eager = SparseTensor(matrix, torch.ones(3), [1, 1, 3, 3])
    assert eager.indices is matrix and eager.index_source() is matrix and eager.row_positions is None
    eager.indices = matrix + 1
    assert torch.equal(eager.indices, matrix + 1)
