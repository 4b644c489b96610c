"""GPU parity of the projection kernel (fp32 ``x @ W^T + b`` on the bf16 matrix cores with exactly
split operands) against float64 arithmetic on the same fp32 inputs.

The qkv and proj layers of the reference are plain ``nn.Linear`` (sparse_swin/swin3d_base.py:606-610);
the bar is the fp32 one: an error per output below 1e-6 of the sum of the absolute products, which is
what an fp32 library GEMM reaches on the same data.
"""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = 1e-6          # of sum_k |x_ik w_jk|


def _run(lib, _lib, x, w, b):
    N, K = x.shape
    P = w.shape[0]
    assert lib.sswin_tall_linear_supported(P, K)
    y = torch.full((N, P), float("nan"), device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.sswin_tall_linear_forward(C.c_void_p(x.data_ptr()), N, K, C.c_void_p(w.data_ptr()),
                                             C.c_void_p(b.data_ptr() if b is not None else None), P,
                                             C.c_void_p(y.data_ptr()), stream))
    torch.cuda.synchronize()
    return y


@pytest.mark.parametrize("N,K,P,bias", [
    (107500, 96, 288, True),        # qkv of stage 1
    (107500, 96, 96, True),         # proj of stage 1
    (25900, 192, 576, True),        # qkv of stage 2: the row-per-lane kernel
    (6500, 192, 192, False),
    (1, 96, 96, True), (31, 16, 96, False), (33, 32, 192, True), (257, 48, 96, True), (1000, 64, 96, False),
    (4097, 80, 288, True), (129, 112, 96, True), (300, 176, 192, True),
    (107500, 384, 96, True),        # second layer of the block's MLP: four chunks of 96 channels
    (3000, 288, 96, False), (700, 768, 192, True),
])
def test_tall_linear_forward(N, K, P, bias):
    from sparseswin3d_amd import _lib
    lib = _lib.load()
    g = torch.Generator().manual_seed(N * 7 + K + P)
    # values over many binades, so that all three pieces of the split carry bits
    x = (torch.randn(N, K, generator=g) * torch.exp2(torch.randint(-6, 7, (N, K), generator=g).float())).cuda()
    w = (torch.randn(P, K, generator=g) * 0.1).cuda()
    b = torch.randn(P, generator=g).cuda() if bias else None
    y = _run(lib, _lib, x, w, b)
    ref = x.double() @ w.double().T
    if bias:
        ref = ref + b.double()
    scale = x.double().abs() @ w.double().abs().T + (b.double().abs() if bias else 0.0)
    err = ((y.double() - ref).abs() / scale).max().item()
    assert not torch.isnan(y).any()
    assert err < TOL, err


def test_tall_linear_exact_cases():
    """Operands that are sums of three bf16 pieces with few products per output: the result is exact,
    so a dropped or doubled piece product shows as a wrong bit."""
    from sparseswin3d_amd import _lib
    lib = _lib.load()
    N, K, P = 200, 32, 96
    x = torch.zeros(N, K)
    w = torch.zeros(P, K)
    rng = np.random.default_rng(3)
    # one nonzero per row of x and per row of w: y[i, j] = x[i, k_i] * w[j, k_i] or 0
    xi = rng.integers(0, K, N)
    x[torch.arange(N), torch.from_numpy(xi)] = torch.from_numpy(rng.integers(1, 2 ** 12, N).astype(np.float32)) / 64
    wj = rng.integers(0, K, P)
    w[torch.arange(P), torch.from_numpy(wj)] = torch.from_numpy(rng.integers(1, 2 ** 12, P).astype(np.float32)) / 128
    y = _run(lib, _lib, x.cuda(), w.cuda(), None).cpu()
    ref = (x.double() @ w.double().T).float()           # 12-bit x 12-bit integers: exact in fp32
    torch.testing.assert_close(y, ref, rtol=0, atol=0)


def test_tall_linear_rejects_unsupported_shapes():
    from sparseswin3d_amd import _lib
    lib = _lib.load()
    assert lib.sswin_tall_linear_supported(288, 96) == 1
    assert lib.sswin_tall_linear_supported(100, 96) == 0             # columns not a multiple of 96
    assert lib.sswin_tall_linear_supported(96, 100) == 0             # channels not a multiple of 16
    assert lib.sswin_tall_linear_supported(96, 384) == 1             # chunks of 96 channels
    assert lib.sswin_tall_linear_supported(96, 208) == 0             # above 192: multiples of 96 only
    assert lib.sswin_tall_linear_supported(96, 864) == 0             # too many channels
    x = torch.zeros(8, 100, device="cuda")
    w = torch.zeros(96, 100, device="cuda")
    y = torch.zeros(8, 96, device="cuda")
    rc = lib.sswin_tall_linear_forward(C.c_void_p(x.data_ptr()), 8, 100, C.c_void_p(w.data_ptr()), None, 96,
                                       C.c_void_p(y.data_ptr()), None)
    assert rc != 0
    with pytest.raises(RuntimeError, match="input channels"):
        _lib.check(rc)


@pytest.mark.parametrize("N,K,P,bias", [
    (107500, 96, 288, True), (107500, 96, 96, True), (1, 96, 96, True), (63, 32, 96, False), (65, 64, 192, True),
    (1000, 96, 96, True), (4099, 96, 288, False), (20000, 32, 288, True),
    (25900, 192, 576, True),        # qkv of stage 2: two passes of 96 columns of x
    (3000, 288, 96, True), (130, 384, 192, False),
])
def test_tall_linear_weight_grad(N, K, P, bias):
    """dW = dY^T X and db = column sums of dY against float64 on the same fp32 inputs; the same bits on
    a second call (partial sums are added in a fixed order)."""
    from sparseswin3d_amd import _lib
    lib = _lib.load()
    g = torch.Generator().manual_seed(N + 3 * K + P)
    x = (torch.randn(N, K, generator=g) * torch.exp2(torch.randint(-4, 5, (N, K), generator=g).float())).cuda()
    dy = (torch.randn(N, P, generator=g) * torch.exp2(torch.randint(-4, 5, (N, P), generator=g).float())).cuda()
    nb = int(lib.sswin_tall_linear_weight_grad_workspace_bytes(N, P, K))
    assert nb > 0
    ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for _ in range(2):
        dw = torch.full((P, K), float("nan"), device="cuda")
        db = torch.full((P,), float("nan"), device="cuda") if bias else None
        _lib.check(lib.sswin_tall_linear_weight_grad(C.c_void_p(dy.data_ptr()), C.c_void_p(x.data_ptr()), N, P, K,
                                                     C.c_void_p(dw.data_ptr()),
                                                     C.c_void_p(db.data_ptr() if bias else None),
                                                     C.c_void_p(ws.data_ptr()), nb, stream))
        torch.cuda.synchronize()
        outs.append((dw, db))
    dw, db = outs[0]
    assert torch.equal(dw, outs[1][0])
    ref = dy.double().T @ x.double()
    scale = dy.double().abs().T @ x.double().abs()
    assert ((dw.double() - ref).abs() / scale).max().item() < TOL
    if bias:
        assert torch.equal(db, outs[1][1])
        refb = dy.double().sum(0)
        assert ((db.double() - refb).abs() / dy.double().abs().sum(0)).max().item() < TOL


@pytest.mark.parametrize("N,P,K", [
    (107500, 288, 96),              # qkv of stage 1
    (25900, 576, 192),              # qkv of stage 2
    (107500, 96, 96), (1, 288, 96), (31, 192, 96), (257, 96, 192), (4097, 288, 96), (300, 384, 288),
])
def test_tall_linear_input_grad(N, P, K):
    """dX = dY W against float64 on the same fp32 inputs."""
    from sparseswin3d_amd import _lib
    lib = _lib.load()
    assert lib.sswin_tall_linear_input_grad_supported(P, K)
    g = torch.Generator().manual_seed(N + P + 5 * K)
    dy = (torch.randn(N, P, generator=g) * torch.exp2(torch.randint(-6, 7, (N, P), generator=g).float())).cuda()
    w = (torch.randn(P, K, generator=g) * 0.1).cuda()
    dx = torch.full((N, K), float("nan"), device="cuda")
    _lib.check(lib.sswin_tall_linear_input_grad(C.c_void_p(dy.data_ptr()), N, P, C.c_void_p(w.data_ptr()), K,
                                                C.c_void_p(dx.data_ptr()),
                                                C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    ref = dy.double() @ w.double()
    scale = dy.double().abs() @ w.double().abs()
    assert not torch.isnan(dx).any()
    assert ((dx.double() - ref).abs() / scale).max().item() < TOL


def test_tall_linear_input_grad_unsupported_shapes():
    from sparseswin3d_amd import _lib
    lib = _lib.load()
    assert lib.sswin_tall_linear_input_grad_supported(100, 96) == 0
    assert lib.sswin_tall_linear_input_grad_supported(96, 64) == 0
    t = torch.zeros(64, 96, device="cuda")
    rc = lib.sswin_tall_linear_input_grad(C.c_void_p(t.data_ptr()), 64, 96, C.c_void_p(t.data_ptr()), 64,
                                          C.c_void_p(t.data_ptr()), None)
    assert rc != 0
    with pytest.raises(RuntimeError, match="input channels"):
        _lib.check(rc)


def test_tall_linear_weight_grad_unsupported_shapes():
    from sparseswin3d_amd import _lib
    lib = _lib.load()
    assert lib.sswin_tall_linear_weight_grad_workspace_bytes(1000, 100, 96) == 0
    assert lib.sswin_tall_linear_weight_grad_workspace_bytes(1000, 96, 160) == 0
    assert lib.sswin_tall_linear_weight_grad_workspace_bytes(1000, 96, 864) == 0
    assert lib.sswin_tall_linear_weight_grad_workspace_bytes(1000, 96, 48) == 0
    assert lib.sswin_tall_linear_weight_grad_workspace_bytes(0, 96, 96) == 0
    t = torch.zeros(64, 96, device="cuda")
    rc = lib.sswin_tall_linear_weight_grad(C.c_void_p(t.data_ptr()), C.c_void_p(t.data_ptr()), 64, 96, 48,
                                           C.c_void_p(t.data_ptr()), None, C.c_void_p(t.data_ptr()), 1024, None)
    assert rc != 0
    with pytest.raises(RuntimeError, match="input channels"):
        _lib.check(rc)


def test_module_projection_matches_library_gemm():
    """tall_linear() of the module (forward and all three gradients through the kernels) against
    nn.Linear in float64."""
    from sparseswin3d_amd.window_attention import tall_linear
    torch.manual_seed(5)
    layer = torch.nn.Linear(96, 288).cuda()
    x = torch.randn(5000, 96, device="cuda", requires_grad=True)
    y = tall_linear(x, layer)
    g = torch.randn_like(y)
    y.backward(g)
    ref_layer = torch.nn.Linear(96, 288).double().cuda()
    ref_layer.load_state_dict({k: v.double() for k, v in layer.state_dict().items()})
    xr = x.detach().double().requires_grad_(True)
    yr = ref_layer(xr)
    yr.backward(g.double())
    torch.testing.assert_close(y.double(), yr, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(x.grad.double(), xr.grad, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(layer.weight.grad.double(), ref_layer.weight.grad, rtol=1e-5, atol=2e-4)
    torch.testing.assert_close(layer.bias.grad.double(), ref_layer.bias.grad, rtol=1e-5, atol=2e-4)
