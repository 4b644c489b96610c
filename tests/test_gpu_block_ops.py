"""GPU parity of the window-blocked products, transposes and the sparse softmax against the
CPU oracle.  Indices and offsets: bit-exact.  Values: fp32 within rel 1e-5 of the fp64 oracle,
fp16/bf16 within rel 2e-2; a product's error is measured against sum_k |a_ik b_kj| of its element, a softmax
entry's against its own value plus the largest value of its row (helpers.close)."""
import zlib

import numpy as np
import pytest
import torch

from helpers import softmax_bwd_mag, close, product_mag, qkv_operands, ragged_window_indices, random_window_indices

pytestmark = pytest.mark.gpu

RTOL = {torch.float32: 1e-5, torch.float64: 1e-12, torch.float16: 2e-2, torch.bfloat16: 2e-2}


def seed_of(*parts):
    return zlib.crc32(repr(parts).encode()) % 100000


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t if dtype is None else t.to(dtype)


def host(t):
    return t.detach().to(torch.float64).cpu().numpy() if t.is_floating_point() else t.cpu().numpy()


@pytest.fixture(scope="module")
def ops():
    from sparseswin3d_amd import custom_ops
    return custom_ops


# window occupancy mixes: tiny, around the 32 / 64 tile edges, full 5^3 windows, empty slots
MIXES = {
    "tiny": [1, 2, 3, 1, 5, 4],
    "edges": [31, 32, 33, 0, 63, 64, 65, 1],
    "full": [125, 124, 100, 7],
    "mixed": [1, 40, 2, 125, 0, 0, 17, 32, 90, 3, 3, 3, 3, 64],
    "wide": [227, 130, 60, 200, 33],      # windows of 7^3 positions: up to 64 blocks of 32 x 32 per group
}
POSITIONS = {"wide": 343}


def build(oracle, mix, H, hd, seed, n=None):
    rng = np.random.default_rng(seed)
    n = POSITIONS.get(mix, 125) if n is None else n
    counts = MIXES[mix]
    ind = ragged_window_indices(rng, counts, n)
    B = len(counts)
    return B, n, qkv_operands(oracle, ind, B, n, H, hd, rng, dtype=np.float64)


def run_forward(ops, oracle, d, dtype):
    """q_k -> softmax -> qk_v on the GPU and in the fp64 oracle; returns both sides."""
    q, kt, v = (dev(d[k], dtype) for k in ("q", "kt", "v"))
    qi, ki = dev(d["qi"]), dev(d["ki"])
    s_idx, s_val, s_shape, c1 = ops.matmul_cuda_naive(q, qi, d["q_shape"], kt, ki, d["k_shape"], "q_k")
    # oracle consumes the same (rounded) inputs in fp64
    q64, kt64, v64 = host(q), host(kt), host(v)
    r_idx, r_val, r_shape, r_c = oracle.matmul_cuda_naive(q64, d["qi"], d["q_shape"], kt64, d["ki"], d["k_shape"], "q_k")
    r_mag = product_mag(oracle, "matmul_cuda_naive", q64, d["qi"], d["q_shape"], kt64, d["ki"], d["k_shape"], "q_k")
    return dict(q=q, kt=kt, v=v, qi=qi, ki=ki, s_idx=s_idx, s_val=s_val, s_shape=s_shape, c1=c1,
                q64=q64, kt64=kt64, v64=v64, r_idx=r_idx, r_val=r_val, r_shape=r_shape, r_c=r_c, r_mag=r_mag)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mix,H,hd", [("tiny", 2, 32), ("edges", 3, 32), ("full", 1, 32), ("mixed", 3, 32),
                                      ("mixed", 2, 16), ("edges", 1, 64), ("wide", 2, 16), ("wide", 1, 48)])
def test_q_k_and_qk_v(ops, oracle, mix, H, hd, dtype):
    B, n, d = build(oracle, mix, H, hd, seed=seed_of(mix, H, hd))
    f = run_forward(ops, oracle, d, dtype)
    # --- q_k
    assert f["s_idx"].dtype == torch.int32 and f["c1"].dtype == torch.int32
    assert f["s_shape"] == f["r_shape"] == [B, H, n, n]
    np.testing.assert_array_equal(host(f["c1"]), f["r_c"])
    np.testing.assert_array_equal(host(f["s_idx"]), f["r_idx"])
    close(host(f["s_val"]), f["r_val"], RTOL[dtype], "q_k values", mag=f["r_mag"])
    # --- qk_v, fed with the oracle's attention so both sides multiply the same numbers
    rows = oracle.unique_consecutive_indices(oracle.flatten_indices(f["r_idx"][:3], f["r_shape"][:3]))
    p64 = oracle.softmax_last_dim_forward(rows, f["r_val"])
    p = dev(p64, dtype)
    o_idx, o_val, o_shape, c2 = ops.matmul_cuda_naive(p, f["s_idx"], f["s_shape"], f["v"], f["qi"], d["q_shape"], "qk_v")
    ro_idx, ro_val, ro_shape, ro_c = oracle.matmul_cuda_naive(host(p), f["r_idx"], f["r_shape"], f["v64"], d["qi"],
                                                             d["q_shape"], "qk_v")
    assert o_shape == ro_shape == [B, H, n, hd]
    np.testing.assert_array_equal(host(c2), ro_c)
    np.testing.assert_array_equal(host(o_idx), ro_idx)
    o_mag = product_mag(oracle, "matmul_cuda_naive", host(p), f["r_idx"], f["r_shape"], f["v64"], d["qi"], d["q_shape"], "qk_v")
    close(host(o_val), ro_val, RTOL[dtype], "qk_v values", mag=o_mag)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16])
@pytest.mark.parametrize("mix,H,hd", [("tiny", 2, 32), ("edges", 2, 32), ("mixed", 3, 32), ("full", 1, 32),
                                      ("mixed", 1, 16), ("edges", 1, 64), ("wide", 2, 16), ("wide", 1, 48)])
@pytest.mark.parametrize("kind", ["rc_cr", "rr_rc", "cr_rr"])
def test_matmul_grad(ops, oracle, mix, H, hd, kind, dtype):
    rng = np.random.default_rng(seed_of(mix, H, hd, kind))
    c = np.repeat(np.array([x for x in MIXES[mix] if x > 0], np.int32), H)
    mat = int((c.astype(np.int64) * hd).sum())
    sq = int((c.astype(np.int64) ** 2).sum())
    n1, n2 = {"rc_cr": (mat, mat), "rr_rc": (sq, mat), "cr_rr": (mat, sq)}[kind]
    m1 = dev(rng.standard_normal(n1), dtype)
    m2 = dev(rng.standard_normal(n2), dtype)
    out = ops.matmul_grad_cuda_naive(m1, m2, dev(c), hd, kind)
    ref = oracle.matmul_grad_cuda_naive(host(m1), host(m2), c, hd, kind)
    assert out.dtype == dtype
    close(host(out), ref, RTOL[dtype], kind, mag=product_mag(oracle, "matmul_grad_cuda_naive", host(m1), host(m2), c, hd, kind))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16])
@pytest.mark.parametrize("mix,hd", [("tiny", 32), ("edges", 32), ("mixed", 32), ("full", 16)])
@pytest.mark.parametrize("kind", ["rc", "rr"])
def test_qkv_transpose(ops, oracle, mix, hd, kind, dtype):
    rng = np.random.default_rng(len(mix) + hd)
    c = np.array([x for x in MIXES[mix] if x > 0], np.int32)
    total = int((c.astype(np.int64) * (hd if kind == "rc" else c)).sum())
    m = dev(rng.standard_normal(total), dtype)
    out = ops.qkv_transpose(m, dev(c), hd, kind)
    ref = oracle.qkv_transpose(host(m), c, hd, kind)
    np.testing.assert_array_equal(host(out), ref)          # pure data movement: exact


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16])
@pytest.mark.parametrize("mix,H,hd", [("tiny", 2, 32), ("edges", 2, 32), ("mixed", 3, 32), ("full", 1, 32),
                                      ("mixed", 1, 16), ("edges", 1, 64), ("wide", 2, 16), ("wide", 1, 48)])
@pytest.mark.parametrize("kind", ["tr_rc", "tc_rr"])
def test_matmul_grad_from_untransposed_operands(ops, oracle, mix, H, hd, kind, dtype):
    """The second gradient of each product read from the operands as the forward pass left them: equal, bit for bit,
    to the reference's composition of two transposes and a product (swin3d_base.py:123-125, 131-133), and within the
    product tolerance of the oracle's composition in fp64."""
    rng = np.random.default_rng(seed_of(mix, H, hd, kind))
    c = np.repeat(np.array([x for x in MIXES[mix] if x > 0], np.int32), H)
    mat = int((c.astype(np.int64) * hd).sum())
    sq = int((c.astype(np.int64) ** 2).sum())
    n1, n2, t1, t2, prod = {"tr_rc": (sq, mat, "rr", "rc", "rr_rc"), "tc_rr": (mat, sq, "rc", "rr", "cr_rr")}[kind]
    m1 = dev(rng.standard_normal(n1), dtype)
    m2 = dev(rng.standard_normal(n2), dtype)
    cd = dev(c)
    out = ops.matmul_grad_untransposed(m1, m2, cd, hd, kind)
    composed = ops.matmul_grad_cuda_naive(ops.qkv_transpose(m1, cd, hd, t1), ops.qkv_transpose(m2, cd, hd, t2), cd, hd, prod)
    assert out.dtype == dtype and torch.equal(out, composed)
    r1, r2 = oracle.qkv_transpose(host(m1), c, hd, t1), oracle.qkv_transpose(host(m2), c, hd, t2)
    ref = oracle.matmul_grad_cuda_naive(r1, r2, c, hd, prod)
    close(host(out), ref, RTOL[dtype], kind, mag=product_mag(oracle, "matmul_grad_cuda_naive", r1, r2, c, hd, prod))


def test_backward_identities_through_transposes(ops, oracle):
    """The backward of 'q_k' as the reference's autograd Function composes it
    (sparse_swin/swin3d_base.py:119-126) against plain per-group matrix algebra in fp64."""
    B, n, d = build(oracle, "mixed", 2, 32, seed=9)
    f = run_forward(ops, oracle, d, torch.float32)
    rng = np.random.default_rng(1)
    g_np = rng.standard_normal(f["s_val"].numel()).astype(np.float32)
    g = dev(g_np)
    c, C_ = f["c1"], 32
    dq = ops.matmul_grad_cuda_naive(g, f["kt"], c, C_, "rr_rc")
    qt = ops.qkv_transpose(f["q"], c, C_, "rc")
    gt = ops.qkv_transpose(g, c, C_, "rr")
    dkt = ops.matmul_grad_cuda_naive(qt, gt, c, C_, "cr_rr")
    # plain algebra per group
    cs = f["r_c"]
    q64, kt64 = f["q64"], f["kt64"]
    dq_ref, dkt_ref, dq_mag, dkt_mag = [], [], [], []
    po = mo = 0
    for cg in cs:
        cg = int(cg)
        Q = q64[mo:mo + cg * C_].reshape(cg, C_)
        Kt = kt64[mo:mo + cg * C_].reshape(C_, cg)
        dS = g_np[po:po + cg * cg].astype(np.float64).reshape(cg, cg)
        dq_ref.append((dS @ Kt.T).ravel())
        dkt_ref.append((Q.T @ dS).ravel())
        dq_mag.append((np.abs(dS) @ np.abs(Kt.T)).ravel())
        dkt_mag.append((np.abs(Q.T) @ np.abs(dS)).ravel())
        po += cg * cg
        mo += cg * C_
    close(host(dq), np.concatenate(dq_ref), 1e-5, "dQ", mag=np.concatenate(dq_mag))
    close(host(dkt), np.concatenate(dkt_ref), 1e-5, "dK^T", mag=np.concatenate(dkt_mag))
    assert torch.equal(ops.matmul_grad_untransposed(f["q"], g, c, C_, "tc_rr"), dkt)


# ------------------------------------------------------------------------------------------ softmax
def _rows(lengths):
    return np.repeat(np.arange(len(lengths)), lengths).astype(np.int32)


ROW_MIXES = {
    "short": [1, 2, 3, 16, 17, 31, 32, 33, 1, 1],
    "windows": [125] * 40 + [7] * 30 + [64] * 9,
    "cross_tile": [2047, 1, 2048, 2049, 5000, 3, 4096 + 17],
    "single_long": [10_000],
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("mix", list(ROW_MIXES))
def test_softmax_forward_backward(ops, oracle, mix, dtype):
    rng = np.random.default_rng(len(mix))
    rows = _rows(ROW_MIXES[mix])
    v = rng.standard_normal(len(rows)) * 3.0
    v[rng.random(len(rows)) < 0.2] -= 100.0                    # masked entries of shifted windows
    v64 = host(dev(v, dtype))
    y = ops.softmax_last_dim_forward(dev(rows), dev(v, dtype))
    y_ref = oracle.softmax_last_dim_forward(rows, v64)
    close(host(y), y_ref, RTOL[dtype] if dtype == torch.float64 else 1e-5, "softmax fwd", seg=rows)
    g = rng.standard_normal(len(rows))
    gx = ops.softmax_last_dim_backward(dev(rows), y, dev(g, dtype))
    gx_ref = oracle.softmax_last_dim_backward(rows, host(y), host(dev(g, dtype)))
    close(host(gx), gx_ref, RTOL[dtype] if dtype == torch.float64 else 1e-5, "softmax bwd",
          mag=softmax_bwd_mag(rows, host(y), host(dev(g, dtype))))


def test_softmax_all_negative_rows_keep_zero_max(ops, oracle):
    # rows whose maximum is below zero: the subtracted maximum is 0, not the row maximum
    rows = _rows([4, 4, 1])
    v = np.array([-1, -2, -3, -4, -30, -31, -32, -33, -5], np.float32)
    y = ops.softmax_last_dim_forward(dev(rows), dev(v)).cpu().numpy().astype(np.float64)
    ref = oracle.softmax_last_dim_forward(rows, v.astype(np.float64))
    close(y, ref, 1e-5, "negative rows", seg=rows)
    assert abs(y[4:8].sum() - 1.0) > 1e-6          # the 1e-8 term is visible for exp(-30)-sized sums


def test_softmax_views_inside_an_allocation(ops, oracle):
    """Row ids and values that start 4 bytes into their allocations (the kernels use 16-byte moves)."""
    rng = np.random.default_rng(21)
    rows = _rows([5, 1, 2047, 40, 3000])
    v = rng.standard_normal(len(rows) + 1).astype(np.float32)
    rows_d = dev(np.concatenate([[0], rows]).astype(np.int32))[1:]
    y = ops.softmax_last_dim_forward(rows_d, dev(v)[1:])
    close(host(y), oracle.softmax_last_dim_forward(rows, v[1:].astype(np.float64)), 1e-5, "views fwd", seg=rows)
    g = rng.standard_normal(len(rows) + 1).astype(np.float32)
    gx = ops.softmax_last_dim_backward(rows_d, y, dev(g)[1:])
    close(host(gx), oracle.softmax_last_dim_backward(rows, host(y), g[1:].astype(np.float64)), 1e-5, "views bwd",
          mag=softmax_bwd_mag(rows, host(y), g[1:]))


def test_softmax_deterministic(ops):
    rng = np.random.default_rng(0)
    rows = dev(_rows([37] * 5000))
    v = dev(rng.standard_normal(37 * 5000).astype(np.float32))
    a = ops.softmax_last_dim_forward(rows, v)
    b = ops.softmax_last_dim_forward(rows, v)
    assert torch.equal(a, b)


# ------------------------------------------------------------------------------------------ errors
def test_error_behaviour(ops, oracle):
    B, n, d = build(oracle, "tiny", 1, 32, seed=3)
    q, kt = dev(d["q"], torch.float32), dev(d["kt"], torch.float32)
    qi, ki = dev(d["qi"]), dev(d["ki"])
    with pytest.raises(RuntimeError, match="Invalid mul_type"):
        ops.matmul_cuda_naive(q, qi, d["q_shape"], kt, ki, d["k_shape"], "k_q")
    with pytest.raises(RuntimeError, match="not int32"):
        ops.matmul_cuda_naive(q, qi.long(), d["q_shape"], kt, ki.long(), d["k_shape"], "q_k")
    with pytest.raises(RuntimeError, match="does not match"):
        ops.matmul_cuda_naive(q, qi, d["q_shape"], kt.double(), ki, d["k_shape"], "q_k")
    with pytest.raises(RuntimeError, match="Invalid shapes"):
        ops.matmul_cuda_naive(q, qi, d["q_shape"], kt, ki, [B, 1, 16, n], "q_k")
    c = dev(np.array([1, 2], np.int32))
    with pytest.raises(RuntimeError, match="Invalid mul_type"):
        ops.matmul_grad_cuda_naive(q, kt, c, 32, "rc_rc")
    with pytest.raises(RuntimeError, match="Invalid mul_type"):
        ops.qkv_transpose(q, c, 32, "cr")


def test_empty_operands(ops):
    e_idx = torch.empty((4, 0), dtype=torch.int32, device="cuda")
    e_val = torch.empty(0, dtype=torch.float32, device="cuda")
    idx, val, shape, c = ops.matmul_cuda_naive(e_val, e_idx, [4, 2, 125, 32], e_val, e_idx, [4, 2, 32, 125], "q_k")
    assert idx.shape == (4, 0) and val.numel() == 0 and c.numel() == 0 and shape == [4, 2, 125, 125]
    assert ops.softmax_last_dim_forward(torch.empty(0, dtype=torch.int32, device="cuda"), e_val).numel() == 0


@pytest.mark.parametrize("mix", sorted(MIXES))
@pytest.mark.parametrize("H,hd", [(3, 32), (2, 16), (1, 64)])
def test_permute_of_an_attention_output_without_a_sort(ops, oracle, mix, H, hd):
    """SparseTensor.permute((0, 2, 1, 3)) (reference swin3d_base.py:47-59) on a 'qk_v' product: the order
    derived from the group structure equals the stable sort of the permuted hash, bit for bit."""
    from sparseswin3d_amd.window_attention import SparseTensor
    B, n, d = build(oracle, mix, H, hd, seed_of("permute", mix, H, hd))
    idx = dev(d["qi"])                                       # coalesced (window, head, pos, channel)
    val = dev(np.arange(idx.shape[1], dtype=np.float32))
    shape = [B, H, n, hd]
    order = ops.permute_heads_order(idx, shape)
    assert order is not None
    perm = d["qi"][[0, 2, 1, 3]]
    want = oracle.sort_indices(oracle.flatten_indices(np.ascontiguousarray(perm), [B, n, H, hd]))
    np.testing.assert_array_equal(host(order), want)
    out = SparseTensor(idx, val, shape).permute((0, 2, 1, 3))
    np.testing.assert_array_equal(host(out.indices), perm[:, want])
    np.testing.assert_array_equal(host(out.values), want.astype(np.float64))
    assert out.shape == [B, n, H, hd]


def test_permute_falls_back_to_the_sort_when_heads_differ(ops, oracle):
    """Heads of one window with different positions: the structure check fails on the device and permute
    sorts, as the reference always does."""
    from sparseswin3d_amd.window_attention import SparseTensor
    # window 0: head 0 holds positions {1, 4}, head 1 holds {1, 5}; window 2: one head only
    rows = [(0, 0, 1), (0, 0, 4), (0, 1, 1), (0, 1, 5), (2, 0, 3)]
    hd = 4
    idx = np.array([[w, h, p, ch] for (w, h, p) in rows for ch in range(hd)], np.int32).T.copy()
    shape = [3, 2, 8, hd]
    assert ops.permute_heads_order(dev(idx), shape) is None
    out = SparseTensor(dev(idx), dev(np.arange(idx.shape[1], dtype=np.float32)), shape).permute((0, 2, 1, 3))
    perm = idx[[0, 2, 1, 3]]
    want = oracle.sort_indices(oracle.flatten_indices(np.ascontiguousarray(perm), [3, 8, 2, hd]))
    np.testing.assert_array_equal(host(out.indices), perm[:, want])
    np.testing.assert_array_equal(host(out.values), want.astype(np.float64))


@pytest.mark.parametrize("what", ["positions", "heads", "windows"])
def test_permute_sorts_a_tensor_that_is_not_coalesced(ops, oracle, what):
    """Equal positions in every head of a window are not enough for the order to follow from the group structure: the
    tensor must be coalesced too.  Positions out of order inside a group, heads out of order inside a window, or windows
    out of order fail the device check, and permute sorts, as the reference always does."""
    from sparseswin3d_amd.window_attention import SparseTensor
    hd = 4
    rows = {"positions": [(0, 0, 4), (0, 0, 1), (0, 1, 4), (0, 1, 1), (2, 0, 3), (2, 1, 3)],
            "heads": [(0, 1, 1), (0, 1, 4), (0, 0, 1), (0, 0, 4), (2, 0, 3), (2, 1, 3)],
            "windows": [(2, 0, 3), (2, 1, 3), (0, 0, 1), (0, 0, 4), (0, 1, 1), (0, 1, 4)]}[what]
    idx = np.array([[w, h, p, ch] for (w, h, p) in rows for ch in range(hd)], np.int32).T.copy()
    shape = [3, 2, 8, hd]
    assert ops.permute_heads_order(dev(idx), shape) is None
    out = SparseTensor(dev(idx), dev(np.arange(idx.shape[1], dtype=np.float32)), shape).permute((0, 2, 1, 3))
    perm = idx[[0, 2, 1, 3]]
    want = oracle.sort_indices(oracle.flatten_indices(np.ascontiguousarray(perm), [3, 8, 2, hd]))
    np.testing.assert_array_equal(host(out.indices), perm[:, want])
    np.testing.assert_array_equal(host(out.values), want.astype(np.float64))


@pytest.mark.parametrize("mix", sorted(MIXES))
@pytest.mark.parametrize("H,hd", [(3, 32), (2, 16)])
def test_softmax_rows_from_the_group_sizes(ops, oracle, mix, H, hd):
    """Row ids of the softmax over a 'q_k' product (reference swin3d_base.py:140-150: hash of the first three index rows,
    then unique_consecutive) from the group sizes alone: bit-exact against the oracle's hash + unique_consecutive, and
    softmax_last_dim gives the same result either way."""
    from sparseswin3d_amd.window_attention import SparseTensor, softmax_last_dim
    B, n, d = build(oracle, mix, H, hd, seed_of("rows", mix, H, hd))
    f = run_forward(ops, oracle, d, torch.float32)
    want = oracle.unique_consecutive_indices(oracle.flatten_indices(f["r_idx"][:3], f["r_shape"][:3]))
    rows = ops.softmax_rows_from_counts(f["c1"], f["s_val"].numel())
    np.testing.assert_array_equal(host(rows), want)
    with_counts = softmax_last_dim(SparseTensor(f["s_idx"], f["s_val"], f["s_shape"], f["c1"]))
    generic = softmax_last_dim(SparseTensor(f["s_idx"], f["s_val"], f["s_shape"]))
    assert torch.equal(with_counts.values, generic.values)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16])
@pytest.mark.parametrize("mix,H,hd", [("mixed", 3, 32), ("edges", 2, 16)])
def test_index_matrices_written_on_demand(ops, oracle, mix, H, hd, dtype):
    """spspmm_block_naive leaves the product's [4, nnz] index matrix unwritten until it is read: the attention
    (q_k -> bias -> softmax -> qk_v) goes through without it, and reading it afterwards gives the matrix the
    operator returns.  The library's values-only and indices-only halves equal the full call bit for bit."""
    from sparseswin3d_amd.window_attention import SparseTensor, _LazyIndices, softmax_last_dim, spspmm_block_naive
    B, n, d = build(oracle, mix, H, hd, seed=seed_of("lazy", mix, H, hd))
    f = run_forward(ops, oracle, d, dtype)
    q = SparseTensor(f["qi"], f["q"], d["q_shape"])
    kt = SparseTensor(_LazyIndices(lambda: f["ki"]), f["kt"], d["k_shape"])        # K^T's matrix: never needed
    v = SparseTensor(f["qi"], f["v"], d["q_shape"])
    s = spspmm_block_naive(q * 0.5, kt, "q_k")
    p = softmax_last_dim(s)
    o = spspmm_block_naive(p, v, "qk_v")
    for t in (kt, s, p, o):
        assert isinstance(t._idx, _LazyIndices) and t._idx.value is None
    assert torch.equal(s.row_positions, f["qi"][2, ::hd])
    full_idx, full_val, _, _ = ops.matmul_cuda_naive(f["q"] * 0.5, f["qi"], d["q_shape"], f["kt"], f["ki"], d["k_shape"], "q_k")
    assert torch.equal(s.values, full_val)
    assert torch.equal(s.indices, full_idx) and p.indices is s.indices             # one matrix, written once
    o_idx, o_val, _, _ = ops.matmul_cuda_naive(p.values.to(dtype), full_idx, s.shape, f["v"], f["qi"], d["q_shape"], "qk_v")
    assert torch.equal(o.values, o_val) and torch.equal(o.indices, o_idx)
    np.testing.assert_array_equal(host(o.indices), oracle.matmul_cuda_naive(
        host(p.values), f["r_idx"], f["r_shape"], f["v64"], d["qi"], d["q_shape"], "qk_v")[0])
    # the two halves through the operator module
    only_idx, none_val, _, c = ops.block_product(None, f["qi"], d["q_shape"], None, None, d["k_shape"], "q_k", values=False)
    none_idx, only_val, _, _ = ops.block_product(f["q"] * 0.5, f["qi"], d["q_shape"], f["kt"], None, d["k_shape"], "q_k",
                                                 indices=False)
    assert none_val is None and none_idx is None
    assert torch.equal(only_idx, full_idx) and torch.equal(only_val, full_val) and torch.equal(c, f["c1"])
    with pytest.raises(RuntimeError, match="nothing asked for"):
        ops.block_product(f["q"], f["qi"], d["q_shape"], f["kt"], f["ki"], d["k_shape"], "q_k", values=False, indices=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window,mix,use_mask", [((5, 5, 5), "mixed", True), ((5, 5, 5), "edges", False), ((7, 7, 7), "full", True)])
def test_table_bias_and_mask_in_one_pass(ops, oracle, window, mix, use_mask, dtype):
    """sp_add_rpb + sp_add_mask of the reference (swin3d_base.py:557-581) against the single pass over a 'q_k' product:
    same values bit for bit (the reference's two roundings are kept), same gradient of the values, table gradient
    within fp32 rel 1e-5 of autograd's index_add (another summation order)."""
    from sparseswin3d_amd.window_attention import (SparseTensor, WindowAttentionSparse, sp_add_mask, sp_add_rpb,
                                                   sp_add_table_bias_and_mask)
    H, hd = 3, 16
    n = window[0] * window[1] * window[2]
    rng = np.random.default_rng(seed_of("bias", window, mix))
    counts = MIXES[mix] + ([300, 129] if n > 125 else [])
    ind = ragged_window_indices(rng, counts, n)
    B = len(counts)
    d = qkv_operands(oracle, ind, B, n, H, hd, rng, dtype=np.float64)
    f = run_forward(ops, oracle, d, torch.float32)
    attn_mod = WindowAttentionSparse(H * hd, H, window, qkv_bias=False).cuda()
    with torch.no_grad():
        attn_mod.relative_position_bias_table.normal_(0, 0.5)
    mask = dev(rng.integers(0, 27, size=(5, n)).astype(np.int8)) if use_mask else None
    vals = f["s_val"].to(dtype)
    up = torch.randn_like(vals)

    v1 = vals.clone().requires_grad_(True)
    fast = sp_add_table_bias_and_mask(SparseTensor(f["s_idx"], v1, f["s_shape"], f["c1"]),
                                      attn_mod.relative_position_bias_table, attn_mod._table_index(n), mask)
    assert fast is not None
    fast.values.backward(up)
    g_table_fast = attn_mod.relative_position_bias_table.grad.clone()
    attn_mod.relative_position_bias_table.grad = None

    v2 = vals.clone().requires_grad_(True)
    ref = sp_add_rpb(SparseTensor(f["s_idx"], v2, f["s_shape"]), attn_mod.relative_position_bias(n, dtype))
    if mask is not None:
        ref = sp_add_mask(ref, mask)
    ref.values.backward(up)
    assert torch.equal(fast.values, ref.values)
    assert torch.equal(v1.grad, v2.grad)
    # the table gradient is the sum of the upstream gradient over the entries that read a table row: checked against
    # that sum formed in fp64 on the host, relative to the sum of their magnitudes (autograd's index_add in the
    # values' own type is not a reference for 16-bit values)
    table_index = attn_mod._table_index(n)
    rel = host(attn_mod.relative_position_index)[:n, :n].astype(np.int64)
    r_idx = f["r_idx"]
    cell = rel[r_idx[2], r_idx[3]]
    rows_t = attn_mod.relative_position_bias_table.shape[0]
    want = np.zeros((rows_t, H))
    mag = np.zeros((rows_t, H))
    np.add.at(want, (cell, r_idx[1]), host(up))
    np.add.at(mag, (cell, r_idx[1]), np.abs(host(up)))
    close(host(g_table_fast), want, 1e-5 if dtype == torch.float32 else 2e-2, "d bias table", mag=mag)
    if dtype == torch.float32:
        close(host(attn_mod.relative_position_bias_table.grad), want, 1e-5, "d bias table (autograd)", mag=mag)
    # the entry point that takes the gathered [H, n, n] bias gives the same bits as the one that reads the table
    gp = ops.group_plan(f["c1"])
    dense = attn_mod.relative_position_bias(n, torch.float32).detach()
    row_pos = ops.group_row_positions(f["s_idx"], gp)
    assert torch.equal(row_pos[:gp.rows], f["qi"][2, ::hd])            # = the Q operand's position row, one entry per token
    assert torch.equal(ops.group_add_bias_mask(vals, row_pos, gp, n, dense, mask), fast.values.detach())
