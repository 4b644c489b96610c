"""Pins of the CPU oracle (runs without a GPU).

The reference ships no tests, golden vectors or fixtures for this path, so each oracle function
is pinned against something it does not share code with: a numpy / torch / scipy library
routine, a closed form derived from the reference's index conventions, a dense brute-force
computation, or an invariant.  Each check is chosen so that a plausible slip (dropped stride,
swapped rows 2/3 of the K^T layout, transposed operand, missing +1e-8, max not clamped at 0)
fails it.
"""
import numpy as np
import pytest
import scipy.special
import torch

from helpers import qkv_operands, ragged_window_indices, random_window_indices


# ------------------------------------------------------------------------------------------ index ops
@pytest.mark.parametrize("sizes", [[7, 5], [4, 3, 9], [6, 2, 8, 4], [3, 125, 24, 32]])
def test_flatten_is_ravel_multi_index(oracle, sizes):
    rng = np.random.default_rng(len(sizes))
    idx = np.stack([rng.integers(0, s, size=500) for s in sizes]).astype(np.int32)
    ref = np.ravel_multi_index(tuple(idx.astype(np.int64)), sizes).astype(np.int32)
    np.testing.assert_array_equal(oracle.flatten_indices(idx, sizes), ref)


def test_flatten_ignores_first_size_and_wraps(oracle):
    idx = np.array([[50000, 3], [23, 1], [124, 7], [767, 2]], np.int32)
    sizes = [1, 24, 125, 768]                       # sizes[0] never enters the strides
    exact = (idx[0].astype(np.int64) * 24 * 125 * 768 + idx[1].astype(np.int64) * 125 * 768
             + idx[2].astype(np.int64) * 768 + idx[3])
    wrapped = ((exact + 2**31) % 2**32 - 2**31).astype(np.int32)
    assert exact[0] >= 2**31                        # the first column really overflows int32
    np.testing.assert_array_equal(oracle.flatten_indices(idx, sizes), wrapped)


def test_sort_is_stable_argsort(oracle):
    rng = np.random.default_rng(0)
    keys = rng.integers(-100, 100, size=5000).astype(np.int32)
    np.testing.assert_array_equal(oracle.sort_indices(keys), np.argsort(keys, kind="stable").astype(np.int32))


def test_unique_consecutive_matches_torch(oracle):
    rng = np.random.default_rng(1)
    x = rng.integers(0, 4, size=3000).astype(np.int32)           # unsorted: runs, not values, count
    ref = torch.unique_consecutive(torch.from_numpy(x), return_inverse=True)[1].numpy()
    np.testing.assert_array_equal(oracle.unique_consecutive_indices(x), ref.astype(np.int32))
    x64 = np.sort(rng.integers(0, 10**12, size=1000))
    ref = torch.unique_consecutive(torch.from_numpy(x64), return_inverse=True)[1].numpy()
    np.testing.assert_array_equal(oracle.unique_consecutive_indices(x64), ref.astype(np.int32))


@pytest.mark.parametrize("maxnum", [-1, 700])
def test_return_inverse_matches_numpy_unique(oracle, maxnum):
    rng = np.random.default_rng(2)
    x = rng.integers(0, 600, size=2000).astype(np.int32)
    uniq, inv = np.unique(x, return_inverse=True)
    out, cnt = oracle.return_inverse(x, maxnum)
    assert cnt == len(uniq)
    np.testing.assert_array_equal(out, inv.astype(np.int32))


# ------------------------------------------------------------------------------------------ qkv indices
def test_qkv_sparse_indices_brute_force_and_closed_forms(oracle):
    rng = np.random.default_rng(3)
    B, n, H, hd = 9, 27, 3, 8
    ind = random_window_indices(rng, B, n, 60)
    N, D = len(ind), H * hd
    iqv, sqv, ik, sk = oracle.qkv_sparse_indices(ind, B, n, H, hd)
    # brute force: all E 4-tuples in input order, lexsort = argsort of the row-major hash
    e = np.arange(N * D)
    v, h, ch = e // D, (e % D) // hd, e % hd
    qv_rows = np.stack([ind[v, 0], h, ind[v, 1], ch])
    k_rows = np.stack([ind[v, 0], h, ch, ind[v, 1]])
    np.testing.assert_array_equal(iqv, qv_rows)
    np.testing.assert_array_equal(ik, k_rows)
    np.testing.assert_array_equal(sqv, np.lexsort(qv_rows[::-1]))
    np.testing.assert_array_equal(sk, np.lexsort(k_rows[::-1]))
    # closed forms: token rank T_k + i, destination slots of both layouts
    key = ind[:, 0].astype(np.int64) * n + ind[:, 1]
    order = np.argsort(key)
    wins, counts = np.unique(ind[order, 0], return_counts=True)
    T = np.concatenate([[0], np.cumsum(counts)[:-1]])
    slot_qv = np.empty(N * D, np.int64)
    slot_k = np.empty(N * D, np.int64)
    r = 0
    for k, c in enumerate(counts):
        for i in range(c):
            vox = order[r]
            for hh in range(H):
                base = hd * (H * T[k] + hh * c)
                for cc in range(hd):
                    slot_qv[base + i * hd + cc] = vox * D + hh * hd + cc
                    slot_k[base + cc * c + i] = vox * D + hh * hd + cc
            r += 1
    np.testing.assert_array_equal(sqv, slot_qv)
    np.testing.assert_array_equal(sk, slot_k)


# ------------------------------------------------------------------------------------------ products
def _dense_scores(ind, qkv, B, n):
    N, _, H, hd = qkv.shape
    Q = np.zeros((B, H, n, hd))
    K = np.zeros((B, H, n, hd))
    V = np.zeros((B, H, n, hd))
    present = np.zeros((B, n), bool)
    for t in range(N):
        w, p = ind[t]
        Q[w, :, p], K[w, :, p], V[w, :, p] = qkv[t, 0], qkv[t, 1], qkv[t, 2]
        present[w, p] = True
    return Q, K, V, present


def test_matmul_q_k_and_qk_v_against_dense_brute_force(oracle):
    rng = np.random.default_rng(4)
    counts = [3, 0, 1, 7, 0, 12, 2]
    B, n, H, hd = len(counts), 16, 2, 4
    ind = ragged_window_indices(rng, counts, n)
    d = qkv_operands(oracle, ind, B, n, H, hd, rng, dtype=np.float64)
    Q, K, V, present = _dense_scores(ind, d["qkv"], B, n)
    idx, val, shape, c = oracle.matmul_cuda_naive(d["q"], d["qi"], d["q_shape"], d["kt"], d["ki"], d["k_shape"], "q_k")
    S = np.einsum("bhid,bhjd->bhij", Q, K)
    mask = np.broadcast_to(present[:, None, :, None] & present[:, None, None, :], S.shape)
    assert shape == [B, H, n, n]
    np.testing.assert_array_equal(idx, np.stack(np.nonzero(mask)))          # coalesced COO order
    np.testing.assert_allclose(val, S[mask], rtol=1e-12, atol=1e-12)
    # offsets: _c per non-empty (window, head), sums
    nz = np.array([x for x in counts if x > 0])
    np.testing.assert_array_equal(c, np.repeat(nz, H))
    assert c.sum() == H * len(ind) and (c.astype(np.int64) ** 2).sum() == len(val)
    # attention @ V
    P = np.where(mask, rng.random(S.shape), 0.0)
    o_idx, o_val, o_shape, c2 = oracle.matmul_cuda_naive(P[mask], idx, shape, d["v"], d["qi"], d["q_shape"], "qk_v")
    O = np.einsum("bhij,bhjd->bhid", P, V)
    omask = np.broadcast_to(present[:, None, :, None], O.shape)
    assert o_shape == [B, H, n, hd]
    np.testing.assert_array_equal(o_idx, np.stack(np.nonzero(omask)))
    np.testing.assert_allclose(o_val, O[omask], rtol=1e-12, atol=1e-12)
    np.testing.assert_array_equal(c2, c)


def test_matmul_fp32_accumulates_in_fp32(oracle):
    rng = np.random.default_rng(5)
    ind = ragged_window_indices(rng, [20, 9], 27)
    d = qkv_operands(oracle, ind, 2, 27, 1, 32, rng, dtype=np.float32)
    _, v32, _, _ = oracle.matmul_cuda_naive(d["q"], d["qi"], d["q_shape"], d["kt"], d["ki"], d["k_shape"], "q_k")
    _, v64, _, _ = oracle.matmul_cuda_naive(d["q"].astype(np.float64), d["qi"], d["q_shape"],
                                            d["kt"].astype(np.float64), d["ki"], d["k_shape"], "q_k")
    assert v32.dtype == np.float32
    err = np.abs(v32 - v64)
    assert 0 < err.max() < 1e-4


@pytest.mark.parametrize("kind", ["rc_cr", "rr_rc", "cr_rr"])
def test_matmul_grad_per_group_numpy(oracle, kind):
    rng = np.random.default_rng(6)
    c, C = np.array([3, 1, 6, 2], np.int32), 5
    mats = [rng.standard_normal((int(x), C)) for x in c]            # [c x C]
    sqs = [rng.standard_normal((int(x), int(x))) for x in c]        # [c x c]
    if kind == "rc_cr":      # m1 [c x C] . m2[c x C]^T
        m1, m2, ref = mats, [rng.standard_normal(m.shape) for m in mats], None
        ref = [a @ b.T for a, b in zip(m1, m2)]
    elif kind == "rr_rc":    # m1 [c x c] . m2[C x c]^T
        m1, m2 = sqs, [rng.standard_normal((C, int(x))) for x in c]
        ref = [a @ b.T for a, b in zip(m1, m2)]
    else:                    # m1 [C x c] . m2[c x c]^T
        m1, m2 = [rng.standard_normal((C, int(x))) for x in c], sqs
        ref = [a @ b.T for a, b in zip(m1, m2)]
    cat = lambda xs: np.concatenate([x.ravel() for x in xs])
    out = oracle.matmul_grad_cuda_naive(cat(m1), cat(m2), c, C, kind)
    np.testing.assert_allclose(out, cat(ref), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("kind", ["rc", "rr"])
def test_qkv_transpose_is_per_group_T(oracle, kind):
    rng = np.random.default_rng(7)
    c, C = np.array([4, 1, 3], np.int32), 6
    blocks = [rng.standard_normal((int(x), C if kind == "rc" else int(x))) for x in c]
    out = oracle.qkv_transpose(np.concatenate([b.ravel() for b in blocks]), c, C, kind)
    np.testing.assert_array_equal(out, np.concatenate([b.T.ravel() for b in blocks]))


def test_backward_products_are_the_gradients_of_the_forward(oracle):
    """dQ, dK^T of S = Q K through the reference's composition equal torch.autograd's."""
    rng = np.random.default_rng(8)
    c, C = np.array([5, 2, 7], np.int32), 4
    q = rng.standard_normal(int(c.sum()) * C)
    kt = rng.standard_normal(int(c.sum()) * C)
    g = rng.standard_normal(int((c.astype(np.int64) ** 2).sum()))
    dq = oracle.matmul_grad_cuda_naive(g, kt, c, C, "rr_rc")
    dkt = oracle.matmul_grad_cuda_naive(oracle.qkv_transpose(q, c, C, "rc"), oracle.qkv_transpose(g, c, C, "rr"),
                                        c, C, "cr_rr")
    qt, ktt = torch.tensor(q, requires_grad=True), torch.tensor(kt, requires_grad=True)
    mo = po = 0
    loss = 0
    for cg in c:
        cg = int(cg)
        S = qt[mo:mo + cg * C].reshape(cg, C) @ ktt[mo:mo + cg * C].reshape(C, cg)
        loss = loss + (S.reshape(-1) * torch.tensor(g[po:po + cg * cg])).sum()
        mo += cg * C
        po += cg * cg
    loss.backward()
    np.testing.assert_allclose(dq, qt.grad.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dkt, ktt.grad.numpy(), rtol=1e-12, atol=1e-12)


# ------------------------------------------------------------------------------------------ softmax
def test_softmax_forward_against_scipy_and_invariants(oracle):
    rng = np.random.default_rng(9)
    lengths = [1, 5, 32, 2, 125]
    rows = np.repeat(np.arange(len(lengths)), lengths).astype(np.int32)
    v = rng.standard_normal(len(rows)) * 4
    y = oracle.softmax_last_dim_forward(rows, v)
    s = 0
    for n in lengths:
        seg = v[s:s + n]
        ref = scipy.special.softmax(seg)
        denom = np.exp(seg - max(0.0, seg.max())).sum()
        # differs from the textbook softmax only by the 1e-8 added to the row sum
        np.testing.assert_allclose(y[s:s + n], ref * denom / (denom + 1e-8), rtol=1e-13)
        assert abs(y[s:s + n].sum() - (1 - 1e-8 / (denom + 1e-8))) < 1e-13
        s += n
    assert (y >= 0).all()


def test_softmax_zero_clamped_max_and_epsilon_are_observable(oracle):
    rows = np.zeros(3, np.int32)
    v = np.array([-20.0, -21.0, -22.0])
    y = oracle.softmax_last_dim_forward(rows, v)
    e = np.exp(v)                                  # maximum is clamped at 0, so no shift happens
    np.testing.assert_allclose(y, e / (e.sum() + 1e-8), rtol=1e-14)
    assert abs(y.sum() - 1) > 1e-3                 # textbook softmax would sum to 1
    # single-element row
    y1 = oracle.softmax_last_dim_forward(np.zeros(1, np.int32), np.array([3.0]))
    np.testing.assert_allclose(y1, [1 / (1 + 1e-8)], rtol=1e-15)


def test_softmax_backward_closed_form_and_autograd(oracle):
    rng = np.random.default_rng(10)
    lengths = [1, 4, 9]
    rows = np.repeat(np.arange(len(lengths)), lengths).astype(np.int32)
    v = rng.standard_normal(len(rows))
    g = rng.standard_normal(len(rows))
    y = oracle.softmax_last_dim_forward(rows, v)
    gx = oracle.softmax_last_dim_backward(rows, y, g)
    s = 0
    for n in lengths:
        yy, gg = y[s:s + n], g[s:s + n]
        np.testing.assert_allclose(gx[s:s + n], yy * (gg - (gg * yy).sum()), rtol=1e-12, atol=1e-15)
        s += n
    # autograd of the textbook softmax agrees up to the 1e-8 term
    vt = torch.tensor(v, requires_grad=True)
    outs = torch.cat([torch.softmax(vt[a:b], 0) for a, b in ((0, 1), (1, 5), (5, 14))])
    (outs * torch.tensor(g)).sum().backward()
    np.testing.assert_allclose(gx, vt.grad.numpy(), atol=1e-7)
    assert abs(gx[0]) < 1e-7                       # a single-element row has (almost) zero gradient


def test_readme_softmax_equals_operator_softmax_on_ordinary_rows(oracle):
    from oracle import cpu_path
    rng = np.random.default_rng(11)
    rows = np.repeat(np.arange(50), 20).astype(np.int32)
    v = rng.standard_normal(1000)
    a = cpu_path.sparse_softmax_readme(torch.tensor(v), torch.tensor(rows.astype(np.int64)), 50).numpy()
    b = cpu_path.sparse_softmax_ops(torch.tensor(v), torch.tensor(rows.astype(np.int64)), 50).numpy()
    np.testing.assert_allclose(b, oracle.softmax_last_dim_forward(rows, v), rtol=1e-13)
    np.testing.assert_allclose(a, b, rtol=1e-7)


# ------------------------------------------------------------------------------------------ module path
def test_cpu_path_equals_dense_window_attention():
    from oracle import cpu_path
    from sparseswin3d_amd import synth
    torch.manual_seed(0)
    c4, _ = synth.with_batch([synth.box_surfaces_scene(seed=3, grid=(25, 25, 25), n_boxes=2)])
    for shift in ((0, 0, 0), (2, 2, 2)):
        idx, nw, n = synth.window_indices(c4, (25, 25, 25), (5, 5, 5), shift)
        N, D, H = len(idx), 32, 2
        f = torch.randn(N, D, dtype=torch.float64)
        qw, qb = torch.randn(3 * D, D, dtype=torch.float64) * 0.2, torch.randn(3 * D, dtype=torch.float64)
        pw, pb = torch.randn(D, D, dtype=torch.float64) * 0.2, torch.randn(D, dtype=torch.float64)
        rpb = torch.randn(H, n, n, dtype=torch.float64)
        mask = synth.shift_region_mask((25, 25, 25), (5, 5, 5), (2, 2, 2)) if any(shift) else None
        a = cpu_path.window_attention_cpu(f, idx, n, H, qw, qb, pw, pb, rpb, mask, softmax="readme")
        b = cpu_path.dense_window_attention_reference(f, idx, n, H, qw, qb, pw, pb, rpb, mask)
        np.testing.assert_allclose(a.numpy(), b.numpy(), rtol=1e-10, atol=1e-12)


def _region_brute_force(dims, ws, ss):
    """Region of every cell of the shifted grid, one cell at a time: along each axis the three
    slices [:-ws], [-ws:-s], [-s:] are applied in this order and the last one that holds the
    coordinate wins (Python slice semantics: s == 0 makes the middle slice empty and the last
    one the whole axis)."""
    def axis(v, extent, w, s):
        r = None
        for k, sl in enumerate((slice(-w), slice(-w, -s), slice(-s, None))):
            if v in range(extent)[sl]:
                r = k
        return r
    nd, nh, nw = (dims[a] // ws[a] for a in range(3))
    out = np.zeros((nd * nh * nw, ws[0] * ws[1] * ws[2]), np.int8)
    for z in range(dims[0]):
        for y in range(dims[1]):
            for x in range(dims[2]):
                win = ((z // ws[0]) * nh + y // ws[1]) * nw + x // ws[2]
                pos = ((z % ws[0]) * ws[1] + y % ws[1]) * ws[2] + x % ws[2]
                out[win, pos] = 9 * axis(z, dims[0], ws[0], ss[0]) + 3 * axis(y, dims[1], ws[1], ss[1]) \
                    + axis(x, dims[2], ws[2], ss[2])
    return out


@pytest.mark.parametrize("dims,ws,ss", [((15, 10, 20), (5, 5, 5), (2, 2, 2)), ((6, 8, 4), (3, 4, 2), (1, 2, 1)),
                                        ((5, 10, 5), (5, 5, 5), (0, 2, 0)), ((4, 4, 4), (2, 2, 2), (0, 0, 0))])
def test_shift_mask_matches_cell_by_cell_construction(dims, ws, ss):
    from oracle import grid
    from sparseswin3d_amd import synth
    ref = _region_brute_force(dims, ws, ss)
    np.testing.assert_array_equal(grid.shift_mask(dims, ws, ss), ref)
    np.testing.assert_array_equal(synth.shift_region_mask(dims, ws, ss), ref)
    if all(ss) and all(d > w for d, w in zip(dims, ws)):
        assert ref.max() == 26


def test_oracle_window_indices_match_dense_roll_and_partition():
    """The step-by-step pad / roll / partition of the oracle against torch.roll + reshape on a
    dense volume of voxel ids, with a grid that needs padding and two batch items."""
    from oracle import grid as og
    grid, ws, shift = (9, 13, 5), (5, 5, 5), (2, 2, 2)
    padded = (10, 15, 5)
    vol = torch.arange(2 * int(np.prod(padded))).reshape(2, *padded)
    rolled = torch.roll(vol, shifts=tuple(-s for s in shift), dims=(1, 2, 3))
    parts = rolled.reshape(2, 2, 5, 3, 5, 1, 5).permute(0, 1, 3, 5, 2, 4, 6).reshape(-1, 125)   # [window, pos] -> id
    bb, zz, yy, xx = np.meshgrid(np.arange(2), *[np.arange(g) for g in grid], indexing="ij")
    c4 = np.stack([bb.ravel(), zz.ravel(), yy.ravel(), xx.ravel()], 1).astype(np.int32)
    idx, nw, n = og.window_indices(c4, grid, ws, shift)
    assert (nw, n) == (6, 125)
    vox_id = ((c4[:, 0] * padded[0] + c4[:, 1]) * padded[1] + c4[:, 2]) * padded[2] + c4[:, 3]
    np.testing.assert_array_equal(parts.numpy()[idx[:, 0], idx[:, 1]], vox_id)


def test_oracle_downsample_against_dictionary_brute_force():
    from oracle import grid as og
    rng = np.random.default_rng(8)
    c4 = np.unique(np.stack([rng.integers(0, 2, 400), rng.integers(0, 9, 400), rng.integers(0, 7, 400),
                             rng.integers(0, 11, 400)], 1), axis=0).astype(np.int32)
    c4 = c4[rng.permutation(len(c4))]
    f = rng.standard_normal((len(c4), 8))
    coords, pooled, inverse = og.downsample(c4, f)
    cells = {}
    for row, feat in zip(c4, f):
        cells.setdefault((row[0], row[1] // 2, row[2] // 2, row[3] // 2), []).append(feat)
    keys = sorted(cells)
    np.testing.assert_array_equal(coords, np.array(keys, np.int32))
    np.testing.assert_allclose(pooled, np.stack([np.mean(cells[k], 0) for k in keys]), rtol=1e-12)
    assert all(tuple(coords[inverse[i]]) == (c4[i, 0], c4[i, 1] // 2, c4[i, 2] // 2, c4[i, 3] // 2) for i in range(len(c4)))


def test_window_indices_match_dense_roll_and_partition():
    """Sparse pad/roll/partition arithmetic against torch.roll + reshape on a dense id volume."""
    from sparseswin3d_amd import synth
    grid, ws, shift = (10, 15, 5), (5, 5, 5), (2, 2, 2)
    vol = torch.arange(int(np.prod(grid))).reshape(grid)
    rolled = torch.roll(vol, shifts=tuple(-s for s in shift), dims=(0, 1, 2))
    parts = rolled.reshape(2, 5, 3, 5, 1, 5).permute(0, 2, 4, 1, 3, 5).reshape(-1, 125)   # [window, pos] -> voxel id
    zz, yy, xx = np.meshgrid(*[np.arange(g) for g in grid], indexing="ij")
    c4, _ = synth.with_batch([np.stack([zz.ravel(), yy.ravel(), xx.ravel()], 1)])
    idx, nw, n = synth.window_indices(c4, grid, ws, shift)
    vox_id = (c4[:, 1] * grid[1] + c4[:, 2]) * grid[2] + c4[:, 3]
    np.testing.assert_array_equal(parts.numpy()[idx[:, 0], idx[:, 1]], vox_id)
