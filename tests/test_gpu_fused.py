"""The fused window-attention path: token plan bit-exact against closed forms, module results
equal to the operator-by-operator path and to the CPU path (fp32 rel 1e-5, 16-bit rel 2e-2)."""
import numpy as np
import pytest
import torch

from helpers import score_grad_mag, PATHS, close, ragged_window_indices, random_window_indices, set_path

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


@pytest.mark.parametrize("case", ["random", "ragged", "single", "big", "wide", "wide125"])
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
    elif case == "big":
        B, n, H = 20000, 125, 3
        ind = random_window_indices(rng, B, n, 120000)
    elif case == "wide":             # enough window slots for the per-block phases to take four slots per thread
        B, n, H = 300000, 8, 1
        ind = random_window_indices(rng, B, n, 250000)
    else:                            # the same with four bitmap words per slot and several heads
        B, n, H = 70000, 125, 3
        ind = random_window_indices(rng, B, n, 150000)
    tokens, plan, A, c_max = _closed_form_plan(ind, n, H)
    tp = TokenPlan(torch.from_numpy(ind).cuda(), B, n, H)
    assert (tp.G, tp.A, tp.c_max) == (plan.shape[1], A, c_max)
    np.testing.assert_array_equal(tp.tokens.view(5, -1).cpu().numpy(), tokens)
    np.testing.assert_array_equal(tp.plan.view(5, -1)[:, :tp.G].cpu().numpy(), plan)


def test_token_plans_in_one_batch_equal_single_plans():
    """Several plans built by shared launches (different voxel counts, window counts, window sizes, head counts,
    one of them empty, one without task descriptors) hold the same bits as plans built one by one; a bad index in
    one plan of a batch is reported for that plan only."""
    from sparseswin3d_amd import _lib
    from sparseswin3d_amd.fused import TokenPlan
    rng = np.random.default_rng(11)
    specs = [(random_window_indices(rng, 50, 125, 1500), 50, 125, 3, True),
             (ragged_window_indices(rng, [1, 0, 125, 2, 0, 0, 33, 64, 5, 17, 1, 1, 100], 125), 13, 125, 6, True),
             (random_window_indices(rng, 20000, 125, 120000), 20000, 125, 3, True),
             (np.zeros((0, 2), np.int32), 7, 27, 2, True),
             (random_window_indices(rng, 3000, 8, 9000), 3000, 8, 1, False),
             (random_window_indices(rng, 700, 64, 20000), 700, 64, 4, True),
             (random_window_indices(rng, 270000, 27, 90000), 270000, 27, 2, True)]   # its call uses the wide blocks
    dev = [(torch.from_numpy(ind).cuda(), B, n, H, tasks) for ind, B, n, H, tasks in specs]
    plans = TokenPlan.batch(dev)                         # seven plans: two library calls
    assert len(plans) == len(specs)
    for spec, tp in zip(dev, plans):
        tp.finish()
        one = TokenPlan(*spec[:4], tasks=spec[4])
        assert (tp.G, tp.windows, tp.A, tp.c_max, list(tp.bucket_counts)) == \
               (one.G, one.windows, one.A, one.c_max, list(one.bucket_counts))
        assert torch.equal(tp.tokens[:5 * tp.N], one.tokens[:5 * one.N])
        assert torch.equal(tp.plan.view(5, -1)[:, :tp.G], one.plan.view(5, -1)[:, :one.G])
        if spec[4] and tp.G:
            # descriptors of a bucket, as sets: their order inside a bucket is the same here, but not promised
            a, b = tp.tasks[:16 * tp.g_cap].view(4, tp.g_cap, 4), one.tasks[:16 * one.g_cap].view(4, one.g_cap, 4)
            for k in range(4):
                m = int(tp.bucket_counts[k])
                assert torch.equal(a[k, :m], b[k, :m])
            # the token records behind the descriptors: one per (window, tile of 32 tokens), the bucket of four tiles
            # first, inside a bucket by window, then tile; entry l = (voxel, pos) of token 32 tile + l of the window,
            # the window's last token again behind it
            H = spec[3]
            n_rec = sum(int(tp.bucket_counts[k]) // H * (k + 1) for k in range(4))
            ra = tp.tasks[16 * tp.g_cap:16 * tp.g_cap + 64 * n_rec].view(n_rec, 32, 2).cpu().numpy()
            rb = one.tasks[16 * one.g_cap:16 * one.g_cap + 64 * n_rec].view(n_rec, 32, 2).cpu().numpy()
            np.testing.assert_array_equal(ra, rb)
            tok = tp.tokens.view(5, -1).cpu().numpy()
            desc = a.cpu().numpy()
            first = 0
            for k in (3, 2, 1, 0):
                for wslot in range(int(tp.bucket_counts[k]) // H):
                    T, c = int(desc[k, wslot * H, 0]), int(desc[k, wslot * H, 1]) & 0xff
                    for tile in range(k + 1):
                        ranks = T + np.minimum(32 * tile + np.arange(32), c - 1)
                        want = np.stack([tok[0, ranks], tok[3, ranks]], 1)
                        np.testing.assert_array_equal(ra[first + wslot * (k + 1) + tile], want)
                first += int(tp.bucket_counts[k]) // H * (k + 1)
    # a plan that keeps the voxel order only (what the stride-2 merge reads) holds the same first row and group table
    lean = TokenPlan(dev[4][0], 3000, 8, 1, tasks=False, order_only=True)
    assert lean.tokens.numel() == lean.N and torch.equal(lean.tokens, plans[4].tokens[:lean.N])
    assert torch.equal(lean.plan.view(5, -1)[:, :lean.G], plans[4].plan.view(5, -1)[:, :lean.G])
    descs = (_lib.TokenPlanDesc * 1)()
    descs[0].N, descs[0].B, descs[0].n, descs[0].H, descs[0].flags = 4, 4, 8, 1, 6
    totals = torch.zeros(9, dtype=torch.int64)               # the library clears it before it looks at the rest
    descs[0].totals_out = totals.data_ptr()
    descs[0].indices = descs[0].tokens = descs[0].plan = descs[0].ws = dev[4][0].data_ptr()    # never reached
    descs[0].g_cap, descs[0].ws_bytes = 4, 1 << 20
    assert _lib.load().sswin_token_plan_batch(descs, 1, None) != 0 and b"flags" in _lib.load().sswin_last_error()
    # errors stay with their plan
    good = specs[0][0]
    bad = np.concatenate([good[:400], np.array([[50, 3]], np.int32), good[400:]])
    p_bad, p_good = TokenPlan.batch([(torch.from_numpy(bad).cuda(), 50, 125, 3), dev[1][:4]])
    with pytest.raises(RuntimeError, match="outside"):
        p_bad.finish()
    assert p_good.finish().G == plans[1].G
    # more than four descriptors in one library call are refused
    descs = (_lib.TokenPlanDesc * 5)()
    assert _lib.load().sswin_token_plan_batch(descs, 5, None) != 0
    assert b"between 0 and 4" in _lib.load().sswin_last_error()
    assert _lib.load().sswin_token_plan_batch(None, 0, None) == 0


def test_token_plan_rejects_bad_indices():
    """Indices outside [0,B) x [0,n) and repeated (window, pos) pairs are skipped on the device (every kernel
    exits normally, nothing is written through them) and reported when the totals are decoded."""
    from sparseswin3d_amd.fused import TokenPlan
    rng = np.random.default_rng(5)
    B, n, H = 40, 125, 3
    good = random_window_indices(rng, B, n, 900)
    for bad_row, what in (([B, 3], "outside"), ([-1, 0], "outside"), ([2, n], "outside"), ([5, -7], "outside"),
                          (list(good[17]), "distinct")):
        ind = np.concatenate([good[:400], np.array([bad_row], np.int32), good[400:]])
        with pytest.raises(RuntimeError, match=what):
            TokenPlan(torch.from_numpy(ind).cuda(), B, n, H)
    tp = TokenPlan(torch.from_numpy(good).cuda(), B, n, H)     # and the library still works
    assert tp.G == len(np.unique(good[:, 0])) * H


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
    for path in PATHS:
        set_path(attn, path)
        attn.zero_grad()
        f = feats.clone().requires_grad_(True)
        out = attn(SparseVoxelTensor(f, torch.from_numpy(idx).cuda(), (n,), nw), mask).features
        out.backward(up)
        res[path] = [t.detach().cpu().numpy() for t in
                      (out, f.grad, attn.qkv.weight.grad, attn.relative_position_bias_table.grad)]
    for path in ("resident", "fused"):
        for a, b, what in zip(res[path], res["operators"], ("out", "d feats", "d qkv.w", "d bias table")):
            close(a, b, 1e-5, f"{path}: {what}")


@pytest.mark.parametrize("dtype,dim,heads", [(torch.float32, 96, 3), (torch.float32, 48, 3), (torch.bfloat16, 64, 2)])
def test_fused_products_with_32_and_64_bit_addresses(dtype, dim, heads, monkeypatch):
    """The fused-path products address token rows through buffer descriptors; tensors beyond 2^31 bytes take kernels
    with 64-bit addresses (SSWIN_FUSED_WIDE=1 sends everything there).  The two split the last tokens of a reduction
    between the lane halves differently, so the sums agree to rounding, not bit for bit."""
    from sparseswin3d_amd import synth
    from sparseswin3d_amd.window_attention import SparseVoxelTensor
    c4, _ = synth.with_batch([synth.box_surfaces_scene(seed=5, grid=(40, 40, 40), n_boxes=4)])
    idx, nw, n = synth.window_indices(c4, (40, 40, 40), (5, 5, 5), (2, 2, 2))
    mask = torch.from_numpy(synth.shift_region_mask((40, 40, 40), (5, 5, 5), (2, 2, 2))).cuda()
    attn = _modules(dim, heads, dtype)
    set_path(attn, "fused")
    feats = torch.randn(len(idx), dim, device="cuda").to(dtype)
    up = torch.randn(len(idx), dim, device="cuda").to(dtype)
    res = []
    for wide in ("0", "1"):
        monkeypatch.setenv("SSWIN_FUSED_WIDE", wide)
        attn.zero_grad()
        f = feats.clone().requires_grad_(True)
        out = attn(SparseVoxelTensor(f, torch.from_numpy(idx).cuda(), (n,), nw), mask).features
        out.backward(up)
        res.append([t.detach().double().cpu().numpy() for t in (out, f.grad, attn.qkv.weight.grad, attn.relative_position_bias_table.grad)])
    for a, b, what in zip(res[0], res[1], ("out", "d feats", "d qkv.w", "d bias table")):
        close(a, b, 1e-5 if dtype == torch.float32 else 2e-2, f"descriptor against 64-bit addresses: {what}")


@pytest.mark.parametrize("H", [1, 3])
def test_softmax_over_the_rows_of_the_groups(oracle, H):
    """The fused path's softmax takes its rows from the group table.  Against the fp64 oracle of the operator
    (zero-initialised maximum, + 1e-8), forward and backward, out of place and in place, on group sizes around the
    edges of its three lane layouts (16, 32, 64 lanes per row; 2 and 6 values per lane) and with rows that are all
    negative (their maximum stays 0, ops.cu:128-167)."""
    from helpers import softmax_bwd_mag
    from sparseswin3d_amd import fused
    rng = np.random.default_rng(77 + H)
    counts = [1, 16, 17, 0, 32, 33, 64, 65, 128, 129, 300, 5, 2, 343]
    n = 343
    ind = ragged_window_indices(rng, counts, n)
    tp = fused.TokenPlan(torch.from_numpy(ind).cuda(), len(counts), n, H)
    plan = tp.plan.view(5, -1)[:, :tp.G].cpu().numpy()
    rows = np.empty(tp.A, np.int32)
    r0 = 0
    for c, sq in zip(plan[0], plan[2]):
        rows[sq:sq + c * c] = r0 + np.repeat(np.arange(c), c)
        r0 += c
    x = rng.standard_normal(tp.A).astype(np.float32) * 3
    x[rows % 7 == 3] = -np.abs(x[rows % 7 == 3]) - 1.0          # whole rows below zero
    g = rng.standard_normal(tp.A).astype(np.float32)
    xd, gd = torch.from_numpy(x).cuda(), torch.from_numpy(g).cuda()
    y = torch.empty_like(xd)
    fused._group_softmax(tp, False, xd, None, y)
    ref_y = oracle.softmax_last_dim_forward(rows, x.astype(np.float64))
    close(y.cpu().numpy(), ref_y, 1e-5, "group softmax forward", seg=rows)
    y2 = xd.clone()
    fused._group_softmax(tp, False, y2, None, y2)
    assert torch.equal(y, y2)
    gx = torch.empty_like(xd)
    fused._group_softmax(tp, True, y, gd, gx)
    yh = y.double().cpu().numpy()
    ref_gx = oracle.softmax_last_dim_backward(rows, yh, g.astype(np.float64))
    close(gx.cpu().numpy(), ref_gx, 1e-5, "group softmax backward", mag=softmax_bwd_mag(rows, yh, g))
    g2 = gd.clone()
    fused._group_softmax(tp, True, y, g2, g2)
    assert torch.equal(gx, g2)


@pytest.mark.parametrize("path", ["resident", "fused"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_16bit_against_cpu_fp64(dtype, path):
    from oracle import cpu_path
    from sparseswin3d_amd import synth
    from sparseswin3d_amd.window_attention import SparseVoxelTensor
    c4, _ = synth.with_batch([synth.filled_blob_scene(seed=4, grid=(10, 10, 10), fill=0.9)])
    idx, nw, n = synth.window_indices(c4, (10, 10, 10), (5, 5, 5), (2, 2, 2))
    mask_np = synth.shift_region_mask((10, 10, 10), (5, 5, 5), (2, 2, 2))
    attn = _modules(64, 2, dtype)
    set_path(attn, path)
    feats = (torch.randn(len(idx), 64) * 0.5).to(dtype)
    x = SparseVoxelTensor(feats.cuda(), torch.from_numpy(idx).cuda(), (n,), nw)
    out = attn(x, torch.from_numpy(mask_np).cuda()).features
    p = {k: v.detach().double().cpu() for k, v in attn.state_dict().items()}
    rpb = p["relative_position_bias_table"][p["relative_position_index"].reshape(-1).long()].reshape(n, n, -1).permute(2, 0, 1)
    ref = cpu_path.window_attention_cpu(feats.double(), idx, n, 2, p["qkv.weight"], p["qkv.bias"], p["proj.weight"],
                                        p["proj.bias"], rpb, mask_np)
    close(out.detach().double().cpu().numpy(), ref.numpy(), 2e-2, f"{path} {dtype}")


@pytest.mark.parametrize("family", ["fp32mfma", "x16"])
@pytest.mark.parametrize("mix", ["tiny", "edges", "full", "mixed"])
@pytest.mark.parametrize("use_mask", [False, True], ids=["nomask", "mask"])
def test_resident_kernels_on_ragged_windows(mix, use_mask, family, monkeypatch):
    """Window-resident forward/backward through the C ABI on hand-picked occupancies (1 token,
    around the 32/64/96 tile edges, full 125-token windows, empty slots) against dense fp64
    attention per window; also checks the bucket counts of the task list.  Both kernel families on fp32 tokens:
    the fp32 matrix instructions and the 16-bit operands with every value split into two fp16 pieces."""
    import ctypes as C
    monkeypatch.setenv("SSWIN_WATTN", family)
    from sparseswin3d_amd import _lib
    from sparseswin3d_amd.fused import TokenPlan, _ptr
    mixes = {"tiny": [1, 2, 3, 1, 5, 4], "edges": [31, 32, 33, 0, 63, 64, 65, 1, 95, 96, 97],
             "full": [125, 124, 100, 7], "mixed": [1, 40, 2, 125, 0, 0, 17, 32, 90, 3, 3, 3, 3, 64]}
    counts = mixes[mix]
    rng = np.random.default_rng(len(mix) + use_mask)
    n, H, hd = 125, 3, 32
    D = H * hd
    ind = ragged_window_indices(rng, counts, n)
    N, B = len(ind), len(counts)
    tp = TokenPlan(torch.from_numpy(ind).cuda(), B, n, H)
    want = [sum(1 for c in counts if 32 * b < c <= 32 * (b + 1)) * H for b in range(4)]
    assert list(tp.bucket_counts) == want and tp.oversize_groups == 0
    qkv = torch.randn(N, 3 * D, dtype=torch.float64)
    bias = torch.randn(H, n, n, dtype=torch.float64)
    d_out = torch.randn(N, D, dtype=torch.float64)
    mask = torch.from_numpy(rng.integers(0, 3, size=(4, n)).astype(np.int8)) if use_mask else None
    scale = hd ** -0.5

    lib = _lib.load()
    q32 = qkv.float().cuda()
    b32 = bias.float().cuda()
    do32 = d_out.float().cuda()
    m_dev = None if mask is None else mask.cuda()
    out = torch.full((N, D), float("nan"), device="cuda")
    lse = torch.empty(H * N, device="cuda")
    dqkv = torch.full((N, 3 * D), float("nan"), device="cuda")
    ds = torch.full((tp.A,), float("nan"), device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    nmw = 0 if mask is None else mask.shape[0]
    _lib.check(lib.sswin_window_attention_forward(
        0, _ptr(tp.tasks), tp.g_cap, tp.bucket_counts, _ptr(tp.tokens), N, H, hd, _ptr(q32), 3 * D, 0, _ptr(q32), 3 * D, D,
        _ptr(q32), 3 * D, 2 * D, C.c_float(scale), _ptr(b32), n, _ptr(m_dev), nmw, _ptr(out), D, 0, _ptr(lse), stream))
    _lib.check(lib.sswin_window_attention_backward(
        0, _ptr(tp.tasks), tp.g_cap, tp.bucket_counts, _ptr(tp.tokens), N, H, hd, _ptr(q32), 3 * D, 0, _ptr(q32), 3 * D, D,
        _ptr(q32), 3 * D, 2 * D, C.c_float(scale), _ptr(b32), n, _ptr(m_dev), nmw, _ptr(out), D, 0, _ptr(do32), D, 0,
        _ptr(lse), _ptr(dqkv), 3 * D, 0, _ptr(dqkv), 3 * D, D, _ptr(dqkv), 3 * D, 2 * D, _ptr(ds), 3, stream))

    # dense fp64 reference per window with autograd
    qkv_r = q32.double().cpu().requires_grad_(True)
    bias_r = b32.double().cpu().requires_grad_(True)
    ref = torch.zeros(N, D, dtype=torch.float64)
    order = np.lexsort((ind[:, 1], ind[:, 0]))
    pieces = []
    bias_mag = torch.zeros(H, n, n, dtype=torch.float64)
    plan_h = tp.plan.view(5, -1)[:, :tp.G].cpu().numpy()       # rows: c, first row, first entry, window, head
    sq_of = {(int(plan_h[3, g]), int(plan_h[4, g])): int(plan_h[2, g]) for g in range(tp.G)}
    ds_ref, ds_mag = np.zeros(tp.A), np.zeros(tp.A)
    for w in np.unique(ind[:, 0]):
        vox = torch.from_numpy(order[ind[order, 0] == w])
        pos = torch.from_numpy(ind[vox.numpy(), 1].astype(np.int64))
        x = qkv_r[vox].reshape(len(vox), 3, H, hd)
        s = torch.einsum("ihc,jhc->hij", x[:, 0] * scale, x[:, 1]) + bias_r[:, pos][:, :, pos]
        if mask is not None:
            r = mask[int(w) % mask.shape[0]].long()[pos]
            s = s + (r[None, :] != r[:, None]).double() * -100.0
        m = s.max(-1, keepdim=True).values.clamp(min=0)
        e = (s - m).exp()
        p = e / (e.sum(-1, keepdim=True) + 1e-8)
        pieces.append((vox, torch.einsum("hij,jhc->ihc", p, x[:, 2]).reshape(len(vox), D)))
        with torch.no_grad():           # dS = P (dP - D) itself and what it is conditioned by, per entry and per bias cell
            dO_w = do32.double().cpu()[vox].reshape(len(vox), H, hd)
            O_w = pieces[-1][1].reshape(len(vox), H, hd)
            cw = len(vox)
            for hh in range(H):
                mag_wh = score_grad_mag(p[hh], dO_w[:, hh], x[:, 2, hh], O_w[:, hh])
                bias_mag[hh][pos[:, None], pos[None, :]] += mag_wh
                dP = dO_w[:, hh] @ x[:, 2, hh].t()
                sq0 = sq_of[(int(w), hh)]
                ds_ref[sq0:sq0 + cw * cw] = (p[hh] * (dP - (dO_w[:, hh] * O_w[:, hh]).sum(-1, keepdim=True))).reshape(-1).numpy()
                ds_mag[sq0:sq0 + cw * cw] = mag_wh.reshape(-1).numpy()
    ref = torch.zeros(N, D, dtype=torch.float64).index_put((torch.cat([v for v, _ in pieces]),),
                                                            torch.cat([o for _, o in pieces]))
    ref.backward(do32.double().cpu())
    close(out.cpu().numpy(), ref.detach().numpy(), 1e-5, "O")
    close(dqkv.cpu().numpy(), qkv_r.grad.numpy(), 1e-5, "d qkv")
    # the per-side kernels (sides 1 and 2)
    for sides, cols in ((1, slice(0, D)), (2, slice(D, 3 * D))):
        part = torch.full((N, 3 * D), float("nan"), device="cuda")
        ds2 = torch.full((tp.A,), float("nan"), device="cuda")
        _lib.check(lib.sswin_window_attention_backward(
            0, _ptr(tp.tasks), tp.g_cap, tp.bucket_counts, _ptr(tp.tokens), N, H, hd, _ptr(q32), 3 * D, 0, _ptr(q32), 3 * D, D,
            _ptr(q32), 3 * D, 2 * D, C.c_float(scale), _ptr(b32), n, _ptr(m_dev), nmw, _ptr(out), D, 0, _ptr(do32), D, 0,
            _ptr(lse), _ptr(part), 3 * D, 0, _ptr(part), 3 * D, D, _ptr(part), 3 * D, 2 * D, _ptr(ds2), sides, stream))
        got, want_g = part.cpu().numpy(), qkv_r.grad.numpy()
        # a token's dQ alone can be zero where dK and dV are not (a window of one token: dS = P (dP - D) = 0 from two
        # equal numbers of ordinary size): measured against the token's whole gradient row
        close(got[:, cols], want_g[:, cols], 1e-5, f"sides={sides}",
              mag=np.abs(want_g[:, cols]) + np.abs(want_g).max(axis=1, keepdims=True))
        other = np.ones(3 * D, bool)
        other[cols] = False
        assert np.isnan(got[:, other]).all()                 # the other side is not touched
        if sides != 1:
            close(ds2.cpu().numpy(), ds_ref, 1e-5, "dS of the key-side kernel", mag=ds_mag)
    close(ds.cpu().numpy(), ds_ref, 1e-5, "dS of the one-launch backward", mag=ds_mag)
    # bias gradient from the stored dS
    d_bias = torch.zeros(H, n, n, device="cuda")
    nbytes = lib.sswin_fused_bias_grad_workspace_bytes(tp.G, H, n)
    ws = torch.empty(int(nbytes), dtype=torch.uint8, device="cuda")
    _lib.check(lib.sswin_fused_bias_grad(_ptr(tp.plan), tp.g_cap, tp.G, _ptr(tp.tokens), N, H, n, _ptr(ds), _ptr(d_bias),
                                         _ptr(ws), nbytes, stream))
    assert not torch.isnan(ds).any()
    close(d_bias.cpu().numpy(), bias_r.grad.numpy(), 1e-5, "d bias", mag=bias_mag.numpy())


@pytest.mark.parametrize("mix,H", [("tiny", 1), ("mixed", 3), ("full", 2), ("many", 3), ("crowd", 3)])
def test_bias_table_gradient(mix, H):
    """d_table[rel(p_i, p_j), h] = sum of dS: the table-gradient kernel against a numpy scatter."""
    import ctypes as C
    from sparseswin3d_amd import _lib
    from sparseswin3d_amd.fused import BiasTableIndex, TokenPlan, _ptr
    from sparseswin3d_amd.window_attention import relative_position_index_3d
    rng = np.random.default_rng(len(mix) + H)
    mixes = {"tiny": [1, 2, 3, 1, 5, 4], "mixed": [1, 40, 2, 125, 0, 0, 17, 32, 90, 3, 3, 3, 3, 64, 65, 70],
             "full": [125, 124, 100, 7], "many": list(rng.integers(0, 60, size=700)),
             # more than 64 windows per window slice of the kernel (128 slices for three heads): a wavefront
             # fetches window headers more than once
             "crowd": list(rng.integers(0, 5, size=9000))}
    counts = [int(c) for c in mixes[mix]]
    n, rows = 125, 729
    ind = ragged_window_indices(rng, counts, n)
    tp = TokenPlan(torch.from_numpy(ind).cuda(), len(counts), n, H)
    rel = relative_position_index_3d((5, 5, 5))
    ti = BiasTableIndex.build(rel.cuda(), rows)
    assert ti is not None
    ds = rng.standard_normal(tp.A).astype(np.float32)
    lib = _lib.load()
    out = torch.full((rows, H), float("nan"), device="cuda")
    nbytes = lib.sswin_bias_table_grad_workspace_bytes(tp.G, H, rows)
    ws = torch.empty(int(nbytes), dtype=torch.uint8, device="cuda")
    ds_d = torch.from_numpy(ds).cuda()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.sswin_bias_table_grad(_ptr(tp.plan), tp.g_cap, tp.G, _ptr(tp.tokens), tp.N, H, n, _ptr(ti.code),
                                         ti.offset0, rows, _ptr(ds_d), _ptr(out), _ptr(ws), nbytes, stream))
    # reference: walk the plan on the host
    plan = tp.plan.view(5, -1)[:, :tp.G].cpu().numpy()
    pos = tp.tokens.view(5, -1)[3].cpu().numpy()
    ref = np.zeros((rows, H))
    mag = np.zeros((rows, H))
    reln = rel.numpy()
    for g in range(tp.G):
        c, T, sq, _, h = (int(v) for v in plan[:, g])
        p = pos[T:T + c]
        np.add.at(ref[:, h], reln[p][:, p].reshape(-1), ds[sq:sq + c * c].astype(np.float64))
        np.add.at(mag[:, h], reln[p][:, p].reshape(-1), np.abs(ds[sq:sq + c * c].astype(np.float64)))
    close(out.cpu().numpy(), ref, 1e-5, "d table", mag=mag)
    out2 = torch.empty_like(out)
    _lib.check(lib.sswin_bias_table_grad(_ptr(tp.plan), tp.g_cap, tp.G, _ptr(tp.tokens), tp.N, H, n, _ptr(ti.code),
                                         ti.offset0, rows, _ptr(ds_d), _ptr(out2), _ptr(ws), nbytes, stream))
    assert torch.equal(out, out2)                       # same bits on every run
    # the same gradient with the batches dealt from the plan's task descriptors (what the module calls when every
    # window holds at most 128 tokens): same reference, and the same bits on every run
    res = []
    for _ in range(2):
        o = torch.full((rows, H), float("nan"), device="cuda")
        _lib.check(lib.sswin_bias_table_grad_tasks(_ptr(tp.tasks), tp.g_cap, tp.bucket_counts, tp.G, _ptr(tp.tokens), tp.N, H, n,
                                                   _ptr(ti.code), ti.offset0, rows, _ptr(ds_d), _ptr(o), _ptr(ws), nbytes, stream))
        res.append(o)
    close(res[0].cpu().numpy(), ref, 1e-5, "d table, batches from the task descriptors", mag=mag)
    assert torch.equal(res[0], res[1])


def test_bias_from_table_matches_the_gather():
    """sswin_bias_from_table against table[relative_position_index].permute(2, 0, 1)
    (sparse_swin/swin3d_base.py:644-647): a copy, so bit-exact."""
    import ctypes as C
    from sparseswin3d_amd import _lib, fused
    from sparseswin3d_amd.window_attention import relative_position_index_3d
    lib = _lib.load()
    for ws, H in (((5, 5, 5), 3), ((3, 4, 2), 2), ((1, 1, 1), 1)):
        n = ws[0] * ws[1] * ws[2]
        rows = (2 * ws[0] - 1) * (2 * ws[1] - 1) * (2 * ws[2] - 1)
        index = relative_position_index_3d(ws).cuda()
        ti = fused.BiasTableIndex.build(index, rows)
        assert ti is not None
        table = torch.randn(rows, H, device="cuda")
        out = torch.full((H, n, n), float("nan"), device="cuda")
        _lib.check(lib.sswin_bias_from_table(C.c_void_p(table.data_ptr()), rows, H, C.c_void_p(ti.code.data_ptr()), ti.offset0,
                                             n, C.c_void_p(out.data_ptr()),
                                             C.c_void_p(torch.cuda.current_stream().cuda_stream)))
        ref = table[index.reshape(-1)].reshape(n, n, H).permute(2, 0, 1)
        assert torch.equal(out, ref)


def test_sums_over_nothing_are_zero():
    """The two reductions with an early exit for empty input (column sums of a matrix without rows, the bias-table
    gradient of a product without groups) write zeros, through a kernel rather than a memset node."""
    import ctypes as C
    from sparseswin3d_amd import _lib
    lib = _lib.load()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = torch.full((96,), 7.0, device="cuda")
    _lib.check(lib.sswin_column_sum(None, 0, 0, 96, C.c_void_p(out.data_ptr()), None, 0, stream))
    assert torch.count_nonzero(out) == 0
    table = torch.full((729, 3), 7.0, device="cuda")
    _lib.check(lib.sswin_bias_table_grad(None, 0, 0, None, 0, 3, 125, None, 0, 729, None, C.c_void_p(table.data_ptr()),
                                         None, 0, stream))
    assert torch.count_nonzero(table) == 0
    table.fill_(7.0)
    counts = (C.c_int64 * 4)(0, 0, 0, 0)
    _lib.check(lib.sswin_bias_table_grad_tasks(None, 0, counts, 0, None, 0, 3, 125, None, 0, 729, None,
                                               C.c_void_p(table.data_ptr()), None, 0, stream))
    assert torch.count_nonzero(table) == 0
    # nothing to do for a plan without groups: no launch, no pointer touched
    _lib.check(lib.sswin_group_softmax(0, None, 0, 0, 0, 3, 1, None, None, None, stream))
    _lib.check(lib.sswin_fused_score_grad(0, None, 0, 0, None, 0, 3, 16, 1, None, 0, 0, None, 0, 0, None, 0, 0, None, None, stream))


def test_entry_points_of_the_fused_path_reject_what_they_cannot_do():
    """Error behaviour of the entry points that take sizes the kernels are built around."""
    import ctypes as C
    from sparseswin3d_amd import _lib
    from sparseswin3d_amd.fused import TokenPlan, _ptr
    lib = _lib.load()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(1)
    ind = ragged_window_indices(rng, [3, 40, 7], 125)
    tp = TokenPlan(torch.from_numpy(ind).cuda(), 3, 125, 2)
    x = torch.zeros(tp.A, device="cuda")
    with pytest.raises(RuntimeError, match="384 at most"):
        _lib.check(lib.sswin_group_softmax(0, _ptr(tp.plan), tp.g_cap, tp.G, tp.N, tp.H, 385, _ptr(x), None, _ptr(x), stream))
    with pytest.raises(RuntimeError, match="null pointer"):
        _lib.check(lib.sswin_group_softmax(1, _ptr(tp.plan), tp.g_cap, tp.G, tp.N, tp.H, tp.c_max, _ptr(x), None, _ptr(x), stream))
    table = torch.zeros(729, 2, device="cuda")
    short = (C.c_int64 * 4)(2, 0, 0, 0)                      # fewer groups in the buckets than the plan holds
    with pytest.raises(RuntimeError, match="have no descriptor"):
        _lib.check(lib.sswin_bias_table_grad_tasks(_ptr(tp.tasks), tp.g_cap, short, tp.G, _ptr(tp.tokens), tp.N, 2, 125,
                                                   _ptr(x), 0, 729, _ptr(x), _ptr(table), _ptr(x), 1 << 30, stream))
