"""Shifted-window block and stage built around :class:`WindowAttentionSparse`.

Host-side mirror of the caller side of the reference's ``sparse_swin/swin3d_base.py``:
window/shift clamping (ref ``:276-300``), sparse window partition / reverse (``:336-413``),
padding and cyclic roll of voxel indices (``:501-554``), the 27-region shift mask
(``:416-452``), ``SwinTransformerBlock`` (``:680-782``) and ``BasicLayer`` (``:785-873``).
All of it is integer arithmetic on an [N, 4] (batch, d, h, w) int32 index tensor plus plain
torch modules; the attention itself runs in the HIP operators.
"""
from __future__ import annotations

import collections
import copy
import ctypes as C
from typing import List, Sequence

import torch
import torch.nn as nn
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from . import _lib
from .window_attention import WindowAttentionSparse, prefetch_plans, replace_feature, tall_linear

_DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def _i32x3(v):
    return (C.c_int32 * 3)(*(int(e) for e in v))


def _stream(device):
    return _lib.stream_handle(device)


def get_window_size(x_size, window_size, shift_size=None):
    """Clamp the window (and zero the shift) along axes where the grid is not larger."""
    ws = list(window_size)
    ss = list(shift_size) if shift_size is not None else None
    for i, extent in enumerate(x_size):
        if extent <= window_size[i]:
            ws[i] = extent
            if ss is not None:
                ss[i] = 0
    return tuple(ws) if ss is None else (tuple(ws), tuple(ss))


def _window_grid(spatial, window_size):
    return [s // w for s, w in zip(spatial, window_size)]


def window_partition_sparse(x, window_size):
    """(batch, d, h, w) voxel indices -> (window id, position inside the window); in place."""
    d, h, w = x.spatial_shape
    nd, nh, nw = _window_grid((d, h, w), window_size)
    wd, wh, ww = window_size
    i = x.indices
    window = i[:, 0] * (nd * nh * nw) + (i[:, 1] // wd) * (nh * nw) + (i[:, 2] // wh) * nw + (i[:, 3] // ww)
    pos = (i[:, 1] % wd) * (wh * ww) + (i[:, 2] % wh) * ww + (i[:, 3] % ww)
    batch = x.batch_size
    x.indices = torch.stack([window, pos], dim=1)
    x.spatial_shape = (wd * wh * ww,)
    x.batch_size = batch * nd * nh * nw
    return x


def window_reverse_sparse(x, original_shape, window_size):
    """Inverse of :func:`window_partition_sparse`; in place."""
    b, d, h, w, _ = original_shape
    nd, nh, nw = _window_grid((d, h, w), window_size)
    wd, wh, ww = window_size
    window, pos = x.indices[:, 0], x.indices[:, 1]
    per_batch = nd * nh * nw
    batch, cell = window // per_batch, window % per_batch
    zd = (cell // (nh * nw)) * wd + pos // (wh * ww)
    zh = ((cell % (nh * nw)) // nw) * wh + (pos % (wh * ww)) // ww
    zw = (cell % nw) * ww + pos % ww
    x.indices = torch.stack([batch, zd, zh, zw], dim=1)
    x.spatial_shape = [d, h, w]
    x.batch_size = b
    return x


def pad_sparse_tensor(x, pad_l, pad_r, pad_t, pad_b, pad_d0=0, pad_d1=0):
    """Grow the spatial shape; leading pads shift the indices."""
    idx = x.indices.clone()
    idx[:, 1] += pad_d0
    idx[:, 2] += pad_t
    idx[:, 3] += pad_l
    x.indices = idx
    x.spatial_shape = (x.spatial_shape[0] + pad_d0 + pad_d1, x.spatial_shape[1] + pad_t + pad_b,
                       x.spatial_shape[2] + pad_l + pad_r)
    return x


def roll_sparse_tensor(x, shifts, dims):
    """Cyclic shift of voxel indices along spatial dims 1..3."""
    idx = x.indices.clone()
    for shift, dim in zip(shifts, dims):
        if dim < 1 or dim > 3:
            raise ValueError("Dimension out of bounds for spatial shift. Must be 1, 2, or 3.")
        idx[:, dim] = (idx[:, dim] + shift) % x.spatial_shape[dim - 1]
    x.indices = idx
    return x


def window_partition(x: torch.Tensor, window_size: List[int]) -> torch.Tensor:
    """Dense [b, d, h, w, c] -> [b * windows, tokens per window, c]."""
    b, d, h, w, c = x.shape
    wd, wh, ww = window_size
    x = x.view(b, d // wd, wd, h // wh, wh, w // ww, ww, c)
    return x.permute(0, 1, 3, 5, 2, 4, 6, 7).contiguous().view(-1, wd * wh * ww, c)


def compute_mask(dims: List[int], window_size: List[int], shift_size: List[int], device, private: bool = False) -> torch.Tensor:
    """int8 [windows, tokens per window] region ids (27 regions) of the shifted grid.

    The reference assigns 27 slices of a dense volume and partitions it (ref ``:416-452``);
    here one kernel evaluates the region of every (window, position) directly.

    The returned tensor is shared: every call with the same shapes, device and stream gets the same tensor
    (``private=True`` returns a copy of its own).  A caller that writes into a shared mask is detected by the tensor's
    version counter at the next call, which then builds the mask again."""
    device = torch.device(device)
    if device.type != "cuda":
        raise RuntimeError("compute_mask runs on the GPU only; there is no CPU fallback")
    if device.index is None:
        device = torch.device("cuda", torch.cuda.current_device())
    # the mask is a function of the three shapes alone, and a stage asks for the same one in every forward pass:
    # the last few are kept (per device and stream, read-only by convention), 256 MB at most
    key = (tuple(int(e) for e in dims), tuple(int(e) for e in window_size), tuple(int(e) for e in shift_size),
           device.index, torch.cuda.current_stream(device).cuda_stream)
    mask = _MASKS.get(key)
    if mask is not None and mask._version == 0:              # written to by a caller: not the mask any more
        _MASKS.move_to_end(key)
        return mask.clone() if private else mask
    windows = 1
    for extent, w in zip(dims, window_size):
        windows *= extent // w
    n = window_size[0] * window_size[1] * window_size[2]
    mask = torch.empty((windows, n), dtype=torch.int8, device=device)
    with _lib.on_device(device):
        _lib.check(_lib.load().sswin_shift_mask(_i32x3(dims), _i32x3(window_size), _i32x3(shift_size), _ptr(mask),
                                                _stream(device)))
    _MASKS[key] = mask
    while len(_MASKS) > 8 or (len(_MASKS) > 1 and sum(m.numel() for m in _MASKS.values()) > _MASK_CACHE_BYTES):
        _MASKS.popitem(last=False)
    return mask.clone() if private else mask


_MASKS = collections.OrderedDict()
_MASK_CACHE_BYTES = 256 << 20


def sparse_window_indices(indices: torch.Tensor, batch_size: int, dims: Sequence[int], window_size: Sequence[int],
                          shift_size: Sequence[int] = (0, 0, 0)) -> torch.Tensor:
    """int32 [N, 4] (batch, d, h, w) -> int32 [N, 2] (window slot, position) of the grid of
    padded extents ``dims`` rolled by ``-shift_size``: :func:`pad_sparse_tensor` (trailing pads),
    :func:`roll_sparse_tensor` and :func:`window_partition_sparse` in one kernel."""
    if indices.device.type != "cuda":
        raise RuntimeError("sparse_window_indices runs on the GPU only; there is no CPU fallback")
    if indices.dtype != torch.int32 or indices.dim() != 2 or indices.shape[1] != 4:
        raise RuntimeError("sparse_window_indices: indices must be int32 [N, 4]")
    indices = indices.contiguous()
    out = torch.empty((indices.shape[0], 2), dtype=torch.int32, device=indices.device)
    with _lib.on_device(indices.device):
        _lib.check(_lib.load().sswin_window_indices(_ptr(indices), indices.shape[0], int(batch_size), _i32x3(dims),
                                                    _i32x3(window_size), _i32x3(shift_size), _ptr(out),
                                                    _stream(indices.device)))
    return out


class _PoolWindows(Function):
    """Sum or mean of the feature rows of every non-empty window, in (window, position) order."""

    @staticmethod
    def forward(ctx, features, plan, mean):
        features = features.contiguous()
        M, channels = plan.windows, features.shape[1]
        out = torch.empty((M, channels), dtype=features.dtype, device=features.device)
        with _lib.on_device(features.device):
            _lib.check(_lib.load().sswin_pool_windows(
                _DTYPE_CODE[features.dtype], 0, 1 if mean else 0, _ptr(plan.plan), plan.g_cap, M, _ptr(plan.tokens),
                plan.N, _ptr(features), channels, channels, _ptr(out), channels, _stream(features.device)))
        ctx.plan, ctx.mean = plan, mean
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        plan = ctx.plan
        grad = grad.contiguous()
        channels = grad.shape[1]
        g_in = torch.empty((plan.N, channels), dtype=grad.dtype, device=grad.device)
        with _lib.on_device(grad.device):
            _lib.check(_lib.load().sswin_pool_windows(
                _DTYPE_CODE[grad.dtype], 1, 1 if ctx.mean else 0, _ptr(plan.plan), plan.g_cap, plan.windows,
                _ptr(plan.tokens), plan.N, _ptr(grad), channels, channels, _ptr(g_in), channels, _stream(grad.device)))
        return g_in, None, None


def downsample_plan_request(x, factor: int = 2):
    """What the token plan of the ``floor(coord / factor)`` merge is built from: the arguments
    ``(indices, window slots, positions per window, heads = 1, tasks = False, order_only = True)`` of
    ``TokenPlan`` / ``TokenPlan.batch``.  It depends on the voxel coordinates only, so a stage can enqueue it together with
    the plans of its attention blocks and hand the plan to :func:`downsample_plan` later."""
    f = int(factor)
    dims = [-(-int(e) // f) * f for e in x.spatial_shape]
    idx = sparse_window_indices(x.indices, x.batch_size, dims, (f, f, f))
    slots = x.batch_size * (dims[0] // f) * (dims[1] // f) * (dims[2] // f)
    return idx, slots, f * f * f, 1, False, True


def downsample_plan(x, factor: int = 2, plan=None):
    """Token plan of the ``floor(coord / factor)`` merge: windows of ``factor``^3 cells, one head.
    Returns ``(plan, merged coordinates int32 [M, 4], merged spatial shape)``.  ``plan``: a plan made earlier
    from :func:`downsample_plan_request` of the same voxels (possibly still in flight)."""
    from .fused import TokenPlan
    f = int(factor)
    dims = [-(-int(e) // f) * f for e in x.spatial_shape]
    win = (f, f, f)
    if plan is None:
        req = downsample_plan_request(x, f)
        plan = TokenPlan(*req[:4], tasks=req[4], order_only=req[5])
    plan.finish()
    coords = torch.empty((plan.windows, 4), dtype=torch.int32, device=x.indices.device)
    with _lib.on_device(coords.device):
        _lib.check(_lib.load().sswin_window_coords(_ptr(plan.plan), plan.g_cap, plan.windows, _i32x3(dims), _i32x3(win),
                                                   _ptr(coords), _stream(coords.device)))
    return plan, coords, [e // f for e in dims]


class PoolDownsample(nn.Module):
    """Stride-2 merge between stages: voxels with the same ``floor(coord / 2)`` become one voxel.

    Stands where the reference builds ``spconv.SparseConv3d(dim, 2*dim, kernel_size=2, stride=2)``
    (ref ``:950-976``; spconv is not available here): same output coordinates (deduplicated
    ``floor(coord/2)``, ascending (batch, d, h, w)), the children's rows averaged instead of
    weighted per tap, then ``norm`` and a bias-free ``Linear(dim, 2*dim)``."""

    def __init__(self, dim: int, norm_layer=nn.LayerNorm, spatial_dims: int = 3, indice_key=None) -> None:
        super().__init__()
        if spatial_dims != 3:
            raise ValueError("PoolDownsample handles three spatial dimensions")
        self.dim = dim
        self.norm = norm_layer(dim) if norm_layer is not None else nn.Identity()
        self.reduction = nn.Linear(dim, 2 * dim, bias=False)

    def plan_request(self, x):
        """Arguments of the token plan this merge needs for ``x``'s voxels (see :func:`downsample_plan_request`)."""
        return downsample_plan_request(x, 2)

    def forward(self, x, plan=None):
        plan, coords, shape = downsample_plan(x, 2, plan)
        pooled = _PoolWindows.apply(x.features, plan, True)
        out = copy.copy(x)
        out.indices, out.spatial_shape = coords, shape
        out.features = tall_linear(self.norm(pooled), self.reduction)
        return out


_ACTIVATIONS = {"GELU": nn.GELU, "RELU": nn.ReLU, "LEAKYRELU": nn.LeakyReLU, "SILU": nn.SiLU, "SWISH": nn.SiLU,
                "TANH": nn.Tanh, "SIGMOID": nn.Sigmoid, "ELU": nn.ELU}


def get_act_layer(name: str):
    try:
        return _ACTIVATIONS[name.upper()]()
    except KeyError:
        raise ValueError(f"Unknown activation '{name}'.") from None


class MLP(nn.Module):
    """Two-layer feed-forward block: linear, activation, dropout, linear, dropout."""

    def __init__(self, hidden_size: int, mlp_dim: int, dropout_rate: float = 0.0, act="GELU"):
        super().__init__()
        if not 0 <= dropout_rate <= 1:
            raise ValueError("dropout_rate should be between 0 and 1.")
        self.linear1 = nn.Linear(hidden_size, mlp_dim or hidden_size)
        self.linear2 = nn.Linear(mlp_dim or hidden_size, hidden_size)
        self.fn = get_act_layer(act) if isinstance(act, str) else act
        self.drop1 = nn.Dropout(dropout_rate)
        self.drop2 = nn.Dropout(dropout_rate)

    def forward(self, x):
        # tall 2-D fp32 inputs on the GPU take the projection kernels of the attention (same results as
        # nn.Linear to fp32 rounding); anything else is nn.Linear itself
        return self.drop2(tall_linear(self.drop1(self.fn(tall_linear(x, self.linear1))), self.linear2))


class DropPath(nn.Module):
    """Stochastic depth: drops whole rows with probability ``drop_prob`` during training."""

    def __init__(self, drop_prob: float = 0.0, scale_by_keep: bool = True):
        super().__init__()
        if not 0 <= drop_prob <= 1:
            raise ValueError("Drop path prob should be between 0 and 1.")
        self.drop_prob = drop_prob
        self.scale_by_keep = scale_by_keep

    def forward(self, x):
        if self.drop_prob == 0.0 or not self.training:
            return x
        keep = 1.0 - self.drop_prob
        mask = x.new_empty((x.shape[0],) + (1,) * (x.ndim - 1)).bernoulli_(keep)
        if keep > 0.0 and self.scale_by_keep:
            mask.div_(keep)
        return x * mask


class SwinTransformerBlock(nn.Module):
    """norm -> (shifted) window attention -> residual -> norm -> MLP -> residual."""

    def __init__(self, dim: int, num_heads: int, window_size: Sequence[int], shift_size: Sequence[int],
                 mlp_ratio: float = 4.0, qkv_bias: bool = True, drop: float = 0.0, attn_drop: float = 0.0,
                 drop_path: float = 0.0, act_layer: str = "GELU", norm_layer=nn.LayerNorm,
                 use_checkpoint: bool = False) -> None:
        super().__init__()
        self.dim = dim
        self.num_heads = num_heads
        self.window_size = window_size
        self.shift_size = shift_size
        self.mlp_ratio = mlp_ratio
        self.use_checkpoint = use_checkpoint
        self.norm1 = norm_layer(dim)
        self.attn = WindowAttentionSparse(dim, window_size=self.window_size, num_heads=num_heads,
                                          qkv_bias=qkv_bias, attn_drop=attn_drop, proj_drop=drop)
        self.drop_path = DropPath(drop_path) if drop_path > 0.0 else nn.Identity()
        self.norm2 = norm_layer(dim)
        self.mlp = MLP(hidden_size=dim, mlp_dim=int(dim * mlp_ratio), act=act_layer, dropout_rate=drop)

    def window_view(self, x):
        """``x`` seen as (window, position) tokens for this block's shift, and whether the block is shifted."""
        d, h, w = x.spatial_shape
        window_size, shift_size = get_window_size((d, h, w), self.window_size, self.shift_size)
        shifted = any(s > 0 for s in shift_size)
        # pad (trailing), roll by -shift and partition in one pass; the voxel list itself keeps its
        # (batch, d, h, w) indices, so the reverse / roll back / un-pad of the reference
        # (ref :760-771) has nothing left to do.  Blocks of a stage with the same shift share the
        # window indices and the token plan through ``x.window_cache``.
        cache = getattr(x, "window_cache", None)
        key = (tuple(window_size), tuple(shift_size))
        view = cache.get(key) if cache is not None else None
        if view is None:
            dims = [-(-e // ws) * ws for e, ws in zip((d, h, w), window_size)]
            view = copy.copy(x)
            view.window_cache = None
            view.indices = sparse_window_indices(x.indices, x.batch_size, dims, window_size, shift_size)
            view.spatial_shape = (window_size[0] * window_size[1] * window_size[2],)
            view.batch_size = x.batch_size * (dims[0] // window_size[0]) * (dims[1] // window_size[1]) * (dims[2] // window_size[2])
            view.plan_cache = {}
            if cache is not None:
                cache[key] = view
        return replace_feature(view, x.features), shifted

    def prefetch(self, x):
        """Enqueue this block's window indices and token plan (see ``WindowAttentionSparse.prefetch_plan``);
        needs ``x.window_cache``."""
        if getattr(x, "window_cache", None) is not None:
            self.attn.prefetch_plan(self.window_view(x)[0])

    @staticmethod
    def prefetch_all(blocks, x, extra=()):
        """The same for all blocks of a stage at once: their token plans share one set of launches.  ``extra``:
        further ``TokenPlan`` argument tuples to build in the same launches; their plans are returned."""
        if getattr(x, "window_cache", None) is None:
            return prefetch_plans([], extra)
        return prefetch_plans([(blk.attn, blk.window_view(x)[0]) for blk in blocks], extra)[len(blocks):]

    def forward_part1(self, x, mask_matrix):
        x = replace_feature(x, self.norm1(x.features))
        view, shifted = self.window_view(x)
        out = self.attn(view, mask=mask_matrix if shifted else None)
        return replace_feature(x, out.features)

    def forward_part2(self, x):
        x = replace_feature(x, self.norm2(x.features))
        return replace_feature(x, self.drop_path(self.mlp(x.features)))

    def forward(self, x, mask_matrix):
        shortcut = x
        x = self.forward_part1(x, mask_matrix)
        x = replace_feature(x, shortcut.features + self.drop_path(x.features))
        return replace_feature(x, x.features + self.forward_part2(x).features)


class BasicLayer(nn.Module):
    """One stage: ``depth`` blocks alternating no shift / shift by half a window."""

    def __init__(self, dim: int, depth: int, num_heads: int, window_size: Sequence[int], drop_path,
                 mlp_ratio: float = 4.0, qkv_bias: bool = False, drop: float = 0.0, attn_drop: float = 0.0,
                 norm_layer=nn.LayerNorm, downsample=None, use_checkpoint: bool = False,
                 indice_key=None) -> None:
        super().__init__()
        self.window_size = window_size
        self.shift_size = tuple(i // 2 for i in window_size)
        self.no_shift = tuple(0 for _ in window_size)
        self.depth = depth
        self.use_checkpoint = use_checkpoint
        self.blocks = nn.ModuleList([
            SwinTransformerBlock(dim=dim, num_heads=num_heads, window_size=self.window_size,
                                 shift_size=self.no_shift if i % 2 == 0 else self.shift_size,
                                 mlp_ratio=mlp_ratio, qkv_bias=qkv_bias, drop=drop, attn_drop=attn_drop,
                                 drop_path=drop_path[i] if isinstance(drop_path, list) else drop_path,
                                 norm_layer=norm_layer, use_checkpoint=use_checkpoint)
            for i in range(depth)])
        self.downsample = downsample
        if callable(self.downsample):
            self.downsample = downsample(dim=dim, norm_layer=norm_layer, spatial_dims=len(self.window_size),
                                         indice_key=indice_key)

    def forward(self, x):
        d, h, w = x.spatial_shape
        window_size, shift_size = get_window_size((d, h, w), self.window_size, self.shift_size)
        padded = [-(-s // ws) * ws for s, ws in zip((d, h, w), window_size)]
        # The mask is built whenever the layer has a shift; unshifted blocks ignore it.
        attn_mask = compute_mask(padded, window_size, shift_size, x.features.device)
        x = copy.copy(x)
        x.window_cache = {}                      # (window, shift) -> window indices and token plans of this stage
        # the plans need the voxel indices only: all of them are enqueued now, so that only the first block waits
        # for totals from the GPU
        # (and the plan of the stride-2 merge behind the blocks, when the merge can say what it needs)
        merge_plan = None
        if self.downsample is not None and hasattr(self.downsample, "plan_request"):
            merge_plan, = SwinTransformerBlock.prefetch_all(self.blocks, x, [self.downsample.plan_request(x)])
        else:
            SwinTransformerBlock.prefetch_all(self.blocks, x)
        for blk in self.blocks:
            x = blk(x, attn_mask)
        x.window_cache = None
        if self.downsample is not None:
            x = self.downsample(x, merge_plan) if merge_plan is not None else self.downsample(x)
        return x
