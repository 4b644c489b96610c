"""Seeded synthetic voxel scenes and window-partition index arithmetic (numpy only).

The scenes stand in for ScanNet rooms, which cannot be downloaded here.  Every
function is deterministic in its ``seed`` so that the CPU oracle, the HIP path
and the benchmark all see identical inputs.

The window-partition arithmetic restates, as pure int32 math on an ``[N, 4]``
``(batch, z, y, x)`` coordinate array, what the reference does on a spconv
tensor: pad to a multiple of the window (reference
``sparse_swin/swin3d_base.py:745-749``), cyclic roll by ``-shift``
(``:529-554``), and ``(window_id, pos_in_window)`` (``:336-372``).
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np


# --------------------------------------------------------------------------- #
# geometry
# --------------------------------------------------------------------------- #
def _box_surface(lo, hi):
    """Integer voxels on the surface of the axis-aligned box [lo, hi] (inclusive)."""
    z0, y0, x0 = lo
    z1, y1, x1 = hi
    zz, yy, xx = np.meshgrid(
        np.arange(z0, z1 + 1), np.arange(y0, y1 + 1), np.arange(x0, x1 + 1), indexing="ij"
    )
    on = (
        (zz == z0) | (zz == z1) | (yy == y0) | (yy == y1) | (xx == x0) | (xx == x1)
    )
    return np.stack([zz[on], yy[on], xx[on]], axis=1)


def _dedupe(coords, grid):
    """Drop duplicate voxels, keep first occurrence order-independent (sorted by key)."""
    key = (coords[:, 0].astype(np.int64) * grid[1] + coords[:, 1]) * grid[2] + coords[:, 2]
    _, first = np.unique(key, return_index=True)
    return coords[np.sort(first)]


def box_surfaces_scene(seed: int = 1, grid=(128, 128, 128), n_boxes: int = 8):
    """Surfaces of ``n_boxes`` random axis-aligned boxes inside ``grid``.

    Returns int32 ``[N, 3]`` (z, y, x) voxel coordinates in a random (seeded) order,
    so the caller's voxel order is unrelated to window order.
    """
    rng = np.random.default_rng(seed)
    parts = []
    g = np.asarray(grid)
    for _ in range(n_boxes):
        size = rng.integers(g // 10, g // 4 + 1)
        lo = np.array([rng.integers(0, g[i] - size[i]) for i in range(3)])
        parts.append(_box_surface(lo, lo + size))
    c = _dedupe(np.concatenate(parts, 0), grid)
    c = c[rng.permutation(len(c))]
    return c.astype(np.int32)


def room_scene(seed: int = 2, grid=(256, 256, 96), footprint=(168, 152), wall_height=52,
               n_furniture: int = 20, rough: float = 0.5):
    """A ScanNet-like room voxelised on ``grid`` = (x, y, z) extents, z up.

    Floor, four walls and ``n_furniture`` random box surfaces standing on the floor.  The floor
    and the walls are rough, as scanned surfaces are: a fraction ``rough`` of their voxels sits one
    voxel further along the surface normal, and the two levels straddle a boundary of the
    ``floor(coord / 2)`` grid, so that down-sampling keeps about 1/3 of the voxels (a perfectly
    flat one-voxel sheet would keep 1/4).  Returned coordinates are int32 ``[N, 3]`` ordered
    (d, h, w) = (x, y, z) in a seeded random order.
    """
    rng = np.random.default_rng(seed)
    jit = np.random.default_rng(seed + 1000)          # roughness: its own stream, the furniture layout does not move
    gx, gy, gz = grid
    fx, fy = footprint
    ox, oy = (gx - fx) // 2, (gy - fy) // 2
    parts = []

    def level(size):
        return (jit.random(size) < rough).astype(np.int64)

    # floor at z = 1 or 2
    xx, yy = np.meshgrid(np.arange(ox, ox + fx), np.arange(oy, oy + fy), indexing="ij")
    parts.append(np.stack([xx.ravel(), yy.ravel(), 1 + level(xx.size)], 1))
    # walls, displaced outwards
    for x, sign in ((ox, -1), (ox + fx - 1, 1)):
        yy, zz = np.meshgrid(np.arange(oy, oy + fy), np.arange(wall_height), indexing="ij")
        parts.append(np.stack([x + sign * level(yy.size), yy.ravel(), zz.ravel()], 1))
    for y, sign in ((oy, -1), (oy + fy - 1, 1)):
        xx, zz = np.meshgrid(np.arange(ox, ox + fx), np.arange(wall_height), indexing="ij")
        parts.append(np.stack([xx.ravel(), y + sign * level(xx.size), zz.ravel()], 1))
    # furniture: boxes standing on the floor
    for _ in range(n_furniture):
        sx, sy = rng.integers(10, 36, size=2)
        sz = rng.integers(8, 32)
        x0 = rng.integers(ox + 1, ox + fx - sx - 1)
        y0 = rng.integers(oy + 1, oy + fy - sy - 1)
        parts.append(_box_surface((x0, y0, 0), (x0 + sx, y0 + sy, sz)))
    c = _dedupe(np.concatenate(parts, 0), grid)
    c = c[rng.permutation(len(c))]
    return c.astype(np.int32)


def filled_blob_scene(seed: int = 4, grid=(32, 32, 12), fill: float = 0.9):
    """Volumetric (mostly filled) scene: windows hold close to ws^3 tokens."""
    rng = np.random.default_rng(seed)
    zz, yy, xx = np.meshgrid(*[np.arange(g) for g in grid], indexing="ij")
    c = np.stack([zz.ravel(), yy.ravel(), xx.ravel()], 1)
    keep = rng.random(len(c)) < fill
    c = c[keep]
    c = c[rng.permutation(len(c))]
    return c.astype(np.int32)


def volumetric_scene(seed: int = 4, coarse=(30, 30, 10), levels: int = 3, fill: float = 0.9, density: float = 0.5):
    """A volumetric scene on the fine grid ``coarse * 2**levels``: a fraction ``fill`` of the cells of the
    coarse grid is solid, and a solid cell holds a fraction ``density`` of its fine voxels (at least one).
    ``levels`` passes of :func:`downsample_coords` give back exactly the solid coarse cells."""
    rng = np.random.default_rng(seed)
    f = 2 ** levels
    solid = rng.random(coarse) < fill
    fine = np.repeat(np.repeat(np.repeat(solid, f, 0), f, 1), f, 2) & (rng.random(tuple(g * f for g in coarse)) < density)
    # every solid cell keeps at least its first fine voxel
    fine[::f, ::f, ::f] |= solid
    c = np.argwhere(fine)
    c = c[rng.permutation(len(c))]
    return c.astype(np.int32)


def downsample_coords(coords: np.ndarray, factor: int = 2):
    """floor(coord / factor) with dedupe.

    Returns ``(new_coords [M,3] int32, inverse [N] int64)`` where ``inverse[i]`` is the
    merged voxel that input voxel ``i`` fell into (for mean-pooling features).  The merged
    voxels keep the order of their first contributing input voxel.
    """
    q = coords // factor
    span = q.max(0).astype(np.int64) + 1
    key = (q[:, 0].astype(np.int64) * span[1] + q[:, 1]) * span[2] + q[:, 2]
    uniq, first, inv = np.unique(key, return_index=True, return_inverse=True)
    order = np.argsort(first, kind="stable")        # merged voxels in first-seen order
    rank = np.empty_like(order)
    rank[order] = np.arange(len(order))
    return q[first[order]].astype(np.int32), rank[inv]


def mean_pool(features: np.ndarray, inverse: np.ndarray, m: int):
    """Average the features of voxels merged by :func:`downsample_coords`."""
    out = np.zeros((m, features.shape[1]), dtype=np.float64)
    np.add.at(out, inverse, features)
    cnt = np.bincount(inverse, minlength=m).astype(np.float64)
    return (out / cnt[:, None]).astype(features.dtype)


def with_batch(coords_list):
    """Concatenate per-room ``[N_i, 3]`` coords into ``[N, 4]`` (batch, d, h, w) int32.

    Also returns the int32 cumulative batch offsets (Pointcept's ``offset`` convention).
    """
    out = []
    for b, c in enumerate(coords_list):
        out.append(np.concatenate([np.full((len(c), 1), b, np.int32), c.astype(np.int32)], 1))
    offsets = np.cumsum([len(c) for c in coords_list]).astype(np.int32)
    return np.concatenate(out, 0), offsets


# --------------------------------------------------------------------------- #
# window partition arithmetic
# --------------------------------------------------------------------------- #
def effective_window(spatial_shape, window_size, shift_size):
    """Clamp window/shift when the grid is not larger than the window.

    Restates ``get_window_size`` (reference ``sparse_swin/swin3d_base.py:276-300``).
    """
    ws = list(window_size)
    ss = list(shift_size)
    for i, extent in enumerate(spatial_shape):
        if extent <= window_size[i]:
            ws[i] = extent
            ss[i] = 0
    return tuple(ws), tuple(ss)


def padded_shape(spatial_shape, window_size):
    return tuple(int(-(-s // w) * w) for s, w in zip(spatial_shape, window_size))


def window_indices(coords4: np.ndarray, spatial_shape, window_size, shift_size=(0, 0, 0)):
    """``(window_id, pos_in_window)`` int32 ``[N, 2]`` for ``[N, 4]`` (b, d, h, w) voxels.

    pad (right/bottom only) -> roll by ``-shift`` modulo the padded extent -> partition.
    Returns ``(indices [N,2] int32, n_windows_per_batch, tokens_per_window)``.
    """
    ws = tuple(int(w) for w in window_size)
    pshape = padded_shape(spatial_shape, ws)
    c = coords4.astype(np.int64)
    zyx = [(c[:, 1 + i] - shift_size[i]) % pshape[i] for i in range(3)]
    nw = [pshape[i] // ws[i] for i in range(3)]
    win = (c[:, 0] * nw[0] * nw[1] * nw[2]
           + (zyx[0] // ws[0]) * nw[1] * nw[2]
           + (zyx[1] // ws[1]) * nw[2]
           + (zyx[2] // ws[2]))
    pos = (zyx[0] % ws[0]) * ws[1] * ws[2] + (zyx[1] % ws[1]) * ws[2] + (zyx[2] % ws[2])
    idx = np.stack([win, pos], 1).astype(np.int32)
    return idx, nw[0] * nw[1] * nw[2], ws[0] * ws[1] * ws[2]


def shift_region_mask(pshape, window_size, shift_size):
    """int8 ``[nW, n]`` region ids of the shifted-window mask.

    The padded volume is cut into 27 regions by the slices ``[:-ws]``, ``[-ws:-shift]``,
    ``[-shift:]`` along each axis and partitioned into windows
    (reference ``sparse_swin/swin3d_base.py:436-452``).
    """
    d, h, w = pshape
    img = np.zeros((d, h, w), np.int8)
    cnt = 0

    def cuts(ws, ss):
        return (slice(-ws), slice(-ws, -ss), slice(-ss, None))

    for sd in cuts(window_size[0], shift_size[0]):
        for sh in cuts(window_size[1], shift_size[1]):
            for sw in cuts(window_size[2], shift_size[2]):
                img[sd, sh, sw] = cnt
                cnt += 1
    wd, wh, ww = window_size
    v = img.reshape(d // wd, wd, h // wh, wh, w // ww, ww).transpose(0, 2, 4, 1, 3, 5)
    return np.ascontiguousarray(v.reshape(-1, wd * wh * ww))


@dataclass
class SceneStats:
    n_voxels: int
    n_window_slots: int
    n_windows: int          # non-empty
    c_max: int
    c_mean: float
    sum_c2: int             # S2 = sum over windows of c^2
    histogram: np.ndarray   # histogram[c] = number of windows holding c tokens

    def describe(self, heads: int, head_dim: int = 32):
        e = self.n_voxels * heads * head_dim
        return {
            "N": self.n_voxels, "windows": self.n_windows, "G": self.n_windows * heads,
            "c_max": self.c_max, "c_mean": round(self.c_mean, 2), "S2": self.sum_c2,
            "E": e, "A": heads * self.sum_c2,
        }


def scene_stats(win_idx: np.ndarray, n_window_slots: int) -> SceneStats:
    cnt = np.bincount(win_idx[:, 0], minlength=n_window_slots)
    nz = cnt[cnt > 0]
    return SceneStats(
        n_voxels=len(win_idx), n_window_slots=int(n_window_slots), n_windows=int(len(nz)),
        c_max=int(nz.max()), c_mean=float(nz.mean()), sum_c2=int((nz.astype(np.int64) ** 2).sum()),
        histogram=np.bincount(nz),
    )


# --------------------------------------------------------------------------- #
# the five named configurations
# --------------------------------------------------------------------------- #
@dataclass
class Workload:
    name: str
    coords4: np.ndarray          # [N,4] int32 (batch, d, h, w)
    spatial_shape: tuple
    batch_size: int
    dim: int
    heads: int
    window: tuple = (5, 5, 5)
    dtype: str = "fp32"


def config1():
    c = box_surfaces_scene(seed=1, grid=(128, 128, 128), n_boxes=8)
    c4, _ = with_batch([c])
    return Workload("cfg1_boxes20k", c4, (128, 128, 128), 1, 96, 3)


def config2():
    c = room_scene(seed=2)
    c4, _ = with_batch([c])
    return Workload("cfg2_room100k", c4, (256, 256, 96), 1, 96, 3)


def config3():
    c = room_scene(seed=2)
    c2, _ = downsample_coords(c, 2)
    c4, _ = with_batch([c2])
    return Workload("cfg3_room40k", c4, (128, 128, 48), 1, 192, 6)


def config4():
    # a volumetric scene of about two million voxels on a 240 x 240 x 80 grid, down-sampled by floor(coord / 2)
    # three times: about 8k voxels, most windows hold 100-125 tokens
    c = volumetric_scene(seed=4, coarse=(30, 30, 10), levels=3, fill=0.9)
    for _ in range(3):
        c, _ = downsample_coords(c, 2)
    c4, _ = with_batch([c])
    return Workload("cfg4_dense8k", c4, (30, 30, 10), 1, 768, 24, dtype="bf16")


def config_ref7():
    """The room of configuration 2 in the reference's own attention setting (config/scannet/semseg-swin-0-base.py:11-31:
    window 7, 48 channels in 3 heads of 16)."""
    c = room_scene(seed=2)
    c4, _ = with_batch([c])
    return Workload("ref7_room100k_window7_heads16", c4, (256, 256, 96), 1, 48, 3, window=(7, 7, 7))


def config5_rooms(n_rooms: int = 4):
    rooms = [room_scene(seed=50 + i) for i in range(n_rooms)]
    c4, offsets = with_batch(rooms)
    return Workload("cfg5_rooms400k", c4, (256, 256, 96), n_rooms, 96, 3, dtype="bf16"), offsets
