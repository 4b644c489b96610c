"""CPU restatement of the voxel-grid glue of a stage (test infrastructure; never imported by the
product).  Each function follows the reference's own sequence of steps on numpy arrays.

* window_indices: pad_sparse_tensor -> roll_sparse_tensor -> window_partition_sparse
  (sparse_swin/swin3d_base.py:501-527, 529-554, 336-372), one step after the other.
* shift_mask: compute_mask (:416-452): a dense int8 volume, 27 slice assignments, dense
  window_partition (:375-413).
* downsample: output coordinates and child-to-output pairs of the stride-2, kernel-2 sparse
  convolution the reference places between stages (:950-976; spconv's rule: out = floor(in / 2),
  outputs deduplicated), with mean pooling of the children as the feature rule.

Pins (tests/test_oracle_pins.py): torch.roll + reshape on a dense id volume for window_indices, a
per-element brute force for shift_mask, numpy.unique / numpy.add.at for downsample."""
import numpy as np


def get_window_size(x_size, window_size, shift_size):
    """swin3d_base.py:276-300"""
    ws, ss = list(window_size), list(shift_size)
    for i in range(len(x_size)):
        if x_size[i] <= window_size[i]:
            ws[i] = x_size[i]
            ss[i] = 0
    return tuple(ws), tuple(ss)


def window_indices(coords4, spatial_shape, window_size, shift_size):
    """(window slot, position) int32 [N,2], slots per batch item, positions per window."""
    idx = np.array(coords4, dtype=np.int64, copy=True)
    shape = list(spatial_shape)
    # pad: only trailing pads are used by the block (:735-738), so indices stay, the shape grows
    for a in range(3):
        shape[a] += (window_size[a] - shape[a] % window_size[a]) % window_size[a]
    # roll by -shift along the three spatial dims (:529-554)
    for a in range(3):
        idx[:, 1 + a] = (idx[:, 1 + a] - shift_size[a]) % shape[a]
    # partition (:336-372)
    nd, nh, nw = (shape[a] // window_size[a] for a in range(3))
    wd, wh, ww = window_size
    window = idx[:, 0] * (nd * nh * nw) + (idx[:, 1] // wd) * (nh * nw) + (idx[:, 2] // wh) * nw + idx[:, 3] // ww
    pos = (idx[:, 1] % wd) * (wh * ww) + (idx[:, 2] % wh) * ww + idx[:, 3] % ww
    return np.stack([window, pos], 1).astype(np.int32), nd * nh * nw, wd * wh * ww


def shift_mask(dims, window_size, shift_size):
    """int8 [windows, positions] region ids (:416-452)."""
    d, h, w = dims
    img = np.zeros((d, h, w), np.int8)
    cnt = 0
    for sd in (slice(-window_size[0]), slice(-window_size[0], -shift_size[0]), slice(-shift_size[0], None)):
        for sh in (slice(-window_size[1]), slice(-window_size[1], -shift_size[1]), slice(-shift_size[1], None)):
            for sw in (slice(-window_size[2]), slice(-window_size[2], -shift_size[2]), slice(-shift_size[2], None)):
                img[sd, sh, sw] = cnt
                cnt += 1
    wd, wh, ww = window_size
    v = img.reshape(d // wd, wd, h // wh, wh, w // ww, ww).transpose(0, 2, 4, 1, 3, 5)
    return np.ascontiguousarray(v.reshape(-1, wd * wh * ww))


def downsample(coords4, features, mean=True):
    """(merged coords int32 [M,4] ascending in (batch, d, h, w), pooled features [M,C], inverse [N])."""
    q = np.array(coords4, dtype=np.int64, copy=True)
    q[:, 1:] //= 2
    uniq, inverse = np.unique(q, axis=0, return_inverse=True)      # rows sorted lexicographically
    inverse = inverse.reshape(-1)
    out = np.zeros((len(uniq), features.shape[1]), np.float64)
    np.add.at(out, inverse, features.astype(np.float64))
    if mean:
        out /= np.bincount(inverse, minlength=len(uniq))[:, None]
    return uniq.astype(np.int32), out, inverse
