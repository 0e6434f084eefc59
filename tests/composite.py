"""Independent float64 composite of the cost-volume op, used to pin the CPU oracle.

It restates, in numpy, the TensorFlow composite that the reference's own unit tests
compare the op against (``build_sampler_coordinate`` + ``cost_aggregate_tfa``,
custom_helper_op/python/ops/op_tests/cost_volume_op_test.py:136-171 and
cost_volume_v2_op_test.py:155-172): scale homogeneous pixel coordinates by depth,
``matvec`` with R, add T, perspective divide, subtract the half-pixel, strict
open-interval validity, textbook bilinear resampling with zeros outside the image
(what ``tfa.image.resampler`` does), then the reduce over views.

Nothing here shares code or operation order with the oracle: the projection is
``R @ (depth * p) + T`` (the oracle follows the kernel's ``(R @ p) * depth + T``), and
the bilinear gather is the four-corner formula over whole arrays.
"""
import numpy as np
from scipy.ndimage import map_coordinates


def sampler_coordinates(Rs, Ts, depth, half_centor=True):
    """depth ``[B,H,W,D]`` -> xy ``[B,N,H,W,D,2]`` (x = column, y = row), z>0 mask."""
    B, H, W, D = depth.shape
    off = 0.5 if half_centor else 0.0
    xs, ys = np.meshgrid(np.arange(W) + off, np.arange(H) + off)
    base = np.stack([xs, ys, np.ones_like(xs)], -1)                      # [H,W,3]
    coord = depth[..., None] * base[None, :, :, None, :]                  # [B,H,W,D,3]
    smp = np.einsum("bnij,bhwdj->bnhwdi", Rs, coord) + Ts[:, :, None, None, None, :]
    front = smp[..., 2:3] > 0
    with np.errstate(divide="ignore", invalid="ignore"):
        xy = np.where(front, smp[..., :2] / smp[..., 2:3], 0.0)
    if half_centor:
        xy = xy - 0.5
    return xy, front[..., 0]


def validity(xy, front, srcH, srcW):
    lim = np.array([srcW - 1, srcH - 1], dtype=xy.dtype)
    return front & np.all((xy > 0.0) & (xy < lim), axis=-1)


def bilinear_zero_pad(img, x, y):
    """img ``[h,w,C]``; x,y arrays of any shape -> ``x.shape + [C]``; zeros outside."""
    h, w, _ = img.shape
    x0 = np.floor(x).astype(np.int64)
    y0 = np.floor(y).astype(np.int64)
    out = 0.0
    for dy in (0, 1):
        for dx in (0, 1):
            xi, yi = x0 + dx, y0 + dy
            wgt = (1 - np.abs(x - xi)) * (1 - np.abs(y - yi))
            ok = (xi >= 0) & (xi < w) & (yi >= 0) & (yi < h)
            v = img[np.clip(yi, 0, h - 1), np.clip(xi, 0, w - 1)]
            out = out + np.where(ok, wgt, 0.0)[..., None] * v
    return out


def bilinear_scipy(img, x, y):
    """Library twin of :func:`bilinear_zero_pad` (scipy's order-1 spline == bilinear)."""
    return np.stack([map_coordinates(img[..., c], [y, x], order=1, mode="constant", cval=0.0)
                     for c in range(img.shape[-1])], -1)


def warp_views(src, xy, valid, sampler=bilinear_zero_pad):
    """src ``[B,N,h,w,C]`` -> warped ``[B,N,H,W,D,C]`` (invalid samples read at -1000)."""
    B, N = src.shape[:2]
    xy = np.where(valid[..., None], xy, -1000.0)
    out = np.empty(xy.shape[:-1] + (src.shape[-1],), dtype=np.float64)
    for b in range(B):
        for n in range(N):
            out[b, n] = sampler(src[b, n].astype(np.float64), xy[b, n, ..., 0], xy[b, n, ..., 1])
    return out


def cost_volume_composite(ref, src, depth, Rs, Ts, reduce="MEAN", half_centor=True, groups=None,
                          sampler=bilinear_zero_pad):
    """Returns (cost ``[B,H,W,D,C|G]``, per-view validity ``[B,N,H,W,D]``, xy).

    ``groups=None``: V1, squared difference, mean/min over views.
    ``groups=G``: V2, channel-group dot product, mean/max over views.
    Like the reference composite the reduce runs over *all* N views, so it equals the
    op only where every view is valid (MEAN) -- the reference test masks accordingly.
    """
    ref = ref.astype(np.float64)
    xy, front = sampler_coordinates(Rs.astype(np.float64), Ts.astype(np.float64),
                                    depth.astype(np.float64), half_centor)
    valid = validity(xy, front, src.shape[2], src.shape[3])
    warped = warp_views(src, xy, valid, sampler)
    r = ref[:, None, :, :, None, :]
    if groups is None:
        per_view = (warped - r) ** 2
        cost = per_view.mean(1) if reduce == "MEAN" else per_view.min(1)
    else:
        prod = warped * r
        per_view = prod.reshape(prod.shape[:-1] + (groups, prod.shape[-1] // groups)).sum(-1)
        cost = per_view.mean(1) if reduce == "MEAN" else per_view.max(1)
    return cost, valid, xy, per_view
