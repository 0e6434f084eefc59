"""TEST INFRASTRUCTURE -- numpy front end of the CPU oracle (``libchop_oracle.so``).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.  The product package never does.

Every function takes and returns C-contiguous numpy arrays in the reference op's
layouts (custom_helper_op/cc/ops/custom_helper_ops.cc:190-307):
ref ``[B,H,W,C]``, src ``[B,N,srcH,srcW,C]``, base_plane ``[B,H,W,1]``,
offsets ``[B,D]``, depth_grid ``[B,H,W,D]``, Rs ``[B,N,3,3]``, Ts ``[B,N,3]``,
cost ``[B,H,W,D,C|G]``, mask int32 ``[B,H,W,D,1]`` (MEAN) or ``[B,H,W,D,C|G]`` (MIN).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libchop_oracle.so")
_lib = None

MEAN, MIN = 0, 1
_REDUCE = {"MEAN": 0, "MIN": 1, 0: 0, 1: 1}


def build(force=False):
    """Compile the oracle with the Makefile beside this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B"] if force else ["make", "-C", _HERE], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32"
    if dtype == np.float64:
        return "f64"
    raise TypeError("oracle computes in float32 or float64 only, got %s" % dtype)


def _p(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(0)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def _i64(*v):
    return [ctypes.c_int64(int(x)) for x in v]


def _check(rc, name):
    if rc != 0:
        raise ValueError("%s failed with oracle status %d" % (name, rc))


def _outputs(out, cost_shape, mask_shape, dt):
    """Fresh output arrays, or the caller's (already touched, so that a timed call does not
    pay for the first-touch page faults of a new allocation)."""
    if out is None:
        return np.empty(cost_shape, dt), np.empty(mask_shape, np.int32)
    cost, mask = out
    assert cost.shape == cost_shape and cost.dtype == dt and cost.flags.c_contiguous
    assert mask.shape == mask_shape and mask.dtype == np.int32 and mask.flags.c_contiguous
    return cost, mask


def cost_volume_fwd(ref, src, base_plane, offsets, Rs, Ts, reduce="MEAN", half_centor=True,
                    threads=1, out=None):
    dt = ref.dtype
    sfx = _sfx(dt)
    ref, src, base_plane, offsets, Rs, Ts = (_c(x, dt) for x in (ref, src, base_plane, offsets, Rs, Ts))
    B, H, W, C = ref.shape
    N, sH, sW = src.shape[1:4]
    D = offsets.shape[1]
    r = _REDUCE[reduce]
    cost, mask = _outputs(out, (B, H, W, D, C), (B, H, W, D, 1 if r == 0 else C), dt)
    fn = getattr(lib(), "chop_oracle_cost_volume_fwd_" + sfx)
    rc = fn(r, int(bool(half_centor)), *_i64(B, H, W, C, D, N, sH, sW), _p(ref), _p(src),
            _p(base_plane), _p(offsets), _p(Rs), _p(Ts), _p(cost), _p(mask), int(threads))
    _check(rc, "cost_volume_fwd")
    return cost, mask


def cost_volume_bwd(ref, src, base_plane, offsets, Rs, Ts, cost_grad, mask, reduce="MEAN",
                    half_centor=True, threads=1):
    dt = ref.dtype
    sfx = _sfx(dt)
    ref, src, base_plane, offsets, Rs, Ts, cost_grad = (
        _c(x, dt) for x in (ref, src, base_plane, offsets, Rs, Ts, cost_grad))
    mask = _c(mask, np.int32)
    B, H, W, C = ref.shape
    N, sH, sW = src.shape[1:4]
    D = offsets.shape[1]
    ref_grad = np.empty_like(ref)
    src_grad = np.empty_like(src)
    bp_grad = np.empty_like(base_plane)
    fn = getattr(lib(), "chop_oracle_cost_volume_bwd_" + sfx)
    rc = fn(_REDUCE[reduce], int(bool(half_centor)), *_i64(B, H, W, C, D, N, sH, sW), _p(ref),
            _p(src), _p(base_plane), _p(offsets), _p(Rs), _p(Ts), _p(cost_grad), _p(mask),
            _p(ref_grad), _p(src_grad), _p(bp_grad), int(threads))
    _check(rc, "cost_volume_bwd")
    return ref_grad, src_grad, bp_grad


def cost_aggregate_fwd(ref, src, base_plane, offsets, Rs, Ts, reduce="MEAN", half_centor=True,
                       threads=1):
    """cost [B,H,W,D] and mask [B,H,W,D] (MEAN: valid-view count, MIN: winning view or -1)."""
    dt = ref.dtype
    sfx = _sfx(dt)
    ref, src, base_plane, offsets, Rs, Ts = (_c(x, dt) for x in (ref, src, base_plane, offsets, Rs, Ts))
    B, H, W, C = ref.shape
    N, sH, sW = src.shape[1:4]
    D = offsets.shape[1]
    cost = np.empty((B, H, W, D), dt)
    mask = np.empty((B, H, W, D), np.int32)
    fn = getattr(lib(), "chop_oracle_cost_aggregate_fwd_" + sfx)
    rc = fn(_REDUCE[reduce], int(bool(half_centor)), *_i64(B, H, W, C, D, N, sH, sW), _p(ref),
            _p(src), _p(base_plane), _p(offsets), _p(Rs), _p(Ts), _p(cost), _p(mask), int(threads))
    _check(rc, "cost_aggregate_fwd")
    return cost, mask


def cost_aggregate_bwd(ref, src, base_plane, offsets, Rs, Ts, cost_grad, mask, reduce="MEAN",
                       half_centor=True, threads=1):
    dt = ref.dtype
    sfx = _sfx(dt)
    ref, src, base_plane, offsets, Rs, Ts, cost_grad = (
        _c(x, dt) for x in (ref, src, base_plane, offsets, Rs, Ts, cost_grad))
    mask = _c(mask, np.int32)
    B, H, W, C = ref.shape
    N, sH, sW = src.shape[1:4]
    D = offsets.shape[1]
    ref_grad = np.empty_like(ref)
    src_grad = np.empty_like(src)
    bp_grad = np.empty_like(base_plane)
    fn = getattr(lib(), "chop_oracle_cost_aggregate_bwd_" + sfx)
    rc = fn(_REDUCE[reduce], int(bool(half_centor)), *_i64(B, H, W, C, D, N, sH, sW), _p(ref),
            _p(src), _p(base_plane), _p(offsets), _p(Rs), _p(Ts), _p(cost_grad), _p(mask),
            _p(ref_grad), _p(src_grad), _p(bp_grad), int(threads))
    _check(rc, "cost_aggregate_bwd")
    return ref_grad, src_grad, bp_grad


def cost_volume_v2_fwd(ref, src, depth_grid, Rs, Ts, reduce="MEAN", groups=1, half_centor=True,
                       threads=1, out=None):
    dt = ref.dtype
    sfx = _sfx(dt)
    ref, src, depth_grid, Rs, Ts = (_c(x, dt) for x in (ref, src, depth_grid, Rs, Ts))
    B, H, W, C = ref.shape
    N, sH, sW = src.shape[1:4]
    D = depth_grid.shape[3]
    r = _REDUCE[reduce]
    G = int(groups)
    cost, mask = _outputs(out, (B, H, W, D, max(G, 0)), (B, H, W, D, 1 if r == 0 else max(G, 0)), dt)
    fn = getattr(lib(), "chop_oracle_cost_volume_v2_fwd_" + sfx)
    rc = fn(r, int(bool(half_centor)), *_i64(B, H, W, C, D, N, sH, sW, G), _p(ref), _p(src),
            _p(depth_grid), _p(Rs), _p(Ts), _p(cost), _p(mask), int(threads))
    _check(rc, "cost_volume_v2_fwd")
    return cost, mask


def cost_volume_grid_fwd(ref, src, depth_grid, Rs, Ts, reduce="MEAN", half_centor=True, threads=1):
    """CostVolume's squared-difference reduce over per-voxel hypotheses ``depth_grid``."""
    dt = ref.dtype
    sfx = _sfx(dt)
    ref, src, depth_grid, Rs, Ts = (_c(x, dt) for x in (ref, src, depth_grid, Rs, Ts))
    B, H, W, C = ref.shape
    N, sH, sW = src.shape[1:4]
    D = depth_grid.shape[3]
    r = _REDUCE[reduce]
    cost, mask = _outputs(None, (B, H, W, D, C), (B, H, W, D, 1 if r == 0 else C), dt)
    fn = getattr(lib(), "chop_oracle_cost_volume_grid_fwd_" + sfx)
    rc = fn(r, int(bool(half_centor)), *_i64(B, H, W, C, D, N, sH, sW), _p(ref), _p(src),
            _p(depth_grid), _p(Rs), _p(Ts), _p(cost), _p(mask), int(threads))
    _check(rc, "cost_volume_grid_fwd")
    return cost, mask


def cost_volume_grid_bwd(ref, src, depth_grid, Rs, Ts, cost_grad, mask, reduce="MEAN",
                         half_centor=True, threads=1):
    dt = ref.dtype
    sfx = _sfx(dt)
    ref, src, depth_grid, Rs, Ts, cost_grad = (
        _c(x, dt) for x in (ref, src, depth_grid, Rs, Ts, cost_grad))
    mask = _c(mask, np.int32)
    B, H, W, C = ref.shape
    N, sH, sW = src.shape[1:4]
    D = depth_grid.shape[3]
    ref_grad = np.empty_like(ref)
    src_grad = np.empty_like(src)
    dg_grad = np.empty_like(depth_grid)
    fn = getattr(lib(), "chop_oracle_cost_volume_grid_bwd_" + sfx)
    rc = fn(_REDUCE[reduce], int(bool(half_centor)), *_i64(B, H, W, C, D, N, sH, sW), _p(ref),
            _p(src), _p(depth_grid), _p(Rs), _p(Ts), _p(cost_grad), _p(mask), _p(ref_grad),
            _p(src_grad), _p(dg_grad), int(threads))
    _check(rc, "cost_volume_grid_bwd")
    return ref_grad, src_grad, dg_grad


def cost_volume_v2_bwd(ref, src, depth_grid, Rs, Ts, cost_grad, mask, reduce="MEAN", groups=1,
                       half_centor=True, threads=1):
    dt = ref.dtype
    sfx = _sfx(dt)
    ref, src, depth_grid, Rs, Ts, cost_grad = (
        _c(x, dt) for x in (ref, src, depth_grid, Rs, Ts, cost_grad))
    mask = _c(mask, np.int32)
    B, H, W, C = ref.shape
    N, sH, sW = src.shape[1:4]
    D = depth_grid.shape[3]
    ref_grad = np.empty_like(ref)
    src_grad = np.empty_like(src)
    dg_grad = np.empty_like(depth_grid)
    fn = getattr(lib(), "chop_oracle_cost_volume_v2_bwd_" + sfx)
    rc = fn(_REDUCE[reduce], int(bool(half_centor)), *_i64(B, H, W, C, D, N, sH, sW, int(groups)),
            _p(ref), _p(src), _p(depth_grid), _p(Rs), _p(Ts), _p(cost_grad), _p(mask),
            _p(ref_grad), _p(src_grad), _p(dg_grad), int(threads))
    _check(rc, "cost_volume_v2_bwd")
    return ref_grad, src_grad, dg_grad


def cost_volume_v3_fwd(ref, src, base_plane, offsets, Rs, Ts, reduce="MEAN", groups=1,
                       half_centor=True, threads=1):
    """cost [B,H,W,D,1]; mask [B,H,W,D,1] (MEAN) or [B,H,W,D,3] (MIN: view, ref group, src group)."""
    dt = ref.dtype
    sfx = _sfx(dt)
    ref, src, base_plane, offsets, Rs, Ts = (_c(x, dt) for x in (ref, src, base_plane, offsets, Rs, Ts))
    B, H, W, C = ref.shape
    N, sH, sW = src.shape[1:4]
    D = offsets.shape[1]
    r = _REDUCE[reduce]
    cost = np.empty((B, H, W, D, 1), dt)
    mask = np.empty((B, H, W, D, 1 if r == 0 else 3), np.int32)
    fn = getattr(lib(), "chop_oracle_cost_volume_v3_fwd_" + sfx)
    rc = fn(r, int(bool(half_centor)), *_i64(B, H, W, C, D, N, sH, sW, int(groups)), _p(ref),
            _p(src), _p(base_plane), _p(offsets), _p(Rs), _p(Ts), _p(cost), _p(mask), int(threads))
    _check(rc, "cost_volume_v3_fwd")
    return cost, mask


def cost_volume_v3_bwd(ref, src, base_plane, offsets, Rs, Ts, cost_grad, mask, reduce="MEAN",
                       groups=1, half_centor=True, threads=1):
    dt = ref.dtype
    sfx = _sfx(dt)
    ref, src, base_plane, offsets, Rs, Ts, cost_grad = (
        _c(x, dt) for x in (ref, src, base_plane, offsets, Rs, Ts, cost_grad))
    mask = _c(mask, np.int32)
    B, H, W, C = ref.shape
    N, sH, sW = src.shape[1:4]
    D = offsets.shape[1]
    ref_grad = np.empty_like(ref)
    src_grad = np.empty_like(src)
    bp_grad = np.empty_like(base_plane)
    fn = getattr(lib(), "chop_oracle_cost_volume_v3_bwd_" + sfx)
    rc = fn(_REDUCE[reduce], int(bool(half_centor)), *_i64(B, H, W, C, D, N, sH, sW, int(groups)),
            _p(ref), _p(src), _p(base_plane), _p(offsets), _p(Rs), _p(Ts), _p(cost_grad),
            _p(mask), _p(ref_grad), _p(src_grad), _p(bp_grad), int(threads))
    _check(rc, "cost_volume_v3_bwd")
    return ref_grad, src_grad, bp_grad


def feature_aggregate_fwd(src, base_plane, offsets, Rs, Ts, half_centor=True, threads=1):
    """mapped_feature [B,H,W,D,N,C] and mapped_mask [B,H,W,D,N,1]; H, W from base_plane."""
    dt = src.dtype
    sfx = _sfx(dt)
    src, base_plane, offsets, Rs, Ts = (_c(x, dt) for x in (src, base_plane, offsets, Rs, Ts))
    B, N, sH, sW, C = src.shape
    H, W = base_plane.shape[1:3]
    D = offsets.shape[1]
    mapped = np.empty((B, H, W, D, N, C), dt)
    mask = np.empty((B, H, W, D, N, 1), np.int32)
    fn = getattr(lib(), "chop_oracle_feature_aggregate_fwd_" + sfx)
    rc = fn(int(bool(half_centor)), *_i64(B, H, W, C, D, N, sH, sW), _p(src), _p(base_plane),
            _p(offsets), _p(Rs), _p(Ts), _p(mapped), _p(mask), int(threads))
    _check(rc, "feature_aggregate_fwd")
    return mapped, mask


def feature_aggregate_bwd(src, base_plane, offsets, Rs, Ts, mapped_grad, mapped_mask,
                          half_centor=True, threads=1):
    dt = src.dtype
    sfx = _sfx(dt)
    src, base_plane, offsets, Rs, Ts, mapped_grad = (
        _c(x, dt) for x in (src, base_plane, offsets, Rs, Ts, mapped_grad))
    mapped_mask = _c(mapped_mask, np.int32)
    B, N, sH, sW, C = src.shape
    H, W = base_plane.shape[1:3]
    D = offsets.shape[1]
    src_grad = np.empty_like(src)
    bp_grad = np.empty_like(base_plane)
    fn = getattr(lib(), "chop_oracle_feature_aggregate_bwd_" + sfx)
    rc = fn(int(bool(half_centor)), *_i64(B, H, W, C, D, N, sH, sW), _p(src), _p(base_plane),
            _p(offsets), _p(Rs), _p(Ts), _p(mapped_grad), _p(mapped_mask), _p(src_grad),
            _p(bp_grad), int(threads))
    _check(rc, "feature_aggregate_bwd")
    return src_grad, bp_grad


def cost_default_fill(cost, cost_mask, default_cost, reduce="MEAN"):
    """``tf.where(cost_mask > 0, cost, default)`` (MEAN) / ``cost_mask >= 0`` (MIN), as the
    reference's layers apply it (custom_helper_op/python/layers/custom_layers.py:52-57, :78-83);
    the mask broadcasts over a trailing axis of the cost."""
    valid = (cost_mask > 0) if _REDUCE[reduce] == 0 else (cost_mask >= 0)
    while valid.ndim < cost.ndim:
        valid = valid[..., None]
    return np.where(valid, cost, np.asarray(default_cost, cost.dtype))


def cost_default_fill_grad(out_grad, cost_mask, reduce="MEAN"):
    """Gradient of that ``where``: ``(cost_grad, default_grad)``."""
    valid = (cost_mask > 0) if _REDUCE[reduce] == 0 else (cost_mask >= 0)
    while valid.ndim < out_grad.ndim:
        valid = valid[..., None]
    valid = np.broadcast_to(valid, out_grad.shape)
    return np.where(valid, out_grad, 0), np.where(valid, 0, out_grad).sum(dtype=np.float64)


def combine_projection(ref_cam, src_cam, scale):
    """Line-by-line numpy restatement of the reference helper
    (custom_helper_op/python/ops/op_tests/cost_volume_op_test.py:115-134) for one camera pair:
    ``ref_cam, src_cam [2,4,4]``, ``scale [3]`` -> ``(R [3,3], T [3,1])``."""
    ref_R, ref_T = ref_cam[0, :3, :3], ref_cam[0, :3, 3:]
    ref_K = ref_cam[1, :3, :3] * scale[:, None]
    src_R, src_T = src_cam[0, :3, :3], src_cam[0, :3, 3:]
    src_K = src_cam[1, :3, :3] * scale[:, None]
    ref_K[0, 2] = ref_K[0, 2] + 0.5
    ref_K[1, 2] = ref_K[1, 2] + 0.5
    src_K[0, 2] = src_K[0, 2] + 0.5
    src_K[1, 2] = src_K[1, 2] + 0.5
    ref_K_inv = np.linalg.inv(ref_K)
    delta_R = src_R @ ref_R.T
    delta_T = src_T - delta_R @ ref_T
    return src_K @ (delta_R @ ref_K_inv), src_K @ delta_T


def sample_coords(base_plane, offsets, Rs, Ts, src_hw, half_centor=True, depth_grid=None):
    """Per-(voxel, view) source coordinates ``[B,H,W,D,N]``: (sw, sh, fh, fw, state)."""
    if depth_grid is not None:
        dt = depth_grid.dtype
        depth_grid = _c(depth_grid, dt)
        B, H, W, D = depth_grid.shape
        base_plane = offsets = None
    else:
        dt = base_plane.dtype
        base_plane, offsets = _c(base_plane, dt), _c(offsets, dt)
        B, H, W = base_plane.shape[:3]
        D = offsets.shape[1]
    sfx = _sfx(dt)
    Rs, Ts = _c(Rs, dt), _c(Ts, dt)
    N = Rs.shape[1]
    sH, sW = src_hw
    shape = (B, H, W, D, N)
    sw, sh = np.empty(shape, dt), np.empty(shape, dt)
    fh, fw, st = (np.empty(shape, np.int32) for _ in range(3))
    fn = getattr(lib(), "chop_oracle_sample_coords_" + sfx)
    rc = fn(int(bool(half_centor)), *_i64(B, H, W, D, N, sH, sW), _p(base_plane), _p(offsets),
            _p(depth_grid), _p(Rs), _p(Ts), _p(sw), _p(sh), _p(fh), _p(fw), _p(st))
    _check(rc, "sample_coords")
    return sw, sh, fh, fw, st
