"""Host-side mirror of the reference's Python operator interface for the cost volume.

Same names, argument order, defaults and outputs as
custom_helper_op/python/ops/custom_helper_ops.py:32-197 (``cost_volume``,
``cost_volume_v2``, ``cost_volume_v3``, ``cost_aggregate``, ``feature_aggregate`` and the
gradients registered for them), with torch tensors standing in
for TensorFlow tensors: torch supplies device memory and the current HIP stream, the
arithmetic is done by ``libchop_costvol.so`` through its C ABI.  The shape checks are the
ones ``CostVolumeOp::Compute`` performs (custom_helper_op/cc/kernels/
cost_volume_kernels.cc:91-106, :220-243; cost_volume_kernels_v2.cc:93-110), raised as
``InvalidArgumentError``.

float32/float64 follow the registered ops; float16/bfloat16 feature tensors use the
library's 16-bit storage extension (depth inputs and camera matrices must then be
float32).
"""
import torch

from . import _lib

_REDUCE = {"MEAN": 0, "MIN": 1}
_STORAGE16 = {torch.float16: 1, torch.bfloat16: 2}


class InvalidArgumentError(ValueError):
    """What ``OP_REQUIRES(..., errors::InvalidArgument(...))`` becomes on this side."""


def _reduce_code(reduce_method):
    if reduce_method not in _REDUCE:
        # the reference aborts the process here (LOG(FATAL), cost_volume_kernels.cc:71)
        raise InvalidArgumentError(
            "Invalid reduce method %r. Supported types: MEAN, MIN" % (reduce_method,))
    return _REDUCE[reduce_method]


def _require(cond, msg):
    if not cond:
        raise InvalidArgumentError(msg)


def _ptr(t):
    return t.data_ptr() if t is not None else None


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _prep(t, dtype, device, name):
    t = torch.as_tensor(t)
    _require(t.dtype == dtype, "%s must have dtype %s, got %s" % (name, dtype, t.dtype))
    _require(t.device == device, "%s must live on %s" % (name, device))
    return t.contiguous()


def _real_dtype(dtype):
    _require(dtype in (torch.float32, torch.float64, torch.float16, torch.bfloat16),
             "dtype must be float32 or float64 (float16/bfloat16 storage as an extension)")
    return torch.float32 if dtype in _STORAGE16 else dtype


def _check_common(ref_image, src_images, Rs, Ts):
    _require(ref_image.dim() == 4, "ref image must have rank 4")
    B, H, W, C = ref_image.shape
    _require(src_images.dim() == 5 and src_images.shape[0] == B and src_images.shape[2] == H
             and src_images.shape[3] == W and src_images.shape[4] == C,
             "src_images must have rank 5, and must compate to ref_image")
    N = src_images.shape[1]
    _require(Rs.dim() == 4 and tuple(Rs.shape) == (B, N, 3, 3),
             "Rs must have rank 2, and must compate to ref_image")
    _require(Ts.dim() == 3 and tuple(Ts.shape) == (B, N, 3),
             "Ts must have rank 2, and must compate to ref_image")
    return B, H, W, C, N


def _check_v1(ref_image, src_images, base_plane, offsets, Rs, Ts):
    B, H, W, C, N = _check_common(ref_image, src_images, Rs, Ts)
    _require(base_plane.dim() == 4 and tuple(base_plane.shape) == (B, H, W, 1),
             "base_plane must have rank 4, and must compate to ref_image")
    _require(offsets.dim() == 2 and offsets.shape[0] == B,
             "offsets must have rank 2, and must compate to ref_image")
    return B, H, W, C, N, offsets.shape[1]


def _check_v2(ref_image, src_images, depth_grid, Rs, Ts, groups):
    B, H, W, C, N = _check_common(ref_image, src_images, Rs, Ts)
    _require(depth_grid.dim() == 4 and tuple(depth_grid.shape[:3]) == (B, H, W),
             "depth_grid must have rank 4, and must compate to ref_image")
    _require(isinstance(groups, int) and groups > 0 and C % groups == 0,
             "image_channels must be divisible by groups")
    return B, H, W, C, N, depth_grid.shape[3]


def _check_grid16(ref_image, src_images, depth_grid, Rs, Ts):
    """Per-voxel hypotheses for the squared-difference op: an extension of the 16-bit storage
    entry points (the registered CostVolume op only knows base_plane + offsets)."""
    _require(ref_image.dtype in _STORAGE16,
             "depth_grid with the squared-difference op needs float16 or bfloat16 features")
    B, H, W, C, N = _check_common(ref_image, src_images, Rs, Ts)
    _require(depth_grid.dim() == 4 and tuple(depth_grid.shape[:3]) == (B, H, W),
             "depth_grid must have rank 4, and must compate to ref_image")
    return B, H, W, C, N, depth_grid.shape[3]


def cost_volume_raw(ref_image, src_images, base_plane, offsets, Rs, Ts, reduce_method="MEAN",
                    half_centor=True, depth_grid=None):
    """Forward op without autograd: returns ``(cost [B,H,W,D,C], cost_mask int32)``.
    ``depth_grid`` ([B,H,W,D] float32, 16-bit feature storage only) replaces
    ``base_plane + offsets`` (which may then be ``None``) by per-voxel hypotheses."""
    lib = _lib.load()
    red = _reduce_code(reduce_method)
    dt, dev = ref_image.dtype, ref_image.device
    rdt = _real_dtype(dt)
    ref_image = _prep(ref_image, dt, dev, "ref_image")
    src_images = _prep(src_images, dt, dev, "src_images")
    Rs, Ts = _prep(Rs, rdt, dev, "Rs"), _prep(Ts, rdt, dev, "Ts")
    if depth_grid is not None:
        depth_grid = _prep(depth_grid, rdt, dev, "depth_grid")
        B, H, W, C, N, D = _check_grid16(ref_image, src_images, depth_grid, Rs, Ts)
        base_plane = offsets = None
    else:
        base_plane = _prep(base_plane, rdt, dev, "base_plane")
        offsets = _prep(offsets, rdt, dev, "offsets")
        B, H, W, C, N, D = _check_v1(ref_image, src_images, base_plane, offsets, Rs, Ts)
    cost = torch.empty((B, H, W, D, C), dtype=dt, device=dev)
    mask = torch.empty((B, H, W, D, 1 if red == 0 else C), dtype=torch.int32, device=dev)
    dims = (B, H, W, C, D, N, src_images.shape[2], src_images.shape[3])
    if dt in _STORAGE16:
        rc = lib.chop_cost_volume_fwd_16(_stream(cost), _STORAGE16[dt], red, int(half_centor), *dims,
                                         _ptr(ref_image), _ptr(src_images), _ptr(base_plane),
                                         _ptr(offsets), _ptr(depth_grid), _ptr(Rs), _ptr(Ts),
                                         _ptr(cost), _ptr(mask))
    else:
        fn = lib.chop_cost_volume_fwd_f32 if dt == torch.float32 else lib.chop_cost_volume_fwd_f64
        rc = fn(_stream(cost), red, int(half_centor), *dims, _ptr(ref_image), _ptr(src_images),
                _ptr(base_plane), _ptr(offsets), _ptr(Rs), _ptr(Ts), _ptr(cost), _ptr(mask))
    _lib.check(rc)
    return cost, mask


def cost_volume_grad(ref_image, src_images, base_plane, offsets, rs, ts, cost_grad, cost_mask,
                     reduce_method="MEAN", half_centor=True, need_depth_grad=True,
                     depth_grid=None):
    """The ``CostVolumeGrad`` op: ``(ref_image_grad, src_images_grad, base_plane_grad)``.
    With ``need_depth_grad=False`` the third result is ``None`` and the kernels skip the
    depth-derivative work (the registered op always computes it).  With ``depth_grid``
    (16-bit feature storage only) the third result is the gradient of ``depth_grid``,
    ``[B,H,W,D]``, zero on the voxels the mask skips."""
    lib = _lib.load()
    red = _reduce_code(reduce_method)
    dt, dev = ref_image.dtype, ref_image.device
    rdt = _real_dtype(dt)
    ref_image = _prep(ref_image, dt, dev, "ref_image")
    src_images = _prep(src_images, dt, dev, "src_images")
    rs, ts = _prep(rs, rdt, dev, "Rs"), _prep(ts, rdt, dev, "Ts")
    cost_grad = _prep(cost_grad, dt, dev, "cost_grad")
    cost_mask = _prep(cost_mask, torch.int32, dev, "cost_mask")
    if depth_grid is not None:
        depth_grid = _prep(depth_grid, rdt, dev, "depth_grid")
        B, H, W, C, N, D = _check_grid16(ref_image, src_images, depth_grid, rs, ts)
        base_plane = offsets = None
    else:
        base_plane = _prep(base_plane, rdt, dev, "base_plane")
        offsets = _prep(offsets, rdt, dev, "offsets")
        B, H, W, C, N, D = _check_v1(ref_image, src_images, base_plane, offsets, rs, ts)
    _require(tuple(cost_grad.shape) == (B, H, W, D, C),
             "cost_grad must have rank 5, and must compate to ref_image")
    _require(tuple(cost_mask.shape) == (B, H, W, D, 1 if red == 0 else C),
             "cost_mask must have rank 5, and must compate to ref_image")
    ref_grad = torch.empty_like(ref_image)
    src_grad = torch.empty_like(src_images)
    bp_grad = None
    if need_depth_grad:
        bp_grad = torch.empty_like(depth_grid if depth_grid is not None else base_plane)
    dims = (B, H, W, C, D, N, src_images.shape[2], src_images.shape[3])
    if dt in _STORAGE16:
        need = lib.chop_cost_volume_bwd16_workspace_bytes(B, H, W, C, N, *dims[6:])
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
        rc = lib.chop_cost_volume_bwd_16(_stream(ref_grad), _STORAGE16[dt], red, int(half_centor),
                                         *dims, _ptr(ref_image), _ptr(src_images),
                                         _ptr(base_plane), _ptr(offsets), _ptr(depth_grid),
                                         _ptr(rs), _ptr(ts),
                                         _ptr(cost_grad), _ptr(cost_mask), _ptr(ref_grad),
                                         _ptr(src_grad), _ptr(bp_grad), _ptr(ws), need)
    else:
        fn = lib.chop_cost_volume_bwd_f32 if dt == torch.float32 else lib.chop_cost_volume_bwd_f64
        rc = fn(_stream(ref_grad), red, int(half_centor), *dims, _ptr(ref_image), _ptr(src_images),
                _ptr(base_plane), _ptr(offsets), _ptr(rs), _ptr(ts), _ptr(cost_grad),
                _ptr(cost_mask), _ptr(ref_grad), _ptr(src_grad), _ptr(bp_grad))
    _lib.check(rc)
    return ref_grad, src_grad, bp_grad


def _prep_default(default_cost, rdt, dev):
    default_cost = _prep(default_cost, rdt, dev, "default_cost")
    _require(default_cost.numel() == 1, "default_cost must be a scalar")
    return default_cost


def cost_volume_v2_raw(ref_image, src_images, depth_grid, Rs, Ts, reduce_method="MEAN", groups=None,
                       half_centor=True, default_cost=None):
    """``default_cost`` (a device scalar): written instead of the cost wherever no view was
    accepted -- ``CostMapLayerV2``'s fill, done by the op's own store."""
    lib = _lib.load()
    red = _reduce_code(reduce_method)
    dt, dev = ref_image.dtype, ref_image.device
    rdt = _real_dtype(dt)
    ref_image = _prep(ref_image, dt, dev, "ref_image")
    src_images = _prep(src_images, dt, dev, "src_images")
    depth_grid = _prep(depth_grid, rdt, dev, "depth_grid")
    Rs, Ts = _prep(Rs, rdt, dev, "Rs"), _prep(Ts, rdt, dev, "Ts")
    B, H, W, C, N, D = _check_v2(ref_image, src_images, depth_grid, Rs, Ts, groups)
    cost = torch.empty((B, H, W, D, groups), dtype=dt, device=dev)
    mask = torch.empty((B, H, W, D, 1 if red == 0 else groups), dtype=torch.int32, device=dev)
    dims = (B, H, W, C, D, N, src_images.shape[2], src_images.shape[3])
    if default_cost is not None:
        default_cost = _prep_default(default_cost, rdt, dev)
        if dt in _STORAGE16:
            rc = lib.chop_cost_volume_v2_fwd_fill_16(
                _stream(cost), _STORAGE16[dt], red, int(half_centor), *dims, groups,
                _ptr(ref_image), _ptr(src_images), _ptr(depth_grid), _ptr(Rs), _ptr(Ts),
                _ptr(default_cost), _ptr(cost), _ptr(mask))
        else:
            fn = (lib.chop_cost_volume_v2_fwd_fill_f32 if dt == torch.float32
                  else lib.chop_cost_volume_v2_fwd_fill_f64)
            rc = fn(_stream(cost), red, int(half_centor), *dims, groups, _ptr(ref_image),
                    _ptr(src_images), _ptr(depth_grid), _ptr(Rs), _ptr(Ts), _ptr(default_cost),
                    _ptr(cost), _ptr(mask))
    elif dt in _STORAGE16:
        rc = lib.chop_cost_volume_v2_fwd_16(_stream(cost), _STORAGE16[dt], red, int(half_centor),
                                            *dims, groups, _ptr(ref_image), _ptr(src_images),
                                            _ptr(depth_grid), _ptr(Rs), _ptr(Ts), _ptr(cost),
                                            _ptr(mask))
    else:
        fn = (lib.chop_cost_volume_v2_fwd_f32 if dt == torch.float32
              else lib.chop_cost_volume_v2_fwd_f64)
        rc = fn(_stream(cost), red, int(half_centor), *dims, groups, _ptr(ref_image),
                _ptr(src_images), _ptr(depth_grid), _ptr(Rs), _ptr(Ts), _ptr(cost), _ptr(mask))
    _lib.check(rc)
    return cost, mask


def cost_volume_grad_v2(ref_image, src_images, depth_grid, rs, ts, cost_grad, cost_mask,
                        reduce_method="MEAN", groups=None, half_centor=True,
                        need_depth_grad=True):
    """The ``CostVolumeGradV2`` op: ``(ref_image_grad, src_images_grad, depth_grid_grad)``;
    ``need_depth_grad=False`` as in :func:`cost_volume_grad`."""
    lib = _lib.load()
    red = _reduce_code(reduce_method)
    dt, dev = ref_image.dtype, ref_image.device
    rdt = _real_dtype(dt)
    ref_image = _prep(ref_image, dt, dev, "ref_image")
    src_images = _prep(src_images, dt, dev, "src_images")
    depth_grid = _prep(depth_grid, rdt, dev, "depth_grid")
    rs, ts = _prep(rs, rdt, dev, "Rs"), _prep(ts, rdt, dev, "Ts")
    cost_grad = _prep(cost_grad, dt, dev, "cost_grad")
    cost_mask = _prep(cost_mask, torch.int32, dev, "cost_mask")
    B, H, W, C, N, D = _check_v2(ref_image, src_images, depth_grid, rs, ts, groups)
    _require(tuple(cost_grad.shape) == (B, H, W, D, groups),
             "cost_grad must have rank 5, and must compate to ref_image")
    _require(tuple(cost_mask.shape) == (B, H, W, D, 1 if red == 0 else groups),
             "cost_mask must have rank 5, and must compate to ref_image")
    ref_grad = torch.empty_like(ref_image)
    src_grad = torch.empty_like(src_images)
    dg_grad = torch.empty_like(depth_grid) if need_depth_grad else None
    dims = (B, H, W, C, D, N, src_images.shape[2], src_images.shape[3])
    if dt in _STORAGE16:
        need = lib.chop_cost_volume_bwd16_workspace_bytes(B, H, W, C, N, *dims[6:])
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
        rc = lib.chop_cost_volume_v2_bwd_16(_stream(ref_grad), _STORAGE16[dt], red,
                                            int(half_centor), *dims, groups, _ptr(ref_image),
                                            _ptr(src_images), _ptr(depth_grid), _ptr(rs), _ptr(ts),
                                            _ptr(cost_grad), _ptr(cost_mask), _ptr(ref_grad),
                                            _ptr(src_grad), _ptr(dg_grad), _ptr(ws), need)
    else:
        fn = (lib.chop_cost_volume_v2_bwd_f32 if dt == torch.float32
              else lib.chop_cost_volume_v2_bwd_f64)
        rc = fn(_stream(ref_grad), red, int(half_centor), *dims, groups, _ptr(ref_image),
                _ptr(src_images), _ptr(depth_grid), _ptr(rs), _ptr(ts), _ptr(cost_grad),
                _ptr(cost_mask), _ptr(ref_grad), _ptr(src_grad), _ptr(dg_grad))
    _lib.check(rc)
    return ref_grad, src_grad, dg_grad


def cost_aggregate_raw(ref_image, src_images, base_plane, offsets, Rs, Ts, reduce_method="MEAN",
                       half_centor=True, default_cost=None):
    """The ``CostAggregate`` op without autograd: ``(cost [B,H,W,D], cost_mask int32 [B,H,W,D])``
    (shapes: custom_helper_op/cc/ops/custom_helper_ops.cc:46-58; checks:
    cost_aggregate_kernels.cc:85-106).  float32 and float64 only, as registered.
    ``default_cost`` as in :func:`cost_volume_v2_raw` (``CostMapLayer``'s fill)."""
    lib = _lib.load()
    red = _reduce_code(reduce_method)
    dt, dev = ref_image.dtype, ref_image.device
    _require(dt in (torch.float32, torch.float64), "dtype must be float32 or float64")
    ref_image = _prep(ref_image, dt, dev, "ref_image")
    src_images = _prep(src_images, dt, dev, "src_images")
    base_plane = _prep(base_plane, dt, dev, "base_plane")
    offsets = _prep(offsets, dt, dev, "offsets")
    Rs, Ts = _prep(Rs, dt, dev, "Rs"), _prep(Ts, dt, dev, "Ts")
    B, H, W, C, N, D = _check_v1(ref_image, src_images, base_plane, offsets, Rs, Ts)
    cost = torch.empty((B, H, W, D), dtype=dt, device=dev)
    mask = torch.empty((B, H, W, D), dtype=torch.int32, device=dev)
    dims = (B, H, W, C, D, N, src_images.shape[2], src_images.shape[3])
    if default_cost is not None:
        default_cost = _prep_default(default_cost, dt, dev)
        fn = (lib.chop_cost_aggregate_fwd_fill_f32 if dt == torch.float32
              else lib.chop_cost_aggregate_fwd_fill_f64)
        rc = fn(_stream(cost), red, int(half_centor), *dims, _ptr(ref_image), _ptr(src_images),
                _ptr(base_plane), _ptr(offsets), _ptr(Rs), _ptr(Ts), _ptr(default_cost), _ptr(cost),
                _ptr(mask))
    else:
        fn = lib.chop_cost_aggregate_fwd_f32 if dt == torch.float32 else lib.chop_cost_aggregate_fwd_f64
        rc = fn(_stream(cost), red, int(half_centor), *dims, _ptr(ref_image), _ptr(src_images),
                _ptr(base_plane), _ptr(offsets), _ptr(Rs), _ptr(Ts), _ptr(cost), _ptr(mask))
    _lib.check(rc)
    return cost, mask


def cost_aggregate_grad(ref_image, src_images, base_plane, offsets, rs, ts, cost_grad, cost_mask,
                        reduce_method="MEAN", half_centor=True, need_depth_grad=True):
    """The ``CostAggregateGrad`` op: ``(ref_image_grad, src_images_grad, base_plane_grad)``
    (checks: cost_aggregate_kernels.cc:196-226); ``need_depth_grad=False`` as in
    :func:`cost_volume_grad`."""
    lib = _lib.load()
    red = _reduce_code(reduce_method)
    dt, dev = ref_image.dtype, ref_image.device
    _require(dt in (torch.float32, torch.float64), "dtype must be float32 or float64")
    ref_image = _prep(ref_image, dt, dev, "ref_image")
    src_images = _prep(src_images, dt, dev, "src_images")
    base_plane = _prep(base_plane, dt, dev, "base_plane")
    offsets = _prep(offsets, dt, dev, "offsets")
    rs, ts = _prep(rs, dt, dev, "Rs"), _prep(ts, dt, dev, "Ts")
    cost_grad = _prep(cost_grad, dt, dev, "cost_grad")
    cost_mask = _prep(cost_mask, torch.int32, dev, "cost_mask")
    B, H, W, C, N, D = _check_v1(ref_image, src_images, base_plane, offsets, rs, ts)
    _require(tuple(cost_grad.shape) == (B, H, W, D),
             "cost_grad must have rank 4, and must compate to ref_image")
    _require(tuple(cost_mask.shape) == (B, H, W, D),
             "cost_mask must have rank 4, and must compate to ref_image")
    ref_grad = torch.empty_like(ref_image)
    src_grad = torch.empty_like(src_images)
    bp_grad = torch.empty_like(base_plane) if need_depth_grad else None
    dims = (B, H, W, C, D, N, src_images.shape[2], src_images.shape[3])
    fn = lib.chop_cost_aggregate_bwd_f32 if dt == torch.float32 else lib.chop_cost_aggregate_bwd_f64
    rc = fn(_stream(ref_grad), red, int(half_centor), *dims, _ptr(ref_image), _ptr(src_images),
            _ptr(base_plane), _ptr(offsets), _ptr(rs), _ptr(ts), _ptr(cost_grad), _ptr(cost_mask),
            _ptr(ref_grad), _ptr(src_grad), _ptr(bp_grad))
    _lib.check(rc)
    return ref_grad, src_grad, bp_grad


def _check_v3_groups(C, groups):
    # cost_volume_kernels_v3.cc:111-115
    _require(isinstance(groups, int) and groups > 0 and C % groups == 0,
             "image_channels and groups_ must match")
    _require(C // groups <= 8, "image_channels / groups_ less than MAX_SUBCHANNELS_SIZE(8)")


def cost_volume_v3_raw(ref_image, src_images, base_plane, offsets, Rs, Ts, reduce_method="MEAN",
                       groups=None, half_centor=True):
    """The ``CostVolumeV3`` op without autograd: ``(cost [B,H,W,D,1], cost_mask int32
    [B,H,W,D,1] (MEAN) or [B,H,W,D,3] (MIN: view, reference group, source group))``
    (shapes: custom_helper_op/cc/ops/custom_helper_ops.cc:311-347; checks:
    cost_volume_kernels_v3.cc:94-115).  float32 and float64, as registered."""
    lib = _lib.load()
    red = _reduce_code(reduce_method)
    dt, dev = ref_image.dtype, ref_image.device
    _require(dt in (torch.float32, torch.float64), "dtype must be float32 or float64")
    ref_image = _prep(ref_image, dt, dev, "ref_image")
    src_images = _prep(src_images, dt, dev, "src_images")
    base_plane = _prep(base_plane, dt, dev, "base_plane")
    offsets = _prep(offsets, dt, dev, "offsets")
    Rs, Ts = _prep(Rs, dt, dev, "Rs"), _prep(Ts, dt, dev, "Ts")
    B, H, W, C, N, D = _check_v1(ref_image, src_images, base_plane, offsets, Rs, Ts)
    _check_v3_groups(C, groups)
    cost = torch.empty((B, H, W, D, 1), dtype=dt, device=dev)
    mask = torch.empty((B, H, W, D, 1 if red == 0 else 3), dtype=torch.int32, device=dev)
    dims = (B, H, W, C, D, N, src_images.shape[2], src_images.shape[3])
    fn = lib.chop_cost_volume_v3_fwd_f32 if dt == torch.float32 else lib.chop_cost_volume_v3_fwd_f64
    rc = fn(_stream(cost), red, int(half_centor), *dims, groups, _ptr(ref_image), _ptr(src_images),
            _ptr(base_plane), _ptr(offsets), _ptr(Rs), _ptr(Ts), _ptr(cost), _ptr(mask))
    _lib.check(rc)
    return cost, mask


def cost_volume_grad_v3(ref_image, src_images, base_plane, offsets, rs, ts, cost_grad, cost_mask,
                        reduce_method="MEAN", groups=None, half_centor=True):
    """The ``CostVolumeGradV3`` op: ``(ref_image_grad, src_images_grad, base_plane_grad)``
    (checks: cost_volume_kernels_v3.cc:231-255)."""
    lib = _lib.load()
    red = _reduce_code(reduce_method)
    dt, dev = ref_image.dtype, ref_image.device
    _require(dt in (torch.float32, torch.float64), "dtype must be float32 or float64")
    ref_image = _prep(ref_image, dt, dev, "ref_image")
    src_images = _prep(src_images, dt, dev, "src_images")
    base_plane = _prep(base_plane, dt, dev, "base_plane")
    offsets = _prep(offsets, dt, dev, "offsets")
    rs, ts = _prep(rs, dt, dev, "Rs"), _prep(ts, dt, dev, "Ts")
    cost_grad = _prep(cost_grad, dt, dev, "cost_grad")
    cost_mask = _prep(cost_mask, torch.int32, dev, "cost_mask")
    B, H, W, C, N, D = _check_v1(ref_image, src_images, base_plane, offsets, rs, ts)
    _check_v3_groups(C, groups)
    _require(tuple(cost_grad.shape) == (B, H, W, D, 1),
             "cost_grad must have rank 5, and must compate to ref_image")
    _require(tuple(cost_mask.shape) == (B, H, W, D, 1 if red == 0 else 3),
             "cost_mask must have rank 5, and must compate to ref_image")
    ref_grad = torch.empty_like(ref_image)
    src_grad = torch.empty_like(src_images)
    bp_grad = torch.empty_like(base_plane)
    dims = (B, H, W, C, D, N, src_images.shape[2], src_images.shape[3])
    fn = lib.chop_cost_volume_v3_bwd_f32 if dt == torch.float32 else lib.chop_cost_volume_v3_bwd_f64
    rc = fn(_stream(ref_grad), red, int(half_centor), *dims, groups, _ptr(ref_image),
            _ptr(src_images), _ptr(base_plane), _ptr(offsets), _ptr(rs), _ptr(ts), _ptr(cost_grad),
            _ptr(cost_mask), _ptr(ref_grad), _ptr(src_grad), _ptr(bp_grad))
    _lib.check(rc)
    return ref_grad, src_grad, bp_grad


def _check_feature(src_images, base_plane, offsets, Rs, Ts):
    # feature_aggregate_kernels.cc:69-92
    _require(src_images.dim() == 5, "src_images must have rank 5")
    B, N, srcH, srcW, C = src_images.shape
    _require(base_plane.dim() == 4 and base_plane.shape[0] == B and base_plane.shape[3] == 1,
             "base_plane must have rank 4, and must compate to ref_image")
    H, W = base_plane.shape[1:3]
    _require(offsets.dim() == 2 and offsets.shape[0] == B,
             "offsets must have rank 2, and must compate to ref_image")
    _require(Rs.dim() == 4 and tuple(Rs.shape) == (B, N, 3, 3),
             "Rs must have rank 2, and must compate to ref_image")
    _require(Ts.dim() == 3 and tuple(Ts.shape) == (B, N, 3),
             "Ts must have rank 2, and must compate to ref_image")
    return B, H, W, C, offsets.shape[1], N, srcH, srcW


def feature_aggregate_raw(src_images, base_plane, offsets, Rs, Ts, half_centor=True):
    """The ``FeatureAggregate`` op without autograd: ``(mapped_feature [B,H,W,D,N,C],
    mapped_mask int32 [B,H,W,D,N,1])``; H and W are base_plane's (shapes:
    custom_helper_op/cc/ops/custom_helper_ops.cc:414-440)."""
    lib = _lib.load()
    dt, dev = src_images.dtype, src_images.device
    _require(dt in (torch.float32, torch.float64), "dtype must be float32 or float64")
    src_images = _prep(src_images, dt, dev, "src_images")
    base_plane = _prep(base_plane, dt, dev, "base_plane")
    offsets = _prep(offsets, dt, dev, "offsets")
    Rs, Ts = _prep(Rs, dt, dev, "Rs"), _prep(Ts, dt, dev, "Ts")
    B, H, W, C, D, N, srcH, srcW = dims = _check_feature(src_images, base_plane, offsets, Rs, Ts)
    mapped = torch.empty((B, H, W, D, N, C), dtype=dt, device=dev)
    mask = torch.empty((B, H, W, D, N, 1), dtype=torch.int32, device=dev)
    fn = (lib.chop_feature_aggregate_fwd_f32 if dt == torch.float32
          else lib.chop_feature_aggregate_fwd_f64)
    rc = fn(_stream(mapped), int(half_centor), *dims, _ptr(src_images), _ptr(base_plane),
            _ptr(offsets), _ptr(Rs), _ptr(Ts), _ptr(mapped), _ptr(mask))
    _lib.check(rc)
    return mapped, mask


def feature_aggregate_grad(src_images, base_plane, offsets, rs, ts, mapped_feature_grad,
                           mapped_mask, half_centor=True):
    """The ``FeatureAggregateGrad`` op: ``(src_images_grad, base_plane_grad)``
    (checks: feature_aggregate_kernels.cc:176-210)."""
    lib = _lib.load()
    dt, dev = src_images.dtype, src_images.device
    _require(dt in (torch.float32, torch.float64), "dtype must be float32 or float64")
    src_images = _prep(src_images, dt, dev, "src_images")
    base_plane = _prep(base_plane, dt, dev, "base_plane")
    offsets = _prep(offsets, dt, dev, "offsets")
    rs, ts = _prep(rs, dt, dev, "Rs"), _prep(ts, dt, dev, "Ts")
    mapped_feature_grad = _prep(mapped_feature_grad, dt, dev, "mapped_feature_grad")
    mapped_mask = _prep(mapped_mask, torch.int32, dev, "mapped_mask")
    B, H, W, C, D, N, srcH, srcW = dims = _check_feature(src_images, base_plane, offsets, rs, ts)
    _require(tuple(mapped_feature_grad.shape) == (B, H, W, D, N, C),
             "mapped_feature_grad must have rank 6, and must compate to src_images")
    _require(tuple(mapped_mask.shape) == (B, H, W, D, N, 1),
             "mapped_mask must have rank 6, and must compate to src_images")
    src_grad = torch.empty_like(src_images)
    bp_grad = torch.empty_like(base_plane)
    fn = (lib.chop_feature_aggregate_bwd_f32 if dt == torch.float32
          else lib.chop_feature_aggregate_bwd_f64)
    rc = fn(_stream(src_grad), int(half_centor), *dims, _ptr(src_images), _ptr(base_plane),
            _ptr(offsets), _ptr(rs), _ptr(ts), _ptr(mapped_feature_grad), _ptr(mapped_mask),
            _ptr(src_grad), _ptr(bp_grad))
    _lib.check(rc)
    return src_grad, bp_grad


class _CostVolume(torch.autograd.Function):
    """Forward = CostVolume, backward = the gradient registered for it
    (custom_helper_ops.py:41-61): the Grad op is fed the forward's cost_mask, the incoming
    gradient of cost_mask is ignored, offsets/Rs/Ts receive no gradient."""

    @staticmethod
    def forward(ctx, ref_image, src_images, base_plane, offsets, Rs, Ts, reduce_method, half_centor):
        cost, mask = cost_volume_raw(ref_image, src_images, base_plane, offsets, Rs, Ts,
                                     reduce_method, half_centor)
        ctx.save_for_backward(ref_image, src_images, base_plane, offsets, Rs, Ts, mask)
        ctx.attrs = (reduce_method, half_centor)
        ctx.mark_non_differentiable(mask)
        return cost, mask

    @staticmethod
    def backward(ctx, grad_out, _grad_mask):
        ref_image, src_images, base_plane, offsets, Rs, Ts, mask = ctx.saved_tensors
        rg, sg, bg = cost_volume_grad(ref_image, src_images, base_plane, offsets, Rs, Ts,
                                      grad_out.contiguous(), mask, *ctx.attrs,
                                      need_depth_grad=ctx.needs_input_grad[2])
        return rg, sg, bg, None, None, None, None, None


class _CostVolumeV2(torch.autograd.Function):
    """CostVolumeV2 with its registered gradient (custom_helper_ops.py:74-94)."""

    @staticmethod
    def forward(ctx, ref_image, src_images, depth_grid, Rs, Ts, reduce_method, groups, half_centor):
        cost, mask = cost_volume_v2_raw(ref_image, src_images, depth_grid, Rs, Ts, reduce_method,
                                        groups, half_centor)
        ctx.save_for_backward(ref_image, src_images, depth_grid, Rs, Ts, mask)
        ctx.attrs = (reduce_method, groups, half_centor)
        ctx.mark_non_differentiable(mask)
        return cost, mask

    @staticmethod
    def backward(ctx, grad_out, _grad_mask):
        ref_image, src_images, depth_grid, Rs, Ts, mask = ctx.saved_tensors
        rg, sg, dg = cost_volume_grad_v2(ref_image, src_images, depth_grid, Rs, Ts,
                                         grad_out.contiguous(), mask, *ctx.attrs,
                                         need_depth_grad=ctx.needs_input_grad[2])
        return rg, sg, dg, None, None, None, None, None


class _CostAggregate(torch.autograd.Function):
    """CostAggregate with its registered gradient (custom_helper_ops.py:141-161)."""

    @staticmethod
    def forward(ctx, ref_image, src_images, base_plane, offsets, Rs, Ts, reduce_method, half_centor):
        cost, mask = cost_aggregate_raw(ref_image, src_images, base_plane, offsets, Rs, Ts,
                                        reduce_method, half_centor)
        ctx.save_for_backward(ref_image, src_images, base_plane, offsets, Rs, Ts, mask)
        ctx.attrs = (reduce_method, half_centor)
        ctx.mark_non_differentiable(mask)
        return cost, mask

    @staticmethod
    def backward(ctx, grad_out, _grad_mask):
        ref_image, src_images, base_plane, offsets, Rs, Ts, mask = ctx.saved_tensors
        rg, sg, bg = cost_aggregate_grad(ref_image, src_images, base_plane, offsets, Rs, Ts,
                                         grad_out.contiguous(), mask, *ctx.attrs,
                                         need_depth_grad=ctx.needs_input_grad[2])
        return rg, sg, bg, None, None, None, None, None


def _default_grad(grad_out, mask, reduce_method, like):
    """Gradient of the layers' scalar default: the upstream gradient summed over the voxels
    that received it (one reduction kernel; 16-bit storage is read as stored and summed in
    float, without a widened copy)."""
    lib = _lib.load()
    red = _reduce_code(reduce_method)
    g = grad_out.contiguous()
    n_mask = mask.numel()
    inner = g.numel() // n_mask if n_mask else 1
    out = torch.empty((), dtype=_real_dtype(g.dtype), device=g.device)
    if g.dtype in _STORAGE16:
        _lib.check(lib.chop_cost_default_fill_grad_16(_stream(out), _STORAGE16[g.dtype], red, n_mask,
                                                      inner, _ptr(g), _ptr(mask), None, _ptr(out)))
    else:
        fn = (lib.chop_cost_default_fill_grad_f32 if g.dtype == torch.float32
              else lib.chop_cost_default_fill_grad_f64)
        _lib.check(fn(_stream(out), red, n_mask, inner, _ptr(g), _ptr(mask), None, _ptr(out)))
    return out.to(like.dtype).reshape(like.shape)


class _CostVolumeV2Filled(torch.autograd.Function):
    """``CostMapLayerV2.call`` (custom_layers.py:77-83) as one forward kernel: CostVolumeV2 whose
    store writes ``default_cost`` where no view was accepted.  The op's registered gradient
    skips exactly those voxels, so it takes the upstream gradient as it is."""

    @staticmethod
    def forward(ctx, ref_image, src_images, depth_grid, Rs, Ts, default_cost, reduce_method, groups,
                half_centor):
        cost, mask = cost_volume_v2_raw(ref_image, src_images, depth_grid, Rs, Ts, reduce_method,
                                        groups, half_centor, default_cost=default_cost)
        ctx.save_for_backward(ref_image, src_images, depth_grid, Rs, Ts, mask, default_cost)
        ctx.attrs = (reduce_method, groups, half_centor)
        ctx.mark_non_differentiable(mask)
        return cost, mask

    @staticmethod
    def backward(ctx, grad_out, _grad_mask):
        ref_image, src_images, depth_grid, Rs, Ts, mask, default_cost = ctx.saved_tensors
        rg, sg, dg = cost_volume_grad_v2(ref_image, src_images, depth_grid, Rs, Ts,
                                         grad_out.contiguous(), mask, *ctx.attrs,
                                         need_depth_grad=ctx.needs_input_grad[2])
        dd = (_default_grad(grad_out, mask, ctx.attrs[0], default_cost)
              if ctx.needs_input_grad[5] else None)
        return rg, sg, dg, None, None, dd, None, None, None


class _CostAggregateFilled(torch.autograd.Function):
    """``CostMapLayer.call`` (custom_layers.py:51-57) as one forward kernel."""

    @staticmethod
    def forward(ctx, ref_image, src_images, base_plane, offsets, Rs, Ts, default_cost, reduce_method,
                half_centor):
        cost, mask = cost_aggregate_raw(ref_image, src_images, base_plane, offsets, Rs, Ts,
                                        reduce_method, half_centor, default_cost=default_cost)
        ctx.save_for_backward(ref_image, src_images, base_plane, offsets, Rs, Ts, mask, default_cost)
        ctx.attrs = (reduce_method, half_centor)
        ctx.mark_non_differentiable(mask)
        return cost, mask

    @staticmethod
    def backward(ctx, grad_out, _grad_mask):
        ref_image, src_images, base_plane, offsets, Rs, Ts, mask, default_cost = ctx.saved_tensors
        rg, sg, bg = cost_aggregate_grad(ref_image, src_images, base_plane, offsets, Rs, Ts,
                                         grad_out.contiguous(), mask, *ctx.attrs,
                                         need_depth_grad=ctx.needs_input_grad[2])
        dd = (_default_grad(grad_out, mask, ctx.attrs[0], default_cost)
              if ctx.needs_input_grad[6] else None)
        return rg, sg, bg, None, None, None, dd, None, None


def cost_volume_v2_filled(ref_image, src_images, depth_grid, Rs, Ts, default_cost,
                          reduce_method="MEAN", groups=None, half_centor=True):
    """CostVolumeV2 followed by ``where(valid(cost_mask), cost, default_cost)``, fused into one
    kernel; differentiable in the images, the depth grid and the scalar."""
    return _CostVolumeV2Filled.apply(ref_image, src_images, depth_grid, Rs, Ts, default_cost,
                                     reduce_method, groups, half_centor)


def cost_aggregate_filled(ref_image, src_images, base_plane, offsets, Rs, Ts, default_cost,
                          reduce_method="MEAN", half_centor=True):
    """CostAggregate followed by the same fill, fused into one kernel."""
    return _CostAggregateFilled.apply(ref_image, src_images, base_plane, offsets, Rs, Ts,
                                      default_cost, reduce_method, half_centor)


class _CostVolumeV3(torch.autograd.Function):
    """CostVolumeV3 with its registered gradient (custom_helper_ops.py:107-131)."""

    @staticmethod
    def forward(ctx, ref_image, src_images, base_plane, offsets, Rs, Ts, reduce_method, groups,
                half_centor):
        cost, mask = cost_volume_v3_raw(ref_image, src_images, base_plane, offsets, Rs, Ts,
                                        reduce_method, groups, half_centor)
        ctx.save_for_backward(ref_image, src_images, base_plane, offsets, Rs, Ts, mask)
        ctx.attrs = (reduce_method, groups, half_centor)
        ctx.mark_non_differentiable(mask)
        return cost, mask

    @staticmethod
    def backward(ctx, grad_out, _grad_mask):
        ref_image, src_images, base_plane, offsets, Rs, Ts, mask = ctx.saved_tensors
        rg, sg, bg = cost_volume_grad_v3(ref_image, src_images, base_plane, offsets, Rs, Ts,
                                         grad_out.contiguous(), mask, *ctx.attrs)
        return rg, sg, bg, None, None, None, None, None, None


class _FeatureAggregate(torch.autograd.Function):
    """FeatureAggregate with its registered gradient (custom_helper_ops.py:174-195)."""

    @staticmethod
    def forward(ctx, src_images, base_plane, offsets, Rs, Ts, half_centor):
        mapped, mask = feature_aggregate_raw(src_images, base_plane, offsets, Rs, Ts, half_centor)
        ctx.save_for_backward(src_images, base_plane, offsets, Rs, Ts, mask)
        ctx.half_centor = half_centor
        ctx.mark_non_differentiable(mask)
        return mapped, mask

    @staticmethod
    def backward(ctx, grad_out, _grad_mask):
        src_images, base_plane, offsets, Rs, Ts, mask = ctx.saved_tensors
        sg, bg = feature_aggregate_grad(src_images, base_plane, offsets, Rs, Ts,
                                        grad_out.contiguous(), mask, ctx.half_centor)
        return sg, bg, None, None, None, None


def cost_volume(ref_image, src_images, base_plane, offsets, Rs, Ts, reduce_method="MEAN",
                half_centor=True, name=None):
    """``custom_helper_op.cost_volume``: returns ``(cost, cost_mask)``; differentiable with
    respect to ref_image, src_images and base_plane."""
    del name
    offsets = torch.as_tensor(offsets, device=ref_image.device)
    Rs = torch.as_tensor(Rs, device=ref_image.device)
    Ts = torch.as_tensor(Ts, device=ref_image.device)
    return _CostVolume.apply(ref_image, src_images, base_plane, offsets, Rs, Ts, reduce_method,
                             half_centor)


def cost_volume_v2(ref_image, src_images, depth_grid, Rs, Ts, reduce_method="MEAN", groups=None,
                   half_centor=True, name=None):
    """``custom_helper_op.cost_volume_v2``: returns ``(cost [B,H,W,D,groups], cost_mask)``."""
    del name
    depth_grid = torch.as_tensor(depth_grid, device=ref_image.device)
    Rs = torch.as_tensor(Rs, device=ref_image.device)
    Ts = torch.as_tensor(Ts, device=ref_image.device)
    return _CostVolumeV2.apply(ref_image, src_images, depth_grid, Rs, Ts, reduce_method, groups,
                               half_centor)


def cost_aggregate(ref_image, src_images, base_plane, offsets, Rs, Ts, reduce_method="MEAN",
                   half_centor=True, name=None):
    """``custom_helper_op.cost_aggregate`` (custom_helper_ops.py:133-138): returns
    ``(cost [B,H,W,D], cost_mask [B,H,W,D])``; differentiable with respect to ref_image,
    src_images and base_plane."""
    del name
    offsets = torch.as_tensor(offsets, device=ref_image.device)
    Rs = torch.as_tensor(Rs, device=ref_image.device)
    Ts = torch.as_tensor(Ts, device=ref_image.device)
    return _CostAggregate.apply(ref_image, src_images, base_plane, offsets, Rs, Ts, reduce_method,
                                half_centor)


def cost_volume_v3(ref_image, src_images, base_plane, offsets, Rs, Ts, reduce_method="MEAN",
                   groups=None, half_centor=True, name=None):
    """``custom_helper_op.cost_volume_v3`` (custom_helper_ops.py:99-104): returns
    ``(cost [B,H,W,D,1], cost_mask)``; differentiable with respect to ref_image, src_images and
    base_plane."""
    del name
    offsets = torch.as_tensor(offsets, device=ref_image.device)
    Rs = torch.as_tensor(Rs, device=ref_image.device)
    Ts = torch.as_tensor(Ts, device=ref_image.device)
    return _CostVolumeV3.apply(ref_image, src_images, base_plane, offsets, Rs, Ts, reduce_method,
                               groups, half_centor)


def feature_aggregate(src_images, base_plane, offsets, Rs, Ts, half_centor=True, name=None):
    """``custom_helper_op.feature_aggregate`` (custom_helper_ops.py:166-171): returns
    ``(mapped_feature [B,H,W,D,N,C], mapped_mask [B,H,W,D,N,1])``; differentiable with respect
    to src_images and base_plane."""
    del name
    offsets = torch.as_tensor(offsets, device=src_images.device)
    Rs = torch.as_tensor(Rs, device=src_images.device)
    Ts = torch.as_tensor(Ts, device=src_images.device)
    return _FeatureAggregate.apply(src_images, base_plane, offsets, Rs, Ts, half_centor)


class _DefaultFill(torch.autograd.Function):
    """``tf.where(valid(cost_mask), cost, default_cost)`` with its gradient, as one kernel each
    way (custom_helper_op/python/layers/custom_layers.py:52-57, :78-83)."""

    @staticmethod
    def forward(ctx, cost, cost_mask, default_cost, reduce_method):
        lib = _lib.load()
        red = _reduce_code(reduce_method)
        dt, dev = cost.dtype, cost.device
        _require(dt in (torch.float32, torch.float64), "dtype must be float32 or float64")
        cost = _prep(cost, dt, dev, "cost")
        cost_mask = _prep(cost_mask, torch.int32, dev, "cost_mask")
        default_cost = _prep(default_cost, dt, dev, "default_cost")
        _require(default_cost.numel() == 1, "default_cost must be a scalar")
        n_mask = cost_mask.numel()
        _require(n_mask > 0 and cost.numel() % n_mask == 0 or cost.numel() == 0,
                 "cost_mask must cover cost with a whole number of elements per entry")
        inner = cost.numel() // n_mask if n_mask else 1
        out = torch.empty_like(cost)
        fn = lib.chop_cost_default_fill_f32 if dt == torch.float32 else lib.chop_cost_default_fill_f64
        _lib.check(fn(_stream(out), red, n_mask, inner, _ptr(cost), _ptr(cost_mask),
                      _ptr(default_cost), _ptr(out)))
        ctx.save_for_backward(cost_mask)
        ctx.attrs = (red, n_mask, inner, default_cost.shape)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        lib = _lib.load()
        (cost_mask,) = ctx.saved_tensors
        red, n_mask, inner, dshape = ctx.attrs
        grad_out = grad_out.contiguous()
        cost_grad = torch.empty_like(grad_out)
        default_grad = torch.empty(dshape, dtype=grad_out.dtype, device=grad_out.device)
        fn = (lib.chop_cost_default_fill_grad_f32 if grad_out.dtype == torch.float32
              else lib.chop_cost_default_fill_grad_f64)
        _lib.check(fn(_stream(cost_grad), red, n_mask, inner, _ptr(grad_out), _ptr(cost_mask),
                      _ptr(cost_grad), _ptr(default_grad)))
        return cost_grad, None, default_grad, None


def cost_default_fill(cost, cost_mask, default_cost, reduce_method="MEAN"):
    """``where(cost_mask > 0, cost, default_cost)`` for MEAN, ``cost_mask >= 0`` for MIN: what
    ``CostMapLayer`` / ``CostMapLayerV2`` apply to the op's outputs; differentiable with respect
    to ``cost`` and the scalar ``default_cost``.  ``cost_mask`` may have one entry per cost
    element or one per row of the last axis."""
    return _DefaultFill.apply(cost, cost_mask, default_cost, reduce_method)


def combine_projection(ref_cam, src_cam, scale):
    """The relative projection the ops take, computed on the device
    (custom_helper_op/python/ops/op_tests/cost_volume_op_test.py:115-134).
    ``ref_cam [B,2,4,4]`` (or ``[2,4,4]``), ``src_cam [B,N,2,4,4]`` (or ``[2,4,4]``), ``scale [3]``
    -> ``(Rs [B,N,3,3], Ts [B,N,3])``; the unbatched form returns ``(R [3,3], T [3,1])`` like the
    reference helper."""
    lib = _lib.load()
    single = ref_cam.dim() == 3
    dt, dev = ref_cam.dtype, ref_cam.device
    _require(dt in (torch.float32, torch.float64), "dtype must be float32 or float64")
    if single:
        _require(tuple(ref_cam.shape) == (2, 4, 4) and tuple(src_cam.shape) == (2, 4, 4),
                 "cameras must be [2,4,4]")
        ref_cam, src_cam = ref_cam[None], src_cam[None, None]
    ref_cam = _prep(ref_cam, dt, dev, "ref_cam")
    src_cam = _prep(src_cam, dt, dev, "src_cam")
    scale = _prep(scale, dt, dev, "scale")
    _require(ref_cam.dim() == 4 and tuple(ref_cam.shape[1:]) == (2, 4, 4), "ref_cam must be [B,2,4,4]")
    B = ref_cam.shape[0]
    _require(src_cam.dim() == 5 and src_cam.shape[0] == B and tuple(src_cam.shape[2:]) == (2, 4, 4),
             "src_cam must be [B,N,2,4,4]")
    _require(tuple(scale.shape) == (3,), "scale must have 3 entries")
    N = src_cam.shape[1]
    Rs = torch.empty((B, N, 3, 3), dtype=dt, device=dev)
    Ts = torch.empty((B, N, 3), dtype=dt, device=dev)
    fn = lib.chop_combine_projection_f32 if dt == torch.float32 else lib.chop_combine_projection_f64
    _lib.check(fn(_stream(Rs), B, N, _ptr(ref_cam), _ptr(src_cam), _ptr(scale), _ptr(Rs), _ptr(Ts)))
    if single:
        return Rs[0, 0], Ts[0, 0][:, None]
    return Rs, Ts


def sample_coords(base_plane, offsets, Rs, Ts, src_hw, half_centor=True, depth_grid=None):
    """Diagnostic: per-(voxel, view) sample coordinates ``[B,H,W,D,N]`` as the kernels
    compute them: ``(sw, sh, fh, fw, state)``."""
    lib = _lib.load()
    if depth_grid is not None:
        dt, dev = depth_grid.dtype, depth_grid.device
        depth_grid = depth_grid.contiguous()
        B, H, W, D = depth_grid.shape
    else:
        dt, dev = base_plane.dtype, base_plane.device
        base_plane, offsets = base_plane.contiguous(), offsets.contiguous()
        B, H, W = base_plane.shape[:3]
        D = offsets.shape[1]
    Rs, Ts = _prep(Rs, dt, dev, "Rs"), _prep(Ts, dt, dev, "Ts")
    N = Rs.shape[1]
    shape = (B, H, W, D, N)
    sw, sh = (torch.empty(shape, dtype=dt, device=dev) for _ in range(2))
    fh, fw, st = (torch.empty(shape, dtype=torch.int32, device=dev) for _ in range(3))
    fn = (lib.chop_cost_volume_sample_coords_f32 if dt == torch.float32
          else lib.chop_cost_volume_sample_coords_f64)
    rc = fn(_stream(sw), int(half_centor), B, H, W, D, N, src_hw[0], src_hw[1], _ptr(base_plane),
            _ptr(offsets), _ptr(depth_grid), _ptr(Rs), _ptr(Ts), _ptr(sw), _ptr(sh), _ptr(fh),
            _ptr(fw), _ptr(st))
    _lib.check(rc)
    return sw, sh, fh, fw, st
