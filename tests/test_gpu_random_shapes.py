"""GPU parity on seeded random shapes: CostVolume and CostVolumeV2, both reduces, float32 and
float64, whatever kernel family the library picks for the shape (tiled, strip or general).
The fixed-shape tests cover the benchmark and reference shapes; this sweep is for what lies
between them: odd image sizes (ragged two-row tiles), fewer depths than a chunk, channel
counts on both sides of the tiled kernels' list, one to seven views, batch 1 and 2."""
import numpy as np
import pytest

import custom_helper_op_amd as chop
from custom_helper_op_amd import _lib
from custom_helper_op_amd.configs import reference_test_case
from gpu_util import assert_backward_close, assert_forward_close, dev, host

pytestmark = pytest.mark.gpu

TILED_CHANNELS = (4, 8, 16, 32, 64)


def _case(seed):
    rng = np.random.default_rng(5000 + seed)
    B = int(rng.integers(1, 3))
    N = int(rng.integers(1, 8))
    H = int(rng.integers(3, 24))
    W = int(rng.integers(3, 38))
    D = int(rng.integers(1, 41))
    C = int(rng.choice([1, 2, 3, 4, 5, 8, 9, 12, 16, 24, 32, 33, 40, 64]))
    dtype = np.float64 if rng.random() < 0.3 else np.float32
    reduce = "MIN" if rng.random() < 0.4 else "MEAN"
    half = bool(rng.random() < 0.7)
    camera = int(rng.integers(0, 4))
    t = reference_test_case(camera, B, N, H, W, C, D, dtype, seed=seed)
    # different views, some of them partly out of the frustum
    t["Ts"] = (t["Ts"] + rng.uniform(-2.0, 2.0, t["Ts"].shape)).astype(dtype)
    divisors = [g for g in (1, 2, 3, 4, 5, 8) if C % g == 0]
    groups = int(rng.choice(divisors))
    return t, (B, N, H, W, C, D), dtype, reduce, half, groups


@pytest.mark.parametrize("seed", range(48))
def test_random_shape(oracle, seed):
    t, shape, dtype, reduce, half, groups = _case(seed)
    B, N, H, W, C, D = shape
    print("\n[case] seed %d: B%d N%d %dx%d C%d D%d %s %s half=%s groups=%d" % (
        seed, B, N, H, W, C, D, np.dtype(dtype).name, reduce, half, groups), flush=True)
    lib = _lib.load()
    args = tuple(t[k] for k in ("ref", "src", "base_plane", "offsets", "Rs", "Ts"))
    d_args = [dev(x) for x in args]
    rng = np.random.default_rng(seed)

    want_cost, want_mask = oracle.cost_volume_fwd(*args, reduce, half)
    cost, mask = chop.cost_volume_raw(*d_args, reduce, half)
    family = lib.chop_last_kernel_family()
    assert family == (2 if dtype == np.float32 and C in TILED_CHANNELS and N <= 6 else 3), family
    assert np.array_equal(host(mask), want_mask)
    if family == 3 or reduce == "MIN":
        assert np.array_equal(host(cost), want_cost)  # literal operand order: bit-identical
    else:
        assert_forward_close(host(cost), want_cost)
    cg = rng.standard_normal(want_cost.shape).astype(dtype)
    want = oracle.cost_volume_bwd(*args, cg, want_mask, reduce, half)
    got = chop.cost_volume_grad(*d_args, dev(cg), mask, reduce, half)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)

    depth_grid = (t["base_plane"] + t["offsets"][:, None, None, :]).astype(dtype)
    a2 = (t["ref"], t["src"], depth_grid, t["Rs"], t["Ts"])
    d2 = [dev(x) for x in a2]
    want_cost, want_mask = oracle.cost_volume_v2_fwd(*a2, reduce, groups, half)
    cost, mask = chop.cost_volume_v2_raw(*d2, reduce, groups, half)
    family = lib.chop_last_kernel_family()
    assert np.array_equal(host(mask), want_mask)
    if family == 3 or reduce == "MIN":
        assert np.array_equal(host(cost), want_cost)
    else:
        assert_forward_close(host(cost), want_cost, atol=1e-5)
    cg = rng.standard_normal(want_cost.shape).astype(dtype)
    want = oracle.cost_volume_v2_bwd(*a2, cg, want_mask, reduce, groups, half)
    got = chop.cost_volume_grad_v2(*d2, dev(cg), mask, reduce, groups, half)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)


@pytest.mark.parametrize("seed", range(100, 132))
def test_random_shape_other_ops(oracle, seed):
    """CostAggregate, CostVolumeV3 and FeatureAggregate on the same kind of shapes.  Forward
    values: masks and every index bit-exact; CostVolumeV3 and FeatureAggregate bit-identical in
    every family, CostAggregate MEAN within 1e-5 where the tiled kernels serve it."""
    t, shape, dtype, reduce, half, _ = _case(seed)
    B, N, H, W, C, D = shape
    print("\n[case] seed %d: B%d N%d %dx%d C%d D%d %s %s half=%s" % (
        seed, B, N, H, W, C, D, np.dtype(dtype).name, reduce, half), flush=True)
    lib = _lib.load()
    tol = 1e-4 if dtype == np.float32 else 1e-10
    args = tuple(t[k] for k in ("ref", "src", "base_plane", "offsets", "Rs", "Ts"))
    d_args = [dev(x) for x in args]
    rng = np.random.default_rng(seed)

    want_cost, want_mask = oracle.cost_aggregate_fwd(*args, reduce, half)
    cost, mask = chop.cost_aggregate_raw(*d_args, reduce, half)
    assert np.array_equal(host(mask), want_mask)
    if lib.chop_last_kernel_family() != 2 or reduce == "MIN":
        assert np.array_equal(host(cost), want_cost)  # general and strip kernels: bit-identical
    else:
        assert_forward_close(host(cost), want_cost)
    cg = rng.standard_normal(want_cost.shape).astype(dtype)
    want = oracle.cost_aggregate_bwd(*args, cg, want_mask, reduce, half)
    got = chop.cost_aggregate_grad(*d_args, dev(cg), mask, reduce, half)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w, tol)

    # at most 8 channels per group (MAX_SUBCHANNELS_SIZE, cost_volume_v3.h:35)
    groups = int(rng.choice([g for g in range(1, C + 1) if C % g == 0 and C // g <= 8]))
    signed = dict(t, ref=t["ref"] - 5, src=t["src"] - 5)  # some maxima stay at the seed
    for tt in (t, signed):
        a3 = tuple(tt[k] for k in ("ref", "src", "base_plane", "offsets", "Rs", "Ts"))
        d3 = [dev(x) for x in a3]
        want_cost, want_mask = oracle.cost_volume_v3_fwd(*a3, reduce, groups, half)
        cost, mask = chop.cost_volume_v3_raw(*d3, reduce, groups, half)
        assert np.array_equal(host(mask), want_mask)
        assert np.array_equal(host(cost), want_cost)
        cg = rng.standard_normal(want_cost.shape).astype(dtype)
        want = oracle.cost_volume_v3_bwd(*a3, cg, want_mask, reduce, groups, half)
        got = chop.cost_volume_grad_v3(*d3, dev(cg), mask, reduce, groups, half)
        for g, w in zip(got, want):
            assert_backward_close(host(g), w, tol)

    af = tuple(t[k] for k in ("src", "base_plane", "offsets", "Rs", "Ts"))
    df = [dev(x) for x in af]
    want, want_mask = oracle.feature_aggregate_fwd(*af, half)
    mapped, mask = chop.feature_aggregate_raw(*df, half)
    tiled = dtype == np.float32 and C in TILED_CHANNELS and N <= 6
    assert lib.chop_last_kernel_family() == (2 if tiled else 3)
    assert np.array_equal(host(mask), want_mask)
    assert np.array_equal(host(mapped), want)
    g = rng.standard_normal(want.shape).astype(dtype)
    want_g = oracle.feature_aggregate_bwd(*af, g, want_mask, half)
    got_g = chop.feature_aggregate_grad(*df, dev(g), mask, half)
    for a, b in zip(got_g, want_g):
        assert_backward_close(host(a), b, tol)


@pytest.mark.parametrize("seed", range(200, 224))
def test_random_shape_16bit_storage(oracle, seed):
    """float16 / bfloat16 feature storage with float32 arithmetic: the float32 oracle on the
    quantised inputs, masks bit-exact, values within 1e-2 (the outputs themselves are rounded to
    11 or 8 significant bits).  CostVolume over planes and over a depth grid, CostVolumeV2."""
    import torch
    from custom_helper_op_amd.configs import quantise
    from gpu_util import TORCH_DTYPE, rms
    t, shape, _, reduce, half, groups = _case(seed)
    B, N, H, W, C, D = shape
    storage = "f16" if seed % 2 else "bf16"
    print("\n[case] seed %d: B%d N%d %dx%d C%d D%d %s %s half=%s groups=%d" % (
        seed, B, N, H, W, C, D, storage, reduce, half, groups), flush=True)
    td = TORCH_DTYPE[storage]
    f32 = np.float32
    ref, src = quantise(t["ref"].astype(f32), storage), quantise(t["src"].astype(f32), storage)
    bp, off, Rs, Ts = (t[k].astype(f32) for k in ("base_plane", "offsets", "Rs", "Ts"))
    rng = np.random.default_rng(seed)

    def close(got, want, mask=None):
        if mask is not None and reduce == "MIN":
            # an element no view reached keeps the float seed, rounded to the storage type:
            # FLT_MAX becomes +inf in both 16-bit types, the correlation's 1.18e-38 stays (bf16)
            # or becomes 0 (f16); the mask (-1) is what marks such an element
            empty = mask < 0
            assert np.all(np.isinf(got[empty]) | (np.abs(got[empty]) < 1e-37))
            got, want = got[~empty], want[~empty]
        np.testing.assert_allclose(got, want, rtol=1e-2, atol=1e-2 * max(rms(want), 1e-30))

    want_cost, want_mask = oracle.cost_volume_fwd(ref, src, bp, off, Rs, Ts, reduce, half)
    ins = [dev(ref, td), dev(src, td), dev(bp), dev(off), dev(Rs), dev(Ts)]
    cost, mask = chop.cost_volume_raw(*ins, reduce, half)
    assert cost.dtype == td
    assert np.array_equal(host(mask), want_mask)
    close(host(cost), want_cost, want_mask)
    cg = quantise(rng.standard_normal(want_cost.shape).astype(f32), storage)
    want = oracle.cost_volume_bwd(ref, src, bp, off, Rs, Ts, cg, want_mask, reduce, half)
    got = chop.cost_volume_grad(*ins, dev(cg, td), mask, reduce, half)
    assert got[2].dtype == torch.float32
    for g, w in zip(got, want):
        close(host(g), w)

    grid = (bp * (1.0 + 0.01 * (np.arange(D, dtype=f32) - D // 2))[None, None, None]).astype(f32)
    want_cost, want_mask = oracle.cost_volume_grid_fwd(ref, src, grid, Rs, Ts, reduce, half)
    gins = [dev(ref, td), dev(src, td), None, None, dev(Rs), dev(Ts)]
    cost, mask = chop.cost_volume_raw(*gins, reduce, half, depth_grid=dev(grid))
    assert np.array_equal(host(mask), want_mask)
    close(host(cost), want_cost, want_mask)
    want = oracle.cost_volume_grid_bwd(ref, src, grid, Rs, Ts, cg, want_mask, reduce, half)
    got = chop.cost_volume_grad(*gins, dev(cg, td), mask, reduce, half, depth_grid=dev(grid))
    assert got[2].shape == (B, H, W, D)
    for g, w in zip(got, want):
        close(host(g), w)

    want_cost, want_mask = oracle.cost_volume_v2_fwd(ref, src, grid, Rs, Ts, reduce, groups, half)
    vins = [dev(ref, td), dev(src, td), dev(grid), dev(Rs), dev(Ts)]
    cost, mask = chop.cost_volume_v2_raw(*vins, reduce, groups, half)
    assert np.array_equal(host(mask), want_mask)
    close(host(cost), want_cost, want_mask)
    cg = quantise(rng.standard_normal(want_cost.shape).astype(f32), storage)
    want = oracle.cost_volume_v2_bwd(ref, src, grid, Rs, Ts, cg, want_mask, reduce, groups, half)
    got = chop.cost_volume_grad_v2(*vins, dev(cg, td), mask, reduce, groups, half)
    for g, w in zip(got, want):
        close(host(g), w)
