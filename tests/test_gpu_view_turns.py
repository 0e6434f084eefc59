"""Narrow pixels on large images: the backward kernels in which one workgroup goes through all
views of its pixel tile in turn (up to 8 channels, at least 10240 pixel tiles), so that the
pixel-owned gradients need neither atomics nor a zero fill.  Every op that reaches those
kernels, forward and backward against the oracle; `chop_last_views_per_workgroup` confirms
that the launch really took that form."""
import numpy as np
import pytest
import torch

import custom_helper_op_amd as chop
from custom_helper_op_amd import _lib
from custom_helper_op_amd.configs import make_workload, quantise, reference_test_case
from gpu_util import TORCH_DTYPE, assert_backward_close, assert_forward_close, dev, host, rms

pytestmark = pytest.mark.gpu

HW8 = (400, 840)    # 336000 pixels: 10500 tiles of 32 pixels (8 channels)
HW4 = (660, 1000)   # 660000 pixels: 10330 tiles of 64 pixels (4 channels)
KEYS = ("ref", "src", "base_plane", "offsets", "Rs", "Ts")


@pytest.fixture(autouse=True)
def _announce(request):
    print("\n[case] %s" % request.node.nodeid, flush=True)
    _lib.load().chop_set_kernel_family(0)
    yield


def _turns(views):
    lib = _lib.load()
    assert lib.chop_last_kernel_family() == 2
    assert lib.chop_last_views_per_workgroup() == views


def _v1_case(C, hw, D=3):
    """Configuration 1's generator (8 channels, two source views) at another size."""
    wl = make_workload(1, hw=hw, depth=D, with_cost_grad=False)
    t = wl.tensors
    if C != wl.C:
        t["ref"] = np.ascontiguousarray(t["ref"][..., :C])
        t["src"] = np.ascontiguousarray(t["src"][..., :C])
    # a third view, so that the turns are more than two
    t["src"] = np.concatenate([t["src"], t["src"][:, :1, ::-1].copy()], axis=1)
    t["Rs"] = np.concatenate([t["Rs"], t["Rs"][:, 1:2]], axis=1)
    t["Ts"] = np.concatenate([t["Ts"], t["Ts"][:, 1:2] * np.float32(-0.7)], axis=1)
    return {k: np.ascontiguousarray(v) for k, v in t.items()}


@pytest.mark.parametrize("C,hw", [(8, HW8), (4, HW4)])
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_cost_volume(oracle, C, hw, reduce):
    t = _v1_case(C, hw)
    args = tuple(t[k] for k in KEYS)
    want_cost, want_mask = oracle.cost_volume_fwd(*args, reduce, threads=16)
    ins = [dev(x) for x in args]
    cost, mask = chop.cost_volume_raw(*ins, reduce)
    assert np.array_equal(host(mask), want_mask)
    cg = np.random.default_rng(C).standard_normal(want_cost.shape).astype(np.float32)
    want = oracle.cost_volume_bwd(*args, cg, want_mask, reduce, threads=16)
    got = chop.cost_volume_grad(*ins, dev(cg), mask, reduce)
    _turns(3)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)
    # without the depth gradient (another instantiation of the kernel)
    got = chop.cost_volume_grad(*ins, dev(cg), mask, reduce, need_depth_grad=False)
    _turns(3)
    for g, w in zip(got[:2], want[:2]):
        assert_backward_close(host(g), w)


@pytest.mark.parametrize("groups", [2, 4, 8])
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_cost_volume_v2(oracle, groups, reduce):
    t = _v1_case(8, HW8, D=4)
    depth_grid = (t["base_plane"] + t["offsets"][:, None, None, :]).astype(np.float32)
    depth_grid *= (1 + 0.01 * np.random.default_rng(2).standard_normal(depth_grid.shape)).astype(np.float32)
    args = (t["ref"], t["src"], depth_grid, t["Rs"], t["Ts"])
    want_cost, want_mask = oracle.cost_volume_v2_fwd(*args, reduce, groups, threads=16)
    ins = [dev(x) for x in args]
    cost, mask = chop.cost_volume_v2_raw(*ins, reduce, groups)
    assert np.array_equal(host(mask), want_mask)
    cg = np.random.default_rng(groups).standard_normal(want_cost.shape).astype(np.float32)
    want = oracle.cost_volume_v2_bwd(*args, cg, want_mask, reduce, groups, threads=16)
    got = chop.cost_volume_grad_v2(*ins, dev(cg), mask, reduce, groups)
    _turns(3)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)


@pytest.mark.parametrize("storage", ["f16", "bf16"])
def test_cost_volume_16bit_depth_grid(oracle, storage):
    """16-bit storage over per-voxel hypotheses (the fp32 gradient images of the workspace)."""
    t = _v1_case(8, HW8, D=4)
    td = TORCH_DTYPE[storage]
    ref, src = quantise(t["ref"], storage), quantise(t["src"], storage)
    depth_grid = (t["base_plane"] + t["offsets"][:, None, None, :]).astype(np.float32)
    want_cost, want_mask = oracle.cost_volume_grid_fwd(ref, src, depth_grid, t["Rs"], t["Ts"], threads=16)
    cg = quantise(np.random.default_rng(3).standard_normal(want_cost.shape).astype(np.float32), storage)
    want = oracle.cost_volume_grid_bwd(ref, src, depth_grid, t["Rs"], t["Ts"], cg, want_mask, threads=16)
    d_ref, d_src = dev(ref, td), dev(src, td)
    d_rs, d_ts, d_dg = dev(t["Rs"]), dev(t["Ts"]), dev(depth_grid)
    cost, mask = chop.cost_volume_raw(d_ref, d_src, None, None, d_rs, d_ts, depth_grid=d_dg)
    assert np.array_equal(host(mask), want_mask)
    got = chop.cost_volume_grad(d_ref, d_src, None, None, d_rs, d_ts, dev(cg, td), mask, depth_grid=d_dg)
    _turns(3)
    for g, w in zip(got, want):
        np.testing.assert_allclose(host(g), w, rtol=1e-2, atol=1e-2 * max(rms(w), 1e-30))


@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_cost_aggregate(oracle, reduce):
    t = _v1_case(8, HW8)
    args = tuple(t[k] for k in KEYS)
    want_cost, want_mask = oracle.cost_aggregate_fwd(*args, reduce, threads=16)
    ins = [dev(x) for x in args]
    cost, mask = chop.cost_aggregate_raw(*ins, reduce)
    assert np.array_equal(host(mask), want_mask)
    cg = np.random.default_rng(5).standard_normal(want_cost.shape).astype(np.float32)
    want = oracle.cost_aggregate_bwd(*args, cg, want_mask, reduce, threads=16)
    got = chop.cost_aggregate_grad(*ins, dev(cg), mask, reduce)
    _turns(3)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)


@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_cost_volume_v3(oracle, reduce):
    t = _v1_case(8, HW8)
    args = tuple(t[k] for k in KEYS)
    want_cost, want_mask = oracle.cost_volume_v3_fwd(*args, reduce, 2, threads=16)
    ins = [dev(x) for x in args]
    cost, mask = chop.cost_volume_v3_raw(*ins, reduce, 2)
    assert np.array_equal(host(mask), want_mask)
    assert np.array_equal(host(cost), want_cost)
    cg = np.random.default_rng(6).standard_normal(want_cost.shape).astype(np.float32)
    want = oracle.cost_volume_v3_bwd(*args, cg, want_mask, reduce, 2)
    got = chop.cost_volume_grad_v3(*ins, dev(cg), mask, reduce, 2)
    _turns(3)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)


def test_feature_aggregate(oracle):
    t = _v1_case(8, HW8)
    args = tuple(t[k] for k in ("src", "base_plane", "offsets", "Rs", "Ts"))
    want_feat, want_mask = oracle.feature_aggregate_fwd(*args, threads=16)
    ins = [dev(x) for x in args]
    feat, mask = chop.feature_aggregate_raw(*ins)
    assert np.array_equal(host(mask), want_mask)
    assert np.array_equal(host(feat), want_feat)
    cg = np.random.default_rng(7).standard_normal(want_feat.shape).astype(np.float32)
    want = oracle.feature_aggregate_bwd(*args, cg, want_mask)
    got = chop.feature_aggregate_grad(*ins, dev(cg), mask)
    _turns(3)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)


@pytest.mark.parametrize("op", ["cost_volume", "cost_volume_f16", "cost_aggregate", "cost_aggregate_min",
                                "feature_aggregate"])
def test_both_32_channel_gradient_kernels(oracle, op):
    """The 32-channel gradients exist slimmed (four waves per SIMD, 6 x 8 scatter window) and
    wide (three waves, 8 x 8): both against the oracle, on a sweep long enough for the window
    to move (and for cells to leave the smaller one), and the launcher's own choice by the
    number of source views."""
    lib = _lib.load()
    B, H, W, C, D = 1, 24, 36, 32, 40
    rng = np.random.default_rng(41)
    for N, want_auto in ((2, 6), (5, 8)):
        t = reference_test_case(2, B, N, H, W, C, D, np.float32, seed=70 + N)
        args = tuple(t[k] for k in ("ref", "src", "base_plane", "offsets", "Rs", "Ts"))
        if op.startswith("cost_volume"):
            half = op.endswith("f16")
            if half:
                q = lambda x: x.astype(np.float16).astype(np.float32)
                args = (q(args[0]), q(args[1])) + args[2:]
            _, mask = oracle.cost_volume_fwd(*args, "MEAN")
            cg = rng.normal(size=(B, H, W, D, C)).astype(np.float32)
            if half:
                cg = cg.astype(np.float16).astype(np.float32)
            want = oracle.cost_volume_bwd(*args, cg, mask, "MEAN")
            dt = torch.float16 if half else None
            ins = [dev(args[0], dt), dev(args[1], dt)] + [dev(x) for x in args[2:]]
            run = lambda: chop.cost_volume_grad(*ins, dev(cg, dt), dev(mask), "MEAN")
            rtol = 1e-2 if half else 1e-4
        elif op.startswith("cost_aggregate"):
            reduce = "MIN" if op.endswith("min") else "MEAN"
            _, mask = oracle.cost_aggregate_fwd(*args, reduce)
            cg = rng.normal(size=(B, H, W, D)).astype(np.float32)
            want = oracle.cost_aggregate_bwd(*args, cg, mask, reduce)
            ins = [dev(x) for x in args]
            run = lambda: chop.cost_aggregate_grad(*ins, dev(cg), dev(mask), reduce)
            rtol = 1e-4
        else:
            fargs = args[1:]
            _, mask = oracle.feature_aggregate_fwd(*fargs)
            cg = rng.normal(size=(B, H, W, D, N, C)).astype(np.float32)
            want = oracle.feature_aggregate_bwd(*fargs, cg, mask)
            ins = [dev(x) for x in fargs]
            run = lambda: chop.feature_aggregate_grad(*ins, dev(cg), dev(mask))
            rtol = 1e-4
        for rows in (6, 8, 0):
            print("\n[case] %s N=%d window %d" % (op, N, rows), flush=True)
            lib.chop_set_backward_window(rows)
            try:
                got = run()
                assert lib.chop_last_kernel_family() == 2
                assert lib.chop_last_backward_window() == (rows if rows else want_auto)
            finally:
                lib.chop_set_backward_window(0)
            for g, w in zip(got, want):
                assert_backward_close(host(g), w, rtol=rtol)
