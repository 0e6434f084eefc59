"""GPU parity of the CostVolumeV3 and FeatureAggregate entry points against the CPU oracle.

Bars: masks (view counts, winning view / group indices, 0/1 sample masks) bit-exact; the
forward values of these kernels follow the oracle's operation order, so they are compared
bit for bit as well; gradients within 1e-4 (the atomics land in another order).
The shapes are the reference tests' parameter sets (cost_volume_v3_op_test.py:178-191,
feature_aggregate_op_test.py:163-172) plus wider channel counts.
"""
import numpy as np
import pytest
import torch

import custom_helper_op_amd as chop
from custom_helper_op_amd import _lib
from custom_helper_op_amd.configs import make_workload, reference_test_case
from gpu_util import assert_backward_close, dev, host

pytestmark = pytest.mark.gpu

KEYS = ("ref", "src", "base_plane", "offsets", "Rs", "Ts")
FKEYS = ("src", "base_plane", "offsets", "Rs", "Ts")
# (B, N, H, W, C, D, groups)
V3_SHAPES = [(1, 1, 12, 16, 9, 5, 3), (1, 2, 12, 16, 9, 9, 3), (2, 2, 12, 18, 9, 10, 3),
             (2, 3, 12, 16, 9, 6, 3), (1, 2, 20, 24, 32, 7, 4), (1, 3, 9, 11, 8, 4, 1),
             (1, 2, 10, 12, 6, 5, 6)]
F_SHAPES = [(1, 1, 12, 16, 3, 5), (2, 2, 12, 18, 9, 10), (2, 3, 12, 16, 4, 6), (1, 2, 20, 24, 32, 19),
            (1, 2, 9, 11, 6, 4)]


@pytest.fixture(autouse=True)
def _announce(request):
    print("\n[case] %s" % request.node.nodeid, flush=True)
    yield


def _inputs(t, keys=KEYS):
    return [dev(t[k]) for k in keys]


def _args(t, keys=KEYS):
    return tuple(t[k] for k in keys)


# ---- CostVolumeV3 -------------------------------------------------------------------------
@pytest.mark.parametrize("shape", V3_SHAPES)
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_v3_forward(oracle, shape, reduce, dtype):
    B, N, H, W, C, D, G = shape
    for case in range(4):
        t = reference_test_case(case, B, N, H, W, C, D, dtype, seed=case)
        if case == 3:   # signed features: some views' maxima stay at the seed
            t["ref"] = t["ref"] - 5
            t["src"] = t["src"] - 5
        want_cost, want_mask = oracle.cost_volume_v3_fwd(*_args(t), reduce, G)
        cost, mask = chop.cost_volume_v3_raw(*_inputs(t), reduce, G)
        assert cost.shape == (B, H, W, D, 1)
        assert mask.shape == (B, H, W, D, 1 if reduce == "MEAN" else 3)
        assert np.array_equal(host(mask), want_mask)
        assert np.array_equal(host(cost), want_cost)


@pytest.mark.parametrize("half", [True, False])
def test_v3_forward_negative_correlations(oracle, half):
    # every correlation negative: MIN records nothing, MEAN returns the seed
    rng = np.random.default_rng(3)
    t = reference_test_case(1, 1, 2, 10, 12, 6, 5, np.float32, seed=5)
    t["src"] = -np.abs(t["src"]) - 0.1
    for reduce in ("MEAN", "MIN"):
        want_cost, want_mask = oracle.cost_volume_v3_fwd(*_args(t), reduce, 3, half)
        cost, mask = chop.cost_volume_v3_raw(*_inputs(t), reduce, 3, half)
        assert np.array_equal(host(mask), want_mask)
        assert np.array_equal(host(cost), want_cost)
        cg = dev(rng.normal(size=want_cost.shape).astype(np.float32))
        got = chop.cost_volume_grad_v3(*_inputs(t), cg, mask, reduce, 3, half)
        assert all(not host(g).any() for g in got)   # nothing exceeded the seed: no gradient


@pytest.mark.parametrize("shape", V3_SHAPES)
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_v3_backward(oracle, shape, reduce, dtype):
    B, N, H, W, C, D, G = shape
    rng = np.random.default_rng(29)
    for case in (1, 3):
        t = reference_test_case(case, B, N, H, W, C, D, dtype, seed=10 + case)
        _, mask = oracle.cost_volume_v3_fwd(*_args(t), reduce, G)
        cg = rng.normal(size=(B, H, W, D, 1)).astype(dtype)
        want = oracle.cost_volume_v3_bwd(*_args(t), cg, mask, reduce, G)
        lib = _lib.load()
        # the one-thread-per-voxel kernel, then the strip kernel (lane per channel: any group
        # width, float and double), which is also what an unforced call picks for these shapes
        # unless the tiled kernels take them
        for family, ran in ((1, (1,)), (2, (3,)), (0, (2, 3))):
            lib.chop_set_kernel_family(family)
            try:
                got = chop.cost_volume_grad_v3(*_inputs(t), dev(cg), dev(mask), reduce, G)
                assert lib.chop_last_kernel_family() in ran
            finally:
                lib.chop_set_kernel_family(0)
            for g, w in zip(got, want):
                assert g.shape == w.shape
                assert_backward_close(host(g), w, rtol=1e-4 if dtype == np.float32 else 1e-10)


@pytest.mark.parametrize("C,G", [(8, 1), (8, 2), (16, 2), (16, 4), (32, 4), (32, 8), (64, 8),
                                 (64, 16)])
@pytest.mark.parametrize("N", [1, 3])
def test_v3_tiled_widths(oracle, C, G, N):
    """Groups of 4 and 8 channels (one lane or two per group) at 2, 4, 8 and 16 lanes per
    pixel run the tiled kernels in float32.  Forward: cost and all indices bit for bit, like
    the one-thread-per-voxel kernel.  Gradient: within the backward bar, including the best
    pair it finds again for MEAN."""
    B, H, W, D = 2, 20, 24, 21
    lib = _lib.load()
    rng = np.random.default_rng(C + G + N)
    for case in (1, 3):
        t = reference_test_case(case, B, N, H, W, C, D, np.float32, seed=200 + case)
        for reduce in ("MEAN", "MIN"):
            want_cost, mask = oracle.cost_volume_v3_fwd(*_args(t), reduce, G)
            for family in (1, 0):
                lib.chop_set_kernel_family(family)
                cost, got_mask = chop.cost_volume_v3_raw(*_inputs(t), reduce, G)
                assert lib.chop_last_kernel_family() == (2 if family == 0 else 1)
                assert np.array_equal(host(got_mask), mask)
                assert np.array_equal(host(cost), want_cost)
            if reduce == "MIN":
                # recorded groups outside the image's groups: such voxels are skipped
                mask = mask.copy()
                flat = mask.reshape(-1, 3)
                hit = np.flatnonzero(flat[:, 0] >= 0)
                flat[hit[::7], 1] = G
                flat[hit[3::11], 2] = -1
            cg = rng.normal(size=(B, H, W, D, 1)).astype(np.float32)
            want = oracle.cost_volume_v3_bwd(*_args(t), cg, mask, reduce, G)
            for family in (1, 0):
                lib.chop_set_kernel_family(family)
                got = chop.cost_volume_grad_v3(*_inputs(t), dev(cg), dev(mask), reduce, G)
                assert lib.chop_last_kernel_family() == (2 if family == 0 else 1)
                for g, w in zip(got, want):
                    assert_backward_close(host(g), w)
    lib.chop_set_kernel_family(0)


@pytest.mark.parametrize("C,G", [(16, 4), (32, 4), (64, 8)])
def test_v3_tiled_ties(oracle, C, G):
    """Equal correlations: the first pair in (source group, reference group) order wins, in
    the lanes' tournament as in the reference's loop.  Constant images make every pair tie;
    reference groups 1 and 2 doubled make those two tie ahead of the rest."""
    B, N, H, W, D = 1, 2, 12, 16, 9
    lib = _lib.load()
    t = reference_test_case(1, B, N, H, W, C, D, np.float32, seed=5)
    t["src"] = np.ones_like(t["src"])
    rng = np.random.default_rng(3)
    for variant in (0, 1):
        ref = np.ones_like(t["ref"])
        if variant == 1:
            sub = C // G
            ref[..., sub:3 * sub] = 2.0
        t["ref"] = ref
        _, mask = oracle.cost_volume_v3_fwd(*_args(t), "MEAN", G)
        want_cost, want_win = oracle.cost_volume_v3_fwd(*_args(t), "MIN", G)
        lib.chop_set_kernel_family(0)
        cost, win = chop.cost_volume_v3_raw(*_inputs(t), "MIN", G)
        assert lib.chop_last_kernel_family() == 2
        assert np.array_equal(host(win), want_win) and np.array_equal(host(cost), want_cost)
        seen = want_win.reshape(-1, 3)
        seen = seen[seen[:, 0] >= 0]
        assert len(seen) and (seen[:, 0] == 0).all() and (seen[:, 2] == 0).all()
        assert (seen[:, 1] == (0 if variant == 0 else 1)).all()
        cg = rng.normal(size=(B, H, W, D, 1)).astype(np.float32)
        want = oracle.cost_volume_v3_bwd(*_args(t), cg, mask, "MEAN", G)
        # the whole reference gradient sits in the winning group
        sub = C // G
        first = slice(0, sub) if variant == 0 else slice(sub, 2 * sub)
        outside = np.delete(want[0], np.r_[first], axis=-1)
        assert np.abs(want[0][..., first]).max() > 0 and not outside.any()
        for family, ran in ((0, 2), (2, 3)):   # tiled, then the strip kernel's search
            lib.chop_set_kernel_family(family)
            try:
                got = chop.cost_volume_grad_v3(*_inputs(t), dev(cg), dev(mask), "MEAN", G)
                assert lib.chop_last_kernel_family() == ran
            finally:
                lib.chop_set_kernel_family(0)
            assert_backward_close(host(got[0]), want[0])
            assert_backward_close(host(got[1]), want[1])
            # constant images: the depth gradient is exactly zero in the reference's form
            # (differences of equal taps); the tiled kernel sums four weights that cancel
            assert not want[2].any() and np.abs(host(got[2])).max() < 1e-6


def test_v3_backward_full_size(oracle):
    """CostVolumeV3's gradient on the benchmark workload's tensors, both reduces."""
    t = make_workload(2, with_cost_grad=False).tensors
    ins = _inputs(t)
    rng = np.random.default_rng(11)
    cg = rng.normal(size=(1, 128, 160, 192, 1)).astype(np.float32)
    for reduce in ("MEAN", "MIN"):
        _, mask = chop.cost_volume_v3_raw(*ins, reduce, 4)
        got = chop.cost_volume_grad_v3(*ins, dev(cg), mask, reduce, 4)
        assert _lib.load().chop_last_kernel_family() == 2
        want = oracle.cost_volume_v3_bwd(*_args(t), cg, host(mask), reduce, 4)
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)
        # the strip kernel (what float64 and other group widths run) on the same tensors
        lib = _lib.load()
        lib.chop_set_kernel_family(2)
        try:
            got = chop.cost_volume_grad_v3(*ins, dev(cg), mask, reduce, 4)
            assert lib.chop_last_kernel_family() == 3
        finally:
            lib.chop_set_kernel_family(0)
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)


def test_v3_autograd_and_errors(oracle):
    t = reference_test_case(3, 2, 2, 8, 10, 6, 4, np.float64, seed=2)
    ins = _inputs(t)
    for k in range(3):
        ins[k].requires_grad_(True)
    cost, mask = chop.cost_volume_v3(*ins, reduce_method="MEAN", groups=3)
    assert not mask.requires_grad
    w = torch.linspace(0.5, 1.5, cost.numel(), dtype=cost.dtype, device=cost.device).reshape(cost.shape)
    (cost * w).sum().backward()
    want = oracle.cost_volume_v3_bwd(*_args(t), host(w), host(mask), "MEAN", 3)
    for k in range(3):
        assert_backward_close(host(ins[k].grad), want[k], rtol=1e-10)
    with pytest.raises(chop.InvalidArgumentError):
        chop.cost_volume_v3_raw(*_inputs(t), "MEAN", 4)          # groups does not divide C
    t18 = reference_test_case(1, 1, 1, 4, 4, 18, 2, np.float32, seed=1)
    with pytest.raises(chop.InvalidArgumentError):
        chop.cost_volume_v3_raw(*_inputs(t18), "MEAN", 2)        # 9 channels per group
    with pytest.raises(chop.InvalidArgumentError):
        chop.cost_volume_v3_raw(*_inputs(t), "MAX", 3)
    # the C ABI reports the same conditions by status
    lib = _lib.load()
    ins = _inputs(t18)
    cost = torch.empty(1, 4, 4, 2, 1, device="cuda")
    mask = torch.empty(1, 4, 4, 2, 1, dtype=torch.int32, device="cuda")
    rc = lib.chop_cost_volume_v3_fwd_f32(None, 0, 1, 1, 4, 4, 18, 2, 1, 4, 4, 2,
                                         *[x.data_ptr() for x in ins], cost.data_ptr(), mask.data_ptr())
    assert rc == 4 and b"8 channels" in lib.chop_last_error_string()
    rc = lib.chop_cost_volume_v3_fwd_f32(None, 0, 1, 0, 4, 4, 16, 2, 1, 4, 4, 2, *([None] * 8))
    assert rc == 0                                              # empty batch: nothing to do


# ---- FeatureAggregate ---------------------------------------------------------------------
@pytest.mark.parametrize("shape", F_SHAPES)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("half", [True, False])
def test_feature_forward(oracle, shape, dtype, half):
    B, N, H, W, C, D = shape
    for case in range(4):
        t = reference_test_case(case, B, N, H, W, C, D, dtype, seed=case)
        want, want_mask = oracle.feature_aggregate_fwd(*_args(t, FKEYS), half)
        mapped, mask = chop.feature_aggregate_raw(*_inputs(t, FKEYS), half)
        assert mapped.shape == (B, H, W, D, N, C) and mask.shape == (B, H, W, D, N, 1)
        assert np.array_equal(host(mask), want_mask)
        assert np.array_equal(host(mapped), want)


def test_feature_forward_other_source_size(oracle):
    rng = np.random.default_rng(4)
    B, N, sH, sW, C, H, W, D = 2, 2, 9, 14, 8, 5, 6, 4
    t = dict(src=rng.normal(size=(B, N, sH, sW, C)).astype(np.float32),
             base_plane=rng.uniform(2, 3, (B, H, W, 1)).astype(np.float32),
             offsets=rng.uniform(-0.2, 0.2, (B, D)).astype(np.float32),
             Rs=np.tile(np.eye(3, dtype=np.float32)[None, None], (B, N, 1, 1)),
             Ts=rng.uniform(0.5, 6.0, (B, N, 3)).astype(np.float32))
    want, want_mask = oracle.feature_aggregate_fwd(*_args(t, FKEYS))
    mapped, mask = chop.feature_aggregate_raw(*_inputs(t, FKEYS))
    assert want_mask.any() and not want_mask.all()
    assert np.array_equal(host(mask), want_mask)
    assert np.array_equal(host(mapped), want)
    g = rng.normal(size=want.shape).astype(np.float32)
    want_g = oracle.feature_aggregate_bwd(*_args(t, FKEYS), g, want_mask)
    got_g = chop.feature_aggregate_grad(*_inputs(t, FKEYS), dev(g), mask)
    for a, b in zip(got_g, want_g):
        assert_backward_close(host(a), b)


@pytest.mark.parametrize("shape", F_SHAPES)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_feature_backward(oracle, shape, dtype):
    B, N, H, W, C, D = shape
    rng = np.random.default_rng(31)
    for case in (1, 3):
        t = reference_test_case(case, B, N, H, W, C, D, dtype, seed=20 + case)
        _, mask = oracle.feature_aggregate_fwd(*_args(t, FKEYS))
        g = rng.normal(size=(B, H, W, D, N, C)).astype(dtype)
        want = oracle.feature_aggregate_bwd(*_args(t, FKEYS), g, mask)
        got = chop.feature_aggregate_grad(*_inputs(t, FKEYS), dev(g), dev(mask))
        for a, b in zip(got, want):
            assert a.shape == b.shape
            assert_backward_close(host(a), b, rtol=1e-4 if dtype == np.float32 else 1e-10)


@pytest.mark.parametrize("C", [4, 8, 16, 32, 64])
@pytest.mark.parametrize("N", [1, 3])
@pytest.mark.parametrize("family", [pytest.param(1, id="general"), pytest.param(2, id="strip"),
                                    pytest.param(0, id="auto")])
def test_feature_tiled_channel_widths(oracle, C, N, family):
    """Every lanes-per-pixel variant of the tiled kernels (C = 4 x a power of two, float32),
    on an image whose pixel count is no multiple of the tile; the general and the strip kernels
    on the same inputs for comparison.  Forward values are bit-identical in all families."""
    lib = _lib.load()
    lib.chop_set_kernel_family(family)
    try:
        B, H, W, D = 2, 20, 23, 21
        t = reference_test_case(3, B, N, H, W, C, D, np.float32, seed=C + N)
        want, want_mask = oracle.feature_aggregate_fwd(*_args(t, FKEYS))
        mapped, mask = chop.feature_aggregate_raw(*_inputs(t, FKEYS))
        assert lib.chop_last_kernel_family() == {1: 1, 2: 3, 0: 2}[family]
        assert np.array_equal(host(mask), want_mask)
        assert np.array_equal(host(mapped), want)
        g = np.random.default_rng(C).normal(size=want.shape).astype(np.float32)
        want_g = oracle.feature_aggregate_bwd(*_args(t, FKEYS), g, want_mask)
        got_g = chop.feature_aggregate_grad(*_inputs(t, FKEYS), dev(g), mask)
        assert lib.chop_last_kernel_family() == {1: 1, 2: 3, 0: 2}[family]
        for a, b in zip(got_g, want_g):
            assert_backward_close(host(a), b)
    finally:
        lib.chop_set_kernel_family(0)


def test_feature_autograd_and_errors(oracle):
    t = reference_test_case(3, 1, 2, 8, 10, 4, 5, np.float64, seed=6)
    ins = _inputs(t, FKEYS)
    ins[0].requires_grad_(True)
    ins[1].requires_grad_(True)
    mapped, mask = chop.feature_aggregate(*ins)
    assert not mask.requires_grad
    w = torch.linspace(-1, 1, mapped.numel(), dtype=mapped.dtype, device=mapped.device).reshape(mapped.shape)
    (mapped * w).sum().backward()
    want = oracle.feature_aggregate_bwd(*_args(t, FKEYS), host(w), host(mask))
    assert_backward_close(host(ins[0].grad), want[0], rtol=1e-10)
    assert_backward_close(host(ins[1].grad), want[1], rtol=1e-10)
    bad = _inputs(t, FKEYS)
    with pytest.raises(chop.InvalidArgumentError):
        chop.feature_aggregate_raw(bad[0][0], *bad[1:])            # src_images rank 4
    with pytest.raises(chop.InvalidArgumentError):
        chop.feature_aggregate_raw(bad[0], bad[1], bad[2], bad[3][:, :1], bad[4])
    lib = _lib.load()
    rc = lib.chop_feature_aggregate_fwd_f32(None, 1, 1, 2, 2, 2, 2, 1, 2, 2, *([None] * 7))
    assert rc == 1 and b"null pointer" in lib.chop_last_error_string()
    rc = lib.chop_feature_aggregate_fwd_f32(None, 1, 1, 2, 2, 2, 0, 1, 2, 2, *([None] * 7))
    assert rc == 0                                                   # no depth hypotheses


def test_full_size_benchmark_tensors(oracle):
    """The benchmark workload's tensors (B1 N2 128x160 C32 D192) in full: CostVolumeV3 with
    4 groups (both reduces) and FeatureAggregate, against the multi-threaded oracle."""
    t = make_workload(2, with_cost_grad=False).tensors
    ins = _inputs(t)
    for reduce in ("MEAN", "MIN"):
        cost, mask = chop.cost_volume_v3_raw(*ins, reduce, 4)
        assert _lib.load().chop_last_kernel_family() == 2
        want_cost, want_mask = oracle.cost_volume_v3_fwd(*_args(t), reduce, 4, threads=16)
        assert np.array_equal(host(mask), want_mask)
        assert np.array_equal(host(cost), want_cost)
        del cost, mask
    fin = [ins[k] for k in (1, 2, 3, 4, 5)]
    mapped, fmask = chop.feature_aggregate_raw(*fin)
    assert _lib.load().chop_last_kernel_family() == 2
    want, want_mask = oracle.feature_aggregate_fwd(*_args(t, FKEYS), threads=16)
    assert np.array_equal(host(fmask), want_mask)
    assert np.array_equal(host(mapped), want)
    del mapped, want
    # gradient at full size: linearity in the upstream gradient and the known total
    # (every accepted sample's four weights sum to 1, so sum(src_grad) = sum of the
    # upstream gradient over accepted samples)
    g = torch.randn(1, 128, 160, 192, 2, 32, device="cuda")
    sg, bg = chop.feature_aggregate_grad(*fin, g, fmask)
    assert _lib.load().chop_last_kernel_family() == 2
    total = (g.double() * fmask.double()).sum().item()
    assert abs(sg.double().sum().item() - total) < 1e-6 * g.double().abs().sum().item()
    sg2, bg2 = chop.feature_aggregate_grad(*fin, 2 * g, fmask)
    assert_backward_close(host(sg2), 2 * host(sg))
    assert_backward_close(host(bg2), 2 * host(bg))
    want_sg, want_bg = oracle.feature_aggregate_bwd(*_args(t, FKEYS), host(g), want_mask)
    assert_backward_close(host(sg), want_sg)
    assert_backward_close(host(bg), want_bg)
