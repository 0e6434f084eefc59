"""GPU checks of the callers around the ops: the layers' default fill (bit-exact: it only
selects), its gradient, ``combine_projection`` and the two cost-map layers end to end."""
import numpy as np
import pytest
import torch

import custom_helper_op_amd as chop
from custom_helper_op_amd import _lib
from custom_helper_op_amd.configs import reference_test_case
from gpu_util import assert_backward_close, dev, host
from test_oracle_callers import random_cam

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _announce(request):
    print("\n[case] %s" % request.node.nodeid, flush=True)
    yield


@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_default_fill(oracle, reduce, dtype):
    rng = np.random.default_rng(3)
    for shape, mshape in (((2, 5, 7, 9), (2, 5, 7, 9)), ((2, 5, 7, 9, 4), (2, 5, 7, 9, 1)),
                          ((1, 33, 65, 17, 4), (1, 33, 65, 17, 4))):
        cost = rng.normal(size=shape).astype(dtype)
        mask = rng.integers(-1, 3, mshape).astype(np.int32)
        default = torch.tensor(0.375, dtype=getattr(torch, np.dtype(dtype).name), device="cuda",
                               requires_grad=True)
        c = dev(cost).requires_grad_(True)
        out = chop.cost_default_fill(c, dev(mask), default, reduce)
        assert np.array_equal(host(out), oracle.cost_default_fill(cost, mask, 0.375, reduce))
        g = rng.normal(size=shape).astype(dtype)
        out.backward(dev(g))
        want_cg, want_dg = oracle.cost_default_fill_grad(g, mask, reduce)
        assert np.array_equal(host(c.grad), want_cg)
        tol = 1e-4 if dtype == np.float32 else 1e-11
        assert abs(float(default.grad) - want_dg) <= tol * max(1.0, np.abs(g).sum() ** 0.5)
        # a second call starts the scalar's gradient from zero again
        default.grad = None
        chop.cost_default_fill(c, dev(mask), default, reduce).backward(dev(g))
        assert abs(float(default.grad) - want_dg) <= tol * max(1.0, np.abs(g).sum() ** 0.5)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_combine_projection(oracle, dtype):
    rng = np.random.default_rng(11)
    B, N = 3, 4
    ref = np.stack([random_cam(rng) for _ in range(B)])
    src = np.stack([np.stack([random_cam(rng) for _ in range(N)]) for _ in range(B)])
    scale = np.array([0.25, 0.5, 1.0])
    Rs, Ts = chop.combine_projection(dev(ref.astype(dtype)), dev(src.astype(dtype)),
                                     dev(scale.astype(dtype)))
    assert Rs.shape == (B, N, 3, 3) and Ts.shape == (B, N, 3)
    tol = 2e-5 if dtype == np.float32 else 1e-12
    for b in range(B):
        for n in range(N):
            R, T = oracle.combine_projection(ref[b].copy(), src[b, n].copy(), scale)
            np.testing.assert_allclose(host(Rs)[b, n], R, rtol=tol, atol=tol * np.abs(R).max())
            np.testing.assert_allclose(host(Ts)[b, n], T[:, 0], rtol=tol, atol=tol * np.abs(T).max())
    # the unbatched form of the reference helper
    R1, T1 = chop.combine_projection(dev(ref[0].astype(dtype)), dev(src[0, 0].astype(dtype)),
                                     dev(scale.astype(dtype)))
    assert R1.shape == (3, 3) and T1.shape == (3, 1)
    assert np.array_equal(host(R1), host(Rs)[0, 0]) and np.array_equal(host(T1)[:, 0], host(Ts)[0, 0])
    with pytest.raises(chop.InvalidArgumentError):
        chop.combine_projection(dev(ref.astype(dtype)), dev(src[:2].astype(dtype)), dev(scale.astype(dtype)))
    lib = _lib.load()
    assert lib.chop_combine_projection_f32(None, 1, 1, None, None, None, None, None) == 1
    assert lib.chop_combine_projection_f32(None, 0, 4, None, None, None, None, None) == 0
    assert lib.chop_cost_default_fill_f32(None, 5, 1, 1, None, None, None, None) == 3
    assert lib.chop_cost_default_fill_f32(None, 0, 4, 0, None, None, None, None) == 2


@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_cost_map_layers(oracle, reduce):
    t = reference_test_case(3, 2, 2, 10, 12, 8, 6, np.float32, seed=4)
    t["Ts"][:, 1, 2] = -40.0                           # the second view sees nothing
    t["Ts"][0, 0, 0] = 400.0                           # and the first one nothing of batch item 0
    keys = ("ref", "src", "base_plane", "offsets", "Rs", "Ts")
    layer = chop.CostMapLayer(reduce_method=reduce, default_type="DYNAMIC").cuda()
    with torch.no_grad():
        layer.default_cost.fill_(0.25)
    ins = [dev(t[k]) for k in keys]
    ins[0].requires_grad_(True)
    cost, mask = layer(ins)
    want_cost, want_mask = oracle.cost_aggregate_fwd(*[t[k] for k in keys], reduce)
    assert np.array_equal(host(mask), want_mask)
    want = oracle.cost_default_fill(want_cost, want_mask, np.float32(0.25), reduce)
    np.testing.assert_allclose(host(cost), want, rtol=1e-5, atol=1e-6)
    empty = (want_mask <= 0) if reduce == "MEAN" else (want_mask < 0)
    assert empty.any() and not empty.all()
    cost.sum().backward()
    assert float(layer.default_cost.grad) == pytest.approx(float(empty.sum()), rel=1e-6)
    assert ins[0].grad is not None and np.isfinite(host(ins[0].grad)).all()
    frozen = chop.CostMapLayer(reduce_method=reduce, default_type="CONSTANT")
    assert not frozen.default_cost.requires_grad

    depth_grid = (t["base_plane"] + t["offsets"][:, None, None, :]).astype(np.float32)
    layer2 = chop.CostMapLayerV2(reduce_method=reduce, groups=4, default_type=torch.tensor(1.5)).cuda()
    ins2 = [dev(t["ref"]), dev(t["src"]), dev(depth_grid), dev(t["Rs"]), dev(t["Ts"])]
    cost2, mask2 = layer2(ins2)
    want_cost2, want_mask2 = oracle.cost_volume_v2_fwd(t["ref"], t["src"], depth_grid, t["Rs"], t["Ts"],
                                                       reduce, 4)
    assert np.array_equal(host(mask2), want_mask2)
    want2 = oracle.cost_default_fill(want_cost2, want_mask2, np.float32(1.5), reduce)
    np.testing.assert_allclose(host(cost2), want2, rtol=1e-5, atol=1e-5)


FAMILIES = [pytest.param(1, id="general"), pytest.param(2, id="strip"), pytest.param(0, id="auto")]


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_fill_folded_into_the_forward(oracle, family, reduce, dtype):
    """The ops with a default_cost write, in one kernel, exactly what the plain op followed by
    the layers' `where` gives: the op's own output with the default selected in, bit for bit
    (every kernel family; CostAggregate and CostVolumeV2, which the two layers run)."""
    lib = _lib.load()
    lib.chop_set_kernel_family(family)
    try:
        t = reference_test_case(3, 2, 2, 20, 24, 8, 9, dtype, seed=6)
        t["Ts"][:, 1, 2] = -40.0                       # the second view sees nothing
        t["Ts"][0, 0, 0] = 400.0                       # and the first one nothing of batch item 0
        keys = ("ref", "src", "base_plane", "offsets", "Rs", "Ts")
        td = getattr(torch, np.dtype(dtype).name)
        default = torch.tensor(-0.625, dtype=td, device="cuda")
        ins = [dev(t[k]) for k in keys]
        plain, mask = chop.cost_aggregate_raw(*ins, reduce)
        fam_plain = lib.chop_last_kernel_family()
        filled, mask_f = chop.cost_aggregate_raw(*ins, reduce, default_cost=default)
        assert lib.chop_last_kernel_family() == fam_plain
        assert np.array_equal(host(mask_f), host(mask))
        want = oracle.cost_default_fill(host(plain), host(mask), dtype(-0.625), reduce)
        assert np.array_equal(host(filled), want)
        empty = (host(mask) <= 0) if reduce == "MEAN" else (host(mask) < 0)
        assert empty.any() and not empty.all()

        grid = (t["base_plane"] + t["offsets"][:, None, None, :]).astype(dtype)
        ins2 = [dev(t["ref"]), dev(t["src"]), dev(grid), dev(t["Rs"]), dev(t["Ts"])]
        for groups in (4, 8, 1):
            plain, mask = chop.cost_volume_v2_raw(*ins2, reduce, groups)
            fam_plain = lib.chop_last_kernel_family()
            filled, mask_f = chop.cost_volume_v2_raw(*ins2, reduce, groups, default_cost=default)
            assert lib.chop_last_kernel_family() == fam_plain
            assert np.array_equal(host(mask_f), host(mask))
            want = oracle.cost_default_fill(host(plain), host(mask), dtype(-0.625), reduce)
            assert np.array_equal(host(filled), want), groups
    finally:
        lib.chop_set_kernel_family(0)


@pytest.mark.parametrize("storage", [torch.float16, torch.bfloat16])
def test_cost_map_layer_v2_16bit(oracle, storage):
    """CostMapLayerV2 on 16-bit features (the op beneath it supports them): forward against the
    float32 oracle on the quantised inputs, and the scalar's gradient."""
    from custom_helper_op_amd.configs import quantise
    name = "f16" if storage == torch.float16 else "bf16"
    t = reference_test_case(3, 1, 2, 16, 24, 8, 6, np.float32, seed=9)
    t["Ts"][:, 1, 2] = -40.0
    ref, src = quantise(t["ref"] * 0.1, name), quantise(t["src"] * 0.1, name)
    grid = (t["base_plane"] + t["offsets"][:, None, None, :]).astype(np.float32)
    layer = chop.CostMapLayerV2(reduce_method="MEAN", groups=4, default_type="DYNAMIC").cuda()
    with torch.no_grad():
        layer.default_cost.fill_(0.5)
    cost, mask = layer([dev(ref, storage), dev(src, storage), dev(grid), dev(t["Rs"]), dev(t["Ts"])])
    assert cost.dtype == storage
    want_cost, want_mask = oracle.cost_volume_v2_fwd(ref, src, grid, t["Rs"], t["Ts"], "MEAN", 4)
    assert np.array_equal(host(mask), want_mask)
    want = oracle.cost_default_fill(want_cost, want_mask, np.float32(0.5), "MEAN")
    np.testing.assert_allclose(host(cost), want, rtol=1e-2, atol=1e-2)
    empty = want_mask <= 0
    assert empty.any() and not empty.all()
    cost.float().sum().backward()
    assert float(layer.default_cost.grad) == pytest.approx(float(empty.sum()) * 4, rel=1e-3)
