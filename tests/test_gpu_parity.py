"""GPU parity: the HIP library (through its C ABI) against the CPU oracle on identical
seeded inputs.  Bars: sample coordinates, truncated indices, acceptance and masks
bit-exact; fp32 forward values within 1e-5 relative; fp32 backward within 1e-4 relative;
16-bit storage within 1e-2."""
import numpy as np
import pytest
import torch

import custom_helper_op_amd as chop
from custom_helper_op_amd import _lib
from custom_helper_op_amd.configs import make_workload, quantise, reference_test_case
from gpu_util import (TORCH_DTYPE, assert_backward_close, assert_forward_close, dev, host, rms)

pytestmark = pytest.mark.gpu

FAMILIES = [pytest.param(1, id="general"), pytest.param(2, id="strip"), pytest.param(0, id="auto")]


@pytest.fixture(autouse=True)
def _announce(request):
    print("\n[case] %s" % request.node.nodeid, flush=True)
    yield
    _lib.load().chop_set_kernel_family(0)


def _assert_family(family, expect_tiled=True):
    """Which kernels served the last call: 1 general, 2 tiled, 3 strip.  Under the automatic
    selection the benchmark shapes must really run the tiled kernels; what those decline
    (float64, channel counts other than 4 x 2^k) goes to the strip kernels."""
    got = _lib.load().chop_last_kernel_family()
    want = {1: 1, 2: 3, 0: 2 if expect_tiled else 3}[family]
    assert got == want, (got, want)


def _v1_inputs(t, dtype=None):
    keys = ("ref", "src", "base_plane", "offsets", "Rs", "Ts")
    return [dev(t[k].astype(dtype) if dtype else t[k]) for k in keys]


# ---- coordinates ---------------------------------------------------------------------------
@pytest.mark.parametrize("index,hw", [(1, None), (5, (48, 64))])
@pytest.mark.parametrize("half", [True, False])
def test_sample_coordinates_bit_exact(oracle, index, hw, half):
    wl = make_workload(index, hw=hw, with_cost_grad=False, batch=1)
    t = wl.tensors
    want = oracle.sample_coords(t["base_plane"], t["offsets"], t["Rs"], t["Ts"], (wl.H, wl.W), half)
    got = chop.sample_coords(dev(t["base_plane"]), dev(t["offsets"]), dev(t["Rs"]), dev(t["Ts"]),
                             (wl.H, wl.W), half)
    names = ("sw", "sh", "fh", "fw", "state")
    for n, g, w in zip(names, got, want):
        g = host(g)
        assert g.dtype == w.dtype
        assert np.array_equal(g.view(np.int32), w.view(np.int32)), n  # bit patterns
    assert 0.02 < (want[4] == 2).mean() < 1.0


def test_sample_coordinates_bit_exact_f64_and_depth_grid(oracle):
    t = reference_test_case(3, 2, 3, 12, 16, 3, 6, np.float64, seed=8)
    want = oracle.sample_coords(t["base_plane"], t["offsets"], t["Rs"], t["Ts"], (12, 16))
    got = chop.sample_coords(dev(t["base_plane"]), dev(t["offsets"]), dev(t["Rs"]), dev(t["Ts"]),
                             (12, 16))
    for g, w in zip(got, want):
        assert np.array_equal(host(g), w)
    wl = make_workload(4, hw=(32, 40), with_cost_grad=False, batch=1)
    dg = wl.tensors["depth_grid"]
    want = oracle.sample_coords(None, None, wl.tensors["Rs"], wl.tensors["Ts"], (32, 40),
                                depth_grid=dg)
    got = chop.sample_coords(None, None, dev(wl.tensors["Rs"]), dev(wl.tensors["Ts"]), (32, 40),
                             depth_grid=dev(dg))
    for g, w in zip(got, want):
        assert np.array_equal(host(g).view(np.int32), w.view(np.int32))


# ---- V1 forward ----------------------------------------------------------------------------
REF_SHAPES = [(1, 1, 12, 16, 3, 5), (1, 2, 12, 16, 3, 9), (2, 2, 12, 18, 5, 10), (2, 3, 12, 16, 3, 6)]


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("shape", REF_SHAPES)
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_v1_forward_reference_shapes(oracle, family, shape, reduce, dtype):
    """The reference unit tests' shapes and four camera cases (cost_volume_op_test.py:174-263)."""
    _lib.load().chop_set_kernel_family(family)
    B, N, H, W, C, D = shape
    for case in range(4):
        t = reference_test_case(case, B, N, H, W, C, D, dtype, seed=case)
        want_cost, want_mask = oracle.cost_volume_fwd(**t, reduce=reduce)
        cost, mask = chop.cost_volume_raw(*_v1_inputs(t), reduce)
        _assert_family(family, expect_tiled=False)  # C = 3 or 5: never the tiled kernels
        assert np.array_equal(host(mask), want_mask)
        # general and strip kernels keep the literal operation order: same bits
        assert np.array_equal(host(cost), want_cost)


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("half", [True, False])
def test_v1_forward_tiny_config_full(oracle, family, half):
    """Benchmark configuration 1 at full size, forward only."""
    _lib.load().chop_set_kernel_family(family)
    wl = make_workload(1)
    t = wl.tensors
    want_cost, want_mask = oracle.cost_volume_fwd(t["ref"], t["src"], t["base_plane"], t["offsets"],
                                                  t["Rs"], t["Ts"], "MEAN", half, threads=8)
    cost, mask = chop.cost_volume_raw(*_v1_inputs(t), "MEAN", half)
    _assert_family(family)
    assert cost.shape == (1, 64, 80, 32, 8) and mask.shape == (1, 64, 80, 32, 1)
    assert np.array_equal(host(mask), want_mask)
    assert_forward_close(host(cost), want_cost)
    assert (want_mask == wl.N).mean() > 0.5


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("index,hw,depth", [(2, (32, 40), None), (5, (36, 48), 32)])
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_v1_forward_benchmark_shapes(oracle, family, index, hw, depth, reduce):
    _lib.load().chop_set_kernel_family(family)
    wl = make_workload(index, hw=hw, depth=depth, with_cost_grad=False, batch=min(2, _SPEC_B[index]))
    t = wl.tensors
    want_cost, want_mask = oracle.cost_volume_fwd(t["ref"], t["src"], t["base_plane"], t["offsets"],
                                                  t["Rs"], t["Ts"], reduce, threads=8)
    cost, mask = chop.cost_volume_raw(*_v1_inputs(t), reduce)
    _assert_family(family)
    assert np.array_equal(host(mask), want_mask)
    if reduce == "MIN":
        # both kernel families evaluate the MIN reduce in the literal operation order
        assert np.array_equal(host(cost), want_cost)
    else:
        assert_forward_close(host(cost), want_cost)


_SPEC_B = {1: 1, 2: 1, 3: 1, 4: 2, 5: 4}


# ---- V1 backward ---------------------------------------------------------------------------
@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("shape", REF_SHAPES)
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_v1_backward_reference_shapes(oracle, family, shape, reduce, dtype):
    _lib.load().chop_set_kernel_family(family)
    B, N, H, W, C, D = shape
    rng = np.random.default_rng(17)
    for case in (1, 3):
        t = reference_test_case(case, B, N, H, W, C, D, dtype, seed=case)
        _, mask = oracle.cost_volume_fwd(**t, reduce=reduce)
        cg = rng.standard_normal((B, H, W, D, C)).astype(dtype)
        want = oracle.cost_volume_bwd(**t, cost_grad=cg, mask=mask, reduce=reduce)
        got = chop.cost_volume_grad(*_v1_inputs(t), dev(cg), dev(mask), reduce)
        _assert_family(family, expect_tiled=False)
        tol = 1e-4 if dtype == np.float32 else 1e-10
        for g, w in zip(got, want):
            assert g.shape == w.shape
            assert_backward_close(host(g), w, tol)


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("index,hw,depth", [(2, (32, 40), None), (5, (36, 48), 32)])
def test_v1_backward_benchmark_shapes(oracle, family, index, hw, depth):
    _lib.load().chop_set_kernel_family(family)
    wl = make_workload(index, hw=hw, depth=depth, batch=min(2, _SPEC_B[index]))
    t = wl.tensors
    args = (t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
    _, mask = oracle.cost_volume_fwd(*args, threads=8)
    want = oracle.cost_volume_bwd(*args, t["cost_grad"], mask, threads=1)
    got = chop.cost_volume_grad(*_v1_inputs(t), dev(t["cost_grad"]), dev(mask))
    _assert_family(family)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)
    # conservation: ref_grad and src_grad cancel in sum (each g enters as -g and as four
    # taps whose weights sum to one)
    rg, sg = host(got[0]).astype(np.float64), host(got[1]).astype(np.float64)
    assert abs(rg.sum() + sg.sum()) < 1e-4 * np.abs(rg).sum()


# ---- V2 ------------------------------------------------------------------------------------
@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_v2_forward_backward_reference_shapes(oracle, family, reduce, dtype):
    """cost_volume_v2_op_test.py:174-263: C=9, groups=3, depth_grid = base + offsets."""
    _lib.load().chop_set_kernel_family(family)
    rng = np.random.default_rng(23)
    for (B, N, H, W, D) in [(1, 1, 12, 16, 5), (1, 2, 12, 16, 9), (2, 2, 12, 18, 10), (2, 3, 12, 16, 6)]:
        for case in (0, 1, 3):
            t = reference_test_case(case, B, N, H, W, 9, D, dtype, seed=case + 40)
            dg = (t["base_plane"] + t["offsets"][:, None, None, :]).astype(dtype)
            want_cost, want_mask = oracle.cost_volume_v2_fwd(t["ref"], t["src"], dg, t["Rs"],
                                                             t["Ts"], reduce, 3)
            ins = [dev(t["ref"]), dev(t["src"]), dev(dg), dev(t["Rs"]), dev(t["Ts"])]
            cost, mask = chop.cost_volume_v2_raw(*ins, reduce, 3)
            _assert_family(family, expect_tiled=False)  # C = 9
            assert np.array_equal(host(mask), want_mask)
            assert np.array_equal(host(cost), want_cost)
            cg = rng.standard_normal(want_cost.shape).astype(dtype)
            want = oracle.cost_volume_v2_bwd(t["ref"], t["src"], dg, t["Rs"], t["Ts"], cg,
                                             want_mask, reduce, 3)
            got = chop.cost_volume_grad_v2(*ins, dev(cg), dev(want_mask), reduce, 3)
            _assert_family(family, expect_tiled=False)
            tol = 1e-4 if dtype == np.float32 else 1e-10
            for g, w in zip(got, want):
                assert_backward_close(host(g), w, tol)


@pytest.mark.parametrize("family", FAMILIES)
def test_v2_groupwise_config_f32(oracle, family):
    """Benchmark configuration 4's shape family (C=8, groups=4, D=8 per-pixel hypotheses)
    in float32 at reduced resolution."""
    _lib.load().chop_set_kernel_family(family)
    wl = make_workload(4, hw=(64, 80), batch=2)
    t = wl.tensors
    want_cost, want_mask = oracle.cost_volume_v2_fwd(t["ref"], t["src"], t["depth_grid"], t["Rs"],
                                                     t["Ts"], "MEAN", 4, threads=8)
    ins = [dev(t[k]) for k in ("ref", "src", "depth_grid", "Rs", "Ts")]
    cost, mask = chop.cost_volume_v2_raw(*ins, "MEAN", 4)
    _assert_family(family)
    assert np.array_equal(host(mask), want_mask)
    assert_forward_close(host(cost), want_cost, atol=1e-5)
    want = oracle.cost_volume_v2_bwd(t["ref"], t["src"], t["depth_grid"], t["Rs"], t["Ts"],
                                     t["cost_grad"], want_mask, "MEAN", 4)
    got = chop.cost_volume_grad_v2(*ins, dev(t["cost_grad"]), dev(want_mask), "MEAN", 4)
    _assert_family(family)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)


# ---- 16-bit storage ------------------------------------------------------------------------
def _assert_16bit_close(got, want, storage):
    """1e-2 relative, floor 1e-2 * rms: the output itself is rounded to 8 (bf16) or 11
    (fp16) significant bits."""
    np.testing.assert_allclose(got, want, rtol=1e-2, atol=1e-2 * max(rms(want), 1e-30))


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("storage", ["f16", "bf16"])
def test_v1_16bit_storage(oracle, family, storage):
    """Benchmark configuration 3's shape family (C=16, N=4, D=32, smooth base plane):
    fp32 oracle on the quantised inputs, 1e-2."""
    _lib.load().chop_set_kernel_family(family)
    wl = make_workload(3, hw=(48, 64))
    t = wl.tensors
    ref, src, cg = (quantise(t[k], storage) for k in ("ref", "src", "cost_grad"))
    want_cost, want_mask = oracle.cost_volume_fwd(ref, src, t["base_plane"], t["offsets"], t["Rs"],
                                                  t["Ts"], threads=8)
    td = TORCH_DTYPE[storage]
    ins = [dev(ref, td), dev(src, td), dev(t["base_plane"]), dev(t["offsets"]), dev(t["Rs"]),
           dev(t["Ts"])]
    cost, mask = chop.cost_volume_raw(*ins)
    _assert_family(family)
    assert cost.dtype == td
    assert np.array_equal(host(mask), want_mask)
    _assert_16bit_close(host(cost), want_cost, storage)
    want = oracle.cost_volume_bwd(ref, src, t["base_plane"], t["offsets"], t["Rs"], t["Ts"], cg,
                                  want_mask)
    got = chop.cost_volume_grad(*ins, dev(cg, td), dev(want_mask))
    _assert_family(family)
    assert got[0].dtype == td and got[1].dtype == td and got[2].dtype == torch.float32
    for g, w in zip(got, want):
        _assert_16bit_close(host(g), w, storage)


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("storage", ["bf16", "f16"])
def test_v2_16bit_storage(oracle, family, storage):
    """Benchmark configuration 4 (bf16 group-wise correlation) at reduced resolution."""
    _lib.load().chop_set_kernel_family(family)
    wl = make_workload(4, hw=(64, 80), batch=2)
    t = wl.tensors
    ref, src, cg = (quantise(t[k], storage) for k in ("ref", "src", "cost_grad"))
    want_cost, want_mask = oracle.cost_volume_v2_fwd(ref, src, t["depth_grid"], t["Rs"], t["Ts"],
                                                     "MEAN", 4, threads=8)
    td = TORCH_DTYPE[storage]
    ins = [dev(ref, td), dev(src, td), dev(t["depth_grid"]), dev(t["Rs"]), dev(t["Ts"])]
    cost, mask = chop.cost_volume_v2_raw(*ins, "MEAN", 4)
    assert np.array_equal(host(mask), want_mask)
    _assert_16bit_close(host(cost), want_cost, storage)
    want = oracle.cost_volume_v2_bwd(ref, src, t["depth_grid"], t["Rs"], t["Ts"], cg, want_mask,
                                     "MEAN", 4)
    got = chop.cost_volume_grad_v2(*ins, dev(cg, td), dev(want_mask), "MEAN", 4)
    _assert_family(family)
    for g, w in zip(got, want):
        _assert_16bit_close(host(g), w, storage)


# ---- the registered gradient, end to end ------------------------------------------------------
def test_autograd_matches_grad_op(oracle):
    """forward -> keep cost_mask -> Grad op with the upstream gradient, the call pattern
    of the gradient registered in custom_helper_ops.py:41-61."""
    wl = make_workload(2, hw=(16, 20), depth=24)
    t = wl.tensors
    ins = _v1_inputs(t)
    for x in ins[:3]:
        x.requires_grad_(True)
    cost, mask = chop.cost_volume(*ins)
    assert not mask.requires_grad
    cg = dev(t["cost_grad"])
    (cost * cg).sum().backward()
    _, m = oracle.cost_volume_fwd(t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
    want = oracle.cost_volume_bwd(t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"],
                                  t["Ts"], t["cost_grad"], m)
    for x, w in zip(ins[:3], want):
        assert_backward_close(host(x.grad), w)
    assert ins[3].grad is None and ins[4].grad is None and ins[5].grad is None


@pytest.mark.parametrize("family", FAMILIES)
def test_backward_without_the_depth_gradient(oracle, family):
    """A NULL third gradient: ref_grad and src_grad are those of the full call, the depth
    gradient is neither written nor computed (V1 both reductions, V2 fp32 and bf16,
    CostAggregate, and through autograd when the planes do not require a gradient)."""
    _lib.load().chop_set_kernel_family(family)
    wl = make_workload(2, hw=(24, 40), depth=24)
    t = wl.tensors
    args = (t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
    for reduce in ("MEAN", "MIN"):
        _, mask = oracle.cost_volume_fwd(*args, reduce)
        cg = t["cost_grad"]
        want = oracle.cost_volume_bwd(*args, cg, mask, reduce)
        got = chop.cost_volume_grad(*_v1_inputs(t), dev(cg), dev(mask), reduce,
                                    need_depth_grad=False)
        _assert_family(family)
        assert got[2] is None
        assert_backward_close(host(got[0]), want[0])
        assert_backward_close(host(got[1]), want[1])
    _, amask = oracle.cost_aggregate_fwd(*args)
    acg = np.ascontiguousarray(t["cost_grad"][..., 0])
    want = oracle.cost_aggregate_bwd(*args, acg, amask)
    got = chop.cost_aggregate_grad(*_v1_inputs(t), dev(acg), dev(amask), need_depth_grad=False)
    _assert_family(family)
    assert got[2] is None
    assert_backward_close(host(got[0]), want[0])
    assert_backward_close(host(got[1]), want[1])

    wl4 = make_workload(4, hw=(32, 40), batch=1)
    t4 = wl4.tensors
    v2 = (t4["ref"], t4["src"], t4["depth_grid"], t4["Rs"], t4["Ts"])
    _, m4 = oracle.cost_volume_v2_fwd(*v2, "MEAN", 4)
    want = oracle.cost_volume_v2_bwd(*v2, t4["cost_grad"], m4, "MEAN", 4)
    ins = [dev(x) for x in v2]
    got = chop.cost_volume_grad_v2(*ins, dev(t4["cost_grad"]), dev(m4), "MEAN", 4,
                                   need_depth_grad=False)
    _assert_family(family)
    assert got[2] is None
    assert_backward_close(host(got[0]), want[0])
    assert_backward_close(host(got[1]), want[1])
    ins16 = [dev(v2[0], torch.bfloat16), dev(v2[1], torch.bfloat16)] + ins[2:]
    got = chop.cost_volume_grad_v2(*ins16, dev(t4["cost_grad"], torch.bfloat16), dev(m4),
                                   "MEAN", 4, need_depth_grad=False)
    assert got[2] is None
    _assert_16bit_close(host(got[0]), want[0], "bf16")
    _assert_16bit_close(host(got[1]), want[1], "bf16")

    ins = _v1_inputs(t)
    ins[0].requires_grad_(True), ins[1].requires_grad_(True)
    cost, _ = chop.cost_volume(*ins)
    (cost * dev(t["cost_grad"])).sum().backward()
    _, mask = oracle.cost_volume_fwd(*args)
    want = oracle.cost_volume_bwd(*args, t["cost_grad"], mask)
    assert_backward_close(host(ins[0].grad), want[0])
    assert_backward_close(host(ins[1].grad), want[1])
    assert ins[2].grad is None


def test_empty_and_degenerate_inputs():
    z = lambda *s: torch.zeros(*s, device="cuda")
    cost, mask = chop.cost_volume_raw(z(1, 0, 4, 3), z(1, 2, 0, 4, 3), z(1, 0, 4, 1), z(1, 5),
                                      z(1, 2, 3, 3), z(1, 2, 3))
    assert cost.shape == (1, 0, 4, 5, 3) and mask.shape == (1, 0, 4, 5, 1)
    # no source views: every count is zero and the cost row stays zero
    ref = torch.randn(1, 4, 5, 3, device="cuda")
    cost, mask = chop.cost_volume_raw(ref, z(1, 0, 4, 5, 3), torch.ones(1, 4, 5, 1, device="cuda"),
                                      torch.ones(1, 2, device="cuda"), z(1, 0, 3, 3), z(1, 0, 3))
    assert int(mask.abs().sum()) == 0 and float(cost.abs().sum()) == 0
    rg, sg, bg = chop.cost_volume_grad(ref, z(1, 0, 4, 5, 3), torch.ones(1, 4, 5, 1, device="cuda"),
                                       torch.ones(1, 2, device="cuda"), z(1, 0, 3, 3), z(1, 0, 3),
                                       torch.ones_like(cost), mask)
    assert float(rg.abs().sum()) == 0 and float(bg.abs().sum()) == 0 and sg.numel() == 0
    # every sample behind the camera
    src = torch.randn(1, 2, 4, 5, 3, device="cuda")
    Rs = torch.eye(3, device="cuda").expand(1, 2, 3, 3).contiguous()
    Ts = torch.tensor([0.0, 0.0, -100.0], device="cuda").expand(1, 2, 3).contiguous()
    cost, mask = chop.cost_volume_raw(ref, src, torch.ones(1, 4, 5, 1, device="cuda"),
                                      torch.ones(1, 2, device="cuda"), Rs, Ts)
    assert int(mask.abs().sum()) == 0 and float(cost.abs().sum()) == 0
    cmin, mmin = chop.cost_volume_raw(ref, src, torch.ones(1, 4, 5, 1, device="cuda"),
                                      torch.ones(1, 2, device="cuda"), Rs, Ts, "MIN")
    assert bool((mmin == -1).all()) and bool((cmin == torch.finfo(torch.float32).max).all())


# ---- committed golden vectors ------------------------------------------------------------------
@pytest.mark.parametrize("family", FAMILIES)
def test_golden_vectors(family):
    """The fixtures of tests/golden/costvol_golden.npz (frozen oracle outputs)."""
    import os
    _lib.load().chop_set_kernel_family(family)
    blob = np.load(os.path.join(os.path.dirname(__file__), "golden", "costvol_golden.npz"))
    names = sorted({k.split("/")[0] for k in blob.files})
    for name in names:
        print("[golden]", name, flush=True)
        op, red, groups, half = (int(x) for x in blob[name + "/attrs"])
        t = {k.split("/")[-1]: blob[k] for k in blob.files if k.startswith(name + "/in/")}
        red_s = "MEAN" if red == 0 else "MIN"
        want_cost, want_mask = blob[name + "/out/cost"], blob[name + "/out/mask"]
        if op == 0:
            ins = [dev(t[k]) for k in ("ref", "src", "base_plane", "offsets", "Rs", "Ts")]
            cost, mask = chop.cost_volume_raw(*ins, red_s, bool(half))
            got = chop.cost_volume_grad(*ins, dev(t["cost_grad"]), dev(want_mask), red_s, bool(half))
        elif op == 2:
            ins = [dev(t[k]) for k in ("ref", "src", "base_plane", "offsets", "Rs", "Ts")]
            cost, mask = chop.cost_aggregate_raw(*ins, red_s, bool(half))
            got = chop.cost_aggregate_grad(*ins, dev(t["cost_grad"]), dev(want_mask), red_s,
                                           bool(half))
        elif op == 3:
            ins = [dev(t[k]) for k in ("ref", "src", "base_plane", "offsets", "Rs", "Ts")]
            cost, mask = chop.cost_volume_v3_raw(*ins, red_s, groups, bool(half))
            got = chop.cost_volume_grad_v3(*ins, dev(t["cost_grad"]), dev(want_mask), red_s, groups,
                                           bool(half))
        elif op == 4:
            ins = [dev(t[k]) for k in ("src", "base_plane", "offsets", "Rs", "Ts")]
            cost, mask = chop.feature_aggregate_raw(*ins, bool(half))
            got = chop.feature_aggregate_grad(*ins, dev(t["cost_grad"]), dev(want_mask), bool(half))
        else:
            ins = [dev(t[k]) for k in ("ref", "src", "depth_grid", "Rs", "Ts")]
            cost, mask = chop.cost_volume_v2_raw(*ins, red_s, groups, bool(half))
            got = chop.cost_volume_grad_v2(*ins, dev(t["cost_grad"]), dev(want_mask), red_s, groups,
                                           bool(half))
        assert np.array_equal(host(mask), want_mask), name
        if family in (1, 2) or op >= 3:   # literal operation order: same bits
            assert np.array_equal(host(cost), want_cost), name
        else:
            assert_forward_close(host(cost), want_cost, atol=1e-5 if op == 1 else 1e-6)
        tol = 1e-4 if want_cost.dtype == np.float32 else 1e-10
        keys = ("src_grad", "depth_grad") if op == 4 else ("ref_grad", "src_grad", "depth_grad")
        for g, k in zip(got, keys):
            assert_backward_close(host(g), blob[name + "/out/" + k], tol)


# ---- per-voxel hypotheses for the squared difference (cascade fine stage, exact form) ----------
@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("storage", ["f16", "bf16"])
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_v1_16bit_depth_grid(oracle, family, storage, reduce):
    """chop_cost_volume_{fwd,bwd}_16 with a depth_grid: the cascade workload's multiplicative
    hypotheses coarse * (1 + 0.02 k), N = 4 views, so that the per-voxel depth gradient of
    the tiled kernels is added up over the view groups."""
    _lib.load().chop_set_kernel_family(family)
    wl = make_workload(3, hw=(40, 56))
    t = wl.tensors
    ref, src, cg = (quantise(t[k], storage) for k in ("ref", "src", "cost_grad"))
    grid = t["depth_grid"]
    assert grid.shape == (1, 40, 56, 32)
    want_cost, want_mask = oracle.cost_volume_grid_fwd(ref, src, grid, t["Rs"], t["Ts"], reduce,
                                                       threads=8)
    td = TORCH_DTYPE[storage]
    d_ref, d_src, d_grid, d_rs, d_ts = dev(ref, td), dev(src, td), dev(grid), dev(t["Rs"]), dev(t["Ts"])
    cost, mask = chop.cost_volume_raw(d_ref, d_src, None, None, d_rs, d_ts, reduce, depth_grid=d_grid)
    _assert_family(family)
    assert np.array_equal(host(mask), want_mask)
    if reduce == "MEAN":
        _assert_16bit_close(host(cost), want_cost, storage)
    else:  # rows no view reaches keep the float maximum, which does not fit 16 bits
        ok = want_mask >= 0
        np.testing.assert_allclose(host(cost)[ok], want_cost[ok], rtol=1e-2,
                                   atol=1e-2 * rms(want_cost[ok]))
    want = oracle.cost_volume_grid_bwd(ref, src, grid, t["Rs"], t["Ts"], cg, want_mask, reduce)
    got = chop.cost_volume_grad(d_ref, d_src, None, None, d_rs, d_ts, dev(cg, td), dev(want_mask),
                                reduce, depth_grid=d_grid)
    _assert_family(family)
    assert got[2].shape == grid.shape and got[2].dtype == torch.float32
    for g, w in zip(got, want):
        _assert_16bit_close(host(g), w, storage)
    # no depth gradient wanted: the other two are unchanged
    two = chop.cost_volume_grad(d_ref, d_src, None, None, d_rs, d_ts, dev(cg, td), dev(want_mask),
                                reduce, need_depth_grad=False, depth_grid=d_grid)
    assert two[2] is None
    _assert_16bit_close(host(two[0]), want[0], storage)
    _assert_16bit_close(host(two[1]), want[1], storage)


def test_depth_grid_needs_16bit_storage():
    wl = make_workload(3, hw=(8, 8))
    t = wl.tensors
    with pytest.raises(chop.InvalidArgumentError):
        chop.cost_volume_raw(dev(t["ref"]), dev(t["src"]), None, None, dev(t["Rs"]), dev(t["Ts"]),
                             depth_grid=dev(t["depth_grid"]))


# ---- full benchmark sizes -----------------------------------------------------------------------
@pytest.mark.parametrize("form", ["plane", "grid"])
def test_cascade_fine_full_size(oracle, form):
    """Benchmark configuration 3 at its real size (f16 storage, B1 N4 256x320 C16 D32), both
    forms: base_plane + additive offsets (the registered op's) and the exact per-pixel
    multiplicative hypotheses through depth_grid."""
    wl = make_workload(3)
    t = wl.tensors
    ref, src, cg = (quantise(t[k], "f16") for k in ("ref", "src", "cost_grad"))
    td = torch.float16
    d_ref, d_src, d_rs, d_ts = dev(ref, td), dev(src, td), dev(t["Rs"]), dev(t["Ts"])
    if form == "plane":
        args = (ref, src, t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
        want_cost, want_mask = oracle.cost_volume_fwd(*args, threads=16)
        want = oracle.cost_volume_bwd(*args, cg, want_mask, threads=16)
        cost, mask = chop.cost_volume_raw(d_ref, d_src, dev(t["base_plane"]), dev(t["offsets"]), d_rs, d_ts)
        _assert_family(0)
        got = chop.cost_volume_grad(d_ref, d_src, dev(t["base_plane"]), dev(t["offsets"]), d_rs, d_ts,
                                    dev(cg, td), mask)
    else:
        args = (ref, src, t["depth_grid"], t["Rs"], t["Ts"])
        want_cost, want_mask = oracle.cost_volume_grid_fwd(*args, threads=16)
        want = oracle.cost_volume_grid_bwd(*args, cg, want_mask, threads=16)
        d_grid = dev(t["depth_grid"])
        cost, mask = chop.cost_volume_raw(d_ref, d_src, None, None, d_rs, d_ts, depth_grid=d_grid)
        _assert_family(0)
        got = chop.cost_volume_grad(d_ref, d_src, None, None, d_rs, d_ts, dev(cg, td), mask,
                                    depth_grid=d_grid)
    _assert_family(0)
    assert cost.shape == (1, 256, 320, 32, 16)
    assert np.array_equal(host(mask), want_mask)
    _assert_16bit_close(host(cost), want_cost, "f16")
    for g, w in zip(got, want):
        _assert_16bit_close(host(g), w, "f16")


def test_group_correlation_full_size(oracle):
    """Benchmark configuration 4 at its real size (bf16 storage, B2 N4 512x640 C8 G4 D8)."""
    wl = make_workload(4)
    t = wl.tensors
    ref, src, cg = (quantise(t[k], "bf16") for k in ("ref", "src", "cost_grad"))
    args = (ref, src, t["depth_grid"], t["Rs"], t["Ts"])
    want_cost, want_mask = oracle.cost_volume_v2_fwd(*args, "MEAN", 4, threads=16)
    want = oracle.cost_volume_v2_bwd(*args, cg, want_mask, "MEAN", 4, threads=16)
    td = torch.bfloat16
    ins = [dev(ref, td), dev(src, td), dev(t["depth_grid"]), dev(t["Rs"]), dev(t["Ts"])]
    cost, mask = chop.cost_volume_v2_raw(*ins, "MEAN", 4)
    _assert_family(0)
    assert cost.shape == (2, 512, 640, 8, 4)
    assert np.array_equal(host(mask), want_mask)
    _assert_16bit_close(host(cost), want_cost, "bf16")
    got = chop.cost_volume_grad_v2(*ins, dev(cg, td), mask, "MEAN", 4)
    _assert_family(0)
    for g, w in zip(got, want):
        _assert_16bit_close(host(g), w, "bf16")



def test_mvsnet_stage_full_size(oracle):
    """Benchmark configuration 2 at its real size, forward and backward, against the oracle
    (the oracle takes a few seconds on the box's host cores)."""
    wl = make_workload(2)
    t = wl.tensors
    args = (t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
    want_cost, want_mask = oracle.cost_volume_fwd(*args, threads=16)
    ins = _v1_inputs(t)
    cost, mask = chop.cost_volume_raw(*ins)
    _assert_family(0)
    assert cost.shape == (1, 128, 160, 192, 32)
    assert np.array_equal(host(mask), want_mask)
    # (how much of the comparison rests on the absolute floors: under one element in a hundred)
    assert assert_forward_close(host(cost), want_cost, what="cost") < 0.01
    del cost
    want = oracle.cost_volume_bwd(*args, t["cost_grad"], want_mask, threads=16)
    got = chop.cost_volume_grad(*ins, dev(t["cost_grad"]), mask)
    _assert_family(0)
    for g, w, name in zip(got, want, ("ref_grad", "src_grad", "base_plane_grad")):
        assert assert_backward_close(host(g), w, what=name) < 0.01


def test_large_batch_stress_full_size():
    """Benchmark configuration 5 at its real size (7.25 GB cost volume): size-independent
    properties on the whole result, the oracle on one band of one batch item."""
    import oracle
    wl = make_workload(5, with_cost_grad=False)
    t = wl.tensors
    ins = _v1_inputs(t)
    cost, mask = chop.cost_volume_raw(*ins)
    _assert_family(0)
    assert cost.shape == (4, 288, 384, 128, 32) and cost.numel() == 1811939328
    assert int(mask.min()) >= 0 and int(mask.max()) <= wl.N
    out_of_frustum = 1.0 - float(mask.float().mean()) / wl.N
    print("[stress] samples outside every frustum: %.1f%%" % (100 * out_of_frustum), flush=True)
    assert 0.05 < out_of_frustum < 0.95
    assert float(cost.min()) >= 0.0
    assert float((cost.abs() * (mask == 0)).max()) == 0.0  # rows no view reaches stay zero
    b, r0, r1 = 3, 100, 116
    band = (t["ref"][b:b + 1, r0:r1], t["src"][b:b + 1], t["base_plane"][b:b + 1, r0:r1],
            t["offsets"][b:b + 1], t["Rs"][b:b + 1], t["Ts"][b:b + 1])
    # the oracle runs on reference rows 0..r1 of that batch item (rows above the band are
    # computed and dropped) so that every pixel keeps its own coordinates
    want_cost, want_mask = oracle.cost_volume_fwd(
        t["ref"][b:b + 1, :r1], band[1], t["base_plane"][b:b + 1, :r1], band[3], band[4], band[5],
        threads=16)
    got_cost = host(cost[b, r0:r1])
    got_mask = host(mask[b, r0:r1])
    assert np.array_equal(got_mask, want_mask[0, r0:r1])
    assert_forward_close(got_cost, want_cost[0, r0:r1])
    # backward: linearity in the upstream gradient and conservation, on the full size
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    cg = torch.randn(cost.shape, device="cuda", generator=gen)
    del cost
    g1 = chop.cost_volume_grad(*ins, cg, mask)
    _assert_family(0)
    # ref_grad and base_plane_grad are owned by their pixel: a band of them against the oracle
    # run on that band alone (the first rows of a batch item, so no rows above it are needed)
    b, r1 = 2, 16
    want = oracle.cost_volume_bwd(t["ref"][b:b + 1, :r1], t["src"][b:b + 1], t["base_plane"][b:b + 1, :r1],
                                  t["offsets"][b:b + 1], t["Rs"][b:b + 1], t["Ts"][b:b + 1],
                                  host(cg[b:b + 1, :r1]), host(mask[b:b + 1, :r1]), threads=16)
    assert_backward_close(host(g1[0][b:b + 1, :r1]), want[0], what="ref_grad band")
    assert_backward_close(host(g1[2][b:b + 1, :r1]), want[2], what="base_plane_grad band")
    rg, sg = g1[0].double(), g1[1].double()
    assert abs(float(rg.sum() + sg.sum())) < 1e-4 * float(rg.abs().sum())
    cg.mul_(2.0)
    g2 = chop.cost_volume_grad(*ins, cg, mask)
    for a1, a2 in zip(g1, g2):
        scale = float(a1.abs().max())
        assert float((a2 - 2 * a1).abs().max()) <= 2e-4 * scale
    # Six source views: the launcher took the wide form of the 32-channel kernel (three waves
    # per SIMD, 8 x 8 scatter window).  The slimmed form (four waves, 6 x 8 window), in which
    # far more of this workload's cells stick out of the window and go to memory on their own,
    # must agree with it.
    lib = _lib.load()
    assert lib.chop_last_backward_window() == 8
    lib.chop_set_backward_window(6)
    try:
        g3 = chop.cost_volume_grad(*ins, cg, mask)
        assert lib.chop_last_backward_window() == 6
    finally:
        lib.chop_set_backward_window(0)
    for a2, a3 in zip(g2, g3):
        scale = float(a2.abs().max())
        assert float((a3 - a2).abs().max()) <= 2e-4 * scale
    assert_backward_close(host(g3[0][b:b + 1, :r1]) / 2, want[0], what="ref_grad band, slimmed kernel")


def test_volume_above_two_to_the_31_elements():
    """The stress configuration with six batch items: 2.72 G cost elements (10.9 GB), so the
    whole last batch item lies beyond element 2^31, where the reference switches to 64-bit
    indices (cost_volume_kernels_gpu.cu.cc:313, :619).  The library's own choice of kernels
    and the general kernels forced onto the same shape: mask bit-exact and cost within 1e-5
    on a band of the last batch item, whole-volume properties, and for the backward
    conservation plus the pixel-owned gradients of the band against the oracle."""
    import oracle
    wl = make_workload(5, with_cost_grad=False, batch=6)
    t = wl.tensors
    assert wl.B * wl.H * wl.W * wl.D * wl.C > 2 ** 31 + 2 ** 29
    ins = _v1_inputs(t)
    b, r1 = wl.B - 1, 16
    assert b * wl.H * wl.W * wl.D * wl.C > 2 ** 31   # the band's rows start beyond 2^31
    band = (t["ref"][b:b + 1, :r1], t["src"][b:b + 1], t["base_plane"][b:b + 1, :r1],
            t["offsets"][b:b + 1], t["Rs"][b:b + 1], t["Ts"][b:b + 1])
    want_cost, want_mask = oracle.cost_volume_fwd(*band, threads=16)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(31)
    cg = torch.randn((wl.B, wl.H, wl.W, wl.D, wl.C), device="cuda", generator=gen)
    want = oracle.cost_volume_bwd(*band, host(cg[b:b + 1, :r1]), want_mask, threads=16)
    for family in (0, 1):
        print("[case] above 2^31 elements, kernel family %d" % family, flush=True)
        _lib.load().chop_set_kernel_family(family)
        cost, mask = chop.cost_volume_raw(*ins)
        _assert_family(family)
        assert cost.numel() == 2717908992
        assert np.array_equal(host(mask[b, :r1]), want_mask[0])
        if family == 1:
            assert np.array_equal(host(cost[b, :r1]), want_cost[0])   # literal operand order
        else:
            assert_forward_close(host(cost[b, :r1]), want_cost[0])
        assert int(mask.min()) >= 0 and int(mask.max()) <= wl.N
        assert float(cost.min()) >= 0.0
        assert float((cost[b].abs() * (mask[b] == 0)).max()) == 0.0
        del cost
        g = chop.cost_volume_grad(*ins, cg, mask)
        _assert_family(family)
        rg, sg = g[0].double(), g[1].double()
        assert abs(float(rg.sum() + sg.sum())) < 1e-4 * float(rg.abs().sum())
        assert float(sg[b].abs().sum()) > 0.0
        assert_backward_close(host(g[0][b:b + 1, :r1]), want[0], what="ref_grad band")
        assert_backward_close(host(g[2][b:b + 1, :r1]), want[2], what="base_plane_grad band")
        del g, rg, sg, mask
        torch.cuda.empty_cache()


# ---- five views: the six-view instantiation with one view missing ----------------------------
@pytest.mark.parametrize("C", [8, 16, 32])
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_five_views(oracle, C, reduce):
    B, N, H, W, D = 1, 5, 14, 18, 11
    t = reference_test_case(3, B, N, H, W, C, D, np.float32, seed=C)
    t["Ts"] = t["Ts"] + np.linspace(-2, 2, N, dtype=np.float32)[None, :, None]   # five different views
    args = tuple(t[k] for k in ("ref", "src", "base_plane", "offsets", "Rs", "Ts"))
    want_cost, want_mask = oracle.cost_volume_fwd(*args, reduce)
    cost, mask = chop.cost_volume_raw(*_v1_inputs(t), reduce)
    _assert_family(0)
    assert np.array_equal(host(mask), want_mask)
    if reduce == "MIN":
        assert np.array_equal(host(cost), want_cost)
    else:
        assert_forward_close(host(cost), want_cost)
    cg = np.random.default_rng(C).standard_normal(want_cost.shape).astype(np.float32)
    want = oracle.cost_volume_bwd(*args, cg, want_mask, reduce)
    got = chop.cost_volume_grad(*_v1_inputs(t), dev(cg), mask, reduce)
    _assert_family(0)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)
    groups = C // 4
    depth_grid = (t["base_plane"] + t["offsets"][:, None, None, :]).astype(np.float32)
    a2 = (t["ref"], t["src"], depth_grid, t["Rs"], t["Ts"])
    want_cost, want_mask = oracle.cost_volume_v2_fwd(*a2, reduce, groups)
    cost, mask = chop.cost_volume_v2_raw(*[dev(x) for x in a2], reduce, groups)
    _assert_family(0)
    assert np.array_equal(host(mask), want_mask)
    if reduce == "MIN":
        assert np.array_equal(host(cost), want_cost)
    else:
        assert_forward_close(host(cost), want_cost, atol=1e-5)


# ---- strip kernels: several view groups, with and without carried runs --------------------------
@pytest.mark.parametrize("C,N,dtype", [(5, 9, np.float64), (40, 9, np.float64), (24, 7, np.float32),
                                       (3, 17, np.float32), (33, 3, np.float64)])
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_strip_many_views(oracle, C, N, dtype, reduce):
    """The strip kernels reproject min(N, max(1, lanes per pixel / 8)) views per phase 1 and keep
    the runs that are open at the end of a chunk in LDS as long as that takes at most 16 KiB
    (N <= 7 in float64, N <= 14 in float32).  These shapes cover one view at a time (C = 3, 5),
    groups of four and eight with a remainder (C = 24, 33, 40) and both sides of the limit;
    D = 21 leaves a ragged last chunk."""
    B, H, W, D = 1, 10, 14, 21
    t = reference_test_case(3, B, N, H, W, C, D, dtype, seed=C + N)
    t["Ts"] = (t["Ts"] + np.linspace(-1, 1, N)[None, :, None]).astype(dtype)   # N different views
    args = tuple(t[k] for k in ("ref", "src", "base_plane", "offsets", "Rs", "Ts"))
    want_cost, want_mask = oracle.cost_volume_fwd(*args, reduce)
    _lib.load().chop_set_kernel_family(2)
    cost, mask = chop.cost_volume_raw(*_v1_inputs(t), reduce)
    _assert_family(2)
    assert np.array_equal(host(mask), want_mask)
    assert np.array_equal(host(cost), want_cost)   # literal operand order: bit-identical
    cg = np.random.default_rng(C).standard_normal(want_cost.shape).astype(dtype)
    want = oracle.cost_volume_bwd(*args, cg, want_mask, reduce)
    got = chop.cost_volume_grad(*_v1_inputs(t), dev(cg), mask, reduce)
    _assert_family(2)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)
    if C in (24, 40):
        groups = 8
        depth_grid = (t["base_plane"] + t["offsets"][:, None, None, :]).astype(dtype)
        a2 = (t["ref"], t["src"], depth_grid, t["Rs"], t["Ts"])
        want_cost, want_mask = oracle.cost_volume_v2_fwd(*a2, reduce, groups)
        cost, mask = chop.cost_volume_v2_raw(*[dev(x) for x in a2], reduce, groups)
        _assert_family(2)
        assert np.array_equal(host(mask), want_mask)
        assert np.array_equal(host(cost), want_cost)
        cg = np.random.default_rng(N).standard_normal(want_cost.shape).astype(dtype)
        want = oracle.cost_volume_v2_bwd(*a2, cg, want_mask, reduce, groups)
        got = chop.cost_volume_grad_v2(*[dev(x) for x in a2], dev(cg), mask, reduce, groups)
        _assert_family(2)
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)


@pytest.mark.parametrize("C,N", [(12, 3), (32, 2), (20, 1)])
def test_strip_float64_wide_pixels(oracle, C, N):
    """Float64 with 16 lanes or more per pixel and few views: the strip gradient kernels then put
    a texel cache in LDS between the runs and memory, end every run with its chunk instead of
    carrying it, and run in their four-waves-per-SIMD form.  Every op that reaches them, both
    reduces; D = 21 leaves a ragged last chunk."""
    B, H, W, D = 1, 11, 15, 21
    t = reference_test_case(3, B, N, H, W, C, D, np.float64, seed=3 * C + N)
    t["Ts"] = (t["Ts"] + np.linspace(-1, 1, N)[None, :, None]).astype(np.float64)
    args = tuple(t[k] for k in ("ref", "src", "base_plane", "offsets", "Rs", "Ts"))
    ins = [dev(x) for x in args]
    rng = np.random.default_rng(C + N)
    groups = 4
    depth_grid = t["base_plane"] + t["offsets"][:, None, None, :]
    a2 = (t["ref"], t["src"], depth_grid, t["Rs"], t["Ts"])
    in2 = [dev(x) for x in a2]
    for reduce in ("MEAN", "MIN"):
        want_cost, want_mask = oracle.cost_volume_fwd(*args, reduce)
        cost, mask = chop.cost_volume_raw(*ins, reduce)
        _assert_family(2)
        assert np.array_equal(host(mask), want_mask) and np.array_equal(host(cost), want_cost)
        cg = rng.standard_normal(want_cost.shape)
        want = oracle.cost_volume_bwd(*args, cg, want_mask, reduce)
        got = chop.cost_volume_grad(*ins, dev(cg), mask, reduce)
        _assert_family(2)
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)

        want_cost, want_mask = oracle.cost_volume_v2_fwd(*a2, reduce, groups)
        cost, mask = chop.cost_volume_v2_raw(*in2, reduce, groups)
        assert np.array_equal(host(mask), want_mask) and np.array_equal(host(cost), want_cost)
        cg = rng.standard_normal(want_cost.shape)
        want = oracle.cost_volume_v2_bwd(*a2, cg, want_mask, reduce, groups)
        got = chop.cost_volume_grad_v2(*in2, dev(cg), mask, reduce, groups)
        _assert_family(2)
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)

        want_cost, want_mask = oracle.cost_aggregate_fwd(*args, reduce)
        cost, mask = chop.cost_aggregate_raw(*ins, reduce)
        assert np.array_equal(host(mask), want_mask)
        cg = rng.standard_normal(want_cost.shape)
        want = oracle.cost_aggregate_bwd(*args, cg, want_mask, reduce)
        got = chop.cost_aggregate_grad(*ins, dev(cg), mask, reduce)
        _assert_family(2)
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)

        want_cost, want_mask = oracle.cost_volume_v3_fwd(*args, reduce, groups)
        cost, mask = chop.cost_volume_v3_raw(*ins, reduce, groups)
        assert np.array_equal(host(mask), want_mask)
        cg = rng.standard_normal(want_cost.shape)
        want = oracle.cost_volume_v3_bwd(*args, cg, want_mask, reduce, groups)
        got = chop.cost_volume_grad_v3(*ins, dev(cg), mask, reduce, groups)
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)

    fargs = args[1:]
    want_feat, want_mask = oracle.feature_aggregate_fwd(*fargs)
    feat, mask = chop.feature_aggregate_raw(*ins[1:])
    assert np.array_equal(host(mask), want_mask) and np.array_equal(host(feat), want_feat)
    cg = rng.standard_normal(want_feat.shape)
    want = oracle.feature_aggregate_bwd(*fargs, cg, want_mask)
    got = chop.feature_aggregate_grad(*ins[1:], dev(cg), mask)
    _assert_family(2)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)


# ---- samples that jump far between consecutive depths ------------------------------------------
@pytest.mark.parametrize("C", [4, 8, 16, 32, 64])
def test_backward_cells_outside_the_scatter_window(oracle, C):
    """A sideways camera offset close to the scene: consecutive depth hypotheses land many
    texels apart, so most cells lie outside the kernel's scatter window and take its direct
    path to memory.  One case per lanes-per-pixel variant; FeatureAggregate's gradient runs
    the same kernel."""
    rng, geo = np.random.default_rng(C), np.random.default_rng(4)   # one geometry for all widths
    B, N, H, W, D = 1, 2, 12, 72, 14
    t = dict(base_plane=geo.uniform(1.0, 1.2, (B, H, W, 1)).astype(np.float32),
             offsets=geo.permutation(np.linspace(0.0, 3.0, D)).astype(np.float32)[None].repeat(B, 0),
             ref=rng.normal(size=(B, H, W, C)).astype(np.float32),
             src=rng.normal(size=(B, N, H, W, C)).astype(np.float32),
             Rs=np.tile(np.eye(3, dtype=np.float32)[None, None], (B, N, 1, 1)),
             Ts=np.array([[[40.0, 3.0, 0.0], [-35.0, -2.0, 0.0]]], np.float32).repeat(B, 0))
    args = tuple(t[k] for k in ("ref", "src", "base_plane", "offsets", "Rs", "Ts"))
    sw, sh, fh, fw, state = oracle.sample_coords(t["base_plane"], t["offsets"], t["Rs"], t["Ts"], (H, W))
    ok = state == 2
    jump = np.abs(np.diff(np.where(ok, fw, 0), axis=3))[ok[:, :, :, 1:] & ok[:, :, :, :-1]]
    assert ok.mean() > 0.2 and np.median(jump) >= 6 and jump.max() > 20   # a chunk spans far more than the 16 texel columns of a window
    want_cost, want_mask = oracle.cost_volume_fwd(*args)
    cost, mask = chop.cost_volume_raw(*_v1_inputs(t))
    _assert_family(0)
    assert np.array_equal(host(mask), want_mask)
    assert_forward_close(host(cost), want_cost)
    cg = rng.standard_normal(want_cost.shape).astype(np.float32)
    want = oracle.cost_volume_bwd(*args, cg, want_mask)
    got = chop.cost_volume_grad(*_v1_inputs(t), dev(cg), mask)
    _assert_family(0)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)
    fkeys = ("src", "base_plane", "offsets", "Rs", "Ts")
    _, fmask = oracle.feature_aggregate_fwd(*[t[k] for k in fkeys])
    fg = rng.standard_normal(fmask.shape[:-1] + (C,)).astype(np.float32)
    want = oracle.feature_aggregate_bwd(*[t[k] for k in fkeys], fg, fmask)
    got = chop.feature_aggregate_grad(*[dev(t[k]) for k in fkeys], dev(fg), dev(fmask))
    _assert_family(0)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)


# ---- every lanes-per-pixel variant of the tiled kernels -------------------------------------
@pytest.mark.parametrize("C", [4, 8, 16, 32, 64])
@pytest.mark.parametrize("N", [1, 3])
def test_tiled_channel_widths(oracle, C, N):
    """C = 4, 8, 16, 32, 64 select 1, 2, 4, 8 and 16 lanes per pixel, each with its own record
    path, window size and prefetch depth; D = 21 leaves a partial last chunk everywhere."""
    B, H, W, D = 2, 20, 24, 21
    rng = np.random.default_rng(C + N)
    for case in (1, 3):
        t = reference_test_case(case, B, N, H, W, C, D, np.float32, seed=100 + case)
        args = tuple(t[k] for k in ("ref", "src", "base_plane", "offsets", "Rs", "Ts"))
        want_cost, want_mask = oracle.cost_volume_fwd(*args)
        cost, mask = chop.cost_volume_raw(*_v1_inputs(t))
        _assert_family(0)
        assert np.array_equal(host(mask), want_mask)
        assert_forward_close(host(cost), want_cost)
        cg = rng.standard_normal(want_cost.shape).astype(np.float32)
        want = oracle.cost_volume_bwd(*args, cg, want_mask)
        got = chop.cost_volume_grad(*_v1_inputs(t), dev(cg), dev(want_mask))
        _assert_family(0)
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)
        # group correlation with per-voxel depths on the same tensors
        groups = C // 2
        grid = (t["base_plane"] + t["offsets"][:, None, None, :]).astype(np.float32)
        a2 = (t["ref"], t["src"], grid, t["Rs"], t["Ts"])
        want_cost, want_mask = oracle.cost_volume_v2_fwd(*a2, "MEAN", groups)
        ins = [dev(x) for x in a2]
        cost, mask = chop.cost_volume_v2_raw(*ins, "MEAN", groups)
        _assert_family(0)
        assert np.array_equal(host(mask), want_mask)
        assert_forward_close(host(cost), want_cost, atol=1e-5)
        cg = rng.standard_normal(want_cost.shape).astype(np.float32)
        want = oracle.cost_volume_v2_bwd(*a2, cg, want_mask, "MEAN", groups)
        got = chop.cost_volume_grad_v2(*ins, dev(cg), dev(want_mask), "MEAN", groups)
        _assert_family(0)
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)
        # MIN / MAX reduces: winners and values bit for bit
        want_cost, want_mask = oracle.cost_volume_fwd(*args, "MIN")
        cost, mask = chop.cost_volume_raw(*_v1_inputs(t), "MIN")
        _assert_family(0)
        assert np.array_equal(host(mask), want_mask) and np.array_equal(host(cost), want_cost)
        cg = rng.standard_normal(want_cost.shape).astype(np.float32)
        want = oracle.cost_volume_bwd(*args, cg, want_mask, "MIN")
        got = chop.cost_volume_grad(*_v1_inputs(t), dev(cg), dev(want_mask), "MIN")
        _assert_family(0)
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)
        want_cost, want_mask = oracle.cost_volume_v2_fwd(*a2, "MIN", groups)
        cost, mask = chop.cost_volume_v2_raw(*ins, "MIN", groups)
        _assert_family(0)
        assert np.array_equal(host(mask), want_mask) and np.array_equal(host(cost), want_cost)
        cg = rng.standard_normal(want_cost.shape).astype(np.float32)
        want = oracle.cost_volume_v2_bwd(*a2, cg, want_mask, "MIN", groups)
        got = chop.cost_volume_grad_v2(*ins, dev(cg), dev(want_mask), "MIN", groups)
        _assert_family(0)
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)
        # minimum of the summed squared difference: the tiled forward adds the channels in
        # the reference's order (staged through LDS), so winner and cost are bit-exact
        want_cost, want_mask = oracle.cost_aggregate_fwd(*args, "MIN")
        cost, mask = chop.cost_aggregate_raw(*_v1_inputs(t), "MIN")
        _assert_family(0)
        assert np.array_equal(host(mask), want_mask) and np.array_equal(host(cost), want_cost)
        cg = rng.standard_normal(want_cost.shape).astype(np.float32)
        want = oracle.cost_aggregate_bwd(*args, cg, want_mask, "MIN")
        got = chop.cost_aggregate_grad(*_v1_inputs(t), dev(cg), dev(want_mask), "MIN")
        _assert_family(0)
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)
        # summed squared difference
        want_cost, want_mask = oracle.cost_aggregate_fwd(*args)
        cost, mask = chop.cost_aggregate_raw(*_v1_inputs(t))
        _assert_family(0)
        assert np.array_equal(host(mask), want_mask)
        assert_forward_close(host(cost), want_cost)
        cg = rng.standard_normal(want_cost.shape).astype(np.float32)
        want = oracle.cost_aggregate_bwd(*args, cg, want_mask)
        got = chop.cost_aggregate_grad(*_v1_inputs(t), dev(cg), dev(want_mask))
        _assert_family(0)
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)


# ---- HIP graph capture ----------------------------------------------------------------------
def test_entry_points_replay_in_a_hip_graph(oracle):
    """The entry points only enqueue kernels (their zero fills are kernels too), so a caller
    may capture them.  One graph holds a CostVolume forward and backward call, a backward call
    without the depth gradient and a CostVolumeV3 forward and backward call; it is replayed
    several times on changing inputs, with eager work and synchronisations in between, and
    every replay is checked against the oracle."""
    lib = _lib.load()
    B, N, H, W, C, D = 1, 2, 16, 20, 32, 24
    t = reference_test_case(3, B, N, H, W, C, D, np.float32, seed=77)
    keys = ("ref", "src", "base_plane", "offsets", "Rs", "Ts")
    ins = {k: dev(t[k]) for k in keys}
    cost = torch.empty((B, H, W, D, C), device="cuda")
    mask = torch.empty((B, H, W, D, 1), dtype=torch.int32, device="cuda")
    cg = torch.empty_like(cost)
    grads = [torch.empty_like(ins["ref"]), torch.empty_like(ins["src"]), torch.empty_like(ins["base_plane"])]
    grads2 = [torch.empty_like(ins["ref"]), torch.empty_like(ins["src"])]
    cost3 = torch.empty((B, H, W, D, 1), device="cuda")
    mask3 = torch.empty((B, H, W, D, 1), dtype=torch.int32, device="cuda")
    cg3 = torch.empty_like(cost3)
    grads3 = [torch.empty_like(g) for g in grads]
    dims = (B, H, W, C, D, N, H, W)

    def step():
        s = torch.cuda.current_stream().cuda_stream
        p = [ins[k].data_ptr() for k in keys]
        assert lib.chop_cost_volume_fwd_f32(s, 0, 1, *dims, *p, cost.data_ptr(), mask.data_ptr()) == 0
        assert lib.chop_cost_volume_bwd_f32(s, 0, 1, *dims, *p, cg.data_ptr(), mask.data_ptr(),
                                            *[g.data_ptr() for g in grads]) == 0
        assert lib.chop_cost_volume_bwd_f32(s, 0, 1, *dims, *p, cg.data_ptr(), mask.data_ptr(),
                                            *[g.data_ptr() for g in grads2], None) == 0
        assert lib.chop_cost_volume_v3_fwd_f32(s, 0, 1, *dims, 4, *p, cost3.data_ptr(),
                                               mask3.data_ptr()) == 0
        assert lib.chop_last_kernel_family() == 2
        assert lib.chop_cost_volume_v3_bwd_f32(s, 0, 1, *dims, 4, *p, cg3.data_ptr(),
                                               mask3.data_ptr(), *[g.data_ptr() for g in grads3]) == 0
        assert lib.chop_last_kernel_family() == 2

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step()
    rng = np.random.default_rng(5)
    for replay in range(4):
        new_ref = rng.uniform(0, 10, t["ref"].shape).astype(np.float32)
        new_cg = rng.standard_normal(cost.shape).astype(np.float32)
        ins["ref"].copy_(dev(new_ref))          # eager work between the replays
        cg.copy_(dev(new_cg))
        new_cg3 = rng.standard_normal(cost3.shape).astype(np.float32)
        cg3.copy_(dev(new_cg3))
        for g in grads + grads2 + grads3:
            g.fill_(float("nan"))               # the graph has to zero what it accumulates into
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        args = (new_ref,) + tuple(t[k] for k in keys[1:])
        want_cost, want_mask = oracle.cost_volume_fwd(*args)
        want = oracle.cost_volume_bwd(*args, new_cg, want_mask)
        assert np.array_equal(host(mask), want_mask), replay
        assert_forward_close(host(cost), want_cost)
        for g, w in zip(grads, want):
            assert_backward_close(host(g), w)
        for g, w in zip(grads2, want[:2]):
            assert_backward_close(host(g), w)
        want_cost3, want_mask3 = oracle.cost_volume_v3_fwd(*args, "MEAN", 4)
        assert np.array_equal(host(mask3), want_mask3) and np.array_equal(host(cost3), want_cost3)
        for g, w in zip(grads3, oracle.cost_volume_v3_bwd(*args, new_cg3, want_mask3, "MEAN", 4)):
            assert_backward_close(host(g), w)
