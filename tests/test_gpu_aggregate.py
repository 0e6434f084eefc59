"""GPU parity of the CostAggregate entry points against the CPU oracle (same bars as the
cost volume: masks bit-exact, fp32 forward 1e-5, fp32 backward 1e-4)."""
import numpy as np
import pytest
import torch

import custom_helper_op_amd as chop
from custom_helper_op_amd import _lib
from custom_helper_op_amd.configs import make_workload, reference_test_case
from gpu_util import assert_backward_close, assert_forward_close, dev, host

pytestmark = pytest.mark.gpu

FAMILIES = [pytest.param(1, id="general"), pytest.param(2, id="strip"), pytest.param(0, id="auto")]
# (B, N, H, W, C, D): the reference tests' parameter sets plus channel counts the tiled
# kernels take (multiples of 4) and ones they do not
SHAPES = [(1, 1, 12, 16, 3, 5), (1, 2, 12, 16, 8, 9), (2, 2, 12, 18, 5, 10), (2, 3, 12, 16, 16, 6),
          (1, 2, 20, 24, 32, 19)]
KEYS = ("ref", "src", "base_plane", "offsets", "Rs", "Ts")


@pytest.fixture(autouse=True)
def _announce(request):
    print("\n[case] %s" % request.node.nodeid, flush=True)
    yield
    _lib.load().chop_set_kernel_family(0)


def _inputs(t):
    return [dev(t[k]) for k in KEYS]


def _args(t):
    return tuple(t[k] for k in KEYS)


def _expect_family(family, C, reduce, dtype, backward=False):
    """Which kernels served the last call (1 general, 2 tiled, 3 strip).  Left to itself the
    library gives float32 with a channel count of 4 times a power of two to the tiled kernels
    and everything else (float64, other channel counts) to the strip kernels."""
    tiled = dtype == np.float32 and C in (4, 8, 16, 32, 64)
    want = {1: 1, 2: 3, 0: 2 if tiled else 3}[family]
    got = _lib.load().chop_last_kernel_family()
    assert got == want, (got, want, family, C, reduce, dtype)


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_forward(oracle, family, shape, reduce, dtype):
    _lib.load().chop_set_kernel_family(family)
    B, N, H, W, C, D = shape
    for case in range(4):
        t = reference_test_case(case, B, N, H, W, C, D, dtype, seed=case)
        want_cost, want_mask = oracle.cost_aggregate_fwd(*_args(t), reduce)
        cost, mask = chop.cost_aggregate_raw(*_inputs(t), reduce)
        _expect_family(family, C, reduce, dtype)
        assert cost.shape == (B, H, W, D) and mask.shape == (B, H, W, D)
        assert np.array_equal(host(mask), want_mask)
        if _lib.load().chop_last_kernel_family() != 2 or reduce == "MIN":
            assert np.array_equal(host(cost), want_cost)  # literal operation order: same bits
        else:
            assert_forward_close(host(cost), want_cost)


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_backward(oracle, family, shape, reduce, dtype):
    _lib.load().chop_set_kernel_family(family)
    B, N, H, W, C, D = shape
    rng = np.random.default_rng(23)
    for case in (1, 3):
        t = reference_test_case(case, B, N, H, W, C, D, dtype, seed=case)
        _, mask = oracle.cost_aggregate_fwd(*_args(t), reduce)
        cg = rng.standard_normal((B, H, W, D)).astype(dtype)
        want = oracle.cost_aggregate_bwd(*_args(t), cg, mask, reduce)
        got = chop.cost_aggregate_grad(*_inputs(t), dev(cg), dev(mask), reduce)
        _expect_family(family, C, reduce, dtype, backward=True)
        tol = 1e-4 if dtype == np.float32 else 1e-10
        for g, w in zip(got, want):
            assert g.shape == w.shape
            assert_backward_close(host(g), w, tol)


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("index,hw,depth", [(2, (32, 40), None), (5, (36, 48), 32)])
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_benchmark_cameras(oracle, family, index, hw, depth, reduce):
    _lib.load().chop_set_kernel_family(family)
    wl = make_workload(index, hw=hw, depth=depth, with_cost_grad=False, batch=1)
    t = wl.tensors
    want_cost, want_mask = oracle.cost_aggregate_fwd(*_args(t), reduce, threads=8)
    cost, mask = chop.cost_aggregate_raw(*_inputs(t), reduce)
    assert np.array_equal(host(mask), want_mask)
    assert_forward_close(host(cost), want_cost)
    cg = np.random.default_rng(3).standard_normal(want_cost.shape).astype(np.float32)
    want = oracle.cost_aggregate_bwd(*_args(t), cg, want_mask, reduce)
    got = chop.cost_aggregate_grad(*_inputs(t), dev(cg), dev(want_mask), reduce)
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)
    rg, sg = host(got[0]).astype(np.float64), host(got[1]).astype(np.float64)
    assert abs(rg.sum() + sg.sum()) < 1e-4 * np.abs(rg).sum()


def test_autograd_matches_grad_op():
    t = reference_test_case(3, 2, 2, 12, 18, 8, 7, np.float32, seed=5)
    x = _inputs(t)
    for k in (0, 1, 2):
        x[k].requires_grad_(True)
    cost, mask = chop.cost_aggregate(*x)
    assert not mask.requires_grad
    w = torch.randn_like(cost)
    (cost * w).sum().backward()
    rg, sg, bg = chop.cost_aggregate_grad(*[v.detach() for v in x], w, mask)
    assert torch.equal(x[0].grad, rg) or torch.allclose(x[0].grad, rg, rtol=1e-4, atol=1e-6)
    assert torch.allclose(x[1].grad, sg, rtol=1e-4, atol=1e-5)
    assert torch.allclose(x[2].grad, bg, rtol=1e-4, atol=1e-5)


def test_errors_and_empty():
    t = reference_test_case(1, 1, 2, 6, 8, 4, 3, np.float32, seed=2)
    x = _inputs(t)
    with pytest.raises(chop.InvalidArgumentError):
        chop.cost_aggregate_raw(*x, reduce_method="MAX")
    with pytest.raises(chop.InvalidArgumentError):
        chop.cost_aggregate_raw(x[0], x[1][:, :, :-1], *x[2:])
    with pytest.raises(chop.InvalidArgumentError):
        chop.cost_aggregate_grad(*x, torch.zeros(1, 6, 8, 3, 4, device="cuda"),
                                 torch.zeros(1, 6, 8, 3, dtype=torch.int32, device="cuda"))
    # zero depth hypotheses: a successful no-op
    cost, mask = chop.cost_aggregate_raw(x[0], x[1], x[2], x[3][:, :0], x[4], x[5])
    assert cost.shape == (1, 6, 8, 0) and mask.shape == (1, 6, 8, 0)


def test_mvsnet_stage_full_size(oracle):
    """The benchmark workload's tensors through CostAggregate (forward and backward)."""
    wl = make_workload(2, with_cost_grad=False)
    t = wl.tensors
    want_cost, want_mask = oracle.cost_aggregate_fwd(*_args(t), "MEAN", threads=8)
    cost, mask = chop.cost_aggregate_raw(*_inputs(t), "MEAN")
    assert _lib.load().chop_last_kernel_family() == 2
    assert np.array_equal(host(mask), want_mask)
    assert_forward_close(host(cost), want_cost)
    cg = np.random.default_rng(9).standard_normal(want_cost.shape).astype(np.float32)
    want = oracle.cost_aggregate_bwd(*_args(t), cg, want_mask, "MEAN", threads=8)
    got = chop.cost_aggregate_grad(*_inputs(t), dev(cg), mask, "MEAN")
    assert _lib.load().chop_last_kernel_family() == 2
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)
