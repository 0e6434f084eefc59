"""Source images of another size than the reference image, through the raw C ABI.

The reference's functors receive the source size separately from the output grid's
(cost_volume_kernels.cc:38-39, cost_aggregate_kernels.cc, cost_volume_kernels_v2.cc:38-39),
although its Compute methods only ever pass equal sizes; the C ABI accepts what the functors
accept.  The Python wrappers keep the reference's shape check, so these cases call the library
directly: CostVolume, CostVolumeV2 and CostAggregate, every kernel family, both reduces,
forward and backward against the oracle."""
import numpy as np
import pytest
import torch

from custom_helper_op_amd import _lib
from custom_helper_op_amd.configs import reference_test_case
from gpu_util import assert_backward_close, assert_forward_close, dev, host

pytestmark = pytest.mark.gpu

FAMILIES = [pytest.param(1, id="general"), pytest.param(2, id="strip"), pytest.param(0, id="auto")]
SIZES = [((12, 16), (17, 23)), ((14, 20), (9, 13))]   # (H, W) of the output grid, (srcH, srcW)


@pytest.fixture(autouse=True)
def _announce(request):
    print("\n[case] %s" % request.node.nodeid, flush=True)
    yield
    _lib.load().chop_set_kernel_family(0)


def _case(hw, src_hw, C, N, D, dtype, seed):
    """The reference tests' inputs for the output grid (camera case 1), source images of
    `src_hw` filled independently."""
    H, W = hw
    t = reference_test_case(1, 1, N, H, W, C, D, dtype, seed=seed)
    rng = np.random.default_rng(seed + 100)
    t["src"] = rng.standard_normal((1, N, src_hw[0], src_hw[1], C)).astype(dtype)
    # source intrinsics scaled to the source size (the samples then span the source image),
    # a small rotation about the optical axis, and a different offset per view
    Rs = t["Rs"].astype(np.float64)
    a = 0.06
    rot = np.array([[np.cos(a), -np.sin(a), 0.4], [np.sin(a), np.cos(a), -0.3], [0, 0, 1.0]])
    scale = np.diag([src_hw[1] / W, src_hw[0] / H, 1.0])
    t["Rs"] = (scale @ rot @ Rs).astype(dtype)
    t["Ts"] = (t["Ts"] + np.linspace(-25.0, 25.0, N)[None, :, None] * np.array([1.0, 0.6, 0.0])).astype(dtype)
    return t


def _family_served(family, tiled_shape):
    got = _lib.load().chop_last_kernel_family()
    want = {1: 1, 2: 3, 0: 2 if tiled_shape else 3}[family]
    assert got == want, (got, want)


def _p(t):
    return t.data_ptr()


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("hw,src_hw", SIZES)
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("C,dtype", [(8, np.float32), (5, np.float32), (8, np.float64)])
def test_cost_volume_other_source_size(oracle, family, hw, src_hw, reduce, C, dtype):
    lib = _lib.load()
    lib.chop_set_kernel_family(family)
    sfx = "f32" if dtype == np.float32 else "f64"
    tiled = C == 8 and dtype == np.float32
    N, D = 2, 11
    t = _case(hw, src_hw, C, N, D, dtype, seed=C)
    args = tuple(t[k] for k in ("ref", "src", "base_plane", "offsets", "Rs", "Ts"))
    want_cost, want_mask = oracle.cost_volume_fwd(*args, reduce)
    assert (want_mask != (0 if reduce == "MEAN" else -1)).mean() > 0.2   # the case exercises the taps
    d = [dev(x) for x in args]
    H, W = hw
    red = 0 if reduce == "MEAN" else 1
    dims = (1, H, W, C, D, N, src_hw[0], src_hw[1])
    cost = torch.empty(want_cost.shape, dtype=d[0].dtype, device="cuda")
    mask = torch.empty(want_mask.shape, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    _lib.check(getattr(lib, "chop_cost_volume_fwd_" + sfx)(stream, red, 1, *dims, *map(_p, d), _p(cost),
                                                          _p(mask)))
    _family_served(family, tiled)
    assert np.array_equal(host(mask), want_mask)
    if tiled and family == 0 and reduce == "MEAN":
        assert_forward_close(host(cost), want_cost)
    else:
        assert np.array_equal(host(cost), want_cost)
    cg = np.random.default_rng(C).standard_normal(want_cost.shape).astype(dtype)
    want = oracle.cost_volume_bwd(*args, cg, want_mask, reduce)
    grads = [torch.empty_like(d[0]), torch.empty_like(d[1]), torch.empty_like(d[2])]
    _lib.check(getattr(lib, "chop_cost_volume_bwd_" + sfx)(stream, red, 1, *dims, *map(_p, d),
                                                          _p(dev(cg)), _p(mask), *map(_p, grads)))
    _family_served(family, tiled)
    assert grads[1].shape == (1, N, src_hw[0], src_hw[1], C)
    for g, w in zip(grads, want):
        assert_backward_close(host(g), w)


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("hw,src_hw", SIZES)
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("C,groups,dtype", [(8, 4, np.float32), (6, 3, np.float32), (8, 2, np.float64)])
def test_cost_volume_v2_other_source_size(oracle, family, hw, src_hw, reduce, C, groups, dtype):
    lib = _lib.load()
    lib.chop_set_kernel_family(family)
    sfx = "f32" if dtype == np.float32 else "f64"
    tiled = C == 8 and dtype == np.float32
    N, D = 2, 7
    t = _case(hw, src_hw, C, N, D, dtype, seed=C + groups)
    depth_grid = (t["base_plane"] + t["offsets"][:, None, None, :]).astype(dtype)
    depth_grid = depth_grid * (1 + 0.01 * np.random.default_rng(3).standard_normal(depth_grid.shape)).astype(dtype)
    args = (t["ref"], t["src"], depth_grid, t["Rs"], t["Ts"])
    want_cost, want_mask = oracle.cost_volume_v2_fwd(*args, reduce, groups)
    d = [dev(x) for x in args]
    H, W = hw
    red = 0 if reduce == "MEAN" else 1
    dims = (1, H, W, C, D, N, src_hw[0], src_hw[1])
    cost = torch.empty(want_cost.shape, dtype=d[0].dtype, device="cuda")
    mask = torch.empty(want_mask.shape, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    _lib.check(getattr(lib, "chop_cost_volume_v2_fwd_" + sfx)(stream, red, 1, *dims, groups,
                                                             *map(_p, d), _p(cost), _p(mask)))
    _family_served(family, tiled)
    assert np.array_equal(host(mask), want_mask)
    if tiled and family == 0 and reduce == "MEAN":
        assert_forward_close(host(cost), want_cost, atol=1e-5)
    else:
        assert np.array_equal(host(cost), want_cost)
    cg = np.random.default_rng(C).standard_normal(want_cost.shape).astype(dtype)
    want = oracle.cost_volume_v2_bwd(*args, cg, want_mask, reduce, groups)
    grads = [torch.empty_like(d[0]), torch.empty_like(d[1]), torch.empty_like(d[2])]
    _lib.check(getattr(lib, "chop_cost_volume_v2_bwd_" + sfx)(stream, red, 1, *dims, groups,
                                                             *map(_p, d), _p(dev(cg)), _p(mask),
                                                             *map(_p, grads)))
    _family_served(family, tiled)
    for g, w in zip(grads, want):
        assert_backward_close(host(g), w)


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("hw,src_hw", SIZES)
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("C,dtype", [(8, np.float32), (5, np.float32), (8, np.float64)])
def test_cost_aggregate_other_source_size(oracle, family, hw, src_hw, reduce, C, dtype):
    lib = _lib.load()
    lib.chop_set_kernel_family(family)
    sfx = "f32" if dtype == np.float32 else "f64"
    tiled = C == 8 and dtype == np.float32
    N, D = 3, 11
    t = _case(hw, src_hw, C, N, D, dtype, seed=C + 1)
    args = tuple(t[k] for k in ("ref", "src", "base_plane", "offsets", "Rs", "Ts"))
    want_cost, want_mask = oracle.cost_aggregate_fwd(*args, reduce)
    d = [dev(x) for x in args]
    H, W = hw
    red = 0 if reduce == "MEAN" else 1
    dims = (1, H, W, C, D, N, src_hw[0], src_hw[1])
    cost = torch.empty(want_cost.shape, dtype=d[0].dtype, device="cuda")
    mask = torch.empty(want_mask.shape, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    _lib.check(getattr(lib, "chop_cost_aggregate_fwd_" + sfx)(stream, red, 1, *dims, *map(_p, d),
                                                             _p(cost), _p(mask)))
    _family_served(family, tiled)
    assert np.array_equal(host(mask), want_mask)
    if tiled and family == 0 and reduce == "MEAN":
        assert_forward_close(host(cost), want_cost)
    else:
        assert np.array_equal(host(cost), want_cost)
    cg = np.random.default_rng(C).standard_normal(want_cost.shape).astype(dtype)
    want = oracle.cost_aggregate_bwd(*args, cg, want_mask, reduce)
    grads = [torch.empty_like(d[0]), torch.empty_like(d[1]), torch.empty_like(d[2])]
    _lib.check(getattr(lib, "chop_cost_aggregate_bwd_" + sfx)(stream, red, 1, *dims, *map(_p, d),
                                                             _p(dev(cg)), _p(mask), *map(_p, grads)))
    _family_served(family, tiled)
    for g, w in zip(grads, want):
        assert_backward_close(host(g), w)
