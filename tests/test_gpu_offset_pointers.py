"""Callers whose buffers do not start on a 16-byte boundary (a slice of a larger allocation:
legal for a `const float *`).  The tiled kernels use 16-byte accesses and decline such calls;
the strip and general kernels, the zero fill and the 16-bit narrowing pass must take them with
every pointer only element-aligned and give the oracle's results."""
import numpy as np
import pytest
import torch

import custom_helper_op_amd as chop
from custom_helper_op_amd import _lib
from custom_helper_op_amd.configs import reference_test_case
from gpu_util import assert_backward_close, assert_forward_close, dev, host, rms

pytestmark = pytest.mark.gpu

KEYS = ("ref", "src", "base_plane", "offsets", "Rs", "Ts")
TILED = 2


@pytest.fixture(autouse=True)
def _announce(request):
    print("\n[case] %s" % request.node.nodeid, flush=True)
    _lib.load().chop_set_kernel_family(0)
    yield


def shifted_empty(shape, dtype):
    """A contiguous tensor that starts one element past a 16-byte boundary."""
    n = int(np.prod(shape))
    flat = torch.empty(n + 8, dtype=dtype, device="cuda")
    assert flat.data_ptr() % 16 == 0
    out = flat[1:1 + n].view(*shape)
    assert out.data_ptr() % 16 == out.element_size() and out.is_contiguous()
    return out


def shifted(x, dtype=None):
    src = dev(x, dtype)
    out = shifted_empty(tuple(src.shape), src.dtype)
    out.copy_(src)
    return out


def _case(N, H, W, C, D, seed, camera=3):
    t = reference_test_case(camera, 1, N, H, W, C, D, np.float32, seed=seed)
    return tuple(t[k] for k in KEYS)


@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("which", ["all", "outputs"])
def test_cost_volume_f32_raw_abi(oracle, reduce, which):
    """CostVolume and its gradient through the C ABI, 32 channels (a shape the tiled kernels
    serve when aligned): every pointer shifted, or only the outputs."""
    lib = _lib.load()
    N, H, W, C, D = 2, 14, 22, 32, 11
    args = _case(N, H, W, C, D, seed=11)
    want_cost, want_mask = oracle.cost_volume_fwd(*args, reduce)
    put = shifted if which == "all" else dev
    ins = [put(x) for x in args]
    red = 0 if reduce == "MEAN" else 1
    cost = shifted_empty((1, H, W, D, C), torch.float32)
    mask = shifted_empty((1, H, W, D, 1 if red == 0 else C), torch.int32)
    stream = torch.cuda.current_stream().cuda_stream
    dims = (1, H, W, C, D, N, H, W)
    _lib.check(lib.chop_cost_volume_fwd_f32(stream, red, 1, *dims, *[x.data_ptr() for x in ins],
                                            cost.data_ptr(), mask.data_ptr()))
    assert lib.chop_last_kernel_family() != TILED
    assert np.array_equal(host(mask), want_mask)
    if red == 0:
        assert_forward_close(host(cost), want_cost)
    else:
        assert np.array_equal(host(cost), want_cost)
    cg = np.random.default_rng(12).standard_normal(want_cost.shape).astype(np.float32)
    want = oracle.cost_volume_bwd(*args, cg, want_mask, reduce)
    d_cg = put(cg)
    ref_grad = shifted_empty((1, H, W, C), torch.float32)
    src_grad = shifted_empty((1, N, H, W, C), torch.float32)
    bp_grad = shifted_empty((1, H, W, 1), torch.float32)
    for g in (ref_grad, src_grad, bp_grad):
        g.fill_(float("nan"))     # the library zeroes what it accumulates into
    _lib.check(lib.chop_cost_volume_bwd_f32(stream, red, 1, *dims, *[x.data_ptr() for x in ins],
                                            d_cg.data_ptr(), mask.data_ptr(), ref_grad.data_ptr(),
                                            src_grad.data_ptr(), bp_grad.data_ptr()))
    assert lib.chop_last_kernel_family() != TILED
    for g, w in zip((ref_grad, src_grad, bp_grad), want):
        assert_backward_close(host(g), w)


@pytest.mark.parametrize("storage", ["f16", "bf16"])
@pytest.mark.parametrize("which", ["all", "outputs"])
def test_cost_volume_16_raw_abi(oracle, storage, which):
    """The 16-bit entry points: float32 accumulation in the (aligned) workspace, then the
    narrowing pass into gradient buffers that start two bytes past a 16-byte boundary."""
    lib = _lib.load()
    td = torch.float16 if storage == "f16" else torch.bfloat16
    code = 1 if storage == "f16" else 2
    N, H, W, C, D = 3, 13, 21, 16, 10
    q = lambda x: dev(x, td).float().cpu().numpy()
    args = _case(N, H, W, C, D, seed=21)
    args = (q(args[0]), q(args[1])) + args[2:]
    want_cost, want_mask = oracle.cost_volume_fwd(*args, "MEAN")
    put = shifted if which == "all" else dev
    ins = [put(args[0], td), put(args[1], td)] + [put(x) for x in args[2:]]
    cost = shifted_empty((1, H, W, D, C), td)
    mask = shifted_empty((1, H, W, D, 1), torch.int32)
    stream = torch.cuda.current_stream().cuda_stream
    dims = (1, H, W, C, D, N, H, W)
    p = [x.data_ptr() for x in ins]
    _lib.check(lib.chop_cost_volume_fwd_16(stream, code, 0, 1, *dims, p[0], p[1], p[2], p[3], None,
                                           p[4], p[5], cost.data_ptr(), mask.data_ptr()))
    assert lib.chop_last_kernel_family() != TILED
    assert np.array_equal(host(mask), want_mask)
    eps = 2.0 ** -10 if storage == "f16" else 2.0 ** -7
    np.testing.assert_allclose(host(cost), want_cost, rtol=2 * eps, atol=1e-6)
    cg = q(np.random.default_rng(22).standard_normal(want_cost.shape).astype(np.float32))
    want = oracle.cost_volume_bwd(*args, cg, want_mask, "MEAN")
    d_cg = put(cg, td)
    ref_grad = shifted_empty((1, H, W, C), td)
    src_grad = shifted_empty((1, N, H, W, C), td)
    bp_grad = shifted_empty((1, H, W, 1), torch.float32)
    need = lib.chop_cost_volume_bwd16_workspace_bytes(1, H, W, C, N, H, W)
    ws = torch.empty(max(need, 256), dtype=torch.uint8, device="cuda")
    _lib.check(lib.chop_cost_volume_bwd_16(stream, code, 0, 1, *dims, p[0], p[1], p[2], p[3], None,
                                           p[4], p[5], d_cg.data_ptr(), mask.data_ptr(),
                                           ref_grad.data_ptr(), src_grad.data_ptr(),
                                           bp_grad.data_ptr(), ws.data_ptr(), need))
    assert lib.chop_last_kernel_family() != TILED
    for g, w in zip((ref_grad, src_grad), want[:2]):
        np.testing.assert_allclose(host(g), w, rtol=2 * eps, atol=2 * eps * max(rms(w), 1e-30))
    assert_backward_close(host(bp_grad), want[2])


def test_other_ops_shifted_inputs(oracle):
    """CostVolumeV2, CostAggregate, CostVolumeV3 and FeatureAggregate with every input shifted
    (the wrappers allocate the outputs)."""
    lib = _lib.load()
    N, H, W, C, D = 2, 12, 20, 16, 9
    args = _case(N, H, W, C, D, seed=31)
    ins = [shifted(x) for x in args]
    rng = np.random.default_rng(32)

    depth_grid = (args[2] + args[3][:, None, None, :]).astype(np.float32)
    v2 = (args[0], args[1], depth_grid, args[4], args[5])
    v2_ins = [ins[0], ins[1], shifted(depth_grid), ins[4], ins[5]]
    want_cost, want_mask = oracle.cost_volume_v2_fwd(*v2, "MEAN", 4)
    cost, mask = chop.cost_volume_v2_raw(*v2_ins, "MEAN", 4)
    assert lib.chop_last_kernel_family() != TILED
    assert np.array_equal(host(mask), want_mask)
    assert_forward_close(host(cost), want_cost, atol=1e-5)
    cg = rng.standard_normal(want_cost.shape).astype(np.float32)
    want = oracle.cost_volume_v2_bwd(*v2, cg, want_mask, "MEAN", 4)
    got = chop.cost_volume_grad_v2(*v2_ins, shifted(cg), shifted(want_mask), "MEAN", 4)
    assert lib.chop_last_kernel_family() != TILED
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)

    for reduce in ("MEAN", "MIN"):
        want_cost, want_mask = oracle.cost_aggregate_fwd(*args, reduce)
        cost, mask = chop.cost_aggregate_raw(*ins, reduce)
        assert lib.chop_last_kernel_family() != TILED
        assert np.array_equal(host(mask), want_mask)
        assert_forward_close(host(cost), want_cost, atol=1e-5)
        cg = rng.standard_normal(want_cost.shape).astype(np.float32)
        want = oracle.cost_aggregate_bwd(*args, cg, want_mask, reduce)
        got = chop.cost_aggregate_grad(*ins, shifted(cg), shifted(want_mask), reduce)
        assert lib.chop_last_kernel_family() != TILED
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)

        want_cost, want_mask = oracle.cost_volume_v3_fwd(*args, reduce, 4)
        cost, mask = chop.cost_volume_v3_raw(*ins, reduce, 4)
        assert lib.chop_last_kernel_family() != TILED
        assert np.array_equal(host(mask), want_mask)
        assert_forward_close(host(cost), want_cost, atol=1e-5)
        cg = rng.standard_normal(want_cost.shape).astype(np.float32)
        want = oracle.cost_volume_v3_bwd(*args, cg, want_mask, reduce, 4)
        got = chop.cost_volume_grad_v3(*ins, shifted(cg), shifted(want_mask), reduce, 4)
        assert lib.chop_last_kernel_family() != TILED
        for g, w in zip(got, want):
            assert_backward_close(host(g), w)

    feat_args = args[1:]
    want_feat, want_mask = oracle.feature_aggregate_fwd(*feat_args)
    feat, mask = chop.feature_aggregate_raw(*ins[1:])
    assert lib.chop_last_kernel_family() != TILED
    assert np.array_equal(host(mask), want_mask)
    assert np.array_equal(host(feat), want_feat)
    cg = rng.standard_normal(want_feat.shape).astype(np.float32)
    want = oracle.feature_aggregate_bwd(*feat_args, cg, want_mask)
    got = chop.feature_aggregate_grad(*ins[1:], shifted(cg), shifted(want_mask))
    assert lib.chop_last_kernel_family() != TILED
    for g, w in zip(got, want):
        assert_backward_close(host(g), w)
