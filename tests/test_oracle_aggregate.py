"""Pins the CPU oracle's CostAggregate functions (CPU only).

The reference's own test of this op (cost_aggregate_op_test.py) follows the cost-volume
tests: unseeded inputs against a TensorFlow composite, and finite differences for the
gradient.  Here the aggregate oracle is pinned by
 (1) the independently pinned cost-volume oracle: MEAN aggregate = mean over channels of
     the MEAN cost volume, and its gradient = the cost-volume gradient fed the upstream
     gradient broadcast over channels and divided by C,
 (2) the float64 composite (sum of squared differences over channels, mean / min over
     the valid views), which also pins the MIN reduce and its winning view,
 (3) a scalar brute-force loop on tiny inputs, and
 (4) central finite differences of the forward in float64 for both reduces.
"""
import numpy as np
import pytest
from scipy.spatial.transform import Rotation

import composite
from custom_helper_op_amd.configs import reference_test_case
from test_oracle_backward import _close, _numeric

REF_SHAPES = [(1, 1, 12, 16, 5), (1, 2, 12, 16, 9), (2, 2, 12, 18, 10), (2, 3, 12, 16, 6)]


def _args(t):
    return (t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])


@pytest.mark.parametrize("shape", REF_SHAPES)
@pytest.mark.parametrize("case", [0, 1, 2, 3])
def test_mean_is_channel_mean_of_cost_volume(oracle, shape, case):
    B, N, H, W, D = shape
    for dtype, tol in ((np.float64, 1e-12), (np.float32, 2e-6)):
        t = reference_test_case(case, B, N, H, W, 5, D, dtype, seed=3 * case + B + N)
        cost, mask = oracle.cost_aggregate_fwd(*_args(t), "MEAN")
        vol, vmask = oracle.cost_volume_fwd(*_args(t), "MEAN")
        assert cost.shape == (B, H, W, D) and mask.shape == (B, H, W, D)
        assert np.array_equal(mask, vmask[..., 0])
        np.testing.assert_allclose(cost, vol.astype(np.float64).mean(-1), rtol=tol, atol=tol)
        assert np.all(cost[mask == 0] == 0)


@pytest.mark.parametrize("shape", REF_SHAPES)
@pytest.mark.parametrize("case", [1, 2, 3])
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_matches_composite(oracle, shape, case, reduce):
    B, N, H, W, D = shape
    C = 3
    t = reference_test_case(case, B, N, H, W, C, D, np.float64, seed=20 + 10 * case + B + N)
    cost, mask = oracle.cost_aggregate_fwd(*_args(t), reduce)
    depth = t["base_plane"] + t["offsets"][:, None, None, :]
    _, valid, xy, per_view = composite.cost_volume_composite(t["ref"], t["src"], depth, t["Rs"],
                                                             t["Ts"], "MEAN")
    lim = np.array([W - 1, H - 1], dtype=np.float64)
    safe = ~((np.abs(xy) < 1e-9) | (np.abs(xy - lim) < 1e-9)).any(-1).any(1)
    ssd = per_view.sum(-1)                      # [B,N,H,W,D] sum over channels
    cnt = valid.sum(1)
    if reduce == "MEAN":
        want = (ssd * valid).sum(1) / (np.maximum(cnt, 1) * C)
        assert np.array_equal(mask[safe], cnt[safe])
        np.testing.assert_allclose(cost[safe], want[safe], rtol=1e-9, atol=1e-12)
    else:
        big = np.where(valid, ssd, np.inf)
        best = big.min(1)
        arg = np.where(np.isfinite(best), big.argmin(1), -1)
        has = safe & (cnt > 0)
        np.testing.assert_allclose(cost[has], best[has] / C, rtol=1e-9, atol=1e-12)
        assert np.array_equal(mask[has], arg[has])
        none = safe & (cnt == 0)
        assert np.all(cost[none] == 0) and np.all(mask[none] == -1)


def _brute(ref, src, depth, Rs, Ts, reduce, half):
    B, H, W, C = ref.shape
    N, sH, sW = src.shape[1:4]
    D = depth.shape[-1]
    cost = np.zeros((B, H, W, D))
    mask = np.zeros((B, H, W, D), np.int32)
    o = 0.5 if half else 0.0
    for b in range(B):
        for h in range(H):
            for w in range(W):
                for d in range(D):
                    best, used = (0.0, 0) if reduce == "MEAN" else (np.inf, -1)
                    for n in range(N):
                        p = Rs[b, n] @ np.array([w + o, h + o, 1.0]) * depth[b, h, w, d] + Ts[b, n]
                        if p[2] <= 0:
                            continue
                        x, y = p[0] / p[2] - o, p[1] / p[2] - o
                        if not (0 < y < sH - 1 and 0 < x < sW - 1):
                            continue
                        fy, fx = int(y), int(x)
                        dy, dx = y - fy, x - fx
                        s = ((1 - dy) * (1 - dx) * src[b, n, fy, fx] + (1 - dy) * dx * src[b, n, fy, fx + 1]
                             + dy * dx * src[b, n, fy + 1, fx + 1] + dy * (1 - dx) * src[b, n, fy + 1, fx])
                        ssd = float(((s - ref[b, h, w]) ** 2).sum())
                        if reduce == "MEAN":
                            best += ssd
                            used += 1
                        elif best > ssd:
                            best, used = ssd, n
                    mask[b, h, w, d] = used
                    if reduce == "MEAN":
                        cost[b, h, w, d] = best / (used * C) if used > 0 else 0.0
                    else:
                        cost[b, h, w, d] = best / C if used >= 0 else 0.0
    return cost, mask


@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("half", [True, False])
def test_brute_force_tiny(oracle, reduce, half):
    rng = np.random.default_rng(5)
    B, N, H, W, C, D = 2, 3, 5, 6, 4, 3
    ref = rng.normal(size=(B, H, W, C))
    src = rng.normal(size=(B, N, H, W, C))
    base = rng.uniform(2, 3, (B, H, W, 1))
    offsets = rng.uniform(-0.5, 0.5, (B, D))
    Rs = np.empty((B, N, 3, 3))
    Ts = rng.uniform(-1.5, 1.5, (B, N, 3))
    for b in range(B):
        for n in range(N):
            Rs[b, n] = Rotation.from_euler("xyz", rng.uniform(-4, 4, 3), degrees=True).as_matrix()
    Ts[0, 0, 2] = -10.0  # one view entirely behind the reference camera
    cost, mask = oracle.cost_aggregate_fwd(ref, src, base, offsets, Rs, Ts, reduce, half)
    bc, bm = _brute(ref, src, base + offsets[:, None, None, :], Rs, Ts, reduce, half)
    assert np.array_equal(mask, bm)
    np.testing.assert_allclose(cost, bc, rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("shape", REF_SHAPES[1:])
@pytest.mark.parametrize("case", [1, 3])
def test_mean_gradient_is_cost_volume_gradient(oracle, shape, case):
    B, N, H, W, D = shape
    C = 4
    t = reference_test_case(case, B, N, H, W, C, D, np.float64, seed=31 + case + B + N)
    rng = np.random.default_rng(1)
    _, mask = oracle.cost_aggregate_fwd(*_args(t), "MEAN")
    cg = rng.normal(size=(B, H, W, D))
    got = oracle.cost_aggregate_bwd(*_args(t), cg, mask, "MEAN")
    vol_cg = np.repeat(cg[..., None] / C, C, axis=-1)
    want = oracle.cost_volume_bwd(*_args(t), vol_cg, mask[..., None], "MEAN")
    for g, w in zip(got, want):
        np.testing.assert_allclose(g, w, rtol=1e-12, atol=1e-13)
    # threads only change the order in which src_grad ranges are summed
    got4 = oracle.cost_aggregate_bwd(*_args(t), cg, mask, "MEAN", threads=4)
    assert np.array_equal(got4[0], got[0]) and np.array_equal(got4[2], got[2])
    np.testing.assert_allclose(got4[1], got[1], rtol=1e-12, atol=1e-13)


def _loss(oracle, t, reduce):
    cost, mask = oracle.cost_aggregate_fwd(*_args(t), reduce)
    ok = (mask > 0) if reduce == "MEAN" else (mask >= 0)
    return np.where(ok, cost, 0.0).mean(), mask, cost.size


@pytest.mark.parametrize("shape,reduce", [(s, "MEAN") for s in REF_SHAPES[:2]] +
                         [(s, "MIN") for s in REF_SHAPES[1:3]])
@pytest.mark.parametrize("case", [1, 3])
def test_gradient_against_finite_differences(oracle, shape, case, reduce):
    B, N, H, W, D = shape
    t = reference_test_case(case, B, N, H, W, 4, D, np.float64, seed=70 + 7 * case + B + 2 * N)
    fn = lambda tt: _loss(oracle, tt, reduce)
    _, mask, numel = fn(t)
    ok = (mask > 0) if reduce == "MEAN" else (mask >= 0)
    cg = np.where(ok, 1.0 / numel, 0.0)
    rg, sg, bg = oracle.cost_aggregate_bwd(*_args(t), cg, mask, reduce)
    _close(rg, _numeric(fn, t, "ref", 1e-4))
    _close(sg, _numeric(fn, t, "src", 1e-4))
    _close(bg, _numeric(fn, t, "base_plane", 1e-6), rtol=2e-4)
    assert np.abs(sg).max() > 0
    # conservation: every g goes to ref_grad as -g and to four taps whose weights sum to 1
    assert abs(rg.sum() + sg.sum()) < 1e-9 * max(1.0, np.abs(sg).sum())


def test_status_codes(oracle):
    import ctypes
    fn = oracle.lib().chop_oracle_cost_aggregate_fwd_f32
    z = ctypes.c_void_p(0)
    dims = [ctypes.c_int64(v) for v in (1, 2, 2, 1, 1, 1, 2, 2)]
    assert fn(7, 1, *dims, z, z, z, z, z, z, z, z, 1) == 3          # bad reduce
    dims[0] = ctypes.c_int64(-1)
    assert fn(0, 1, *dims, z, z, z, z, z, z, z, z, 1) == 2          # bad dims
    dims[0] = ctypes.c_int64(0)
    assert fn(0, 1, *dims, z, z, z, z, z, z, z, z, 1) == 0          # empty: no-op
