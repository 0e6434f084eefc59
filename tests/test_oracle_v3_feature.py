"""Pins the CPU oracle's CostVolumeV3 and FeatureAggregate functions (CPU only).

The reference tests these ops like the others (cost_volume_v3_op_test.py:136-265 and
feature_aggregate_op_test.py:173-267): unseeded inputs against a TensorFlow composite built
on ``tfa.image.resampler``, and finite differences for the gradients.  No vectors exist, so
the oracle is pinned by
 (1) the float64 numpy composite (independent projection order, whole-array bilinear
     gather) with the reference's shapes, camera cases and masking,
 (2) the already pinned V2 oracle on the special cases that reduce to it: V3 with one group
     is the V2 correlation with one group; FeatureAggregate of one view is the V2
     correlation against a reference image of ones with one channel per group (bit-exact),
 (3) scalar brute-force loops on tiny inputs, including data whose correlations are all
     negative (the seed ``numeric_limits<T>::min()`` then wins) and exact ties,
 (4) central finite differences of the forward in float64.
"""
import ctypes

import numpy as np
import pytest
from scipy.spatial.transform import Rotation

import composite
from custom_helper_op_amd.configs import reference_test_case
from test_oracle_backward import _close, _numeric

REF_SHAPES = [(1, 1, 12, 16, 5), (1, 2, 12, 16, 9), (2, 2, 12, 18, 10), (2, 3, 12, 16, 6)]
TINY = np.finfo(np.float64).tiny


def _args(t):
    return (t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])


def _warped(t, half=True):
    depth = t["base_plane"] + t["offsets"][:, None, None, :]
    xy, front = composite.sampler_coordinates(t["Rs"], t["Ts"], depth, half)
    valid = composite.validity(xy, front, t["src"].shape[2], t["src"].shape[3])
    lim = np.array([t["src"].shape[3] - 1, t["src"].shape[2] - 1], dtype=np.float64)
    safe = ~((np.abs(xy) < 1e-9) | (np.abs(xy - lim) < 1e-9)).any(-1)     # [B,N,H,W,D]
    return composite.warp_views(t["src"], xy, valid), valid, safe


# ---- CostVolumeV3 -------------------------------------------------------------------------
@pytest.mark.parametrize("shape", REF_SHAPES)
@pytest.mark.parametrize("case", [1, 2, 3])
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_v3_matches_composite(oracle, shape, case, reduce):
    B, N, H, W, D = shape
    C, G = 9, 3                                    # the reference tests use C=9, groups=3
    t = reference_test_case(case, B, N, H, W, C, D, np.float64, seed=40 + 10 * case + B + N)
    cost, mask = oracle.cost_volume_v3_fwd(*_args(t), reduce, G)
    assert cost.shape == (B, H, W, D, 1)
    assert mask.shape == (B, H, W, D, 1 if reduce == "MEAN" else 3)
    warped, valid, safe = _warped(t)
    wg = warped.reshape(B, N, H, W, D, G, C // G)
    rg = t["ref"].reshape(B, H, W, G, C // G)
    # corr[b,n,h,w,d,gi,gs] = <ref group gi, source group gs>
    corr = np.einsum("bhwik,bnhwdsk->bnhwdis", rg, wg)
    best = corr.max(axis=(-2, -1))                                     # [B,N,H,W,D]
    safe = safe.all(1)
    cnt = valid.sum(1)
    if reduce == "MEAN":
        want = (best * valid).sum(1) / np.maximum(cnt, 1)
        assert np.array_equal(mask[..., 0][safe], cnt[safe])
        np.testing.assert_allclose(cost[..., 0][safe], want[safe], rtol=1e-9, atol=1e-12)
        assert np.all(cost[..., 0][safe & (cnt == 0)] == 0)
    else:
        big = np.where(valid, best, -np.inf)
        top = big.max(1)
        has = safe & (cnt > 0)
        np.testing.assert_allclose(cost[..., 0][has], top[has], rtol=1e-9, atol=1e-12)
        n_win = big.argmax(1)
        flat = np.take_along_axis(corr, n_win[:, None, ..., None, None], 1)[:, 0]
        pair = flat.reshape(flat.shape[:-2] + (-1,)).argmax(-1)
        assert np.array_equal(mask[..., 0][has], n_win[has])
        assert np.array_equal(mask[..., 1][has], (pair // G)[has])     # reference group
        assert np.array_equal(mask[..., 2][has], (pair % G)[has])      # source group
        none = safe & (cnt == 0)
        assert np.all(mask[none] == -1) and np.all(cost[..., 0][none] == 0)


def _brute_v3(ref, src, depth, Rs, Ts, reduce, groups, half):
    B, H, W, C = ref.shape
    N, sH, sW = src.shape[1:4]
    D = depth.shape[-1]
    sub = C // groups
    cost = np.zeros((B, H, W, D, 1))
    mask = np.zeros((B, H, W, D, 1 if reduce == "MEAN" else 3), np.int32)
    o = 0.5 if half else 0.0
    for b in range(B):
        for h in range(H):
            for w in range(W):
                for d in range(D):
                    total, used, top, win = 0.0, 0, TINY, (-1, -1, -1)
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
                        view_top = TINY
                        for gs in range(groups):
                            for gi in range(groups):
                                v = float(np.dot(s[gs * sub:(gs + 1) * sub], ref[b, h, w, gi * sub:(gi + 1) * sub]))
                                view_top = max(view_top, v)
                                if v > top:
                                    top, win = v, (n, gi, gs)
                        total += view_top
                        used += 1
                    if reduce == "MEAN":
                        mask[b, h, w, d, 0] = used
                        cost[b, h, w, d, 0] = total / used if used else 0.0
                    else:
                        mask[b, h, w, d] = win
                        cost[b, h, w, d, 0] = top if win[0] >= 0 else 0.0
    return cost, mask


@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("half", [True, False])
@pytest.mark.parametrize("sign", ["mixed", "negative"])
def test_v3_brute_force_tiny(oracle, reduce, half, sign):
    rng = np.random.default_rng(11)
    B, N, H, W, C, D, G = 2, 3, 5, 6, 6, 3, 3
    ref = rng.normal(size=(B, H, W, C))
    src = rng.normal(size=(B, N, H, W, C))
    if sign == "negative":       # every correlation is negative: the seed survives
        ref, src = np.abs(ref) + 0.1, -np.abs(src) - 0.1
    base = rng.uniform(2, 3, (B, H, W, 1))
    offsets = rng.uniform(-0.5, 0.5, (B, D))
    Rs = np.empty((B, N, 3, 3))
    Ts = rng.uniform(-1.5, 1.5, (B, N, 3))
    for b in range(B):
        for n in range(N):
            Rs[b, n] = Rotation.from_euler("xyz", rng.uniform(-4, 4, 3), degrees=True).as_matrix()
    Ts[0, 0, 2] = -10.0
    cost, mask = oracle.cost_volume_v3_fwd(ref, src, base, offsets, Rs, Ts, reduce, G, half)
    bc, bm = _brute_v3(ref, src, base + offsets[:, None, None, :], Rs, Ts, reduce, G, half)
    assert np.array_equal(mask, bm)
    np.testing.assert_allclose(cost, bc, rtol=1e-10, atol=1e-300)
    if sign == "negative" and reduce == "MIN":
        assert np.all(mask == -1) and np.all(cost == 0)
    if sign == "negative" and reduce == "MEAN":
        assert np.all(cost[mask > 0] == TINY)


def test_v3_ties_keep_the_first_pair(oracle):
    # identical channel groups on both sides: every pair ties, the first (gs=0, gi=0) of the
    # first accepted view must be recorded (strict "<" at cost_volume_kernels_gpu_v3.cu.cc:243)
    t = reference_test_case(1, 1, 2, 8, 9, 6, 3, np.float64, seed=2)
    t["ref"][..., 2:4] = t["ref"][..., 0:2]
    t["ref"][..., 4:6] = t["ref"][..., 0:2]
    t["src"][..., 2:4] = t["src"][..., 0:2]
    t["src"][..., 4:6] = t["src"][..., 0:2]
    t["src"][:, 1] = t["src"][:, 0]
    cost, mask = oracle.cost_volume_v3_fwd(*_args(t), "MIN", 3)
    won = mask[..., 0] >= 0
    assert won.any()
    assert np.all(mask[won] == 0)


@pytest.mark.parametrize("shape", REF_SHAPES[1:])
@pytest.mark.parametrize("case", [1, 3])
def test_v3_single_group_is_v2(oracle, shape, case):
    B, N, H, W, D = shape
    C = 5
    t = reference_test_case(case, B, N, H, W, C, D, np.float64, seed=51 + case + B + N)
    depth_grid = t["base_plane"] + t["offsets"][:, None, None, :]
    for reduce in ("MEAN", "MIN"):
        cost, mask = oracle.cost_volume_v3_fwd(*_args(t), reduce, 1)
        c2, m2 = oracle.cost_volume_v2_fwd(t["ref"], t["src"], depth_grid, t["Rs"], t["Ts"], reduce, 1)
        assert np.array_equal(mask[..., :1], m2)
        ok = (m2 > 0) if reduce == "MEAN" else (m2 >= 0)
        assert np.array_equal(np.where(ok, cost, 0), np.where(ok, c2, 0))  # features are positive
        if reduce == "MIN":
            assert np.all(mask[..., 1:][m2[..., 0] >= 0] == 0)
        cg = np.random.default_rng(3).normal(size=cost.shape)
        rg, sg, bg = oracle.cost_volume_v3_bwd(*_args(t), cg, mask, reduce, 1)
        rg2, sg2, dg2 = oracle.cost_volume_v2_bwd(t["ref"], t["src"], depth_grid, t["Rs"], t["Ts"],
                                                  cg, m2, reduce, 1)
        np.testing.assert_allclose(rg, rg2, rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(sg, sg2, rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(bg[..., 0], dg2.sum(-1), rtol=1e-10, atol=1e-12)


def _loss_v3(oracle, t, reduce, groups):
    cost, mask = oracle.cost_volume_v3_fwd(*_args(t), reduce, groups)
    ok = (mask[..., :1] > 0) if reduce == "MEAN" else (mask[..., :1] >= 0)
    return np.where(ok, cost, 0.0).mean(), mask, cost.size


@pytest.mark.parametrize("shape,reduce", [(s, "MEAN") for s in REF_SHAPES[:2]] +
                         [(s, "MIN") for s in REF_SHAPES[1:3]])
@pytest.mark.parametrize("case", [1, 3])
def test_v3_gradient_against_finite_differences(oracle, shape, case, reduce):
    B, N, H, W, D = shape
    t = reference_test_case(case, B, N, H, W, 6, D, np.float64, seed=90 + 7 * case + B + 2 * N)
    fn = lambda tt: _loss_v3(oracle, tt, reduce, 3)
    _, mask, numel = fn(t)
    ok = (mask[..., :1] > 0) if reduce == "MEAN" else (mask[..., :1] >= 0)
    cg = np.where(ok, 1.0 / numel, 0.0)
    rg, sg, bg = oracle.cost_volume_v3_bwd(*_args(t), cg, mask, reduce, 3)
    # the correlation is bilinear in (ref, src): central differences are exact unless the
    # winning pair changes inside the step
    _close(rg, _numeric(fn, t, "ref", 1e-5))
    _close(sg, _numeric(fn, t, "src", 1e-5))
    _close(bg, _numeric(fn, t, "base_plane", 1e-6), rtol=2e-4)
    assert np.abs(sg).max() > 0 and np.abs(rg).max() > 0


def test_v3_status_codes(oracle):
    fn = oracle.lib().chop_oracle_cost_volume_v3_fwd_f32
    z = ctypes.c_void_p(0)

    def call(reduce, B, C, G):
        dims = [ctypes.c_int64(v) for v in (B, 2, 2, C, 1, 1, 2, 2, G)]
        return fn(reduce, 1, *dims, z, z, z, z, z, z, z, z, 1)

    assert call(7, 0, 4, 2) == 3          # bad reduce
    assert call(0, -1, 4, 2) == 2         # bad dims
    assert call(0, 0, 4, 3) == 4          # groups does not divide C
    assert call(0, 0, 18, 2) == 4         # more than 8 channels per group (cost_volume_v3.h:35)
    assert call(0, 0, 16, 2) == 0         # empty: no-op


# ---- FeatureAggregate ---------------------------------------------------------------------
@pytest.mark.parametrize("shape", REF_SHAPES)
@pytest.mark.parametrize("case", [0, 1, 2, 3])
def test_feature_matches_composite(oracle, shape, case):
    B, N, H, W, D = shape
    C = 3
    t = reference_test_case(case, B, N, H, W, C, D, np.float64, seed=60 + 10 * case + B + N)
    mapped, mask = oracle.feature_aggregate_fwd(t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
    assert mapped.shape == (B, H, W, D, N, C) and mask.shape == (B, H, W, D, N, 1)
    warped, valid, safe = _warped(t)
    want = np.where(valid[..., None], warped, 0.0).transpose(0, 2, 3, 4, 1, 5)
    safe = safe.transpose(0, 2, 3, 4, 1)
    assert np.array_equal(mask[..., 0][safe], valid.transpose(0, 2, 3, 4, 1)[safe].astype(np.int32))
    np.testing.assert_allclose(mapped[safe], want[safe], rtol=1e-10, atol=1e-12)
    assert np.all(mapped[mask[..., 0] == 0] == 0)
    assert set(np.unique(mask)) <= {0, 1}


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("half", [True, False])
def test_feature_is_v2_against_ones(oracle, dtype, half):
    # one channel per group and a reference of ones: the V2 correlation of a single view is
    # 0 + sample*1, i.e. the sample itself, rounding included
    B, N, H, W, C, D = 2, 3, 10, 12, 4, 5
    t = reference_test_case(3, B, N, H, W, C, D, dtype, seed=8)
    mapped, mask = oracle.feature_aggregate_fwd(t["src"], t["base_plane"], t["offsets"], t["Rs"],
                                                t["Ts"], half)
    depth_grid = t["base_plane"] + t["offsets"][:, None, None, :]
    ones = np.ones((B, H, W, C), dtype)
    for n in range(N):
        c2, m2 = oracle.cost_volume_v2_fwd(ones, t["src"][:, n:n + 1], depth_grid, t["Rs"][:, n:n + 1],
                                           t["Ts"][:, n:n + 1], "MEAN", C, half)
        assert np.array_equal(mask[..., n, :], m2)
        assert np.array_equal(mapped[..., n, :], c2)
    assert mask.any() and not mask.all()


def test_feature_output_size_follows_base_plane(oracle):
    # the output grid is base_plane's; the source images may be larger or smaller
    # (feature_aggregate_kernels.cc:72-81)
    rng = np.random.default_rng(4)
    B, N, sH, sW, C, H, W, D = 1, 2, 9, 14, 3, 5, 6, 4
    src = rng.normal(size=(B, N, sH, sW, C))
    base = rng.uniform(2, 3, (B, H, W, 1))
    offsets = rng.uniform(-0.2, 0.2, (B, D))
    Rs = np.tile(np.eye(3)[None, None], (B, N, 1, 1))
    Ts = rng.uniform(0.5, 6.0, (B, N, 3))
    mapped, mask = oracle.feature_aggregate_fwd(src, base, offsets, Rs, Ts)
    assert mapped.shape == (B, H, W, D, N, C)
    depth = base + offsets[:, None, None, :]
    xy, front = composite.sampler_coordinates(Rs, Ts, depth, True)
    valid = composite.validity(xy, front, sH, sW)
    want = np.where(valid[..., None], composite.warp_views(src, xy, valid), 0.0).transpose(0, 2, 3, 4, 1, 5)
    assert np.array_equal(mask[..., 0], valid.transpose(0, 2, 3, 4, 1).astype(np.int32))
    np.testing.assert_allclose(mapped, want, rtol=1e-10, atol=1e-12)
    assert mask.any()


def _loss_feature(oracle, t, weights):
    mapped, mask = oracle.feature_aggregate_fwd(t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
    return float((mapped * weights).sum()), mask, mapped.size


@pytest.mark.parametrize("shape", REF_SHAPES[:3])
@pytest.mark.parametrize("case", [1, 3])
def test_feature_gradient_against_finite_differences(oracle, shape, case):
    B, N, H, W, D = shape
    C = 3
    t = reference_test_case(case, B, N, H, W, C, D, np.float64, seed=120 + 7 * case + B + 2 * N)
    weights = np.random.default_rng(9).normal(size=(B, H, W, D, N, C))
    fn = lambda tt: _loss_feature(oracle, tt, weights)
    _, mask, _ = fn(t)
    sg, bg = oracle.feature_aggregate_bwd(t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"],
                                          weights, mask)
    _close(sg, _numeric(fn, t, "src", 1e-3))              # linear in src: exact
    _close(bg, _numeric(fn, t, "base_plane", 1e-6), rtol=2e-4)
    assert np.abs(sg).max() > 0 and np.abs(bg).max() > 0
    # a masked-out sample receives nothing: zero weights where the mask is 1 kill the gradient
    sg0, bg0 = oracle.feature_aggregate_bwd(t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"],
                                            weights * (mask == 0), mask)
    assert not sg0.any() and not bg0.any()


def test_feature_gradient_is_v2_gradient_against_ones(oracle):
    B, N, H, W, C, D = 1, 2, 8, 10, 4, 5
    t = reference_test_case(3, B, N, H, W, C, D, np.float64, seed=17)
    g = np.random.default_rng(2).normal(size=(B, H, W, D, N, C))
    _, mask = oracle.feature_aggregate_fwd(t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
    sg, bg = oracle.feature_aggregate_bwd(t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"], g, mask)
    depth_grid = t["base_plane"] + t["offsets"][:, None, None, :]
    ones = np.ones((B, H, W, C))
    bsum = 0.0
    for n in range(N):
        _, sg2, dg2 = oracle.cost_volume_v2_bwd(ones, t["src"][:, n:n + 1], depth_grid, t["Rs"][:, n:n + 1],
                                                t["Ts"][:, n:n + 1], g[..., n, :], mask[..., n, :], "MEAN", C)
        np.testing.assert_allclose(sg[:, n], sg2[:, 0], rtol=1e-12, atol=1e-13)
        bsum = bsum + dg2.sum(-1)
    np.testing.assert_allclose(bg[..., 0], bsum, rtol=1e-10, atol=1e-12)


def test_feature_status_codes(oracle):
    fn = oracle.lib().chop_oracle_feature_aggregate_fwd_f64
    z = ctypes.c_void_p(0)
    dims = [ctypes.c_int64(v) for v in (-1, 2, 2, 1, 1, 1, 2, 2)]
    assert fn(1, *dims, z, z, z, z, z, z, z, 1) == 2
    dims[0] = ctypes.c_int64(0)
    assert fn(1, *dims, z, z, z, z, z, z, z, 1) == 0
