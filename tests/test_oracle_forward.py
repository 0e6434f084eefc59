"""Pins the CPU oracle's forward functions (CPU only).

The reference ships no golden vectors for this path (its tests draw unseeded random
inputs and compare with a TensorFlow composite), so the oracle is pinned by
 (1) an independent float64 composite restating that TensorFlow composite, with the
     reference tests' own shapes, camera cases, masking and rtol=1e-5
     (cost_volume_op_test.py:174-263, cost_volume_v2_op_test.py:174-263),
 (2) scipy's order-1 ``map_coordinates`` as a library twin of the bilinear gather,
 (3) closed-form camera set-ups (integer shifts, a 90 degree rotation),
 (4) a scalar brute-force loop on tiny inputs, and
 (5) invariants of the op's definition.
"""
import numpy as np
import pytest
from scipy.spatial.transform import Rotation

import composite
from custom_helper_op_amd.configs import make_workload, reference_test_case

# (B, N, H, W, D): the reference's parameter sets (cost_volume_op_test.py:174-187)
REF_SHAPES = [(1, 1, 12, 16, 5), (1, 2, 12, 16, 9), (2, 2, 12, 18, 10), (2, 3, 12, 16, 6)]


def _depth(t):
    return t["base_plane"] + t["offsets"][:, None, None, :]


def _away_from_edges(xy, srcH, srcW, eps=1e-9):
    """True where no coordinate sits within eps of a validity boundary."""
    lim = np.array([srcW - 1, srcH - 1], dtype=np.float64)
    near = (np.abs(xy) < eps) | (np.abs(xy - lim) < eps)
    return ~near.any(-1)


@pytest.mark.parametrize("shape", REF_SHAPES)
@pytest.mark.parametrize("case", [0, 1, 2, 3])
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_v1_matches_reference_composite(oracle, shape, case, reduce):
    B, N, H, W, D = shape
    t = reference_test_case(case, B, N, H, W, 3, D, np.float64, seed=10 * case + B + N)
    cost, mask = oracle.cost_volume_fwd(**t, reduce=reduce)
    ref_cost, valid, xy, per_view = composite.cost_volume_composite(
        t["ref"], t["src"], _depth(t), t["Rs"], t["Ts"], reduce)
    # the reference test's criterion: all views valid (MEAN) / any valid (MIN), interior
    if reduce == "MEAN":
        sel = np.broadcast_to(mask >= N, cost.shape)
    else:
        sel = mask >= 0
    a = np.where(sel, cost, 0.0)[:, 1:-1, 1:-1]
    b = np.where(sel, ref_cost, 0.0)[:, 1:-1, 1:-1]
    if reduce == "MEAN":
        np.testing.assert_allclose(a, b, rtol=1e-5, atol=1e-6)
    else:
        # the composite takes the minimum over ALL views (invalid ones sample zeros), so
        # it is only comparable where every view is valid
        full = np.broadcast_to((valid.sum(1) == N)[..., None], cost.shape)[:, 1:-1, 1:-1]
        np.testing.assert_allclose(a[full], b[full], rtol=1e-5, atol=1e-6)
    # stronger than the reference's criterion: count and partial means everywhere
    safe = _away_from_edges(xy, H, W).all(1)
    cnt = valid.sum(1)
    if reduce == "MEAN":
        assert np.array_equal(mask[..., 0][safe], cnt[safe])
        part = (per_view * valid[..., None]).sum(1) / np.maximum(cnt, 1)[..., None]
        np.testing.assert_allclose(cost[safe], part[safe], rtol=1e-9, atol=1e-9)
    else:
        big = np.where(valid[..., None], per_view, np.inf)
        best = big.min(1)
        arg = np.where(np.isfinite(best), big.argmin(1), -1)
        has = safe & (cnt > 0)
        np.testing.assert_allclose(cost[has], best[has], rtol=1e-9, atol=1e-9)
        assert np.array_equal(mask[has], arg[has])
        none = safe & (cnt == 0)
        assert np.all(cost[none] == np.finfo(np.float64).max) and np.all(mask[none] == -1)


@pytest.mark.parametrize("shape", REF_SHAPES)
@pytest.mark.parametrize("case", [0, 1, 3])
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_v2_matches_reference_composite(oracle, shape, case, reduce):
    B, N, H, W, D = shape
    t = reference_test_case(case, B, N, H, W, 9, D, np.float64, seed=100 + 10 * case + B + N)
    depth = _depth(t)[..., :]
    cost, mask = oracle.cost_volume_v2_fwd(t["ref"], t["src"], depth, t["Rs"], t["Ts"], reduce, 3)
    ref_cost, valid, xy, per_view = composite.cost_volume_composite(
        t["ref"], t["src"], depth, t["Rs"], t["Ts"], reduce, groups=3)
    sel = np.broadcast_to(mask >= N, cost.shape) if reduce == "MEAN" else mask >= 0
    full = np.broadcast_to((valid.sum(1) == N)[..., None], cost.shape)
    sel = sel & full
    np.testing.assert_allclose(np.where(sel, cost, 0)[:, 1:-1, 1:-1],
                               np.where(sel, ref_cost, 0)[:, 1:-1, 1:-1], rtol=1e-5, atol=1e-6)
    safe = _away_from_edges(xy, H, W).all(1)
    cnt = valid.sum(1)
    if reduce == "MEAN":
        assert np.array_equal(mask[..., 0][safe], cnt[safe])
        part = (per_view * valid[..., None]).sum(1) / np.maximum(cnt, 1)[..., None]
        np.testing.assert_allclose(cost[safe], part[safe], rtol=1e-9, atol=1e-9)
    else:
        # "MIN" of V2 keeps the LARGER correlation, seeded with the smallest positive
        # normal (cost_volume_kernels_gpu_v2.cu.cc:179, :227-230)
        tiny = np.finfo(np.float64).tiny
        big = np.where(valid[..., None], per_view, -np.inf)
        best = np.maximum(big.max(1), tiny)
        arg = np.where(big.max(1) > tiny, big.argmax(1), -1)
        np.testing.assert_allclose(cost[safe], best[safe], rtol=1e-9, atol=0)
        assert np.array_equal(mask[safe], arg[safe])


@pytest.mark.parametrize("index", [1, 2, 5])
def test_v1_composite_on_benchmark_cameras(oracle, index):
    """Same comparison on the benchmark's camera generator (rotation + translation through
    intrinsics), where most voxels see every view and samples are genuinely fractional."""
    wl = make_workload(index, hw=(20, 28), depth=12, batch=1, with_cost_grad=False)
    t = {k: v.astype(np.float64) for k, v in wl.tensors.items()}
    cost, mask = oracle.cost_volume_fwd(t["ref"], t["src"], t["base_plane"], t["offsets"],
                                        t["Rs"], t["Ts"])
    ref_cost, valid, xy, per_view = composite.cost_volume_composite(
        t["ref"], t["src"], _depth(t), t["Rs"], t["Ts"])
    safe = _away_from_edges(xy, wl.H, wl.W).all(1)
    cnt = valid.sum(1)
    assert (cnt > 0).mean() > 0.25
    assert np.array_equal(mask[..., 0][safe], cnt[safe])
    part = (per_view * valid[..., None]).sum(1) / np.maximum(cnt, 1)[..., None]
    np.testing.assert_allclose(cost[safe], part[safe], rtol=1e-9, atol=1e-9)


def test_bilinear_against_scipy(oracle):
    t = reference_test_case(1, 1, 2, 12, 16, 3, 9, np.float64, seed=5)
    cost, mask = oracle.cost_volume_fwd(**t)
    ref_cost, valid, *_ = composite.cost_volume_composite(
        t["ref"], t["src"], _depth(t), t["Rs"], t["Ts"], sampler=composite.bilinear_scipy)
    full = np.broadcast_to(mask >= 2, cost.shape)
    assert full.mean() > 0.3
    np.testing.assert_allclose(cost[full], ref_cost[full], rtol=1e-9, atol=1e-12)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_closed_form_integer_shift(oracle, dtype):
    """R = I, depth constant d0, T = (2 d0, 1 d0, 0): every sample lands exactly on the
    source texel one row down, two columns right, so cost = (src[h+1,w+2] - ref[h,w])^2."""
    rng = np.random.default_rng(3)
    B, N, H, W, C, D, d0 = 1, 2, 9, 11, 4, 3, 4.0
    ref = rng.uniform(0, 10, (B, H, W, C)).astype(dtype)
    src = rng.uniform(0, 10, (B, N, H, W, C)).astype(dtype)
    base = np.full((B, H, W, 1), d0, dtype)
    offsets = np.zeros((B, D), dtype)
    Rs = np.tile(np.eye(3, dtype=dtype)[None, None], (B, N, 1, 1))
    Ts = np.tile(np.array([2 * d0, 1 * d0, 0], dtype)[None, None], (B, N, 1))
    cost, mask = oracle.cost_volume_fwd(ref, src, base, offsets, Rs, Ts)
    # (w+.5)*4 + 8 and the divide by 4 are exact in binary floating point
    expect = np.zeros_like(cost)
    emask = np.zeros(mask.shape, np.int32)
    for h in range(H):
        for w in range(W):
            sh, sw = h + 1, w + 2
            if 0 < sh < H - 1 and 0 < sw < W - 1:
                e = ((src[0, :, sh, sw] - ref[0, h, w][None]) ** 2)
                acc = e[0] + e[1]
                expect[0, h, w, :] = (acc / dtype(2))[None]
                emask[0, h, w, :] = N
    assert np.array_equal(mask, emask)
    assert np.array_equal(cost, expect)  # weights are exactly (1,0,0,0): bit-exact


def test_closed_form_rotation_z(oracle):
    """R = 90 degrees about z, T = (H d0, 0, 0), constant depth: pixel centre (x,y) maps to
    (H - y, x), i.e. ref[h,w] meets src[row = w, col = H-1-h] with no interpolation."""
    rng = np.random.default_rng(4)
    B, N, H, W, C, D, d0 = 1, 1, 6, 8, 2, 2, 2.0
    ref = rng.uniform(0, 10, (B, H, W, C))
    src = rng.uniform(0, 10, (B, N, H, W, C))
    Rz = np.array([[0.0, -1.0, 0.0], [1.0, 0.0, 0.0], [0.0, 0.0, 1.0]])
    Rs = np.tile(Rz[None, None], (B, N, 1, 1))
    Ts = np.tile(np.array([H * d0, 0.0, 0.0])[None, None], (B, N, 1))
    cost, mask = oracle.cost_volume_fwd(ref, src, np.full((B, H, W, 1), d0), np.zeros((B, D)),
                                        Rs, Ts)
    for h in range(H):
        for w in range(W):
            row, col = w, H - 1 - h
            ok = 0 < row < H - 1 and 0 < col < W - 1
            assert np.all(mask[0, h, w] == int(ok))
            want = (src[0, 0, row, col] - ref[0, h, w]) ** 2 if ok else np.zeros(C)
            np.testing.assert_allclose(cost[0, h, w, 0], want, rtol=1e-12, atol=1e-12)


def _brute_force(ref, src, depth, Rs, Ts, reduce, half, groups=None):
    """Scalar restatement from the op's definition (Python floats, float64)."""
    B, H, W, C = ref.shape
    N, sH, sW = src.shape[1:4]
    D = depth.shape[3]
    OC = C if groups is None else groups
    cost = np.zeros((B, H, W, D, OC))
    mask = np.zeros((B, H, W, D, 1 if reduce == "MEAN" else OC), np.int32)
    for b in range(B):
        for h in range(H):
            for w in range(W):
                for d in range(D):
                    px = np.array([w + 0.5 * half, h + 0.5 * half, 1.0])
                    per_view = []
                    for n in range(N):
                        q = (Rs[b, n] @ px) * depth[b, h, w, d] + Ts[b, n]
                        if q[2] <= 0:
                            continue
                        x, y = q[0] / q[2] - 0.5 * half, q[1] / q[2] - 0.5 * half
                        if not (0 < y < sH - 1 and 0 < x < sW - 1):
                            continue
                        fy, fx = int(y), int(x)
                        ay, ax = y - fy, x - fx
                        s = ((1 - ay) * (1 - ax) * src[b, n, fy, fx] + (1 - ay) * ax * src[b, n, fy, fx + 1]
                             + ay * ax * src[b, n, fy + 1, fx + 1] + ay * (1 - ax) * src[b, n, fy + 1, fx])
                        if groups is None:
                            per_view.append((n, (s - ref[b, h, w]) ** 2))
                        else:
                            per_view.append((n, (s * ref[b, h, w]).reshape(groups, -1).sum(-1)))
                    if reduce == "MEAN":
                        mask[b, h, w, d, 0] = len(per_view)
                        if per_view:
                            cost[b, h, w, d] = sum(v for _, v in per_view) / len(per_view)
                    else:
                        seed = np.finfo(np.float64).max if groups is None else np.finfo(np.float64).tiny
                        best = np.full(OC, seed)
                        arg = np.full(OC, -1)
                        for n, v in per_view:
                            better = (best > v) if groups is None else (best < v)
                            best = np.where(better, v, best)
                            arg = np.where(better, n, arg)
                        cost[b, h, w, d], mask[b, h, w, d] = best, arg
    return cost, mask


@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
@pytest.mark.parametrize("half", [True, False])
def test_brute_force_tiny(oracle, reduce, half):
    rng = np.random.default_rng(11)
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
    depth = base + offsets[:, None, None, :]
    cost, mask = oracle.cost_volume_fwd(ref, src, base, offsets, Rs, Ts, reduce, half)
    bc, bm = _brute_force(ref, src, depth, Rs, Ts, reduce, half)
    assert np.array_equal(mask, bm)
    np.testing.assert_allclose(cost, bc, rtol=1e-10, atol=1e-12)
    cost2, mask2 = oracle.cost_volume_v2_fwd(ref, src, depth, Rs, Ts, reduce, 2, half)
    bc2, bm2 = _brute_force(ref, src, depth, Rs, Ts, reduce, half, groups=2)
    assert np.array_equal(mask2, bm2)
    np.testing.assert_allclose(cost2, bc2, rtol=1e-10, atol=1e-12)


def test_invariants_and_threads(oracle):
    wl = make_workload(5, hw=(24, 32), depth=16, batch=2, with_cost_grad=False)
    t = wl.tensors
    args = (t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
    cost, mask = oracle.cost_volume_fwd(*args)
    assert mask.min() >= 0 and mask.max() <= wl.N
    assert 0.02 < (mask < wl.N).mean() < 0.98  # wide-baseline cameras: both kinds occur
    assert cost.min() >= 0
    assert np.all(cost[np.broadcast_to(mask == 0, cost.shape)] == 0)
    # more threads: identical forward bits
    cost4, mask4 = oracle.cost_volume_fwd(*args, threads=4)
    assert np.array_equal(cost, cost4) and np.array_equal(mask, mask4)
    # permuting the source views
    perm = np.array([3, 0, 5, 1, 4, 2])
    pargs = (t["ref"], t["src"][:, perm], t["base_plane"], t["offsets"], t["Rs"][:, perm],
             t["Ts"][:, perm])
    pcost, pmask = oracle.cost_volume_fwd(*pargs)
    assert np.array_equal(mask, pmask)
    np.testing.assert_allclose(cost, pcost, rtol=2e-6, atol=1e-6)
    mcost, mmask = oracle.cost_volume_fwd(*args, reduce="MIN")
    pmcost, pmmask = oracle.cost_volume_fwd(*pargs, reduce="MIN")
    assert mmask.min() >= -1 and mmask.max() <= wl.N - 1
    assert np.array_equal(mcost, pmcost)  # a minimum does not depend on the order
    hit = mmask >= 0
    assert np.array_equal(perm[pmmask[hit]], mmask[hit]) or (mcost[hit] == 0).any()
    # float32 oracle against float64 oracle on the same (float32-representable) inputs
    a64 = tuple(x.astype(np.float64) for x in args)
    cost64, mask64 = oracle.cost_volume_fwd(*a64)
    same = mask64 == mask
    assert same.mean() > 0.999
    sel = np.broadcast_to(same, cost.shape)
    np.testing.assert_allclose(cost[sel], cost64[sel], rtol=1e-4, atol=1e-5)


def test_sample_coords_match_composite(oracle):
    t = reference_test_case(3, 2, 3, 12, 16, 3, 6, np.float64, seed=8)
    sw, sh, fh, fw, st = oracle.sample_coords(t["base_plane"], t["offsets"], t["Rs"], t["Ts"],
                                              (12, 16))
    xy, front = composite.sampler_coordinates(t["Rs"], t["Ts"], _depth(t))
    valid = composite.validity(xy, front, 12, 16)
    xy = np.moveaxis(xy, 1, 4)         # [B,H,W,D,N,2]
    valid = np.moveaxis(valid, 1, 4)
    front = np.moveaxis(front, 1, 4)
    assert np.array_equal(st >= 1, front) and 0.05 < front.mean() < 0.999
    np.testing.assert_allclose(sw[front], xy[..., 0][front], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(sh[front], xy[..., 1][front], rtol=1e-12, atol=1e-12)
    assert np.array_equal(st == 2, valid)
    assert np.array_equal(fh[valid], np.floor(xy[..., 1][valid]).astype(np.int32))
    assert np.array_equal(fw[valid], np.floor(xy[..., 0][valid]).astype(np.int32))
    _, mask = oracle.cost_volume_fwd(**t)
    assert np.array_equal((st == 2).sum(-1), mask[..., 0])


def test_status_codes(oracle):
    z = np.zeros
    with pytest.raises(ValueError):
        oracle.cost_volume_v2_fwd(z((1, 2, 2, 5)), z((1, 1, 2, 2, 5)), z((1, 2, 2, 1)),
                                  z((1, 1, 3, 3)), z((1, 1, 3)), "MEAN", 2)
    # zero-sized work is a successful no-op
    c, m = oracle.cost_volume_fwd(z((1, 0, 4, 3)), z((1, 2, 0, 4, 3)), z((1, 0, 4, 1)), z((1, 5)),
                                  z((1, 2, 3, 3)), z((1, 2, 3)))
    assert c.shape == (1, 0, 4, 5, 3) and m.shape == (1, 0, 4, 5, 1)
