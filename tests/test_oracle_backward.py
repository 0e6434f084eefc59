"""Pins the CPU oracle's backward functions (CPU only).

The reference's gradient test (cost_volume_op_test.py:400-463, V2:
cost_volume_v2_op_test.py:403-466) compares the registered gradient with central
finite differences of ``reduce_mean(where(mask ok, cost, 0))`` in float64 at
rtol=5e-5.  The same criterion is applied here to the oracle's backward, with the
oracle's (independently pinned) forward as the differentiated function.
"""
import numpy as np
import pytest
from scipy.spatial.transform import Rotation

from custom_helper_op_amd.configs import make_workload, reference_test_case

REF_SHAPES = [(1, 1, 12, 16, 5), (1, 2, 12, 16, 9), (2, 2, 12, 18, 10), (2, 3, 12, 16, 6)]


def _loss_v1(oracle, t, reduce):
    cost, mask = oracle.cost_volume_fwd(t["ref"], t["src"], t["base_plane"], t["offsets"],
                                        t["Rs"], t["Ts"], reduce)
    ok = (mask > 0) if reduce == "MEAN" else (mask >= 0)
    return np.where(ok, cost, 0.0).mean(), mask, cost.size


def _loss_v2(oracle, t, reduce, groups):
    cost, mask = oracle.cost_volume_v2_fwd(t["ref"], t["src"], t["depth_grid"], t["Rs"], t["Ts"],
                                           reduce, groups)
    ok = (mask > 0) if reduce == "MEAN" else (mask >= 0)
    return np.where(ok, cost, 0.0).mean(), mask, cost.size


def _numeric(loss_fn, t, key, delta):
    """Central differences; NaN where the perturbation changed the mask (valid-view count
    or arg-min view), because the registered gradient is the derivative at fixed mask."""
    x = t[key]
    base_mask = loss_fn(t)[1]
    g = np.zeros_like(x)
    flat, gf = x.reshape(-1), g.reshape(-1)
    for i in range(flat.size):
        keep = flat[i]
        flat[i] = keep + delta
        hi, m_hi, _ = loss_fn(t)
        flat[i] = keep - delta
        lo, m_lo, _ = loss_fn(t)
        flat[i] = keep
        same = np.array_equal(m_hi, base_mask) and np.array_equal(m_lo, base_mask)
        gf[i] = (hi - lo) / (2 * delta) if same else np.nan
    return g


def _close(analytic, numeric, rtol=5e-5):
    # the reference asserts rtol=5e-5 with assertAllClose's default atol=1e-6
    keep = np.isfinite(numeric)
    assert keep.mean() > 0.98
    a, n = analytic[keep], numeric[keep]
    np.testing.assert_allclose(a, n, rtol=rtol, atol=1e-6 * max(1.0, np.abs(n).max()))


@pytest.mark.parametrize("shape,reduce", [(s, "MEAN") for s in REF_SHAPES] +
                         [(s, "MIN") for s in REF_SHAPES[1:3]])
@pytest.mark.parametrize("case", [0, 1, 3])
def test_v1_gradient_against_finite_differences(oracle, shape, case, reduce):
    B, N, H, W, D = shape
    t = reference_test_case(case, B, N, H, W, 5, D, np.float64, seed=7 * case + B + 2 * N)
    fn = lambda tt: _loss_v1(oracle, tt, reduce)
    _, mask, numel = fn(t)
    ok = (mask > 0) if reduce == "MEAN" else (mask >= 0)
    cg = np.broadcast_to(np.where(ok, 1.0 / numel, 0.0), (B, H, W, D, 5)).copy()
    rg, sg, bg = oracle.cost_volume_bwd(t["ref"], t["src"], t["base_plane"], t["offsets"],
                                        t["Rs"], t["Ts"], cg, mask, reduce)
    # ref/src: the loss is quadratic in them, central differences are exact up to rounding
    _close(rg, _numeric(fn, t, "ref", 1e-4))
    _close(sg, _numeric(fn, t, "src", 1e-4))
    if case != 0:
        # identity cameras put every sample exactly on a texel corner (a kink of the
        # bilinear surface), so the reference skips the depth gradient there too (:435)
        _close(bg, _numeric(fn, t, "base_plane", 1e-6), rtol=2e-4)
    assert np.abs(sg).max() > 0


@pytest.mark.parametrize("shape", REF_SHAPES[1:3])
@pytest.mark.parametrize("case", [1, 3])
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_v2_gradient_against_finite_differences(oracle, shape, case, reduce):
    B, N, H, W, D = shape
    t = reference_test_case(case, B, N, H, W, 6, D, np.float64, seed=50 + 7 * case + B + 2 * N)
    t["depth_grid"] = (t["base_plane"] + t["offsets"][:, None, None, :]).copy()
    fn = lambda tt: _loss_v2(oracle, tt, reduce, 3)
    _, mask, numel = fn(t)
    ok = (mask > 0) if reduce == "MEAN" else (mask >= 0)
    cg = np.broadcast_to(np.where(ok, 1.0 / numel, 0.0), (B, H, W, D, 3)).copy()
    rg, sg, dg = oracle.cost_volume_v2_bwd(t["ref"], t["src"], t["depth_grid"], t["Rs"], t["Ts"],
                                           cg, mask, reduce, 3)
    _close(rg, _numeric(fn, t, "ref", 1e-4))
    _close(sg, _numeric(fn, t, "src", 1e-4))
    _close(dg, _numeric(fn, t, "depth_grid", 1e-6), rtol=2e-4)
    skipped = (mask[..., 0] <= 0) if reduce == "MEAN" else (mask[..., 0] < 0)
    assert np.all(dg[skipped] == 0)


def test_gradient_on_benchmark_cameras(oracle):
    """Finite differences with rotation+translation cameras and a random upstream gradient
    (a linear functional of the cost instead of the mean), V1 MEAN."""
    wl = make_workload(2, hw=(10, 12), depth=6)
    t = {k: v.astype(np.float64) for k, v in wl.tensors.items()}
    t["base_plane"] = t["base_plane"] + 1.7
    cg = t["cost_grad"]
    _, mask = oracle.cost_volume_fwd(t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"],
                                     t["Ts"])

    def fn(tt):
        c, m = oracle.cost_volume_fwd(tt["ref"], tt["src"], tt["base_plane"], tt["offsets"],
                                      tt["Rs"], tt["Ts"])
        assert np.array_equal(m, mask)
        return (c * cg).sum(), m, c.size

    rg, sg, bg = oracle.cost_volume_bwd(t["ref"], t["src"], t["base_plane"], t["offsets"],
                                        t["Rs"], t["Ts"], cg, mask)
    sub = {k: v for k, v in t.items()}
    # all of ref and base_plane, a slab of src
    _close(rg, _numeric(fn, sub, "ref", 1e-4))
    _close(bg, _numeric(fn, sub, "base_plane", 1e-7), rtol=2e-4)
    num_src = _numeric(fn, sub, "src", 1e-4)
    _close(sg, num_src)


def test_conservation_and_threads(oracle):
    """V1: each g goes to ref_grad as -g and to four src_grad taps with weights summing
    to one (cost_volume_kernels_gpu.cu.cc:440-444), so the two gradients cancel in sum."""
    wl = make_workload(5, hw=(24, 32), depth=16, batch=2)
    t = {k: v.astype(np.float64) for k, v in wl.tensors.items()}
    args = (t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
    _, mask = oracle.cost_volume_fwd(*args)
    rg, sg, bg = oracle.cost_volume_bwd(*args, t["cost_grad"], mask)
    scale = np.abs(rg).sum()
    assert abs(rg.sum() + sg.sum()) < 1e-10 * scale
    per_batch = rg.sum((1, 2, 3)) + sg.sum((1, 2, 3, 4))
    assert np.all(np.abs(per_batch) < 1e-10 * scale)
    assert np.all(rg[np.broadcast_to((mask.sum(3) == 0), rg.shape[:3] + (1,))[..., 0]] == 0)
    rg4, sg4, bg4 = oracle.cost_volume_bwd(*args, t["cost_grad"], mask, threads=4)
    assert np.array_equal(rg, rg4) and np.array_equal(bg, bg4)
    np.testing.assert_allclose(sg, sg4, rtol=1e-12, atol=1e-13)
    # float32 oracle on the same inputs
    a32 = tuple(x.astype(np.float32) for x in args)
    _, mask32 = oracle.cost_volume_fwd(*a32)
    r32, s32, b32 = oracle.cost_volume_bwd(*a32, t["cost_grad"].astype(np.float32), mask32)
    rg_m, sg_m, bg_m = oracle.cost_volume_bwd(*args, t["cost_grad"], mask32)
    for a, b in ((r32, rg_m), (s32, sg_m), (b32, bg_m)):
        assert np.abs(a - b).max() <= 2e-4 * np.abs(b).max()


def test_v2_mean_linear_in_ref(oracle):
    """V2 MEAN cost is bilinear in (ref, src): cost(a*ref, src) = a*cost, and the ref
    gradient of <cost, cg> does not depend on ref at all."""
    rng = np.random.default_rng(2)
    t = reference_test_case(1, 1, 2, 8, 10, 6, 4, np.float64, seed=3)
    dg = t["base_plane"] + t["offsets"][:, None, None, :]
    c1, m1 = oracle.cost_volume_v2_fwd(t["ref"], t["src"], dg, t["Rs"], t["Ts"], "MEAN", 2)
    c2, m2 = oracle.cost_volume_v2_fwd(3 * t["ref"], t["src"], dg, t["Rs"], t["Ts"], "MEAN", 2)
    assert np.array_equal(m1, m2)
    np.testing.assert_allclose(c2, 3 * c1, rtol=1e-12)
    cg = rng.normal(size=c1.shape)
    r1, s1, _ = oracle.cost_volume_v2_bwd(t["ref"], t["src"], dg, t["Rs"], t["Ts"], cg, m1, "MEAN", 2)
    r2, s2, _ = oracle.cost_volume_v2_bwd(3 * t["ref"], t["src"], dg, t["Rs"], t["Ts"], cg, m1, "MEAN", 2)
    np.testing.assert_allclose(r1, r2, rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(3 * s1, s2, rtol=1e-12, atol=1e-14)


# ---- squared difference over a depth grid ------------------------------------------------------
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_grid_entry_equals_the_plane_entry_bit_for_bit(oracle, dtype, reduce):
    """chop_oracle_cost_volume_grid_* is the pinned CostVolume oracle with another depth
    source.  On depth_grid = base_plane + offsets (formed in the same precision, the kernel's
    own expression, cost_volume_kernels_gpu.cu.cc:64) every voxel sees the same depth, so cost,
    mask, ref_grad and src_grad must equal the pinned functions' to the bit, and the per-voxel
    depth gradient must add up, in depth order, to the per-pixel one."""
    t = reference_test_case(3, B=2, N=3, H=12, W=18, C=5, D=10, dtype=dtype, seed=21)
    args = (t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
    grid = (t["base_plane"] + t["offsets"][:, None, None, :]).astype(dtype)
    want_cost, want_mask = oracle.cost_volume_fwd(*args, reduce)
    cost, mask = oracle.cost_volume_grid_fwd(t["ref"], t["src"], grid, t["Rs"], t["Ts"], reduce)
    assert np.array_equal(mask, want_mask)
    assert np.array_equal(cost.view(np.uint8), want_cost.view(np.uint8))
    assert (want_mask > 0).any() if reduce == "MEAN" else (want_mask >= 0).any()
    rng = np.random.default_rng(5)
    cg = rng.standard_normal(cost.shape).astype(dtype)
    want = oracle.cost_volume_bwd(*args, cg, want_mask, reduce)
    got = oracle.cost_volume_grid_bwd(t["ref"], t["src"], grid, t["Rs"], t["Ts"], cg, want_mask, reduce)
    assert np.array_equal(got[0], want[0])
    assert np.array_equal(got[1], want[1])
    total = np.zeros(want[2].shape[:3], dtype)
    for d in range(grid.shape[3]):  # the plane entry adds its voxels up in this order (:454)
        total = (total + got[2][..., d]).astype(dtype)
    assert np.array_equal(total, want[2][..., 0])
    # voxels the mask skips get a zero, as in CostVolumeGradV2 (cost_volume_kernels_gpu_v2.cu.cc:375-378)
    skipped = (want_mask[..., 0] <= 0) if reduce == "MEAN" else (want_mask[..., 0] < 0)
    assert skipped.any() and not got[2][skipped].any()
    # several threads: the same forward, the same pixel-owned gradients
    cost4, mask4 = oracle.cost_volume_grid_fwd(t["ref"], t["src"], grid, t["Rs"], t["Ts"], reduce,
                                               threads=4)
    assert np.array_equal(cost4, cost) and np.array_equal(mask4, mask)
    got4 = oracle.cost_volume_grid_bwd(t["ref"], t["src"], grid, t["Rs"], t["Ts"], cg, want_mask,
                                       reduce, threads=4)
    assert np.array_equal(got4[0], got[0]) and np.array_equal(got4[2], got[2])
    np.testing.assert_allclose(got4[1], got[1], rtol=1e-5 if dtype == np.float32 else 1e-12,
                               atol=1e-5 if dtype == np.float32 else 1e-12)
