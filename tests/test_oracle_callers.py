"""Pins the oracle's restatements of the callers around the ops (CPU only): the layers'
default fill and ``combine_projection``.

``combine_projection`` exists only as a helper inside the reference's test files; what it must
satisfy is geometric, so it is pinned by projecting random world points through both cameras
directly and through the relative projection, and by its special cases.
"""
import numpy as np
import pytest
from scipy.spatial.transform import Rotation


def random_cam(rng, dtype=np.float64):
    cam = np.zeros((2, 4, 4), dtype)
    cam[0, :3, :3] = Rotation.from_euler("xyz", rng.uniform(-20, 20, 3), degrees=True).as_matrix()
    cam[0, :3, 3] = rng.uniform(-1, 1, 3)
    cam[0, 3, 3] = 1
    f = rng.uniform(300, 600)
    cam[1, :3, :3] = [[f, 0, rng.uniform(150, 170)], [0, f * rng.uniform(0.9, 1.1), rng.uniform(110, 130)],
                      [0, 0, 1]]
    cam[1, 3] = [425.0, 2.5, 192, 905]        # depth range row of the camera files
    return cam


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_combine_projection_maps_reference_rays_to_source_pixels(oracle, seed):
    rng = np.random.default_rng(seed)
    ref_cam, src_cam = random_cam(rng), random_cam(rng)
    scale = np.array([0.25, 0.5, 1.0])
    R, T = oracle.combine_projection(ref_cam, src_cam, scale)
    assert R.shape == (3, 3) and T.shape == (3, 1)

    def intrinsics(cam):
        K = cam[1, :3, :3] * scale[:, None]
        K[:2, 2] += 0.5
        return K

    X = rng.uniform(-1, 1, (3, 50)) + np.array([[0], [0], [6.0]])      # world points
    ref_c = ref_cam[0, :3, :3] @ X + ref_cam[0, :3, 3:]                  # reference camera frame
    src_c = src_cam[0, :3, :3] @ X + src_cam[0, :3, 3:]
    ref_h = intrinsics(ref_cam) @ ref_c          # = depth * (u, v, 1) in the reference image
    want = intrinsics(src_cam) @ src_c           # = z' * (u', v', 1) in the source image
    np.testing.assert_allclose(R @ ref_h + T, want, rtol=1e-10, atol=1e-9)
    # which is exactly what the ops evaluate: R (u, v, 1) * depth + T, then the perspective divide
    depth = ref_h[2]
    uv1 = ref_h / depth
    np.testing.assert_allclose((R @ uv1) * depth + T, want, rtol=1e-10, atol=1e-9)


def test_combine_projection_special_cases(oracle):
    rng = np.random.default_rng(5)
    cam = random_cam(rng)
    one = np.ones(3)
    R, T = oracle.combine_projection(cam.copy(), cam.copy(), one)
    np.testing.assert_allclose(R, np.eye(3), atol=1e-12)                 # same camera: identity
    np.testing.assert_allclose(T, 0, atol=1e-9)
    other = cam.copy()
    other[0, :3, 3] += [0.3, -0.2, 0.1]                                  # pure translation
    R, T = oracle.combine_projection(cam.copy(), other, one)
    K = cam[1, :3, :3].copy()
    K[:2, 2] += 0.5
    np.testing.assert_allclose(R, np.eye(3), atol=1e-12)
    np.testing.assert_allclose(T[:, 0], K @ np.array([0.3, -0.2, 0.1]), rtol=1e-12)
    # the inputs are not modified (the reference helper scales copies of K)
    before = cam.copy()
    oracle.combine_projection(cam, other, np.array([0.5, 0.5, 1.0]))
    assert np.array_equal(cam, before)


@pytest.mark.parametrize("reduce", ["MEAN", "MIN"])
def test_default_fill_and_gradient(oracle, reduce):
    rng = np.random.default_rng(7)
    cost = rng.normal(size=(2, 3, 4, 5, 6))
    for mask_shape in ((2, 3, 4, 5, 1), (2, 3, 4, 5, 6)):
        mask = rng.integers(-1, 3, mask_shape).astype(np.int32)
        out = oracle.cost_default_fill(cost, mask, 0.75, reduce)
        keep = np.broadcast_to((mask > 0) if reduce == "MEAN" else (mask >= 0), cost.shape)
        assert np.array_equal(out[keep], cost[keep]) and np.all(out[~keep] == 0.75)
        g = rng.normal(size=cost.shape)
        cg, dg = oracle.cost_default_fill_grad(g, mask, reduce)
        # d/d(cost) and d/d(default) of sum(out * g) by finite differences (the map is linear)
        eps = 1e-6
        num = (np.sum(oracle.cost_default_fill(cost, mask, 0.75 + eps, reduce) * g)
               - np.sum(oracle.cost_default_fill(cost, mask, 0.75 - eps, reduce) * g)) / (2 * eps)
        assert abs(num - dg) < 1e-6 * max(1.0, abs(dg))
        assert np.array_equal(cg, np.where(keep, g, 0))
        assert abs(cg.sum() + dg - g.sum()) < 1e-9
