"""Seeded synthetic workloads for the cost-volume operator.

The five workloads mirror the benchmark configurations of this repository
(tiny forward, standard MVSNet stage, cascade fine stage with 16-bit features,
group-wise correlation, large-batch stress).  All tensors are produced on the host
with ``numpy.random.default_rng(1000 + index)`` so that the CPU checker and the GPU
library see identical bits.  The operator takes *pre-combined* camera matrices
(``Rs = K_src R K_ref^-1``, ``Ts = K_src t``), the way the reference's test helper
``combine_projection`` builds them
(custom_helper_op/python/ops/op_tests/cost_volume_op_test.py:115-134).
"""
from dataclasses import dataclass, field
from typing import Dict, Optional

import numpy as np
from scipy.ndimage import zoom
from scipy.spatial.transform import Rotation


@dataclass
class Workload:
    name: str
    op: str                # "v1": CostVolume (base_plane + offsets, squared difference)
                           # "v2": CostVolumeV2 (depth_grid, group-wise correlation)
                           # "agg": CostAggregate (v1's inputs, channels summed: one value/voxel)
                           # "v3": CostVolumeV3 (v1's inputs, best group pair: one value/voxel)
                           # "feat": FeatureAggregate (v1's inputs without ref: N*C values/voxel)
    storage: str           # element type of ref/src/cost/cost_grad: f32, f64, f16, bf16
    B: int
    N: int
    H: int
    W: int
    C: int
    D: int
    groups: int = 1
    backward: bool = True
    reduce_method: str = "MEAN"
    half_centor: bool = True
    grid_form: bool = False  # "v1" with per-voxel hypotheses (depth_grid) instead of plane + offsets
    seed: int = 0
    tensors: Dict[str, np.ndarray] = field(default_factory=dict)

    @property
    def voxels(self) -> int:
        return self.B * self.D * self.H * self.W

    @property
    def out_channels(self) -> int:
        if self.op == "feat":
            return self.N * self.C
        return self.groups if self.op == "v2" else 1 if self.op in ("agg", "v3") else self.C

    def elem_bytes(self) -> int:
        return {"f32": 4, "f64": 8, "f16": 2, "bf16": 2}[self.storage]

    def depth_bytes(self) -> int:
        """Depth inputs, camera matrices and depth gradients stay fp32 for 16-bit storage."""
        return 8 if self.storage == "f64" else 4

    def algorithmic_bytes(self):
        """(forward, backward) compulsory bytes: every operand counted once per pass,
        bilinear taps assumed cache resident, zero-fill folded into the single write."""
        e, f = self.elem_bytes(), self.depth_bytes()
        px = self.B * self.H * self.W
        ref = px * self.C * e
        src = self.B * self.N * self.H * self.W * self.C * e
        cams = self.B * self.N * 12 * f
        if self.op != "v2" and not self.grid_form:
            depth_in = px * f + self.B * self.D * f
            depth_grad = px * f
        else:
            depth_in = px * self.D * f
            depth_grad = px * self.D * f
        cost = self.voxels * self.out_channels * e
        mask = self.voxels * 4 * (1 if self.reduce_method == "MEAN" else self.out_channels)
        if self.op == "agg":
            cost = self.voxels * e  # one value per voxel
        if self.op == "v3":         # mask: view count, or (view, reference group, source group)
            mask = self.voxels * 4 * (1 if self.reduce_method == "MEAN" else 3)
        if self.op == "feat":       # no reference image; one mask entry per (voxel, view)
            ref = 0
            mask = self.voxels * self.N * 4
        fwd = ref + src + depth_in + cams + cost + mask
        bwd = ref + src + depth_in + cams + cost + mask + ref + src + depth_grad
        return fwd, bwd


def intrinsics(H: int, W: int) -> np.ndarray:
    return np.array([[0.8 * W, 0.0, W / 2.0], [0.0, 0.8 * W, H / 2.0], [0.0, 0.0, 1.0]])


def combine_cameras(K_ref, K_src, R_rel, t_rel):
    """``(K_src R K_ref^-1, K_src t)`` in float64."""
    return K_src @ R_rel @ np.linalg.inv(K_ref), K_src @ t_rel


def random_cameras(rng, B, N, H, W, max_deg, max_t):
    K = intrinsics(H, W)
    Rs = np.empty((B, N, 3, 3))
    Ts = np.empty((B, N, 3))
    for b in range(B):
        for n in range(N):
            ang = rng.uniform(-max_deg, max_deg, 3)
            t = rng.uniform(-max_t, max_t, 3)
            R = Rotation.from_euler("xyz", ang, degrees=True).as_matrix()
            Rs[b, n], Ts[b, n] = combine_cameras(K, K, R, t)
    return Rs, Ts


def smooth_field(rng, B, H, W, mean=5.0, std=1.0, lo=None, hi=None):
    """8x10 Gaussian grid, bicubically upsampled to HxW; optionally rescaled to [lo,hi]."""
    out = np.empty((B, H, W))
    for b in range(B):
        g = rng.normal(mean, std, (8, 10))
        f = zoom(g, (H / 8.0, W / 10.0), order=3, mode="nearest", grid_mode=True)
        f = f[:H, :W]
        if lo is not None:
            f = lo + (hi - lo) * (f - f.min()) / max(f.max() - f.min(), 1e-12)
        out[b] = f
    return out


def quantise(x: np.ndarray, storage: str) -> np.ndarray:
    """Round float32 values to the storage type and back (values the kernels will see)."""
    if storage == "f16":
        return x.astype(np.float16).astype(np.float32)
    if storage == "bf16":
        u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
        u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16  # round to nearest even
        return u.astype(np.uint32).view(np.float32).reshape(x.shape)
    return x


_SPECS = {
    # index: name, op, storage, B, N, H, W, C, D, groups, backward, rot deg, |t|
    1: ("tiny_variance_fwd", "v1", "f32", 1, 2, 64, 80, 8, 32, 1, False, 5.0, 0.1),
    2: ("mvsnet_stage", "v1", "f32", 1, 2, 128, 160, 32, 192, 1, True, 5.0, 0.2),
    3: ("cascade_fine_f16", "v1", "f16", 1, 4, 256, 320, 16, 32, 1, True, 5.0, 0.2),
    4: ("groupwise_corr_bf16", "v2", "bf16", 2, 4, 512, 640, 8, 8, 4, True, 5.0, 0.2),
    5: ("large_batch_stress", "v1", "f32", 4, 6, 288, 384, 32, 128, 1, True, 15.0, 0.5),
}


def make_workload(index: int, hw: Optional[tuple] = None, with_cost_grad: bool = True,
                  depth: Optional[int] = None, batch: Optional[int] = None) -> Workload:
    """Build workload ``index`` (1..5).

    ``hw``/``depth``/``batch`` shrink the image, hypothesis count or batch so that a CPU
    check finishes in seconds; the generator, cameras and value distributions stay those
    of the full configuration.  ``with_cost_grad=False`` skips the upstream gradient (the
    largest tensor) for callers that draw it on the device instead.
    """
    name, op, storage, B, N, H, W, C, D, G, backward, deg, tmax = _SPECS[index]
    if hw is not None:
        H, W = hw
    if depth is not None:
        D = depth
    if batch is not None:
        B = batch
    rng = np.random.default_rng(1000 + index)
    wl = Workload(name, op, storage, B, N, H, W, C, D, G, backward, seed=1000 + index)
    f32 = np.float32
    t = wl.tensors
    t["ref"] = quantise(rng.standard_normal((B, H, W, C), dtype=f32), storage)
    t["src"] = quantise(rng.standard_normal((B, N, H, W, C), dtype=f32), storage)
    Rs, Ts = random_cameras(rng, B, N, H, W, deg, tmax)
    t["Rs"], t["Ts"] = Rs.astype(f32), Ts.astype(f32)
    if index == 1:
        t["base_plane"] = np.zeros((B, H, W, 1), f32)
        t["offsets"] = np.tile(np.linspace(2.0, 6.0, D)[None], (B, 1)).astype(f32)
    elif index == 2:
        t["base_plane"] = np.zeros((B, H, W, 1), f32)
        t["offsets"] = np.tile((1.0 / np.linspace(1.0, 1.0 / 10.0, D))[None], (B, 1)).astype(f32)
    elif index == 3:
        coarse = smooth_field(rng, B, H, W, 5.0, 1.0)
        t["base_plane"] = coarse[..., None].astype(f32)
        k = np.arange(D) - D // 2
        # The registered op can only add a per-batch offset to the base plane, so the
        # drop-in form of "coarse +- k*0.02*depth" uses the field's nominal mean depth.
        t["offsets"] = np.tile((k * 0.02 * 5.0)[None], (B, 1)).astype(f32)
        # The exact per-pixel multiplicative form, for the depth_grid entry points.
        t["depth_grid"] = (coarse[..., None] * (1.0 + 0.02 * k)[None, None, None]).astype(f32)
    elif index == 4:
        fld = smooth_field(rng, B, H, W, 5.0, 1.0, lo=2.0, hi=8.0)
        k = np.arange(D) - D // 2
        t["depth_grid"] = (fld[..., None] * (1.0 + 0.02 * k)[None, None, None]).astype(f32)
    elif index == 5:
        t["base_plane"] = np.zeros((B, H, W, 1), f32)
        t["offsets"] = np.tile(np.linspace(0.5, 20.0, D)[None], (B, 1)).astype(f32)
    if backward and with_cost_grad:
        t["cost_grad"] = quantise(
            rng.standard_normal((B, H, W, D, wl.out_channels), dtype=f32), storage)
    return wl


def reference_test_case(case: int, B=1, N=2, H=12, W=16, C=3, D=9, dtype=np.float64, seed=0):
    """Inputs shaped and distributed like the reference's own unit tests
    (cost_volume_op_test.py:188-194): features U(0,10), base depth U(20,30),
    offsets U(-2,2), and one of its four camera set-ups:
    0 identity, 1 T=(3,3,3), 2 adds a 90 degree rotation about z, 3 instead rotates
    22.5 degrees about y (the test reuses T=(3,3,3) for cases 2 and 3, :213-248)."""
    rng = np.random.default_rng(seed)
    ref = rng.uniform(0, 10, (B, H, W, C)).astype(dtype)
    src = rng.uniform(0, 10, (B, N, H, W, C)).astype(dtype)
    base = ((rng.uniform(0, 1, (B, H, W, 1)) + 2) * 10).astype(dtype)
    offsets = (rng.uniform(0, 1, (B, D)) * 4 - 2).astype(dtype)
    R = np.eye(3)
    T = np.zeros(3)
    if case >= 1:
        T = np.array([3.0, 3.0, 3.0])
    if case == 2:
        R = Rotation.from_rotvec(np.pi / 2 * np.array([0, 0, 1.0])).as_matrix()
    if case == 3:
        R = Rotation.from_rotvec(np.pi / 8 * np.array([0, 1.0, 0])).as_matrix()
    Rs = np.tile(R[None, None], (B, N, 1, 1)).astype(dtype)
    Ts = np.tile(T[None, None], (B, N, 1)).astype(dtype)
    return dict(ref=ref, src=src, base_plane=base, offsets=offsets, Rs=Rs, Ts=Ts)
