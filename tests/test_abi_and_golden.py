"""CPU-only checks: the C-ABI library loads and exports every declared symbol, argument
validation answers before any HIP call, the host mirror raises the reference's
InvalidArgument errors, the oracle reproduces the committed golden vectors, and the
workload generator is deterministic."""
import ctypes
import hashlib
import os
import re

import numpy as np
import pytest
import torch

from custom_helper_op_amd import _lib
from custom_helper_op_amd.configs import make_workload, quantise
import custom_helper_op_amd as chop

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden", "costvol_golden.npz")


def declared_functions():
    text = open(os.path.join(ROOT, "include", "chop_costvol.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(chop_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = declared_functions()
    assert len(names) == 49
    for n in names:
        assert hasattr(lib, n), n
    assert set(names) == set(_lib.SIGNATURES), set(names) ^ set(_lib.SIGNATURES)
    assert lib.chop_abi_version() == 1


def test_oracle_exports():
    import oracle
    lib = oracle.lib()
    for sfx in ("f32", "f64"):
        for stem in ("cost_volume_fwd", "cost_volume_bwd", "cost_volume_v2_fwd", "cost_volume_v2_bwd",
                     "cost_aggregate_fwd", "cost_aggregate_bwd", "sample_coords",
                     "cost_volume_grid_fwd", "cost_volume_grid_bwd"):
            assert hasattr(lib, "chop_oracle_%s_%s" % (stem, sfx))


def _fwd_f32(lib, reduce, dims, ptrs):
    return lib.chop_cost_volume_fwd_f32(None, reduce, 1, *dims, *ptrs)


def test_validation_runs_before_any_device_call():
    """Bad arguments are answered with status codes on a machine without a GPU."""
    lib = _lib.load()
    fake = [ctypes.c_void_p(4096)] * 8
    null = [None] * 8
    good = (1, 4, 5, 8, 3, 2, 4, 5)
    assert _fwd_f32(lib, 7, good, fake) == 3 and b"reduce" in lib.chop_last_error_string()
    assert _fwd_f32(lib, 0, (1, -4, 5, 8, 3, 2, 4, 5), fake) == 2
    assert _fwd_f32(lib, 0, (1, 2 ** 40, 5, 8, 3, 2, 4, 5), fake) == 2
    assert _fwd_f32(lib, 0, good, null) == 1 and b"null pointer: ref" in lib.chop_last_error_string()
    # CostAggregate goes through the same validation
    assert lib.chop_cost_aggregate_fwd_f32(None, 7, 1, *good, *fake) == 3
    assert lib.chop_cost_aggregate_fwd_f64(None, 0, 1, *good, *null) == 1
    assert lib.chop_cost_aggregate_bwd_f32(None, 0, 1, *good, *([None] * 11)) == 1
    assert lib.chop_cost_aggregate_bwd_f32(None, 0, 1, 1, 4, 5, 8, 0, 2, 4, 5, *([None] * 8),
                                           *fake[:3]) in (0, 5)  # D = 0: only zero fills
    # zero-sized work: success without touching anything
    assert _fwd_f32(lib, 0, (1, 0, 5, 8, 3, 2, 0, 5), null) == 0
    assert _fwd_f32(lib, 0, (1, 4, 5, 8, 0, 2, 4, 5), null) == 0
    # groups
    rc = lib.chop_cost_volume_v2_fwd_f32(None, 0, 1, *good, 3, *([ctypes.c_void_p(4096)] * 7))
    assert rc == 4 and b"groups" in lib.chop_last_error_string()
    rc = lib.chop_cost_volume_v2_fwd_f64(None, 0, 1, *good, 0, *([ctypes.c_void_p(4096)] * 7))
    assert rc == 4
    # 16-bit storage: enum and workspace
    rc = lib.chop_cost_volume_fwd_16(None, 9, 0, 1, *good, *([ctypes.c_void_p(4096)] * 9))
    assert rc == 3 and b"storage" in lib.chop_last_error_string()
    need = lib.chop_cost_volume_bwd16_workspace_bytes(1, 4, 5, 8, 2, 4, 5)
    assert need == 4 * (320 + 192)  # fp32 images of src_grad and ref_grad, padded to 64 elements
    p = ctypes.c_void_p(4096)
    args = [None, 1, 0, 1, *good] + [p] * 13
    args[4 + 8 + 12] = None                      # workspace pointer
    assert lib.chop_cost_volume_bwd_16(*args, 0) == 6
    args[4 + 8 + 12] = ctypes.c_void_p(4096 + 8)  # misaligned
    assert lib.chop_cost_volume_bwd_16(*args, need) == 6 and b"aligned" in lib.chop_last_error_string()
    args[4 + 8 + 12] = ctypes.c_void_p(4096)
    assert lib.chop_cost_volume_bwd_16(*args, need - 1) == 6 and b"too small" in lib.chop_last_error_string()
    # backward with null outputs
    rc = lib.chop_cost_volume_bwd_f32(None, 0, 1, *good, *([None] * 11))
    assert rc == 1
    assert lib.chop_set_kernel_family(1) in (0, 1)
    assert lib.chop_set_kernel_family(0) == 1


def test_host_mirror_shape_errors():
    """The checks of CostVolumeOp::Compute (cost_volume_kernels.cc:91-106), as exceptions."""
    z = torch.zeros
    ref, src = z(1, 4, 5, 3), z(1, 2, 4, 5, 3)
    bp, off, Rs, Ts = z(1, 4, 5, 1), z(1, 6), z(1, 2, 3, 3), z(1, 2, 3)
    with pytest.raises(chop.InvalidArgumentError, match="ref image must have rank 4"):
        chop.cost_volume_raw(z(4, 5, 3), src, bp, off, Rs, Ts)
    with pytest.raises(chop.InvalidArgumentError, match="src_images must have rank 5"):
        chop.cost_volume_raw(ref, z(1, 2, 4, 6, 3), bp, off, Rs, Ts)
    with pytest.raises(chop.InvalidArgumentError, match="base_plane must have rank 4"):
        chop.cost_volume_raw(ref, src, z(1, 4, 5), off, Rs, Ts)
    with pytest.raises(chop.InvalidArgumentError, match="offsets must have rank 2"):
        chop.cost_volume_raw(ref, src, bp, z(2, 6), Rs, Ts)
    with pytest.raises(chop.InvalidArgumentError, match="Rs must have rank 2"):
        chop.cost_volume_raw(ref, src, bp, off, z(1, 3, 3, 3), Ts)
    with pytest.raises(chop.InvalidArgumentError, match="Ts must have rank 2"):
        chop.cost_volume_raw(ref, src, bp, off, Rs, z(1, 2, 4))
    with pytest.raises(chop.InvalidArgumentError, match="Invalid reduce method"):
        chop.cost_volume_raw(ref, src, bp, off, Rs, Ts, "MAX")
    with pytest.raises(chop.InvalidArgumentError, match="groups"):
        chop.cost_volume_v2_raw(ref, src, z(1, 4, 5, 6), Rs, Ts, "MEAN", 2)
    with pytest.raises(chop.InvalidArgumentError, match="cost_grad must have rank 5"):
        chop.cost_volume_grad(ref, src, bp, off, Rs, Ts, z(1, 4, 5, 6, 2), z(1, 4, 5, 6, 1).int())
    with pytest.raises(chop.InvalidArgumentError, match="dtype"):
        chop.cost_volume_raw(ref, src.double(), bp, off, Rs, Ts)


def _golden_cases():
    blob = np.load(GOLDEN)
    names = sorted({k.split("/")[0] for k in blob.files})
    return blob, names


def test_oracle_reproduces_golden_vectors(oracle):
    blob, names = _golden_cases()
    assert len(names) == 28
    for name in names:
        op, red, groups, half = (int(x) for x in blob[name + "/attrs"])
        t = {k.split("/")[-1]: blob[k] for k in blob.files if k.startswith(name + "/in/")}
        red_s = "MEAN" if red == 0 else "MIN"
        if op == 0:
            a = (t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
            cost, mask = oracle.cost_volume_fwd(*a, red_s, bool(half))
            grads = oracle.cost_volume_bwd(*a, t["cost_grad"], mask, red_s, bool(half))
        elif op == 2:
            a = (t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
            cost, mask = oracle.cost_aggregate_fwd(*a, red_s, bool(half))
            grads = oracle.cost_aggregate_bwd(*a, t["cost_grad"], mask, red_s, bool(half))
        elif op == 3:
            a = (t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
            cost, mask = oracle.cost_volume_v3_fwd(*a, red_s, groups, bool(half))
            grads = oracle.cost_volume_v3_bwd(*a, t["cost_grad"], mask, red_s, groups, bool(half))
        elif op == 4:
            a = (t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
            cost, mask = oracle.feature_aggregate_fwd(*a, bool(half))
            grads = oracle.feature_aggregate_bwd(*a, t["cost_grad"], mask, bool(half))
        else:
            a = (t["ref"], t["src"], t["depth_grid"], t["Rs"], t["Ts"])
            cost, mask = oracle.cost_volume_v2_fwd(*a, red_s, groups, bool(half))
            grads = oracle.cost_volume_v2_bwd(*a, t["cost_grad"], mask, red_s, groups, bool(half))
        assert np.array_equal(cost, blob[name + "/out/cost"]), name
        assert np.array_equal(mask, blob[name + "/out/mask"]), name
        keys = ("src_grad", "depth_grad") if op == 4 else ("ref_grad", "src_grad", "depth_grad")
        for k, g in zip(keys, grads):
            assert np.array_equal(g, blob[name + "/out/" + k]), (name, k)


def test_workload_generator_is_deterministic():
    a = make_workload(2, hw=(8, 10), depth=6)
    b = make_workload(2, hw=(8, 10), depth=6)
    for k in a.tensors:
        assert np.array_equal(a.tensors[k], b.tensors[k])
    digest = hashlib.sha256(a.tensors["Rs"].tobytes() + a.tensors["Ts"].tobytes()).hexdigest()
    assert digest == hashlib.sha256(b.tensors["Rs"].tobytes() + b.tensors["Ts"].tobytes()).hexdigest()
    wl = make_workload(2, with_cost_grad=False)
    assert wl.voxels == 3932160
    assert wl.algorithmic_bytes() == (526992224, 534938464)
    assert make_workload(5, hw=(8, 8), depth=4, batch=1, with_cost_grad=False).N == 6
    x = np.array([1.0, 1.0 + 2 ** -9, 3.14159, -1e-3], np.float32)
    assert np.array_equal(quantise(x, "bf16"),
                          torch.from_numpy(x).to(torch.bfloat16).float().numpy())
    assert np.array_equal(quantise(x, "f16"), x.astype(np.float16).astype(np.float32))
