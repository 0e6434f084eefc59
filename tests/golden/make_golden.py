"""Writes tests/golden/costvol_golden.npz: small inputs with the CPU oracle's outputs.

The reference holds no vectors for this path and cannot be run here (TensorFlow + CUDA), so
these fixtures are produced by this repository's oracle AFTER it passed the pinning tests
(tests/test_oracle_forward.py, tests/test_oracle_backward.py, tests/test_oracle_aggregate.py,
tests/test_oracle_v3_feature.py).  They freeze its behaviour:
the CPU suite checks that the oracle still reproduces them bit for bit, the GPU suite checks
the HIP library against them.  Run from the repository root:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from custom_helper_op_amd.configs import make_workload, reference_test_case  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "costvol_golden.npz")


def cases():
    """name -> (op, dtype, reduce, groups, half_centor, inputs)"""
    out = {}
    for dt, tag in ((np.float64, "f64"), (np.float32, "f32")):
        for case in (1, 3):
            t = reference_test_case(case, 1, 2, 8, 12, 3, 4, dt, seed=case)
            for red in ("MEAN", "MIN"):
                out["v1_ref%d_%s_%s" % (case, red, tag)] = ("v1", red, 1, True, t)
        t = reference_test_case(1, 1, 2, 8, 12, 9, 4, dt, seed=7)
        t = dict(t)
        t["depth_grid"] = (t["base_plane"] + t["offsets"][:, None, None, :]).astype(dt)
        for red in ("MEAN", "MIN"):
            out["v2_ref1_%s_%s" % (red, tag)] = ("v2", red, 3, True, t)
    wl = make_workload(2, hw=(6, 8), depth=8)
    out["v1_bench2_MEAN_f32"] = ("v1", "MEAN", 1, True, wl.tensors)
    out["v1_bench2_nohalf_MEAN_f32"] = ("v1", "MEAN", 1, False, wl.tensors)
    wl = make_workload(4, hw=(8, 12), batch=1)
    out["v2_bench4_MEAN_f32"] = ("v2", "MEAN", 4, True, wl.tensors)
    # CostAggregate (appended last: the cases above keep their random upstream gradients)
    for dt, tag in ((np.float64, "f64"), (np.float32, "f32")):
        t = reference_test_case(3, 1, 2, 8, 12, 8, 4, dt, seed=11)
        for red in ("MEAN", "MIN"):
            out["agg_ref3_%s_%s" % (red, tag)] = ("agg", red, 1, True, t)
    wl = make_workload(2, hw=(6, 8), depth=8)
    out["agg_bench2_MEAN_f32"] = ("agg", "MEAN", 1, True, wl.tensors)
    # CostVolumeV3 and FeatureAggregate (appended last for the same reason)
    for dt, tag in ((np.float64, "f64"), (np.float32, "f32")):
        t = reference_test_case(3, 1, 2, 8, 12, 9, 4, dt, seed=13)
        t["ref"], t["src"] = t["ref"] - 4, t["src"] - 4   # signed: some maxima stay at the seed
        for red in ("MEAN", "MIN"):
            out["v3_ref3_%s_%s" % (red, tag)] = ("v3", red, 3, True, t)
        t = reference_test_case(3, 1, 2, 8, 12, 4, 4, dt, seed=17)
        out["feat_ref3_%s" % tag] = ("feat", "MEAN", 1, True, t)
    wl = make_workload(2, hw=(6, 8), depth=8)
    out["v3_bench2_MEAN_f32"] = ("v3", "MEAN", 4, True, wl.tensors)
    out["feat_bench2_nohalf_f32"] = ("feat", "MEAN", 1, False, wl.tensors)
    return out


def run(op, red, groups, half, t, cost_grad):
    if op == "v1":
        a = (t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
        cost, mask = oracle.cost_volume_fwd(*a, red, half)
        grads = oracle.cost_volume_bwd(*a, cost_grad(cost), mask, red, half)
    elif op == "agg":
        a = (t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
        cost, mask = oracle.cost_aggregate_fwd(*a, red, half)
        grads = oracle.cost_aggregate_bwd(*a, cost_grad(cost), mask, red, half)
    elif op == "v3":
        a = (t["ref"], t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
        cost, mask = oracle.cost_volume_v3_fwd(*a, red, groups, half)
        grads = oracle.cost_volume_v3_bwd(*a, cost_grad(cost), mask, red, groups, half)
    elif op == "feat":
        a = (t["src"], t["base_plane"], t["offsets"], t["Rs"], t["Ts"])
        cost, mask = oracle.feature_aggregate_fwd(*a, half)
        grads = oracle.feature_aggregate_bwd(*a, cost_grad(cost), mask, half)
    else:
        a = (t["ref"], t["src"], t["depth_grid"], t["Rs"], t["Ts"])
        cost, mask = oracle.cost_volume_v2_fwd(*a, red, groups, half)
        grads = oracle.cost_volume_v2_bwd(*a, cost_grad(cost), mask, red, groups, half)
    return cost, mask, grads


def main():
    blob = {}
    rng = np.random.default_rng(2024)
    for name, (op, red, groups, half, t) in cases().items():
        cg_holder = {}

        def cost_grad(cost):
            cg_holder["cg"] = rng.standard_normal(cost.shape).astype(cost.dtype)
            return cg_holder["cg"]

        cost, mask, grads = run(op, red, groups, half, t, cost_grad)
        keys = ("ref", "src", "Rs", "Ts") + (("depth_grid",) if op == "v2" else ("base_plane", "offsets"))
        if op == "feat":
            keys = keys[1:]
        for k in keys:
            blob[name + "/in/" + k] = t[k]
        blob[name + "/in/cost_grad"] = cg_holder["cg"]
        blob[name + "/attrs"] = np.array([{"v1": 0, "v2": 1, "agg": 2, "v3": 3, "feat": 4}[op], 0 if red == "MEAN" else 1, groups,
                                          int(half)], np.int64)
        blob[name + "/out/cost"] = cost
        blob[name + "/out/mask"] = mask
        names = ("src_grad", "depth_grad") if op == "feat" else ("ref_grad", "src_grad", "depth_grad")
        for k, g in zip(names, grads):
            blob[name + "/out/" + k] = g
    np.savez_compressed(OUT, **blob)
    print("wrote %s: %d cases, %.1f KiB" % (OUT, len(cases()), os.path.getsize(OUT) / 1024))


if __name__ == "__main__":
    main()
