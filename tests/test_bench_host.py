"""bench.py without a GPU: the parts of its contract that are host logic.  More than one GPU is
refused with a message (the operator has no multi-GPU path), and the HBM traffic figures under
profiles/ belong to the kernel sources in the tree (otherwise the benchmark line would withhold
them as stale)."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*flags):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags],
                          capture_output=True, text=True, cwd=ROOT, timeout=120)


def test_more_than_one_gpu_is_refused():
    r = _run("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in r.stderr and "--gpus 2" in r.stderr
    assert r.stdout.strip() == ""      # no JSON line that could be taken for a measurement


def test_traffic_counters_belong_to_the_sources_in_the_tree():
    r = _run("--print-kernel-hashes")
    assert r.returncode == 0, r.stderr
    now = json.loads(r.stdout)["kernel_sources"]
    with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
        recorded = json.load(f)
    assert recorded["kernel_sources"] == now
    t = recorded["mvsnet_stage"]
    for direction in ("forward", "backward"):
        assert t[direction]["fetch_bytes"] > 0 and t[direction]["write_bytes"] > 0
