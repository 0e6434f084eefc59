"""The C ABI is re-entrant: the reference's Compute may run concurrently on TensorFlow's
inter-op threads (cost_volume_kernels.cc:59-60 keeps only immutable attributes in the kernel
object).  Four host threads, each with its own stream and its own buffers, drive forward +
backward through the C ABI at the same time; every thread's results are checked against the
CPU oracle."""
import threading

import numpy as np
import pytest
import torch

import custom_helper_op_amd as chop
from custom_helper_op_amd import _lib
from custom_helper_op_amd.configs import make_workload
from gpu_util import assert_backward_close, assert_forward_close, dev, host

pytestmark = pytest.mark.gpu

KEYS = ("ref", "src", "base_plane", "offsets", "Rs", "Ts")


def test_four_host_threads_four_streams(oracle):
    print("\n[case] four host threads on four streams", flush=True)
    lib = _lib.load()
    # different shapes per thread: different kernel instantiations and launch geometries
    shapes = [(2, (32, 40), 48), (2, (24, 32), 64), (1, (32, 40), 32), (5, (16, 24), 32)]
    work = []
    for index, hw, depth in shapes:
        wl = make_workload(index, hw=hw, depth=depth, batch=1)
        t = wl.tensors
        if "cost_grad" not in t:  # the forward-only workload
            t["cost_grad"] = np.random.default_rng(7).standard_normal(
                (wl.B, wl.H, wl.W, wl.D, wl.C)).astype(np.float32)
        want_cost, want_mask = oracle.cost_volume_fwd(*[t[k] for k in KEYS], threads=4)
        want = oracle.cost_volume_bwd(*[t[k] for k in KEYS], t["cost_grad"], want_mask)
        work.append((t, want_cost, want_mask, want))
    results = [None] * len(work)
    errors = []
    start = threading.Barrier(len(work))

    def run(i):
        try:
            t = work[i][0]
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                ins = [dev(t[k]) for k in KEYS]
                cg, mask_in = dev(t["cost_grad"]), dev(work[i][2])
                start.wait()
                out = []
                for _ in range(8):  # several rounds, so that the calls really overlap
                    cost, mask = chop.cost_volume_raw(*ins)
                    grads = chop.cost_volume_grad(*ins, cg, mask_in)
                    assert lib.chop_last_kernel_family() == 2  # thread-local: this thread's call
                    out = [cost, mask, *grads]
                stream.synchronize()
            results[i] = [x.cpu().numpy() for x in out]
        except Exception as e:  # noqa: BLE001 - reported below, in the main thread
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=run, args=(i,)) for i in range(len(work))]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not errors, errors
    for (t, want_cost, want_mask, want), got in zip(work, results):
        assert got is not None
        assert np.array_equal(got[1], want_mask)
        assert_forward_close(got[0], want_cost)
        for g, w in zip(got[2:], want):
            assert_backward_close(g, w)
