"""Benchmark of the cost-volume hot path on one MI355X.

A step is one forward + one backward of the operator (through the C ABI) on one batch of
synthetic input that is already resident in HBM.  Prints one JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload 2] [--no-cpu-baseline]
                  [--no-configs]

``value`` and ``ms_per_step`` are wall-clock over exactly K back-to-back steps.  The
``roofline`` object is per call: HIP-event times of the dominant kernel's entry point with
nothing of the workload in L2 or the memory-side cache (cold: a 1 GiB buffer is overwritten
and then read before every call, so the caches hold clean lines of foreign data), the times
right after the overwrite alone (every line dirty: the call also waits for the write-back of
another kernel's output) and the back-to-back (warm) times beside them, and the rate a plain
fill / copy reaches on this box in the same run.
``configs`` holds the cold forward / backward times of all five benchmark configurations.

The default run is the headline configuration (workload 2, MEAN).  ``--reduce MIN``,
``--aggregate`` (CostAggregate), ``--v3 GROUPS`` (CostVolumeV3) and ``--feature``
(FeatureAggregate), all on the same tensors and for float32 workloads only, time the other
entry points for the tables under profiles/.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published


KERNEL_SOURCES = ("custom_helper_op_amd/csrc/tiled.h", "custom_helper_op_amd/csrc/tiled_launch.inc")


def kernel_source_hashes():
    """git blob hashes (sha1 of "blob <size>\\0" + content) of the sources of the tiled
    kernels.  profiles/hbm_traffic.json records them beside the counters; bench.py reports
    the traffic figure only while they still match (``python bench.py --print-kernel-hashes``
    prints the current ones for that file)."""
    import hashlib
    out = {}
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            data = f.read()
        out[rel] = hashlib.sha1(b"blob %d\0" % len(data) + data).hexdigest()
    return out


class Runner:
    """Pre-allocated buffers + direct C-ABI calls, so a step enqueues kernels and nothing else."""

    def __init__(self, wl, torch, lib):
        self.wl, self.torch, self.lib = wl, torch, lib
        t = wl.tensors
        td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16,
              "f64": torch.float64}[wl.storage]
        self.storage_code = {"f32": 0, "f16": 1, "bf16": 2, "f64": 0}[wl.storage]
        self.f64 = wl.storage == "f64"  # depths, cameras and depth gradients are float64 too
        real = torch.float64 if self.f64 else None
        d = "cuda:0"
        up = lambda k, dt=real: (torch.from_numpy(t[k]).to(d) if dt is None
                                 else torch.from_numpy(t[k]).to(d).to(dt))
        self.ref, self.src = up("ref", td), up("src", td)
        self.Rs, self.Ts = up("Rs"), up("Ts")
        self.v2 = wl.op == "v2"
        self.grid = wl.op == "v1" and wl.grid_form  # squared difference over a depth grid (16-bit only)
        self.agg = wl.op == "agg"
        self.v3, self.feat = wl.op == "v3", wl.op == "feat"
        self.red = 0 if wl.reduce_method == "MEAN" else 1
        if self.v2 or self.grid:
            self.depth_grid = up("depth_grid")
        else:
            self.base_plane, self.offsets = up("base_plane"), up("offsets")
        B, H, W, D, OC = wl.B, wl.H, wl.W, wl.D, wl.out_channels
        self.cost = torch.empty((B, H, W, D, OC), dtype=td, device=d)
        mask_last = wl.N if self.feat else 1 if self.red == 0 else 3 if self.v3 else OC
        self.mask = torch.empty((B, H, W, D, mask_last), dtype=torch.int32, device=d)
        gen = torch.Generator(device=d)
        gen.manual_seed(wl.seed)
        self.cost_grad = torch.randn((B, H, W, D, OC), dtype=torch.float32, device=d,
                                     generator=gen).to(td)
        self.ref_grad = torch.empty_like(self.ref)
        self.src_grad = torch.empty_like(self.src)
        self.depth_grad = torch.empty((B, H, W, D) if self.v2 or self.grid else (B, H, W, 1),
                                      dtype=real or torch.float32, device=d)
        self.dims = (B, H, W, wl.C, D, wl.N, H, W)
        self.ws = None
        self.ws_bytes = 0
        if self.storage_code:
            self.ws_bytes = lib.chop_cost_volume_bwd16_workspace_bytes(B, H, W, wl.C, wl.N, H, W)
            self.ws = torch.empty(max(self.ws_bytes, 256), dtype=torch.uint8, device=d)
        self.stream = torch.cuda.current_stream().cuda_stream

    def forward(self):
        p = lambda x: x.data_ptr()
        lib, s = self.lib, self.stream
        if self.v2:
            if self.storage_code:
                rc = lib.chop_cost_volume_v2_fwd_16(s, self.storage_code, self.red, 1, *self.dims,
                                                    self.wl.groups, p(self.ref), p(self.src),
                                                    p(self.depth_grid), p(self.Rs), p(self.Ts),
                                                    p(self.cost), p(self.mask))
            else:
                rc = lib.chop_cost_volume_v2_fwd_f32(s, self.red, 1, *self.dims, self.wl.groups,
                                                     p(self.ref), p(self.src), p(self.depth_grid),
                                                     p(self.Rs), p(self.Ts), p(self.cost),
                                                     p(self.mask))
        elif self.agg:
            fn = lib.chop_cost_aggregate_fwd_f64 if self.f64 else lib.chop_cost_aggregate_fwd_f32
            rc = fn(s, self.red, 1, *self.dims, p(self.ref), p(self.src), p(self.base_plane),
                    p(self.offsets), p(self.Rs), p(self.Ts), p(self.cost), p(self.mask))
        elif self.v3:
            fn = lib.chop_cost_volume_v3_fwd_f64 if self.f64 else lib.chop_cost_volume_v3_fwd_f32
            rc = fn(s, self.red, 1, *self.dims, self.wl.groups, p(self.ref), p(self.src),
                    p(self.base_plane), p(self.offsets), p(self.Rs), p(self.Ts), p(self.cost),
                    p(self.mask))
        elif self.feat:
            fn = lib.chop_feature_aggregate_fwd_f64 if self.f64 else lib.chop_feature_aggregate_fwd_f32
            rc = fn(s, 1, *self.dims, p(self.src), p(self.base_plane), p(self.offsets), p(self.Rs),
                    p(self.Ts), p(self.cost), p(self.mask))
        elif self.grid:
            rc = lib.chop_cost_volume_fwd_16(s, self.storage_code, self.red, 1, *self.dims, p(self.ref),
                                             p(self.src), None, None, p(self.depth_grid),
                                             p(self.Rs), p(self.Ts), p(self.cost), p(self.mask))
        elif self.storage_code:
            rc = lib.chop_cost_volume_fwd_16(s, self.storage_code, self.red, 1, *self.dims, p(self.ref),
                                             p(self.src), p(self.base_plane), p(self.offsets), None,
                                             p(self.Rs), p(self.Ts), p(self.cost), p(self.mask))
        else:
            fn = lib.chop_cost_volume_fwd_f64 if self.f64 else lib.chop_cost_volume_fwd_f32
            rc = fn(s, self.red, 1, *self.dims, p(self.ref), p(self.src), p(self.base_plane),
                    p(self.offsets), p(self.Rs), p(self.Ts), p(self.cost), p(self.mask))
        if rc:
            raise RuntimeError(lib.chop_last_error_string().decode())

    def backward(self):
        p = lambda x: x.data_ptr()
        lib, s = self.lib, self.stream
        tail = (p(self.cost_grad), p(self.mask), p(self.ref_grad), p(self.src_grad),
                p(self.depth_grad))
        if self.v2:
            if self.storage_code:
                rc = lib.chop_cost_volume_v2_bwd_16(s, self.storage_code, self.red, 1, *self.dims,
                                                    self.wl.groups, p(self.ref), p(self.src),
                                                    p(self.depth_grid), p(self.Rs), p(self.Ts),
                                                    *tail, p(self.ws), self.ws_bytes)
            else:
                rc = lib.chop_cost_volume_v2_bwd_f32(s, self.red, 1, *self.dims, self.wl.groups,
                                                     p(self.ref), p(self.src), p(self.depth_grid),
                                                     p(self.Rs), p(self.Ts), *tail)
        elif self.agg:
            fn = lib.chop_cost_aggregate_bwd_f64 if self.f64 else lib.chop_cost_aggregate_bwd_f32
            rc = fn(s, self.red, 1, *self.dims, p(self.ref), p(self.src), p(self.base_plane),
                    p(self.offsets), p(self.Rs), p(self.Ts), *tail)
        elif self.v3:
            fn = lib.chop_cost_volume_v3_bwd_f64 if self.f64 else lib.chop_cost_volume_v3_bwd_f32
            rc = fn(s, self.red, 1, *self.dims, self.wl.groups, p(self.ref), p(self.src),
                    p(self.base_plane), p(self.offsets), p(self.Rs), p(self.Ts), *tail)
        elif self.feat:
            fn = lib.chop_feature_aggregate_bwd_f64 if self.f64 else lib.chop_feature_aggregate_bwd_f32
            rc = fn(s, 1, *self.dims, p(self.src), p(self.base_plane), p(self.offsets), p(self.Rs),
                    p(self.Ts), p(self.cost_grad), p(self.mask), p(self.src_grad), p(self.depth_grad))
        elif self.grid:
            rc = lib.chop_cost_volume_bwd_16(s, self.storage_code, self.red, 1, *self.dims, p(self.ref),
                                             p(self.src), None, None, p(self.depth_grid),
                                             p(self.Rs), p(self.Ts), *tail, p(self.ws),
                                             self.ws_bytes)
        elif self.storage_code:
            rc = lib.chop_cost_volume_bwd_16(s, self.storage_code, self.red, 1, *self.dims, p(self.ref),
                                             p(self.src), p(self.base_plane), p(self.offsets), None,
                                             p(self.Rs), p(self.Ts), *tail, p(self.ws),
                                             self.ws_bytes)
        else:
            fn = lib.chop_cost_volume_bwd_f64 if self.f64 else lib.chop_cost_volume_bwd_f32
            rc = fn(s, self.red, 1, *self.dims, p(self.ref), p(self.src), p(self.base_plane),
                    p(self.offsets), p(self.Rs), p(self.Ts), *tail)
        if rc:
            raise RuntimeError(lib.chop_last_error_string().decode())


def cpu_baseline(wl, budget_s=12.0):
    """The CPU oracle (a port of the reference kernel's per-voxel loop; the reference has
    no CPU kernel of its own) on the same workload, all host threads the box grants."""
    import numpy as np
    import oracle
    from custom_helper_op_amd.configs import quantise
    threads = max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")), 16))
    t = wl.tensors
    rng = np.random.default_rng(wl.seed)
    # bounded sample: a horizontal band of the image (all views, all depth hypotheses)
    rows = wl.H
    est_voxel_rate = 4.0e6 * threads  # voxel*view*channel/32 per second, conservative
    work = wl.voxels * wl.N * wl.C / 32.0
    if work / est_voxel_rate > budget_s:
        rows = max(8, int(wl.H * budget_s * est_voxel_rate / work))
    sl = slice(0, rows)
    ref, src = t["ref"][:, sl], t["src"]
    cg = quantise(rng.standard_normal((wl.B, rows, wl.W, wl.D, wl.out_channels), dtype=np.float32),
                  wl.storage)
    times = []
    out = None
    if wl.op in ("v1", "v2"):  # the large outputs exist (and are touched) before the clock starts
        oc = wl.out_channels
        out = (np.zeros((wl.B, rows, wl.W, wl.D, oc), np.float32),
               np.zeros((wl.B, rows, wl.W, wl.D, 1 if wl.reduce_method == "MEAN" else oc), np.int32))
    for _ in range(3):
        t0 = time.perf_counter()
        if wl.op == "v1":
            bp = t["base_plane"][:, sl]
            args = (ref, src, bp, t["offsets"], t["Rs"], t["Ts"])
            _, mask = oracle.cost_volume_fwd(*args, wl.reduce_method, threads=threads, out=out)
            oracle.cost_volume_bwd(*args, cg, mask, wl.reduce_method, threads=threads)
        elif wl.op == "agg":
            bp = t["base_plane"][:, sl]
            args = (ref, src, bp, t["offsets"], t["Rs"], t["Ts"])
            _, mask = oracle.cost_aggregate_fwd(*args, wl.reduce_method, threads=threads)
            oracle.cost_aggregate_bwd(*args, cg[..., 0], mask, wl.reduce_method, threads=threads)
        elif wl.op == "v3":
            bp = t["base_plane"][:, sl]
            args = (ref, src, bp, t["offsets"], t["Rs"], t["Ts"])
            _, mask = oracle.cost_volume_v3_fwd(*args, wl.reduce_method, wl.groups, threads=threads)
            oracle.cost_volume_v3_bwd(*args, cg, mask, wl.reduce_method, wl.groups)
        elif wl.op == "feat":
            bp = t["base_plane"][:, sl]
            args = (src, bp, t["offsets"], t["Rs"], t["Ts"])
            _, mask = oracle.feature_aggregate_fwd(*args, threads=threads)
            oracle.feature_aggregate_bwd(*args, cg.reshape(wl.B, rows, wl.W, wl.D, wl.N, wl.C), mask)
        else:
            dg = t["depth_grid"][:, sl]
            args = (ref, src, dg, t["Rs"], t["Ts"])
            _, mask = oracle.cost_volume_v2_fwd(*args, wl.reduce_method, wl.groups, threads=threads,
                                                out=out)
            oracle.cost_volume_v2_bwd(*args, cg, mask, wl.reduce_method, wl.groups, threads=threads)
        times.append(time.perf_counter() - t0)
        if sum(times) > budget_s:
            break
    times.sort()
    med = times[len(times) // 2]
    vox = wl.B * rows * wl.W * wl.D
    return {"value": vox / med, "unit": "voxels/s", "cores": threads, "kind": "port",
            "sample": "%s rows 0..%d of %d (all views, all %d depths), fwd+bwd, median of %d, "
                      "cost and mask pre-allocated" % (wl.name, rows, wl.H, wl.D, len(times))}


def timed_passes(torch, r, passes, scratch, read_back=True):
    """`passes` forward + backward calls with HIP events on the launch stream around each
    call.  With `scratch` (a 1 GiB buffer) every call is preceded by an overwrite of it, so
    that L2 and the memory-side cache hold nothing of the workload: cold-cache times.  With
    `read_back` the buffer is then read once, which leaves the caches full of clean lines;
    without, every line is dirty and the first misses of the call push out another kernel's
    output (kernels whose loads allocate in the caches then wait for those write-backs)."""
    ev = lambda: torch.cuda.Event(enable_timing=True)
    marks = []
    sink = torch.zeros((), dtype=torch.float32, device="cuda:0") if scratch is not None else None

    def flush(value):
        if scratch is not None:
            scratch.fill_(value)
            if read_back:
                sink.add_(scratch.sum())

    for _ in range(passes):
        e0, e1, e2, e3 = ev(), ev(), ev(), ev()
        flush(1.0)
        e0.record()
        r.forward()
        e1.record()
        flush(2.0)
        e2.record()
        r.backward()
        e3.record()
        marks.append((e0, e1, e2, e3))
    torch.cuda.synchronize()
    med = lambda v: sorted(v)[len(v) // 2]
    return (med([m[0].elapsed_time(m[1]) for m in marks]),
            med([m[2].elapsed_time(m[3]) for m in marks]))


def stream_rates(torch):
    """What this box's HBM gives a plain kernel, measured in this run: a 512 MiB fill
    (write-only, the forward's pattern) and a 256 MiB copy (read + write)."""
    n = 128 * 1024 * 1024
    a = torch.empty(n, dtype=torch.float32, device="cuda:0")
    b = torch.empty(n // 2, dtype=torch.float32, device="cuda:0")
    ev = lambda: torch.cuda.Event(enable_timing=True)
    fills, copies = [], []
    for i in range(7):
        e0, e1, e2 = ev(), ev(), ev()
        e0.record()
        a.fill_(float(i))
        e1.record()
        b.copy_(a[:n // 2])
        e2.record()
        torch.cuda.synchronize()
        if i >= 2:
            fills.append(e0.elapsed_time(e1))
            copies.append(e1.elapsed_time(e2))
    med = lambda v: sorted(v)[len(v) // 2]
    del a, b
    return {"fill_GBs": n * 4 / (med(fills) * 1e-3) / 1e9,
            "copy_GBs": n * 4 / (med(copies) * 1e-3) / 1e9}  # copy: n/2 read + n/2 written


def other_configs(torch, lib, make_workload, skip_index, scratch):
    """Forward / backward event times of the BASELINE configurations the headline line is not
    quoted on, each against its own algorithmic bytes (cold-cache, median of 9 after 30 steps)."""
    out = {}
    for index, grid_form in ((1, False), (2, False), (3, False), (3, True), (4, False), (5, False)):
        if index == skip_index:
            continue
        wl = make_workload(index, with_cost_grad=False)
        if grid_form:  # the cascade stage's exact per-pixel hypotheses, coarse * (1 + 0.02 k)
            wl.grid_form = True
            wl.name += "_depth_grid"
        r = Runner(wl, torch, lib)
        # (as for the headline workload: the clock settles over the first ~30 steps after the
        # idle time in which the workload's tensors were generated on the host)
        for _ in range(30):
            r.forward()
            r.backward()
        torch.cuda.synchronize()
        fwd_ms, bwd_ms = timed_passes(torch, r, 9, scratch)
        dirty_fwd, dirty_bwd = timed_passes(torch, r, 9, scratch, read_back=False)
        fwd_b, bwd_b = wl.algorithmic_bytes()
        frac = lambda b, ms: b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS
        out[wl.name] = {
            "workload": "%s B%d N%d %dx%d C%d D%d %s%s" % (
                {"v1": "CostVolume", "v2": "CostVolumeV2"}[wl.op], wl.B, wl.N, wl.H, wl.W, wl.C,
                wl.D, wl.storage, " over depth_grid" if grid_form else ""),
            "voxels": wl.voxels, "forward_ms": fwd_ms, "backward_ms": bwd_ms,
            "forward_frac": frac(fwd_b, fwd_ms), "backward_frac": frac(bwd_b, bwd_ms),
            "fwd_bwd_frac": frac(fwd_b + bwd_b, fwd_ms + bwd_ms),
            "voxels_per_s": wl.voxels / ((fwd_ms + bwd_ms) * 1e-3),
            "after_overwrite_ms": {"forward": dirty_fwd, "backward": dirty_bwd},
            "backward_window_rows": lib.chop_last_backward_window()}
        del r
        torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # (the defaults give the GPU's clocks time to settle: the first ~30 steps after an idle
    # period run up to 15 % slower than the steady state)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--workload", type=int, default=2)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the forward/backward times of the other BASELINE configurations")
    ap.add_argument("--reduce", choices=["MEAN", "MIN"], default="MEAN")
    ap.add_argument("--aggregate", action="store_true",
                    help="time CostAggregate on the workload's tensors (float32 CostVolume workloads)")
    ap.add_argument("--v3", type=int, default=0, metavar="GROUPS",
                    help="time CostVolumeV3 with this many channel groups on the workload's tensors")
    ap.add_argument("--feature", action="store_true",
                    help="time FeatureAggregate on the workload's tensors")
    ap.add_argument("--float64", action="store_true",
                    help="time a float32 CostVolume workload's tensors as float64 (strip kernels)")
    ap.add_argument("--channels", type=int, default=0, metavar="C",
                    help="keep only the first C feature channels of a float32 CostVolume workload")
    ap.add_argument("--kernel-family", choices=["auto", "general", "strip"], default="auto",
                    help="force the one-thread-per-element or the strip kernels instead of the "
                         "library's own choice")
    ap.add_argument("--backward-window", type=int, choices=[0, 6, 8], default=0,
                    help="fix the choice between the two 32-channel gradient kernels (6: four waves "
                         "per SIMD, 6 x 8 scatter window; 8: three waves, 8 x 8) instead of the "
                         "library's own (0)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 256 MiB device copy, as the known-size reference "
                         "that HBM traffic counters of a profiler run are scaled by")
    ap.add_argument("--print-kernel-hashes", action="store_true",
                    help="print the git blob hashes of the tiled kernels' sources and exit")
    a = ap.parse_args()
    if a.print_kernel_hashes:
        print(json.dumps({"kernel_sources": kernel_source_hashes()}, indent=2))
        return
    if a.gpus != 1:
        sys.exit("bench.py: this operator runs on one GPU; --gpus %d is not supported "
                 "(there is no multi-GPU path to measure)" % a.gpus)
    import torch
    from custom_helper_op_amd import _lib
    from custom_helper_op_amd.configs import make_workload
    lib = _lib.load()
    lib.chop_set_kernel_family({"auto": 0, "general": 1, "strip": 2}[a.kernel_family])
    lib.chop_set_backward_window(a.backward_window)
    wl = make_workload(a.workload, with_cost_grad=False)
    wl.reduce_method = a.reduce
    if a.float64 or a.channels:
        if wl.op != "v1" or wl.storage != "f32":
            sys.exit("bench.py: --float64 / --channels need a float32 CostVolume workload (1, 2 or 5), "
                     "alone or with --aggregate / --v3 / --feature")
        if a.channels:
            if not 1 <= a.channels <= wl.C:
                sys.exit("bench.py: --channels must be 1..%d for this workload" % wl.C)
            import numpy as np
            wl.C = a.channels
            for k in ("ref", "src"):
                wl.tensors[k] = np.ascontiguousarray(wl.tensors[k][..., :wl.C])
        if a.float64:
            wl.storage = "f64"
    if a.aggregate:
        if wl.op != "v1" or wl.storage not in ("f32", "f64"):
            sys.exit("bench.py: --aggregate needs a float32 CostVolume workload (1, 2 or 5)")
        wl.op = "agg"
    if a.v3 or a.feature:
        if wl.op != "v1" or wl.storage not in ("f32", "f64"):
            sys.exit("bench.py: --v3 / --feature need a float32 CostVolume workload (1, 2 or 5)")
        wl.op = "v3" if a.v3 else "feat"
        wl.groups = a.v3 if a.v3 else 1
    r = Runner(wl, torch, lib)
    r.forward()
    served = [lib.chop_last_kernel_family()]
    r.backward()
    served.append(lib.chop_last_kernel_family())
    # which of the two 32-channel gradient kernels the launcher took (0: the shape has one only)
    backward_window = lib.chop_last_backward_window()
    served = "/".join({1: "general", 2: "tiled", 3: "strip"}.get(c, str(c)) for c in served)
    for _ in range(a.warmup):
        r.forward()
        r.backward()
    torch.cuda.synchronize()
    if a.calibrate_copy:
        n = 256 * 1024 * 1024 // 4
        src_buf = torch.ones(n, dtype=torch.float32, device="cuda:0")
        dst_buf = torch.empty_like(src_buf)
        for _ in range(3):
            dst_buf.copy_(src_buf)
        torch.cuda.synchronize()
        del src_buf, dst_buf
    # the timed region: exactly `steps` steps, nothing else enqueued in between
    t0 = time.perf_counter()
    for _ in range(a.steps):
        r.forward()
        r.backward()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / a.steps
    # the same K steps as one captured HIP graph (the entry points only enqueue kernels): what
    # a caller who removes the host's launch gaps gets; reported beside ms_per_step, never as it
    graph_ms = None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        eager_stream, r.stream = r.stream, side.cuda_stream
        with torch.cuda.stream(side):
            r.forward()
            r.backward()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(a.steps):
                r.forward()
                r.backward()
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) * 1e3 / a.steps
        del graph
    except Exception as e:  # a profiler or an old runtime may refuse the capture
        print("bench.py: graph replay skipped: %s" % e, file=sys.stderr)
    finally:
        r.stream = eager_stream
    # per-call times, outside the timed region: warm (back to back, as above), cold (a foreign
    # buffer overwritten and read before every call) and right after the overwrite alone; the
    # roofline line is the cold one
    warm_fwd, warm_bwd = timed_passes(torch, r, max(a.steps, 5), None)
    scratch = torch.empty(1 << 28, dtype=torch.float32, device="cuda:0")
    fwd_ms, bwd_ms = timed_passes(torch, r, max(a.steps, 5), scratch)
    dirty_fwd, dirty_bwd = timed_passes(torch, r, max(a.steps, 5), scratch, read_back=False)
    dirty_ms = dirty_bwd if bwd_ms >= fwd_ms else dirty_fwd
    fwd_b, bwd_b = wl.algorithmic_bytes()
    dominant = "backward" if bwd_ms >= fwd_ms else "forward"
    d_ms, d_b = (bwd_ms, bwd_b) if dominant == "backward" else (fwd_ms, fwd_b)
    w_ms = warm_bwd if dominant == "backward" else warm_fwd
    achieved = d_b / (d_ms * 1e-3) / 1e9
    traffic = None
    traffic_source = None
    traffic_stale = None
    try:  # HBM bytes per launch from rocprofv3 counters of a separate run of this command
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            plain = wl.op in ("v1", "v2") and a.reduce == "MEAN" and not (a.float64 or a.channels)
            recorded = json.load(f)
            t = recorded[wl.name if plain and a.kernel_family == "auto" else "-"][dominant]
        # the counters belong to the kernel sources they were taken on: a figure measured on
        # other sources is withheld, not reported
        traffic_stale = recorded.get("kernel_sources") != kernel_source_hashes()
        if not traffic_stale:
            traffic = t["fetch_bytes"] + t["write_bytes"]
        traffic_source = "profiles/hbm_traffic.json (rocprofv3 FETCH_SIZE/WRITE_SIZE of a separate run)"
    except (OSError, KeyError, ValueError):
        pass
    rates = stream_rates(torch)
    stream = rates["copy_GBs"] if dominant == "backward" else rates["fill_GBs"]
    out = {
        "metric": "cost-volume voxels/s (B*D*H*W) fwd+bwd",
        "value": wl.voxels / (ms_per_step * 1e-3),
        "unit": "voxels/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms_per_step,
        "graph_replay_ms_per_step": graph_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": wl.storage, "data": "synthetic",
        "config": {"workload": "%s: %s B%d N%d %dx%d C%d D%d%s %s fwd+bwd" % (
            wl.name, {"v1": "CostVolume", "v2": "CostVolumeV2", "agg": "CostAggregate", "v3": "CostVolumeV3",
                      "feat": "FeatureAggregate"}[wl.op],
            wl.B, wl.N, wl.H, wl.W,
            wl.C, wl.D, " G%d" % wl.groups if wl.op in ("v2", "v3") else "", wl.storage),
            "voxels": wl.voxels, "reduce_method": wl.reduce_method, "half_centor": True,
            "kernels": served, "backward_window_rows": backward_window},
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": achieved,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "timing": "HIP events on the launch stream, a foreign 1 GiB buffer overwritten and then "
                               "read before each call (caches cold and clean), median",
                     "traffic": traffic, "traffic_source": traffic_source,
                     "traffic_stale": traffic_stale,
                     "algorithmic_bytes": {"forward": fwd_b, "backward": bwd_b},
                     "ms": {"forward": fwd_ms, "backward": bwd_ms},
                     "fwd_bwd_frac": (fwd_b + bwd_b) / ((fwd_ms + bwd_ms) * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "warm": {"ms": {"forward": warm_fwd, "backward": warm_bwd},
                              "frac": d_b / (w_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                              "fwd_bwd_frac": (fwd_b + bwd_b) / ((warm_fwd + warm_bwd) * 1e-3) / 1e9
                                              / HBM_PEAK_GBS},
                     "after_overwrite": {"ms": {"forward": dirty_fwd, "backward": dirty_bwd},
                                         "frac": d_b / (dirty_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                         "fwd_bwd_frac": (fwd_b + bwd_b) / ((dirty_fwd + dirty_bwd) * 1e-3)
                                                         / 1e9 / HBM_PEAK_GBS,
                                         "note": "the 1 GiB buffer overwritten and not read: every cache "
                                                 "line dirty with foreign data when the call starts"},
                     "measured_stream_GBs": stream,
                     "measured_stream": {**rates, "used": "copy" if dominant == "backward" else "fill"},
                     "frac_of_measured_stream": achieved / stream},
    }
    if not a.no_configs and wl.op in ("v1", "v2") and a.reduce == "MEAN":
        del r
        torch.cuda.empty_cache()
        out["configs"] = other_configs(torch, lib, make_workload, a.workload, scratch)
        out["configs"][wl.name] = {
            "workload": "headline", "voxels": wl.voxels, "forward_ms": fwd_ms, "backward_ms": bwd_ms,
            "forward_frac": fwd_b / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "backward_frac": bwd_b / (bwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "fwd_bwd_frac": out["roofline"]["fwd_bwd_frac"],
            "voxels_per_s": wl.voxels / ((fwd_ms + bwd_ms) * 1e-3)}
    if not a.no_cpu_baseline and not a.float64:  # (the checker is timed in the workload's own type)
        out["cpu_baseline"] = cpu_baseline(wl)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
