"""The entry point that allocates nothing (chop_cost_volume_bwd_16_static) against the entry
point it is a variant of (chop_cost_volume_bwd_16 with a caller workspace), through the C
ABI: two calls in a row on one GPU, the second with a smaller input, so that what the first
call left in the shared static scratch must not leak into the second.  Both are also held to
the 16-bit bar (1e-2) against the CPU oracle."""
import numpy as np
import pytest
import torch

from custom_helper_op_amd import _lib
from custom_helper_op_amd.configs import make_workload, quantise
from gpu_util import TORCH_DTYPE, dev, host, rms

pytestmark = pytest.mark.gpu

_STORAGE = {"f16": 1, "bf16": 2}


def _ptr(t):
    return t.data_ptr() if t is not None else None


def _run_both(lib, wl, storage, oracle):
    """Runs the workspace entry point and the static-scratch one on the same device inputs."""
    t = wl.tensors
    td = TORCH_DTYPE[storage]
    ref, src, cg = (quantise(t[k], storage) for k in ("ref", "src", "cost_grad"))
    _, want_mask = oracle.cost_volume_fwd(ref, src, t["base_plane"], t["offsets"], t["Rs"], t["Ts"],
                                          threads=8)
    want = oracle.cost_volume_bwd(ref, src, t["base_plane"], t["offsets"], t["Rs"], t["Ts"], cg,
                                  want_mask)
    d_ref, d_src, d_cg = dev(ref, td), dev(src, td), dev(cg, td)
    d_bp, d_off, d_rs, d_ts = (dev(t[k]) for k in ("base_plane", "offsets", "Rs", "Ts"))
    d_mask = dev(want_mask)
    dims = (wl.B, wl.H, wl.W, wl.C, wl.D, wl.N, wl.H, wl.W)
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for static in (False, True):
        rg, sg = torch.empty_like(d_ref), torch.empty_like(d_src)
        bg = torch.empty_like(d_bp)
        # garbage in the outputs: the entry points must overwrite every element
        rg.fill_(7.0), sg.fill_(-3.0), bg.fill_(11.0)
        common = (stream, _STORAGE[storage], 0, 1, *dims, _ptr(d_ref), _ptr(d_src), _ptr(d_bp),
                  _ptr(d_off), None, _ptr(d_rs), _ptr(d_ts), _ptr(d_cg), _ptr(d_mask), _ptr(rg),
                  _ptr(sg), _ptr(bg))
        if static:
            rc = lib.chop_cost_volume_bwd_16_static(*common)
        else:
            need = lib.chop_cost_volume_bwd16_workspace_bytes(wl.B, wl.H, wl.W, wl.C, wl.N, wl.H,
                                                              wl.W)
            ws = torch.empty(need, dtype=torch.uint8, device="cuda")
            rc = lib.chop_cost_volume_bwd_16(*common, _ptr(ws), need)
        _lib.check(rc)
        assert lib.chop_last_kernel_family() == 2  # the tiled kernels served the call
        outs.append([host(x) for x in (rg, sg, bg)])
    return outs, want


@pytest.mark.parametrize("storage", ["f16", "bf16"])
def test_static_scratch_entry_matches_workspace_entry(oracle, storage):
    lib = _lib.load()
    lib.chop_set_kernel_family(0)
    # the larger call first: the second, smaller one runs over what it left in the scratch
    for hw in ((64, 80), (24, 40)):
        print("\n[case] static scratch %s %dx%d" % (storage, hw[0], hw[1]), flush=True)
        wl = make_workload(3, hw=hw)
        assert lib.chop_cost_volume_bwd16_workspace_bytes(
            wl.B, wl.H, wl.W, wl.C, wl.N, wl.H, wl.W) <= lib.chop_static_scratch_bytes()
        (with_ws, with_static), want = _run_both(lib, wl, storage, oracle)
        for a, b, w in zip(with_ws, with_static, want):
            floor = 1e-2 * max(rms(w), 1e-30)
            # the same kernels on the same inputs: the two differ by the order in which the
            # atomics landed, far inside the 16-bit bar
            np.testing.assert_allclose(b, a, rtol=1e-2, atol=floor)
            np.testing.assert_allclose(b, w, rtol=1e-2, atol=floor)


def test_static_scratch_entry_rejects_oversized_shapes():
    lib = _lib.load()
    limit = lib.chop_static_scratch_bytes()
    assert limit == 32 << 20
    # validation happens before any pointer is touched
    B, H, W, C, D, N = 1, 1024, 1024, 32, 4, 4
    assert lib.chop_cost_volume_bwd16_workspace_bytes(B, H, W, C, N, H, W) > limit
    one = torch.zeros(1, device="cuda")
    p = one.data_ptr()
    rc = lib.chop_cost_volume_bwd_16_static(torch.cuda.current_stream().cuda_stream, 1, 0, 1, B, H,
                                            W, C, D, N, H, W, p, p, p, p, None, p, p, p, p, p, p, p)
    assert rc == 6  # CHOP_ERR_WORKSPACE
    assert b"built-in scratch" in lib.chop_last_error_string()


def test_static_scratch_entry_in_a_captured_graph(oracle):
    """The entry point captured into a HIP graph (chop_init() made the one runtime query
    beforehand) and replayed on changed inputs, with eager work and synchronisations
    between the replays: every replay against the oracle for the inputs of that replay."""
    lib = _lib.load()
    lib.chop_set_kernel_family(0)
    _lib.check(lib.chop_init())
    storage = "f16"
    td = TORCH_DTYPE[storage]
    wl = make_workload(3, hw=(24, 40))
    t = wl.tensors
    rng = np.random.default_rng(7)
    ref, src = quantise(t["ref"], storage), quantise(t["src"], storage)
    _, want_mask = oracle.cost_volume_fwd(ref, src, t["base_plane"], t["offsets"], t["Rs"], t["Ts"],
                                          threads=8)
    d_ref, d_src = dev(ref, td), dev(src, td)
    d_cg = dev(quantise(t["cost_grad"], storage), td)
    d_bp, d_off, d_rs, d_ts = (dev(t[k]) for k in ("base_plane", "offsets", "Rs", "Ts"))
    d_mask = dev(want_mask)
    rg, sg, bg = torch.empty_like(d_ref), torch.empty_like(d_src), torch.empty_like(d_bp)
    dims = (wl.B, wl.H, wl.W, wl.C, wl.D, wl.N, wl.H, wl.W)

    def call(stream):
        return lib.chop_cost_volume_bwd_16_static(
            stream, _STORAGE[storage], 0, 1, *dims, _ptr(d_ref), _ptr(d_src), _ptr(d_bp),
            _ptr(d_off), None, _ptr(d_rs), _ptr(d_ts), _ptr(d_cg), _ptr(d_mask), _ptr(rg),
            _ptr(sg), _ptr(bg))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _lib.check(call(side.cuda_stream))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        _lib.check(call(torch.cuda.current_stream().cuda_stream))
    for replay in range(3):
        print("\n[case] captured static-scratch backward, replay %d" % replay, flush=True)
        new_ref = quantise(rng.standard_normal(ref.shape).astype(np.float32), storage)
        new_cg = quantise(rng.standard_normal(t["cost_grad"].shape).astype(np.float32), storage)
        d_ref.copy_(dev(new_ref, td))
        d_cg.copy_(dev(new_cg, td))
        rg.fill_(7.0), sg.fill_(-3.0), bg.fill_(11.0)   # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = oracle.cost_volume_bwd(new_ref, src, t["base_plane"], t["offsets"], t["Rs"], t["Ts"],
                                      new_cg, want_mask)
        for got, w in zip((rg, sg, bg), want):
            np.testing.assert_allclose(host(got), w, rtol=1e-2, atol=1e-2 * max(rms(w), 1e-30))
