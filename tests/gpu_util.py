"""Helpers for the GPU parity tests: numpy <-> device tensors and tolerance checks."""
import numpy as np
import torch

TORCH_DTYPE = {"f32": torch.float32, "f64": torch.float64, "f16": torch.float16,
               "bf16": torch.bfloat16}


def dev(x, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(x)).to("cuda")
    return t.to(dtype) if dtype is not None else t


def host(t):
    torch.cuda.synchronize()
    return t.detach().float().cpu().numpy() if t.dtype in (torch.float16, torch.bfloat16) \
        else t.detach().cpu().numpy()


def rms(x):
    return float(np.sqrt(np.mean(np.square(x.astype(np.float64))))) if x.size else 0.0


def floor_only_fraction(got, want, rtol, atol, what=""):
    """Fraction of the elements that meet `|got - want| <= atol + rtol*|want|` only thanks to
    the absolute term, i.e. that miss the purely relative bar; printed, so that a run shows
    how much of a comparison rests on the floor."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    err = np.abs(got - want)
    floor_only = int(np.count_nonzero(err > rtol * np.abs(want)))
    frac = floor_only / max(want.size, 1)
    print("[tolerance] %s%d of %d elements (%.4f%%) pass through the absolute floor %.3g only"
          % (what + ": " if what else "", floor_only, want.size, 100.0 * frac, atol), flush=True)
    return frac


def assert_forward_close(got, want, rtol=1e-5, atol=1e-6, what="forward"):
    """fp32 forward bar: 1e-5 relative, with the reference tests' absolute floor of 1e-6
    (assertAllClose(rtol=1e-5) in cost_volume_op_test.py:209 uses atol=1e-6).  Returns the
    fraction of elements that pass through the floor only."""
    np.testing.assert_allclose(got, want, rtol=rtol, atol=atol)
    return floor_only_fraction(got, want, rtol, atol, what)


def assert_backward_close(got, want, rtol=1e-4, what="backward"):
    """fp32 backward bar: 1e-4 relative.  Sums of many signed terms are compared with an
    absolute floor of rtol * rms(expected): the order in which atomics land changes the
    rounding of each partial sum by a few ulp of the LARGEST partial sum, which for an
    element that cancels to almost zero is far more than rtol of the element itself.
    Returns the fraction of elements that pass through the floor only."""
    atol = rtol * max(rms(want), 1e-30)
    np.testing.assert_allclose(got, want, rtol=rtol, atol=atol)
    return floor_only_fraction(got, want, rtol, atol, what)
