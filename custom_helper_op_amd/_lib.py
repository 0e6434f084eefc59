"""ctypes binding of ``libchop_costvol.so`` (the C ABI declared in include/chop_costvol.h).

There is no fallback: if the shared library is missing or does not export the expected
symbols, importing the operators fails.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libchop_costvol.so")

_i64, _int, _vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
_DIMS = [_i64] * 8  # B,H,W,C,D,N,srcH,srcW

#: name -> argument types, in the order of include/chop_costvol.h
SIGNATURES = {
    "chop_abi_version": [],
    "chop_init": [],
    "chop_last_error_string": [],
    "chop_set_kernel_family": [_int],
    "chop_last_kernel_family": [],
    "chop_last_views_per_workgroup": [],
    "chop_set_backward_window": [_int],
    "chop_last_backward_window": [],
    "chop_cost_volume_bwd16_workspace_bytes": [_i64] * 7,
}
for _t in ("f32", "f64"):
    SIGNATURES["chop_cost_volume_fwd_" + _t] = [_vp, _int, _int] + _DIMS + [_vp] * 8
    SIGNATURES["chop_cost_volume_bwd_" + _t] = [_vp, _int, _int] + _DIMS + [_vp] * 11
    SIGNATURES["chop_cost_aggregate_fwd_" + _t] = [_vp, _int, _int] + _DIMS + [_vp] * 8
    SIGNATURES["chop_cost_aggregate_bwd_" + _t] = [_vp, _int, _int] + _DIMS + [_vp] * 11
    SIGNATURES["chop_cost_volume_v2_fwd_" + _t] = [_vp, _int, _int] + _DIMS + [_int] + [_vp] * 7
    SIGNATURES["chop_cost_volume_v2_bwd_" + _t] = [_vp, _int, _int] + _DIMS + [_int] + [_vp] * 10
    SIGNATURES["chop_cost_aggregate_fwd_fill_" + _t] = [_vp, _int, _int] + _DIMS + [_vp] * 9
    SIGNATURES["chop_cost_volume_v2_fwd_fill_" + _t] = [_vp, _int, _int] + _DIMS + [_int] + [_vp] * 8
    SIGNATURES["chop_cost_volume_v3_fwd_" + _t] = [_vp, _int, _int] + _DIMS + [_int] + [_vp] * 8
    SIGNATURES["chop_cost_volume_v3_bwd_" + _t] = [_vp, _int, _int] + _DIMS + [_int] + [_vp] * 11
    SIGNATURES["chop_feature_aggregate_fwd_" + _t] = [_vp, _int] + _DIMS + [_vp] * 7
    SIGNATURES["chop_feature_aggregate_bwd_" + _t] = [_vp, _int] + _DIMS + [_vp] * 9
    SIGNATURES["chop_cost_default_fill_" + _t] = [_vp, _int, _i64, _i64] + [_vp] * 4
    SIGNATURES["chop_cost_default_fill_grad_" + _t] = [_vp, _int, _i64, _i64] + [_vp] * 4
    SIGNATURES["chop_combine_projection_" + _t] = [_vp, _i64, _i64] + [_vp] * 5
    SIGNATURES["chop_cost_volume_sample_coords_" + _t] = [_vp, _int] + [_i64] * 7 + [_vp] * 10
SIGNATURES["chop_cost_volume_fwd_16"] = [_vp, _int, _int, _int] + _DIMS + [_vp] * 9
SIGNATURES["chop_cost_volume_bwd_16"] = [_vp, _int, _int, _int] + _DIMS + [_vp] * 13 + [ctypes.c_size_t]
SIGNATURES["chop_cost_volume_bwd_16_static"] = [_vp, _int, _int, _int] + _DIMS + [_vp] * 12
SIGNATURES["chop_static_scratch_bytes"] = []
SIGNATURES["chop_cost_default_fill_grad_16"] = [_vp, _int, _int, _i64, _i64] + [_vp] * 4
SIGNATURES["chop_cost_volume_v2_fwd_16"] = [_vp, _int, _int, _int] + _DIMS + [_int] + [_vp] * 7
SIGNATURES["chop_cost_volume_v2_fwd_fill_16"] = [_vp, _int, _int, _int] + _DIMS + [_int] + [_vp] * 8
SIGNATURES["chop_cost_volume_v2_bwd_16"] = ([_vp, _int, _int, _int] + _DIMS + [_int] + [_vp] * 11
                                            + [ctypes.c_size_t])

_lib = None


class ChopError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("libchop_costvol status %d: %s" % (code, message))
        self.code = code


def load():
    """Load the library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s is missing: build it with `python -m custom_helper_op_amd.build` "
            "(there is no non-HIP fallback)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if a declared symbol is not exported
        fn.argtypes = argtypes
        fn.restype = _int
    lib.chop_last_error_string.restype = ctypes.c_char_p
    lib.chop_cost_volume_bwd16_workspace_bytes.restype = ctypes.c_size_t
    lib.chop_static_scratch_bytes.restype = ctypes.c_size_t
    _lib = lib
    return lib


def check(code):
    if code != 0:
        raise ChopError(code, load().chop_last_error_string().decode())
