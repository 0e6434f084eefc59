"""Static check of the TensorFlow shim (custom_helper_op_amd/tf_shim/cost_volume_ops.cc).
No TensorFlow exists in this image (test_shim_compile.py runs the compiler's syntax check
against stand-in headers); every pointer argument of a forwarding overload has the same type,
so a transposed argument would compile anywhere.
This test parses the overloads and the prototypes of include/chop_costvol.h and checks, per
call: the callee exists, the arity agrees, every argument's type equals the prototype's
parameter type, and the pointer arguments are forwarded in the order the overload received
them.  It then checks that every OpKernel::Compute hands the tensors over in the order of the
reference's functor argument lists (cost_volume_kernels.cc:31-47 forward, :160-179 gradient;
cost_volume_kernels_v2.cc:31-48; cost_aggregate_kernels.cc, cost_volume_kernels_v3.cc and
feature_aggregate_kernels.cc use the same pattern)."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SHIM = os.path.join(ROOT, "custom_helper_op_amd", "tf_shim", "cost_volume_ops.cc")
HEADER = os.path.join(ROOT, "include", "chop_costvol.h")


def _strip_comments(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def _norm_type(t):
    t = " ".join(t.split())
    t = t.replace("int64_t", "int64").replace("int32_t", "int32")
    return t.replace(" *", "*").replace("* ", "*")


def _split_params(text):
    """'const float *a, int b' -> [('const float*', 'a'), ('int', 'b')]"""
    out = []
    for p in text.split(","):
        p = " ".join(p.split())
        if not p or p == "void":
            continue
        m = re.match(r"(.*?)([A-Za-z_][A-Za-z_0-9]*)$", p)
        out.append((_norm_type(m.group(1)), m.group(2)))
    return out


def header_prototypes():
    text = _strip_comments(open(HEADER).read())
    protos = {}
    for m in re.finditer(r"\b(?:int|size_t|const char \*)\s*(chop_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        protos[m.group(1)] = _split_params(m.group(2))
    return protos


def shim_overloads():
    text = _strip_comments(open(SHIM).read())
    pat = re.compile(r"inline int (\w+)\(([^)]*)\)\s*\{\s*return (chop_\w+)\(([^;]*)\);\s*\}", re.S)
    return [(m.group(1), _split_params(m.group(2)), m.group(3),
             [a.strip() for a in m.group(4).split(",")]) for m in pat.finditer(text)]


def test_forwarding_overloads_match_the_header():
    protos = header_prototypes()
    overloads = shim_overloads()
    assert len(overloads) == 20, len(overloads)  # 10 entry-point families x {float, double}
    seen = set()
    for name, params, callee, args in overloads:
        assert callee in protos, callee
        seen.add(callee)
        proto = protos[callee]
        assert len(args) == len(proto), (name, callee, len(args), len(proto))
        types = dict((n, t) for t, n in params)
        order = [n for _, n in params]
        last_pos = -1
        for arg, (want_type, want_name) in zip(args, proto):
            m = re.match(r"(\w+)\[(\d)\]$", arg)
            if m:  # one of the eight dimensions, passed as d[0]..d[7] in header order
                assert types[m.group(1)] == "const int64*", (name, arg)
                assert want_type == "int64", (callee, want_name, want_type)
                dims = ["B", "H", "W", "C", "D", "N", "srcH", "srcW"]
                assert want_name == dims[int(m.group(2))], (callee, arg, want_name)
                continue
            assert arg in types, (name, arg)
            assert types[arg] == want_type, (name, callee, arg, types[arg], want_type)
            # arguments are forwarded in the order they were received
            pos = order.index(arg)
            assert pos > last_pos, (name, callee, arg)
            last_pos = pos
        # float overloads call the f32 entry point, double overloads the f64 one
        elem = "double" if any("double" in t for t, _ in params) else "float"
        assert callee.endswith("_f64" if elem == "double" else "_f32"), (name, callee, elem)
    for family in ("cost_volume", "cost_aggregate", "cost_volume_v2", "cost_volume_v3",
                   "feature_aggregate"):
        for direction in ("fwd", "bwd"):
            for sfx in ("f32", "f64"):
                assert "chop_%s_%s_%s" % (family, direction, sfx) in seen


# Order in which each Compute must hand its tensors to the forwarding overload: the
# reference's functor argument lists (inputs in registration order, then outputs).
_EXPECTED = {
    "Fwd": ["ref", "src", "plane", "offsets", "rs", "ts", "cost", "mask"],
    "Bwd": ["ref", "src", "plane", "offsets", "rs", "ts", "cost_grad", "cost_mask", "g0", "g1", "g2"],
    "FwdAgg": ["ref", "src", "plane", "offsets", "rs", "ts", "cost", "mask"],
    "BwdAgg": ["ref", "src", "plane", "offsets", "rs", "ts", "cost_grad", "cost_mask", "g0", "g1", "g2"],
    "FwdV2": ["ref", "src", "grid", "rs", "ts", "cost", "mask"],
    "BwdV2": ["ref", "src", "grid", "rs", "ts", "cost_grad", "cost_mask", "g0", "g1", "g2"],
    "FwdV3": ["ref", "src", "plane", "offsets", "rs", "ts", "cost", "mask"],
    "BwdV3": ["ref", "src", "plane", "offsets", "rs", "ts", "cost_grad", "cost_mask", "g0", "g1", "g2"],
    "FwdFeat": ["src", "plane", "offsets", "rs", "ts", "mapped", "mask"],
    "BwdFeat": ["src", "plane", "offsets", "rs", "ts", "grad", "mask", "g0", "g1"],
}


def test_compute_bodies_pass_tensors_in_the_reference_order():
    text = _strip_comments(open(SHIM).read())
    calls = re.findall(r"FromChop\((\w+)\(StreamOf\(ctx\),(.*?)\)\)\)\);", text, flags=re.S)
    assert len(calls) == len(_EXPECTED), [c[0] for c in calls]
    for fn, body in calls:
        tensors = re.findall(r"(\w+)(?:\.|->)flat<", body)
        assert tensors == _EXPECTED[fn], (fn, tensors)


# registered input name -> the name its tensor is bound to in Compute
_BOUND = {"ref_image": "ref", "src_images": "src", "base_plane": "plane", "offsets": "offsets",
          "rs": "rs", "ts": "ts", "depth_grid": "grid", "cost_grad": "cost_grad",
          "cost_mask": "cost_mask", "mapped_feature_grad": "grad", "mapped_mask": "mask"}


def test_compute_inputs_are_read_in_registration_order():
    """ctx->input(i) must bind the i-th registered input of the op the kernel class serves:
    the REGISTER_OP block (copied from custom_helper_ops.cc:190-371) fixes the order."""
    text = _strip_comments(open(SHIM).read())
    registered = {}
    for m in re.finditer(r'REGISTER_OP\("(\w+)"\)(.*?);', text, flags=re.S):
        registered[m.group(1)] = re.findall(r'\.Input\("(\w+):', m.group(2))
    assert len(registered) == 10, sorted(registered)
    checked = 0
    for m in re.finditer(r"class (\w+)Op : public OpKernel(.*?)\n};", text, flags=re.S):
        op, body = m.group(1), m.group(2)
        binds = re.findall(r"&(\w+) = ctx->input\((\d+)\)", body)
        assert [int(i) for _, i in binds] == list(range(len(binds))), (op, binds)
        assert [b for b, _ in binds] == [_BOUND[n] for n in registered[op]], (op, binds, registered[op])
        checked += 1
    assert checked == 10
