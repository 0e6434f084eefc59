"""The TensorFlow shim through a real C++ front end, on the CPU.

No TensorFlow exists in this image.  tests/tf_stubs/ holds stand-in declarations of the few
TensorFlow symbols the shim uses (REGISTER_OP, OpKernel, OpKernelContext, Tensor, TensorShape,
OP_REQUIRES*, the shape-inference context); `g++ -std=c++17 -fsyntax-only` against them parses
all of custom_helper_op_amd/tf_shim/cost_volume_ops.cc, instantiates every OpKernel class for
float and double, and type-checks every chop_* call against include/chop_costvol.h.  It proves
nothing about TensorFlow's behaviour."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SHIM = os.path.join(ROOT, "custom_helper_op_amd", "tf_shim", "cost_volume_ops.cc")
STUBS = os.path.join(ROOT, "tests", "tf_stubs")
INCLUDE = os.path.join(ROOT, "include")

pytestmark = pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")


def _syntax_check(path):
    return subprocess.run(
        ["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Wno-comment", "-Wno-unused-function",
         "-Werror", "-DTENSORFLOW_USE_ROCM=1", "-I", STUBS, "-I", INCLUDE, path],
        stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)


def test_shim_parses_and_type_checks():
    r = _syntax_check(SHIM)
    assert r.returncode == 0, r.stdout


def test_the_check_sees_a_wrong_call(tmp_path):
    """The same command rejects a shim whose forwarding call drops an argument or passes a
    pointer of the wrong element type: the check is not vacuous."""
    text = open(SHIM).read()
    call = "e, f, g, o, m);\n}"  # tail of the first forwarding overload (chop_cost_volume_fwd_f32)
    assert call in text
    dropped = tmp_path / "dropped.cc"
    dropped.write_text(text.replace(call, "e, f, g, o);\n}", 1))
    r = _syntax_check(str(dropped))
    assert r.returncode != 0 and "chop_cost_volume_fwd_f32" in r.stdout
    m = re.search(r"inline int Fwd\(void\* s, int r, int h, const int64\* d, const float\* a", text)
    assert m
    wrong = tmp_path / "wrong_type.cc"
    wrong.write_text(text[:m.start()] + text[m.start():].replace("const float* a", "const double* a", 1))
    assert _syntax_check(str(wrong)).returncode != 0
