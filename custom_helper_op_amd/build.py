"""Compiles the HIP sources under csrc/ into libchop_costvol.so (gfx950 only).

Run as ``python -m custom_helper_op_amd.build``.  hipcc cross-compiles without a GPU.
Flags that are part of the numerical contract:
  -ffp-contract=off   no implicit multiply-add fusion (coordinates must be bit-exact);
  -packed-fp32-ops disabled, so the compiler emits no packed fp32 arithmetic.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libchop_costvol.so")
SOURCES = ["tiled_f32_fwd_wide.hip", "tiled_f32_bwd_wide.hip", "tiled_f32_fwd_narrow.hip",
           "tiled_f32_bwd_narrow.hip", "tiled_f16_fwd.hip", "tiled_f16_bwd.hip",
           "tiled_bf16_fwd.hip", "tiled_bf16_bwd.hip", "api.hip", "general.hip", "v3_feature.hip",
           "epilogue.hip", "tiled.hip", "strip.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


def build(verbose=False, extra=()):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [hipcc, *[f for f in FLAGS if f != "-shared"], *extra, "-c",
               os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out = p.communicate()[0].decode()
        # the host pass warns that it does not know the packed-fp32 feature: harmless
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if out.strip():
            print(out, flush=True)
        failed |= p.returncode != 0
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
