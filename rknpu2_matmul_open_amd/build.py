"""Builds librk_npu_matmul.so (HIP kernels + C++ host layer) for gfx950.

    python -m rknpu2_matmul_open_amd.build

The library is built in-tree next to this file.  hipcc cross-compiles without
a GPU present.  Flags that matter for bit-exact results: no fast-math, fp
contraction off (every fused multiply-add in the kernels is an explicit fmaf),
correctly rounded fp32 division (the hipcc default).
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
ROOT = os.path.dirname(HERE)
LIB = os.path.join(HERE, "librk_npu_matmul.so")
SOURCES = ["rk_kernels.hip", "rk_core.cpp", "rk_quant_matmul.cpp", "rk_autotune.cpp", "rk_w4a8.cpp", "rk_w4a8_tune.cpp", "rk_i4.cpp",
           "rk_moe_w8.cpp"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    "-I" + CSRC, "-I" + os.path.join(ROOT, "include"),
]


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
        objs.append(obj)
        cmd = [hipcc] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        if src.endswith(".cpp"):
            cmd.insert(1, "-x")
            cmd.insert(2, "hip")
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            failed = True
            sys.stderr.write("[build] %s FAILED\n%s\n" % (src, out))
        elif verbose and out.strip():
            sys.stderr.write("[build] %s\n%s\n" % (src, out))
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs + ["-lpthread"]
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build())
