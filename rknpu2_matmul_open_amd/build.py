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
SOURCES = ["rk_kernels.hip", "rk_kernels_gemv.hip", "rk_kernels_gemm.hip", "rk_kernels_stream.hip", "rk_core.cpp", "rk_quant_matmul.cpp", "rk_autotune.cpp", "rk_w4a8.cpp", "rk_w4a8_tune.cpp", "rk_i4.cpp",
           "rk_moe_w8.cpp"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # leading scalar kernel arguments arrive in registers at wave start (14 dwords is what the
    # hardware's user registers hold beside the argument pointer)
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
    "-Wall", "-Wno-unused-function",
    "-I" + CSRC, "-I" + os.path.join(ROOT, "include"),
]


# gemm_wk_kernel and gemm_stream_kernel issue their loads from inline assembly and place every
# s_waitcnt by hand: they rely on this compiler not copying or re-using a load's destination
# register between the load and the wait that covers it.  The kernels were validated (parity
# suite on an MI355X) with the compiler named here; any other one may schedule differently, so
# a build with it is REFUSED unless the caller opts in with RK_NPU_HIP_ALLOW_UNVALIDATED_HIPCC=1,
# and then says so loudly: the parity suite (`pytest tests -m gpu` on an MI355X) has to be run
# again before the results of such a build are trusted.  The same holds after any change to
# those kernels' load / wait sequences.
VALIDATED_HIPCC = "HIP version: 7.2.26015"
ALLOW_ENV = "RK_NPU_HIP_ALLOW_UNVALIDATED_HIPCC"


class UnvalidatedToolchain(RuntimeError):
    pass


def check_toolchain(hipcc):
    """Returns the compiler's version line.  A compiler other than the validated one raises
    UnvalidatedToolchain, or -- with RK_NPU_HIP_ALLOW_UNVALIDATED_HIPCC=1 -- warns on stderr."""
    try:
        out = subprocess.run([hipcc, "--version"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                             text=True, check=False).stdout
    except OSError as e:
        raise RuntimeError("cannot run %s: %s" % (hipcc, e))
    line = next((l.strip() for l in out.splitlines() if l.startswith("HIP version:")), "")
    if not line.startswith(VALIDATED_HIPCC):
        what = ("%s reports %r, the inline-assembly load kernels (gemm_wk_kernel, gemm_stream_kernel) were "
                "validated with %r" % (hipcc, line or out[:80], VALIDATED_HIPCC))
        if os.environ.get(ALLOW_ENV) != "1":
            raise UnvalidatedToolchain(what + ".  Set %s=1 to build anyway, then run `pytest tests -m gpu` "
                                       "on an MI355X before trusting the build." % ALLOW_ENV)
        sys.stderr.write("\n[build] WARNING: %s.\n[build] Run `pytest tests -m gpu` on an MI355X before "
                         "trusting results of this build.\n\n" % what)
    return line


def build(verbose=True, audit=True):
    """Compiles and links the library.  audit: also compile the two inline-assembly load units to
    device assembly (alongside the objects) and check the hand-placed waits in it, see
    audit_waits.py; a violation fails the build (RK_NPU_HIP_SKIP_WAIT_AUDIT=1 skips the check)."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    check_toolchain(hipcc)
    audit = audit and os.environ.get("RK_NPU_HIP_SKIP_WAIT_AUDIT") != "1"
    audit_pool = audit_jobs = None
    if audit:
        from concurrent.futures import ThreadPoolExecutor
        from . import audit_waits
        audit_pool = ThreadPoolExecutor(len(audit_waits.UNITS))
        audit_jobs = [audit_pool.submit(audit_waits.device_assembly, u, hipcc, FLAGS) for u in audit_waits.UNITS]
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
    if audit:
        violations, checked = [], 0
        for job in audit_jobs:
            v, c = audit_waits.audit_text(job.result())
            violations += v
            checked += c
        audit_pool.shutdown()
        if violations or not checked:
            for line in violations[:20]:
                sys.stderr.write("[build] wait audit: %s\n" % line)
            raise RuntimeError("wait audit: %d violations in %d kernels (hand-placed waits of the inline-assembly "
                               "load kernels no longer cover their loads in the code this compiler produced)"
                               % (len(violations), checked))
        if verbose:
            sys.stderr.write("[build] wait audit: %d kernels, no violation\n" % checked)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs + ["-lpthread"]
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build())
