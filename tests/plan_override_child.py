"""Child process of tests/test_gpu_plan_override.py: runs dense GEMMs of every operator under the
launch plan forced by RK_NPU_HIP_GEMM_PLAN (read once per process, hence the process of its own)
and checks them against the oracle.  Prints OK <plan> on success."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from rknpu2_matmul_open_amd import capi, ops, workloads  # noqa: E402
from oracle import binding as oracle  # noqa: E402


def bits32(x):
    return np.ascontiguousarray(x, np.float32).view(np.uint32)


def main():
    plan = os.environ["RK_NPU_HIP_GEMM_PLAN"]
    oracle.lib()
    sess = ops.Session()
    rng = np.random.default_rng(31)
    M, N, K = 200, 300, 2100          # more than 128 rows: the large-tile kernel; ragged everywhere

    # int8 weights: raw integer, fp16 and fp32 operators
    A8 = rng.integers(-128, 128, (M, K)).astype(np.int8)
    B8 = rng.integers(-128, 128, (K, N)).astype(np.int8)
    op = ops.W8A8Linear(sess, capi.I8I8I32, M, B8)
    rc, got = op.run(A8)
    assert rc == 0 and np.array_equal(got, oracle.gemm_i8(A8, B8)), "i8i8i32"
    op.close()
    c = workloads.w8a8_case(M, K, N, 3, 4)
    op = ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, M, c["B"], c["w_scale"])
    rc, got = op.run(c["A"])
    assert rc == 0 and np.array_equal(got, oracle.w8a8(c["A"], c["B"], c["w_scale"])["C"]), "f16i8f16"
    op.close()
    A32 = (rng.standard_normal((M, K)) * 3).astype(np.float32)
    op = ops.W8A8Linear(sess, capi.F32I8F32_DYNAMIC, M, c["B"], c["w_scale"])
    rc, got = op.run(A32)
    want = oracle.w8a8(A32, c["B"], c["w_scale"])["C"]
    assert rc == 0 and np.array_equal(bits32(got), bits32(want)), "f32i8f32"
    op.close()

    # int4 weights: integer sums, fp32, fp16, gate/up + SwiGLU
    N4 = 384
    B4 = rng.integers(-8, 8, (K, N4)).astype(np.int8)
    s4 = (rng.random(N4).astype(np.float32) + 0.5) * np.float32(0.01)
    w = ops.W4A8Weights(sess, B4, s4)
    wsp = ops.W4A8Workspace(sess, M, N4, K)
    want = oracle.w4a8(A32, B4, s4)
    rc, acc = wsp.run_i32(w, A32)
    assert rc == 0 and np.array_equal(acc, want["acc"]), "w4a8 i32"
    rc, got = wsp.run_f32(w, A32)
    assert rc == 0 and np.array_equal(bits32(got), bits32(want["C"])), "w4a8 f32"
    A16 = A32.astype(np.float16).view(np.uint16)
    rc, got = wsp.run_f16(w, A16)
    assert rc == 0 and np.array_equal(got, oracle.w4a8(A16, B4, s4)["C"]), "w4a8 f16"
    rc, mid = wsp.run_swiglu_f32(w, A32)
    assert rc == 0 and np.array_equal(bits32(mid), bits32(oracle.w4a8_swiglu(A32, B4, s4, oracle.EXP_POLY)["middle"])), "swiglu"
    wsp.close()
    w.close()
    sess.close()
    print("OK", plan)


if __name__ == "__main__":
    main()
