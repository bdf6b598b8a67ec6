"""Child process of tests/test_gpu_plan_override.py: decode-sized calls (1 to 8 rows) of every
operator with the columns per workgroup of the dot-product kernels forced by RK_NPU_HIP_GEMV_COLS
(read once per process), checked against the oracle -- short rows, and rows long enough for the
larger staging area, for several K chunks and for the chunk-wise scaling of int4 sums.  Prints
OK <columns> on success."""
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
    cols = os.environ["RK_NPU_HIP_GEMV_COLS"]
    oracle.lib()
    sess = ops.Session()
    lib = sess.lib
    rng = np.random.default_rng(int(cols))
    N, K = 520, 1000                      # 17 column blocks, ragged K
    for M in (1, 2, 4, 8):
        # int8 weights: int8 rows as given, fp16 and fp32 rows (device entries: one launch each), and the
        # host-pointer call (rows quantized by a launch of their own, then the plain GEMV)
        A8 = rng.integers(-128, 128, (M, K)).astype(np.int8)
        B8 = rng.integers(-128, 128, (K, N)).astype(np.int8)
        op = ops.W8A8Linear(sess, capi.I8I8I32, M, B8)
        dA, dC = sess.to_device(A8), sess.empty_device(M * N * 4)
        assert op.run_device(dA, dC) == 0 and sess.sync() == 0
        assert np.array_equal(sess.from_device(dC, (M, N), np.int32), oracle.gemm_i8(A8, B8)), ("i8 device", M)
        rc, got = op.run(A8)
        assert rc == 0 and np.array_equal(got, oracle.gemm_i8(A8, B8)), ("i8 host", M)
        sess.free_device(dA)
        sess.free_device(dC)
        op.close()
        c = workloads.w8a8_case(M, K, N, 3 + M, 4)
        for kind, A, dtype in ((capi.F16I8F16_DYNAMIC, c["A"], np.uint16),
                               (capi.F32I8F32_DYNAMIC, (rng.standard_normal((M, K)) * 2).astype(np.float32), np.float32)):
            op = ops.W8A8Linear(sess, kind, M, c["B"], c["w_scale"])
            want = oracle.w8a8(A, c["B"], c["w_scale"])["C"]
            dA, dC = sess.to_device(A), sess.empty_device(M * N * 4)
            assert op.run_device(dA, dC) == 0 and sess.sync() == 0
            got = sess.from_device(dC, (M, N), dtype)
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), ("w8a8 device", kind, M)
            rc, got = op.run(A)
            assert rc == 0 and np.array_equal(got.view(np.uint8), want.view(np.uint8)), ("w8a8 host", kind, M)
            sess.free_device(dA)
            sess.free_device(dC)
            op.close()
        # int4 weights: fp32 and fp16 rows through the device entries, fp32 rows through the host call
        B4 = rng.integers(-8, 8, (K, N)).astype(np.int8)
        s4 = (rng.random(N).astype(np.float32) + 0.5) * np.float32(0.01)
        w = ops.W4A8Weights(sess, B4, s4)
        wsp = ops.W4A8Workspace(sess, M, N, K)
        A32 = (rng.standard_normal((M, K)) * 3).astype(np.float32)
        A16 = A32.astype(np.float16).view(np.uint16)
        want32, want16 = oracle.w4a8(A32, B4, s4)["C"], oracle.w4a8(A16, B4, s4)["C"]
        dA32, dA16, dC = sess.to_device(A32), sess.to_device(A16), sess.empty_device(M * N * 4)
        assert lib.rk_npu_w4a8_run_f32_device(wsp.h, w.h, dA32, dC) == 0 and sess.sync() == 0
        assert np.array_equal(bits32(sess.from_device(dC, (M, N), np.float32)), bits32(want32)), ("w4a8 f32 device", M)
        assert lib.rk_npu_w4a8_run_f16_device(wsp.h, w.h, dA16, dC) == 0 and sess.sync() == 0
        assert np.array_equal(sess.from_device(dC, (M, N), np.uint16), want16), ("w4a8 f16 device", M)
        rc, got = wsp.run_f32(w, A32)
        assert rc == 0 and np.array_equal(bits32(got), bits32(want32)), ("w4a8 host", M)
        for d in (dA32, dA16, dC):
            sess.free_device(d)
        wsp.close()
        w.close()
    # Long rows: several rows that fill the larger staging area of the int8-weight kernels (one chunk,
    # quantized by the kernel), rows beyond it (several chunks behind a quantization launch), fewer rows
    # than the kernel's row count, and int4 weights over enough K chunks that the 16 x code sums are
    # taken off chunk by chunk.
    N = 72                                # 3 column blocks, the last one ragged
    for M, K in ((4, 9000), (3, 10000), (8, 5000), (5, 6000), (5, 20000), (7, 3000)):
        A8 = rng.integers(-128, 128, (M, K)).astype(np.int8)
        B8 = rng.integers(-128, 128, (K, N)).astype(np.int8)
        op = ops.W8A8Linear(sess, capi.I8I8I32, M, B8)
        dA, dC = sess.to_device(A8), sess.empty_device(M * N * 4)
        assert op.run_device(dA, dC) == 0 and sess.sync() == 0
        assert np.array_equal(sess.from_device(dC, (M, N), np.int32), oracle.gemm_i8(A8, B8)), ("long i8 device", M, K)
        sess.free_device(dA)
        sess.free_device(dC)
        op.close()
        c = workloads.w8a8_case(M, K, N, 11 + M, 12)
        for kind, A, dtype in ((capi.F16I8F16_DYNAMIC, c["A"], np.uint16),
                               (capi.F32I8F32_DYNAMIC, (rng.standard_normal((M, K)) * 2).astype(np.float32), np.float32)):
            op = ops.W8A8Linear(sess, kind, M, c["B"], c["w_scale"])
            want = oracle.w8a8(A, c["B"], c["w_scale"])["C"]
            dA, dC = sess.to_device(A), sess.empty_device(M * N * 4)
            assert op.run_device(dA, dC) == 0 and sess.sync() == 0
            got = sess.from_device(dC, (M, N), dtype)
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), ("long w8a8 device", kind, M, K)
            rc, got = op.run(A)          # (host call: rows quantized by a launch of their own)
            assert rc == 0 and np.array_equal(got.view(np.uint8), want.view(np.uint8)), ("long w8a8 host", kind, M, K)
            sess.free_device(dA)
            sess.free_device(dC)
            op.close()
    for M, K in ((4, 70000), (6, 33000)):
        B4 = np.full((K, N), -8, np.int8)
        B4[::3] = 7
        s4 = (rng.random(N).astype(np.float32) + 0.5) * np.float32(0.01)
        w = ops.W4A8Weights(sess, B4, s4)
        wsp = ops.W4A8Workspace(sess, M, N, K)
        A16 = np.where(rng.random((M, K)) < 0.5, -1000.0, 1000.0).astype(np.float16).view(np.uint16)  # every code +-127
        want16 = oracle.w4a8(A16, B4, s4)["C"]
        dA16, dC = sess.to_device(A16), sess.empty_device(M * N * 2)
        assert lib.rk_npu_w4a8_run_f16_device(wsp.h, w.h, dA16, dC) == 0 and sess.sync() == 0
        assert np.array_equal(sess.from_device(dC, (M, N), np.uint16), want16), ("long w4a8 f16 device", M, K)
        sess.free_device(dA16)
        sess.free_device(dC)
        wsp.close()
        w.close()
    sess.close()
    print("OK", cols)


if __name__ == "__main__":
    main()
