"""Times the device-pointer calls of both weight formats over a grid of shapes and row counts.

    python -m rknpu2_matmul_open_amd.sweep_rows --shapes 4096x8192,14336x4096 --rows 1,2,4,8

One line per shape (K x N) and weight format: microseconds per call for each row count, fp16 rows resident
on the device, the step cycling through enough copies of the weights that every call streams them from
HBM.  The calls are `rk_npu_f16i8f16_run_dynamic_device` (int8 weights) and `rk_npu_w4a8_run_f16_device`
(int4 weights); with --int8-rows also `rk_npu_i8i8i32_run_device`.  A measuring aid for the dispatch rules
(columns per workgroup, row limits of the decode kernels, tile shapes of the GEMM kernels): the tuning
variables documented with the library (RK_NPU_HIP_GEMV_COLS, RK_NPU_HIP_GEMV_MAX_ROWS, ...) are read by
the library as usual, so two runs compare two choices.  Results are not checked here (the tests do that).
"""
import argparse
import ctypes as C

import numpy as np

from . import capi, ops


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--shapes", default="4096x4096,4096x14336,14336x4096", help="comma-separated KxN")
    ap.add_argument("--rows", default="1,2,4,8", help="comma-separated row counts")
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--int8-rows", action="store_true", help="also time the exact int8 x int8 product of int8 rows")
    args = ap.parse_args()
    shapes = [tuple(int(v) for v in s.split("x")) for s in args.shapes.split(",")]
    rows = [int(v) for v in args.rows.split(",")]
    sess = ops.Session()
    lib = sess.lib
    rng = np.random.default_rng(0)
    for K, N in shapes:
        B8 = rng.integers(-127, 128, (K, N)).astype(np.int8)
        B4 = rng.integers(-8, 8, (K, N)).astype(np.int8)
        scale = (rng.random(N).astype(np.float32) + 0.5) * np.float32(0.01)
        copies = max(2, int(400e6 // (K * N)))  # more than the memory-side cache holds
        w8 = [ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, 1, B8, scale) for _ in range(copies)]
        w4 = [ops.W4A8Weights(sess, B4, scale) for _ in range(copies)]
        wi = [ops.W8A8Linear(sess, capi.I8I8I32, 1, B8) for _ in range(copies)] if args.int8_rows else []
        lines = {"int8": [], "int4": [], "int8 rows": []}
        for M in rows:
            A = (rng.standard_normal((M, K)) * 2).astype(np.float16).view(np.uint16)
            dA, dC = sess.to_device(A), sess.empty_device(M * N * 4)
            turn = [0]
            st = ops.default_strategy(capi.F16I8F16_DYNAMIC, M, N, K)
            ws = lib.rk_npu_matmul_workspace_create(sess.domain, C.byref(st))

            def step8():
                turn[0] += 1
                assert lib.rk_npu_f16i8f16_run_dynamic_device(ws, w8[turn[0] % copies].w, dA, dC) == 0
            lines["int8"].append("M%d:%.2f" % (M, sess.time_us(step8, args.steps, args.warmup)))
            lib.rk_npu_matmul_workspace_free(ws)
            wsp = ops.W4A8Workspace(sess, M, N, K)

            def step4():
                turn[0] += 1
                assert lib.rk_npu_w4a8_run_f16_device(wsp.h, w4[turn[0] % copies].h, dA, dC) == 0
            lines["int4"].append("M%d:%.2f" % (M, sess.time_us(step4, args.steps, args.warmup)))
            wsp.close()
            if args.int8_rows:
                A8 = rng.integers(-128, 128, (M, K)).astype(np.int8)
                dA8 = sess.to_device(A8)
                sti = ops.default_strategy(capi.I8I8I32, M, N, K)
                wsi = lib.rk_npu_matmul_workspace_create(sess.domain, C.byref(sti))

                def stepi():
                    turn[0] += 1
                    assert lib.rk_npu_i8i8i32_run_device(wsi, wi[turn[0] % copies].w, dA8, dC) == 0
                lines["int8 rows"].append("M%d:%.2f" % (M, sess.time_us(stepi, args.steps, args.warmup)))
                lib.rk_npu_matmul_workspace_free(wsi)
                sess.free_device(dA8)
            sess.free_device(dA)
            sess.free_device(dC)
        for fmt in ("int8", "int4", "int8 rows"):
            if lines[fmt]:
                print("K %5d N %5d %-9s %s" % (K, N, fmt, "  ".join(lines[fmt])), flush=True)
        for h in w8 + wi:
            h.close()
        for h in w4:
            h.close()
    sess.close()


if __name__ == "__main__":
    main()
