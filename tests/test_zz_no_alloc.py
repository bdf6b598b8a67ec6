"""GPU test of the entry point that allocates nothing,
rk_npu_f16i8f16_run_dynamic_noalloc_device, through the C ABI.

Its kernels are those of rk_npu_f16i8f16_run_dynamic_device with the workspace
buffers (quantized rows, row scales, K-split partial tiles) replaced by the
library's static device scratch array.  Bar: outputs bit-identical to that
entry point's and to the CPU oracle's.  Every case makes two calls in a row on
the shared array, the second with a smaller input whose padding would pick up
the first call's leftovers if the entry point did not clear it.
"""
import numpy as np
import pytest

from rknpu2_matmul_open_amd import capi, ops, workloads

pytestmark = pytest.mark.gpu


def _run_both(sess, oracle, M, N, K, seed):
    """Output of the no-allocation call, of the workspace call, and of the oracle for one seeded case."""
    c = workloads.w8a8_case(M, K, N, seed_w=seed, seed_a=seed + 1)
    op = ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, M, c["B"], c["w_scale"])
    dA = sess.to_device(c["A"])
    dC = sess.empty_device(M * N * 2)
    dC2 = sess.to_device(np.full((M, N), 0x7e00, np.uint16))  # NaN bits: every element must be overwritten
    try:
        assert op.run_device(dA, dC) == 0
        assert sess.sync() == 0
        with_workspace = sess.from_device(dC, (M, N), np.uint16)
        assert sess.lib.rk_npu_f16i8f16_run_dynamic_noalloc_device(op.w, M, dA, dC2) == 0
        assert sess.sync() == 0
        without = sess.from_device(dC2, (M, N), np.uint16)
    finally:
        sess.free_device(dA)
        sess.free_device(dC)
        sess.free_device(dC2)
        op.close()
    want = oracle.w8a8(c["A"], c["B"], c["w_scale"])["C"]
    return without, with_workspace, want


# (first call, second smaller call): the MFMA kernel with K split over workgroups (partial tiles in
# the scratch) then a ragged streaming-kernel shape; the large-tile kernel then the fused decode
# GEMV; a decode GEMV of the benchmark's shape then a ragged two-row one; a shape whose rows fit
# the array but whose K-split partial tiles would not (12.6 MB of them: the call runs the GEMM
# unsplit instead of refusing, same bits) then a small one
PAIRS = [((200, 1024, 4096), (17, 300, 200)),
         ((700, 6900, 1100), (1, 520, 1000)),
         ((1, 14336, 4096), (2, 700, 3000)),
         ((192, 4096, 4096), (5, 200, 300))]


@pytest.mark.parametrize("first,second", PAIRS)
def test_noalloc_matches_workspace_entry_point_twice_in_a_row(sess, oracle, first, second):
    for i, (M, N, K) in enumerate((first, second)):
        without, with_workspace, want = _run_both(sess, oracle, M, N, K, seed=31 + i)
        assert np.array_equal(without, with_workspace), "M=%d N=%d K=%d differs from the workspace call" % (M, N, K)
        assert np.array_equal(without, want), "M=%d N=%d K=%d differs from the oracle" % (M, N, K)


def test_noalloc_rejects_what_does_not_fit_and_bad_arguments(sess):
    M, N, K = 4096, 64, 4096   # 16 MiB of quantized rows: beyond the 12 MiB array
    c = workloads.w8a8_case(8, K, N, seed_w=5, seed_a=6)
    op = ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, 8, c["B"], c["w_scale"])
    dA = sess.empty_device(M * K * 2)
    dC = sess.empty_device(M * N * 2)
    lib = sess.lib
    try:
        assert lib.rk_npu_f16i8f16_run_dynamic_noalloc_device(op.w, M, dA, dC) == capi.RK_NPU_ERR_NOMEM
        assert lib.rk_npu_f16i8f16_run_dynamic_noalloc_device(op.w, 0, dA, dC) == capi.RK_NPU_ERR_PARAM
        assert lib.rk_npu_f16i8f16_run_dynamic_noalloc_device(None, 8, dA, dC) == capi.RK_NPU_ERR_PARAM
        assert lib.rk_npu_f16i8f16_run_dynamic_noalloc_device(op.w, 8, None, dC) == capi.RK_NPU_ERR_PARAM
        assert sess.sync() == 0
    finally:
        sess.free_device(dA)
        sess.free_device(dC)
        op.close()
