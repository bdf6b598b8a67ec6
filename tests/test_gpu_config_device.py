"""The five benchmark configurations at full size through the device-pointer entry points.

bench.py times rk_npu_f16i8f16_run_dynamic_device (configs 0 and 1), rk_npu_w4a8_run_f16_device
(config 2), rk_npu_w4a8_run_ffn_f32_device (config 3) and rk_npu_moe_w8_run_f32_device (config 4)
on operands that already lie in device memory.  Those calls share their kernels with the
host-pointer calls but not the source of the rows (no pinned mirror), the decision whether the
quantization is fused into the GEMV / GEMM launch, or the scatter input -- so each of them is
checked here, on the seeded inputs of workloads.CONFIGS, to the same bar as the host-pointer
tests: quantized codes, scales and every output element bit-exact against the CPU oracle
(the counterpart of the reference's tests/test_w4a8.cpp:71-124 and tests/test_moe_w8.cpp:19-44,
which compare the complete call with a CPU restatement on seeded inputs).
"""
import numpy as np
import pytest

from rknpu2_matmul_open_amd import capi, ops, workloads

pytestmark = pytest.mark.gpu


def _bits32(x):
    return np.ascontiguousarray(x, np.float32).view(np.uint32)


@pytest.mark.parametrize("config", [0, 1])
def test_w8a8_configs_device(sess, oracle, config):
    c = workloads.CONFIGS[config]()
    M, K, N = c["M"], c["K"], c["N"]
    op = ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, M, c["B"], c["w_scale"])
    dA, dC = sess.to_device(c["A"]), sess.empty_device(M * N * 2)
    try:
        want = oracle.w8a8(c["A"], c["B"], c["w_scale"])
        for _ in range(2):
            assert op.run_device(dA, dC) == 0
            assert sess.sync() == 0
            q, s = op.read_quantized()
            assert np.array_equal(_bits32(s), _bits32(want["a_scale"]))
            assert np.array_equal(q, want["q"])
            assert np.array_equal(sess.from_device(dC, (M, N), np.uint16), want["C"])
        # the GEMM / GEMV alone on the rows the call left in the workspace (what bench.py
        # times as the kernel without quantization)
        assert sess.lib.rk_npu_hip_upload(sess.ctx, dC, capi.ptr(np.zeros((M, N), np.uint16)), M * N * 2) == 0
        assert sess.lib.rk_npu_matmul_workspace_rerun_gemm_device(op.ws, op.w, dC) == 0
        assert sess.sync() == 0
        assert np.array_equal(sess.from_device(dC, (M, N), np.uint16), want["C"])
    finally:
        sess.free_device(dA)
        sess.free_device(dC)
        op.close()


def test_config2_device(sess, oracle):
    """M=2048, K=4096, N=4096 int4 weights: all 8.4 M codes and all 2048 x 4096 fp16 outputs."""
    c = workloads.CONFIGS[2]()
    M, K, N = c["M"], c["K"], c["N"]
    w = ops.W4A8Weights(sess, c["B"], c["w_scale"])
    wsp = ops.W4A8Workspace(sess, M, N, K)
    dA, dC = sess.to_device(c["A"]), sess.empty_device(M * N * 2)
    try:
        want = oracle.w4a8(c["A"], c["B"], c["w_scale"])
        assert want["rc"] == 0
        for _ in range(2):
            assert sess.lib.rk_npu_w4a8_run_f16_device(wsp.h, w.h, dA, dC) == 0
            assert sess.sync() == 0
            q, s = wsp.read_quantized()
            assert np.array_equal(_bits32(s), _bits32(want["a_scale"]))
            assert np.array_equal(q, want["q"])
            assert np.array_equal(sess.from_device(dC, (M, N), np.uint16), want["C"])
        # the GEMM alone, as bench.py times it
        assert sess.lib.rk_npu_hip_upload(sess.ctx, dC, capi.ptr(np.zeros((M, N), np.uint16)), M * N * 2) == 0
        assert sess.lib.rk_npu_w4a8_workspace_rerun_gemm_device(wsp.h, w.h, dC, 1) == 0
        assert sess.sync() == 0
        assert np.array_equal(sess.from_device(dC, (M, N), np.uint16), want["C"])
    finally:
        sess.free_device(dA)
        sess.free_device(dC)
        wsp.close()
        w.close()


def test_config3_device(sess, oracle):
    """M=128, hidden 4096, intermediate 14336: middle, Down codes and scales, output."""
    c = workloads.CONFIGS[3]()
    M, H, I = c["M"], c["H"], c["I"]
    gw, dw = ops.W4A8Weights(sess, c["B_gu"], c["s_gu"]), ops.W4A8Weights(sess, c["B_down"], c["s_down"])
    gws, dws = ops.W4A8Workspace(sess, M, 2 * I, H), ops.W4A8Workspace(sess, M, H, I)
    dA = sess.to_device(c["x"])
    dmid, dC = sess.empty_device(M * I * 4), sess.empty_device(M * H * 4)
    try:
        want = oracle.w4a8_ffn(c["x"], c["B_gu"], c["s_gu"], c["B_down"], c["s_down"], oracle.EXP_POLY)
        assert want["rc"] == 0
        for _ in range(2):
            assert sess.lib.rk_npu_w4a8_run_ffn_f32_device(gws.h, gw.h, dws.h, dw.h, dA, dmid, dC) == 0
            assert sess.sync() == 0
            assert np.array_equal(_bits32(sess.from_device(dmid, (M, I), np.float32)), _bits32(want["middle"]))
            qd, sd = dws.read_quantized()
            assert np.array_equal(_bits32(sd), _bits32(want["down_scale"]))
            assert np.array_equal(qd, want["q_down"])
            assert np.array_equal(_bits32(sess.from_device(dC, (M, H), np.float32)), _bits32(want["C"]))
    finally:
        for d in (dA, dmid, dC):
            sess.free_device(d)
        for o in (gws, dws, gw, dw):
            o.close()


def test_config4_device(sess, oracle):
    """256 tokens, hidden 2048, 32 experts, top-4, intermediate 1024: the fp32 result."""
    c = workloads.CONFIGS[4]()
    T, H = c["T"], c["H"]
    moe = ops.MoeW8(sess, H, c["I"], c["E"], 0, c["top_k"], 256, c["experts"])
    dx, dids, drt = sess.to_device(c["x"]), sess.to_device(c["ids"]), sess.to_device(c["routes"])
    dout = sess.empty_device(T * H * 4)
    try:
        rc, want = oracle.moe_w8(c["experts"], H, c["I"], c["E"], 0, c["top_k"], c["ids"], c["routes"],
                                 input_f32=c["x"])
        assert rc == 0
        for _ in range(2):
            assert sess.lib.rk_npu_moe_w8_run_f32_device(moe.ws, moe.w, T, dx, dids, drt, dout) == 0
            assert sess.sync() == 0
            got = sess.from_device(dout, (T, H), np.float32)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    finally:
        for d in (dx, dids, drt, dout):
            sess.free_device(d)
        moe.close()
