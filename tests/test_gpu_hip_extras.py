"""The HIP-side additions of include/rk_npu_hip.h that have no counterpart in the reference:
stream capture and replay of *_device calls, the per-kernel profile, the measurement probes.

A captured sequence is checked the way a graph has to be on this hardware: several replays,
with the program's own eager work and synchronizations between them, and EVERY replay compared
with the oracle on inputs that changed since the previous one (a replay that re-used stale
results, or a node that only works the first time, fails this).
"""
import ctypes as C

import numpy as np
import pytest

from rknpu2_matmul_open_amd import capi, ops, workloads

pytestmark = pytest.mark.gpu


def _upload(sess, dst, array):
    a = np.ascontiguousarray(array)
    assert sess.lib.rk_npu_hip_upload(sess.ctx, dst, capi.ptr(a), a.nbytes) == 0


def test_captured_decode_sequence_replays_like_eager_calls(sess, oracle):
    lib = sess.lib
    # a decode step of each kind: fused quantize + GEMV (int8 weights), the same with int4
    # weights, and a routed MoE layer for a handful of tokens
    M, K, N = 1, 1024, 2048 + 96
    c = workloads.w8a8_case(M, K, N, 5, 6)
    lin = ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, M, c["B"], c["w_scale"])
    rng = np.random.default_rng(77)
    B4 = rng.integers(-8, 8, (K, N)).astype(np.int8)
    s4 = (rng.random(N).astype(np.float32) + 0.5) * 0.02
    w4 = ops.W4A8Weights(sess, B4, s4)
    ws4 = ops.W4A8Workspace(sess, M, N, K)
    T, H, E, top_k, I = 8, 128, 6, 2, 64
    mc = workloads.moe_case(T, H, E, top_k, I)
    moe = ops.MoeW8(sess, H, I, E, 0, top_k, 32, mc["experts"])

    dA16 = sess.empty_device(M * K * 2)
    dC16 = sess.empty_device(M * N * 2)
    dA32 = sess.empty_device(M * K * 4)
    dC32 = sess.empty_device(M * N * 4)
    dx = sess.empty_device(T * H * 4)
    dids, drt = sess.to_device(np.ascontiguousarray(mc["ids"], np.int32)), sess.to_device(
        np.ascontiguousarray(mc["routes"], np.float32))
    dout = sess.empty_device(T * H * 4)

    def enqueue():
        assert lin.run_device(dA16, dC16) == 0
        assert lib.rk_npu_w4a8_run_f32_device(ws4.h, w4.h, dA32, dC32) == 0
        assert lib.rk_npu_moe_w8_run_f32_device(moe.ws, moe.w, T, dx, dids, drt, dout) == 0

    def set_inputs(seed):
        r = np.random.default_rng(seed)
        a16 = r.standard_normal((M, K)).astype(np.float16)
        a32 = r.standard_normal((M, K)).astype(np.float32)
        x = r.standard_normal((T, H)).astype(np.float32)
        _upload(sess, dA16, a16.view(np.uint16))
        _upload(sess, dA32, a32)
        _upload(sess, dx, x)
        return a16, a32, x

    def check(a16, a32, x, what):
        got16 = sess.from_device(dC16, (M, N), np.uint16)
        assert np.array_equal(got16, oracle.w8a8(a16.view(np.uint16), c["B"], c["w_scale"])["C"]), what
        got32 = sess.from_device(dC32, (M, N), np.float32)
        want32 = oracle.w4a8(a32, B4, s4)["C"]
        assert np.array_equal(got32.view(np.uint32), want32.view(np.uint32)), what
        gotm = sess.from_device(dout, (T, H), np.float32)
        rc, wantm = oracle.moe_w8(mc["experts"], H, I, E, 0, top_k, mc["ids"], mc["routes"], input_f32=x)
        assert rc == 0 and np.array_equal(gotm.view(np.uint32), wantm.view(np.uint32)), what

    graph = None
    try:
        inputs = set_inputs(1)
        enqueue()                      # once eagerly before capturing
        assert sess.sync() == 0
        check(*inputs, "eager")
        assert lib.rk_npu_hip_capture_begin(sess.ctx) == 0
        enqueue()
        graph = lib.rk_npu_hip_capture_end(sess.ctx)
        assert graph
        for replay in range(4):
            inputs = set_inputs(100 + replay)      # eager work between the replays: uploads ...
            scratch = sess.to_device(np.zeros(4096, np.uint8))  # ... an allocation, a copy
            sess.free_device(scratch)
            assert lib.rk_npu_hip_graph_launch(sess.ctx, graph) == 0
            assert sess.sync() == 0
            check(*inputs, "replay %d" % replay)
            if replay == 1:                         # eager calls of the same operators in between
                inputs = set_inputs(500)
                enqueue()
                assert sess.sync() == 0
                check(*inputs, "eager between replays")
    finally:
        if graph:
            lib.rk_npu_hip_graph_free(graph)
        for d in (dA16, dC16, dA32, dC32, dx, dids, drt, dout):
            sess.free_device(d)
        moe.close()
        ws4.close()
        w4.close()
        lin.close()


def test_capture_misuse_is_reported(sess):
    lib = sess.lib
    assert lib.rk_npu_hip_capture_begin(None) == capi.RK_NPU_ERR_PARAM
    assert not lib.rk_npu_hip_capture_end(None)
    assert lib.rk_npu_hip_graph_launch(sess.ctx, None) == capi.RK_NPU_ERR_PARAM
    lib.rk_npu_hip_graph_free(None)
    # nothing recorded: the capture ends cleanly either way (an empty graph replays, or none is
    # returned), and the context works afterwards
    assert lib.rk_npu_hip_capture_begin(sess.ctx) == 0
    g = lib.rk_npu_hip_capture_end(sess.ctx)
    if g:
        assert lib.rk_npu_hip_graph_launch(sess.ctx, g) == 0
        lib.rk_npu_hip_graph_free(g)
    assert sess.sync() == 0
    d = sess.to_device(np.arange(16, dtype=np.uint32))
    assert np.array_equal(sess.from_device(d, (16,), np.uint32), np.arange(16, dtype=np.uint32))
    sess.free_device(d)


def test_profile_names_the_kernels_of_a_step_in_launch_order(sess):
    M, K, N = 64, 512, 512
    c = workloads.w8a8_case(M, K, N, 0, 1)
    lin = ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, M, c["B"], c["w_scale"])
    dA = sess.to_device(c["A"])
    dC = sess.empty_device(M * N * 2)
    try:
        prof = ops.profile_kernels(sess, lambda: lin.run_device(dA, dC), iters=5)
        names = [k for k, _ in prof]
        assert len(names) == 2 and names[0].startswith("quant_rows") and names[1].startswith("gemm_"), names
        assert all(0.5 < us < 5000.0 for _, us in prof), prof
        # one kernel when the quantization is folded into the decode GEMV
        lin1 = ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, 1, c["B"], c["w_scale"])
        dA1 = sess.to_device(np.ascontiguousarray(c["A"][:1]))
        try:
            prof1 = ops.profile_kernels(sess, lambda: lin1.run_device(dA1, dC), iters=5)
            assert len(prof1) == 1 and prof1[0][0].startswith("gemv_kernel"), prof1
        finally:
            sess.free_device(dA1)
            lin1.close()
        # a second profile on a busy context is refused, and so is an end without a begin
        lib = sess.lib
        assert lib.rk_npu_hip_profile_begin(sess.ctx) == 0
        assert lib.rk_npu_hip_profile_begin(sess.ctx) == capi.RK_NPU_ERR_BUSY
        us = (C.c_double * 4)()
        buf = C.create_string_buffer(64)
        assert lib.rk_npu_hip_profile_end(sess.ctx, buf, len(buf), us, 4) == 0   # nothing was launched
        assert lib.rk_npu_hip_profile_end(sess.ctx, buf, len(buf), us, 4) < 0
    finally:
        sess.free_device(dA)
        sess.free_device(dC)
        lin.close()


def test_measurement_probes_run_and_validate_their_arguments(sess):
    lib = sess.lib
    nbytes = 4 << 20
    src = sess.to_device(np.arange(nbytes // 4, dtype=np.uint32))
    try:
        assert lib.rk_npu_hip_probe_stream_read(sess.ctx, src, nbytes, 131072) == 0
        assert lib.rk_npu_hip_probe_stream_read(sess.ctx, src, nbytes - 4096, 65536) == 0   # ragged last span
        assert sess.sync() == 0
        for bad in ((None, src, nbytes, 131072), (sess.ctx, None, nbytes, 131072), (sess.ctx, src, 0, 131072),
                    (sess.ctx, src, nbytes, 1000), (sess.ctx, src, nbytes, 0)):
            assert lib.rk_npu_hip_probe_stream_read(*bad) == capi.RK_NPU_ERR_PARAM, bad[2:]
        ops_count = C.c_double(0.0)
        assert lib.rk_npu_hip_probe_mfma_i8(sess.ctx, src, 50, C.byref(ops_count)) == 0
        assert sess.sync() == 0
        _, cus, _ = sess.device_info()
        # eight waves per compute unit, four accumulators per wave and iteration
        assert ops_count.value == float(cus) * 8 * 50 * 4 * (2 * 32 * 32 * 32)
        assert lib.rk_npu_hip_probe_mfma_i8(sess.ctx, None, 50, C.byref(ops_count)) == capi.RK_NPU_ERR_PARAM
        assert lib.rk_npu_hip_probe_mfma_i8(sess.ctx, src, 0, C.byref(ops_count)) == capi.RK_NPU_ERR_PARAM
    finally:
        sess.free_device(src)


def test_replay_reports_rejected_input_after_an_earlier_sync(sess, oracle):
    """A decode loop is graph_launch + sync, again and again.  The sync takes the workspaces'
    rejected-input flags off the context's list, so every launch of the graph has to put them
    back: input that turns bad between two replays (a NaN token, an expert id out of range, a
    negative coefficient) must surface as RK_NPU_ERR_PARAM at the sync behind THAT replay, and
    the replay after it, on good input again, must be clean and exact."""
    lib = sess.lib
    T, H, E, top_k, I = 4, 128, 6, 2, 64
    mc = workloads.moe_case(T, H, E, top_k, I)
    moe = ops.MoeW8(sess, H, I, E, 0, top_k, 32, mc["experts"])
    M, K, N = 1, 320, 200
    rng = np.random.default_rng(5)
    B4 = rng.integers(-8, 8, (K, N)).astype(np.int8)
    s4 = (rng.random(N).astype(np.float32) + 0.5) * 0.02
    w4, ws4 = ops.W4A8Weights(sess, B4, s4), ops.W4A8Workspace(sess, M, N, K)
    x = np.ascontiguousarray(mc["x"], np.float32)
    ids, routes = np.ascontiguousarray(mc["ids"], np.int32), np.ascontiguousarray(mc["routes"], np.float32)
    a = rng.standard_normal((M, K)).astype(np.float32)
    dx, dids, drt, dout = sess.to_device(x), sess.to_device(ids), sess.to_device(routes), sess.empty_device(T * H * 4)
    dA, dC = sess.to_device(a), sess.empty_device(M * N * 4)

    def enqueue():
        assert lib.rk_npu_moe_w8_run_f32_device(moe.ws, moe.w, T, dx, dids, drt, dout) == 0
        assert lib.rk_npu_w4a8_run_f32_device(ws4.h, w4.h, dA, dC) == 0

    def good():
        _upload(sess, dx, x)
        _upload(sess, dids, ids)
        _upload(sess, drt, routes)
        _upload(sess, dA, a)

    graph = None
    try:
        enqueue()
        assert sess.sync() == 0
        assert lib.rk_npu_hip_capture_begin(sess.ctx) == 0
        enqueue()
        graph = lib.rk_npu_hip_capture_end(sess.ctx)
        assert graph
        rc, want = oracle.moe_w8(mc["experts"], H, I, E, 0, top_k, ids, routes, input_f32=x)
        want4 = oracle.w4a8(a, B4, s4)["C"]
        assert lib.rk_npu_hip_graph_launch(sess.ctx, graph) == 0
        assert sess.sync() == 0            # <- from here on no flag is registered by an eager call
        bad_x = x.copy(); bad_x[2, 7] = np.nan
        bad_ids = ids.copy(); bad_ids[1, 0] = E + 3
        bad_routes = routes.copy(); bad_routes[3, 1] = -0.25
        bad_a = a.copy(); bad_a[0, 11] = np.inf
        for what, dst, bad in (("NaN token", dx, bad_x), ("expert id", dids, bad_ids),
                               ("negative coefficient", drt, bad_routes), ("Inf row (w4a8)", dA, bad_a)):
            _upload(sess, dst, bad)
            assert lib.rk_npu_hip_graph_launch(sess.ctx, graph) == 0
            assert sess.sync() == capi.RK_NPU_ERR_PARAM, what
            good()
            assert lib.rk_npu_hip_graph_launch(sess.ctx, graph) == 0
            assert sess.sync() == 0, "clean replay after " + what
            assert np.array_equal(sess.from_device(dout, (T, H), np.float32).view(np.uint32), want.view(np.uint32))
            assert np.array_equal(sess.from_device(dC, (M, N), np.float32).view(np.uint32), want4.view(np.uint32))
        # a workspace freed while the graph lives takes its flag with it: a later sync must not
        # read freed memory (the graph itself is not launched again)
        ws4.close()
        assert sess.sync() == 0
    finally:
        if graph:
            lib.rk_npu_hip_graph_free(graph)
        for d in (dx, dids, drt, dout, dA, dC):
            sess.free_device(d)
        moe.close()
        ws4.close()
        w4.close()


def test_closing_a_context_that_is_profiling_releases_the_marker(sess):
    """rk_npu_close between profile_begin and profile_end: the process-wide marker and the
    profile ownership go with the context, so launches on other contexts do not touch freed
    memory and another context can profile afterwards."""
    lib = sess.lib
    other = ops.Session()
    M, K, N = 2, 256, 128
    c = workloads.w8a8_case(M, K, N, 0, 1)
    lin_other = ops.W8A8Linear(other, capi.F16I8F16_DYNAMIC, M, c["B"], c["w_scale"])
    dA = other.to_device(c["A"])
    dC = other.empty_device(M * N * 2)
    assert lib.rk_npu_hip_profile_begin(other.ctx) == 0
    assert lin_other.run_device(dA, dC) == 0        # records an event owned by `other`
    other.free_device(dA)
    other.free_device(dC)
    lin_other.close()
    other.close()                                    # still profiling
    lin = ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, M, c["B"], c["w_scale"])
    dA, dC = sess.to_device(c["A"]), sess.empty_device(M * N * 2)
    try:
        assert lin.run_device(dA, dC) == 0           # would call the stale marker
        assert sess.sync() == 0
        prof = ops.profile_kernels(sess, lambda: lin.run_device(dA, dC), iters=3)   # not BUSY
        assert len(prof) == 1
    finally:
        sess.free_device(dA)
        sess.free_device(dC)
        lin.close()
