"""Failure handling on the GPU box, forced from the host: every kernel still exits normally.

* Allocation failures: the library's test hook makes the n-th next device
  allocation fail.  Every constructor is driven through n = 1, 2, ... until it
  succeeds; each failed attempt must return NULL, leave no device memory behind
  (the domain's live byte count is back where it started) and not disturb a
  good run afterwards.  The reference pins the same paths by interposing its
  allocator with a fail_after counter (tests/test_w4a8_low_cpu.cpp:19-52,
  tests/test_moe_quant.cpp built with --wrap=rk_npu_mem_alloc).
* Rejected routing input on the device-pointer MoE entry point: ids outside
  [0, experts), negative / NaN coefficients and tokens whose scale underflows are
  seen by the scatter kernel and surface as RK_NPU_ERR_PARAM at the next
  rk_npu_hip_sync, where the host-pointer call (and the reference,
  src/rk_npu_moe_w8.cpp:586-601) rejects them up front.
"""
import ctypes as C

import numpy as np
import pytest

from rknpu2_matmul_open_amd import capi, ops, workloads

pytestmark = pytest.mark.gpu

MAX_ALLOCATIONS = 40  # no constructor makes this many device allocations


def _live_bytes(sess):
    st = capi.DomainMemoryStats()
    assert sess.lib.rk_npu_iommu_domain_memory_stats(sess.domain, C.byref(st)) == 0
    return st.live_bytes


def _drive(sess, create):
    """Fail the 1st, 2nd, ... allocation of create() until it succeeds; returns (handle, failures)."""
    lib = sess.lib
    base = _live_bytes(sess)
    try:
        for n in range(1, MAX_ALLOCATIONS):
            lib.rk_npu_hip_fail_alloc_after(n)
            h = create()
            lib.rk_npu_hip_fail_alloc_after(0)
            if h:
                assert n > 1, "the constructor made no device allocation"
                return h, n - 1
            assert sess.sync() == 0
            assert _live_bytes(sess) == base, "failed create #%d leaked device memory" % n
    finally:
        lib.rk_npu_hip_fail_alloc_after(0)
    raise AssertionError("constructor never succeeded")


def test_reclaim_hook_runs_once_and_the_allocation_is_retried(sess, oracle):
    """rk_npu_iommu_domain_set_reclaim (reference include/rk_npu_common.h:147-153): an allocation
    that reports out-of-memory calls the domain's hook once -- which here frees an idle weights
    handle -- and is tried again; the constructor then succeeds, and its result is exact.
    Without a hook the same failure returns NULL."""
    M, K, N = 3, 200, 96
    c = workloads.w8a8_case(M, K, N, 0, 1)
    lib = sess.lib
    B = np.ascontiguousarray(c["B"], np.int8)
    wscale = np.ascontiguousarray(c["w_scale"], np.float32)
    wc = capi.MatmulWeightConfig(K, N, min(K, 2048))

    def create():
        return lib.rk_npu_f16i8f16_weights_create(sess.domain, C.byref(wc), capi.ptr(B), capi.ptr(wscale))

    idle = create()
    assert idle
    base = _live_bytes(sess)
    calls = []

    def hook(cookie):
        calls.append(cookie)
        if idle_box[0]:
            lib.rk_npu_f16i8f16_weights_free(idle_box[0])
            idle_box[0] = None

    idle_box = [idle]
    cb = capi.ReclaimIdleFn(hook)
    try:
        lib.rk_npu_iommu_domain_set_reclaim(sess.domain, cb, C.c_void_p(1234))
        lib.rk_npu_hip_fail_alloc_after(1)
        w = create()
        lib.rk_npu_hip_fail_alloc_after(0)
        assert w, "the allocation was not retried after the hook"
        assert calls == [1234] and idle_box[0] is None
        assert _live_bytes(sess) == base   # one handle freed by the hook, one created
        # a second failure with the hook cleared: plain NULL, no call
        lib.rk_npu_iommu_domain_set_reclaim(sess.domain, None, None)
        lib.rk_npu_hip_fail_alloc_after(1)
        assert not create()
        lib.rk_npu_hip_fail_alloc_after(0)
        assert calls == [1234] and _live_bytes(sess) == base
        # the handle made on the retried allocation computes exactly
        strategy = ops.default_strategy(capi.F16I8F16_DYNAMIC, M, N, K)
        ws = lib.rk_npu_matmul_workspace_create(sess.domain, C.byref(strategy))
        assert ws
        out = np.empty((M, N), np.uint16)
        A = np.ascontiguousarray(c["A"])
        assert lib.rk_npu_f16i8f16_run_dynamic(ws, w, capi.ptr(A), capi.ptr(out)) == 0
        assert np.array_equal(out, oracle.w8a8(c["A"], c["B"], c["w_scale"])["C"])
        lib.rk_npu_matmul_workspace_free(ws)
        lib.rk_npu_f16i8f16_weights_free(w)
    finally:
        lib.rk_npu_hip_fail_alloc_after(0)
        lib.rk_npu_iommu_domain_set_reclaim(sess.domain, None, None)
        if idle_box[0]:
            lib.rk_npu_f16i8f16_weights_free(idle_box[0])


def test_w8a8_constructors_survive_every_allocation_failure(sess, oracle):
    M, K, N = 40, 300, 200
    c = workloads.w8a8_case(M, K, N, 0, 1)
    lib = sess.lib
    B = np.ascontiguousarray(c["B"], np.int8)
    wscale = np.ascontiguousarray(c["w_scale"], np.float32)
    strategy = ops.default_strategy(capi.F16I8F16_DYNAMIC, M, N, K)
    wc = capi.MatmulWeightConfig(K, N, strategy.k_tile)
    w, wfail = _drive(sess, lambda: lib.rk_npu_f16i8f16_weights_create(sess.domain, C.byref(wc), capi.ptr(B), capi.ptr(wscale)))
    ws, sfail = _drive(sess, lambda: lib.rk_npu_matmul_workspace_create(sess.domain, C.byref(strategy)))
    assert wfail >= 2 and sfail >= 4
    try:
        out = np.empty((M, N), np.uint16)
        assert lib.rk_npu_f16i8f16_run_dynamic(ws, w, capi.ptr(c["A"]), capi.ptr(out)) == 0
        assert np.array_equal(out, oracle.w8a8(c["A"], c["B"], c["w_scale"])["C"])
    finally:
        lib.rk_npu_matmul_workspace_free(ws)
        lib.rk_npu_f16i8f16_weights_free(w)


def test_w4a8_constructors_survive_every_allocation_failure(sess, oracle):
    M, K, N = 9, 200, 128
    rng = np.random.default_rng(12)
    B = rng.integers(-8, 8, (K, N)).astype(np.int8)
    wscale = (rng.random(N).astype(np.float32) + 0.5) * 0.02
    A = rng.standard_normal((M, K)).astype(np.float32)
    lib = sess.lib
    wcfg = capi.I4WeightConfig(K, N, 480)
    cfg = capi.W4A8Config()
    lib.rk_npu_w4a8_config_init(C.byref(cfg), M, N, K)
    w, wfail = _drive(sess, lambda: lib.rk_npu_w4a8_weights_create(sess.domain, C.byref(wcfg), capi.ptr(B), capi.ptr(wscale)))
    ws, sfail = _drive(sess, lambda: lib.rk_npu_w4a8_workspace_create(sess.domain, C.byref(cfg)))
    assert wfail >= 3 and sfail >= 5
    try:
        out = np.empty((M, N), np.float32)
        assert lib.rk_npu_w4a8_run_f32(ws, w, capi.ptr(A), capi.ptr(out), None) == 0
        want = oracle.w4a8(A, B, wscale)
        assert np.array_equal(out.view(np.uint32), want["C"].view(np.uint32))
    finally:
        lib.rk_npu_w4a8_workspace_free(ws)
        lib.rk_npu_w4a8_weights_free(w)


@pytest.mark.parametrize("flavour", ["w8", "quant"])
def test_moe_constructors_survive_every_allocation_failure(sess, oracle, flavour):
    T, H, E, top_k, I = 12, 128, 4, 2, 64
    c = workloads.moe_case(T, H, E, top_k, I)
    experts = c["experts"]
    if flavour == "quant":  # INT4 codes in the same arrays
        experts = [(np.clip(g, -8, 7), gs, np.clip(d, -8, 7), ds) for g, gs, d, ds in experts]
    lib = sess.lib
    cfg = capi.MoeConfig()
    lib.rk_npu_moe_w8_config_init(C.byref(cfg), H, I, E, 0, top_k, 32)
    keep = []
    arr = (capi.MoeExpert * len(experts))()
    for i, (g, gs, d, ds) in enumerate(experts):
        g, d = np.ascontiguousarray(g, np.int8), np.ascontiguousarray(d, np.int8)
        gs, ds = np.ascontiguousarray(gs, np.float32), np.ascontiguousarray(ds, np.float32)
        keep += [g, gs, d, ds]
        arr[i] = capi.MoeExpert(g.ctypes.data, gs.ctypes.data, d.ctypes.data, ds.ctypes.data)
    wcreate, wscreate = ops.MoeW8._CREATE[flavour]
    w, wfail = _drive(sess, lambda: getattr(lib, wcreate)(sess.domain, C.byref(cfg.weights), arr))
    ws, sfail = _drive(sess, lambda: getattr(lib, wscreate)(sess.domain, C.byref(cfg)))
    assert wfail >= 5 and sfail >= 15
    try:
        out = np.empty((T, H), np.float32)
        x = np.ascontiguousarray(c["x"], np.float32)
        ids, routes = np.ascontiguousarray(c["ids"], np.int32), np.ascontiguousarray(c["routes"], np.float32)
        assert lib.rk_npu_moe_w8_run_f32(ws, w, T, capi.ptr(x), capi.ptr(ids), capi.ptr(routes), capi.ptr(out), None) == 0
        rc, want = oracle.moe_w8(experts, H, I, E, 0, top_k, ids, routes, input_f32=x)
        assert rc == 0 and np.array_equal(out.view(np.uint32), want.view(np.uint32))
    finally:
        lib.rk_npu_moe_w8_workspace_free(ws)
        lib.rk_npu_moe_w8_weights_free(w)


def test_plain_device_allocation_reports_failure(sess):
    lib = sess.lib
    lib.rk_npu_hip_fail_alloc_after(1)
    try:
        assert not lib.rk_npu_hip_malloc(sess.ctx, 1024)
    finally:
        lib.rk_npu_hip_fail_alloc_after(0)
    d = lib.rk_npu_hip_malloc(sess.ctx, 1024)
    assert d
    lib.rk_npu_hip_free(sess.ctx, d)


def test_moe_device_entry_reports_rejected_routing_input(sess, oracle):
    T, H, E, top_k, I = 16, 128, 6, 2, 64
    c = workloads.moe_case(T, H, E, top_k, I)
    moe = ops.MoeW8(sess, H, I, E, 0, top_k, 32, c["experts"])
    lib = sess.lib
    x = np.ascontiguousarray(c["x"], np.float32)
    ids, routes = np.ascontiguousarray(c["ids"], np.int32), np.ascontiguousarray(c["routes"], np.float32)
    dout = sess.empty_device(T * H * 4)

    def run(x_, ids_, routes_):
        dx, dids, drt = sess.to_device(x_), sess.to_device(ids_), sess.to_device(routes_)
        try:
            assert lib.rk_npu_moe_w8_run_f32_device(moe.ws, moe.w, T, dx, dids, drt, dout) == 0
            return sess.sync()
        finally:
            for d in (dx, dids, drt):
                sess.free_device(d)

    def variants():
        bad = ids.copy(); bad[3, 1] = E
        yield "id == experts", x, bad, routes
        bad = ids.copy(); bad[T - 1, 0] = -1
        yield "negative id", x, bad, routes
        bad = ids.copy(); bad[0, 0] = E + 5
        zero = routes.copy(); zero[0, 0] = 0.0   # (rejected although its coefficient drops the route)
        yield "bad id on a dropped route", x, bad, zero
        bad = routes.copy(); bad[5, 0] = -0.25
        yield "negative coefficient", x, ids, bad
        bad = routes.copy(); bad[7, 1] = np.nan
        yield "NaN coefficient", x, ids, bad
        bad = routes.copy(); bad[2, 0] = np.inf
        yield "Inf coefficient", x, ids, bad
        tiny = x.copy(); tiny[4] = 0.0; tiny[4, 9] = 1e-39   # max / 127 underflows: 1 / scale is not finite
        yield "token whose scale underflows", tiny, ids, routes

    try:
        assert run(x, ids, routes) == 0
        good = sess.from_device(dout, (T, H), np.float32)
        rc, want = oracle.moe_w8(c["experts"], H, I, E, 0, top_k, ids, routes, input_f32=x)
        assert rc == 0 and np.array_equal(good.view(np.uint32), want.view(np.uint32))
        for what, x_, ids_, routes_ in variants():
            # the host-pointer call rejects the same input up front, and so does the oracle
            rc_host, _ = moe.run_f32(x_, ids_, routes_)
            assert rc_host == capi.RK_NPU_ERR_PARAM, what
            if ids_ is ids and routes_ is routes:
                rc_orc, _ = oracle.moe_w8(c["experts"], H, I, E, 0, top_k, ids_, routes_, input_f32=x_)
                assert rc_orc != 0, what
            assert run(x_, ids_, routes_) == capi.RK_NPU_ERR_PARAM, what
            # and the workspace is usable afterwards
            assert run(x, ids, routes) == 0, what
            assert np.array_equal(sess.from_device(dout, (T, H), np.float32).view(np.uint32), good.view(np.uint32)), what
    finally:
        sess.free_device(dout)
        moe.close()
