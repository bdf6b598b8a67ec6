"""GPU parity of the routed W8A8 MoE layer against the CPU oracle.

The oracle evaluates the same formula as the reference's own test oracle
(tests/test_moe_w8.cpp:24-44) with the polynomial exponential and fused
combine; outputs are compared bit-exactly.  The libm flavour is checked to the
reference's relL2 < 1e-6 bar.  Cases follow tests/test_moe_w8.cpp:60-146:
shared expert, duplicate ids, zero coefficients, empty experts, weight
re-binding A/B/A, fp32 == pre-quantized entry on tie anchors, zero input,
NaN / alias / bad id / bad scale rejection, all routes dropped, foreign domain.
"""
import ctypes as C

import numpy as np
import pytest

from rknpu2_matmul_open_amd import capi, ops, workloads

pytestmark = pytest.mark.gpu


def _ref_experts(H, N, E, variant):
    """The deterministic expert tensors of reference tests/test_moe_w8.cpp:64-72."""
    out = []
    for e in range(E + 1):
        i = np.arange(H * 2 * N, dtype=np.int64)
        g = (((i * 17 + i // 19 + e * 11 + variant * 3) % 7) - 3).astype(np.int8).reshape(H, 2 * N)
        j = np.arange(N * H, dtype=np.int64)
        d = (((j * 13 + j // 7 + e * 5 + variant * 2) % 7) - 3).astype(np.int8).reshape(N, H)
        out.append((g, np.full(2 * N, 0.0625, np.float32), d, np.full(H, 0.015625, np.float32)))
    return out


def _rel_l2(got, want):
    d = np.sqrt(((got.astype(np.float64) - want) ** 2).sum())
    n = np.sqrt((want.astype(np.float64) ** 2).sum())
    return d / n if n else (np.inf if d else 0.0)


def test_reference_moe_scenario(sess, oracle):
    H, N, E, TOP, MAX = 64, 32, 3, 2, 256
    a, b = _ref_experts(H, N, E, 0), _ref_experts(H, N, E, 1)
    moe = ops.MoeW8(sess, H, N, E, 1, TOP, MAX, a)
    wb = moe.create_weights(b)
    lib = sess.lib
    try:
        for rows in (1, 5, 128, 256, 1):
            i = np.arange(rows * H, dtype=np.int64)
            x = (((i * 7 + i // 5) % 255) - 127).astype(np.int8).reshape(rows, H)
            scales = np.full(rows, 0.03125, np.float32)
            r = np.arange(rows)[:, None]
            s = np.arange(TOP)[None, :]
            ids = ((r + s) % E).astype(np.int32)
            routes = np.where(s == 0, 0.625, 0.375).astype(np.float32) * np.ones((rows, 1), np.float32)
            ids[0, 0] = ids[0, 1] = 0
            routes[0, 1] = 0  # duplicate index with a dropped route
            for variant in (0, 1, 0):
                w, ex = (wb, b) if variant else (moe.w, a)
                rc, want = oracle.moe_w8(ex, H, N, E, 1, TOP, ids, routes, input_q=x, row_scales=scales)
                assert rc == 0
                t = capi.MoeTimings()
                rc, got = moe.run_quantized(x, scales, ids, routes, weights=w, timings=t)
                assert rc == 0
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (rows, variant)
                rc, libm = oracle.moe_w8(ex, H, N, E, 1, TOP, ids, routes, input_q=x, row_scales=scales,
                                         flavour=oracle.EXP_LIBM)
                assert _rel_l2(got, libm) < 1e-6
                rc, again = moe.run_quantized(x, scales, ids, routes, weights=w)
                assert rc == 0 and np.array_equal(again, got)
            saved = got.copy()
            out = got.copy()
            bad_ids = ids.copy()
            bad_ids[0, 0] = E
            rc, _ = moe.run_quantized(x, scales, bad_ids, routes, out=out)
            assert rc == capi.RK_NPU_ERR_PARAM and np.array_equal(out, saved)
            bad_scales = scales.copy()
            bad_scales[0] = 0
            rc, _ = moe.run_quantized(x, bad_scales, ids, routes, out=out)
            assert rc == capi.RK_NPU_ERR_PARAM
            neg = routes.copy()
            neg[0, 0] = -0.5
            rc, _ = moe.run_quantized(x, scales, ids, neg, out=out)
            assert rc == capi.RK_NPU_ERR_PARAM
            # fp32 entry == pre-quantized entry on tie anchors (nearest-even)
            anchors = np.array([127, -127, .5, 1.5, 2.5, -.5, -1.5, -2.5], np.float32)
            f = np.empty((rows, H), np.float32)
            rr, cc = np.meshgrid(np.arange(rows), np.arange(H), indexing="ij")
            f[:] = ((rr * 13 + cc * 7) % 63 - 31) / 8.0
            f[:, :8] = anchors
            fq = np.empty((rows, H), np.int8)
            fs = np.empty(rows, np.float32)
            for row in range(rows):
                fs[row], fq[row] = oracle.moe_quant_row(f[row])
            assert list(fq[0, :8]) == [127, -127, 0, 2, 2, 0, -2, -2]
            rc, even = moe.run_quantized(fq, fs, ids, routes)
            rc2, from_f32 = moe.run_f32(f, ids, routes)
            assert rc == 0 and rc2 == 0 and np.array_equal(even, from_f32)
            rc, want = oracle.moe_w8(a, H, N, E, 1, TOP, ids, routes, input_f32=f)
            assert np.array_equal(from_f32.view(np.uint32), want.view(np.uint32))
            f[:] = 0
            rc, zero = moe.run_f32(f, ids, routes)
            assert rc == 0 and (zero == 0).all()
            f[0, 0] = np.nan
            rc, _ = moe.run_f32(f, ids, routes)
            assert rc == capi.RK_NPU_ERR_PARAM
            f[0, 0] = 0
            rc = lib.rk_npu_moe_w8_run_f32(moe.ws, moe.w, rows, capi.ptr(f), capi.ptr(ids),
                                           capi.ptr(routes), capi.ptr(f), None)
            assert rc == capi.RK_NPU_ERR_PARAM  # output aliases input
            rc = lib.rk_npu_moe_w8_run_f32(moe.ws, moe.w, MAX + 1, capi.ptr(f), capi.ptr(ids),
                                           capi.ptr(routes), capi.ptr(out), None)
            assert rc == capi.RK_NPU_ERR_PARAM
    finally:
        lib.rk_npu_moe_w8_weights_free(wb)
        moe.close()


def test_single_expert_no_shared_and_empty_routes(sess, oracle):
    H, N = 64, 32
    a = _ref_experts(H, N, 0, 0)[:1]
    moe = ops.MoeW8(sess, H, N, 1, 0, 1, 256, a)
    lib = sess.lib
    try:
        other = lib.rk_npu_iommu_domain_create(sess.ctx, 14)
        foreign = moe.create_weights(a, domain=other)
        for rows in (1, 128, 256):
            x = np.ones((rows, H), np.int8)
            scales = np.full(rows, 0.03125, np.float32)
            routes = np.ones((rows, 1), np.float32)
            ids = np.zeros((rows, 1), np.int32)
            rc, _ = moe.run_quantized(x, scales, ids, routes, weights=foreign)
            assert rc == capi.RK_NPU_ERR_DOMAIN
            rc, got = moe.run_quantized(x, scales, ids, routes)
            rc2, want = oracle.moe_w8(a, H, N, 1, 0, 1, ids, routes, input_q=x, row_scales=scales)
            assert rc == 0 and rc2 == 0 and np.array_equal(got.view(np.uint32), want.view(np.uint32))
            routes[:] = 0
            t = capi.MoeTimings()
            rc, got = moe.run_quantized(x, scales, ids, routes, timings=t, out=got)
            assert rc == 0 and (got == 0).all()
            assert t.gemm_tasks == 0 and t.gather_tasks == 0 and t.middle_tasks == 0 and t.sync_us == 0
            scales[0] = 0
            rc, _ = moe.run_quantized(x, scales, ids, routes)
            assert rc == capi.RK_NPU_ERR_PARAM
        lib.rk_npu_moe_w8_weights_free(foreign)
        lib.rk_npu_iommu_domain_free(other)
    finally:
        moe.close()


@pytest.mark.parametrize("T,H,E,top_k,I,shared", [(7, 64, 4, 2, 32, 0), (33, 128, 8, 3, 96, 1),
                                                   (100, 96, 40, 8, 64, 0), (256, 256, 16, 4, 160, 1),
                                                   (19, 160, 5, 1, 544, 0)])
def test_random_moe_bit_exact(sess, oracle, T, H, E, top_k, I, shared):
    c = workloads.moe_case(T, H, E, top_k, I, seeds=(T, H, E, top_k, I))
    experts = c["experts"]
    if shared:
        experts = experts + [experts[0]]
    moe = ops.MoeW8(sess, H, I, E, shared, top_k, 256, experts)
    try:
        rc, got = moe.run_f32(c["x"], c["ids"], c["routes"])
        rc2, want = oracle.moe_w8(experts, H, I, E, shared, top_k, c["ids"], c["routes"], input_f32=c["x"])
        assert rc == 0 and rc2 == 0
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        assert sess.lib.rk_npu_moe_w8_weights_device_bytes(moe.w) >= (E + shared) * 3 * H * I
        assert sess.lib.rk_npu_moe_w8_workspace_device_bytes(moe.ws) > 0
    finally:
        moe.close()


def test_config4_full(sess, oracle):
    """BASELINE config 4: 256 tokens, hidden 2048, 32 experts, top-4, intermediate 1024."""
    c = workloads.CONFIGS[4]()
    moe = ops.MoeW8(sess, c["H"], c["I"], c["E"], 0, c["top_k"], 256, c["experts"])
    try:
        t = capi.MoeTimings()
        rc, got = moe.run_f32(c["x"], c["ids"], c["routes"], timings=t)
        rc2, want = oracle.moe_w8(c["experts"], c["H"], c["I"], c["E"], 0, c["top_k"], c["ids"],
                                  c["routes"], input_f32=c["x"])
        assert rc == 0 and rc2 == 0
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        assert t.total_us > 0 and t.gate_us > 0 and t.down_us > 0
        rc3, libm = oracle.moe_w8(c["experts"], c["H"], c["I"], c["E"], 0, c["top_k"], c["ids"],
                                  c["routes"], input_f32=c["x"], flavour=oracle.EXP_LIBM)
        assert _rel_l2(got, libm) < 1e-6
        g16 = oracle.half_to_float(oracle.float_to_half(got))
        l16 = oracle.half_to_float(oracle.float_to_half(libm))
        assert np.abs(g16 - l16).max() <= 1e-3 * np.abs(l16).max()
    finally:
        moe.close()


def test_config_validation(sess):
    lib = sess.lib
    cfg = capi.MoeConfig()
    lib.rk_npu_moe_w8_config_init(C.byref(cfg), 64, 32, 3, 1, 2, 256)
    assert (cfg.struct_size, cfg.npu_cores, cfg.cpu_threads, cfg.native_input, cfg.middle,
            cfg.timeout_ms) == (C.sizeof(capi.MoeConfig), 3, 4, 0, 0, 1000)
    def make(**kw):
        c = capi.MoeConfig()
        lib.rk_npu_moe_w8_config_init(C.byref(c), 64, 32, 3, 1, 2, 256)
        for k, v in kw.items():
            if k in ("hidden", "intermediate", "routed_experts", "shared_expert"):
                setattr(c.weights, k, v)
            else:
                setattr(c, k, v)
        h = lib.rk_npu_moe_w8_workspace_create(sess.domain, C.byref(c))
        if h:
            lib.rk_npu_moe_w8_workspace_free(h)
        return bool(h)
    assert make()
    for bad in (dict(struct_size=4), dict(hidden=32), dict(hidden=80), dict(intermediate=16),
                dict(intermediate=48), dict(routed_experts=0), dict(shared_expert=2),
                dict(max_rows=0), dict(max_rows=257), dict(top_k=0), dict(top_k=4), dict(npu_cores=0),
                dict(npu_cores=4), dict(cpu_threads=5), dict(native_input=2), dict(timeout_ms=0),
                dict(timeout_ms=60001), dict(middle=1)):
        assert not make(**bad), bad
