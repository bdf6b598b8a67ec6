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
                                                   (19, 160, 5, 1, 544, 0),
                                                   # the envelope: every assignment slot in use (256 x 8 =
                                                   # 2048) over a thousand experts + the shared one (most
                                                   # buckets hold one or two rows); the widest middle
                                                   (256, 64, 1000, 8, 32, 1), (5, 64, 2, 1, 8192, 0)])
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


def test_moe_extreme_codes_and_magnitudes(sess, oracle):
    """All-extreme operands: every expert code +-127, tokens at +-3e38 / denormal / all-equal
    magnitudes, so that the int32 sums (127 * 127 * K), the scales at both ends of the fp32 range
    and the saturating SiLU branch (|gate| far beyond 80) are exercised together."""
    T, H, E, top_k, I = 12, 256, 3, 2, 96
    rng = np.random.default_rng(99)
    experts = []
    for e in range(E):
        g = np.where(rng.random((H, 2 * I)) < 0.5, -127, 127).astype(np.int8)
        d = np.where(rng.random((I, H)) < 0.5, -127, 127).astype(np.int8)
        if e == 0:
            g[:] = 127
            d[:] = -127
        gs = (rng.random(2 * I).astype(np.float32) + 0.5) * np.float32([1e-3, 1.0, 30.0][e])
        ds = (rng.random(H).astype(np.float32) + 0.5) * np.float32([1e-3, 1.0, 1e-6][e])
        experts.append((g, gs, d, ds))
    x = rng.standard_normal((T, H)).astype(np.float32)
    x[0] = 3.0e38
    x[1] = -3.0e38
    x[2] = np.where(rng.random(H) < 0.5, -1.0, 1.0)           # every |q| = 127
    x[3] = 1e-30
    x[4] = 0.0
    x[5, :] = 0.0
    x[5, 7] = -2.5e-36                                         # a scale close to the smallest accepted
    ids = np.stack([rng.permutation(E)[:top_k] for _ in range(T)]).astype(np.int32)
    routes = (rng.random((T, top_k), dtype=np.float32) + np.float32(0.1))
    routes[2, 0] = 0.0                                         # a dropped route
    moe = ops.MoeW8(sess, H, I, E, 0, top_k, 32, experts)
    try:
        rc, got = moe.run_f32(x, ids, routes)
        rc2, want = oracle.moe_w8(experts, H, I, E, 0, top_k, ids, routes, input_f32=x)
        assert rc == rc2
        if rc == 0:
            # A middle that overflows has no defined result in the reference (its scalar path casts
            # NaN to int, its NEON path saturates): such rows only have to be non-finite on both
            # sides, and must not disturb the other tokens of the batch.
            finite = np.isfinite(want).all(axis=1)
            assert not finite[0] and not finite[1] and finite[2:].all()
            assert not np.isfinite(got[~finite]).all(axis=1).any()
            assert np.array_equal(got[finite].view(np.uint32), want[finite].view(np.uint32))
        # the same call without the overflowing tokens
        keep = [2, 3, 4, 5, 6, 7, 8, 9, 10, 11]
        rc, got = moe.run_f32(x[keep], ids[keep], routes[keep])
        rc2, want = oracle.moe_w8(experts, H, I, E, 0, top_k, ids[keep], routes[keep], input_f32=x[keep])
        assert rc == 0 and rc2 == 0
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
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


# ---- INT4 experts, mixed banks, slot banks, packed records (reference include/rk_npu_moe_w8.h:83-143) ----

def _routes(rng, T, E, top_k):
    ids = np.stack([rng.permutation(E)[:top_k] for _ in range(T)]).astype(np.int32)
    routes = rng.random((T, top_k), dtype=np.float32) + np.float32(0.1)
    return ids, routes


@pytest.mark.parametrize("flavour,shared", [("quant", 0), ("quant", 1), ("w4", 1), ("w4", 0)])
def test_int4_experts_equal_the_int8_path(sess, oracle, flavour, shared):
    """The reference runs one test body against its W8 and its W4 factories (tests/test_moe_w8.cpp:52-57):
    INT4 experts are the W8 arithmetic with codes in [-8, 7]."""
    H, I, E, top_k, T = 128, 64, 5, 2, 37
    experts = _ref_experts(H, I, E, 0)[:E + shared]
    rng = np.random.default_rng(3)
    x = rng.standard_normal((T, H)).astype(np.float32)
    ids, routes = _routes(rng, T, E, top_k)
    moe = ops.MoeW8(sess, H, I, E, shared, top_k, 64, experts, flavour=flavour)
    try:
        rc, got = moe.run_f32(x, ids, routes)
        rc2, want = oracle.moe_w8(experts, H, I, E, shared, top_k, ids, routes, input_f32=x)
        assert rc == 0 and rc2 == 0
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        xq = rng.integers(-127, 128, (T, H), dtype=np.int8)
        sc = rng.random(T, dtype=np.float32) * np.float32(0.05) + np.float32(0.01)
        rc, got = moe.run_quantized(xq, sc, ids, routes)
        rc2, want = oracle.moe_w8(experts, H, I, E, shared, top_k, ids, routes, input_q=xq, row_scales=sc)
        assert rc == 0 and rc2 == 0
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        lib = sess.lib
        # INT4 experts are held as packed nibbles: a record is header + half a byte per weight
        # (+ padding to whole tiles) + scales, and the bank takes about half of an int8 bank
        blob = lib.rk_npu_moe_quant_expert_blob_bytes(moe.w)
        assert (2 * I * H + H * I) // 2 + (2 * I + H) * 4 < blob
        # handles of another expert format do not bind
        w8 = ops.MoeW8(sess, H, I, E, shared, top_k, 64, experts)
        try:
            assert lib.rk_npu_moe_quant_expert_blob_bytes(w8.w) == 0
            b4, b8 = lib.rk_npu_moe_w8_weights_device_bytes(moe.w), lib.rk_npu_moe_w8_weights_device_bytes(w8.w)
            int4_experts = E + shared if flavour == "quant" else E
            images8 = (b8 - (E + shared) * (2 * I + H) * 4) // (E + shared)   # int8 image bytes per expert
            assert b8 - b4 == int4_experts * images8 // 2
            assert moe.run_f32(x, ids, routes, weights=w8.w)[0] == capi.RK_NPU_ERR_PARAM
            assert w8.run_f32(x, ids, routes, weights=moe.w)[0] == capi.RK_NPU_ERR_PARAM
        finally:
            w8.close()
    finally:
        moe.close()


@pytest.mark.parametrize("flavour", ["quant", "w4"])
def test_int4_experts_at_prefill_size_take_the_balanced_launch(sess, oracle, flavour):
    """256 tokens, top-8 of 16 experts + the shared one, hidden 1024, intermediate 1024: the grouped
    GEMMs have about 75 row blocks x 32 (gate/up) and x 16 (down) column pairs, enough units for the
    balanced launch (one workgroup per compute unit) of both, here over packed int4 images; with "w4"
    the shared expert is int8, so the bank holds both formats and every grouped GEMM is one launch
    per format."""
    T, H, E, top_k, I = 256, 1024, 16, 8, 1024
    rng = np.random.default_rng(2024)
    experts = []
    for e in range(E + 1):
        lo, hi = (-8, 7) if (flavour == "quant" or e < E) else (-127, 127)
        experts.append((rng.integers(lo, hi + 1, (H, 2 * I)).astype(np.int8),
                        (rng.random(2 * I).astype(np.float32) + 0.5) * np.float32(0.02),
                        rng.integers(lo, hi + 1, (I, H)).astype(np.int8),
                        (rng.random(H).astype(np.float32) + 0.5) * np.float32(0.02)))
    x = rng.standard_normal((T, H)).astype(np.float32)
    ids, routes = _routes(rng, T, E, top_k)
    moe = ops.MoeW8(sess, H, I, E, 1, top_k, 256, experts, flavour=flavour)
    try:
        rc, got = moe.run_f32(x, ids, routes)
        rc2, want = oracle.moe_w8(experts, H, I, E, 1, top_k, ids, routes, input_f32=x)
        assert rc == 0 and rc2 == 0
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    finally:
        moe.close()


def test_int4_factories_validate_codes_geometry_and_layout(sess):
    lib = sess.lib
    H, I, E = 128, 64, 3
    base = _ref_experts(H, I, E, 0)

    def handle(flavour, experts, shared, h=H, i=I):
        probe = ops.MoeW8.__new__(ops.MoeW8)
        probe.s, probe.flavour = sess, flavour
        probe.cfg = capi.MoeConfig()
        lib.rk_npu_moe_w8_config_init(C.byref(probe.cfg), h, i, E, shared, 2, 8)
        try:
            w = probe.create_weights(experts)
        except RuntimeError:
            return None
        lib.rk_npu_moe_w8_weights_free(w)
        return True
    assert handle("quant", base, 1) and handle("w4", base, 1)
    wide = [list(e) for e in base]
    wide[1][0] = wide[1][0].copy()
    wide[1][0][5, 7] = 8                       # a routed expert outside [-8, 7]
    assert handle("w8", wide, 1) and not handle("quant", wide, 1) and not handle("w4", wide, 1)
    shared_wide = [list(e) for e in base]
    shared_wide[E][2] = shared_wide[E][2].copy()
    shared_wide[E][2][3, 3] = -100             # the shared expert: int8 in the mixed bank, INT4 in the all-INT4 one
    assert handle("w4", shared_wide, 1) and not handle("quant", shared_wide, 1)
    # hidden and intermediate must be multiples of 64 for the INT4 formats
    odd = _ref_experts(96, 64, E, 0)
    assert handle("w8", odd, 1, h=96) and not handle("quant", odd, 1, h=96)
    odd_i = _ref_experts(128, 32, E, 0)
    assert handle("w8", odd_i, 1, i=32) and not handle("w4", odd_i, 1, i=32)
    cfg = capi.MoeConfig()
    lib.rk_npu_moe_w8_config_init(C.byref(cfg), H, I, E, 1, 2, 8)
    cfg.native_input = 1
    assert not lib.rk_npu_moe_quant_workspace_create(sess.domain, C.byref(cfg))
    assert not lib.rk_npu_moe_w4_workspace_create(sess.domain, C.byref(cfg))
    ws = lib.rk_npu_moe_w8_workspace_create(sess.domain, C.byref(cfg))
    assert ws
    lib.rk_npu_moe_w8_workspace_free(ws)


def test_slot_banks_records_and_slot_exchange(sess, oracle):
    """reference include/rk_npu_moe_w8.h:107-143: export from a resident bank, import into empty slots in another
    order, run through the caller's expert -> slot map, exchange slots between banks."""
    lib = sess.lib
    H, I, E, top_k, T = 128, 64, 4, 2, 29
    experts = _ref_experts(H, I, E, 1)[:E]
    rng = np.random.default_rng(8)
    x = rng.standard_normal((T, H)).astype(np.float32)
    ids, routes = _routes(rng, T, E, top_k)
    full = ops.MoeW8(sess, H, I, E, 0, top_k, 32, experts, flavour="quant")
    bank = ops.MoeW8(sess, H, I, E, 0, top_k, 32, None, flavour="quant")
    cfgw = bank.cfg.weights
    bank.w = lib.rk_npu_moe_quant_slots_create(sess.domain, C.byref(cfgw))
    other = lib.rk_npu_moe_quant_slots_create(sess.domain, C.byref(cfgw))
    assert bank.w and other
    try:
        need = lib.rk_npu_moe_quant_expert_blob_bytes(full.w)
        assert need == lib.rk_npu_moe_quant_expert_blob_bytes(bank.w) > 0
        rc2, want = oracle.moe_w8(experts, H, I, E, 0, top_k, ids, routes, input_f32=x)
        assert rc2 == 0
        slot_of = [2, 0, 3, 1]                     # logical expert e lives in slot slot_of[e]
        records = []
        for e in range(E):
            rec = np.zeros(need + 64, np.uint8)    # a larger buffer is allowed (page-aligned stores)
            assert lib.rk_npu_moe_quant_export_expert(full.w, e, capi.ptr(rec), rec.nbytes) == 0
            assert lib.rk_npu_moe_quant_export_expert(full.w, e, capi.ptr(rec), need - 1) == capi.RK_NPU_ERR_PARAM
            records.append(rec)
        assert lib.rk_npu_moe_quant_export_expert(full.w, E, capi.ptr(records[0]), need) == capi.RK_NPU_ERR_PARAM
        t = capi.MoeImportTimings()
        for e in range(E):
            fn = lib.rk_npu_moe_quant_import_expert_timed if e % 2 else None
            if fn:
                assert fn(bank.w, slot_of[e], capi.ptr(records[e]), need, C.byref(t)) == 0 and t.total_us > 0
            else:
                assert lib.rk_npu_moe_quant_import_expert(bank.w, slot_of[e], capi.ptr(records[e]), need) == 0
        mapped = np.asarray(slot_of, np.int32)[ids]
        rc, got = bank.run_f32(x, mapped, routes)
        assert rc == 0 and np.array_equal(got.view(np.uint32), want.view(np.uint32))
        # rejected records leave the slot as it was
        bad = records[0].copy()
        bad[:4] = 0
        assert lib.rk_npu_moe_quant_import_expert(bank.w, slot_of[0], capi.ptr(bad), need) == capi.RK_NPU_ERR_PARAM
        # a record of the library's earlier layout (magic "RKHM", 16-byte header, int8 tiles): larger
        # than today's record for the same geometry, so only the header can give it away
        old = np.zeros(2 * need, np.uint8)
        old[:16] = np.frombuffer(np.array([0x4d484b52, 3, H, I], np.uint32).tobytes(), np.uint8)
        old[16:] = 0x11
        assert lib.rk_npu_moe_quant_import_expert(bank.w, slot_of[0], capi.ptr(old), 2 * need) == capi.RK_NPU_ERR_PARAM
        for field, value in ((4, 1), (6, 12345), (8, 7)):   # layout revision, gate/up image bytes, down image bytes
            bad = records[0].copy()
            bad[4 * field:4 * field + 4] = np.frombuffer(np.uint32(value).tobytes(), np.uint8)
            assert lib.rk_npu_moe_quant_import_expert(bank.w, slot_of[0], capi.ptr(bad), need) == capi.RK_NPU_ERR_PARAM
        bad = records[0].copy()
        bad[need - 4:need] = np.frombuffer(np.float32(-1.0).tobytes(), np.uint8)   # a negative down scale
        assert lib.rk_npu_moe_quant_import_expert(bank.w, slot_of[0], capi.ptr(bad), need) == capi.RK_NPU_ERR_PARAM
        assert lib.rk_npu_moe_quant_import_expert(bank.w, E, capi.ptr(records[0]), need) == capi.RK_NPU_ERR_PARAM
        assert lib.rk_npu_moe_quant_import_expert(bank.w, 0, capi.ptr(records[0]), need - 8) == capi.RK_NPU_ERR_PARAM
        rc, got = bank.run_f32(x, mapped, routes)
        assert rc == 0 and np.array_equal(got.view(np.uint32), want.view(np.uint32))
        # stage expert 0 in another bank, exchange it with the slot that holds expert 1
        assert lib.rk_npu_moe_quant_import_expert(other, 3, capi.ptr(records[0]), need) == 0
        assert lib.rk_npu_moe_quant_swap_slots(bank.w, slot_of[1], other, 3) == 0
        ids0 = np.where(ids == 1, 0, ids)          # route everything that wanted expert 1 to expert 0's new copy
        rc2, want0 = oracle.moe_w8(experts, H, I, E, 0, top_k, ids0, routes, input_f32=x)
        mapped0 = np.where(ids == 1, slot_of[1], np.asarray(slot_of, np.int32)[ids]).astype(np.int32)
        rc, got = bank.run_f32(x, mapped0, routes)
        assert rc == 0 and rc2 == 0 and np.array_equal(got.view(np.uint32), want0.view(np.uint32))
        back = np.zeros(need, np.uint8)            # and the staging bank received expert 1
        assert lib.rk_npu_moe_quant_export_expert(other, 3, capi.ptr(back), need) == 0
        assert np.array_equal(back, records[1][:need])
        assert lib.rk_npu_moe_quant_swap_slots(bank.w, E, other, 0) == capi.RK_NPU_ERR_PARAM
        assert lib.rk_npu_moe_quant_swap_slots(bank.w, 0, full.w, 0) == 0  # same geometry: any two INT4 banks
        assert lib.rk_npu_moe_quant_swap_slots(bank.w, 0, full.w, 0) == 0
    finally:
        lib.rk_npu_moe_w8_weights_free(other)
        bank.close()
        full.close()


def test_mixed_slot_bank_with_resident_shared_expert(sess, oracle):
    """reference include/rk_npu_moe_w8.h:101-106: routed INT4 slots are imported, the shared int8 expert is
    packed at creation and can neither be exported nor imported."""
    lib = sess.lib
    H, I, E, top_k, T = 64, 64, 3, 2, 11
    experts = _ref_experts(H, I, E, 0)
    experts[E] = (experts[E][0] * 30, experts[E][1], experts[E][2] * 30, experts[E][3])  # int8-range shared expert
    rng = np.random.default_rng(2)
    x = rng.standard_normal((T, H)).astype(np.float32)
    ids, routes = _routes(rng, T, E, top_k)
    src = ops.MoeW8(sess, H, I, E, 1, top_k, 16, experts, flavour="w4")
    bank = ops.MoeW8(sess, H, I, E, 1, top_k, 16, None, flavour="w4")
    g, gs, d, ds = [np.ascontiguousarray(a) for a in experts[E]]
    shared = capi.MoeExpert(g.ctypes.data, gs.ctypes.data, d.ctypes.data, ds.ctypes.data)
    bank.w = lib.rk_npu_moe_w4_slots_create(sess.domain, C.byref(bank.cfg.weights), C.byref(shared))
    assert bank.w
    try:
        need = lib.rk_npu_moe_quant_expert_blob_bytes(src.w)
        rec = np.zeros(need, np.uint8)
        for e in range(E):
            assert lib.rk_npu_moe_quant_export_expert(src.w, e, capi.ptr(rec), need) == 0
            assert lib.rk_npu_moe_quant_import_expert(bank.w, e, capi.ptr(rec), need) == 0
        assert lib.rk_npu_moe_quant_export_expert(src.w, E, capi.ptr(rec), need) == capi.RK_NPU_ERR_PARAM
        assert lib.rk_npu_moe_quant_import_expert(bank.w, E, capi.ptr(rec), need) == capi.RK_NPU_ERR_PARAM
        assert lib.rk_npu_moe_quant_swap_slots(bank.w, 0, src.w, 0) == capi.RK_NPU_ERR_PARAM  # all-INT4 banks only
        rc, got = bank.run_f32(x, ids, routes)
        rc2, want = oracle.moe_w8(experts, H, I, E, 1, top_k, ids, routes, input_f32=x)
        assert rc == 0 and rc2 == 0 and np.array_equal(got.view(np.uint32), want.view(np.uint32))
        no_shared = capi.MoeWeightConfig(H, I, E, 0)
        assert not lib.rk_npu_moe_w4_slots_create(sess.domain, C.byref(no_shared), C.byref(shared))
        assert not lib.rk_npu_moe_w4_slots_create(sess.domain, C.byref(bank.cfg.weights), None)
        assert not lib.rk_npu_moe_quant_slots_create(sess.domain, C.byref(bank.cfg.weights))  # needs shared_expert = 0
    finally:
        bank.close()
        src.close()


def _quant_scenario_experts(H, F, E):
    """Expert tensors of the reference's INT4 MoE test (tests/test_moe_quant.cpp:186-198)."""
    out = []
    for e in range(E):
        i = np.arange(H * 2 * F, dtype=np.int64)
        g = ((i * 7 + i // 23 + e * 5) % 15 - 7)
        if e == 0:
            g = np.trunc(g / 4)                 # C++ integer division truncates toward zero
        j = np.arange(F * H, dtype=np.int64)
        d = ((j * 3 + j // 11 + e * 7) % 15 - 7)
        gs = (np.float32(0.001) * (np.arange(2 * F) % 13 + 1).astype(np.float32)).astype(np.float32)
        ds = (np.float32(0.001) * (np.arange(H) % 7 + 1).astype(np.float32)).astype(np.float32)
        out.append((g.astype(np.int8).reshape(H, 2 * F), gs, d.astype(np.int8).reshape(F, H), ds))
    return out


def _sin_input(rows, H):
    i = np.arange(rows * H)
    return (np.sin((i % 97).astype(np.float32) * np.float32(0.13)) * np.float32(0.3)).astype(np.float32).reshape(rows, H)


def test_int4_bank_dense_partial_empty_dense_on_one_workspace(sess, oracle):
    """reference tests/test_moe_quant.cpp:42-83: one workspace through dense, partly dropped, fully dropped and
    dense routes again; every result equals the sum, in slot order, of independent single-route runs."""
    H, F, E, K, rows = 2048, 512, 3, 2, 5
    experts = _quant_scenario_experts(H, F, E)
    moe = ops.MoeW8(sess, H, F, E, 0, K, 128, experts, flavour="quant")
    single = ops.MoeW8(sess, H, F, E, 0, 1, 128, None, flavour="quant")
    try:
        x = _sin_input(rows, H)
        ids = ((np.arange(rows)[:, None] + np.arange(K)[None, :]) % E).astype(np.int32)
        for mode in (0, 1, 2, 0):
            rk = np.arange(rows)[:, None] + np.arange(K)[None, :]
            routes = np.where((mode == 2) | ((mode == 1) & (rk % 2 == 1)), 0.0, 0.25).astype(np.float32)
            t = capi.MoeTimings()
            rc, got = moe.run_f32(x, ids, routes, timings=t)
            assert rc == 0
            if mode == 2:
                assert t.gemm_tasks == 0 and t.gather_tasks == 0 and t.sync_us == 0
            want = np.zeros((rows, H), np.float32)
            for k in range(K):
                rc, part = single.run_f32(x, ids[:, k:k + 1].copy(), np.ones((rows, 1), np.float32), weights=moe.w)
                assert rc == 0
                live = routes[:, k] != 0
                fused = (part.astype(np.float64) * routes[:, k:k + 1].astype(np.float64) + want).astype(np.float32)
                want[live] = fused[live]        # fma: one rounding of the exact product-sum (exact in float64)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), mode
            rc2, ref = oracle.moe_w8(experts, H, F, E, 0, K, ids, routes, input_f32=x)
            assert rc2 == 0 and np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    finally:
        single.close()
        moe.close()


def test_staged_slot_promotion_with_a_concurrent_importer(sess):
    """reference tests/test_moe_quant.cpp:85-183: records are imported into a staging bank by another thread
    while the hot bank computes, then promoted slot by slot; imports into one staging slot run beside
    exchanges of another; the hot bank survives the staging bank's release."""
    import threading
    lib = sess.lib
    H, F, E, K, rows = 2048, 512, 3, 2, 5
    experts = _quant_scenario_experts(H, F, E)
    source = ops.MoeW8(sess, H, F, E, 0, K, 128, experts, flavour="quant")
    hot = ops.MoeW8(sess, H, F, E, 0, 1, 128, None, flavour="quant")
    hot.w = lib.rk_npu_moe_quant_slots_create(sess.domain, C.byref(hot.cfg.weights))
    stage = lib.rk_npu_moe_quant_slots_create(sess.domain, C.byref(hot.cfg.weights))
    assert hot.w and stage
    try:
        bank_bytes = lib.rk_npu_moe_w8_weights_device_bytes(hot.w)
        assert bank_bytes and lib.rk_npu_moe_w8_weights_device_bytes(stage) == bank_bytes
        need = lib.rk_npu_moe_quant_expert_blob_bytes(source.w)
        records = [np.zeros(need, np.uint8) for _ in range(E)]
        for e in range(E):
            assert lib.rk_npu_moe_quant_export_expert(source.w, e, capi.ptr(records[e]), need) == 0
            assert lib.rk_npu_moe_quant_import_expert(hot.w, e, capi.ptr(records[e]), need) == 0
        x = _sin_input(rows, H)
        physical = (np.arange(rows) % E).astype(np.int32)[:, None]
        ones = np.ones((rows, 1), np.float32)
        reference_routes = np.zeros((rows, K), np.float32)
        reference_routes[:, 0] = 1
        for iteration in range(9):                 # an odd number of promotions
            errors = []

            def importer():
                for slot in range(E):
                    t = capi.MoeImportTimings()
                    rec = records[(iteration + slot) % E]
                    rc = lib.rk_npu_moe_quant_import_expert_timed(stage, slot, capi.ptr(rec), need, C.byref(t))
                    if rc or min(t.copy_us, t.validate_us, t.gate_sync_us, t.down_sync_us) < 0 or t.total_us < t.copy_us:
                        errors.append((slot, rc))
            th = threading.Thread(target=importer)
            th.start()
            rc, _ = hot.run_f32(x, physical, ones)
            th.join()
            assert rc == 0 and not errors
            for slot in range(E):
                assert lib.rk_npu_moe_quant_swap_slots(hot.w, slot, stage, slot) == 0
            src_ids = np.repeat(((iteration + np.arange(rows) % E) % E).astype(np.int32)[:, None], K, axis=1)
            rc, want = source.run_f32(x, src_ids, reference_routes)
            rc2, got = hot.run_f32(x, physical, ones)
            assert rc == 0 and rc2 == 0 and np.array_equal(got.view(np.uint32), want.view(np.uint32)), iteration
        done = threading.Event()
        errors = []

        def importer2():
            for _ in range(256):
                if lib.rk_npu_moe_quant_expert_blob_bytes(stage) != need or \
                        lib.rk_npu_moe_quant_import_expert(stage, 1, capi.ptr(records[0]), need):
                    errors.append(1)
            done.set()
        th = threading.Thread(target=importer2)
        th.start()
        swaps = 0
        while not done.is_set():
            assert lib.rk_npu_moe_quant_swap_slots(hot.w, 0, stage, 0) == 0
            swaps += 1
        th.join()
        assert not errors and swaps > 0
        if swaps % 2:
            assert lib.rk_npu_moe_quant_swap_slots(hot.w, 0, stage, 0) == 0
        back = np.zeros(need, np.uint8)
        assert lib.rk_npu_moe_quant_export_expert(stage, 1, capi.ptr(back), need) == 0
        assert np.array_equal(back, records[0])
        lib.rk_npu_moe_w8_weights_free(stage)
        stage = None
        assert lib.rk_npu_moe_w8_weights_device_bytes(hot.w) == bank_bytes
        rc2, again = hot.run_f32(x, physical, ones)
        assert rc2 == 0 and np.array_equal(again.view(np.uint32), want.view(np.uint32))
    finally:
        if stage:
            lib.rk_npu_moe_w8_weights_free(stage)
        hot.close()
        source.close()


def test_mixed_bank_rotating_slots_duplicates_and_dropped_routes(sess, oracle):
    """reference tests/test_moe_quant.cpp:262-342: INT4 records bound to a full-range shared int8 expert; imported
    slots in rotating order equal the independently packed resident bank, with duplicate ids, dropped routes
    and rows whose routed coefficients are all zero (the shared expert still contributes); a batch row equals
    the same row run alone."""
    lib = sess.lib
    H, F, E, K = 2048, 512, 3, 2
    experts = _quant_scenario_experts(H, F, E)
    i = np.arange(H * 2 * F, dtype=np.int64)
    j = np.arange(F * H, dtype=np.int64)
    shared_t = (((i * 11 + i // 19) % 255 - 127).astype(np.int8).reshape(H, 2 * F), np.full(2 * F, 0.0003, np.float32),
                ((j * 13 + j // 17) % 255 - 127).astype(np.int8).reshape(F, H), np.full(H, 0.0004, np.float32))
    allx = experts + [shared_t]
    packed = ops.MoeW8(sess, H, F, E, 0, K, 128, experts, flavour="quant")
    mixed = ops.MoeW8(sess, H, F, E, 1, K, 128, allx, flavour="w4")
    shared = capi.MoeExpert(*[a.ctypes.data for a in shared_t])
    slots = lib.rk_npu_moe_w4_slots_create(sess.domain, C.byref(mixed.cfg.weights), C.byref(shared))
    assert slots
    try:
        need = lib.rk_npu_moe_quant_expert_blob_bytes(packed.w)
        assert lib.rk_npu_moe_quant_expert_blob_bytes(slots) == need == lib.rk_npu_moe_quant_expert_blob_bytes(mixed.w)
        stride = (need + 4095) // 4096 * 4096
        blob, trip = np.zeros(stride, np.uint8), np.zeros(stride, np.uint8)
        for rotation, rows in enumerate((1, 5, 128, 1)):
            for e in range(E):
                slot = (e + rotation) % E
                assert lib.rk_npu_moe_quant_export_expert(packed.w, e, capi.ptr(blob), stride) == 0
                assert lib.rk_npu_moe_quant_export_expert(mixed.w, e, capi.ptr(trip), stride) == 0
                assert np.array_equal(blob, trip)
                assert lib.rk_npu_moe_quant_import_expert(slots, slot, capi.ptr(blob), stride) == 0
                assert lib.rk_npu_moe_quant_export_expert(slots, slot, capi.ptr(trip), stride) == 0
                assert np.array_equal(blob, trip)
            x = _sin_input(rows, H)
            r = np.arange(rows)[:, None]
            k = np.arange(K)[None, :]
            ids = ((r + np.where(r % 2 == 1, k, 0)) % E).astype(np.int32)
            physical = ((ids + rotation) % E).astype(np.int32)
            routes = np.where((r % 3 == 2) | ((r % 3 == 1) & (k > 0)), 0.0, np.where(k > 0, 0.375, 0.875)).astype(np.float32)
            rc, want = mixed.run_f32(x, ids, routes)
            rc2, got = mixed.run_f32(x, physical, routes, weights=slots)
            assert rc == 0 and rc2 == 0 and np.array_equal(got.view(np.uint32), want.view(np.uint32))
            rc3, ref = oracle.moe_w8(allx, H, F, E, 1, K, ids, routes, input_f32=x)
            assert rc3 == 0 and np.array_equal(want.view(np.uint32), ref.view(np.uint32))
            assert np.isfinite(got).all()
            if rows > 2:
                assert (got[2] != 0).any()          # all routed coefficients zero: the shared expert remains
            for row in {0, rows // 2, rows - 1}:
                rc, alone = mixed.run_f32(x[row:row + 1], ids[row:row + 1], routes[row:row + 1])
                assert rc == 0 and np.array_equal(alone[0].view(np.uint32), want[row].view(np.uint32))
    finally:
        lib.rk_npu_moe_w8_weights_free(slots)
        mixed.close()
        packed.close()
