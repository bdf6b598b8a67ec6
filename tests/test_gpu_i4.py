"""GPU parity of the exact W4A4 integer GEMM, after the reference's tests/test_i4.cpp: every output equals the
int64 product (:15-25) with guard words around C untouched (:47-49), over tails, tile settings, core masks and
extreme codes (:141-172); weights shared across M, the producer boundary, BUSY from inside a producer, DOMAIN,
a failing producer followed by a good run, rejected activation / weight codes (:77-121)."""
import ctypes as C

import numpy as np
import pytest

from rknpu2_matmul_open_amd import capi, ops

pytestmark = pytest.mark.gpu


def _exact(a, b):
    # |sum| <= K * 64 < 2**53: the float64 product (BLAS) is the exact integer product
    return np.rint(a.astype(np.float64) @ b.astype(np.float64)).astype(np.int64).astype(np.int32)


def _run(sess, M, K, N, mt, kt, nt, mask, pipe, extreme=False, seed=0):
    lib = sess.lib
    rng = np.random.default_rng(91 + seed)
    if extreme:
        a = np.full((M, K), -8, np.int8)
        b = np.where(np.arange(K * N).reshape(K, N) % N % 2 == 1, 7, -8).astype(np.int8)
    else:
        a = rng.integers(-8, 8, (M, K), dtype=np.int8)
        b = rng.integers(-8, 8, (K, N), dtype=np.int8)
    cfg = capi.I4Config()
    lib.rk_npu_i4_config_init(C.byref(cfg), M, N, K)
    cfg.m_tile, cfg.k_tile, cfg.n_tile, cfg.npu_core_mask, cfg.pipeline = mt, kt, nt, mask, pipe
    cfg.cpu_threads = 4 if M >= 128 else 1
    wc = capi.I4WeightConfig(K, N, kt)
    w = lib.rk_npu_i4i4i32_weights_create(sess.domain, C.byref(wc), capi.ptr(b))
    ws = lib.rk_npu_i4_workspace_create(sess.domain, C.byref(cfg))
    assert w and ws
    try:
        out = np.full(M * N + 32, 0x12345678, np.int32)
        view = out[16:16 + M * N]
        for repeat in range(3):
            if not extreme:
                a.reshape(-1)[repeat % a.size] = repeat - 8
            t = capi.I4Timings()
            assert lib.rk_npu_i4i4i32_run(ws, w, capi.ptr(a), view.ctypes.data_as(C.c_void_p), C.byref(t)) == 0
            assert np.array_equal(view.reshape(M, N), _exact(a, b))
            assert (out[:16] == 0x12345678).all() and (out[-16:] == 0x12345678).all()
            assert t.total_us > 0 and t.submit_us > 0
    finally:
        lib.rk_npu_i4_workspace_free(ws)
        lib.rk_npu_i4i4i32_weights_free(w)


@pytest.mark.parametrize("pipe", [0, 1])
def test_shapes_tiles_and_extreme_codes(sess, pipe):
    _run(sess, 2, 480, 64, 128, 480, 1024, 1, 0)
    _run(sess, 1, 1, 1, 128, 480, 1024, 1, pipe, seed=1)
    _run(sess, 3, 33, 65, 2, 32, 64, 1, pipe, seed=2)
    _run(sess, 129, 513, 193, 32, 256, 64, 1, pipe, seed=3)
    _run(sess, 5, 2048, 128, 4, 480, 64, 1, pipe, extreme=True)
    _run(sess, 2, 64, 8128, 128, 480, 8128, 1, pipe, seed=4)
    _run(sess, 2, 64, 8192, 128, 480, 8128, 1, pipe, seed=5)
    _run(sess, 129, 513, 513, 64, 256, 128, 7, pipe, seed=6)


@pytest.mark.parametrize("mask", [2, 4, 3, 7])
def test_core_masks(sess, mask):
    _run(sess, 7, 511, 257, 3, 480, 64, mask, 1, extreme=True)
    _run(sess, 129, 1025, 257, 64, 256, 128, mask, 1, seed=mask)
    _run(sess, 2, 64, 4161, 128, 480, 4096, 1, 1, seed=9)


def test_prefill_size_is_exact(sess):
    """the dense tiles of the int4 GEMM (128 rows) with int4 activations"""
    _run(sess, 640, 4096, 1536, 128, 480, 1024, 7, 1, seed=11)


def _generated(m, k):
    return (m * 7 + k * 3) % 16 - 8


def test_sharing_producer_busy_domain_and_recovery(sess):
    """reference tests/test_i4.cpp:77-121"""
    lib = sess.lib
    K, N = 513, 193
    b = np.full((K, N), 3, np.int8)
    b2 = np.full((K, N), -2, np.int8)
    wc = capi.I4WeightConfig(K, N, 256)
    other = ops.Session(domain_id=1)
    w = lib.rk_npu_i4i4i32_weights_create(sess.domain, C.byref(wc), capi.ptr(b))
    w2 = lib.rk_npu_i4i4i32_weights_create(sess.domain, C.byref(wc), capi.ptr(b2))
    foreign = lib.rk_npu_i4i4i32_weights_create(other.domain, C.byref(wc), capi.ptr(b))
    assert w and w2 and foreign
    try:
        for M in (1, 5, 131):
            cfg = capi.I4Config()
            lib.rk_npu_i4_config_init(C.byref(cfg), M, N, K)
            cfg.k_tile, cfg.m_tile, cfg.n_tile, cfg.npu_core_mask = 256, (1 if M == 1 else 32), 64, (7 if M == 131 else 1)
            ws = lib.rk_npu_i4_workspace_create(sess.domain, C.byref(cfg))
            assert ws
            a = np.fromfunction(lambda m, k: (m * 7 + k * 3) % 16 - 8, (M, K), dtype=np.int64).astype(np.int8)
            c = np.empty((M, N), np.int32)
            state = {"fail_k": -1, "busy": [], "order": []}

            def produce(user, tile):
                t = tile.contents
                state["order"].append((t.k0, t.m0))
                dummy = np.zeros(K, np.int8)
                state["busy"].append(lib.rk_npu_i4i4i32_run(ws, w, capi.ptr(dummy), capi.ptr(c), None))
                if t.k0 == state["fail_k"]:
                    return capi.RK_NPU_ERR_PARAM
                assert t.bytes == t.rows * t.padded_k // 2 and t.padded_k % 32 == 0
                dst = np.ctypeslib.as_array(t.dst, shape=(t.bytes,))
                assert not dst.any()  # zero-initialised
                kk, mm = np.meshgrid(np.arange(t.k), np.arange(t.rows), indexing="ij")
                index = (kk // 32 * t.rows + mm) * 32 + kk % 32
                q = (((t.m0 + mm) * 7 + (t.k0 + kk) * 3) % 16 - 8) & 15
                np.bitwise_or.at(dst, index // 2, np.where(index & 1, q, q << 4).astype(np.uint8))
                return 0
            cb = capi.I4_INPUT_PRODUCER(produce)
            assert lib.rk_npu_i4i4i32_run_with_producer(ws, w, cb, None, capi.ptr(c), None) == 0
            assert np.array_equal(c, _exact(a, b))
            assert set(state["busy"]) == {capi.RK_NPU_ERR_BUSY}
            assert state["order"] == sorted(state["order"])  # increasing K, then M
            assert len(state["order"]) == 3 * -(-M // cfg.m_tile)
            assert lib.rk_npu_i4i4i32_run(ws, w2, capi.ptr(a), capi.ptr(c), None) == 0
            assert np.array_equal(c, _exact(a, b2))
            assert lib.rk_npu_i4i4i32_run(ws, foreign, capi.ptr(a), capi.ptr(c), None) == capi.RK_NPU_ERR_DOMAIN
            state["fail_k"] = 256
            assert lib.rk_npu_i4i4i32_run_with_producer(ws, w, cb, None, capi.ptr(c), None) == capi.RK_NPU_ERR_PARAM
            state["fail_k"] = -1
            assert lib.rk_npu_i4i4i32_run_with_producer(ws, w, cb, None, capi.ptr(c), None) == 0
            assert np.array_equal(c, _exact(a, b))
            a[-1, -1] = 8
            assert lib.rk_npu_i4i4i32_run(ws, w, capi.ptr(a), capi.ptr(c), None) == capi.RK_NPU_ERR_PARAM
            a[-1, -1] = _generated(M - 1, K - 1)
            assert lib.rk_npu_i4i4i32_run(ws, w, capi.ptr(a), capi.ptr(c), None) == 0
            assert np.array_equal(c, _exact(a, b))
            # weights of another K partition do not bind
            wc3 = capi.I4WeightConfig(K, N, 480)
            w3 = lib.rk_npu_i4i4i32_weights_create(sess.domain, C.byref(wc3), capi.ptr(b))
            assert w3 and lib.rk_npu_i4i4i32_run(ws, w3, capi.ptr(a), capi.ptr(c), None) == capi.RK_NPU_ERR_PARAM
            lib.rk_npu_i4i4i32_weights_free(w3)
            lib.rk_npu_i4_workspace_free(ws)
        b[0, 0] = 8
        assert not lib.rk_npu_i4i4i32_weights_create(sess.domain, C.byref(wc), capi.ptr(b))
        # k_tile above 480 needs the INT16-partial certificate: all -8 certifies 480, not 512
        worst = np.full((1024, 64), -8, np.int8)
        assert not lib.rk_npu_i4i4i32_weights_create(sess.domain, C.byref(capi.I4WeightConfig(1024, 64, 512)),
                                                     capi.ptr(worst))
        mild = np.ones((1024, 64), np.int8)
        ok = lib.rk_npu_i4i4i32_weights_create(sess.domain, C.byref(capi.I4WeightConfig(1024, 64, 1024)), capi.ptr(mild))
        assert ok
        lib.rk_npu_i4i4i32_weights_free(ok)
    finally:
        for h in (w, w2, foreign):
            lib.rk_npu_i4i4i32_weights_free(h)
        other.close()
