"""GPU parity of the W4A8 linear, the fused SwiGLU and the FFN block.

Integer intermediates (int8 activations, int32 accumulators, Down's int8
re-quantized middle) and all fp32 / fp16 outputs are compared bit-exactly with
the CPU oracle evaluated with the polynomial exponential (the flavour the
reference's AArch64 production build runs); the libm flavour is checked within
the reference's own 7e-7 relative bound.
Cases follow the reference's tests/test_w4a8.cpp:21-40,71-162 (tails, zero
row, +-127 extremes, large sums, NaN / -Inf rejection, invalid scale / code,
foreign domain) and tests/test_w4a8_ffn.cpp:63-117.
"""
import ctypes as C

import numpy as np
import pytest

from rknpu2_matmul_open_amd import capi, ops, workloads

pytestmark = pytest.mark.gpu


def _codes(rng, shape, lo=-8, hi=7):
    return rng.integers(lo, hi + 1, shape).astype(np.int8)


def _bits32(x):
    return np.ascontiguousarray(x, np.float32).view(np.uint32)


SHAPES = [(1, 64, 64), (1, 65, 33), (3, 65, 33), (2, 65, 20003), (8, 128, 512), (9, 200, 96),
          (40, 130, 257), (64, 256, 1024), (100, 320, 640), (130, 1000, 300),
          # weight-streaming kernel without the in-workgroup K split (>= 128 column tiles x row blocks),
          # K a single / an odd number of 64-deep super-tiles
          (70, 11000, 192), (33, 33000, 40),
          # >= 160 tiles of 128 x 256: the large-tile kernel (ragged M / N / K, K shorter than its look-ahead)
          (650, 6900, 1000), (641, 6912, 200),
          # decode GEMV variants: 16 columns per workgroup (one row: rolling load window; several rows),
          # 32 columns per workgroup on a wide matrix, K staged in several chunks
          (1, 4096, 4096), (3, 2500, 1000), (1, 9000, 520), (8, 8200, 5000),
          # degenerate and lopsided: single k / column, far more rows than columns, very wide matrices
          (1, 1, 1), (2500, 3, 2), (1, 70001, 64), (9, 70001, 40), (300, 30000, 70),
          # 64-row tiles of the large-tile kernel; K split over workgroups + reduce launch; two / three rows
          # on a wide matrix
          (300, 8448, 200), (200, 96, 5000), (2, 9000, 300), (3, 9000, 200),
          # 129 .. 256 rows on a narrow matrix: the streaming kernel (K split over its waves); beyond its K limit: 64-row tiles
          (200, 2000, 300), (256, 1000, 8300), (150, 96, 17000), (300, 1024, 200), (200, 1, 70), (512, 2, 16384),
          # four to seven rows on a wide matrix: the eight-row decode kernel (rows fit its staging area), the
          # streaming kernel beyond
          (6, 8224, 1000), (7, 9000, 4096), (4, 9000, 4200),
          # up to 128 column blocks: 16 columns per workgroup, two / eight rows behind a quantization launch
          (2, 4000, 300), (8, 3000, 300),
          # 65 .. 128 rows whose 32 x 256 tiles outnumber the compute units: the large-tile kernel
          (70, 22100, 64)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_w4a8_f32_and_f16_bit_exact(sess, oracle, M, N, K):
    rng = np.random.default_rng(M * 7919 + N * 31 + K)
    B = _codes(rng, (K, N))
    ws = (rng.random(N).astype(np.float32) + 0.5) * 0.02
    A = (rng.standard_normal((M, K)) * 2).astype(np.float32)
    if M >= 3:
        A[1, :] = 0.0                                   # zero row -> scale 1
        A[2, : min(K, 8)] = [127, -127, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5][: min(K, 8)]
        A[2, min(K, 8):] = 0.0                          # max 127 -> scale exactly 1, exact ties
    w = ops.W4A8Weights(sess, B, ws)
    wsp = ops.W4A8Workspace(sess, M, N, K)
    try:
        want = oracle.w4a8(A, B, ws)
        rc, acc = wsp.run_i32(w, A)
        assert rc == 0
        q, s = wsp.read_quantized()
        assert np.array_equal(_bits32(s), _bits32(want["a_scale"]))
        assert np.array_equal(q, want["q"])
        assert np.array_equal(acc, want["acc"])
        rc, got = wsp.run_f32(w, A)
        assert rc == 0 and np.array_equal(_bits32(got), _bits32(want["C"]))
        A16 = A.astype(np.float16).view(np.uint16)
        want16 = oracle.w4a8(A16, B, ws)
        rc, got16 = wsp.run_f16(w, A16)
        assert rc == 0 and np.array_equal(got16, want16["C"])
    finally:
        wsp.close()
        w.close()


@pytest.mark.parametrize("M", [1, 2, 9, 200])
def test_w4a8_k_beyond_one_part_of_the_times16_range(sess, oracle, M):
    """K > 2^17: the MFMA kernels carry int4 codes as 16 * code, so one K part may not span more
    than 2^17 k before an extreme int32 sum could wrap; longer K is split into parts (M > 8), and
    the decode kernels (M <= 8) multiply the nibbles as they are.  Extreme codes and activations
    make every wrong split show: |sum| = 127 * 8 * K = 1.35e8, times 16 = 2.16e9 > 2^31."""
    N, K = 96, 131072 + 2048 + 64
    rng = np.random.default_rng(M + 4242)
    B = np.full((K, N), -8, np.int8)
    B[:, 1::2] = 7
    B[:, 2::5] = _codes(rng, (K, len(range(2, N, 5))))
    ws = (rng.random(N).astype(np.float32) + 0.5) * 0.001
    A = (rng.standard_normal((M, K)) * 2).astype(np.float32)
    A[0] = 127.0                                        # q = 127 everywhere
    if M > 1:
        A[M - 1] = -127.0
    w = ops.W4A8Weights(sess, B, ws)
    wsp = ops.W4A8Workspace(sess, M, N, K)
    try:
        want = oracle.w4a8(A, B, ws)
        assert int(np.abs(want["acc"].astype(np.int64)).max()) * 16 > 2**31   # the case is what it claims
        rc, acc = wsp.run_i32(w, A)
        assert rc == 0 and np.array_equal(acc, want["acc"])
        rc, got = wsp.run_f32(w, A)
        assert rc == 0 and np.array_equal(_bits32(got), _bits32(want["C"]))
    finally:
        wsp.close()
        w.close()


@pytest.mark.parametrize("M", [1, 9, 130])
def test_w4a8_k_at_the_api_limit(sess, oracle, M):
    """K = INT32_MAX / 1024, the largest the reference accepts (src/rk_npu_w4a8.cpp:47): with
    q = 127 against a column of -8 the sum is 2.13e9, just inside int32 -- which is what the limit
    is for -- and it must come out exactly from the decode, streaming and large-tile kernels."""
    N, K = 40, 2147483647 // 1024
    rng = np.random.default_rng(M + 77)
    B = _codes(rng, (K, N))
    B[:, 0] = -8
    B[:, 1] = 7
    ws = (rng.random(N).astype(np.float32) + 0.5) * 1e-4
    A = rng.standard_normal((M, K)).astype(np.float32)
    A[0] = 127.0
    w = ops.W4A8Weights(sess, B, ws)
    wsp = ops.W4A8Workspace(sess, M, N, K)
    try:
        want = oracle.w4a8(A, B, ws)
        assert int(np.abs(want["acc"].astype(np.int64)).max()) > 2 ** 31 - 2 ** 25
        rc, acc = wsp.run_i32(w, A)
        assert rc == 0 and np.array_equal(acc, want["acc"])
        rc, got = wsp.run_f32(w, A)
        assert rc == 0 and np.array_equal(_bits32(got), _bits32(want["C"]))
    finally:
        wsp.close()
        w.close()


@pytest.mark.parametrize("M,N,K", [(1, 3_000_001, 40), (9, 3_000_001, 40), (70, 1_000_003, 33), (300_001, 300, 33)])
def test_w4a8_millions_of_columns_or_rows(sess, oracle, M, N, K):
    """No upper limit on M and N in the API (src/rk_npu_w4a8.cpp:47 bounds K only)."""
    rng = np.random.default_rng(M + N + 1)
    B = _codes(rng, (K, N))
    ws = (rng.random(N).astype(np.float32) + 0.5) * 1e-2
    A = rng.standard_normal((M, K)).astype(np.float32)
    w = ops.W4A8Weights(sess, B, ws)
    wsp = ops.W4A8Workspace(sess, M, N, K)
    try:
        rc, got = wsp.run_f32(w, A)
        want = oracle.w4a8(A, B, ws)["C"]
        assert rc == 0 and np.array_equal(_bits32(got), _bits32(want))
    finally:
        wsp.close()
        w.close()


def test_w4a8_extremes_and_tiny_scale(sess, oracle):
    M, N, K = 4, 64, 2048
    B = np.full((K, N), -8, np.int8)
    B[:, 1::2] = 7
    ws = np.full(N, 0.001, np.float32)
    A = np.zeros((M, K), np.float32)
    A[0] = 127.0                      # q = 127 everywhere: |sum| = 127*8*2048 > 2^20
    A[1] = -3.0
    A[2, 0] = np.float32(1e-40)       # denormal maximum: scale floors at FLT_MIN
    A[3, 5] = np.float32(2e-36)
    w = ops.W4A8Weights(sess, B, ws)
    wsp = ops.W4A8Workspace(sess, M, N, K)
    try:
        want = oracle.w4a8(A, B, ws)
        rc, got = wsp.run_f32(w, A)
        q, s = wsp.read_quantized()
        assert rc == 0
        assert np.array_equal(_bits32(s), _bits32(want["a_scale"]))
        assert s[2] == np.finfo(np.float32).tiny
        assert np.array_equal(q, want["q"])
        assert np.array_equal(_bits32(got), _bits32(want["C"]))
    finally:
        wsp.close()
        w.close()


def test_w4a8_rejections(sess):
    lib = sess.lib
    M, N, K = 3, 65, 33
    rng = np.random.default_rng(2)
    B = _codes(rng, (K, N))
    ws = np.full(N, 0.01, np.float32)
    w = ops.W4A8Weights(sess, B, ws)
    wsp = ops.W4A8Workspace(sess, M, N, K)
    try:
        A = rng.standard_normal((M, K)).astype(np.float32)
        sentinel = np.full((M, N), 123.0, np.float32)
        for bad in (np.nan, -np.inf, np.inf):
            Ab = A.copy()
            Ab[1, 7] = bad
            out = sentinel.copy()
            t = capi.W4A8Timings()
            rc = lib.rk_npu_w4a8_run_f32(wsp.h, w.h, capi.ptr(Ab), capi.ptr(out), C.byref(t))
            assert rc == capi.RK_NPU_ERR_PARAM
            assert (out == 123.0).all() and t.submit_us == 0
        # the workspace still works afterwards
        rc, _ = wsp.run_f32(w, A)
        assert rc == 0
        # A == C alias
        buf = np.zeros((M, max(N, K)), np.float32)
        assert lib.rk_npu_w4a8_run_f32(wsp.h, w.h, capi.ptr(buf), capi.ptr(buf), None) == capi.RK_NPU_ERR_PARAM
        # invalid scale / code -> NULL
        cfg = capi.I4WeightConfig(K, N, 480)
        for v in (0.0, -1.0, np.nan, np.inf):
            bs = ws.copy()
            bs[3] = v
            assert not lib.rk_npu_w4a8_weights_create(sess.domain, C.byref(cfg), capi.ptr(B), capi.ptr(bs))
        for v in (8, -9):
            Bb = B.copy()
            Bb[5, 6] = v
            assert not lib.rk_npu_w4a8_weights_create(sess.domain, C.byref(cfg), capi.ptr(Bb), capi.ptr(ws))
        # k_tile mismatch -> PARAM, foreign domain -> DOMAIN
        w2 = ops.W4A8Weights(sess, B, ws, k_tile=32)
        rc, _ = wsp.run_f32(w2, A)
        assert rc == capi.RK_NPU_ERR_PARAM
        w2.close()
        other = lib.rk_npu_iommu_domain_create(sess.ctx, 9)
        foreign = lib.rk_npu_w4a8_weights_create(other, C.byref(cfg), capi.ptr(B), capi.ptr(ws))
        assert foreign
        out = np.empty((M, N), np.float32)
        assert lib.rk_npu_w4a8_run_f32(wsp.h, foreign, capi.ptr(A), capi.ptr(out), None) == capi.RK_NPU_ERR_DOMAIN
        lib.rk_npu_w4a8_weights_free(foreign)
        lib.rk_npu_iommu_domain_free(other)
        # SwiGLU needs N % 64 == 0
        mid = np.empty((M, N // 2 + 1), np.float32)
        assert lib.rk_npu_w4a8_run_swiglu_f32(wsp.h, w.h, capi.ptr(A), capi.ptr(mid), None) == capi.RK_NPU_ERR_PARAM
    finally:
        wsp.close()
        w.close()


SWIGLU_SHAPES = [(1, 64, 64), (1, 4160, 1000), (2, 192, 20003),  # one / two rows: the SwiGLU GEMV (ragged K, K in chunks)
                 (3, 4160, 1000), (4, 192, 20003), (4, 64, 64),     # three / four rows on the same kernel
                 (5, 128, 96), (16, 192, 257), (33, 256, 512), (70, 640, 384),
                 (128, 1024, 512),
                 (20, 32896, 128), (32, 2048, 700),  # weight-streaming kernel: wide grid / K split inside the workgroup
                 (8, 32896, 128), (6, 2048, 700),    # the same with five to eight rows (beyond the SwiGLU GEMV's four)
                 (650, 6912, 520), (641, 7040, 300),  # large-tile kernel (F a multiple of 64 / only of 32)
                 (40, 128, 4100)]  # two 32-row tiles: K split over workgroups, SwiGLU in the reduce launch


@pytest.mark.parametrize("M,N,K", SWIGLU_SHAPES)
def test_swiglu_bit_exact_poly_and_close_to_libm(sess, oracle, M, N, K):
    rng = np.random.default_rng(N * 13 + K + M)
    B = _codes(rng, (K, N), -7, 7)
    ws = (rng.random(N).astype(np.float32) + 0.5) * 0.01
    A = (rng.standard_normal((M, K)) * 1.5).astype(np.float32)
    w = ops.W4A8Weights(sess, B, ws)
    wsp = ops.W4A8Workspace(sess, M, N, K)
    try:
        rc, mid = wsp.run_swiglu_f32(w, A)
        assert rc == 0
        poly = oracle.w4a8_swiglu(A, B, ws, oracle.EXP_POLY)
        assert np.array_equal(_bits32(mid), _bits32(poly["middle"]))
        libm = oracle.w4a8_swiglu(A, B, ws, oracle.EXP_LIBM)["middle"]
        denom = np.maximum(np.abs(libm), 1e-30)
        assert (np.abs(mid - libm) / denom).max() <= 7e-7 + 1e-12
        # the plain run on the same (interleaved) weights must still be in logical column order
        rc, full = wsp.run_f32(w, A)
        assert rc == 0 and np.array_equal(_bits32(full), _bits32(oracle.w4a8(A, B, ws)["C"]))
    finally:
        wsp.close()
        w.close()


FFN_SHAPES = [(1, 64, 64, 64), (2, 256, 2048, 300), (3, 1000, 4160, 300), (4, 256, 2048, 65), (7, 128, 96, 65), (33, 256, 160, 128), (64, 512, 1024, 300),
              (128, 384, 2048, 256),
              # an intermediate beyond 2^17: the down projection's K is split into parts, M <= 8 and M > 8
              (2, 64, 131072 + 2112, 40), (9, 64, 131072 + 2112, 40),
              # many rows (large-tile kernels on both projections), a very long hidden size, many rows x few columns
              (700, 264, 1056, 300), (1, 70000, 96, 40), (5, 70000, 96, 40), (3000, 96, 64, 33), (20000, 64, 32, 1)]


@pytest.mark.parametrize("M,H,I,Nout", FFN_SHAPES)
def test_ffn_bit_exact(sess, oracle, M, H, I, Nout):
    rng = np.random.default_rng(M + H + I)
    B_gu = _codes(rng, (H, 2 * I), -7, 7)
    s_gu = (rng.random(2 * I).astype(np.float32) + 0.5) * 0.01
    B_dn = _codes(rng, (I, Nout), -7, 7)
    s_dn = (rng.random(Nout).astype(np.float32) + 0.5) * 0.01
    x = rng.standard_normal((M, H)).astype(np.float32)
    if M > 2:
        x[1] = 0.0  # zero token -> zero middle row -> Down scale 1
    gw, dw = ops.W4A8Weights(sess, B_gu, s_gu), ops.W4A8Weights(sess, B_dn, s_dn)
    gws, dws = ops.W4A8Workspace(sess, M, 2 * I, H), ops.W4A8Workspace(sess, M, Nout, I)
    try:
        t = capi.W4A8FfnTimings()
        rc, mid, out = ops.w4a8_ffn(sess, gws, gw, dws, dw, x, t)
        assert rc == 0
        want = oracle.w4a8_ffn(x, B_gu, s_gu, B_dn, s_dn, oracle.EXP_POLY)
        assert want["rc"] == 0
        assert np.array_equal(_bits32(mid), _bits32(want["middle"]))
        qd, sd = dws.read_quantized()
        assert np.array_equal(_bits32(sd), _bits32(want["down_scale"]))
        assert np.array_equal(qd, want["q_down"])
        assert np.array_equal(_bits32(out), _bits32(want["C"]))
        assert t.down.activation_scan_us == 0 and t.total_us > 0
        # FFN == swiglu followed by run_f32 on the middle, bitwise
        # (reference tests/test_w4a8_ffn.cpp:153-157)
        rc, mid2 = gws.run_swiglu_f32(gw, x)
        rc2, out2 = dws.run_f32(dw, mid2)
        assert rc == 0 and rc2 == 0
        assert np.array_equal(_bits32(mid2), _bits32(mid)) and np.array_equal(_bits32(out2), _bits32(out))
        # end-to-end against the libm flavour within the benchmark tolerance
        libm = oracle.w4a8_ffn(x, B_gu, s_gu, B_dn, s_dn, oracle.EXP_LIBM)["C"]
        assert np.abs(out - libm).max() <= 1e-3 * max(np.abs(libm).max(), 1e-30)
    finally:
        for o in (gws, dws, gw, dw):
            o.close()


def test_ffn_argument_checks_and_nonfinite_middle(sess):
    lib = sess.lib
    M, H, I, Nout = 4, 64, 64, 64
    rng = np.random.default_rng(1)
    B_gu, B_dn = _codes(rng, (H, 2 * I)), _codes(rng, (I, Nout))
    s_gu = np.full(2 * I, 0.01, np.float32)
    s_dn = np.full(Nout, 0.01, np.float32)
    gw, dw = ops.W4A8Weights(sess, B_gu, s_gu), ops.W4A8Weights(sess, B_dn, s_dn)
    gws, dws = ops.W4A8Workspace(sess, M, 2 * I, H), ops.W4A8Workspace(sess, M, Nout, I)
    dws_m = ops.W4A8Workspace(sess, M + 1, Nout, I)
    try:
        x = rng.standard_normal((M, H)).astype(np.float32)
        mid = np.empty((M, I), np.float32)
        out = np.empty((M, Nout), np.float32)
        run = lib.rk_npu_w4a8_run_ffn_f32
        P = capi.ptr
        assert run(gws.h, gw.h, gws.h, dw.h, P(x), P(mid), P(out), None) == capi.RK_NPU_ERR_PARAM  # same ws
        assert run(gws.h, gw.h, dws.h, dw.h, P(x), P(mid), P(mid), None) == capi.RK_NPU_ERR_PARAM  # middle == C
        assert run(gws.h, gw.h, dws.h, dw.h, P(x), P(mid), P(x), None) == capi.RK_NPU_ERR_PARAM    # A == C
        assert run(gws.h, gw.h, dws_m.h, dw.h, P(x), P(mid), P(out), None) == capi.RK_NPU_ERR_PARAM  # M differs
        assert run(gws.h, dw.h, dws.h, dw.h, P(x), P(mid), P(out), None) == capi.RK_NPU_ERR_PARAM  # wrong weights
        xb = x.copy()
        xb[0, 0] = np.nan
        assert run(gws.h, gw.h, dws.h, dw.h, P(xb), P(mid), P(out), None) == capi.RK_NPU_ERR_PARAM
        assert run(gws.h, gw.h, dws.h, dw.h, P(x), P(mid), P(out), None) == 0
        # huge gate/up scales overflow the middle to +-Inf: rejected before Down writes C
        big = ops.W4A8Weights(sess, B_gu, np.full(2 * I, 1e30, np.float32))
        out[:] = 7.0
        assert run(gws.h, big.h, dws.h, dw.h, P(x * 1e6), P(mid), P(out), None) == capi.RK_NPU_ERR_PARAM
        assert (out == 7.0).all()
        big.close()
    finally:
        for o in (gws, dws, dws_m, gw, dw):
            o.close()


def test_weight_info_and_k_tile_resolution(sess):
    """k_tile = 0 picks the largest partition whose INT16 bound certifies
    (reference src/rk_npu_i4_bounds.cpp); explicit k_tile > 480 must certify."""
    K, N = 2048, 64
    small = np.ones((K, N), np.int8)            # P = 7*K, Q = 8*K: certified up to k with 8k <= 32768 -> 2048? 8*2048=16384 ok
    w = ops.W4A8Weights(sess, small, np.ones(N, np.float32), k_tile=0)
    assert w.info.config.k_tile == 2048 and w.info.safe_k_tile == 2048 and w.info.bound_relaxed == 0
    assert w.info.multiplier == 1.0
    w.close()
    heavy = np.full((K, N), -8, np.int8)        # P = 64 per k: tile t certifies iff 64*t <= 32767 -> t <= 511 -> 480
    w = ops.W4A8Weights(sess, heavy, np.ones(N, np.float32), k_tile=0)
    assert w.info.config.k_tile == 480 and w.info.safe_k_tile == 480
    w.close()
    cfg = capi.I4WeightConfig(K, N, 512)
    s = np.ones(N, np.float32)
    assert not sess.lib.rk_npu_w4a8_weights_create(sess.domain, C.byref(cfg), capi.ptr(heavy), capi.ptr(s))
    h = sess.lib.rk_npu_w4a8_weights_create(sess.domain, C.byref(cfg), capi.ptr(small), capi.ptr(s))
    assert h
    sess.lib.rk_npu_w4a8_weights_free(h)


def test_config2_full_output_and_properties(sess, oracle):
    """BASELINE config 2 at full size (M=2048, K=4096, N=4096, seeds 4/5, 0.5% x20
    outliers): every int8 activation, every fp16 output and every int32
    accumulator exact against the oracle (all 2048 rows), plus a size-independent
    property on the whole output: scaling a token by a power of two scales its
    output row exactly (until fp16 range limits), because the quantized codes are
    unchanged."""
    c = workloads.CONFIGS[2]()
    M, K, N = c["M"], c["K"], c["N"]
    w = ops.W4A8Weights(sess, c["B"], c["w_scale"])
    wsp = ops.W4A8Workspace(sess, M, N, K)
    try:
        rc, got = wsp.run_f16(w, c["A"])
        assert rc == 0
        q, s = wsp.read_quantized()
        want = oracle.w4a8(c["A"], c["B"], c["w_scale"])
        assert want["rc"] == 0 and np.array_equal(_bits32(s), _bits32(want["a_scale"]))
        assert np.array_equal(q, want["q"])
        assert np.array_equal(got, want["C"])
        # int32 accumulators of the whole problem through the probe entry point (same kernels,
        # raw integer epilogue)
        rc, acc = wsp.run_i32(w, oracle.half_to_float(c["A"]))
        assert rc == 0 and np.array_equal(acc, want["acc"])
        half = (oracle.half_to_float(c["A"]) * np.float32(0.5)).astype(np.float16).view(np.uint16)
        rc, got_half = wsp.run_f16(w, half)
        assert rc == 0
        f, fh = oracle.half_to_float(got), oracle.half_to_float(got_half)
        normal = np.abs(f) > 2.0 ** -13   # halves of fp16 normals stay exactly representable
        assert np.array_equal(fh[normal] * 2, f[normal])
    finally:
        wsp.close()
        w.close()


def test_config3_ffn_full(sess, oracle):
    """BASELINE config 3: M=128, hidden 4096, intermediate 14336, seeds 6-9."""
    c = workloads.CONFIGS[3]()
    M, H, I = c["M"], c["H"], c["I"]
    gw, dw = ops.W4A8Weights(sess, c["B_gu"], c["s_gu"]), ops.W4A8Weights(sess, c["B_down"], c["s_down"])
    gws, dws = ops.W4A8Workspace(sess, M, 2 * I, H), ops.W4A8Workspace(sess, M, H, I)
    try:
        rc, mid, out = ops.w4a8_ffn(sess, gws, gw, dws, dw, c["x"])
        assert rc == 0
        want = oracle.w4a8_ffn(c["x"], c["B_gu"], c["s_gu"], c["B_down"], c["s_down"], oracle.EXP_POLY)
        assert np.array_equal(_bits32(mid), _bits32(want["middle"]))
        qd, sd = dws.read_quantized()
        assert np.array_equal(qd, want["q_down"]) and np.array_equal(_bits32(sd), _bits32(want["down_scale"]))
        assert np.array_equal(_bits32(out), _bits32(want["C"]))
        rc, acc = dws.run_i32(dw, mid)
        assert rc == 0 and np.array_equal(acc, want["acc_down"])
        out16 = oracle.float_to_half(out)
        ref16 = oracle.half_to_float(oracle.float_to_half(want["C"]))
        assert np.abs(oracle.half_to_float(out16) - ref16).max() <= 1e-3 * np.abs(ref16).max()
    finally:
        for o in (gws, dws, gw, dw):
            o.close()


def test_k_tile_resolution_against_reference_golden(sess):
    """tests/golden/i4_bounds.json holds what the reference's bound_i4_weights
    answers for seeded code matrices (written by tests/golden/make_golden.py from
    the compiled reference); weights_create must resolve the same tiles."""
    import json
    import os
    from tests.golden.make_golden import i4_matrix
    with open(os.path.join(os.path.dirname(__file__), "golden", "i4_bounds.json")) as f:
        cases = json.load(f)
    for case in cases:
        B = i4_matrix(**case["recipe"])
        K, N = B.shape
        scale = np.ones(N, np.float32)
        if case["auto_k_tile"] > 0:
            w = ops.W4A8Weights(sess, B, scale, k_tile=0)
            assert w.info.safe_k_tile == case["auto_k_tile"], case["recipe"]
            assert w.info.config.k_tile == min(case["auto_k_tile"], 2048, (K + 31) // 32 * 32)
            w.close()
        for tile, ok in case["explicit"].items():
            cfg = capi.I4WeightConfig(K, N, int(tile))
            h = sess.lib.rk_npu_w4a8_weights_create(sess.domain, C.byref(cfg), capi.ptr(B), capi.ptr(scale))
            assert bool(h) == bool(ok), (case["recipe"], tile)
            if h:
                sess.lib.rk_npu_w4a8_weights_free(h)


def test_random_shapes_through_the_launch_plan(sess, oracle):
    """Seeded random shapes of more than 128 rows: whatever tile height and K split the dense plan
    picks (long K with few columns is split over workgroups, wide matrices are not), the int32 sums
    and the fp32 output are the oracle's, for int4 weights here and int8 weights below."""
    rng = np.random.default_rng(424242)
    for case in range(20):
        M = int(rng.integers(129, 900))
        N = int(rng.choice([rng.integers(1, 300), rng.integers(300, 2500)]))
        K = int(rng.choice([rng.integers(1, 300), rng.integers(300, 3000), rng.integers(3000, 14000)]))
        B = _codes(rng, (K, N))
        ws = (rng.random(N).astype(np.float32) + 0.5) * 0.01
        A = rng.standard_normal((M, K)).astype(np.float32)
        w = ops.W4A8Weights(sess, B, ws)
        wsp = ops.W4A8Workspace(sess, M, N, K)
        try:
            want = oracle.w4a8(A, B, ws)
            rc, acc = wsp.run_i32(w, A)
            assert rc == 0 and np.array_equal(acc, want["acc"]), (case, M, N, K)
            rc, got = wsp.run_f32(w, A)
            assert rc == 0 and np.array_equal(_bits32(got), _bits32(want["C"])), (case, M, N, K)
        finally:
            wsp.close()
            w.close()
    for case in range(20):
        M = int(rng.integers(129, 900))
        N = int(rng.choice([rng.integers(1, 300), rng.integers(300, 2500)]))
        K = int(rng.choice([rng.integers(1, 300), rng.integers(300, 3000), rng.integers(3000, 14000)]))
        B = rng.integers(-127, 128, (K, N)).astype(np.int8)
        ws = (rng.random(N).astype(np.float32) + 0.5) * 0.01
        A = rng.standard_normal((M, K)).astype(np.float32)
        op = ops.W8A8Linear(sess, capi.F32I8F32_DYNAMIC, M, B, ws)
        try:
            rc, got = op.run(A)
            want = oracle.w8a8(A, B, ws)["C"]
            assert rc == 0 and np.array_equal(_bits32(got), _bits32(want)), (case, M, N, K)
        finally:
            op.close()
