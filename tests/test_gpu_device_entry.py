"""GPU parity of the device-pointer entry points (include/rk_npu_hip.h) against the CPU oracle.

These calls take operands that already lie in device memory and only enqueue
work, so for decode-sized M they reach the one-launch path in which the GEMV
quantizes its rows itself -- a path the host-pointer calls never take (they
quantize from the pinned mirror with a kernel of its own).  Same bar as the
host-pointer tests: quantized codes, scales and outputs bit-exact.
"""
import numpy as np
import pytest

from rknpu2_matmul_open_amd import capi, ops, workloads

pytestmark = pytest.mark.gpu


def _bits32(x):
    return np.ascontiguousarray(x, np.float32).view(np.uint32)


def _special_rows(A, as_f16):
    """A zero row (scale 1) and a row of exact ties at scale 1 where the row count allows."""
    M, K = A.shape
    if M > 2:
        A[1, :] = 0
        ties = np.array([127, -127, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5], np.float32)[: min(K, 8)]
        A[2, :] = 0
        A[2, : len(ties)] = ties.astype(np.float16).view(np.uint16) if as_f16 else ties
    return A


# M <= 8 with rows that fit the fused GEMV (one launch), every column width of the kernel
# (<= 64 / 65..256 / > 256 column blocks), ragged N and K; the last ones do not fit the fused
# path (rows too long) or have more than 8 rows and take the two-kernel route.  (1, 14336, 4096)
# is the decode shape the benchmark times and (1, 9000, 4100) a ragged neighbour: more than 256
# column blocks AND several groups of loads per wave, the loop the short-K wide cases never enter.
W8_SHAPES = [(1, 64, 64), (1, 200, 200), (1, 513, 1000), (1, 4096, 4096), (1, 2100, 8200), (1, 9000, 520),
             (1, 14336, 4096), (1, 9000, 4100), (2, 14336, 4096),
             (2, 3000, 700), (3, 65, 33), (4, 9000, 300), (4, 4100, 8000), (8, 128, 4096), (8, 8300, 2000),
             (7, 5000, 4100), (2, 2500, 20003), (16, 300, 500),
             (2, 1000, 300), (7, 4100, 300),   # two rows, 8 columns per workgroup; five to eight rows, 16 columns
             # five to eight rows beyond 128 column blocks: whole blocks per workgroup; rows in chunks behind a
             # quantization launch there
             (5, 5120, 300), (8, 5100, 4100), (6, 5088, 1000), (8, 5120, 8300),
             # up to 128 blocks: 16 columns per workgroup for any number of rows (small / large staging area)
             (6, 3000, 300), (8, 4000, 5000), (4, 4000, 300)]


@pytest.mark.parametrize("M,N,K", W8_SHAPES)
@pytest.mark.parametrize("f16", [True, False])
def test_w8a8_dynamic_device(sess, oracle, M, N, K, f16):
    c = workloads.w8a8_case(M, K, N, seed_w=M + N + 1, seed_a=K + 11)
    if f16:
        A = _special_rows(c["A"].copy(), True)
        kind, out_dtype = capi.F16I8F16_DYNAMIC, np.uint16
    else:
        A = _special_rows(oracle.half_to_float(c["A"]).astype(np.float32).reshape(M, K) * 3.0, False)
        kind, out_dtype = capi.F32I8F32_DYNAMIC, np.float32
    op = ops.W8A8Linear(sess, kind, M, c["B"], c["w_scale"])
    dA = sess.to_device(A)
    dC = sess.empty_device(M * N * np.dtype(out_dtype).itemsize)
    try:
        for _ in range(2):  # a second call on the same workspace must give the same answer
            assert op.run_device(dA, dC) == 0
            assert sess.sync() == 0
            got = sess.from_device(dC, (M, N), out_dtype)
            want = oracle.w8a8(A, c["B"], c["w_scale"])
            q, s = op.read_quantized()
            assert np.array_equal(_bits32(s), _bits32(want["a_scale"]))
            assert np.array_equal(q, want["q"])
            if f16:
                assert np.array_equal(got, want["C"])
            else:
                assert np.array_equal(_bits32(got), _bits32(want["C"]))
    finally:
        sess.free_device(dA)
        sess.free_device(dC)
        op.close()


W4_SHAPES = [(1, 64, 64), (1, 65, 33), (1, 4096, 4096), (1, 2100, 8200), (1, 9000, 520), (2, 65, 20003),
             (1, 14336, 4096), (1, 9000, 4100),
             (3, 2500, 1000), (4, 9000, 300), (8, 128, 512), (8, 8200, 2000), (5, 4100, 5000), (12, 200, 300),
             # two rows at every column width of the kernel; four rows, 8 columns; six rows, 16 columns
             (2, 4096, 512), (2, 9000, 300), (2, 1000, 200), (4, 1000, 300), (6, 4100, 300),
             # three to seven rows on a wide matrix whose rows fit the staging area eight at a time: the
             # eight-row kernel with matrix-core products (ragged K, a full 4096); K beyond that: the streaming
             # kernel from three rows on, two rows on the dot products
             (3, 8200, 1000), (5, 9000, 4096), (7, 8224, 300), (6, 14336, 4096), (4, 8200, 4100), (3, 8300, 4100),
             (2, 8300, 4100),
             # a narrower matrix: eight rows that fit the staging area stay on the decode kernel, five to eight
             # longer ones go to the streaming kernel; three and four rows stay up to K = 16384 (in chunks
             # beyond 8192)
             (4, 2000, 8192), (3, 4100, 8300), (4, 2000, 4100), (5, 2000, 4100), (8, 2000, 4096), (3, 2000, 16500),
             # 129 .. 256 column blocks: whole blocks per workgroup, the eight-row kernel from three rows on
             (2, 5120, 4096), (3, 8192, 1000), (4, 6000, 300), (8, 5130, 4096), (2, 5100, 4100),
             # up to 128 blocks: 16 columns per workgroup for any number of rows
             (6, 4000, 1000), (8, 3000, 300), (2, 4000, 300),
             # two rows that do not fit it (K > 16384): the streaming kernel beyond 4096 columns
             (2, 4200, 16500), (2, 2000, 16500)]


@pytest.mark.parametrize("M,N,K", W4_SHAPES)
def test_w4a8_device(sess, oracle, M, N, K):
    rng = np.random.default_rng(M * 7919 + N * 31 + K + 5)
    B = rng.integers(-8, 8, (K, N)).astype(np.int8)
    ws = (rng.random(N).astype(np.float32) + 0.5) * 0.02
    A = _special_rows((rng.standard_normal((M, K)) * 2).astype(np.float32), False)
    A16 = A.astype(np.float16).view(np.uint16)
    lib = sess.lib
    w = ops.W4A8Weights(sess, B, ws)
    wsp = ops.W4A8Workspace(sess, M, N, K)
    dA, dA16 = sess.to_device(A), sess.to_device(A16)
    dC, dC16 = sess.empty_device(M * N * 4), sess.empty_device(M * N * 2)
    try:
        want = oracle.w4a8(A, B, ws)
        assert lib.rk_npu_w4a8_run_f32_device(wsp.h, w.h, dA, dC) == 0
        assert sess.sync() == 0
        q, s = wsp.read_quantized()
        assert np.array_equal(_bits32(s), _bits32(want["a_scale"]))
        assert np.array_equal(q, want["q"])
        assert np.array_equal(_bits32(sess.from_device(dC, (M, N), np.float32)), _bits32(want["C"]))
        want16 = oracle.w4a8(A16, B, ws)
        assert lib.rk_npu_w4a8_run_f16_device(wsp.h, w.h, dA16, dC16) == 0
        assert sess.sync() == 0
        assert np.array_equal(sess.from_device(dC16, (M, N), np.uint16), want16["C"])
    finally:
        for d in (dA, dA16, dC, dC16):
            sess.free_device(d)
        wsp.close()
        w.close()


def test_w4a8_device_rejects_nonfinite_rows(sess):
    """NaN / Inf in a row: the enqueue succeeds, the next sync reports RK_NPU_ERR_PARAM."""
    M, N, K = 2, 96, 200
    rng = np.random.default_rng(3)
    B = rng.integers(-8, 8, (K, N)).astype(np.int8)
    ws = np.full(N, 0.01, np.float32)
    w = ops.W4A8Weights(sess, B, ws)
    wsp = ops.W4A8Workspace(sess, M, N, K)
    A = rng.standard_normal((M, K)).astype(np.float32)
    A[1, 17] = np.inf
    dA, dC = sess.to_device(A), sess.empty_device(M * N * 4)
    try:
        assert sess.lib.rk_npu_w4a8_run_f32_device(wsp.h, w.h, dA, dC) == 0
        assert sess.sync() == capi.RK_NPU_ERR_PARAM
        # the context is usable again afterwards
        A[1, 17] = 1.0
        sess.free_device(dA)
        dA = sess.to_device(A)
        assert sess.lib.rk_npu_w4a8_run_f32_device(wsp.h, w.h, dA, dC) == 0
        assert sess.sync() == 0
    finally:
        sess.free_device(dA)
        sess.free_device(dC)
        wsp.close()
        w.close()


# one / two rows: gate/up + SwiGLU as a GEMV that quantizes its rows itself, and a down GEMV that
# re-quantizes the middle itself; more rows: the MFMA kernels with kernels of their own for both
FFN_SHAPES = [(1, 64, 64, 64), (1, 1000, 4160, 300), (2, 256, 2048, 300), (2, 20003, 96, 65),
              (3, 256, 2048, 300), (4, 1000, 4160, 300), (4, 4096, 1056, 40), (3, 9000, 96, 65),  # three / four rows: the SwiGLU GEMV as well (rows of 9000: behind a quantization launch)
              (5, 128, 96, 65), (8, 512, 1024, 4100), (33, 256, 160, 128)]


@pytest.mark.parametrize("M,H,I,Nout", FFN_SHAPES)
def test_w4a8_ffn_device(sess, oracle, M, H, I, Nout):
    rng = np.random.default_rng(M + H + I + 17)
    B_gu = rng.integers(-7, 8, (H, 2 * I)).astype(np.int8)
    s_gu = (rng.random(2 * I).astype(np.float32) + 0.5) * 0.01
    B_dn = rng.integers(-7, 8, (I, Nout)).astype(np.int8)
    s_dn = (rng.random(Nout).astype(np.float32) + 0.5) * 0.01
    x = rng.standard_normal((M, H)).astype(np.float32)
    if M > 2:
        x[1] = 0.0  # zero token -> zero middle row -> Down scale 1
    gw, dw = ops.W4A8Weights(sess, B_gu, s_gu), ops.W4A8Weights(sess, B_dn, s_dn)
    gws, dws = ops.W4A8Workspace(sess, M, 2 * I, H), ops.W4A8Workspace(sess, M, Nout, I)
    dA = sess.to_device(x)
    dmid, dC = sess.empty_device(M * I * 4), sess.empty_device(M * Nout * 4)
    try:
        want = oracle.w4a8_ffn(x, B_gu, s_gu, B_dn, s_dn, oracle.EXP_POLY)
        assert want["rc"] == 0
        for _ in range(2):
            assert sess.lib.rk_npu_w4a8_run_ffn_f32_device(gws.h, gw.h, dws.h, dw.h, dA, dmid, dC) == 0
            assert sess.sync() == 0
            assert np.array_equal(_bits32(sess.from_device(dmid, (M, I), np.float32)), _bits32(want["middle"]))
            qd, sd = dws.read_quantized()
            assert np.array_equal(_bits32(sd), _bits32(want["down_scale"]))
            assert np.array_equal(qd, want["q_down"])
            assert np.array_equal(_bits32(sess.from_device(dC, (M, Nout), np.float32)), _bits32(want["C"]))
    finally:
        for d in (dA, dmid, dC):
            sess.free_device(d)
        for o in (gws, dws, gw, dw):
            o.close()


def test_w4a8_ffn_device_nonfinite_middle_is_rejected(sess):
    """A middle that overflows to Inf (huge scales) must surface as RK_NPU_ERR_PARAM at the next
    sync, also when the down GEMV scans the middle itself (one row)."""
    M, H, I, Nout = 1, 64, 64, 64
    B_gu = np.full((H, 2 * I), 7, np.int8)
    s_gu = np.full(2 * I, 1e18, np.float32)
    B_dn = np.ones((I, Nout), np.int8)
    s_dn = np.ones(Nout, np.float32)
    x = np.full((M, H), 1e18, np.float32)
    gw, dw = ops.W4A8Weights(sess, B_gu, s_gu), ops.W4A8Weights(sess, B_dn, s_dn)
    gws, dws = ops.W4A8Workspace(sess, M, 2 * I, H), ops.W4A8Workspace(sess, M, Nout, I)
    dA = sess.to_device(x)
    dmid, dC = sess.empty_device(M * I * 4), sess.empty_device(M * Nout * 4)
    try:
        assert sess.lib.rk_npu_w4a8_run_ffn_f32_device(gws.h, gw.h, dws.h, dw.h, dA, dmid, dC) == 0
        assert sess.sync() == capi.RK_NPU_ERR_PARAM
        mid = sess.from_device(dmid, (M, I), np.float32)
        assert not np.isfinite(mid).all()
    finally:
        for d in (dA, dmid, dC):
            sess.free_device(d)
        for o in (gws, dws, gw, dw):
            o.close()


# ---- device pointers that are only element-aligned -------------------------------------------
# The device entry points take any pointer into device memory.  Rows that do not start on a
# 16-byte boundary take the element-wise loaders and outputs the element-wise stores; nothing
# in the interface asks for more than the element's own alignment.

def _offset_copy(sess, array, elems):
    """Device copy of `array` that starts `elems` elements into an allocation -> (base, pointer)."""
    a = np.ascontiguousarray(array)
    base = sess.empty_device(a.nbytes + 64)
    p = base + elems * a.itemsize
    assert sess.lib.rk_npu_hip_upload(sess.ctx, p, capi.ptr(a), a.nbytes) == 0
    return base, p


# int8 rows as given (the exact int8 x int8 product, the call the reference's bench_llm_i8 times):
# for M <= 8 the GEMV stages the caller's row-major rows itself, one launch.  Every column width
# (<= 64 / 65..256 / > 256 column blocks), ragged K (tail chunk, rows that start off a 16-byte
# boundary because K is odd), K beyond one staging chunk (32768 / rows), wide matrices with
# several groups of loads per wave, 5..8 rows; (16, 300, 500) and (130, 520, 777) take the two-kernel route.
I8_SHAPES = [(1, 64, 64), (1, 200, 203), (1, 513, 1000), (1, 4096, 4096), (1, 2100, 8200), (1, 9000, 520),
             (1, 11008, 4096), (1, 9000, 4100), (1, 300, 40001), (2, 14336, 4096), (2, 3000, 700), (3, 65, 33),
             (4, 9000, 301), (4, 4100, 9001), (8, 128, 4096), (8, 8300, 2000), (7, 5000, 4100), (2, 2500, 20003),
             (1, 14336, 4096), (4, 14336, 600), (8, 14336, 300), (2, 100, 300),  # whole blocks (one row: the burst variant); two rows, 8 columns
             (16, 300, 500), (130, 520, 777),
             # several rows: 32 columns per workgroup on 129 .. 256 blocks while K <= 5120 (16 beyond), 16 on up to 64 blocks
             (2, 5120, 4096), (8, 4200, 5120), (4, 5000, 5400), (3, 8192, 300), (4, 2048, 8200), (2, 1000, 4100), (2, 2048, 5400),
             (8, 520, 300), (5, 4096, 4096),
             # 9..128 rows on the streaming kernel behind the re-tiling launch (K split over the waves / not; a K
             # of one and of three k-tiles; ragged last row block)
             (16, 300, 512), (33, 4100, 4096), (128, 11008, 4096), (100, 64, 32), (9, 8448, 96), (64, 520, 2080),
             (97, 9000, 288), (128, 4096, 11008)]


@pytest.mark.parametrize("M,N,K", I8_SHAPES)
@pytest.mark.parametrize("offset", [0, 1])
def test_i8i8i32_device(sess, oracle, M, N, K, offset):
    rng = np.random.default_rng(M * 7 + N + K + offset)
    A = rng.integers(-128, 128, (M, K)).astype(np.int8)
    B = rng.integers(-128, 128, (K, N)).astype(np.int8)
    A[0, : min(K, 40)] = -128
    B[: min(K, 40), 0] = -128
    op = ops.W8A8Linear(sess, capi.I8I8I32, M, B)
    baseA, dA = _offset_copy(sess, A, offset)      # offset 1: rows only byte-aligned
    baseC = sess.empty_device(M * N * 4 + 64)
    dC = baseC + 4 * offset
    try:
        want = oracle.gemm_i8(A, B)
        for _ in range(2):
            assert op.run_device(dA, dC) == 0
            assert sess.sync() == 0
            assert np.array_equal(sess.from_device(dC, (M, N), np.int32), want)
        # the workspace holds the rows as a two-kernel run would have left them
        q = np.empty((M, K), np.int8)
        s = np.empty(M, np.float32)
        assert sess.lib.rk_npu_matmul_workspace_read_quantized(op.ws, capi.ptr(q), capi.ptr(s)) == 0
        assert np.array_equal(q, A)
        # ... so the GEMM can be run again on them
        assert sess.lib.rk_npu_hip_upload(sess.ctx, dC, capi.ptr(np.zeros((M, N), np.int32)), M * N * 4) == 0
        assert sess.lib.rk_npu_matmul_workspace_rerun_gemm_device(op.ws, op.w, dC) == 0
        assert sess.sync() == 0
        assert np.array_equal(sess.from_device(dC, (M, N), np.int32), want)
    finally:
        sess.free_device(baseA)
        sess.free_device(baseC)
        op.close()


@pytest.mark.parametrize("M,N,K", [(1, 9000, 520), (1, 2100, 1000), (4, 300, 200), (40, 300, 260), (300, 520, 200)])
@pytest.mark.parametrize("f16", [True, False])
def test_w8a8_device_pointers_with_element_alignment_only(sess, oracle, M, N, K, f16):
    c = workloads.w8a8_case(M, K, N, seed_w=M + N + 2, seed_a=K + 13)
    if f16:
        A, kind, out_dtype = c["A"], capi.F16I8F16_DYNAMIC, np.uint16
    else:
        A = oracle.half_to_float(c["A"]).astype(np.float32).reshape(M, K) * 2.0
        kind, out_dtype = capi.F32I8F32_DYNAMIC, np.float32
    size = np.dtype(out_dtype).itemsize
    op = ops.W8A8Linear(sess, kind, M, c["B"], c["w_scale"])
    baseA, dA = _offset_copy(sess, A, 1)
    baseC = sess.empty_device(M * N * size + 64)
    dC = baseC + 3 * size
    try:
        assert op.run_device(dA, dC) == 0
        assert sess.sync() == 0
        got = sess.from_device(dC, (M, N), out_dtype)
        want = oracle.w8a8(A, c["B"], c["w_scale"])["C"]
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    finally:
        sess.free_device(baseA)
        sess.free_device(baseC)
        op.close()


@pytest.mark.parametrize("M,N,K", [(1, 9000, 520), (2, 300, 200), (40, 300, 260), (300, 520, 200)])
def test_w4a8_device_pointers_with_element_alignment_only(sess, oracle, M, N, K):
    rng = np.random.default_rng(M + N + K)
    B = rng.integers(-8, 8, (K, N)).astype(np.int8)
    ws = (rng.random(N).astype(np.float32) + 0.5) * 0.02
    A = (rng.standard_normal((M, K)) * 2).astype(np.float32)
    A16 = A.astype(np.float16).view(np.uint16)
    w = ops.W4A8Weights(sess, B, ws)
    wsp = ops.W4A8Workspace(sess, M, N, K)
    baseA, dA = _offset_copy(sess, A, 1)
    baseA16, dA16 = _offset_copy(sess, A16, 3)
    baseC, baseC16 = sess.empty_device(M * N * 4 + 64), sess.empty_device(M * N * 2 + 64)
    dC, dC16 = baseC + 4, baseC16 + 2
    try:
        assert sess.lib.rk_npu_w4a8_run_f32_device(wsp.h, w.h, dA, dC) == 0
        assert sess.lib.rk_npu_w4a8_run_f16_device(wsp.h, w.h, dA16, dC16) == 0
        assert sess.sync() == 0
        assert np.array_equal(_bits32(sess.from_device(dC, (M, N), np.float32)), _bits32(oracle.w4a8(A, B, ws)["C"]))
        assert np.array_equal(sess.from_device(dC16, (M, N), np.uint16), oracle.w4a8(A16, B, ws)["C"])
    finally:
        for d in (baseA, baseA16, baseC, baseC16):
            sess.free_device(d)
        wsp.close()
        w.close()


@pytest.mark.parametrize("T", [3, 70])
def test_moe_device_pointers_with_element_alignment_only(sess, oracle, T):
    H, E, top_k, I = 128, 6, 2, 64
    c = workloads.moe_case(T, H, E, top_k, I)
    moe = ops.MoeW8(sess, H, I, E, 0, top_k, 128, c["experts"])
    x = np.ascontiguousarray(c["x"], np.float32)
    ids, routes = np.ascontiguousarray(c["ids"], np.int32), np.ascontiguousarray(c["routes"], np.float32)
    bx, dx = _offset_copy(sess, x, 1)
    bi, dids = _offset_copy(sess, ids, 1)
    br, drt = _offset_copy(sess, routes, 3)
    bo = sess.empty_device(T * H * 4 + 64)
    dout = bo + 4
    try:
        assert sess.lib.rk_npu_moe_w8_run_f32_device(moe.ws, moe.w, T, dx, dids, drt, dout) == 0
        assert sess.sync() == 0
        rc, want = oracle.moe_w8(c["experts"], H, I, E, 0, top_k, ids, routes, input_f32=x)
        got = sess.from_device(dout, (T, H), np.float32)
        assert rc == 0 and np.array_equal(got.view(np.uint32), want.view(np.uint32))
    finally:
        for d in (bx, bi, br, bo):
            sess.free_device(d)
        moe.close()


def test_i8i8i32_device_random_shapes(sess, oracle):
    """Seeded random shapes through every route of the exact int8 x int8 product: one to eight rows
    (dot products, rows staged by the kernel), up to 128 rows (streaming kernel), more (large tiles,
    with whatever tile height and K split the plan picks)."""
    rng = np.random.default_rng(987654)
    for case in range(36):
        M = int(rng.choice([rng.integers(1, 9), rng.integers(9, 129), rng.integers(129, 700)]))
        N = int(rng.choice([rng.integers(1, 300), rng.integers(300, 3000), rng.integers(3000, 12000)]))
        K = int(rng.choice([rng.integers(1, 200), rng.integers(200, 3000), rng.integers(3000, 12000)]))
        A = rng.integers(-128, 128, (M, K)).astype(np.int8)
        B = rng.integers(-128, 128, (K, N)).astype(np.int8)
        op = ops.W8A8Linear(sess, capi.I8I8I32, M, B)
        offset = case % 2
        baseA, dA = _offset_copy(sess, A, offset)
        dC = sess.empty_device(M * N * 4)
        try:
            assert op.run_device(dA, dC) == 0, (case, M, N, K)
            assert sess.sync() == 0, (case, M, N, K)
            got = sess.from_device(dC, (M, N), np.int32)
            assert np.array_equal(got, oracle.gemm_i8(A, B)), (case, M, N, K)
        finally:
            sess.free_device(baseA)
            sess.free_device(dC)
            op.close()


# The decode dispatch changes kernel at these sizes: 256 / 257 column blocks (16- / 32-column workgroups),
# rows of 4096 / 4097+ elements (eight rows fit the staging area of the wide int4 matrices or not; one
# K chunk or two), three rows (the eight-row kernel on wide int4 matrices) and seven / eight rows (the
# decode kernel's limit there).  Both weight formats through the device entries, fp16 rows.
BOUNDARY_SHAPES = [(M, N, K) for M in (2, 3, 7, 8) for N in (8192, 8224) for K in (4096, 4100)] + \
                  [(1, 8224, 4096), (4, 8193, 4095), (5, 8224, 8200), (6, 8160, 4097)] + \
                  [(M, N, 4096) for M in (1, 2, 3, 5) for N in (4096, 4128)] + \
                  [(M, 5120, K) for M in (1, 2, 4) for K in (5120, 5400)] + \
                  [(M, 2048, K) for M in (2, 4, 6) for K in (5120, 5400)] + [(2, 2080, 4096), (5, 520, 300)]
# (128 / 129 column blocks: 16- / 32-column workgroups for several rows; K up to 5120 / beyond: for a few rows too;
# 64 / 65 blocks: 8 / 16 columns for one row, 16 for several)


@pytest.mark.parametrize("M,N,K", BOUNDARY_SHAPES)
def test_decode_dispatch_boundaries(sess, oracle, M, N, K):
    rng = np.random.default_rng(M * 131 + N + K)
    lib = sess.lib
    c = workloads.w8a8_case(M, K, N, seed_w=N + K, seed_a=M + 11)
    B4 = rng.integers(-8, 8, (K, N)).astype(np.int8)
    s4 = (rng.random(N).astype(np.float32) + 0.5) * np.float32(0.02)
    A16 = c["A"]
    op = ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, M, c["B"], c["w_scale"])
    w = ops.W4A8Weights(sess, B4, s4)
    wsp = ops.W4A8Workspace(sess, M, N, K)
    dA, dC = sess.to_device(A16), sess.empty_device(M * N * 2)
    try:
        assert op.run_device(dA, dC) == 0 and sess.sync() == 0
        assert np.array_equal(sess.from_device(dC, (M, N), np.uint16), oracle.w8a8(A16, c["B"], c["w_scale"])["C"])
        assert lib.rk_npu_w4a8_run_f16_device(wsp.h, w.h, dA, dC) == 0 and sess.sync() == 0
        assert np.array_equal(sess.from_device(dC, (M, N), np.uint16), oracle.w4a8(A16, B4, s4)["C"])
    finally:
        sess.free_device(dA)
        sess.free_device(dC)
        wsp.close()
        w.close()
        op.close()
