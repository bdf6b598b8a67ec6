"""GPU parity of the W8A8 operators against the CPU oracle, through the C ABI.

Bars: int8 activations, per-row scales and int32 accumulators bit-exact;
fp16 / fp32 outputs bit-exact as well (the epilogue is two IEEE multiplies and
one RNE cast, which the oracle states identically), which is stricter than the
1e-3 x absmax tolerance the benchmark configuration allows.
"""
import numpy as np
import pytest

from rknpu2_matmul_open_amd import capi, ops, workloads

pytestmark = pytest.mark.gpu


def _rand_i8(rng, shape, lo=-127, hi=127):
    return rng.integers(lo, hi + 1, shape).astype(np.int8)


# reference examples/demo.cpp:58-62 runs odd shapes such as 17x40x33, 300x48x33, 1x200x200
I32_SHAPES = [(1, 32, 32), (1, 200, 200), (3, 65, 33), (8, 64, 96), (9, 64, 96), (17, 40, 33),
              (33, 130, 70), (64, 256, 256), (65, 257, 129), (128, 512, 384), (300, 48, 33),
              (200, 1000, 520),
              # degenerate and lopsided: single k / column / row, far more rows than anything else,
              # a very wide matrix for one row, for a row block and for many rows
              (1, 1, 1), (5000, 3, 1), (2, 1, 5000), (4100, 40, 70), (1, 70001, 64), (9, 70001, 40), (300, 40000, 33),
              # 64-row tiles of the large-tile kernel (too few 128-row tiles); K split over workgroups + reduce launch
              (330, 6600, 200), (150, 96, 8300),
              # tiles of 128 x 128 with one column block per wave (160 .. 256 of them, more 64-row tiles than that)
              (300, 8448, 200), (257, 8200, 300), (640, 4200, 96),
              # weight-streaming kernel (9 .. 128 rows) without / with the in-workgroup K split; 129 .. 256 rows on a
              # narrow matrix with it (a longer K there: the 64-row tiles above)
              (100, 8448, 160), (128, 96, 3000), (200, 2048, 96), (250, 4000, 200), (130, 96, 4100),
              (400, 1000, 96),  # up to 512 rows on a matrix of up to 1024 columns
              (300, 1, 40), (500, 2, 8000), (129, 33, 1),  # the same, degenerate: one / two columns, a single k
              # 65 .. 128 rows on a very wide matrix: tiles of 64 rows (the case above), the large-tile kernel where
              # even those outnumber the compute units; up to 64 rows stay on the streaming kernel's full-K tiles
              (70, 33000, 64), (40, 33000, 96),
              # >= 160 tiles of 128 x 256: the large-tile kernel (ragged M / N / K, K shorter than its look-ahead)
              (641, 6900, 200), (700, 6900, 1100),
              # decode GEMV: 16 columns per workgroup (65 .. 256 column blocks) / 32 columns (more)
              (1, 2100, 257), (5, 8300, 100)]


@pytest.mark.parametrize("M,N,K", I32_SHAPES)
def test_i8i8i32_exact(sess, oracle, M, N, K):
    rng = np.random.default_rng(M * 1000003 + N * 1009 + K)
    A = _rand_i8(rng, (M, K), -128, 127)
    B = _rand_i8(rng, (K, N), -128, 127)
    op = ops.W8A8Linear(sess, capi.I8I8I32, M, B)
    try:
        rc, got = op.run(A)
        assert rc == 0
        want = oracle.gemm_i8(A, B)
        assert np.array_equal(got, want), "M=%d N=%d K=%d first diff at %s" % (
            M, N, K, np.argwhere(got != want)[:4].tolist())
        rc, again = op.run(A)
        assert rc == 0 and np.array_equal(again, got)
    finally:
        op.close()


def test_i8i8i32_extremes_wrap(sess, oracle):
    # all -128 x -128 over K=131072+64 stays below 2^31; the wrap rule itself is
    # exercised with K large enough that +16384 * K crosses 2^31.
    M, N, K = 2, 64, 131072 + 64
    A = np.full((M, K), -128, np.int8)
    B = np.full((K, N), -128, np.int8)
    op = ops.W8A8Linear(sess, capi.I8I8I32, M, B, k_tile=2048)
    try:
        rc, got = op.run(A)
        assert rc == 0
        want = np.int64(16384) * K
        want = ((want + 2 ** 31) % 2 ** 32) - 2 ** 31
        assert (got == want).all()
    finally:
        op.close()


@pytest.mark.parametrize("M", [1, 9, 64, 200])
def test_i8i8i32_sums_far_beyond_int32_wrap_like_the_exact_product(sess, oracle, M):
    """K = 3 million with extreme columns: the exact sums reach 4.9e10, eleven times the int32
    range, and every kernel family (decode, weight stream, large tile with its K split) has to
    return them modulo 2^32, whatever its order of summation."""
    N, K = 48, 3_000_017
    rng = np.random.default_rng(900 + M)
    B = rng.integers(-128, 128, (K, N)).astype(np.int8)
    B[:, 0] = -128
    B[:, 1] = 127
    A = rng.integers(-128, 128, (M, K)).astype(np.int8)
    A[0] = -128
    op = ops.W8A8Linear(sess, capi.I8I8I32, M, B)
    try:
        rc, got = op.run(A)
        assert rc == 0 and np.array_equal(got, oracle.gemm_i8(A, B))
        # the two constant columns in closed form, independent of the oracle
        row_sums = A.astype(np.int64).sum(axis=1)
        assert -128 * int(row_sums[0]) > 10 * 2 ** 32
        assert np.array_equal(got[:, 0], (row_sums * -128).astype(np.int32))   # (the cast wraps)
        assert np.array_equal(got[:, 1], (row_sums * 127).astype(np.int32))
    finally:
        op.close()


F16_SHAPES = [(1, 64, 64), (1, 513, 1000), (4, 96, 200), (8, 128, 4096), (16, 64, 128),
              (33, 100, 130), (64, 512, 512), (100, 300, 257), (130, 768, 1024),
              (650, 7000, 1100),  # large-tile kernel
              (1, 1, 1), (3000, 2, 3), (1, 70001, 48), (2100, 4100, 130),  # degenerate / lopsided
              # decode GEMV variants: 16 columns per workgroup with the rolling load window (one row),
              # with several rows, with K staged in several chunks; wide matrices with one / several rows
              (1, 4096, 4096), (2, 3000, 700), (8, 4100, 9000), (1, 9000, 520), (4, 9000, 300),
              (2, 9000, 300), (4, 4000, 300),   # two rows on a wide matrix; four rows, 16 columns per workgroup
              (4, 4100, 300), (8, 4000, 5000),  # 129 blocks: whole blocks for four rows; eight rows of 5000 on 16 columns
              # weight-streaming kernel on a wide grid; 128 x 128 tiles with one column block per wave; 64-row
              # tiles of the large-tile kernel; eight rows per quantization workgroup (M >= 4096)
              (100, 8448, 160), (300, 8448, 200), (330, 6600, 200), (4200, 64, 100),
              # full-K tiles of the streaming kernel (up to 64 rows, very wide); 65 .. 128 rows there: large-tile kernel
              (40, 33000, 96), (70, 33000, 64),
              # K split over the waves of 64-column tiles (enough of them that 32-column tiles are not needed)
              (100, 4100, 300),
              # 129 .. 256 rows on a narrow matrix: the streaming kernel
              (250, 1500, 300), (136, 4000, 200), (224, 520, 4100), (500, 520, 300), (260, 3, 3)]


@pytest.mark.parametrize("M,N,K", F16_SHAPES)
def test_f16i8f16_dynamic_bit_exact(sess, oracle, M, N, K):
    c = workloads.w8a8_case(M, K, N, seed_w=M + N, seed_a=K + 7)
    A = c["A"].copy()
    if M > 2:
        A[1, :] = 0                      # all-zero token: scale 1
        A[2, : K // 2] = np.float16(0.5).view(np.uint16)  # many exact .5 multiples -> ties
    op = ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, M, c["B"], c["w_scale"])
    try:
        rc, got = op.run(A)
        assert rc == 0
        want = oracle.w8a8(A, c["B"], c["w_scale"])
        q, s = op.read_quantized()
        assert np.array_equal(s.view(np.uint32), want["a_scale"].view(np.uint32))
        assert np.array_equal(q, want["q"])
        assert np.array_equal(got, want["C"]), "max ulp-ish diff %d" % np.abs(
            got.astype(np.int32) - want["C"].astype(np.int32)).max()
    finally:
        op.close()


# second: many-row quantization path; then 128-row tiles of the large-tile kernel, 128 x 128 tiles with one
# column block per wave, 64-row tiles of the large-tile kernel, K split over workgroups + reduce launch,
# eight rows per quantization workgroup
@pytest.mark.parametrize("M,N,K", [(37, 200, 300), (261, 96, 203), (650, 7000, 300), (300, 8448, 200), (330, 6600, 200),
                                   (261, 96, 3000),
                                   (4200, 64, 100),
                                   # an input / an output of more than 64 MiB: beyond the pinned staging mirrors
                                   (4200, 64, 4100), (4200, 4100, 64)])
def test_f32i8f32_dynamic_and_static(sess, oracle, M, N, K):
    rng = np.random.default_rng(5)
    A = rng.standard_normal((M, K)).astype(np.float32) * 3
    A[0, :8] = [127, -127, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5]
    B = _rand_i8(rng, (K, N))
    ws = (rng.random(N).astype(np.float32) + 0.5) * 0.01
    op = ops.W8A8Linear(sess, capi.F32I8F32_DYNAMIC, M, B, ws)
    try:
        rc, got = op.run(A)
        want = oracle.w8a8(A, B, ws)
        assert rc == 0
        assert np.array_equal(got.view(np.uint32), want["C"].view(np.uint32))
    finally:
        op.close()
    a_scale = (rng.random(M).astype(np.float32) + 0.25) * 0.05
    a_scale[0] = 1.0  # exact ties at .5 multiples with scale 1
    for kind, Ain in ((capi.F32I8F32_STATIC, A), (capi.F16I8F16_STATIC, A.astype(np.float16).view(np.uint16))):
        op = ops.W8A8Linear(sess, kind, M, B, ws)
        try:
            rc, got = op.run(Ain, a_scale)
            want = oracle.w8a8(Ain, B, ws, a_scale_static=a_scale)
            assert rc == 0
            q, _ = op.read_quantized()
            assert np.array_equal(q, want["q"])
            assert np.array_equal(got, want["C"]) if got.dtype == np.uint16 else np.array_equal(
                got.view(np.uint32), want["C"].view(np.uint32))
            bad = a_scale.copy()
            bad[3] = 0
            rc, _ = op.run(Ain, bad)
            assert rc == capi.RK_NPU_ERR_PARAM
            bad[3] = np.inf
            rc, _ = op.run(Ain, bad)
            assert rc == capi.RK_NPU_ERR_PARAM
        finally:
            op.close()


@pytest.mark.parametrize("M,N,K", [(1, 3_000_001, 40), (9, 3_000_001, 40), (70, 1_000_003, 33), (300_001, 300, 33)])
def test_f32i8f32_millions_of_columns_or_rows(sess, oracle, M, N, K):
    """The API puts no upper limit on M and N: grids of ~100 000 column blocks or row blocks,
    outputs of hundreds of MB, element offsets beyond 2^31 bytes."""
    rng = np.random.default_rng(M + N)
    B = rng.integers(-127, 128, (K, N)).astype(np.int8)
    ws = (rng.random(N).astype(np.float32) + 0.5) * 1e-2
    A = rng.standard_normal((M, K)).astype(np.float32)
    op = ops.W8A8Linear(sess, capi.F32I8F32_DYNAMIC, M, B, ws)
    try:
        rc, got = op.run(A)
        want = oracle.w8a8(A, B, ws)["C"]
        assert rc == 0 and np.array_equal(got.view(np.uint32), want.view(np.uint32))
    finally:
        op.close()


@pytest.mark.parametrize("M,N,K,f16", [(1, 300, 600_000, True), (2, 520, 150_000, False), (8, 9000, 40_000, False),
                                       (4, 200, 140_000, True), (3, 64, 100_003, False)])
def test_static_scales_on_rows_beyond_the_pinned_mirror(sess, oracle, M, N, K, f16):
    """Decode-sized calls whose rows exceed 1 MiB are uploaded instead of being read in place from
    the pinned mirror; the caller's scales go through their own mirror."""
    c = workloads.w8a8_case(M, K, N, seed_w=M + N + 5, seed_a=K + 17)
    a_scale = (np.random.default_rng(M + K).random(M).astype(np.float32) + 0.2) * 0.03
    if f16:
        A, kind = c["A"], capi.F16I8F16_STATIC
    else:
        A, kind = oracle.half_to_float(c["A"]).astype(np.float32).reshape(M, K) * 2.0, capi.F32I8F32_STATIC
    op = ops.W8A8Linear(sess, kind, M, c["B"], c["w_scale"])
    try:
        for _ in range(2):
            rc, got = op.run(A, a_scale)
            want = oracle.w8a8(A, c["B"], c["w_scale"], a_scale_static=a_scale)
            assert rc == 0 and np.array_equal(got.view(np.uint8), want["C"].view(np.uint8))
            q, s = op.read_quantized()
            assert np.array_equal(q, want["q"]) and np.array_equal(s.view(np.uint32), a_scale.view(np.uint32))
    finally:
        op.close()


def test_rounding_ties_neighbours_saturation_and_nan(sess, oracle):
    """Static scale 1 makes the code round-half-away(x) itself: every tie k + 0.5, the floats on either
    side of it, the largest float below 0.5 (where x + 0.5 rounds up to 1.0 in fp32), saturation beyond
    +-127, infinities and NaNs of both signs (the reference's comparison chain turns every NaN into 127).
    Rows with a dynamic scale of exactly 1 (max |x| = 127) go through the same values."""
    ties = np.arange(-128, 128, dtype=np.float32) + np.float32(0.5)
    vals = np.concatenate([ties, np.nextafter(ties, np.float32(np.inf)), np.nextafter(ties, np.float32(-np.inf)),
                           np.arange(-130, 131, dtype=np.float32),
                           np.array([0.49999997, -0.49999997, 0.0, -0.0, 126.99999, 127.00001, -127.00001, 1e30,
                                     -1e30, 1e-30, -1e-30, 127.0], np.float32)]).astype(np.float32)
    K = (vals.size + 31) // 32 * 32
    row = np.zeros(K, np.float32)
    row[:vals.size] = vals
    special = row.copy()
    special[:6] = np.array([np.inf, -np.inf, np.nan, -np.nan, 3.5, -3.5], np.float32)
    special[2:4].view(np.uint32)[:] = [0x7fc00001, 0xffc00001]
    M = 300                                   # many-row quantization kernel; 5 rows go through the per-row one below
    A = np.tile(row, (M, 1))
    A[1::2] = row[::-1]
    A[7] = special
    N = 64
    B = np.zeros((K, N), np.int8)
    B[np.arange(K), np.arange(K) % N] = 1     # column n sums the codes at k = n (mod N)
    ws = np.ones(N, np.float32)
    for rows in (M, 5):
        Ain = A[:rows] if rows == M else A[[0, 1, 7, 2, 3]]
        scale = np.ones(rows, np.float32)
        with np.errstate(over="ignore"):      # 1e30 -> inf in fp16, on purpose
            halves = Ain.astype(np.float16).view(np.uint16)
        for kind, x in ((capi.F32I8F32_STATIC, Ain), (capi.F16I8F16_STATIC, halves)):
            op = ops.W8A8Linear(sess, kind, rows, B, ws)
            try:
                rc, got = op.run(x, scale)
                want = oracle.w8a8(x, B, ws, a_scale_static=scale)
                assert rc == 0
                q, _ = op.read_quantized()
                assert np.array_equal(q, want["q"]), np.argwhere(q != want["q"])[:5].tolist()
                assert np.array_equal(got.view(np.uint8), want["C"].view(np.uint8))
            finally:
                op.close()
        clipped = np.clip(Ain, -127, 127)      # max |x| = 127 -> dynamic scale exactly 1
        clipped[np.isnan(clipped)] = 0
        op = ops.W8A8Linear(sess, capi.F32I8F32_DYNAMIC, rows, B, ws)
        try:
            rc, got = op.run(clipped)
            want = oracle.w8a8(clipped, B, ws)
            assert rc == 0 and (want["a_scale"] == 1.0).all()
            q, _ = op.read_quantized()
            assert np.array_equal(q, want["q"])
            assert np.array_equal(got.view(np.uint32), want["C"].view(np.uint32))
        finally:
            op.close()


def test_config0_full(sess, oracle):
    """BASELINE config 0: M=64, K=2048, N=2048, seeds 0/1."""
    c = workloads.CONFIGS[0]()
    op = ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, c["M"], c["B"], c["w_scale"])
    try:
        rc, got = op.run(c["A"])
        want = oracle.w8a8(c["A"], c["B"], c["w_scale"])
        assert rc == 0
        q, s = op.read_quantized()
        assert np.array_equal(q, want["q"])
        assert np.array_equal(got, want["C"])
        # int32 accumulators through the raw-integer operator on the same codes
        raw = ops.W8A8Linear(sess, capi.I8I8I32, c["M"], c["B"])
        try:
            rc, acc = raw.run(want["q"])
            assert rc == 0 and np.array_equal(acc, want["acc"])
        finally:
            raw.close()
    finally:
        op.close()


def test_config1_full_decode(sess, oracle):
    """BASELINE config 1: M=1, K=4096, N=14336, seeds 2/3 (GEMV path)."""
    c = workloads.CONFIGS[1]()
    op = ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, 1, c["B"], c["w_scale"])
    try:
        rc, got = op.run(c["A"])
        want = oracle.w8a8(c["A"], c["B"], c["w_scale"])
        assert rc == 0
        assert np.array_equal(got, want["C"])
        err = np.abs(oracle.half_to_float(got) - oracle.half_to_float(want["C"])).max()
        assert err <= 1e-3 * np.abs(oracle.half_to_float(want["C"])).max()
        raw = ops.W8A8Linear(sess, capi.I8I8I32, 1, c["B"])
        try:
            rc, acc = raw.run(want["q"])
            assert rc == 0 and np.array_equal(acc, want["acc"])
        finally:
            raw.close()
    finally:
        op.close()


def test_weight_sharing_rebinding_and_errors(sess, oracle):
    """reference tests/test_quant_matmul.cpp:231-330: one weight serves several M,
    a workspace can be re-bound to other compatible weights, k_tile mismatch is
    PARAM, foreign domain is DOMAIN, wrong op kind is PARAM."""
    lib = sess.lib
    M, N, K = 8, 96, 96
    rng = np.random.default_rng(11)
    A = _rand_i8(rng, (M, K))
    B0, B1 = _rand_i8(rng, (K, N)), _rand_i8(rng, (K, N))
    op0 = ops.W8A8Linear(sess, capi.I8I8I32, M, B0, k_tile=32)
    op1 = ops.W8A8Linear(sess, capi.I8I8I32, M, B1, k_tile=32)
    opm1 = ops.W8A8Linear(sess, capi.I8I8I32, 1, B0, k_tile=32)
    full = ops.W8A8Linear(sess, capi.I8I8I32, M, B0)  # k_tile = K
    try:
        ref0, ref1 = oracle.gemm_i8(A, B0), oracle.gemm_i8(A, B1)
        out = np.empty((M, N), np.int32)
        for w, ref in ((op0.w, ref0), (op1.w, ref1), (op0.w, ref0)):
            assert lib.rk_npu_i8i8i32_run(op0.ws, w, capi.ptr(A), capi.ptr(out)) == 0
            assert np.array_equal(out, ref)
        out1 = np.empty((1, N), np.int32)
        assert lib.rk_npu_i8i8i32_run(opm1.ws, op0.w, capi.ptr(A), capi.ptr(out1)) == 0
        assert np.array_equal(out1[0], ref0[0])
        # incompatible K partition
        assert lib.rk_npu_i8i8i32_run(full.ws, op0.w, capi.ptr(A), capi.ptr(out)) == capi.RK_NPU_ERR_PARAM
        # NULL arguments
        assert lib.rk_npu_i8i8i32_run(op0.ws, op0.w, None, capi.ptr(out)) == capi.RK_NPU_ERR_PARAM
        assert lib.rk_npu_i8i8i32_run(None, op0.w, capi.ptr(A), capi.ptr(out)) == capi.RK_NPU_ERR_PARAM
        # wrong op kind for this workspace
        assert lib.rk_npu_f16i8f16_run_dynamic(op0.ws, op0.w, capi.ptr(A), capi.ptr(out)) == capi.RK_NPU_ERR_PARAM
        # foreign domain
        other = lib.rk_npu_iommu_domain_create(sess.ctx, 14)
        assert other and lib.rk_npu_iommu_domain_id(other) == 14
        wc = capi.MatmulWeightConfig(K, N, 32)
        import ctypes as C
        foreign = lib.rk_npu_i8i8i32_weights_create(other, C.byref(wc), capi.ptr(B0))
        assert foreign
        assert lib.rk_npu_i8i8i32_run(op0.ws, foreign, capi.ptr(A), capi.ptr(out)) == capi.RK_NPU_ERR_DOMAIN
        lib.rk_npu_i8i8i32_weights_free(foreign)
        lib.rk_npu_iommu_domain_free(other)
        # invalid scales -> NULL
        ws = np.ones(N, np.float32)
        ws[5] = 0
        assert not lib.rk_npu_f16i8f16_weights_create(sess.domain, C.byref(wc), capi.ptr(B0), capi.ptr(ws))
        ws[5] = np.nan
        assert not lib.rk_npu_f16i8f16_weights_create(sess.domain, C.byref(wc), capi.ptr(B0), capi.ptr(ws))
    finally:
        for o in (op0, op1, opm1, full):
            o.close()


def test_busy_two_threads(sess):
    """reference tests/test_quant_matmul.cpp:271-293: two threads hammer one
    workspace; every call is either OK or BUSY and OK results are correct."""
    import threading
    M, N, K = 64, 512, 2048
    rng = np.random.default_rng(3)
    A = _rand_i8(rng, (M, K))
    B = _rand_i8(rng, (K, N))
    op = ops.W8A8Linear(sess, capi.I8I8I32, M, B)
    want = A.astype(np.int32) @ B.astype(np.int32)
    counts = {"ok": 0, "busy": 0, "bad": 0}
    lock = threading.Lock()
    go = threading.Event()

    def hammer():
        out = np.empty((M, N), np.int32)
        go.wait()
        for _ in range(64):
            rc = sess.lib.rk_npu_i8i8i32_run(op.ws, op.w, capi.ptr(A), capi.ptr(out))
            with lock:
                if rc == 0:
                    counts["ok" if np.array_equal(out, want) else "bad"] += 1
                elif rc == capi.RK_NPU_ERR_BUSY:
                    counts["busy"] += 1
                else:
                    counts["bad"] += 1

    try:
        ts = [threading.Thread(target=hammer) for _ in range(2)]
        for t in ts:
            t.start()
        go.set()
        for t in ts:
            t.join()
        assert counts["bad"] == 0 and counts["ok"] > 0
    finally:
        op.close()
