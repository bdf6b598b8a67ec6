"""Pins the CPU oracle (oracle/rk_oracle.c) without a GPU.

Every check here is something other than a retyped formula: the known answers
of the reference's own unit tests, IEEE / numpy as an independent authority,
int64 brute force, algebraic invariants, and special cases with closed forms.
"""
import numpy as np
import pytest

FLT_MIN = np.float32(np.finfo(np.float32).tiny)


# ---- binary16 <-> binary32 ------------------------------------------------
def test_half_exhaustive_against_numpy(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    f = oracle.half_to_float(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(f.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    assert np.isnan(f[nan]).all()
    # round trip: reference tests/test_w4a8_cpu.cpp:122-128
    back = oracle.float_to_half(f)
    assert np.array_equal(back[~nan], bits[~nan])
    assert ((back[nan] & 0x7c00) == 0x7c00).all() and ((back[nan] & 1023) != 0).all()


def test_float_to_half_rne_against_numpy(oracle):
    rng = np.random.default_rng(0)
    x = rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-8, 6, 200000)
    x = np.concatenate([x.astype(np.float32),
                        np.array([0.0, -0.0, 65504, 65519.99, 65520, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8,
                                  np.inf, -np.inf, 6.1035156e-05, 6.0975552e-05], np.float32)])
    # exact ties between two halves: half + half an ulp
    h = rng.integers(0, 0x7bff, 5000).astype(np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    x = np.concatenate([x, ((lo + hi) / 2).astype(np.float32)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.float_to_half(x), want)


# ---- activation quantization ---------------------------------------------
def test_w8_quant_matches_round_of_product_with_reciprocal(oracle):
    """reference tests/test_cpu_kernels.cpp:172-176: q = round(x * (1 / scale)),
    ties away from zero, clamped to +-127; zero row -> scale 1."""
    A = np.array([[127, -127, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 0.49999997, 3.4999998],
                  [0] * 10,
                  [1e-3, -2e-3, 5e-4, 0, 0, 0, 0, 0, 0, 0]], np.float32)
    s = oracle.w8_scales(A)
    assert s[0] == np.float32(1.0) and s[1] == np.float32(1.0)
    assert s[2] == np.float32(2e-3) / np.float32(127)
    q = oracle.w8_quant(A, s)
    assert q[0].tolist() == [127, -127, 1, 2, 3, -1, -2, -3, 0, 3]
    assert (q[1] == 0).all()
    inv = np.float32(1.0) / s[2]
    want = np.clip(np.sign(A[2] * inv) * np.floor(np.abs(A[2] * inv) + np.float32(0.5)), -127, 127)
    assert q[2].tolist() == want.astype(np.int8).tolist()
    # fp16 input path sees the half-rounded values
    A16 = A.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.w8_quant(A16, oracle.w8_scales(A16)),
                          oracle.w8_quant(oracle.half_to_float(A16), oracle.w8_scales(oracle.half_to_float(A16))))


def test_w4a8_scale_rules(oracle):
    """reference tests/test_w4a8_cpu.cpp:34-41,78-88: scale-1 ties, zero row,
    FLT_MIN floor for denormal maxima, NaN / Inf rejection (f32 and f16)."""
    K = 533
    k = np.arange(K)
    A = np.zeros((5, K), np.float32)
    for m in range(1, 5):
        A[m] = np.ldexp((k % 255 - 127).astype(np.float32), m - 3)
        A[m, K - 1] = np.ldexp(np.float32(254.0), m - 3)
    A[1] = (k % 255 - 127).astype(np.float32)
    A[1, 1:5] = [0.5, -0.5, 1.5, -1.5]
    A[1, K - 2] = -0.5
    rc, s, inv = oracle.w4a8_scales(A)
    assert rc == 0 and s[0] == 1 and s[1] == 1           # |max| = 127 -> scale exactly 1
    q = oracle.w4a8_quant(A, inv)
    assert q[1, 1:5].tolist() == [1, -1, 2, -2] and q[1, K - 2] == -1
    assert q[1, 0] == -127 and (q[0] == 0).all()
    for m in range(2, 5):                                 # max = 254 * 2^(m-3): codes are k%255-127 halved...
        ref = np.clip(np.sign(A[m] * inv[m]) * np.floor(np.abs(A[m] * inv[m]) + np.float32(0.5)), -127, 127)
        assert np.array_equal(q[m], ref.astype(np.int8))
    for bad in (np.inf, -np.inf, np.nan):
        B = A.copy()
        B[0, 0] = bad
        assert oracle.w4a8_scales(B)[0] == oracle.ERR_PARAM
    H = A.astype(np.float16).view(np.uint16)
    H[0, 0] = 0x7c00
    assert oracle.w4a8_scales(H)[0] == oracle.ERR_PARAM
    tiny = np.array([[np.float32(1e-45)]], np.float32)    # denorm_min
    rc, s, inv = oracle.w4a8_scales(tiny)
    assert rc == 0 and s[0] == FLT_MIN and np.isfinite(inv[0])


def test_msd_split_identity(oracle):
    """reference tests/test_w4a8_cpu.cpp:71: q == 16*h + l + 8 with both halves in int4 range."""
    for q in range(-128, 128):
        h, l = oracle.msd_split(q)
        assert -8 <= h <= 7 and -8 <= l <= 7 and 16 * h + l + 8 == q


def test_moe_quant_ties_to_even(oracle):
    """reference tests/test_moe_w8.cpp:107-115 anchors and tests/test_moe_cpu.cpp:52-63 (lrint)."""
    x = np.zeros(64, np.float32)
    x[:8] = [127, -127, .5, 1.5, 2.5, -.5, -1.5, -2.5]
    s, q = oracle.moe_quant_row(x)
    assert s == 1.0 and q[:8].tolist() == [127, -127, 0, 2, 2, 0, -2, -2]
    rng = np.random.default_rng(1)
    y = (rng.standard_normal(4096) * 3).astype(np.float32)
    s, q = oracle.moe_quant_row(y)
    assert np.float32(s) == np.abs(y).max() / np.float32(127)
    inv = np.float32(1.0) / np.float32(s)
    assert np.array_equal(q, np.clip(np.rint(y * inv), -127, 127).astype(np.int8))  # rint = ties even
    assert oracle.moe_quant_row(np.zeros(32, np.float32))[0] == 1.0
    y[7] = np.nan
    assert oracle.moe_quant_row(y)[0] == 0.0                                       # validate -> 0
    assert oracle.moe_quant_row(y, validate=False)[0] != 0.0


# ---- integer GEMM -----------------------------------------------------------
@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (3, 5, 7), (17, 40, 33), (4, 600, 129), (9, 65, 1000)])
def test_gemm_brute_force_int64(oracle, M, N, K):
    rng = np.random.default_rng(M * N + K)
    A = rng.integers(-128, 128, (M, K)).astype(np.int8)
    B = rng.integers(-128, 128, (K, N)).astype(np.int8)
    want = A.astype(np.int64) @ B.astype(np.int64)
    assert np.array_equal(oracle.gemm_i8(A, B).astype(np.int64), want)


def test_gemm_invariants(oracle):
    rng = np.random.default_rng(2)
    M, N, K = 6, 70, 200
    A = rng.integers(-127, 128, (M, K)).astype(np.int8)
    B = rng.integers(-127, 128, (K, N)).astype(np.int8)
    C = oracle.gemm_i8(A, B)
    # split-K linearity
    assert np.array_equal(C, oracle.gemm_i8(A[:, :77], B[:77]) + oracle.gemm_i8(A[:, 77:], B[77:]))
    # permuting k on both sides, rows of A, columns of B
    pk, pm, pn = rng.permutation(K), rng.permutation(M), rng.permutation(N)
    assert np.array_equal(C, oracle.gemm_i8(A[:, pk], B[pk]))
    assert np.array_equal(C[pm][:, pn], oracle.gemm_i8(A[pm], B[:, pn]))
    # transposed operand would fail: A @ B != (B.T @ A.T) unless transposed back
    assert np.array_equal(C, oracle.gemm_i8(np.ascontiguousarray(B.T), np.ascontiguousarray(A.T)).T)


def test_gemm_wraps_mod_2_32(oracle):
    K = 131072 + 64
    A = np.full((1, K), -128, np.int8)
    B = np.full((K, 2), -128, np.int8)
    want = ((16384 * K + 2 ** 31) % 2 ** 32) - 2 ** 31
    assert (oracle.gemm_i8(A, B) == want).all()


# ---- dequant ----------------------------------------------------------------
def test_dequant_known_answers(oracle):
    """reference tests/test_w4a8_cpu.cpp:133-142 (values) and
    tests/test_w4a8_reduction.cpp:62-86 (sums above 2^24 round once in int->float)."""
    acc = np.array([[-100001, 0, 1, 2, 2049, 65536, 12345, -45678, 16777217, -33554435]], np.int32)
    a_s = np.array([0.125], np.float32)
    w_s = np.array([1, 1, 1, 1, 1, 1, .003, 2, 1, 3], np.float32)
    out = oracle.dequant(acc, a_s, w_s)
    want = (acc.astype(np.float32) * a_s[0]) * w_s      # numpy float32 ops are IEEE, one rounding each
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    assert out[0, 8] == np.float32(16777216.0) * np.float32(0.125)       # 2^24 + 1 rounds to even
    half = oracle.dequant(acc, a_s, w_s, half=True)
    with np.errstate(over="ignore"):
        assert np.array_equal(half, want.astype(np.float16).view(np.uint16))
    # the order of the two multiplies matters: (acc * ws) * as differs somewhere
    rng = np.random.default_rng(3)
    acc = rng.integers(-2 ** 20, 2 ** 20, (8, 512)).astype(np.int32)
    a_s = (rng.random(8).astype(np.float32) + 0.1) * 0.01
    w_s = (rng.random(512).astype(np.float32) + 0.1) * 0.001
    right = (acc.astype(np.float32) * a_s[:, None]) * w_s[None, :]
    wrong = (acc.astype(np.float32) * w_s[None, :]) * a_s[:, None]
    assert not np.array_equal(right, wrong)
    assert np.array_equal(oracle.dequant(acc, a_s, w_s), right)


# ---- SwiGLU -------------------------------------------------------------------
def _silu_poly_f64_steps(g):
    """Independent evaluation of the polynomial SiLU with every step rounded to
    float32 explicitly (fma emulated in float64, exact for these magnitudes)."""
    f32 = np.float32
    def fma(a, b, c):
        return f32(np.float64(a) * np.float64(b) + np.float64(c))
    g = f32(g)
    x = f32(-g)
    x = min(x, f32(80.0))
    x = max(x, f32(-80.0))
    n = f32(np.floor(fma(x, f32(1.4426950408889634), f32(0.5))))
    r = fma(-n, f32(0.693145751953125), x)
    r = fma(-n, f32(1.428606765330187e-6), r)
    p = f32(1.0) / f32(5040.0)
    for c in (f32(1.0) / f32(720.0), f32(1.0) / f32(120.0), f32(1.0) / f32(24.0), f32(1.0) / f32(6.0),
              f32(0.5), f32(1.0), f32(1.0)):
        p = fma(p, r, c)
    d = f32(f32(1.0) + f32(p * f32(2.0) ** int(n)))
    return f32(-0.0) if g < f32(-80.0) else f32(g / d)


def test_silu_poly_special_cases_and_independent_evaluation(oracle):
    assert oracle.silu_mul(0.0, 3.0, oracle.EXP_POLY) == 0.0                 # g = 0 -> 0 / 2
    assert oracle.silu_mul(1.0, 1.0, oracle.EXP_POLY) == pytest.approx(0.7310585786, rel=2e-7)
    y = np.float32(oracle.silu_mul(-80.5, 2.0, oracle.EXP_POLY))
    assert y == 0.0 and np.signbit(y)                                        # g < -80 -> -0.0 * u
    y = np.float32(oracle.silu_mul(-1000.0, -2.0, oracle.EXP_POLY))
    assert y == 0.0 and not np.signbit(y)
    assert oracle.silu_mul(200.0, 1.0, oracle.EXP_POLY) == 200.0             # saturated exp(-80) vanishes
    assert oracle.silu_mul(-80.0, 1.0, oracle.EXP_POLY) < 0.0                # exactly -80 is still computed
    rng = np.random.default_rng(4)
    gs = np.concatenate([rng.standard_normal(3000) * 4, rng.uniform(-90, 90, 3000),
                         [-80.0, 80.0, -79.999, 1e-30, -1e-30, 88.0, -87.0]]).astype(np.float32)
    for g in gs:
        got = np.float32(oracle.silu_mul(float(g), 1.0, oracle.EXP_POLY))
        want = _silu_poly_f64_steps(g)
        assert got.view(np.uint32) == np.float32(want).view(np.uint32), float(g)


def test_silu_poly_within_reference_bound_of_libm(oracle):
    """reference tests/test_w4a8_swiglu.cpp:62-69: |poly - expf flavour| <= 7e-7 relative."""
    rng = np.random.default_rng(5)
    g = np.concatenate([rng.standard_normal(20000) * 3, rng.uniform(-20, 20, 20000)]).astype(np.float32)
    u = rng.standard_normal(g.size).astype(np.float32)
    worst = 0.0
    for gi, ui in zip(g[:8000], u[:8000]):
        a = oracle.silu_mul(float(gi), float(ui), oracle.EXP_POLY)
        b = oracle.silu_mul(float(gi), float(ui), oracle.EXP_LIBM)
        if b != 0:
            worst = max(worst, abs(a - b) / abs(b))
    assert worst <= 7e-7
    # libm flavour against float64 math
    x = g[:2000].astype(np.float64)
    ref = x / (1 + np.exp(-x)) * u[:2000]
    got = np.array([oracle.silu_mul(float(a), float(b), oracle.EXP_LIBM) for a, b in zip(g[:2000], u[:2000])])
    assert np.allclose(got, ref, rtol=3e-7, atol=1e-30)


def test_swiglu_gate_up_pairing_and_row_max(oracle):
    """gate column n pairs with up column F + n (reference src/rk_npu_w4a8_swiglu.cpp:61-78);
    a swapped or shifted pairing changes the result."""
    rng = np.random.default_rng(6)
    M, F = 5, 96
    acc = rng.integers(-3000, 3000, (M, 2 * F)).astype(np.int32)
    a_s = (rng.random(M).astype(np.float32) + 0.5) * 0.01
    w_s = (rng.random(2 * F).astype(np.float32) + 0.5) * 0.05
    mid, bits = oracle.swiglu(acc, a_s, w_s, oracle.EXP_LIBM)
    g = (acc[:, :F].astype(np.float32) * a_s[:, None]) * w_s[None, :F]
    u = (acc[:, F:].astype(np.float32) * a_s[:, None]) * w_s[None, F:]
    ref = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    assert np.allclose(mid, ref, rtol=1e-6, atol=1e-30)
    assert np.array_equal(bits, np.abs(mid).max(axis=1).view(np.uint32))
    swapped = np.concatenate([acc[:, F:], acc[:, :F]], axis=1)
    assert not np.allclose(oracle.swiglu(swapped, a_s, np.concatenate([w_s[F:], w_s[:F]]), oracle.EXP_LIBM)[0], mid)


def test_finish_scales_boundaries(oracle):
    """reference tests/test_w4a8_ffn.cpp:19-30: bits 0 -> 1; 1 (denormal) and
    0x00800000 (FLT_MIN) -> FLT_MIN floor; 1.0 / 2.0 -> max/127; Inf / NaN -> PARAM."""
    bits = np.array([0, 1, 0x00800000, 0x3f800000, 0x40000000], np.uint32)
    rc, s, inv = oracle.finish_scales(bits)
    assert rc == 0
    assert s[0] == 1 and s[1] == FLT_MIN and s[2] == FLT_MIN
    assert s[3] == np.float32(1.0) / np.float32(127) and s[4] == np.float32(2.0) / np.float32(127)
    assert np.array_equal(inv, np.float32(1.0) / s)
    for bad in (0x7f800000, 0x7fc00000, 0x7f800001):
        assert oracle.finish_scales(np.array([0, bad], np.uint32))[0] == oracle.ERR_PARAM


# ---- composites ---------------------------------------------------------------
def test_w8a8_operator_is_the_composition(oracle):
    rng = np.random.default_rng(7)
    M, K, N = 5, 130, 70
    A = (rng.standard_normal((M, K)) * 2).astype(np.float16).view(np.uint16)
    B = rng.integers(-127, 128, (K, N)).astype(np.int8)
    ws = (rng.random(N).astype(np.float32) + 0.5) * 0.01
    r = oracle.w8a8(A, B, ws)
    s = oracle.w8_scales(A)
    q = oracle.w8_quant(A, s)
    acc = q.astype(np.int64) @ B.astype(np.int64)
    assert np.array_equal(r["q"], q) and np.array_equal(r["acc"], acc)
    assert np.array_equal(r["C"], oracle.dequant(acc.astype(np.int32), s, ws, half=True))


def test_ffn_reuses_row_scale_and_rejects_nonfinite_middle(oracle):
    rng = np.random.default_rng(8)
    M, H, I, Nout = 6, 64, 96, 40
    x = rng.standard_normal((M, H)).astype(np.float32)
    x[2] = 0
    B_gu = rng.integers(-7, 8, (H, 2 * I)).astype(np.int8)
    s_gu = (rng.random(2 * I).astype(np.float32) + 0.5) * 0.02
    B_dn = rng.integers(-7, 8, (I, Nout)).astype(np.int8)
    s_dn = (rng.random(Nout).astype(np.float32) + 0.5) * 0.02
    r = oracle.w4a8_ffn(x, B_gu, s_gu, B_dn, s_dn)
    assert r["rc"] == 0
    # Down of the FFN == plain W4A8 run on the middle (scale from a rescan is the same number)
    plain = oracle.w4a8(r["middle"], B_dn, s_dn)
    assert np.array_equal(plain["q"], r["q_down"]) and np.array_equal(plain["C"], r["C"])
    assert r["down_scale"][2] == 1.0 and (r["middle"][2] == 0).all()
    big = oracle.w4a8_ffn(x * 1e6, B_gu, np.full(2 * I, 1e30, np.float32), B_dn, s_dn)
    assert big["rc"] == oracle.ERR_PARAM


def test_moe_oracle_against_reference_test_formula(oracle):
    """Python restatement of the oracle of reference tests/test_moe_w8.cpp:24-44
    (libm exp, lrint, std::fma) on that test's own deterministic tensors."""
    H, N, E, TOP = 64, 32, 3, 2
    experts = []
    for e in range(E + 1):
        i = np.arange(H * 2 * N, dtype=np.int64)
        g = (((i * 17 + i // 19 + e * 11) % 7) - 3).astype(np.int8).reshape(H, 2 * N)
        j = np.arange(N * H, dtype=np.int64)
        d = (((j * 13 + j // 7 + e * 5) % 7) - 3).astype(np.int8).reshape(N, H)
        experts.append((g, np.full(2 * N, 0.0625, np.float32), d, np.full(H, 0.015625, np.float32)))
    rows = 5
    i = np.arange(rows * H, dtype=np.int64)
    x = (((i * 7 + i // 5) % 255) - 127).astype(np.int8).reshape(rows, H)
    scales = np.full(rows, 0.03125, np.float32)
    ids = np.array([[(r + s) % E for s in range(TOP)] for r in range(rows)], np.int32)
    routes = np.tile(np.array([0.625, 0.375], np.float32), (rows, 1))
    ids[0] = 0
    routes[0, 1] = 0
    rc, got = oracle.moe_w8(experts, H, N, E, 1, TOP, ids, routes, input_q=x, row_scales=scales,
                            flavour=oracle.EXP_LIBM, fused_combine=True)
    assert rc == 0
    want = np.zeros((rows, H), np.float32)
    f32 = np.float32
    for r in range(rows):
        for slot in range(TOP + 1):
            e = ids[r, slot] if slot < TOP else E
            w = routes[r, slot] if slot < TOP else f32(1)
            g, gs, d, ds = experts[e]
            acc = x[r].astype(np.int64) @ g.astype(np.int64)
            gu = (acc.astype(np.float32) * scales[r]) * gs
            gate, up = gu[:N], gu[N:]
            hid = (gate / (f32(1) + np.exp(-gate).astype(np.float32))) * up
            mx = np.abs(hid).max()
            s2 = mx / f32(127) if mx else f32(1)
            q2 = np.clip(np.rint(hid * (f32(1) / s2)), -127, 127).astype(np.int64)
            acc2 = q2 @ d.astype(np.int64)
            val = (acc2.astype(np.float32) * s2) * ds
            # the reference test's oracle applies every slot, including coefficient 0 (adds 0)
            want[r] = (val.astype(np.float64) * np.float64(w) + want[r].astype(np.float64)).astype(np.float32)
    rel = np.sqrt(((got.astype(np.float64) - want) ** 2).sum() / (want.astype(np.float64) ** 2).sum())
    assert rel < 1e-6   # reference bar: tests/test_moe_w8.cpp:93
    # dropped routes and bad ids
    bad = ids.copy()
    bad[1, 0] = E
    assert oracle.moe_w8(experts, H, N, E, 1, TOP, bad, routes, input_q=x, row_scales=scales)[0] == oracle.ERR_PARAM
