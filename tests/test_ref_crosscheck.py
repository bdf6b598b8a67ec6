"""Cross-checks the CPU oracle against the reference's own CPU translation
units (oracle/_ref/libref_cpu.so, compiled in place from the reference
checkout by `make -C oracle ref`).  Skipped where that library was not built.
Bit-exact on everything: scales, int8 codes, dequantized fp32 / fp16, row-scale
reuse, the MoE middle (libm flavour: this is an x86 build of the reference),
and the k_tile certificate.
"""
import numpy as np
import pytest

from oracle import ref_binding as ref

pytestmark = pytest.mark.skipif(not ref.available(), reason="oracle/_ref not built (no reference checkout)")


def _bits(x):
    return np.ascontiguousarray(x, np.float32).view(np.uint32)


def _activations(seed, M, K):
    rng = np.random.default_rng(seed)
    A = (rng.standard_normal((M, K)) * np.float32(10.0) ** rng.integers(-3, 3, (M, 1))).astype(np.float32)
    A[0] = 0
    A[1, : min(K, 8)] = [127, -127, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5][: min(K, 8)]
    A[1, min(K, 8):] = 0
    if M > 2:
        A[2] = np.float32(1e-41)          # denormal row
    return A


@pytest.mark.parametrize("M,K", [(3, 33), (7, 200), (5, 533), (65, 1030)])
def test_w8_scales_and_codes(oracle, M, K):
    A = _activations(M * K, M, K)
    for arr in (A, A.astype(np.float16).view(np.uint16)):
        s = oracle.w8_scales(arr)
        assert np.array_equal(_bits(s), _bits(ref.w8_scales(arr)))
        assert np.array_equal(oracle.w8_quant(arr, s), ref.w8_quant(arr, s))


@pytest.mark.parametrize("M,K", [(3, 33), (5, 533), (65, 4097), (130, 2100)])
def test_w4a8_scales_and_codes(oracle, M, K):
    A = _activations(M + K, M, K)
    for arr in (A, A.astype(np.float16).view(np.uint16)):
        rc, s, inv = oracle.w4a8_scales(arr)
        rc2, s2, inv2 = ref.w4a8_scales(arr)
        assert rc == 0 and rc2 == 0
        assert np.array_equal(_bits(s), _bits(s2)) and np.array_equal(_bits(inv), _bits(inv2))
        rc3, q2 = ref.w4a8_quant(arr, s2, inv2)
        assert rc3 == 0 and np.array_equal(oracle.w4a8_quant(arr, inv), q2)
    B = A.copy()
    B[M - 1, K - 1] = np.nan
    assert oracle.w4a8_scales(B)[0] == ref.w4a8_scales(B)[0] == oracle.ERR_PARAM


@pytest.mark.parametrize("M,N", [(1, 8), (5, 65), (33, 130), (64, 513)])
def test_dequant_both_operators(oracle, M, N):
    rng = np.random.default_rng(M * N)
    acc = rng.integers(-2 ** 27, 2 ** 27, (M, N)).astype(np.int32)
    acc[0, :4] = [16777217, -16777219, 2 ** 31 - 1, -2 ** 31]
    a_s = (rng.random(M).astype(np.float32) + 0.01) * np.float32(10.0) ** rng.integers(-4, 1, M)
    w_s = (rng.random(N).astype(np.float32) + 0.01) * np.float32(10.0) ** rng.integers(-4, 1, N)
    a_s, w_s = a_s.astype(np.float32), w_s.astype(np.float32)
    for half in (False, True):
        got = oracle.dequant(acc, a_s, w_s, half=half)
        assert np.array_equal(got.view(np.uint16 if half else np.uint32),
                              ref.w8_dequant(acc, a_s, w_s, half).view(np.uint16 if half else np.uint32))
        assert np.array_equal(got.view(np.uint16 if half else np.uint32),
                              ref.w4a8_dequant(acc, a_s, w_s, half).view(np.uint16 if half else np.uint32))


def test_split_k_sum_wraps_like_the_reference(oracle):
    rng = np.random.default_rng(9)
    M, N, K = 4, 40, 300
    A = rng.integers(-128, 128, (M, K)).astype(np.int8)
    B = rng.integers(-128, 128, (K, N)).astype(np.int8)
    p0, p1 = oracle.gemm_i8(A[:, :160], B[:160]), oracle.gemm_i8(A[:, 160:], B[160:])
    assert np.array_equal(ref.w8_reduce_two(p0, p1), oracle.gemm_i8(A, B))
    big = np.full((1, 8), 2 ** 31 - 5, np.int32)
    assert np.array_equal(ref.w8_reduce_two(big, big), (big.astype(np.int64) * 2 + 2 ** 31) % 2 ** 32 - 2 ** 31)


def test_finish_scales(oracle):
    rng = np.random.default_rng(10)
    vals = np.abs(rng.standard_normal(500).astype(np.float32)) * np.float32(10.0) ** rng.integers(-42, 30, 500)
    bits = np.concatenate([vals.astype(np.float32).view(np.uint32), np.array([0, 1, 0x00800000, 0x7f7fffff], np.uint32)])
    rc, s, inv = oracle.finish_scales(bits)
    rc2, s2, inv2 = ref.finish_scales(bits)
    assert rc == rc2 == 0 and np.array_equal(_bits(s), _bits(s2)) and np.array_equal(_bits(inv), _bits(inv2))
    for bad in (0x7f800000, 0x7fc00000):
        b = bits.copy()
        b[17] = bad
        assert oracle.finish_scales(b)[0] == ref.finish_scales(b)[0] == oracle.ERR_PARAM


@pytest.mark.parametrize("channels", [32, 96, 512])
def test_moe_middle_row_libm_flavour(oracle, channels):
    """reference src/rk_npu_moe_cpu.cpp:38-114 (scalar branch): dequant, SwiGLU with
    std::exp, row scale without FLT_MIN clamp, nearest-even codes."""
    rng = np.random.default_rng(channels)
    for trial in range(6):
        acc = rng.integers(-40000, 40000, 2 * channels).astype(np.int32)
        if trial == 0:
            acc[:] = 0
        ws = (rng.random(2 * channels).astype(np.float32) + 0.5) * 0.002
        a_s = np.float32(0.013 * (trial + 1))
        s_ref, q_ref = ref.moe_middle_row(acc, ws, float(a_s))
        mid, _ = oracle.swiglu(acc[None, :], np.array([a_s], np.float32), ws, oracle.EXP_LIBM)
        s, q = oracle.moe_quant_row(mid[0], validate=False)
        assert np.float32(s).view(np.uint32) == np.float32(s_ref).view(np.uint32)
        assert np.array_equal(q, q_ref)


def test_k_tile_certificate_matches_golden_and_reference():
    """The certified-tile search lives in the shipped host layer; its answers on
    seeded code matrices are frozen in tests/golden/i4_bounds.json by
    tests/golden/make_golden.py from the reference's bound_i4_weights.  Here the
    fixture itself is re-derived to make sure it is current."""
    import json
    import os
    from tests.golden import make_golden
    path = os.path.join(os.path.dirname(__file__), "golden", "i4_bounds.json")
    with open(path) as f:
        frozen = json.load(f)
    assert frozen == make_golden.i4_bound_cases()
