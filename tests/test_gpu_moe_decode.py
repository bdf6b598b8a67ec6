"""The MoE layer for a handful of tokens through the device-pointer call: up to eight fp32 tokens take
two launches of dot-product kernels instead of the five of the grouped path.  Same arithmetic, so the
outputs are compared bit for bit with the oracle -- and with the grouped path itself (the same tokens
inside a larger call, and through the host-pointer call, which always takes the grouped path).
"""
import numpy as np
import pytest

from rknpu2_matmul_open_amd import capi, ops

pytestmark = pytest.mark.gpu


def _experts(rng, H, I, count, lo, hi):
    out = []
    for _ in range(count):
        g = rng.integers(lo, hi + 1, (H, 2 * I)).astype(np.int8)
        d = rng.integers(lo, hi + 1, (I, H)).astype(np.int8)
        gs = (rng.random(2 * I).astype(np.float32) + 0.5) * np.float32(0.02)
        ds = (rng.random(H).astype(np.float32) + 0.5) * np.float32(0.02)
        out.append((g, gs, d, ds))
    return out


def _routing(rng, T, E, top_k):
    ids = np.stack([rng.permutation(E)[:top_k] for _ in range(T)]).astype(np.int32)
    routes = rng.random((T, top_k), dtype=np.float32) + np.float32(0.1)
    return ids, routes


def _run_device(sess, moe, x, ids, routes):
    T = x.shape[0]
    dx, dids, drt = sess.to_device(x), sess.to_device(ids), sess.to_device(routes)
    dout = sess.empty_device(T * moe.H * 4)
    try:
        rc = sess.lib.rk_npu_moe_w8_run_f32_device(moe.ws, moe.w, T, dx, dids, drt, dout)
        sync = sess.sync()
        return rc, sync, sess.from_device(dout, (T, moe.H), np.float32)
    finally:
        for d in (dx, dids, drt, dout):
            sess.free_device(d)


# (T, H, I, E, top_k, shared): every token count of the path, the smallest and large geometries, a K
# that is not a multiple of the 256 the weights are padded to, many slots, the longest token row; and a
# middle too long for the path (8192: that call takes the grouped path and must agree all the same);
# the last two: output widths at which the down kernel takes 16 columns per workgroup (the others: 8 or 32)
CASES = [(1, 64, 32, 3, 2, 1), (1, 2048, 1024, 32, 4, 0), (2, 128, 64, 6, 2, 0), (3, 96, 160, 5, 3, 1),
         (4, 2048, 1024, 32, 4, 1), (5, 416, 96, 9, 8, 0), (7, 64, 8192, 4, 2, 1), (8, 4096, 512, 16, 4, 0),
         (8, 160, 32, 40, 8, 1), (6, 32768, 32, 2, 1, 0), (2, 2048, 64, 4, 2, 1), (3, 1408, 128, 5, 2, 0),
         (10, 2048, 1024, 32, 4, 1), (12, 256, 128, 12, 4, 0)]


def _flavours(case):
    """The expert formats a geometry can take: INT4 images need hidden and intermediate sizes
    that are multiples of 64, and the mixed format is the one with a shared int8 expert."""
    _, H, I, _, _, shared = case
    out = ["w8"]
    if H % 64 == 0 and I % 64 == 0:
        out.append("quant")
        if shared:
            out.append("w4")
    return out


@pytest.mark.parametrize("T,H,I,E,top_k,shared,flavour", [c + (f,) for c in CASES for f in _flavours(c)])
def test_decode_sized_calls_bit_exact(sess, oracle, T, H, I, E, top_k, shared, flavour):
    rng = np.random.default_rng(T * 1000 + H + I + E)
    int4 = flavour != "w8"
    experts = _experts(rng, H, I, E, -8 if int4 else -127, 7 if int4 else 127)
    if shared:
        wide = flavour != "quant"          # the shared expert of "w4" is int8
        experts += _experts(rng, H, I, 1, -127 if wide else -8, 127 if wide else 7)
    x = (rng.standard_normal((T, H)) * 1.5).astype(np.float32)
    ids, routes = _routing(rng, T, E, top_k)
    moe = ops.MoeW8(sess, H, I, E, shared, top_k, 16, experts, flavour=flavour)
    try:
        rc, sync, got = _run_device(sess, moe, x, ids, routes)
        rc2, want = oracle.moe_w8(experts, H, I, E, shared, top_k, ids, routes, input_f32=x)
        assert rc == 0 and sync == 0 and rc2 == 0
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        # the host-pointer call (grouped path) agrees, and so does a second device call
        rc, host = moe.run_f32(x, ids, routes)
        assert rc == 0 and np.array_equal(host.view(np.uint32), want.view(np.uint32))
        rc, sync, again = _run_device(sess, moe, x, ids, routes)
        assert rc == 0 and sync == 0 and np.array_equal(again.view(np.uint32), want.view(np.uint32))
    finally:
        moe.close()


def test_dropped_duplicate_and_all_zero_routes(sess, oracle):
    """Coefficient 0 drops an assignment, an expert may appear twice in a token's slots, a token
    whose coefficients are all zero yields a zero row (with a shared expert: that expert alone)."""
    H, I, E, top_k, T = 128, 64, 5, 3, 6
    rng = np.random.default_rng(77)
    for shared in (0, 1):
        experts = _experts(rng, H, I, E + shared, -127, 127)
        x = rng.standard_normal((T, H)).astype(np.float32)
        ids, routes = _routing(rng, T, E, top_k)
        routes[0, 1] = 0.0
        ids[1] = [2, 2, 4]                      # duplicate
        routes[2] = 0.0                         # nothing routed
        ids[3] = [0, 0, 0]
        routes[3] = [0.25, 0.0, 0.5]
        x[4] = 0.0                              # an all-zero token: scale 1, codes 0
        moe = ops.MoeW8(sess, H, I, E, shared, top_k, 8, experts)
        try:
            rc, sync, got = _run_device(sess, moe, x, ids, routes)
            rc2, want = oracle.moe_w8(experts, H, I, E, shared, top_k, ids, routes, input_f32=x)
            assert rc == 0 and sync == 0 and rc2 == 0
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
            if not shared:
                assert not got[2].any()
        finally:
            moe.close()


def test_rejected_input_is_reported_by_the_next_sync(sess):
    """The device call cannot look at its operands: a non-finite token, an id out of range and a
    negative or non-finite coefficient raise the context's flag, which the next sync returns as
    ERR_PARAM -- like the grouped path."""
    H, I, E, top_k, T = 64, 32, 4, 2, 3
    rng = np.random.default_rng(5)
    experts = _experts(rng, H, I, E, -127, 127)
    moe = ops.MoeW8(sess, H, I, E, 0, top_k, 8, experts)
    try:
        x = rng.standard_normal((T, H)).astype(np.float32)
        ids, routes = _routing(rng, T, E, top_k)
        rc, sync, _ = _run_device(sess, moe, x, ids, routes)
        assert rc == 0 and sync == 0
        for what in ("nan", "inf", "id_high", "id_negative", "negative", "nan_route"):
            bx, bids, brt = x.copy(), ids.copy(), routes.copy()
            if what == "nan":
                bx[1, 7] = np.nan
            elif what == "inf":
                bx[2, 0] = -np.inf
            elif what == "id_high":
                bids[0, 1] = E
            elif what == "id_negative":
                bids[2, 0] = -1
            elif what == "negative":
                brt[1, 1] = -0.5
            else:
                brt[0, 0] = np.nan
            rc, sync, _ = _run_device(sess, moe, bx, bids, brt)
            assert rc == 0 and sync == capi.RK_NPU_ERR_PARAM, what
            rc, sync, _ = _run_device(sess, moe, x, ids, routes)     # the flag does not stick
            assert rc == 0 and sync == 0, what
    finally:
        moe.close()


def test_extreme_codes_and_token_magnitudes(sess, oracle):
    """Every weight at the end of its range against tokens of +-max: the largest sums the layer can
    produce, for int8 and for INT4 experts (the latter multiplied as 16 x code and shifted back)."""
    H, I, E, top_k, T = 2048, 1024, 2, 2, 2
    for flavour, lo, hi in (("w8", -127, 127), ("quant", -8, 7)):
        experts = []
        for e in range(E):
            g = np.full((H, 2 * I), lo if e == 0 else hi, np.int8)
            d = np.full((I, H), hi if e == 0 else lo, np.int8)
            experts.append((g, np.full(2 * I, 1e-3, np.float32), d, np.full(H, 1e-3, np.float32)))
        x = np.full((T, H), 3.0, np.float32)
        x[1] = -3.0
        ids = np.array([[0, 1], [1, 0]], np.int32)
        routes = np.array([[0.5, 0.5], [0.75, 0.25]], np.float32)
        moe = ops.MoeW8(sess, H, I, E, 0, top_k, 8, experts, flavour=flavour)
        try:
            rc, sync, got = _run_device(sess, moe, x, ids, routes)
            rc2, want = oracle.moe_w8(experts, H, I, E, 0, top_k, ids, routes, input_f32=x)
            assert rc == 0 and sync == 0 and rc2 == 0
            finite = np.isfinite(want).all(axis=1)
            assert np.array_equal(got[finite].view(np.uint32), want[finite].view(np.uint32))
            assert not np.isfinite(got[~finite]).all(axis=1).any()
        finally:
            moe.close()


def test_the_same_tokens_in_a_larger_call_give_the_same_rows(sess, oracle):
    """Eight tokens through the two-launch path and the same eight among forty through the grouped
    path: identical rows."""
    H, I, E, top_k = 256, 128, 12, 4
    rng = np.random.default_rng(11)
    experts = _experts(rng, H, I, E + 1, -127, 127)
    x = rng.standard_normal((40, H)).astype(np.float32)
    ids, routes = _routing(rng, 40, E, top_k)
    moe = ops.MoeW8(sess, H, I, E, 1, top_k, 64, experts)
    try:
        rc, sync, big = _run_device(sess, moe, x, ids, routes)
        assert rc == 0 and sync == 0
        for first in (0, 8, 32):
            rc, sync, small = _run_device(sess, moe, x[first:first + 8], ids[first:first + 8], routes[first:first + 8])
            assert rc == 0 and sync == 0
            assert np.array_equal(small.view(np.uint32), big[first:first + 8].view(np.uint32))
    finally:
        moe.close()


def test_random_geometries(sess, oracle):
    """Seeded random layer geometries, routings (with dropped and duplicate slots) and token counts."""
    rng = np.random.default_rng(20240611)
    for case in range(24):
        T = int(rng.integers(1, 9))
        H = int(rng.integers(2, 33)) * 32
        I = int(rng.integers(1, 17)) * 32
        E = int(rng.integers(1, 13))
        top_k = int(rng.integers(1, min(E, 8) + 1))
        shared = int(rng.integers(0, 2))
        flavour = "quant" if (H % 64 == 0 and I % 64 == 0 and case % 3 == 0) else "w8"
        lo, hi = (-8, 7) if flavour == "quant" else (-127, 127)
        experts = _experts(rng, H, I, E + shared, lo, hi)
        x = (rng.standard_normal((T, H)) * float(rng.choice([0.01, 1.0, 50.0]))).astype(np.float32)
        ids = rng.integers(0, E, (T, top_k)).astype(np.int32)            # duplicates allowed
        routes = rng.random((T, top_k), dtype=np.float32)
        routes[rng.random((T, top_k)) < 0.2] = 0.0                       # dropped slots
        moe = ops.MoeW8(sess, H, I, E, shared, top_k, 8, experts, flavour=flavour)
        try:
            rc, sync, got = _run_device(sess, moe, x, ids, routes)
            rc2, want = oracle.moe_w8(experts, H, I, E, shared, top_k, ids, routes, input_f32=x)
            what = (case, T, H, I, E, top_k, shared, flavour)
            assert rc == 0 and sync == 0 and rc2 == 0, what
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), what
        finally:
            moe.close()
