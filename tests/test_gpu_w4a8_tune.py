"""GPU checks of the W4A8 tuning entry points, after the reference's own
tests/test_w4a8_tune.cpp: a tuned strategy creates weights and a workspace whose
f32 and f16 runs are exact (:18-45), the cache replays the same values with no
re-measurement (:46-75), a changed weight code is refused by the tuned factory
(:76-77), a family shares one K partition and reuses single-M cache entries
(:80-93), an explicitly relaxed K tile is honoured (:104), and a profile
captured from weights finds the cache entry without the codes."""
import ctypes as C
import os

import numpy as np
import pytest

from rknpu2_matmul_open_amd import capi

pytestmark = pytest.mark.gpu


def _allowed():
    mask = 0
    for c in os.sched_getaffinity(0):
        if c < 64:
            mask |= 1 << c
    return mask


def _take_cpus(allowed, count):
    mask = 0
    for cpu in list(range(4, 8)) + list(range(64)):
        if bin(mask).count("1") < count and allowed & (1 << cpu):
            mask |= 1 << cpu
    return mask


def _weights(K, N, seed=13):
    rng = np.random.default_rng(seed)
    return rng.integers(-8, 8, size=(K, N), dtype=np.int8), np.full(N, 0.0078125, np.float32)


def _cfg(lib, M, N, K, half=False, multiplier=1.0, required=0):
    c = capi.W4A8AutotuneConfig()
    lib.rk_npu_w4a8_autotune_config_init(C.byref(c), M, N, K)
    c.activation_type = capi.W4A8_F16 if half else capi.W4A8_F32
    c.warmup, c.loops, c.repeats = 0, 1, 1
    c.allowed_cpu_core_mask = _allowed()
    c.k_tile_multiplier = multiplier
    c.required_k_tile = required
    return c


def _verify(sess, oracle, strategy, B, scale):
    """reference tests/test_w4a8_tune.cpp:18-45"""
    lib = sess.lib
    cfg = strategy.config
    w = lib.rk_npu_w4a8_weights_create_tuned(sess.domain, C.byref(strategy), capi.ptr(B), capi.ptr(scale))
    ws = lib.rk_npu_w4a8_workspace_create(sess.domain, C.byref(cfg))
    try:
        assert w and ws and 0 <= cfg.pipeline <= 2
        info = capi.W4A8WeightInfo()
        assert lib.rk_npu_w4a8_weights_query(w, C.byref(info)) == 0
        assert (info.config.K, info.config.N, info.config.k_tile, info.safe_k_tile, info.bound_relaxed) == (
            cfg.K, cfg.N, cfg.k_tile, strategy.weights.safe_k_tile, strategy.weights.bound_relaxed)
        a = ((np.arange(cfg.M * cfg.K) % 23).astype(np.float32) - 11).reshape(cfg.M, cfg.K) * np.float32(0.0625)
        ah = oracle.float_to_half(a)
        out = np.empty((cfg.M, cfg.N), np.float32)
        oh = np.empty((cfg.M, cfg.N), np.uint16)
        assert lib.rk_npu_w4a8_run_f32(ws, w, capi.ptr(a), capi.ptr(out), None) == 0
        assert lib.rk_npu_w4a8_run_f16(ws, w, capi.ptr(ah), capi.ptr(oh), None) == 0
        want = oracle.w4a8(a, B, scale)
        want_h = oracle.w4a8(ah, B, scale)
        assert want["rc"] == 0 and want_h["rc"] == 0
        assert np.array_equal(out.view(np.uint32), want["C"].view(np.uint32))
        assert np.array_equal(oh, want_h["C"])
    finally:
        lib.rk_npu_w4a8_workspace_free(ws)
        lib.rk_npu_w4a8_weights_free(w)


@pytest.mark.parametrize("M,K,N,half,multiplier,required", [
    (3, 257, 193, False, 1.0, 0),
    (1, 8193, 193, False, 1.0, 480),
    (1, 1057, 193, True, 1.0, 480),
    (65, 1057, 257, True, 1.0, 0),
    (4, 4096, 193, False, 2.1, 0),
])
def test_tune_cache_replay_and_tuned_factories(sess, oracle, tmp_path, M, K, N, half, multiplier, required):
    lib = sess.lib
    B, scale = _weights(K, N)
    c = _cfg(lib, M, N, K, half, multiplier, required)
    path = str(tmp_path / "entry").encode()
    fast, stable = capi.W4A8Strategy(), capi.W4A8Strategy()
    hit = C.c_int(-1)
    assert lib.rk_npu_w4a8_autotune_cached(sess.ctx, C.byref(c), capi.ptr(B), capi.ptr(scale), path, 1, C.byref(fast),
                                           C.byref(stable), C.byref(hit)) == 0 and hit.value == 0
    allowed = _allowed()
    threads = min(4, bin(allowed).count("1"))
    for s in (fast, stable):
        assert (s.config.M, s.config.N, s.config.K) == (M, N, K)
        assert s.cpu_core_mask == _take_cpus(allowed, threads) and s.config.cpu_threads == threads
        assert s.config.npu_core_mask == 7 and s.activation_type == c.activation_type
        assert s.total_us > 0 and s.robust_us >= s.total_us and s.tuning_revision == 5
        assert s.weights.config.k_tile == s.config.k_tile and s.weights.multiplier == multiplier
        if required:
            assert s.config.k_tile == required
        if multiplier == 1.0:
            assert not s.weights.bound_relaxed and s.config.k_tile <= s.weights.safe_k_tile
        _verify(sess, oracle, s, B, scale)
    if multiplier > 1:
        # random codes in [-8, 7] certify about 1000 deep: the widest permitted tile is a relaxed one
        safe = fast.weights.safe_k_tile
        assert fast.weights.bound_relaxed == 1 and safe < fast.config.k_tile == min(2048, int(safe * 2.1) // 32 * 32)
    total = fast.total_us
    # replay: same values, no measurement
    assert lib.rk_npu_w4a8_autotune_cached(sess.ctx, C.byref(c), capi.ptr(B), capi.ptr(scale), path, 0, C.byref(fast),
                                           C.byref(stable), C.byref(hit)) == 0 and hit.value == 1
    assert fast.total_us == total
    f2, s2 = capi.W4A8Strategy(), capi.W4A8Strategy()
    assert lib.rk_npu_w4a8_autotune_cache_load(sess.ctx, C.byref(c), capi.ptr(B), capi.ptr(scale), path, C.byref(f2),
                                               C.byref(s2)) == 0
    assert bytes(f2) == bytes(fast) and bytes(s2) == bytes(stable)
    # the entry belongs to these weights, this shape and this policy
    changed = B.copy()
    changed[0, 0] = 6 if changed[0, 0] == 7 else changed[0, 0] + 1
    assert lib.rk_npu_w4a8_autotune_cache_load(sess.ctx, C.byref(c), capi.ptr(changed), capi.ptr(scale), path,
                                               C.byref(f2), C.byref(s2)) == capi.RK_NPU_ERR_CACHE_MISS
    assert not lib.rk_npu_w4a8_weights_create_tuned(sess.domain, C.byref(fast), capi.ptr(changed), capi.ptr(scale))
    other = _cfg(lib, M, N, K, not half, multiplier, required)
    assert lib.rk_npu_w4a8_autotune_cache_load(sess.ctx, C.byref(other), capi.ptr(B), capi.ptr(scale), path,
                                               C.byref(f2), C.byref(s2)) == capi.RK_NPU_ERR_CACHE_MISS
    # the legacy and the extended search have separate identities
    fx, sx = capi.W4A8StrategyEx(), capi.W4A8StrategyEx()
    assert lib.rk_npu_w4a8_autotune_cache_load_ex(sess.ctx, C.byref(c), capi.ptr(B), capi.ptr(scale), path, C.byref(fx),
                                                  C.byref(sx)) == capi.RK_NPU_ERR_CACHE_MISS
    # save under a new name, load it back
    path2 = str(tmp_path / "copy").encode()
    assert lib.rk_npu_w4a8_autotune_cache_save(sess.ctx, C.byref(c), capi.ptr(B), capi.ptr(scale), path2,
                                               C.byref(fast), C.byref(stable)) == 0
    assert lib.rk_npu_w4a8_autotune_cache_load(sess.ctx, C.byref(c), capi.ptr(B), capi.ptr(scale), path2, C.byref(f2),
                                               C.byref(s2)) == 0 and bytes(f2) == bytes(fast)
    broken = capi.W4A8Strategy.from_buffer_copy(bytes(fast))
    broken.config.k_tile += 32
    assert lib.rk_npu_w4a8_autotune_cache_save(sess.ctx, C.byref(c), capi.ptr(B), capi.ptr(scale), path2,
                                               C.byref(broken), C.byref(stable)) == capi.RK_NPU_ERR_PARAM


def test_extended_strategy_profile_lookup_and_tuned_workspace(sess, oracle, tmp_path):
    lib = sess.lib
    M, K, N = 5, 513, 129
    B, scale = _weights(K, N, seed=5)
    c = _cfg(lib, M, N, K, multiplier=1.0)
    path = str(tmp_path / "ex").encode()
    fast, stable = capi.W4A8StrategyEx(), capi.W4A8StrategyEx()
    hit = C.c_int(-1)
    assert lib.rk_npu_w4a8_autotune_cached_ex(sess.ctx, C.byref(c), capi.ptr(B), capi.ptr(scale), path, 0,
                                              C.byref(fast), C.byref(stable), C.byref(hit)) == 0 and hit.value == 0
    assert (fast.execution.struct_size, fast.execution.input_layout, fast.execution.reduce_backend) == (
        C.sizeof(capi.W4A8Options), 0, 0)
    w = lib.rk_npu_w4a8_weights_create_tuned_ex(sess.domain, C.byref(fast), capi.ptr(B), capi.ptr(scale))
    ws = lib.rk_npu_w4a8_workspace_create_tuned_ex(sess.domain, C.byref(fast))
    assert w and ws
    try:
        a = np.random.default_rng(1).standard_normal((M, K)).astype(np.float32)
        out = np.empty((M, N), np.float32)
        assert lib.rk_npu_w4a8_run_f32(ws, w, capi.ptr(a), capi.ptr(out), None) == 0
        assert np.array_equal(out.view(np.uint32), oracle.w4a8(a, B, scale)["C"].view(np.uint32))
        # a profile captured from the weights finds the entry without codes, scales or device work
        prof = lib.rk_npu_w4a8_tuning_profile_from_weights(w)
        assert prof and lib.rk_npu_w4a8_tuning_profile_fingerprint(prof) == fast.base.weight_fingerprint != 0
        f2, s2 = capi.W4A8StrategyEx(), capi.W4A8StrategyEx()
        assert lib.rk_npu_w4a8_autotune_cache_load_profile_ex(sess.ctx, C.byref(c), prof, path, C.byref(f2),
                                                              C.byref(s2)) == 0
        assert bytes(f2) == bytes(fast)
        env = _cfg(lib, M, N, K, multiplier=0.0)  # "read the environment" is not an explicit policy
        assert lib.rk_npu_w4a8_autotune_cache_load_profile_ex(sess.ctx, C.byref(env), prof, path, C.byref(f2),
                                                              C.byref(s2)) == capi.RK_NPU_ERR_PARAM
        lib.rk_npu_w4a8_tuning_profile_free(prof)
    finally:
        lib.rk_npu_w4a8_workspace_free(ws)
        lib.rk_npu_w4a8_weights_free(w)
    stale = capi.W4A8StrategyEx.from_buffer_copy(bytes(fast))
    stale.base.tuning_revision = 4
    assert not lib.rk_npu_w4a8_workspace_create_tuned_ex(sess.domain, C.byref(stale))


def test_family_shares_one_k_partition_and_reuses_entries(sess, tmp_path):
    """reference tests/test_w4a8_tune.cpp:80-93"""
    lib = sess.lib
    K, N = 513, 193
    ms = (C.c_int * 3)(1, 4, 32)
    freq = (C.c_double * 3)(1, 2, 1)
    B = np.ones((K, N), np.int8)
    scale = np.full(N, 0.01, np.float32)
    f = capi.W4A8FamilyConfig()
    lib.rk_npu_w4a8_family_config_init(C.byref(f), N, K, 1, ms)
    f.base.warmup, f.base.loops, f.base.repeats = 0, 1, 1
    f.base.allowed_cpu_core_mask = _allowed()
    f.frequencies = freq
    directory = str(tmp_path / "family").encode()
    fast, stable = capi.W4A8FamilySummary(), capi.W4A8FamilySummary()
    fs, ss = (capi.W4A8Strategy * 3)(), (capi.W4A8Strategy * 3)()
    hits, misses = C.c_int(0), C.c_int(0)

    def run():
        return lib.rk_npu_w4a8_autotune_family_cached(sess.ctx, C.byref(f), capi.ptr(B), capi.ptr(scale), directory, 0,
                                                      C.byref(fast), fs, C.byref(stable), ss, C.byref(hits),
                                                      C.byref(misses))
    assert run() == 0 and hits.value == 0 and misses.value > 0
    f.m_count = 3
    assert run() == 0 and hits.value > 0 and misses.value > 0
    assert run() == 0 and hits.value > 0 and misses.value == 0
    before = fast.weighted_total_us
    freq[0] = 100
    assert run() == 0 and hits.value > 0 and misses.value == 0
    assert fast.weighted_total_us != before or fs[0].total_us == fs[1].total_us == fs[2].total_us
    for i in range(3):
        assert fs[i].config.M == ms[i] and fs[i].config.k_tile == fast.weights.config.k_tile
        assert ss[i].config.k_tile == stable.weights.config.k_tile and 0 <= fs[i].config.pipeline <= 2
    assert fast.weight_fingerprint == fs[0].weight_fingerprint != 0
    want = sum(w * fs[i].total_us for i, w in enumerate((100, 2, 1))) / 103
    assert abs(fast.weighted_total_us - want) <= 1e-9 * want
    # uncached family, extended strategies
    fsx = (capi.W4A8StrategyEx * 3)()
    assert lib.rk_npu_w4a8_autotune_family_ex(sess.ctx, C.byref(f), capi.ptr(B), capi.ptr(scale), C.byref(fast), fsx,
                                              None, None) == 0
    assert fsx[2].base.config.M == 32 and fsx[2].execution.struct_size == C.sizeof(capi.W4A8Options)
    dup = (C.c_int * 3)(1, 4, 4)
    f.m_values = dup
    assert run() == capi.RK_NPU_ERR_PARAM


def test_policy_rejections(sess):
    """reference src/rk_npu_w4a8_tune_policy.cpp:37-45,68 and tests/test_w4a8_tune.cpp:104-108"""
    lib = sess.lib
    K, N = 1024, 64
    B = np.full((K, N), -8, np.int8)
    scale = np.ones(N, np.float32)
    s = capi.W4A8Strategy()

    def tune(c, codes=B, scales=scale):
        return lib.rk_npu_w4a8_autotune(sess.ctx, C.byref(c), capi.ptr(codes), capi.ptr(scales), C.byref(s), None)
    # all -8: 480 is the widest certified tile (512 * 64 = 32768 > 32767)
    c = _cfg(lib, 3, N, K)
    assert tune(c) == 0 and s.weights.safe_k_tile == 480 and s.config.k_tile == 480 and not s.weights.bound_relaxed
    c = _cfg(lib, 3, N, K, required=512)
    assert tune(c) == capi.RK_NPU_ERR_PARAM            # not certified and not relaxed
    c = _cfg(lib, 3, N, K, multiplier=1.5, required=736)
    assert tune(c) == capi.RK_NPU_ERR_PARAM            # beyond 480 * 1.5 = 720 -> limit 704
    c = _cfg(lib, 3, N, K, multiplier=1.5, required=704)
    # The NPU saturates its INT16 partials on this tile and the reference rejects it after its sample run;
    # accumulation is int32 here, the result is exact and the relaxed strategy is returned as such.
    assert tune(c) == 0 and s.config.k_tile == 704 and s.weights.bound_relaxed == 1
    for field, value in (("required_k_tile", 48), ("k_tile_multiplier", 0.5), ("loops", 0), ("repeats", 0),
                         ("warmup", -1), ("timeout_ms", 0), ("allowed_npu_core_mask", 8), ("activation_type", 2)):
        c = _cfg(lib, 3, N, K)
        setattr(c, field, value)
        assert tune(c) == capi.RK_NPU_ERR_PARAM, field
    bad = B.copy()
    bad[5, 5] = 8
    assert tune(_cfg(lib, 3, N, K), codes=bad) == capi.RK_NPU_ERR_PARAM
    bad_scale = scale.copy()
    bad_scale[3] = 0
    assert tune(_cfg(lib, 3, N, K), scales=bad_scale) == capi.RK_NPU_ERR_PARAM
    c = _cfg(lib, 3, N, K)
    assert lib.rk_npu_w4a8_autotune(sess.ctx, C.byref(c), capi.ptr(B), capi.ptr(scale), None, None) == capi.RK_NPU_ERR_PARAM
