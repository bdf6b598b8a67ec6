"""GPU checks of the W8A8 tuning entry points: the assertions the reference's
own tests/test_quant_matmul.cpp:429-600 makes about them (resources fixed from
the masks, measured times, cache value round trip and backend key, joint K
partition of a family, hit / miss accounting, required_k_tile), and that a
returned strategy creates a workspace whose run is exact."""
import ctypes as C
import os
import shutil

import numpy as np
import pytest

from rknpu2_matmul_open_amd import capi, ops

pytestmark = pytest.mark.gpu

M, N, K = 4, 96, 64


def _allowed():
    mask = 0
    for c in os.sched_getaffinity(0):
        if c < 64:
            mask |= 1 << c
    return mask


def _take_cpus(allowed, count):
    """reference tests/test_quant_matmul.cpp:78-85"""
    mask = 0
    for cpu in list(range(4, 8)) + list(range(64)):
        if bin(mask).count("1") < count and allowed & (1 << cpu):
            mask |= 1 << cpu
    return mask


def _cfg(lib, m=M, n=N, k=K):
    cfg = capi.MatmulAutotuneConfig()
    lib.rk_npu_matmul_autotune_config_init(C.byref(cfg), m, n, k)
    cfg.allowed_cpu_core_mask = _allowed()
    cfg.warmup, cfg.loops, cfg.repeats = 0, 2, 1
    return cfg


def test_autotune_each_kind_and_cache_round_trip(sess, tmp_path, monkeypatch):
    lib = sess.lib
    allowed = _allowed()
    threads = min(4, bin(allowed).count("1"))
    cpus = _take_cpus(allowed, threads)
    names = ["rk_npu_i8i8i32_autotune", "rk_npu_f16i8f16_dynamic_autotune", "rk_npu_f16i8f16_static_autotune",
             "rk_npu_f32i8f32_dynamic_autotune", "rk_npu_f32i8f32_static_autotune"]
    cfg = _cfg(lib)
    for kind, name in enumerate(names):
        fast, stable = capi.MatmulStrategy(), capi.MatmulStrategy()
        assert getattr(lib, name)(sess.ctx, C.byref(cfg), C.byref(fast), C.byref(stable)) == 0
        assert fast.op_kind == kind and fast.total_us > 0 and stable.robust_us >= stable.total_us
        assert fast.npu_core_mask == 7 and stable.npu_core_mask == 7
        assert fast.cpu_threads == threads and fast.cpu_core_mask == cpus and stable.cpu_core_mask == cpus
        assert fast.k_tile == K and fast.wave_count == 1
        req = capi.WorkspaceRequirements()
        assert lib.rk_npu_matmul_workspace_memory_query(C.byref(fast), C.byref(req)) == 0
        if kind == capi.I8I8I32:
            path = str(tmp_path / "panel.tune").encode()
            panel = capi.MatmulStrategy.from_buffer_copy(fast)
            panel.a_layout, panel.c_layout = 0, 1  # NORMAL / PANEL8: a value round trip
            loaded, loaded2 = capi.MatmulStrategy(), capi.MatmulStrategy()
            assert lib.rk_npu_matmul_autotune_cache_save(sess.ctx, path, kind, C.byref(cfg), C.byref(panel),
                                                         C.byref(panel)) == 0
            assert lib.rk_npu_matmul_autotune_cache_load(sess.ctx, path, kind, C.byref(cfg), C.byref(loaded),
                                                         C.byref(loaded2)) == 0
            assert loaded.c_layout == 1 and loaded2.c_layout == 1 and loaded.total_us == panel.total_us
            assert bytes(loaded) == bytes(panel)
            # another backend setting, another shape, another kind: all misses
            monkeypatch.setenv("RK_NPU_I8_NPU_REDUCE", "1")
            assert lib.rk_npu_matmul_autotune_cache_load(sess.ctx, path, kind, C.byref(cfg), C.byref(loaded),
                                                         C.byref(loaded2)) == capi.RK_NPU_ERR_CACHE_MISS
            monkeypatch.delenv("RK_NPU_I8_NPU_REDUCE")
            other = _cfg(lib, M + 1)
            assert lib.rk_npu_matmul_autotune_cache_load(sess.ctx, path, kind, C.byref(other), C.byref(loaded),
                                                         C.byref(loaded2)) == capi.RK_NPU_ERR_CACHE_MISS
            assert lib.rk_npu_matmul_autotune_cache_load(sess.ctx, path, 1, C.byref(cfg), C.byref(loaded),
                                                         C.byref(loaded2)) == capi.RK_NPU_ERR_CACHE_MISS
            assert lib.rk_npu_matmul_autotune_cache_load(sess.ctx, str(tmp_path / "absent").encode(), kind,
                                                         C.byref(cfg), C.byref(loaded),
                                                         C.byref(loaded2)) == capi.RK_NPU_ERR_CACHE_MISS
            (tmp_path / "junk.tune").write_text("not a cache file\n")
            assert lib.rk_npu_matmul_autotune_cache_load(sess.ctx, str(tmp_path / "junk.tune").encode(), kind,
                                                         C.byref(cfg), C.byref(loaded),
                                                         C.byref(loaded2)) == capi.RK_NPU_ERR_CACHE_MISS
    # masks: a single allowed core / CPU; N with one 32-wide group
    fixed = _cfg(lib)
    fixed.allowed_cpu_core_mask = _take_cpus(allowed, 1)
    fixed.allowed_npu_core_mask = 4
    fast = capi.MatmulStrategy()
    assert lib.rk_npu_i8i8i32_autotune(sess.ctx, C.byref(fixed), C.byref(fast), None) == 0
    assert fast.npu_core_mask == 4 and fast.cpu_threads == 1 and fast.cpu_core_mask == fixed.allowed_cpu_core_mask
    fixed.N, fixed.allowed_npu_core_mask = 32, 7
    assert lib.rk_npu_i8i8i32_autotune(sess.ctx, C.byref(fixed), C.byref(fast), None) == 0
    assert fast.npu_core_mask == 1 and fast.cpu_threads == 1
    # argument errors
    assert lib.rk_npu_i8i8i32_autotune(sess.ctx, C.byref(fixed), None, None) == capi.RK_NPU_ERR_PARAM
    fixed.loops = 0
    assert lib.rk_npu_i8i8i32_autotune(sess.ctx, C.byref(fixed), C.byref(fast), None) == capi.RK_NPU_ERR_PARAM


def test_cached_tune_and_tuned_strategy_runs_exactly(sess, oracle, tmp_path):
    lib = sess.lib
    cfg = _cfg(lib, 33, 130, 70)
    path = str(tmp_path / "one.tune").encode()
    fast, stable, hit = capi.MatmulStrategy(), capi.MatmulStrategy(), C.c_int(-1)
    assert lib.rk_npu_matmul_autotune_cached(sess.ctx, C.byref(cfg), capi.I8I8I32, path, 0, C.byref(fast),
                                             C.byref(stable), C.byref(hit)) == 0 and hit.value == 0
    again = capi.MatmulStrategy()
    assert lib.rk_npu_matmul_autotune_cached(sess.ctx, C.byref(cfg), capi.I8I8I32, path, 0, C.byref(again), None,
                                             C.byref(hit)) == 0 and hit.value == 1
    assert bytes(again) == bytes(fast)
    assert lib.rk_npu_matmul_autotune_cached(sess.ctx, C.byref(cfg), capi.I8I8I32, path, 1, C.byref(again), None,
                                             C.byref(hit)) == 0 and hit.value == 0  # refresh skips the load
    rng = np.random.default_rng(3)
    A = rng.integers(-128, 128, (33, 70)).astype(np.int8)
    B = rng.integers(-128, 128, (70, 130)).astype(np.int8)
    op = ops.W8A8Linear(sess, capi.I8I8I32, 33, B, strategy=fast)
    try:
        rc, got = op.run(A)
        assert rc == 0 and np.array_equal(got, oracle.gemm_i8(A, B))
    finally:
        op.close()


def test_family_tuning_and_its_cache(sess, tmp_path):
    lib = sess.lib
    ms = (C.c_int * 2)(1, 128)
    freq = (C.c_double * 2)(4.0, 1.0)
    fam = capi.MatmulFamilyAutotuneConfig()
    lib.rk_npu_matmul_family_autotune_config_init(C.byref(fam), N, K, 2, ms)
    fam.frequencies = freq
    fam.allowed_cpu_core_mask = _allowed()
    fam.warmup, fam.loops, fam.repeats = 0, 1, 1
    cache_dir = tmp_path / "family"
    hits, misses = C.c_int(), C.c_int()
    kind = capi.F16I8F16_DYNAMIC
    one = capi.MatmulFamilyAutotuneConfig.from_buffer_copy(fam)
    one.m_count = 1
    s1, st1 = capi.MatmulFamilySummary(), capi.MatmulFamilySummary()
    a1, b1 = (capi.MatmulStrategy * 1)(), (capi.MatmulStrategy * 1)()
    assert lib.rk_npu_matmul_autotune_family_cached(sess.ctx, C.byref(one), kind, str(cache_dir).encode(), 1,
                                                    C.byref(s1), a1, C.byref(st1), b1, C.byref(hits),
                                                    C.byref(misses)) == 0
    assert hits.value == 0 and misses.value > 0
    fs, ss = capi.MatmulFamilySummary(), capi.MatmulFamilySummary()
    fa, sa = (capi.MatmulStrategy * 2)(), (capi.MatmulStrategy * 2)()

    def cached():
        return lib.rk_npu_matmul_autotune_family_cached(sess.ctx, C.byref(fam), kind, str(cache_dir).encode(), 0,
                                                        C.byref(fs), fa, C.byref(ss), sa, C.byref(hits),
                                                        C.byref(misses))

    assert cached() == 0
    assert fs.weight_config.K == K and fs.weight_config.N == N
    assert fa[0].k_tile == fs.weight_config.k_tile == fa[1].k_tile
    assert fa[0].M == 1 and fa[1].M == 128 and fa[1].op_kind == kind
    assert fs.weighted_total_us > 0 and hits.value > 0 and misses.value > 0
    k_tile, total = fs.weight_config.k_tile, fs.weighted_total_us
    assert cached() == 0
    assert hits.value > 0 and misses.value == 0 and fs.weight_config.k_tile == k_tile
    assert fs.weighted_total_us == total
    freq2 = (C.c_double * 2)(1.0, 16.0)
    fam.frequencies = freq2
    assert cached() == 0 and hits.value > 0 and misses.value == 0
    want = (fa[0].total_us * 1.0 + fa[1].total_us * 16.0) / 17.0
    assert abs(fs.weighted_total_us - want) <= 1e-9 * want
    fam.frequencies = freq
    shutil.rmtree(cache_dir)
    assert lib.rk_npu_f32i8f32_dynamic_autotune_family(sess.ctx, C.byref(fam), C.byref(fs), fa, C.byref(ss), sa) == 0
    assert fa[0].op_kind == capi.F32I8F32_DYNAMIC and fa[1].k_tile == fs.weight_config.k_tile
    assert fs.weighted_total_us > 0 and ss.weighted_robust_us >= ss.weighted_total_us
    # a later single-M tune constrained to the family's K partition
    constrained = _cfg(lib, 4, N, K)
    constrained.required_k_tile = fs.weight_config.k_tile
    fast = capi.MatmulStrategy()
    assert lib.rk_npu_f16i8f16_dynamic_autotune(sess.ctx, C.byref(constrained), C.byref(fast), None) == 0
    assert fast.k_tile == fs.weight_config.k_tile
    # argument errors: a summary without its array, duplicate M
    assert lib.rk_npu_i8i8i32_autotune_family(sess.ctx, C.byref(fam), C.byref(fs), None, None,
                                              None) == capi.RK_NPU_ERR_PARAM
    dup = (C.c_int * 2)(8, 8)
    fam.m_values = dup
    assert lib.rk_npu_i8i8i32_autotune_family(sess.ctx, C.byref(fam), C.byref(fs), fa, None,
                                              None) == capi.RK_NPU_ERR_PARAM
