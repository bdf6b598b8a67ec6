"""The C-ABI boundary without a GPU: headers are valid C99, the shared library
loads and exports every function the headers declare, struct layouts seen by a
C compiler equal the ctypes mirror, defaults and the CPU-only queries return
the numbers the reference's own tests pin, and opening a context on a machine
without a device fails cleanly (no compute path is entered)."""
import ctypes as C
import os
import re
import subprocess
import sys

import numpy as np
import pytest

from rknpu2_matmul_open_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")
HEADERS = ["rk_npu_common.h", "rk_npu_quant_matmul.h", "rk_npu_matmul_i4.h", "rk_npu_w4a8.h",
           "rk_npu_w4a8_tune.h", "rk_npu_moe_w8.h", "rk_npu_hip.h"]


@pytest.fixture(scope="module")
def lib():
    return capi.load_library()


def _declared_functions():
    names = set()
    for h in HEADERS:
        text = open(os.path.join(INC, h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        for m in re.finditer(r"\b(rk_npu_[a-z0-9_]+)\s*\(", text):
            names.add(m.group(1))
    return names


def test_headers_compile_as_c99(tmp_path):
    """reference tests/test_quant_header.c, test_w4a8_header.c, test_moe_w8_header.c:
    plain-C translation units keep the headers valid C."""
    for h in HEADERS:
        src = tmp_path / (h + ".c")
        src.write_text('#include "%s"\nint main(void) { return 0; }\n' % h)
        subprocess.check_call(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-I", INC, "-c", str(src),
                               "-o", str(tmp_path / "o.o")])


def test_library_exports_every_declared_function(lib):
    declared = _declared_functions()
    assert len(declared) > 60
    missing = [n for n in sorted(declared) if not hasattr(lib, n)]
    assert not missing, missing
    # and the ctypes mirror binds exactly those
    assert set(capi.EXPORTED_SYMBOLS) == declared


def test_struct_layouts_match_the_c_compiler(tmp_path):
    pairs = [("rk_npu_matmul_strategy", capi.MatmulStrategy), ("rk_npu_matmul_autotune_config", capi.MatmulAutotuneConfig),
             ("rk_npu_matmul_weight_config", capi.MatmulWeightConfig),
             ("rk_npu_matmul_family_autotune_config", capi.MatmulFamilyAutotuneConfig),
             ("rk_npu_matmul_family_summary", capi.MatmulFamilySummary),
             ("rk_npu_matmul_workspace_requirements", capi.WorkspaceRequirements),
             ("rk_npu_matmul_weight_requirements", capi.WeightRequirements),
             ("rk_npu_i4_weight_config", capi.I4WeightConfig), ("rk_npu_i4_memory_info", capi.I4MemoryInfo),
             ("rk_npu_i4_config", capi.I4Config), ("rk_npu_i4_timings", capi.I4Timings),
             ("rk_npu_i4_input_tile", capi.I4InputTile),
             ("rk_npu_w4a8_config", capi.W4A8Config), ("rk_npu_w4a8_memory_info", capi.W4A8MemoryInfo),
             ("rk_npu_w4a8_options", capi.W4A8Options), ("rk_npu_w4a8_memory_info_ex", capi.W4A8MemoryInfoEx),
             ("rk_npu_w4a8_timings", capi.W4A8Timings), ("rk_npu_w4a8_weight_info", capi.W4A8WeightInfo),
             ("rk_npu_w4a8_ffn_timings", capi.W4A8FfnTimings),
             ("rk_npu_w4a8_autotune_config", capi.W4A8AutotuneConfig), ("rk_npu_w4a8_strategy", capi.W4A8Strategy),
             ("rk_npu_w4a8_strategy_ex", capi.W4A8StrategyEx), ("rk_npu_w4a8_family_config", capi.W4A8FamilyConfig),
             ("rk_npu_w4a8_family_summary", capi.W4A8FamilySummary),
             ("rk_npu_moe_w8_weight_config", capi.MoeWeightConfig), ("rk_npu_moe_w8_config", capi.MoeConfig),
             ("rk_npu_moe_w8_expert", capi.MoeExpert), ("rk_npu_moe_w8_timings", capi.MoeTimings),
             ("rk_npu_moe_import_timings", capi.MoeImportTimings),
             ("rk_npu_domain_memory_stats", capi.DomainMemoryStats)]
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "rk_npu_hip.h"', '#include "rk_npu_w4a8_tune.h"',
             "int main(void) {"]
    for cname, ct in pairs:
        lines.append('printf("%s %%zu", sizeof(%s));' % (cname, cname))
        for fname, _ in ct._fields_:
            lines.append('printf(" %%zu", offsetof(%s, %s));' % (cname, fname))
        lines.append('printf("\\n");')
    lines.append("return 0; }")
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c99", "-I", INC, str(src), "-o", str(exe)])
    out = subprocess.check_output([str(exe)]).decode().splitlines()
    for line, (cname, ct) in zip(out, pairs):
        parts = line.split()
        assert parts[0] == cname
        assert int(parts[1]) == C.sizeof(ct), cname
        for off, (fname, _) in zip(parts[2:], ct._fields_):
            assert int(off) == getattr(ct, fname).offset, (cname, fname)


def test_error_codes_and_strings(lib):
    assert (capi.RK_NPU_OK, capi.RK_NPU_ERR_OPEN, capi.RK_NPU_ERR_IOCTL, capi.RK_NPU_ERR_PARAM,
            capi.RK_NPU_ERR_NOMEM, capi.RK_NPU_ERR_SUBMIT, capi.RK_NPU_ERR_BUSY, capi.RK_NPU_ERR_DOMAIN,
            capi.RK_NPU_ERR_IO, capi.RK_NPU_ERR_CACHE_MISS) == (0, -1, -2, -3, -4, -5, -6, -7, -8, -9)
    assert lib.rk_npu_strerror(0) == b"ok"
    assert lib.rk_npu_strerror(-3) == b"bad argument"
    assert lib.rk_npu_strerror(-6) == b"workspace is already running"
    assert lib.rk_npu_strerror(-9) == b"tuning cache miss"
    assert lib.rk_npu_strerror(-77) == b"unknown error"
    assert len({lib.rk_npu_strerror(c) for c in range(0, -10, -1)}) == 10


def test_defaults_of_config_init(lib):
    """reference src/rk_npu_w4a8.cpp:162-168, src/rk_npu_moe_w8.cpp:824-826,
    src/rk_npu_quant_matmul.cpp:1522-1535."""
    w = capi.W4A8Config()
    lib.rk_npu_w4a8_config_init(C.byref(w), 7, 65, 513)
    assert (w.M, w.N, w.K, w.m_tile, w.k_tile, w.n_tile, w.npu_core_mask, w.timeout_ms, w.pipeline,
            w.cpu_threads) == (7, 65, 513, 64, 480, 1024, 1, 500, 1, 1)
    o = capi.W4A8Options()
    lib.rk_npu_w4a8_options_init(C.byref(o))
    assert (o.struct_size, o.input_layout, o.reduce_backend) == (C.sizeof(capi.W4A8Options), 0, 0)
    m = capi.MoeConfig()
    lib.rk_npu_moe_w8_config_init(C.byref(m), 2048, 512, 64, 1, 8, 256)
    assert (m.struct_size, m.weights.hidden, m.weights.intermediate, m.weights.routed_experts,
            m.weights.shared_expert, m.max_rows, m.top_k, m.npu_cores, m.cpu_threads, m.native_input,
            m.middle, m.timeout_ms) == (C.sizeof(capi.MoeConfig), 2048, 512, 64, 1, 256, 8, 3, 4, 0, 0, 1000)
    a = capi.MatmulAutotuneConfig()
    lib.rk_npu_matmul_autotune_config_init(C.byref(a), 3, 4, 5)
    assert (a.M, a.N, a.K, a.allowed_npu_core_mask, a.allowed_cpu_core_mask, a.warmup, a.loops, a.repeats,
            a.timeout_ms, a.verbose, a.required_k_tile) == (3, 4, 5, 7, 0, 2, 8, 3, 500, 0, 0)
    lib.rk_npu_w4a8_config_init(None, 1, 1, 1)   # NULL is ignored
    lib.rk_npu_moe_w8_config_init(None, 1, 1, 1, 0, 1, 1)


def test_w4a8_memory_query_pins(lib):
    """reference tests/test_w4a8_cpu.cpp:143-152 and tests/test_w4a8_reduction.cpp:112-119."""
    cfg = capi.W4A8Config()
    lib.rk_npu_w4a8_config_init(C.byref(cfg), 3, 65, 513)
    mem = capi.W4A8MemoryInfo()
    assert lib.rk_npu_w4a8_memory_query(C.byref(cfg), C.byref(mem)) == 0
    assert mem.weight_metadata_bytes == 65 * 8 == 520
    assert mem.cpu_scratch_bytes == 3 * 128 * 4 + 3 * 8 == 1560
    assert mem.backend.wave_count == 2 and mem.backend.packed_weight_bytes == 544 * 128 // 2
    cfg.m_tile = 65
    assert lib.rk_npu_w4a8_memory_query(C.byref(cfg), C.byref(mem)) == capi.RK_NPU_ERR_PARAM
    cfg.m_tile = 64
    cfg.K = (2 ** 31 - 1) // 1024 + 1
    assert lib.rk_npu_w4a8_memory_query(C.byref(cfg), C.byref(mem)) == capi.RK_NPU_ERR_PARAM
    lib.rk_npu_w4a8_config_init(C.byref(cfg), 128, 4096, 11008)
    ex = capi.W4A8MemoryInfoEx()
    assert lib.rk_npu_w4a8_memory_query_ex(C.byref(cfg), None, C.byref(ex)) == 0
    assert ex.base.backend.partial_bytes == 2 * 256 * 4096 * 2 == 4194304
    assert ex.effective_reduce_backend == capi.W4A8_REDUCE_CPU
    # option handling: NPU reduce is effective only for M > 16; CHAIN + NPU reduce is rejected
    opt = capi.W4A8Options()
    lib.rk_npu_w4a8_options_init(C.byref(opt))
    opt.reduce_backend = capi.W4A8_REDUCE_NPU
    assert lib.rk_npu_w4a8_memory_query_ex(C.byref(cfg), C.byref(opt), C.byref(ex)) == 0
    assert ex.effective_reduce_backend == capi.W4A8_REDUCE_NPU
    cfg.pipeline = capi.W4A8_CHAIN
    assert lib.rk_npu_w4a8_memory_query_ex(C.byref(cfg), C.byref(opt), C.byref(ex)) == capi.RK_NPU_ERR_PARAM
    cfg.pipeline = capi.W4A8_PIPELINED
    cfg.M = 16
    assert lib.rk_npu_w4a8_memory_query_ex(C.byref(cfg), C.byref(opt), C.byref(ex)) == 0
    assert ex.effective_reduce_backend == capi.W4A8_REDUCE_CPU
    opt.struct_size = 3
    assert lib.rk_npu_w4a8_memory_query_ex(C.byref(cfg), C.byref(opt), C.byref(ex)) == capi.RK_NPU_ERR_PARAM
    for field, bad in (("k_tile", 0), ("k_tile", 48), ("k_tile", 2080), ("n_tile", 32), ("n_tile", 100),
                       ("n_tile", 8192), ("npu_core_mask", 5), ("npu_core_mask", 0), ("timeout_ms", 0),
                       ("cpu_threads", 0), ("cpu_threads", 5), ("pipeline", 3), ("M", 0), ("N", 0)):
        lib.rk_npu_w4a8_config_init(C.byref(cfg), 8, 256, 512)
        setattr(cfg, field, bad)
        assert lib.rk_npu_w4a8_memory_query(C.byref(cfg), C.byref(mem)) == capi.RK_NPU_ERR_PARAM, (field, bad)
    lib.rk_npu_w4a8_config_init(C.byref(cfg), 8, 64, 512)
    cfg.npu_core_mask = 3     # two cores need two 64-column blocks
    assert lib.rk_npu_w4a8_memory_query(C.byref(cfg), C.byref(mem)) == capi.RK_NPU_ERR_PARAM


def test_w8_memory_queries_and_k_partition(lib):
    """reference tests/test_quant_matmul.cpp:239-254 (M=8, N=K=96) and
    src/rk_npu_quant_matmul.cpp:1131-1142 (partition policy)."""
    from rknpu2_matmul_open_amd.ops import default_strategy
    M, N, K = 8, 96, 96
    for k_tile, waves in ((K, 1), (32, 3)):
        s = default_strategy(capi.I8I8I32, M, N, K, k_tile=k_tile, n_tile=32 if k_tile == 32 else N)
        if k_tile == 32:
            s.npu_core_mask = 7
        req = capi.WorkspaceRequirements()
        assert lib.rk_npu_matmul_workspace_memory_query(C.byref(s), C.byref(req)) == 0
        assert req.wave_count == waves
        assert req.input_bytes == min(waves, 2) * M * ((min(k_tile, K) + 31) // 32 * 32)
        assert req.output_bytes == min(waves, 3) * M * N * 4
        assert req.buffer_count == 2 * waves + min(waves, 2) + min(waves, 3)
        wc = capi.MatmulWeightConfig(K, N, k_tile)
        wr = capi.WeightRequirements()
        assert lib.rk_npu_i8i8i32_weights_memory_query(C.byref(wc), C.byref(wr)) == 0
        assert (wr.packed_b_bytes, wr.scale_bytes, wr.buffer_count, wr.wave_count) == (K * N, 0, 1, waves)
        assert lib.rk_npu_f16i8f16_weights_memory_query(C.byref(wc), C.byref(wr)) == 0
        assert wr.scale_bytes == N * 4 and wr.bytes == K * N + N * 4
    bad = default_strategy(capi.I8I8I32, M, N, K)
    for field, v in (("k_tile", 0), ("k_tile", K + 1), ("n_tile", 3073), ("npu_core_mask", 5),
                     ("cpu_threads", 2), ("cpu_core_mask", 0), ("a_layout", 4), ("c_layout", 3), ("op_kind", 9)):
        s = default_strategy(capi.I8I8I32, M, N, K)
        setattr(s, field, v)
        req = capi.WorkspaceRequirements()
        assert lib.rk_npu_matmul_workspace_memory_query(C.byref(s), C.byref(req)) == capi.RK_NPU_ERR_PARAM, field
    q = lib.rk_npu_matmul_k_partition_query
    assert q(0, 10, 10) == q(1, 0, 1) == q(1, 10, 11) == capi.RK_NPU_ERR_PARAM
    assert q(4, 8192, 3100) == 0                          # M <= 4 always eligible
    assert q(8, 8192, 2560) == capi.RK_NPU_ERR_PARAM      # split with a tile > 2048 not 1024-aligned
    assert q(8, 8192, 3072) == 0
    assert q(8, 3500, 3500) == capi.RK_NPU_ERR_PARAM      # a wave in (3072, 4096)
    assert q(8, 4096, 4096) == 0 and q(128, 4096, 2048) == 0


def test_open_without_device_fails_cleanly(lib):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    assert not lib.rk_npu_open(None)
    assert not lib.rk_npu_open(b"/dev/dri/renderD128")
    assert not lib.rk_npu_open(b"hip:")
    # NULL handles are tolerated by every free / close
    lib.rk_npu_close(None)
    lib.rk_npu_iommu_domain_free(None)
    lib.rk_npu_matmul_workspace_free(None)
    lib.rk_npu_i8i8i32_weights_free(None)
    lib.rk_npu_f16i8f16_weights_free(None)
    lib.rk_npu_f32i8f32_weights_free(None)
    lib.rk_npu_w4a8_weights_free(None)
    lib.rk_npu_w4a8_workspace_free(None)
    lib.rk_npu_moe_w8_weights_free(None)
    lib.rk_npu_moe_w8_workspace_free(None)
    assert lib.rk_npu_iommu_domain_id(None) == 0xFFFFFFFF
    assert not lib.rk_npu_iommu_domain_create(None, 0)
    assert lib.rk_npu_moe_w8_weights_device_bytes(None) == 0
    # NULL handles in run calls are argument errors, not crashes
    assert lib.rk_npu_i8i8i32_run(None, None, None, None) == capi.RK_NPU_ERR_PARAM
    assert lib.rk_npu_w4a8_run_f32(None, None, None, None, None) == capi.RK_NPU_ERR_PARAM
    assert lib.rk_npu_moe_w8_run_f32(None, None, 1, None, None, None, None, None) == capi.RK_NPU_ERR_PARAM


def test_autotune_entry_points_without_a_context(lib):
    """reference src/rk_npu_quant_matmul.cpp:1536-1550 (family defaults) and the
    argument checks every tuning / cache call makes before touching a device."""
    ms = (C.c_int * 2)(1, 128)
    fam = capi.MatmulFamilyAutotuneConfig()
    lib.rk_npu_matmul_family_autotune_config_init(C.byref(fam), 96, 64, 2, ms)
    assert (fam.K, fam.N, fam.m_count, fam.allowed_npu_core_mask, fam.allowed_cpu_core_mask) == (64, 96, 2, 7, 0)
    assert (fam.warmup, fam.loops, fam.repeats, fam.timeout_ms, fam.verbose) == (2, 8, 3, 500, 0)
    assert not fam.frequencies and fam.m_values[1] == 128
    lib.rk_npu_matmul_family_autotune_config_init(None, 1, 1, 0, None)
    cfg = capi.MatmulAutotuneConfig()
    lib.rk_npu_matmul_autotune_config_init(C.byref(cfg), 4, 96, 64)
    s1, s2 = capi.MatmulStrategy(), capi.MatmulStrategy()
    P = capi.RK_NPU_ERR_PARAM
    assert lib.rk_npu_i8i8i32_autotune(None, C.byref(cfg), C.byref(s1), C.byref(s2)) == P
    assert lib.rk_npu_matmul_autotune_cache_load(None, b"/tmp/x.tune", 0, C.byref(cfg), C.byref(s1), C.byref(s2)) == P
    assert lib.rk_npu_matmul_autotune_cache_save(None, b"/tmp/x.tune", 0, C.byref(cfg), C.byref(s1), C.byref(s2)) == P
    assert lib.rk_npu_matmul_autotune_cached(None, C.byref(cfg), 0, None, 0, C.byref(s1), C.byref(s2), None) == P
    summ = capi.MatmulFamilySummary()
    arr = (capi.MatmulStrategy * 2)()
    assert lib.rk_npu_f16i8f16_dynamic_autotune_family(None, C.byref(fam), C.byref(summ), arr, None, None) == P
    hits, misses = C.c_int(5), C.c_int(5)
    assert lib.rk_npu_matmul_autotune_family_cached(None, C.byref(fam), 1, None, 0, C.byref(summ), arr, None, None,
                                                    C.byref(hits), C.byref(misses)) == P
    assert (hits.value, misses.value) == (0, 0)
    wc = capi.MatmulWeightConfig(64, 96, 64)
    w = np.zeros((64, 96), np.float32)
    assert not lib.rk_npu_f16i8f16_weights_create_from_f32_compress(None, C.byref(wc), capi.ptr(w), 4.0)
    assert not lib.rk_npu_f32i8f32_weights_create_from_f32_compress(None, C.byref(wc), capi.ptr(w), 4.0)


def test_int4_moe_entry_points_without_a_device(lib):
    """W4 / mixed / slot-bank / packed-record entry points of the reference
    (include/rk_npu_moe_w8.h:83-143): refused without a domain or handle, buffers untouched."""
    cfg = capi.MoeWeightConfig(64, 64, 3, 1)
    full = capi.MoeConfig()
    lib.rk_npu_moe_w8_config_init(C.byref(full), 64, 64, 3, 1, 2, 8)
    for fn in (lib.rk_npu_moe_quant_weights_create, lib.rk_npu_moe_quant_weights_create_full_k,
               lib.rk_npu_moe_w4_weights_create, lib.rk_npu_moe_w4_slots_create):
        assert not fn(None, C.byref(cfg), None)
    assert not lib.rk_npu_moe_quant_slots_create(None, C.byref(cfg))
    assert not lib.rk_npu_moe_quant_workspace_create(None, C.byref(full))
    assert not lib.rk_npu_moe_w4_workspace_create(None, C.byref(full))
    assert lib.rk_npu_moe_quant_expert_blob_bytes(None) == 0
    buf = np.full(64, 7, np.uint8)
    assert lib.rk_npu_moe_quant_export_expert(None, 0, capi.ptr(buf), 64) == capi.RK_NPU_ERR_PARAM
    assert lib.rk_npu_moe_quant_import_expert(None, 0, capi.ptr(buf), 64) == capi.RK_NPU_ERR_PARAM
    assert lib.rk_npu_moe_quant_import_expert_timed(None, 0, capi.ptr(buf), 64, None) == capi.RK_NPU_ERR_PARAM
    assert lib.rk_npu_moe_quant_swap_slots(None, 0, None, 0) == capi.RK_NPU_ERR_PARAM
    assert (buf == 7).all()


def test_package_fails_loudly_without_the_library(monkeypatch, tmp_path):
    monkeypatch.setenv("RK_NPU_MATMUL_LIB", str(tmp_path / "missing.so"))
    monkeypatch.setattr(capi, "_LIB", None)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        capi.load_library()


def test_w4a8_tune_entry_points_without_a_context(lib):
    """reference src/rk_npu_w4a8_tune_policy.cpp:178-185 (defaults) and the NULL / argument checks of
    src/rk_npu_w4a8_tune.cpp:124-127, src/rk_npu_w4a8_tune_cache.cpp:71,88,111,
    src/rk_npu_w4a8_tune_family.cpp:14-15: every entry point refuses before touching a device."""
    c = capi.W4A8AutotuneConfig()
    lib.rk_npu_w4a8_autotune_config_init(C.byref(c), 3, 193, 257)
    assert (c.M, c.N, c.K, c.activation_type, c.allowed_npu_core_mask, c.allowed_cpu_core_mask, c.warmup, c.loops,
            c.repeats, c.timeout_ms, c.verbose, c.required_k_tile, c.k_tile_multiplier) == (
                3, 193, 257, capi.W4A8_F32, 7, 0, 2, 8, 3, 500, 0, 0, 0.0)
    ms = (C.c_int * 2)(1, 4)
    f = capi.W4A8FamilyConfig()
    lib.rk_npu_w4a8_family_config_init(C.byref(f), 193, 257, 2, ms)
    assert (f.base.M, f.base.N, f.base.K, f.m_count, f.m_values[1], bool(f.frequencies)) == (1, 193, 257, 2, 4, False)
    B = np.zeros((257, 193), np.int8)
    sc = np.full(193, 0.01, np.float32)
    s, sx = capi.W4A8Strategy(), capi.W4A8StrategyEx()
    hit = C.c_int(7)
    P = capi.RK_NPU_ERR_PARAM
    assert lib.rk_npu_w4a8_autotune(None, C.byref(c), capi.ptr(B), capi.ptr(sc), C.byref(s), None) == P
    assert lib.rk_npu_w4a8_autotune_ex(None, C.byref(c), capi.ptr(B), capi.ptr(sc), C.byref(sx), None) == P
    assert lib.rk_npu_w4a8_autotune_cached(None, C.byref(c), capi.ptr(B), capi.ptr(sc), None, 0, C.byref(s), None,
                                           C.byref(hit)) == P and hit.value == 0
    assert lib.rk_npu_w4a8_autotune_cached_ex(None, C.byref(c), capi.ptr(B), capi.ptr(sc), None, 0, C.byref(sx), None,
                                              None) == P
    assert lib.rk_npu_w4a8_autotune_cache_load(None, C.byref(c), capi.ptr(B), capi.ptr(sc), None, C.byref(s),
                                               C.byref(s)) == P
    assert lib.rk_npu_w4a8_autotune_cache_save(None, C.byref(c), capi.ptr(B), capi.ptr(sc), None, C.byref(s),
                                               C.byref(s)) == P
    assert lib.rk_npu_w4a8_autotune_cache_load_ex(None, C.byref(c), capi.ptr(B), capi.ptr(sc), None, C.byref(sx),
                                                  C.byref(sx)) == P
    assert lib.rk_npu_w4a8_autotune_cache_save_ex(None, C.byref(c), capi.ptr(B), capi.ptr(sc), None, C.byref(sx),
                                                  C.byref(sx)) == P
    assert lib.rk_npu_w4a8_autotune_cache_load_profile_ex(None, C.byref(c), None, None, C.byref(sx), C.byref(sx)) == P
    fam, fs = capi.W4A8FamilySummary(), (capi.W4A8Strategy * 2)()
    fsx = (capi.W4A8StrategyEx * 2)()
    assert lib.rk_npu_w4a8_autotune_family(None, C.byref(f), capi.ptr(B), capi.ptr(sc), C.byref(fam), fs, None, None) == P
    assert lib.rk_npu_w4a8_autotune_family_ex(None, C.byref(f), capi.ptr(B), capi.ptr(sc), C.byref(fam), fsx, None,
                                              None) == P
    hits, misses = C.c_int(5), C.c_int(5)
    assert lib.rk_npu_w4a8_autotune_family_cached(None, C.byref(f), capi.ptr(B), capi.ptr(sc), None, 0, C.byref(fam), fs,
                                                  None, None, C.byref(hits), C.byref(misses)) == P
    assert (hits.value, misses.value) == (0, 0)
    assert lib.rk_npu_w4a8_autotune_family_cached_ex(None, C.byref(f), capi.ptr(B), capi.ptr(sc), None, 0, C.byref(fam),
                                                     fsx, None, None, None, None) == P
    assert not lib.rk_npu_w4a8_weights_create_tuned(None, C.byref(s), capi.ptr(B), capi.ptr(sc))
    assert not lib.rk_npu_w4a8_weights_create_tuned_ex(None, C.byref(sx), capi.ptr(B), capi.ptr(sc))
    assert not lib.rk_npu_w4a8_workspace_create_tuned_ex(None, C.byref(sx))  # revision 0 is not a tuned strategy
    assert not lib.rk_npu_w4a8_tuning_profile_from_weights(None)
    assert lib.rk_npu_w4a8_tuning_profile_fingerprint(None) == 0
    lib.rk_npu_w4a8_tuning_profile_free(None)


def _i4_code(packed, index):
    q = (int(packed[index // 2]) >> (0 if index & 1 else 4)) & 15
    return q - 16 if q >= 8 else q


def test_i4_host_side(lib):
    """reference tests/test_i4_cpu.cpp:16-31 (native K32 activation panel: signed codes, padding, guard bytes,
    rejected code) and :49-59,81-89 (memory accounting and range checks)."""
    for k in (1, 31, 32, 33, 127, 479, 480, 991, 992, 1472, 1984, 2048):
        rows, pk, lda = 3, (k + 31) // 32 * 32, k + 7
        a = ((np.arange(5 * lda) * 7 % 16) - 8).astype(np.int8)
        packed = np.full(rows * pk // 2 + 16, 0x5A, np.uint8)
        t = capi.I4InputTile(1, rows, 2, k, pk, packed.ctypes.data_as(C.POINTER(C.c_uint8)), rows * pk // 2)
        assert lib.rk_npu_i4_pack_a_tile(C.byref(t), capi.ptr(a), lda) == 0
        for m in range(rows):
            for j in range(pk):
                want = int(a[(m + 1) * lda + j + 2]) if j < k else 0
                assert _i4_code(packed, (j // 32 * rows + m) * 32 + j % 32) == want
        assert (packed[-16:] == 0x5A).all()
        a[lda + 2] = 8
        assert lib.rk_npu_i4_pack_a_tile(C.byref(t), capi.ptr(a), lda) == capi.RK_NPU_ERR_PARAM
        t.bytes -= 1
        a[lda + 2] = 0
        assert lib.rk_npu_i4_pack_a_tile(C.byref(t), capi.ptr(a), lda) == capi.RK_NPU_ERR_PARAM
    cfg = capi.I4Config()
    lib.rk_npu_i4_config_init(C.byref(cfg), 129, 65, 513)
    assert (cfg.M, cfg.N, cfg.K, cfg.m_tile, cfg.k_tile, cfg.n_tile, cfg.npu_core_mask, cfg.timeout_ms,
            cfg.pipeline, cfg.cpu_threads) == (129, 65, 513, 128, 480, 1024, 1, 500, 1, 1)
    cfg.m_tile, cfg.n_tile = 64, 64
    info = capi.I4MemoryInfo()
    assert lib.rk_npu_i4_memory_query(C.byref(cfg), C.byref(info)) == 0
    assert (info.wave_count, info.tasks_per_wave, info.packed_weight_bytes) == (2, 6, 34816)
    assert info.input_bytes == 2 * 129 * 480 // 2 and info.partial_bytes == 2 * 129 * 128 * 2
    cfg.k_tile = 512
    assert lib.rk_npu_i4_memory_query(C.byref(cfg), C.byref(info)) == 0
    P = capi.RK_NPU_ERR_PARAM
    cfg.k_tile = 2080
    assert lib.rk_npu_i4_memory_query(C.byref(cfg), C.byref(info)) == P
    cfg.k_tile, cfg.npu_core_mask = 480, 5
    assert lib.rk_npu_i4_memory_query(C.byref(cfg), C.byref(info)) == P
    cfg.npu_core_mask, cfg.K = 1, 2 ** 31 - 1
    assert lib.rk_npu_i4_memory_query(C.byref(cfg), C.byref(info)) == P
    for n in (4160, 8128):
        lib.rk_npu_i4_config_init(C.byref(cfg), 2, n, 64)
        cfg.n_tile = n
        assert lib.rk_npu_i4_memory_query(C.byref(cfg), C.byref(info)) == 0 and info.tasks_per_wave == 1
    cfg.n_tile = 8192
    assert lib.rk_npu_i4_memory_query(C.byref(cfg), C.byref(info)) == P
    lib.rk_npu_i4_config_init(C.byref(cfg), 2, 8192, 64)  # only the tile is capped: 8192 = 8128 + 64
    cfg.n_tile = 8128
    assert lib.rk_npu_i4_memory_query(C.byref(cfg), C.byref(info)) == 0 and info.tasks_per_wave == 2
    for field, value in (("m_tile", 0), ("m_tile", 129), ("n_tile", 96), ("pipeline", 2), ("cpu_threads", 5),
                         ("timeout_ms", 0), ("M", 0), ("npu_core_mask", 7)):
        lib.rk_npu_i4_config_init(C.byref(cfg), 4, 128, 64)
        setattr(cfg, field, value)
        assert lib.rk_npu_i4_memory_query(C.byref(cfg), C.byref(info)) == P, field
    wc = capi.I4WeightConfig(513, 65, 480)
    nbytes = C.c_uint64(0)
    assert lib.rk_npu_i4_weights_memory_query(C.byref(wc), C.byref(nbytes)) == 0 and nbytes.value == 544 * 128 // 2
    wc.k_tile = 0
    assert lib.rk_npu_i4_weights_memory_query(C.byref(wc), C.byref(nbytes)) == P
    # no device needed to be refused
    B = np.zeros((513, 65), np.int8)
    assert not lib.rk_npu_i4i4i32_weights_create(None, C.byref(wc), capi.ptr(B))
    assert not lib.rk_npu_i4_workspace_create(None, C.byref(cfg))
    assert lib.rk_npu_i4i4i32_run(None, None, capi.ptr(B), capi.ptr(B), None) == P
    lib.rk_npu_i4i4i32_weights_free(None)
    lib.rk_npu_i4_workspace_free(None)


def test_build_refuses_a_compiler_it_was_not_validated_with(tmp_path, capsys, monkeypatch):
    """The inline-assembly load kernels depend on how one hipcc schedules around hand-placed
    waits: the build records that compiler's version, refuses any other, and only builds with
    it -- warning loudly -- when the caller opts in through the environment."""
    from rknpu2_matmul_open_amd import build
    monkeypatch.delenv(build.ALLOW_ENV, raising=False)
    line = build.check_toolchain(os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"))
    assert line.startswith(build.VALIDATED_HIPCC)       # this image's compiler is the validated one
    assert "WARNING" not in capsys.readouterr().err
    other = tmp_path / "hipcc"
    other.write_text("#!/bin/sh\necho 'HIP version: 9.9.99999-deadbeef'\n")
    other.chmod(0o755)
    with pytest.raises(build.UnvalidatedToolchain) as refused:
        build.check_toolchain(str(other))
    assert "gemm_wk_kernel" in str(refused.value) and build.VALIDATED_HIPCC in str(refused.value)
    assert build.ALLOW_ENV in str(refused.value)
    monkeypatch.setenv(build.ALLOW_ENV, "1")
    assert build.check_toolchain(str(other)) == "HIP version: 9.9.99999-deadbeef"
    err = capsys.readouterr().err
    assert "WARNING" in err and "gemm_wk_kernel" in err and build.VALIDATED_HIPCC in err
