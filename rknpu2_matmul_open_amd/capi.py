"""ctypes mirror of include/rk_npu_*.h.

Struct layouts and enumerator values are the ones the headers declare; the
functions are bound with explicit argtypes so a wrong call fails in Python
instead of corrupting memory.  Nothing here computes anything.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))

RK_NPU_OK = 0
RK_NPU_ERR_OPEN = -1
RK_NPU_ERR_IOCTL = -2
RK_NPU_ERR_PARAM = -3
RK_NPU_ERR_NOMEM = -4
RK_NPU_ERR_SUBMIT = -5
RK_NPU_ERR_BUSY = -6
RK_NPU_ERR_DOMAIN = -7
RK_NPU_ERR_IO = -8
RK_NPU_ERR_CACHE_MISS = -9

# rk_npu_matmul_op_kind
I8I8I32, F16I8F16_DYNAMIC, F16I8F16_STATIC, F32I8F32_DYNAMIC, F32I8F32_STATIC = range(5)
# rk_npu_w4a8_pipeline / layouts / reduce backends
W4A8_SERIAL, W4A8_PIPELINED, W4A8_CHAIN = range(3)
W4A8_INPUT_NATIVE, W4A8_INPUT_PANEL8 = range(2)
W4A8_REDUCE_CPU, W4A8_REDUCE_NPU = range(2)
MOE_MIDDLE_CPU, MOE_MIDDLE_NPU_LUT = range(2)


class DomainMemoryStats(C.Structure):
    _fields_ = [("live_bytes", C.c_uint64), ("peak_bytes", C.c_uint64),
                ("creates", C.c_uint64), ("destroys", C.c_uint64)]


class MatmulAutotuneConfig(C.Structure):
    _fields_ = [("M", C.c_int), ("N", C.c_int), ("K", C.c_int),
                ("allowed_npu_core_mask", C.c_uint32), ("allowed_cpu_core_mask", C.c_uint64),
                ("warmup", C.c_int), ("loops", C.c_int), ("repeats", C.c_int),
                ("timeout_ms", C.c_uint32), ("verbose", C.c_int), ("required_k_tile", C.c_int)]


class MatmulWeightConfig(C.Structure):
    _fields_ = [("K", C.c_int), ("N", C.c_int), ("k_tile", C.c_int)]


class MatmulFamilyAutotuneConfig(C.Structure):
    _fields_ = [("K", C.c_int), ("N", C.c_int), ("m_count", C.c_int), ("m_values", C.POINTER(C.c_int)),
                ("frequencies", C.POINTER(C.c_double)), ("allowed_npu_core_mask", C.c_uint32),
                ("allowed_cpu_core_mask", C.c_uint64), ("warmup", C.c_int), ("loops", C.c_int),
                ("repeats", C.c_int), ("timeout_ms", C.c_uint32), ("verbose", C.c_int)]


class MatmulFamilySummary(C.Structure):
    _fields_ = [("weight_config", MatmulWeightConfig), ("weighted_total_us", C.c_double),
                ("weighted_robust_us", C.c_double)]


class MatmulStrategy(C.Structure):
    _fields_ = [("op_kind", C.c_int), ("M", C.c_int), ("N", C.c_int), ("K", C.c_int),
                ("k_tile", C.c_int), ("n_tile", C.c_int), ("a_layout", C.c_int),
                ("wave_count", C.c_int), ("n_groups", C.c_int), ("npu_core_mask", C.c_uint32),
                ("cpu_core_mask", C.c_uint64), ("cpu_threads", C.c_int),
                ("input_us", C.c_double), ("npu_us", C.c_double), ("sync_us", C.c_double),
                ("output_us", C.c_double), ("total_us", C.c_double), ("jitter_pct", C.c_double),
                ("robust_us", C.c_double), ("c_layout", C.c_int)]


class WorkspaceRequirements(C.Structure):
    _fields_ = [("bytes", C.c_uint64), ("input_bytes", C.c_uint64), ("output_bytes", C.c_uint64),
                ("control_bytes", C.c_uint64), ("wave_count", C.c_uint32), ("buffer_count", C.c_uint32)]


class WeightRequirements(C.Structure):
    _fields_ = [("bytes", C.c_uint64), ("packed_b_bytes", C.c_uint64), ("scale_bytes", C.c_uint64),
                ("wave_count", C.c_uint32), ("buffer_count", C.c_uint32)]


class I4WeightConfig(C.Structure):
    _fields_ = [("K", C.c_int), ("N", C.c_int), ("k_tile", C.c_int)]


class I4MemoryInfo(C.Structure):
    _fields_ = [("packed_weight_bytes", C.c_uint64), ("input_bytes", C.c_uint64),
                ("partial_bytes", C.c_uint64), ("control_bytes", C.c_uint64),
                ("wave_count", C.c_uint32), ("tasks_per_wave", C.c_uint32)]


class I4Config(C.Structure):
    _fields_ = [("M", C.c_int), ("N", C.c_int), ("K", C.c_int), ("m_tile", C.c_int), ("k_tile", C.c_int),
                ("n_tile", C.c_int), ("npu_core_mask", C.c_uint32), ("timeout_ms", C.c_uint32),
                ("pipeline", C.c_int), ("cpu_threads", C.c_int)]


class I4Timings(C.Structure):
    _fields_ = [("pack_us", C.c_double), ("sync_us", C.c_double), ("submit_us", C.c_double),
                ("reduce_us", C.c_double), ("total_us", C.c_double)]


class I4InputTile(C.Structure):
    _fields_ = [("m0", C.c_int), ("rows", C.c_int), ("k0", C.c_int), ("k", C.c_int), ("padded_k", C.c_int),
                ("dst", C.POINTER(C.c_uint8)), ("bytes", C.c_uint64)]


I4_INPUT_PRODUCER = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(I4InputTile))


class W4A8Config(C.Structure):
    _fields_ = [("M", C.c_int), ("N", C.c_int), ("K", C.c_int), ("m_tile", C.c_int),
                ("k_tile", C.c_int), ("n_tile", C.c_int), ("npu_core_mask", C.c_uint32),
                ("timeout_ms", C.c_uint32), ("pipeline", C.c_int), ("cpu_threads", C.c_int)]


class W4A8MemoryInfo(C.Structure):
    _fields_ = [("backend", I4MemoryInfo), ("weight_metadata_bytes", C.c_uint64),
                ("cpu_scratch_bytes", C.c_uint64)]


class W4A8Options(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("input_layout", C.c_int), ("reduce_backend", C.c_int)]


class W4A8MemoryInfoEx(C.Structure):
    _fields_ = [("base", W4A8MemoryInfo), ("reduction_output_bytes", C.c_uint64),
                ("reduction_weight_bytes", C.c_uint64), ("reduction_control_bytes", C.c_uint64),
                ("workspace_bytes", C.c_uint64), ("effective_reduce_backend", C.c_int)]


class W4A8Timings(C.Structure):
    _fields_ = [("activation_scan_us", C.c_double), ("quant_pack_us", C.c_double),
                ("sync_us", C.c_double), ("submit_us", C.c_double), ("reduce_us", C.c_double),
                ("dequant_us", C.c_double), ("total_us", C.c_double)]


class W4A8WeightInfo(C.Structure):
    _fields_ = [("config", I4WeightConfig), ("safe_k_tile", C.c_int), ("multiplier", C.c_double),
                ("bound_relaxed", C.c_int)]


class W4A8FfnTimings(C.Structure):
    _fields_ = [("gate_up", W4A8Timings), ("down", W4A8Timings), ("total_us", C.c_double)]


# rk_npu_w4a8_tune.h
W4A8_F32, W4A8_F16 = 0, 1


class W4A8AutotuneConfig(C.Structure):
    _fields_ = [("M", C.c_int), ("N", C.c_int), ("K", C.c_int), ("activation_type", C.c_int),
                ("allowed_npu_core_mask", C.c_uint32), ("allowed_cpu_core_mask", C.c_uint64),
                ("warmup", C.c_int), ("loops", C.c_int), ("repeats", C.c_int), ("timeout_ms", C.c_uint32),
                ("verbose", C.c_int), ("required_k_tile", C.c_int), ("k_tile_multiplier", C.c_double)]


class W4A8Strategy(C.Structure):
    _fields_ = [("config", W4A8Config), ("activation_type", C.c_int), ("cpu_core_mask", C.c_uint64),
                ("weights", W4A8WeightInfo), ("weight_fingerprint", C.c_uint64),
                ("tuning_revision", C.c_uint32), ("input_us", C.c_double), ("npu_us", C.c_double),
                ("sync_us", C.c_double), ("output_us", C.c_double), ("total_us", C.c_double),
                ("jitter_pct", C.c_double), ("robust_us", C.c_double)]


class W4A8StrategyEx(C.Structure):
    _fields_ = [("base", W4A8Strategy), ("execution", W4A8Options)]


class W4A8FamilyConfig(C.Structure):
    _fields_ = [("base", W4A8AutotuneConfig), ("m_count", C.c_int), ("m_values", C.POINTER(C.c_int)),
                ("frequencies", C.POINTER(C.c_double))]


class W4A8FamilySummary(C.Structure):
    _fields_ = [("weights", W4A8WeightInfo), ("weight_fingerprint", C.c_uint64),
                ("weighted_total_us", C.c_double), ("weighted_robust_us", C.c_double)]


class MoeWeightConfig(C.Structure):
    _fields_ = [("hidden", C.c_int), ("intermediate", C.c_int), ("routed_experts", C.c_int),
                ("shared_expert", C.c_int)]


class MoeConfig(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("weights", MoeWeightConfig), ("max_rows", C.c_int),
                ("top_k", C.c_int), ("npu_cores", C.c_int), ("cpu_threads", C.c_int),
                ("native_input", C.c_int), ("middle", C.c_int), ("timeout_ms", C.c_uint32)]


class MoeExpert(C.Structure):
    _fields_ = [("gate_up", C.c_void_p), ("gate_up_scales", C.c_void_p),
                ("down", C.c_void_p), ("down_scales", C.c_void_p)]


class MoeTimings(C.Structure):
    _fields_ = [("input_us", C.c_double), ("schedule_us", C.c_double), ("build_us", C.c_double),
                ("sync_us", C.c_double), ("gather_us", C.c_double), ("gate_us", C.c_double),
                ("middle_npu_us", C.c_double), ("middle_cpu_us", C.c_double),
                ("down_us", C.c_double), ("combine_us", C.c_double), ("lut_load_us", C.c_double),
                ("total_us", C.c_double), ("gather_tasks", C.c_uint32),
                ("middle_tasks", C.c_uint32), ("gemm_tasks", C.c_uint32)]


class MoeImportTimings(C.Structure):
    _fields_ = [("copy_us", C.c_double), ("validate_us", C.c_double), ("gate_sync_us", C.c_double),
                ("down_sync_us", C.c_double), ("total_us", C.c_double)]


P = C.c_void_p
ReclaimIdleFn = C.CFUNCTYPE(None, C.c_void_p)   # rk_npu_reclaim_idle_fn
_PROTOTYPES = {
    # rk_npu_common.h
    "rk_npu_open": (P, [C.c_char_p]),
    "rk_npu_close": (None, [P]),
    "rk_npu_iommu_domain_create": (P, [P, C.c_uint32]),
    "rk_npu_iommu_domain_free": (None, [P]),
    "rk_npu_iommu_domain_id": (C.c_uint32, [P]),
    "rk_npu_iommu_domain_memory_stats": (C.c_int, [P, C.POINTER(DomainMemoryStats)]),
    "rk_npu_iommu_domain_set_reclaim": (None, [P, P, P]),
    "rk_npu_strerror": (C.c_char_p, [C.c_int]),
    # rk_npu_quant_matmul.h
    "rk_npu_matmul_autotune_config_init": (None, [C.POINTER(MatmulAutotuneConfig), C.c_int, C.c_int, C.c_int]),
    "rk_npu_matmul_k_partition_query": (C.c_int, [C.c_int, C.c_int, C.c_int]),
    "rk_npu_matmul_family_autotune_config_init": (None, [C.POINTER(MatmulFamilyAutotuneConfig), C.c_int, C.c_int,
                                                         C.c_int, C.POINTER(C.c_int)]),
    "rk_npu_i8i8i32_autotune": (C.c_int, [P, C.POINTER(MatmulAutotuneConfig), P, P]),
    "rk_npu_f16i8f16_dynamic_autotune": (C.c_int, [P, C.POINTER(MatmulAutotuneConfig), P, P]),
    "rk_npu_f16i8f16_static_autotune": (C.c_int, [P, C.POINTER(MatmulAutotuneConfig), P, P]),
    "rk_npu_f32i8f32_dynamic_autotune": (C.c_int, [P, C.POINTER(MatmulAutotuneConfig), P, P]),
    "rk_npu_f32i8f32_static_autotune": (C.c_int, [P, C.POINTER(MatmulAutotuneConfig), P, P]),
    "rk_npu_matmul_autotune_cache_load": (C.c_int, [P, C.c_char_p, C.c_int, C.POINTER(MatmulAutotuneConfig), P, P]),
    "rk_npu_matmul_autotune_cache_save": (C.c_int, [P, C.c_char_p, C.c_int, C.POINTER(MatmulAutotuneConfig), P, P]),
    "rk_npu_matmul_autotune_cached": (C.c_int, [P, C.POINTER(MatmulAutotuneConfig), C.c_int, C.c_char_p, C.c_int, P, P,
                                                C.POINTER(C.c_int)]),
    "rk_npu_i8i8i32_autotune_family": (C.c_int, [P, C.POINTER(MatmulFamilyAutotuneConfig), P, P, P, P]),
    "rk_npu_f16i8f16_dynamic_autotune_family": (C.c_int, [P, C.POINTER(MatmulFamilyAutotuneConfig), P, P, P, P]),
    "rk_npu_f16i8f16_static_autotune_family": (C.c_int, [P, C.POINTER(MatmulFamilyAutotuneConfig), P, P, P, P]),
    "rk_npu_f32i8f32_dynamic_autotune_family": (C.c_int, [P, C.POINTER(MatmulFamilyAutotuneConfig), P, P, P, P]),
    "rk_npu_f32i8f32_static_autotune_family": (C.c_int, [P, C.POINTER(MatmulFamilyAutotuneConfig), P, P, P, P]),
    "rk_npu_matmul_autotune_family_cached": (C.c_int, [P, C.POINTER(MatmulFamilyAutotuneConfig), C.c_int, C.c_char_p,
                                                       C.c_int, P, P, P, P, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "rk_npu_f16i8f16_weights_create_from_f32_compress": (P, [P, C.POINTER(MatmulWeightConfig), P, C.c_float]),
    "rk_npu_f32i8f32_weights_create_from_f32_compress": (P, [P, C.POINTER(MatmulWeightConfig), P, C.c_float]),
    "rk_npu_matmul_workspace_memory_query": (C.c_int, [C.POINTER(MatmulStrategy), C.POINTER(WorkspaceRequirements)]),
    "rk_npu_i8i8i32_weights_memory_query": (C.c_int, [C.POINTER(MatmulWeightConfig), C.POINTER(WeightRequirements)]),
    "rk_npu_f16i8f16_weights_memory_query": (C.c_int, [C.POINTER(MatmulWeightConfig), C.POINTER(WeightRequirements)]),
    "rk_npu_f32i8f32_weights_memory_query": (C.c_int, [C.POINTER(MatmulWeightConfig), C.POINTER(WeightRequirements)]),
    "rk_npu_matmul_workspace_create": (P, [P, C.POINTER(MatmulStrategy)]),
    "rk_npu_matmul_workspace_free": (None, [P]),
    "rk_npu_i8i8i32_weights_create": (P, [P, C.POINTER(MatmulWeightConfig), P]),
    "rk_npu_i8i8i32_weights_create_compress": (P, [P, C.POINTER(MatmulWeightConfig), P]),
    "rk_npu_i8i8i32_weights_free": (None, [P]),
    "rk_npu_i8i8i32_run": (C.c_int, [P, P, P, P]),
    "rk_npu_f16i8f16_weights_create": (P, [P, C.POINTER(MatmulWeightConfig), P, P]),
    "rk_npu_f16i8f16_weights_create_compress": (P, [P, C.POINTER(MatmulWeightConfig), P, P]),
    "rk_npu_f16i8f16_weights_free": (None, [P]),
    "rk_npu_f16i8f16_run_dynamic": (C.c_int, [P, P, P, P]),
    "rk_npu_f16i8f16_run_static": (C.c_int, [P, P, P, P, P]),
    "rk_npu_f32i8f32_weights_create": (P, [P, C.POINTER(MatmulWeightConfig), P, P]),
    "rk_npu_f32i8f32_weights_create_compress": (P, [P, C.POINTER(MatmulWeightConfig), P, P]),
    "rk_npu_f32i8f32_weights_compressed_layout_generation": (C.c_uint64, [P]),
    "rk_npu_f32i8f32_weights_free": (None, [P]),
    "rk_npu_f32i8f32_run_dynamic": (C.c_int, [P, P, P, P]),
    "rk_npu_f32i8f32_run_static": (C.c_int, [P, P, P, P, P]),
    # rk_npu_w4a8.h
    "rk_npu_w4a8_config_init": (None, [C.POINTER(W4A8Config), C.c_int, C.c_int, C.c_int]),
    "rk_npu_w4a8_options_init": (None, [C.POINTER(W4A8Options)]),
    "rk_npu_w4a8_memory_query": (C.c_int, [C.POINTER(W4A8Config), C.POINTER(W4A8MemoryInfo)]),
    "rk_npu_w4a8_memory_query_ex": (C.c_int, [C.POINTER(W4A8Config), C.POINTER(W4A8Options), C.POINTER(W4A8MemoryInfoEx)]),
    "rk_npu_w4a8_weights_create": (P, [P, C.POINTER(I4WeightConfig), P, P]),
    "rk_npu_w4a8_weights_free": (None, [P]),
    "rk_npu_w4a8_weights_query": (C.c_int, [P, C.POINTER(W4A8WeightInfo)]),
    "rk_npu_w4a8_workspace_create": (P, [P, C.POINTER(W4A8Config)]),
    "rk_npu_w4a8_workspace_create_ex": (P, [P, C.POINTER(W4A8Config), C.POINTER(W4A8Options)]),
    "rk_npu_w4a8_workspace_free": (None, [P]),
    "rk_npu_w4a8_run_f32": (C.c_int, [P, P, P, P, C.POINTER(W4A8Timings)]),
    "rk_npu_w4a8_run_f16": (C.c_int, [P, P, P, P, C.POINTER(W4A8Timings)]),
    "rk_npu_w4a8_run_swiglu_f32": (C.c_int, [P, P, P, P, C.POINTER(W4A8Timings)]),
    "rk_npu_w4a8_run_ffn_f32": (C.c_int, [P, P, P, P, P, P, P, C.POINTER(W4A8FfnTimings)]),
    # rk_npu_matmul_i4.h
    "rk_npu_i4_config_init": (None, [C.POINTER(I4Config), C.c_int, C.c_int, C.c_int]),
    "rk_npu_i4_memory_query": (C.c_int, [C.POINTER(I4Config), C.POINTER(I4MemoryInfo)]),
    "rk_npu_i4_weights_memory_query": (C.c_int, [C.POINTER(I4WeightConfig), C.POINTER(C.c_uint64)]),
    "rk_npu_i4i4i32_weights_create": (P, [P, C.POINTER(I4WeightConfig), P]),
    "rk_npu_i4i4i32_weights_free": (None, [P]),
    "rk_npu_i4_workspace_create": (P, [P, C.POINTER(I4Config)]),
    "rk_npu_i4_workspace_free": (None, [P]),
    "rk_npu_i4i4i32_run": (C.c_int, [P, P, P, P, C.POINTER(I4Timings)]),
    "rk_npu_i4i4i32_run_with_producer": (C.c_int, [P, P, I4_INPUT_PRODUCER, C.c_void_p, P, C.POINTER(I4Timings)]),
    "rk_npu_i4_pack_a_tile": (C.c_int, [C.POINTER(I4InputTile), P, C.c_int]),
    # rk_npu_w4a8_tune.h
    "rk_npu_w4a8_autotune_config_init": (None, [C.POINTER(W4A8AutotuneConfig), C.c_int, C.c_int, C.c_int]),
    "rk_npu_w4a8_family_config_init": (None, [C.POINTER(W4A8FamilyConfig), C.c_int, C.c_int, C.c_int,
                                              C.POINTER(C.c_int)]),
    "rk_npu_w4a8_tuning_profile_from_weights": (P, [P]),
    "rk_npu_w4a8_tuning_profile_free": (None, [P]),
    "rk_npu_w4a8_tuning_profile_fingerprint": (C.c_uint64, [P]),
    "rk_npu_w4a8_autotune_cache_load_profile_ex": (C.c_int, [P, C.POINTER(W4A8AutotuneConfig), P, C.c_char_p,
                                                             C.POINTER(W4A8StrategyEx), C.POINTER(W4A8StrategyEx)]),
    "rk_npu_w4a8_autotune": (C.c_int, [P, C.POINTER(W4A8AutotuneConfig), P, P, C.POINTER(W4A8Strategy),
                                       C.POINTER(W4A8Strategy)]),
    "rk_npu_w4a8_autotune_cached": (C.c_int, [P, C.POINTER(W4A8AutotuneConfig), P, P, C.c_char_p, C.c_int,
                                              C.POINTER(W4A8Strategy), C.POINTER(W4A8Strategy),
                                              C.POINTER(C.c_int)]),
    "rk_npu_w4a8_autotune_cache_load": (C.c_int, [P, C.POINTER(W4A8AutotuneConfig), P, P, C.c_char_p,
                                                  C.POINTER(W4A8Strategy), C.POINTER(W4A8Strategy)]),
    "rk_npu_w4a8_autotune_cache_save": (C.c_int, [P, C.POINTER(W4A8AutotuneConfig), P, P, C.c_char_p,
                                                  C.POINTER(W4A8Strategy), C.POINTER(W4A8Strategy)]),
    "rk_npu_w4a8_weights_create_tuned": (P, [P, C.POINTER(W4A8Strategy), P, P]),
    "rk_npu_w4a8_autotune_family": (C.c_int, [P, C.POINTER(W4A8FamilyConfig), P, P,
                                              C.POINTER(W4A8FamilySummary), C.POINTER(W4A8Strategy),
                                              C.POINTER(W4A8FamilySummary), C.POINTER(W4A8Strategy)]),
    "rk_npu_w4a8_autotune_family_cached": (C.c_int, [P, C.POINTER(W4A8FamilyConfig), P, P, C.c_char_p, C.c_int,
                                                     C.POINTER(W4A8FamilySummary), C.POINTER(W4A8Strategy),
                                                     C.POINTER(W4A8FamilySummary), C.POINTER(W4A8Strategy),
                                                     C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "rk_npu_w4a8_autotune_ex": (C.c_int, [P, C.POINTER(W4A8AutotuneConfig), P, P, C.POINTER(W4A8StrategyEx),
                                          C.POINTER(W4A8StrategyEx)]),
    "rk_npu_w4a8_autotune_cached_ex": (C.c_int, [P, C.POINTER(W4A8AutotuneConfig), P, P, C.c_char_p, C.c_int,
                                                 C.POINTER(W4A8StrategyEx), C.POINTER(W4A8StrategyEx),
                                                 C.POINTER(C.c_int)]),
    "rk_npu_w4a8_autotune_cache_load_ex": (C.c_int, [P, C.POINTER(W4A8AutotuneConfig), P, P, C.c_char_p,
                                                     C.POINTER(W4A8StrategyEx), C.POINTER(W4A8StrategyEx)]),
    "rk_npu_w4a8_autotune_cache_save_ex": (C.c_int, [P, C.POINTER(W4A8AutotuneConfig), P, P, C.c_char_p,
                                                     C.POINTER(W4A8StrategyEx), C.POINTER(W4A8StrategyEx)]),
    "rk_npu_w4a8_weights_create_tuned_ex": (P, [P, C.POINTER(W4A8StrategyEx), P, P]),
    "rk_npu_w4a8_workspace_create_tuned_ex": (P, [P, C.POINTER(W4A8StrategyEx)]),
    "rk_npu_w4a8_autotune_family_ex": (C.c_int, [P, C.POINTER(W4A8FamilyConfig), P, P,
                                                 C.POINTER(W4A8FamilySummary), C.POINTER(W4A8StrategyEx),
                                                 C.POINTER(W4A8FamilySummary), C.POINTER(W4A8StrategyEx)]),
    "rk_npu_w4a8_autotune_family_cached_ex": (C.c_int, [P, C.POINTER(W4A8FamilyConfig), P, P, C.c_char_p, C.c_int,
                                                        C.POINTER(W4A8FamilySummary), C.POINTER(W4A8StrategyEx),
                                                        C.POINTER(W4A8FamilySummary), C.POINTER(W4A8StrategyEx),
                                                        C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    # rk_npu_moe_w8.h
    "rk_npu_moe_w8_config_init": (None, [C.POINTER(MoeConfig)] + [C.c_int] * 6),
    "rk_npu_moe_w8_weights_create": (P, [P, C.POINTER(MoeWeightConfig), C.POINTER(MoeExpert)]),
    "rk_npu_moe_w8_weights_free": (None, [P]),
    "rk_npu_moe_w8_workspace_create": (P, [P, C.POINTER(MoeConfig)]),
    "rk_npu_moe_w8_workspace_free": (None, [P]),
    "rk_npu_moe_w8_weights_device_bytes": (C.c_uint64, [P]),
    "rk_npu_moe_w8_workspace_device_bytes": (C.c_uint64, [P]),
    "rk_npu_moe_w8_run_quantized": (C.c_int, [P, P, C.c_int, P, P, P, P, P, C.POINTER(MoeTimings)]),
    "rk_npu_moe_w8_run_f32": (C.c_int, [P, P, C.c_int, P, P, P, P, C.POINTER(MoeTimings)]),
    # other expert formats: exported, always declining
    "rk_npu_moe_quant_weights_create": (P, [P, C.POINTER(MoeWeightConfig), C.POINTER(MoeExpert)]),
    "rk_npu_moe_quant_weights_create_full_k": (P, [P, C.POINTER(MoeWeightConfig), C.POINTER(MoeExpert)]),
    "rk_npu_moe_quant_workspace_create": (P, [P, C.POINTER(MoeConfig)]),
    "rk_npu_moe_w4_weights_create": (P, [P, C.POINTER(MoeWeightConfig), C.POINTER(MoeExpert)]),
    "rk_npu_moe_w4_workspace_create": (P, [P, C.POINTER(MoeConfig)]),
    "rk_npu_moe_w4_slots_create": (P, [P, C.POINTER(MoeWeightConfig), C.POINTER(MoeExpert)]),
    "rk_npu_moe_quant_slots_create": (P, [P, C.POINTER(MoeWeightConfig)]),
    "rk_npu_moe_quant_expert_blob_bytes": (C.c_uint64, [P]),
    "rk_npu_moe_quant_export_expert": (C.c_int, [P, C.c_int, P, C.c_uint64]),
    "rk_npu_moe_quant_import_expert": (C.c_int, [P, C.c_int, P, C.c_uint64]),
    "rk_npu_moe_quant_import_expert_timed": (C.c_int, [P, C.c_int, P, C.c_uint64, P]),
    "rk_npu_moe_quant_swap_slots": (C.c_int, [P, C.c_int, P, C.c_int]),
    # rk_npu_hip.h
    "rk_npu_hip_stream": (P, [P]),
    "rk_npu_hip_device": (C.c_int, [P]),
    "rk_npu_hip_device_info": (C.c_int, [P, C.c_char_p, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "rk_npu_hip_sync": (C.c_int, [P]),
    "rk_npu_hip_malloc": (P, [P, C.c_size_t]),
    "rk_npu_hip_free": (None, [P, P]),
    "rk_npu_hip_upload": (C.c_int, [P, P, P, C.c_size_t]),
    "rk_npu_hip_download": (C.c_int, [P, P, P, C.c_size_t]),
    "rk_npu_hip_copy": (C.c_int, [P, P, P, C.c_size_t]),
    "rk_npu_hip_event_create": (P, []),
    "rk_npu_hip_event_free": (None, [P]),
    "rk_npu_hip_event_record": (C.c_int, [P, P]),
    "rk_npu_hip_event_elapsed_us": (C.c_int, [P, P, C.POINTER(C.c_double)]),
    "rk_npu_i8i8i32_run_device": (C.c_int, [P, P, P, P]),
    "rk_npu_f16i8f16_run_dynamic_device": (C.c_int, [P, P, P, P]),
    "rk_npu_f32i8f32_run_dynamic_device": (C.c_int, [P, P, P, P]),
    "rk_npu_w4a8_run_f16_device": (C.c_int, [P, P, P, P]),
    "rk_npu_w4a8_run_f32_device": (C.c_int, [P, P, P, P]),
    "rk_npu_w4a8_run_ffn_f32_device": (C.c_int, [P, P, P, P, P, P, P]),
    "rk_npu_moe_w8_run_f32_device": (C.c_int, [P, P, C.c_int, P, P, P, P]),
    "rk_npu_matmul_workspace_rerun_gemm_device": (C.c_int, [P, P, P]),
    "rk_npu_w4a8_workspace_rerun_gemm_device": (C.c_int, [P, P, P, C.c_int]),
    "rk_npu_matmul_workspace_read_quantized": (C.c_int, [P, P, P]),
    "rk_npu_w4a8_workspace_read_quantized": (C.c_int, [P, P, P]),
    "rk_npu_w4a8_run_i32": (C.c_int, [P, P, P, P]),
    "rk_npu_hip_fail_alloc_after": (None, [C.c_int]),
    "rk_npu_hip_probe_stream_read": (C.c_int, [P, P, C.c_size_t, C.c_size_t]),
    "rk_npu_hip_probe_mfma_i8": (C.c_int, [P, P, C.c_int, C.POINTER(C.c_double)]),
    "rk_npu_hip_profile_begin": (C.c_int, [P]),
    "rk_npu_hip_profile_end": (C.c_int, [P, C.c_char_p, C.c_size_t, C.POINTER(C.c_double), C.c_int]),
    "rk_npu_hip_capture_begin": (C.c_int, [P]),
    "rk_npu_hip_capture_end": (P, [P]),
    "rk_npu_hip_graph_launch": (C.c_int, [P, P]),
    "rk_npu_hip_graph_free": (None, [P]),
    "rk_npu_f16i8f16_run_dynamic_noalloc_device": (C.c_int, [P, C.c_int, P, P]),
}

EXPORTED_SYMBOLS = tuple(_PROTOTYPES)
_LIB = None


def lib_path():
    """In-tree library, or the file named by RK_NPU_MATMUL_LIB (to try out a
    differently built copy without touching the tree)."""
    return os.environ.get("RK_NPU_MATMUL_LIB") or os.path.join(HERE, "librk_npu_matmul.so")


def load_library():
    """Load librk_npu_matmul.so and bind every prototype.  Raises if it is not built."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = lib_path()
    if not os.path.exists(path):
        raise RuntimeError(
            "%s is missing: build it with `python -m rknpu2_matmul_open_amd.build` "
            "(there is no CPU fallback)" % path)
    lib = C.CDLL(path)
    for name, (restype, argtypes) in _PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _LIB = lib
    return lib


def ptr(array):
    """Address of a numpy array's data as c_void_p (array must stay alive)."""
    return C.c_void_p(array.ctypes.data)
