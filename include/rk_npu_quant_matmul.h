/*
 * rk_npu_quant_matmul.h -- W8A8 single-GEMM operators on MI355X.
 *
 *   i8i8i32   int8 A[M,K] x int8 B[K,N] -> int32 C[M,N]      (exact, wraps mod 2^32)
 *   f16i8f16  fp16 A[M,K] x int8 B[K,N] -> fp16 C[M,N]
 *   f32i8f32  fp32 A[M,K] x int8 B[K,N] -> fp32 C[M,N]
 *
 * Caller-visible names, struct layouts, enumerator values and defaults follow
 * the reference's include/rk_npu_quant_matmul.h (types :44-176, entry points
 * :180-188 and :301-416).  Each declaration below cites the reference
 * interface it replaces.
 *
 * Numerical contract of the floating operators (fp32 arithmetic throughout):
 *   dynamic: s[m] = maxabs(A[m,:]) > 0 ? maxabs/127 : 1 ;  static: s[m] given
 *   q[m,k]  = clamp(round_half_away(A[m,k] * (1/s[m])), -127, 127)
 *   acc     = sum_k q[m,k] * B[k,n]                      (exact int32)
 *   C[m,n]  = ((float)acc * s[m]) * w_scale[n]           (two roundings, this
 *             order), then one round-to-nearest-even cast for fp16 output.
 *
 * Life cycle: strategy -> workspace_create (fixed M, owns device scratch) ;
 * weights_create (copies and re-tiles B into device memory, immutable,
 * independent of M) ; blocking run(host A -> host C) ; free.  A, C and the
 * scale arrays are compact row-major host buffers.  fp16 values are raw IEEE
 * binary16 bit patterns in uint16_t.
 *
 * Fields of rk_npu_matmul_strategy that describe RK3588 resources (k_tile,
 * n_tile, layouts, core masks, cpu_threads) are validated for range exactly as
 * the reference does and otherwise ignored: the GPU kernels choose their own
 * tiling.  k_tile still takes part in the weights <-> workspace match.
 */
#ifndef RK_NPU_QUANT_MATMUL_H
#define RK_NPU_QUANT_MATMUL_H

#include "rk_npu_common.h"

#ifdef __cplusplus
extern "C" {
#endif

/* reference include/rk_npu_quant_matmul.h:44-50 */
typedef enum rk_npu_matmul_op_kind {
    RK_NPU_MATMUL_I8I8I32 = 0,
    RK_NPU_MATMUL_F16I8F16_DYNAMIC = 1,
    RK_NPU_MATMUL_F16I8F16_STATIC = 2,
    RK_NPU_MATMUL_F32I8F32_DYNAMIC = 3,
    RK_NPU_MATMUL_F32I8F32_STATIC = 4,
} rk_npu_matmul_op_kind;

/* reference :52-59.  Range-checked only. */
typedef enum rk_npu_matmul_a_layout {
    RK_NPU_MATMUL_A_LAYOUT_NORMAL = 0,
    RK_NPU_MATMUL_A_LAYOUT_NATIVE_K16_M16 = 1,
    RK_NPU_MATMUL_A_LAYOUT_PANEL8 = 2,
    RK_NPU_MATMUL_A_LAYOUT_PANEL16 = 3,
} rk_npu_matmul_a_layout;

/* reference :61-66.  Range-checked only. */
typedef enum rk_npu_matmul_c_layout {
    RK_NPU_MATMUL_C_LAYOUT_NATIVE = 0,
    RK_NPU_MATMUL_C_LAYOUT_PANEL8 = 1,
    RK_NPU_MATMUL_C_LAYOUT_PANEL16 = 2,
} rk_npu_matmul_c_layout;

/* reference :68-93 */
typedef struct rk_npu_matmul_autotune_config {
    int M;
    int N;
    int K;
    uint32_t allowed_npu_core_mask;
    uint64_t allowed_cpu_core_mask;
    int warmup;
    int loops;
    int repeats;
    uint32_t timeout_ms;
    int verbose;
    int required_k_tile;
} rk_npu_matmul_autotune_config;

/* reference :95-99.  Key under which immutable weights are shared. */
typedef struct rk_npu_matmul_weight_config {
    int K;
    int N;
    int k_tile; /* 1..K */
} rk_npu_matmul_weight_config;

/* reference :101-115.  One K partition is chosen for all m_values (distinct,
 * > 0); frequencies (finite, > 0) weight the summary, NULL = equal weights. */
typedef struct rk_npu_matmul_family_autotune_config {
    int K;
    int N;
    int m_count;
    const int* m_values;
    const double* frequencies;
    uint32_t allowed_npu_core_mask;
    uint64_t allowed_cpu_core_mask;
    int warmup;
    int loops;
    int repeats;
    uint32_t timeout_ms;
    int verbose;
} rk_npu_matmul_family_autotune_config;

/* reference :117-147 */
typedef struct rk_npu_matmul_strategy {
    rk_npu_matmul_op_kind op_kind;
    int M;
    int N;
    int K;
    int k_tile;
    int n_tile;
    rk_npu_matmul_a_layout a_layout;
    int wave_count;
    int n_groups;
    uint32_t npu_core_mask;
    uint64_t cpu_core_mask;
    int cpu_threads;
    double input_us;
    double npu_us;
    double sync_us;
    double output_us;
    double total_us;
    double jitter_pct;
    double robust_us;
    rk_npu_matmul_c_layout c_layout;
} rk_npu_matmul_strategy;

/* reference :149-152 */
typedef struct rk_npu_i8i8i32_weights rk_npu_i8i8i32_weights;
typedef struct rk_npu_f16i8f16_weights rk_npu_f16i8f16_weights;
typedef struct rk_npu_f32i8f32_weights rk_npu_f32i8f32_weights;
typedef struct rk_npu_matmul_workspace rk_npu_matmul_workspace;

/* reference :154-158 */
typedef struct rk_npu_matmul_family_summary {
    rk_npu_matmul_weight_config weight_config;
    double weighted_total_us;
    double weighted_robust_us;
} rk_npu_matmul_family_summary;

/* reference :161-176.  The byte counts reproduce the reference's logical
 * payload formulas (they describe the RK3588 buffers a caller would have
 * budgeted for), not the HBM footprint of this build. */
typedef struct rk_npu_matmul_workspace_requirements {
    uint64_t bytes;
    uint64_t input_bytes;
    uint64_t output_bytes;
    uint64_t control_bytes;
    uint32_t wave_count;
    uint32_t buffer_count;
} rk_npu_matmul_workspace_requirements;

typedef struct rk_npu_matmul_weight_requirements {
    uint64_t bytes;
    uint64_t packed_b_bytes;
    uint64_t scale_bytes;
    uint32_t wave_count;
    uint32_t buffer_count;
} rk_npu_matmul_weight_requirements;

/* Defaults {M,N,K, npu mask 7, cpu mask 0, warmup 2, loops 8, repeats 3,
 * timeout 500 ms, verbose 0, required_k_tile 0}  (reference :180-181). */
void rk_npu_matmul_autotune_config_init(rk_npu_matmul_autotune_config* cfg,
                                        int M, int N, int K);

/* Defaults {K, N, m_count, m_values, frequencies NULL, npu mask 7, cpu mask 0,
 * warmup 2, loops 8, repeats 3, timeout 500 ms, verbose 0} (reference :182-184). */
void rk_npu_matmul_family_autotune_config_init(rk_npu_matmul_family_autotune_config* cfg, int N,
                                               int K, int m_count, const int* m_values);

/* CPU-only policy query kept for callers that probe K partitions before
 * creating weights (reference :188). */
int rk_npu_matmul_k_partition_query(int M, int K, int k_tile);

/* Tuning (reference :190-215).  The reference searches NPU tile sizes and
 * layouts; those knobs do not change what this build executes, so each call
 * returns one canonical strategy -- core / CPU masks fixed from the allowed
 * masks exactly as the reference fixes them, k_tile = required_k_tile or
 * min(K, 2048), the widest safe n_tile, plain layouts -- whose total_us /
 * robust_us are measured: the blocking host API is timed on seeded synthetic
 * tensors with cfg's warmup / loops / repeats.  `fastest` and `stable` receive
 * the same strategy; either may be NULL, not both. */
int rk_npu_i8i8i32_autotune(rk_npu_ctx* ctx, const rk_npu_matmul_autotune_config* cfg,
                            rk_npu_matmul_strategy* fastest, rk_npu_matmul_strategy* stable);
int rk_npu_f16i8f16_dynamic_autotune(rk_npu_ctx* ctx, const rk_npu_matmul_autotune_config* cfg,
                                     rk_npu_matmul_strategy* fastest, rk_npu_matmul_strategy* stable);
int rk_npu_f16i8f16_static_autotune(rk_npu_ctx* ctx, const rk_npu_matmul_autotune_config* cfg,
                                    rk_npu_matmul_strategy* fastest, rk_npu_matmul_strategy* stable);
int rk_npu_f32i8f32_dynamic_autotune(rk_npu_ctx* ctx, const rk_npu_matmul_autotune_config* cfg,
                                     rk_npu_matmul_strategy* fastest, rk_npu_matmul_strategy* stable);
int rk_npu_f32i8f32_static_autotune(rk_npu_ctx* ctx, const rk_npu_matmul_autotune_config* cfg,
                                    rk_npu_matmul_strategy* fastest, rk_npu_matmul_strategy* stable);

/* Result cache (reference :217-251).  One text file holds both strategies and
 * the key (op kind, shape, normalised masks, measurement settings,
 * required_k_tile, backend environment switches).  Load returns
 * RK_NPU_ERR_CACHE_MISS when the file is absent, malformed or keyed
 * differently; save writes a temporary file and renames it.  `cached` loads or
 * tunes-and-saves; NULL cache_path = $XDG_CACHE_HOME/rk_npu_matmul or
 * $HOME/.cache/rk_npu_matmul with a name derived from the key; refresh != 0
 * skips the load; a failed save never hides a good result; cache_hit is
 * optional.  The file format is this library's own (not readable by the
 * reference and vice versa). */
int rk_npu_matmul_autotune_cache_load(rk_npu_ctx* ctx, const char* cache_path,
                                      rk_npu_matmul_op_kind kind,
                                      const rk_npu_matmul_autotune_config* cfg,
                                      rk_npu_matmul_strategy* fastest,
                                      rk_npu_matmul_strategy* stable);
int rk_npu_matmul_autotune_cache_save(rk_npu_ctx* ctx, const char* cache_path,
                                      rk_npu_matmul_op_kind kind,
                                      const rk_npu_matmul_autotune_config* cfg,
                                      const rk_npu_matmul_strategy* fastest,
                                      const rk_npu_matmul_strategy* stable);
int rk_npu_matmul_autotune_cached(rk_npu_ctx* ctx, const rk_npu_matmul_autotune_config* cfg,
                                  rk_npu_matmul_op_kind kind, const char* cache_path, int refresh,
                                  rk_npu_matmul_strategy* fastest, rk_npu_matmul_strategy* stable,
                                  int* cache_hit);

/* Family tuning (reference :253-294): one K partition for all M values;
 * strategy arrays have m_count entries in m_values order; a summary and its
 * array are both NULL or both non-NULL, at least one pair is required.  The
 * cached form keeps one single-M cache file per M in cache_directory (NULL =
 * the per-user default) and counts hits / misses. */
int rk_npu_i8i8i32_autotune_family(rk_npu_ctx* ctx, const rk_npu_matmul_family_autotune_config* cfg,
                                   rk_npu_matmul_family_summary* fastest_summary,
                                   rk_npu_matmul_strategy* fastest_strategies,
                                   rk_npu_matmul_family_summary* stable_summary,
                                   rk_npu_matmul_strategy* stable_strategies);
int rk_npu_f16i8f16_dynamic_autotune_family(rk_npu_ctx* ctx,
                                            const rk_npu_matmul_family_autotune_config* cfg,
                                            rk_npu_matmul_family_summary* fastest_summary,
                                            rk_npu_matmul_strategy* fastest_strategies,
                                            rk_npu_matmul_family_summary* stable_summary,
                                            rk_npu_matmul_strategy* stable_strategies);
int rk_npu_f16i8f16_static_autotune_family(rk_npu_ctx* ctx,
                                           const rk_npu_matmul_family_autotune_config* cfg,
                                           rk_npu_matmul_family_summary* fastest_summary,
                                           rk_npu_matmul_strategy* fastest_strategies,
                                           rk_npu_matmul_family_summary* stable_summary,
                                           rk_npu_matmul_strategy* stable_strategies);
int rk_npu_f32i8f32_dynamic_autotune_family(rk_npu_ctx* ctx,
                                            const rk_npu_matmul_family_autotune_config* cfg,
                                            rk_npu_matmul_family_summary* fastest_summary,
                                            rk_npu_matmul_strategy* fastest_strategies,
                                            rk_npu_matmul_family_summary* stable_summary,
                                            rk_npu_matmul_strategy* stable_strategies);
int rk_npu_f32i8f32_static_autotune_family(rk_npu_ctx* ctx,
                                           const rk_npu_matmul_family_autotune_config* cfg,
                                           rk_npu_matmul_family_summary* fastest_summary,
                                           rk_npu_matmul_strategy* fastest_strategies,
                                           rk_npu_matmul_family_summary* stable_summary,
                                           rk_npu_matmul_strategy* stable_strategies);
int rk_npu_matmul_autotune_family_cached(rk_npu_ctx* ctx,
                                         const rk_npu_matmul_family_autotune_config* cfg,
                                         rk_npu_matmul_op_kind kind, const char* cache_directory,
                                         int refresh, rk_npu_matmul_family_summary* fastest_summary,
                                         rk_npu_matmul_strategy* fastest_strategies,
                                         rk_npu_matmul_family_summary* stable_summary,
                                         rk_npu_matmul_strategy* stable_strategies, int* cache_hits,
                                         int* cache_misses);

/* Logical byte accounting (reference :301-312). */
int rk_npu_matmul_workspace_memory_query(const rk_npu_matmul_strategy* strategy,
                                         rk_npu_matmul_workspace_requirements* out);
int rk_npu_i8i8i32_weights_memory_query(const rk_npu_matmul_weight_config* config,
                                        rk_npu_matmul_weight_requirements* out);
int rk_npu_f16i8f16_weights_memory_query(const rk_npu_matmul_weight_config* config,
                                         rk_npu_matmul_weight_requirements* out);
int rk_npu_f32i8f32_weights_memory_query(const rk_npu_matmul_weight_config* config,
                                         rk_npu_matmul_weight_requirements* out);

/* A workspace is fixed to one op kind and one exact M, owns all device scratch
 * and is non-reentrant: a second concurrent run returns RK_NPU_ERR_BUSY.
 * NULL on an invalid strategy or allocation failure (reference :313-315). */
rk_npu_matmul_workspace* rk_npu_matmul_workspace_create(
    rk_npu_iommu_domain* domain, const rk_npu_matmul_strategy* strategy);
void rk_npu_matmul_workspace_free(rk_npu_matmul_workspace* workspace);

/* ---- int8 x int8 -> int32 (reference :319-338) ---- */
rk_npu_i8i8i32_weights* rk_npu_i8i8i32_weights_create(
    rk_npu_iommu_domain* domain, const rk_npu_matmul_weight_config* config,
    const int8_t* B_rowmajor);
/* The reference's compressed storage is lossless; here it is the same device
 * layout as the plain constructor (reference :328-330). */
rk_npu_i8i8i32_weights* rk_npu_i8i8i32_weights_create_compress(
    rk_npu_iommu_domain* domain, const rk_npu_matmul_weight_config* config,
    const int8_t* B_rowmajor);
void rk_npu_i8i8i32_weights_free(rk_npu_i8i8i32_weights* weights);
int rk_npu_i8i8i32_run(rk_npu_matmul_workspace* workspace,
                       const rk_npu_i8i8i32_weights* weights,
                       const int8_t* A_rowmajor, int32_t* C_rowmajor);

/* ---- fp16 x int8 -> fp16 (reference :345-384) ----
 * w_scale[N] must be finite and > 0.  B and w_scale are copied. */
rk_npu_f16i8f16_weights* rk_npu_f16i8f16_weights_create(
    rk_npu_iommu_domain* domain, const rk_npu_matmul_weight_config* config,
    const int8_t* B_rowmajor, const float* w_scale);
rk_npu_f16i8f16_weights* rk_npu_f16i8f16_weights_create_compress(
    rk_npu_iommu_domain* domain, const rk_npu_matmul_weight_config* config,
    const int8_t* B_rowmajor, const float* w_scale);
void rk_npu_f16i8f16_weights_free(rk_npu_f16i8f16_weights* weights);
int rk_npu_f16i8f16_run_dynamic(rk_npu_matmul_workspace* workspace,
                                const rk_npu_f16i8f16_weights* weights,
                                const uint16_t* A_fp16_rowmajor,
                                uint16_t* C_fp16_rowmajor);
/* a_scale[M]: finite, > 0, caller-owned for the duration of the call. */
int rk_npu_f16i8f16_run_static(rk_npu_matmul_workspace* workspace,
                               const rk_npu_f16i8f16_weights* weights,
                               const uint16_t* A_fp16_rowmajor,
                               const float* a_scale,
                               uint16_t* C_fp16_rowmajor);

/* ---- fp32 x int8 -> fp32 (reference :388-416) ---- */
rk_npu_f32i8f32_weights* rk_npu_f32i8f32_weights_create(
    rk_npu_iommu_domain* domain, const rk_npu_matmul_weight_config* config,
    const int8_t* B_rowmajor, const float* w_scale);
rk_npu_f32i8f32_weights* rk_npu_f32i8f32_weights_create_compress(
    rk_npu_iommu_domain* domain, const rk_npu_matmul_weight_config* config,
    const int8_t* B_rowmajor, const float* w_scale);
/* Always 0: no compressed layouts exist in this build (reference :398-399). */
uint64_t rk_npu_f32i8f32_weights_compressed_layout_generation(
    const rk_npu_f32i8f32_weights* weights);

/* fp32 weights quantized under a bits-per-weight budget for the NPU's lossless
 * weight decompressor (reference :351-359,400-402).  That storage format does
 * not exist here: both constructors report the budget search as unmet (NULL). */
rk_npu_f16i8f16_weights* rk_npu_f16i8f16_weights_create_from_f32_compress(
    rk_npu_iommu_domain* domain, const rk_npu_matmul_weight_config* config, const float* B_rowmajor,
    float target_bpw);
rk_npu_f32i8f32_weights* rk_npu_f32i8f32_weights_create_from_f32_compress(
    rk_npu_iommu_domain* domain, const rk_npu_matmul_weight_config* config, const float* B_rowmajor,
    float target_bpw);
void rk_npu_f32i8f32_weights_free(rk_npu_f32i8f32_weights* weights);
int rk_npu_f32i8f32_run_dynamic(rk_npu_matmul_workspace* workspace,
                                const rk_npu_f32i8f32_weights* weights,
                                const float* A_fp32_rowmajor,
                                float* C_fp32_rowmajor);
int rk_npu_f32i8f32_run_static(rk_npu_matmul_workspace* workspace,
                               const rk_npu_f32i8f32_weights* weights,
                               const float* A_fp32_rowmajor,
                               const float* a_scale,
                               float* C_fp32_rowmajor);

#ifdef __cplusplus
}
#endif
#endif /* RK_NPU_QUANT_MATMUL_H */
