/*
 * rk_npu_w4a8_tune.h -- tuning, strategy-cache and "tuned" factory entry
 * points of the W4A8 operator on MI355X.
 *
 * Names, struct layouts and defaults follow the reference's
 * include/rk_npu_w4a8_tune.h (types :9-77, entry points :82-162), so a caller
 * that tunes, caches and then creates weights / workspaces from a strategy
 * links unchanged.
 *
 * What a tuning call does here.  The reference searches K/M/N tiles, CPU team
 * size, serial / pipelined / chained submission and the panel8 input layout.
 * None of these changes what the GPU executes, so ONE canonical strategy per
 * shape is returned (fastest == stable): the core / CPU sets the reference
 * would fix from the masks, k_tile = required_k_tile or the widest tile the
 * weight-bound policy permits, m_tile = min(64, M), n_tile = min(1024, N share
 * of a core), native input, CPU reduction, pipelined, the full CPU team.
 * Real, and identical in meaning to the reference:
 *   - the weight profile: largest certified K tile (INT16-partial bound of the
 *     reference's NPU path), the set of certified tiles, the multiplier policy
 *     and a fingerprint of codes + scales; it decides which k_tile is legal
 *     and binds strategies and cache entries to one weight matrix;
 *   - the timings: complete blocking calls on the reference's deterministic
 *     calibration tensor, warmup / loops / repeats as configured; the output
 *     is verified against a CPU restatement first (ERR_PARAM on mismatch);
 *   - the cache contract: value round trip, RK_NPU_ERR_CACHE_MISS on any
 *     mismatch of shape, dtype, resources, policy, weights or revision, no
 *     device work on a hit, atomic save.  The file format is this library's
 *     own (text); caches are not interchangeable with the reference's.
 * Difference: a relaxed strategy (multiplier > 1) can not saturate here
 * (int32 accumulation), so a tile the reference rejects after its sample run
 * is accepted.
 */
#ifndef RK_NPU_W4A8_TUNE_H
#define RK_NPU_W4A8_TUNE_H

#include "rk_npu_w4a8.h"

#ifdef __cplusplus
extern "C" {
#endif

/* reference :9-12 */
typedef enum rk_npu_w4a8_activation_type {
    RK_NPU_W4A8_F32 = 0,
    RK_NPU_W4A8_F16 = 1
} rk_npu_w4a8_activation_type;

/* reference :14-24 */
typedef struct rk_npu_w4a8_autotune_config {
    int M, N, K;
    rk_npu_w4a8_activation_type activation_type;
    uint32_t allowed_npu_core_mask; /* subset of 7; 0 = all                              */
    uint64_t allowed_cpu_core_mask; /* 0 = current affinity; up to 4 CPUs, 4..7 first    */
    int warmup, loops, repeats;     /* >= 0, > 0, > 0                                    */
    uint32_t timeout_ms;            /* > 0                                               */
    int verbose;                    /* != 0: one line per measured strategy on stderr    */
    int required_k_tile;            /* 0, or a multiple of 32 <= min(align32(K), 2048)   */
    double k_tile_multiplier;       /* 0: RK_NPU_W4A8_K_TILE_MULTIPLIER (1 if unset); >= 1 */
} rk_npu_w4a8_autotune_config;

/* reference :26-36 */
typedef struct rk_npu_w4a8_strategy {
    rk_npu_w4a8_config config;
    rk_npu_w4a8_activation_type activation_type;
    uint64_t cpu_core_mask;
    rk_npu_w4a8_weight_info weights;
    uint64_t weight_fingerprint; /* codes and scales; not a security hash */
    uint32_t tuning_revision;
    double input_us, npu_us, sync_us, output_us, total_us; /* medians over the repeats */
    double jitter_pct, robust_us;                          /* spread; total + spread/2  */
} rk_npu_w4a8_strategy;

/* reference :42-45.  execution is always {native input, CPU reduction} here. */
typedef struct rk_npu_w4a8_strategy_ex {
    rk_npu_w4a8_strategy base;
    rk_npu_w4a8_options execution;
} rk_npu_w4a8_strategy_ex;

/* Bounds and identity of a weight matrix, copied out of a weights handle; it
 * owns no device memory and outlives the handle.  (reference :51-58) */
typedef struct rk_npu_w4a8_tuning_profile rk_npu_w4a8_tuning_profile;
rk_npu_w4a8_tuning_profile* rk_npu_w4a8_tuning_profile_from_weights(const rk_npu_w4a8_weights* weights);
void rk_npu_w4a8_tuning_profile_free(rk_npu_w4a8_tuning_profile* profile);
/* 0 for NULL */
uint64_t rk_npu_w4a8_tuning_profile_fingerprint(const rk_npu_w4a8_tuning_profile* profile);
/* Cache lookup from a captured profile: no weight scan, no device work, no
 * write; cfg->k_tile_multiplier must equal the profile's (an explicit value,
 * not 0).  (reference :59-62) */
int rk_npu_w4a8_autotune_cache_load_profile_ex(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* cfg,
                                               const rk_npu_w4a8_tuning_profile* profile, const char* cache_path,
                                               rk_npu_w4a8_strategy_ex* fastest, rk_npu_w4a8_strategy_ex* stable);

/* reference :64-74 */
typedef struct rk_npu_w4a8_family_config {
    rk_npu_w4a8_autotune_config base; /* M ignored */
    int m_count;
    const int* m_values;       /* distinct, > 0 */
    const double* frequencies; /* finite > 0; NULL = equal */
} rk_npu_w4a8_family_config;
typedef struct rk_npu_w4a8_family_summary {
    rk_npu_w4a8_weight_info weights; /* the K partition shared by all M */
    uint64_t weight_fingerprint;
    double weighted_total_us, weighted_robust_us;
} rk_npu_w4a8_family_summary;

/* {M, N, K, F32, npu 7, cpu 0, warmup 2, loops 8, repeats 3, 500 ms, quiet,
 *  no required tile, multiplier 0}  (reference :79) */
void rk_npu_w4a8_autotune_config_init(rk_npu_w4a8_autotune_config* cfg, int M, int N, int K);
/* base as above with M = 1  (reference :80-81) */
void rk_npu_w4a8_family_config_init(rk_npu_w4a8_family_config* cfg, int N, int K, int m_count,
                                    const int* m_values);

/* B[K,N] codes and w_scale[N] are the weights the strategy is for.  Either of
 * fastest / stable may be NULL, not both.  (reference :101-105) */
int rk_npu_w4a8_autotune(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* cfg, const int8_t* B,
                         const float* w_scale, rk_npu_w4a8_strategy* fastest, rk_npu_w4a8_strategy* stable);
/* refresh != 0 re-measures and overwrites.  cache_path NULL: a file under
 * $XDG_CACHE_HOME/rk_npu_w4a8 or $HOME/.cache/rk_npu_w4a8.  *cache_hit = 1 when
 * the result came from the file.  (reference :103-105) */
int rk_npu_w4a8_autotune_cached(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* cfg, const int8_t* B,
                                const float* w_scale, const char* cache_path, int refresh,
                                rk_npu_w4a8_strategy* fastest, rk_npu_w4a8_strategy* stable, int* cache_hit);
/* RK_NPU_ERR_CACHE_MISS when absent or stale.  (reference :109-114) */
int rk_npu_w4a8_autotune_cache_load(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* cfg, const int8_t* B,
                                    const float* w_scale, const char* cache_path, rk_npu_w4a8_strategy* fastest,
                                    rk_npu_w4a8_strategy* stable);
int rk_npu_w4a8_autotune_cache_save(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* cfg, const int8_t* B,
                                    const float* w_scale, const char* cache_path,
                                    const rk_npu_w4a8_strategy* fastest, const rk_npu_w4a8_strategy* stable);

/* Re-validates weights and policy against the strategy (a changed code or
 * scale gives NULL), then creates exactly the selected K partition, relaxed or
 * not.  Create the workspace from strategy->config.  (reference :119-120) */
rk_npu_w4a8_weights* rk_npu_w4a8_weights_create_tuned(rk_npu_iommu_domain* domain,
                                                      const rk_npu_w4a8_strategy* strategy, const int8_t* B,
                                                      const float* w_scale);

/* One K partition for every M; per-M results go through the single-M cache
 * entries.  Each requested summary needs a strategy array of m_count
 * elements.  (reference :124-132) */
int rk_npu_w4a8_autotune_family(rk_npu_ctx* ctx, const rk_npu_w4a8_family_config* cfg, const int8_t* B,
                                const float* w_scale, rk_npu_w4a8_family_summary* fastest,
                                rk_npu_w4a8_strategy* fastest_strategies, rk_npu_w4a8_family_summary* stable,
                                rk_npu_w4a8_strategy* stable_strategies);
int rk_npu_w4a8_autotune_family_cached(rk_npu_ctx* ctx, const rk_npu_w4a8_family_config* cfg, const int8_t* B,
                                       const float* w_scale, const char* cache_directory, int refresh,
                                       rk_npu_w4a8_family_summary* fastest, rk_npu_w4a8_strategy* fastest_strategies,
                                       rk_npu_w4a8_family_summary* stable, rk_npu_w4a8_strategy* stable_strategies,
                                       int* cache_hits, int* cache_misses);

/* The _ex forms carry the input layout and have their own cache identity
 * (reference :141-162). */
int rk_npu_w4a8_autotune_ex(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* cfg, const int8_t* B,
                            const float* w_scale, rk_npu_w4a8_strategy_ex* fastest, rk_npu_w4a8_strategy_ex* stable);
int rk_npu_w4a8_autotune_cached_ex(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* cfg, const int8_t* B,
                                   const float* w_scale, const char* cache_path, int refresh,
                                   rk_npu_w4a8_strategy_ex* fastest, rk_npu_w4a8_strategy_ex* stable, int* cache_hit);
int rk_npu_w4a8_autotune_cache_load_ex(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* cfg, const int8_t* B,
                                       const float* w_scale, const char* cache_path, rk_npu_w4a8_strategy_ex* fastest,
                                       rk_npu_w4a8_strategy_ex* stable);
int rk_npu_w4a8_autotune_cache_save_ex(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* cfg, const int8_t* B,
                                       const float* w_scale, const char* cache_path,
                                       const rk_npu_w4a8_strategy_ex* fastest, const rk_npu_w4a8_strategy_ex* stable);
rk_npu_w4a8_weights* rk_npu_w4a8_weights_create_tuned_ex(rk_npu_iommu_domain* domain,
                                                         const rk_npu_w4a8_strategy_ex* strategy, const int8_t* B,
                                                         const float* w_scale);
rk_npu_w4a8_workspace* rk_npu_w4a8_workspace_create_tuned_ex(rk_npu_iommu_domain* domain,
                                                             const rk_npu_w4a8_strategy_ex* strategy);
int rk_npu_w4a8_autotune_family_ex(rk_npu_ctx* ctx, const rk_npu_w4a8_family_config* cfg, const int8_t* B,
                                   const float* w_scale, rk_npu_w4a8_family_summary* fastest,
                                   rk_npu_w4a8_strategy_ex* fastest_strategies, rk_npu_w4a8_family_summary* stable,
                                   rk_npu_w4a8_strategy_ex* stable_strategies);
int rk_npu_w4a8_autotune_family_cached_ex(rk_npu_ctx* ctx, const rk_npu_w4a8_family_config* cfg, const int8_t* B,
                                          const float* w_scale, const char* cache_directory, int refresh,
                                          rk_npu_w4a8_family_summary* fastest,
                                          rk_npu_w4a8_strategy_ex* fastest_strategies,
                                          rk_npu_w4a8_family_summary* stable,
                                          rk_npu_w4a8_strategy_ex* stable_strategies, int* cache_hits,
                                          int* cache_misses);

#ifdef __cplusplus
}
#endif
#endif
