/*
 * rk_npu_w4a8.h -- W4A8 linear, fused gate/up + SwiGLU, and the complete FFN
 * block (gate/up -> SwiGLU -> Down) on MI355X.
 *
 * Weights are symmetric signed INT4 codes (one int8_t per code, [-8,7]) with
 * one positive FP32 scale per output channel; activations are quantized per
 * token to INT8.  Names, struct layouts, enumerators and defaults follow the
 * reference's include/rk_npu_w4a8.h (types :16-92, entry points :94-188).
 *
 * Numerical contract (fp32 arithmetic):
 *   s[m]   = maxabs(A[m,:]) == 0 ? 1 : max(maxabs/127, FLT_MIN)
 *   q[m,k] = clamp(round_half_away(A[m,k] * (1/s[m])), -127, 127)
 *   acc    = sum_k q[m,k] * B[k,n]                        (exact int32)
 *   C[m,n] = ((float)acc * s[m]) * w_scale[n]  (-> one RNE cast for fp16)
 * NaN / Inf anywhere in A is rejected with RK_NPU_ERR_PARAM before the GEMM.
 *
 * SwiGLU: weight columns are [gate(F), up(F)], N = 2F, N % 64 == 0.
 *   middle[m,n] = (g / (1 + exp(-g))) * u, where exp is the reference's
 *   degree-7 fp32 polynomial with the argument clamped to [-80,80] and
 *   g < -80 giving -0.0 (reference src/rk_npu_swiglu_fp32_neon.h:13-51 --
 *   the flavour its AArch64 production build runs).
 * FFN: Down's row scale comes from the per-row max |middle| collected while
 *   middle is produced (no second scan); a non-finite middle row is rejected
 *   with RK_NPU_ERR_PARAM before Down runs.
 *
 * The reference splits each INT8 activation into two INT4 rows and certifies
 * INT16 partial sums per k_tile; the MFMA path multiplies int8 x int4 into
 * int32 directly, so m_tile / k_tile / n_tile / pipeline / core mask /
 * cpu_threads are validated for range exactly as the reference does and
 * otherwise unused.  k_tile still takes part in the weights <-> workspace match.
 */
#ifndef RK_NPU_W4A8_H
#define RK_NPU_W4A8_H

#include "rk_npu_matmul_i4.h"

#ifdef __cplusplus
extern "C" {
#endif

/* reference :16-20.  All three run the same GPU path. */
typedef enum rk_npu_w4a8_pipeline {
    RK_NPU_W4A8_SERIAL = 0,
    RK_NPU_W4A8_PIPELINED = 1,
    RK_NPU_W4A8_CHAIN = 2
} rk_npu_w4a8_pipeline;

/* reference :22-32 */
typedef struct rk_npu_w4a8_config {
    int M, N, K;            /* M >= 1, N >= 1, 1 <= K <= INT32_MAX/1024 */
    int m_tile;             /* 1..64 (1..256 with the panel8 option)    */
    int k_tile;             /* 32..2048, multiple of 32                  */
    int n_tile;             /* 64..8128, multiple of 64                  */
    uint32_t npu_core_mask; /* 1, 2, 4, 3 or 7                           */
    uint32_t timeout_ms;    /* > 0                                       */
    int pipeline;           /* rk_npu_w4a8_pipeline                      */
    int cpu_threads;        /* 1..4                                      */
} rk_npu_w4a8_config;

/* reference :34-39 */
typedef struct rk_npu_w4a8_memory_info {
    rk_npu_i4_memory_info backend;
    uint64_t weight_metadata_bytes;
    uint64_t cpu_scratch_bytes;
} rk_npu_w4a8_memory_info;

/* reference :51-63 */
typedef enum rk_npu_w4a8_input_layout {
    RK_NPU_W4A8_INPUT_NATIVE = 0,
    RK_NPU_W4A8_INPUT_PANEL8 = 1
} rk_npu_w4a8_input_layout;
typedef enum rk_npu_w4a8_reduce_backend {
    RK_NPU_W4A8_REDUCE_CPU = 0,
    RK_NPU_W4A8_REDUCE_NPU = 1
} rk_npu_w4a8_reduce_backend;
typedef struct rk_npu_w4a8_options {
    uint32_t struct_size; /* set by rk_npu_w4a8_options_init */
    rk_npu_w4a8_input_layout input_layout;
    rk_npu_w4a8_reduce_backend reduce_backend;
} rk_npu_w4a8_options;

/* reference :64-75 */
typedef struct rk_npu_w4a8_memory_info_ex {
    rk_npu_w4a8_memory_info base;
    uint64_t reduction_output_bytes;
    uint64_t reduction_weight_bytes;
    uint64_t reduction_control_bytes;
    uint64_t workspace_bytes;
    rk_npu_w4a8_reduce_backend effective_reduce_backend;
} rk_npu_w4a8_memory_info_ex;

/* Per-call stage times in microseconds (reference :76-83).  Here:
 * activation_scan_us + quant_pack_us = the quantize kernel, submit_us = the
 * GEMM kernel, reduce_us = epilogue-side kernels (SwiGLU row-scale finish),
 * sync_us = host<->device copies, total_us = the whole blocking call. */
typedef struct rk_npu_w4a8_timings {
    double activation_scan_us;
    double quant_pack_us, sync_us, submit_us, reduce_us;
    double dequant_us, total_us;
} rk_npu_w4a8_timings;

typedef struct rk_npu_w4a8_weights rk_npu_w4a8_weights;
typedef struct rk_npu_w4a8_workspace rk_npu_w4a8_workspace;

/* reference :87-92 */
typedef struct rk_npu_w4a8_weight_info {
    rk_npu_i4_weight_config config; /* resolved K / N / k_tile */
    int safe_k_tile;
    double multiplier;
    int bound_relaxed;
} rk_npu_w4a8_weight_info;

/* {M, N, K, m_tile 64, k_tile 480, n_tile 1024, mask 1, timeout 500,
 *  pipeline PIPELINED, cpu_threads 1}  (reference :94) */
void rk_npu_w4a8_config_init(rk_npu_w4a8_config* cfg, int M, int N, int K);
/* {sizeof, NATIVE, CPU}  (reference :96) */
void rk_npu_w4a8_options_init(rk_npu_w4a8_options* options);
/* Range validation + the reference's logical byte accounting (:95, :97-99). */
int rk_npu_w4a8_memory_query(const rk_npu_w4a8_config* cfg, rk_npu_w4a8_memory_info* out);
int rk_npu_w4a8_memory_query_ex(const rk_npu_w4a8_config* cfg,
                                const rk_npu_w4a8_options* options,
                                rk_npu_w4a8_memory_info_ex* out);

/* B[K,N] codes in [-8,7], w_scale[N] finite > 0; both copied, then B is
 * stored as packed nibbles in an MFMA-tiled device layout.  cfg->k_tile == 0
 * resolves to the largest tile the reference's INT16 bound certifies for
 * these codes (<= 2048); an explicit k_tile > 480 must certify or creation
 * fails.  NULL on invalid input or allocation failure.  (reference :114-118) */
rk_npu_w4a8_weights* rk_npu_w4a8_weights_create(rk_npu_iommu_domain* domain,
                                                const rk_npu_i4_weight_config* cfg,
                                                const int8_t* B, const float* w_scale);
void rk_npu_w4a8_weights_free(rk_npu_w4a8_weights* weights);
int rk_npu_w4a8_weights_query(const rk_npu_w4a8_weights* weights, rk_npu_w4a8_weight_info* info);

/* All device scratch for one exact M is allocated here; runs allocate nothing.
 * workspace k_tile == 0 is rejected.  (reference :119-127) */
rk_npu_w4a8_workspace* rk_npu_w4a8_workspace_create(rk_npu_iommu_domain* domain,
                                                    const rk_npu_w4a8_config* cfg);
rk_npu_w4a8_workspace* rk_npu_w4a8_workspace_create_ex(rk_npu_iommu_domain* domain,
                                                       const rk_npu_w4a8_config* cfg,
                                                       const rk_npu_w4a8_options* options);
void rk_npu_w4a8_workspace_free(rk_npu_w4a8_workspace* workspace);

/* Blocking; BUSY on concurrent use of one workspace; A != C; timings may be
 * NULL.  (reference :143-146) */
int rk_npu_w4a8_run_f32(rk_npu_w4a8_workspace* workspace, const rk_npu_w4a8_weights* weights,
                        const float* A, float* C, rk_npu_w4a8_timings* timings);
int rk_npu_w4a8_run_f16(rk_npu_w4a8_workspace* workspace, const rk_npu_w4a8_weights* weights,
                        const uint16_t* A, uint16_t* C, rk_npu_w4a8_timings* timings);

/* middle[M, N/2] = SwiGLU(gate, up); requires N % 64 == 0 and the CPU reduce
 * option.  (reference :162-164) */
int rk_npu_w4a8_run_swiglu_f32(rk_npu_w4a8_workspace* workspace,
                               const rk_npu_w4a8_weights* weights, const float* A,
                               float* middle, rk_npu_w4a8_timings* timings);

/* reference :166-169 */
typedef struct rk_npu_w4a8_ffn_timings {
    rk_npu_w4a8_timings gate_up, down;
    double total_us;
} rk_npu_w4a8_ffn_timings;

/* A[M, gate_up.K] -> middle[M, F] -> C[M, down.N], all fp32, mutually
 * non-aliasing; gate_up.N == 2F, down.K == F, same M / ctx / domain, distinct
 * workspaces, both held BUSY for the call; down.activation_scan_us == 0.
 * (reference :185-188) */
int rk_npu_w4a8_run_ffn_f32(rk_npu_w4a8_workspace* gate_up,
                            const rk_npu_w4a8_weights* gate_up_weights,
                            rk_npu_w4a8_workspace* down,
                            const rk_npu_w4a8_weights* down_weights, const float* A,
                            float* middle, float* C, rk_npu_w4a8_ffn_timings* timings);

#ifdef __cplusplus
}
#endif
#endif /* RK_NPU_W4A8_H */
