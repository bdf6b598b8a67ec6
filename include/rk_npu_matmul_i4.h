/*
 * rk_npu_matmul_i4.h -- exact W4A4 integer GEMM on MI355X, and the two INT4
 * structs that rk_npu_w4a8.h embeds.
 *
 *   C[M,N] (int32) = A[M,K] * B[K,N],  A and B signed INT4 codes given as one
 *   int8_t per code in [-8, 7]; no scales, no zero points.
 *
 * Names, struct layouts and defaults follow the reference's
 * include/rk_npu_matmul_i4.h (types :21-55, entry points :57-107).  The
 * reference runs INT4 x INT4 on the NPU into INT16 partials per K tile and
 * widens them on the CPU; here the codes go through the same int4-weight MFMA
 * GEMM as the W4A8 operator (activations held as int8) and accumulate in int32
 * directly, so m_tile / k_tile / n_tile / core mask / pipeline / cpu_threads
 * are validated for range exactly as the reference does and otherwise unused.
 * K <= INT32_MAX/64 guarantees that every dot product fits int32.
 *
 * Weights depend only on K / N / k_tile and may be shared by workspaces of any
 * M.  Workspaces are fixed-shape and non-reentrant (RK_NPU_ERR_BUSY).  The
 * context must outlive its weights and workspaces.  Calls are blocking.
 */
#ifndef RK_NPU_MATMUL_I4_H
#define RK_NPU_MATMUL_I4_H

#include "rk_npu_common.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Sharing key of an INT4 weight matrix B[K,N] (reference :21-24).
 * k_tile: multiple of 32 in 32..2048 (a tile above 480 must pass the INT16
 * partial-sum certificate of the reference for these codes), or 0 when passed
 * to rk_npu_w4a8_weights_create to let the library choose. */
typedef struct rk_npu_i4_weight_config {
    int K, N;
    int k_tile;
} rk_npu_i4_weight_config;

/* reference :26-35 */
typedef struct rk_npu_i4_config {
    int M, N, K;
    int m_tile;             /* 1..128                                         */
    int k_tile;             /* 32..2048, multiple of 32; must match the weights */
    int n_tile;             /* 64..8128, multiple of 64                       */
    uint32_t npu_core_mask; /* 1, 2, 4, 3 or 7; N needs that many 64-blocks   */
    uint32_t timeout_ms;    /* > 0                                            */
    int pipeline;           /* 0 or 1                                         */
    int cpu_threads;        /* 1..4                                           */
} rk_npu_i4_config;

/* Logical RK3588 buffer sizes as the reference accounts them (reference
 * :37-44), for callers that budget memory from these numbers.  control_bytes
 * (NPU command words and task descriptors) is reported as 0. */
typedef struct rk_npu_i4_memory_info {
    uint64_t packed_weight_bytes;
    uint64_t input_bytes;
    uint64_t partial_bytes;
    uint64_t control_bytes;
    uint32_t wave_count;
    uint32_t tasks_per_wave;
} rk_npu_i4_memory_info;

/* reference :46-51.  pack_us: producer calls / code checks / upload staging;
 * submit_us: device work; sync_us: waiting for it; reduce_us: result copy. */
typedef struct rk_npu_i4_timings {
    double pack_us, sync_us, submit_us, reduce_us, total_us;
} rk_npu_i4_timings;

typedef struct rk_npu_i4i4i32_weights rk_npu_i4i4i32_weights;
typedef struct rk_npu_i4_workspace rk_npu_i4_workspace;

/* {M, N, K, m_tile 128, k_tile 480, n_tile 1024, mask 1, 500 ms, pipeline 1,
 *  cpu_threads 1}  (reference :57) */
void rk_npu_i4_config_init(rk_npu_i4_config* cfg, int M, int N, int K);
/* Range validation + logical byte accounting (reference :58-59). */
int rk_npu_i4_memory_query(const rk_npu_i4_config* cfg, rk_npu_i4_memory_info* out);
int rk_npu_i4_weights_memory_query(const rk_npu_i4_weight_config* cfg, uint64_t* bytes);

/* B[K,N] is validated and packed once; it may be released afterwards.  NULL on
 * an invalid config, a code outside [-8,7], an uncertified k_tile > 480 or an
 * allocation failure.  (reference :66-68) */
rk_npu_i4i4i32_weights* rk_npu_i4i4i32_weights_create(rk_npu_iommu_domain* domain,
                                                      const rk_npu_i4_weight_config* cfg, const int8_t* B);
void rk_npu_i4i4i32_weights_free(rk_npu_i4i4i32_weights* weights);
rk_npu_i4_workspace* rk_npu_i4_workspace_create(rk_npu_iommu_domain* domain, const rk_npu_i4_config* cfg);
void rk_npu_i4_workspace_free(rk_npu_i4_workspace* workspace);

/* A[M,K] and C[M,N] must not alias.  A code outside [-8,7] returns
 * RK_NPU_ERR_PARAM (nothing is masked or truncated).  timings may be NULL.
 * Weights must match K / N / k_tile (PARAM) and the context / domain (DOMAIN).
 * (reference :76-78) */
int rk_npu_i4i4i32_run(rk_npu_i4_workspace* workspace, const rk_npu_i4i4i32_weights* weights,
                       const int8_t* A, int32_t* C, rk_npu_i4_timings* timings);

/* Input produced by the caller instead of read from A: `producer` is invoked
 * serially on the calling thread for each K tile and M panel, in increasing K
 * then M order.  dst is a zero-initialised [padded_k/32][rows][32] array of
 * INT4 codes, two per byte, the even element in the HIGH nibble; only the k
 * logical codes need writing.  dst is valid during the callback only.  A
 * non-zero return aborts the run with that code.  (reference :89-98) */
typedef struct rk_npu_i4_input_tile {
    int m0, rows, k0, k, padded_k;
    uint8_t* dst;
    uint64_t bytes;
} rk_npu_i4_input_tile;
typedef int (*rk_npu_i4_input_producer)(void* user, const rk_npu_i4_input_tile* tile);

int rk_npu_i4i4i32_run_with_producer(rk_npu_i4_workspace* workspace, const rk_npu_i4i4i32_weights* weights,
                                     rk_npu_i4_input_producer producer, void* user, int32_t* C,
                                     rk_npu_i4_timings* timings);

/* Host helper for producers: packs rows m0.. and columns k0.. of the full
 * matrix A (row stride lda >= k0 + k) into tile->dst, validating the codes.
 * (reference :102-103) */
int rk_npu_i4_pack_a_tile(const rk_npu_i4_input_tile* tile, const int8_t* A, int lda);

#ifdef __cplusplus
}
#endif
#endif /* RK_NPU_MATMUL_I4_H */
