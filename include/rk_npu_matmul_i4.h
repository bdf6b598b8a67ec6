/*
 * rk_npu_matmul_i4.h -- the two INT4 structs that rk_npu_w4a8.h embeds.
 *
 * Only rk_npu_i4_weight_config and rk_npu_i4_memory_info of the reference's
 * include/rk_npu_matmul_i4.h (:21-24 and :37-44) are on the W4A8 path; the
 * exact W4A4 integer operator declared in the rest of that header is not part
 * of this library.
 */
#ifndef RK_NPU_MATMUL_I4_H
#define RK_NPU_MATMUL_I4_H

#include "rk_npu_common.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Sharing key of an INT4 weight matrix B[K,N] (reference :21-24).
 * k_tile: multiple of 32 in 32..2048, or 0 when passed to
 * rk_npu_w4a8_weights_create to let the library choose. */
typedef struct rk_npu_i4_weight_config {
    int K, N;
    int k_tile;
} rk_npu_i4_weight_config;

/* Logical RK3588 buffer sizes as the reference accounts them (reference
 * :37-44).  Reported for callers that budget memory from these numbers. */
typedef struct rk_npu_i4_memory_info {
    uint64_t packed_weight_bytes;
    uint64_t input_bytes;
    uint64_t partial_bytes;
    uint64_t control_bytes;
    uint32_t wave_count;
    uint32_t tasks_per_wave;
} rk_npu_i4_memory_info;

#ifdef __cplusplus
}
#endif
#endif /* RK_NPU_MATMUL_I4_H */
