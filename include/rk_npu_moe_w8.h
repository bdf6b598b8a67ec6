/*
 * rk_npu_moe_w8.h -- routed W8A8 SwiGLU experts (optional shared expert) on
 * MI355X.  The router is external: callers pass top-k expert ids and
 * coefficients.  Names, struct layouts and defaults follow the reference's
 * include/rk_npu_moe_w8.h (types :12-65, entry points :69-81 and :148-173).
 *
 * Numerical contract (fp32 arithmetic):
 *   token quantization: s = maxabs ? maxabs/127 : 1 ; q = RNE(clamp(x*(1/s), -127, 127))
 *   gate/up:  g = ((float)acc_g * s) * gs[n],  u = ((float)acc_u * s) * gs[I+n]
 *   hidden  = (g / (1 + exp(-g))) * u   with the degree-7 fp32 exp of the
 *             reference (src/rk_npu_swiglu_fp32_neon.h:13-51)
 *   s2      = maxabs(hidden) ? maxabs/127 : 1 ; q2 = RNE(clamp(hidden*(1/s2)))
 *   out[t,n] = sum over slots in order of fma(((float)acc2 * s2) * ds[n], w_slot, out)
 *             with the shared expert last and coefficient 1.
 * Routes with coefficient 0 are dropped before any device work; a call whose
 * every route is dropped zero-fills the output.
 *
 * Differences from the RK3588 limits: intermediate may be up to 8192 (the
 * reference stops at 512 because of a fixed CPU scratch row); npu_cores,
 * cpu_threads, native_input and timeout_ms are range-checked and unused.
 * INT4 experts, mixed banks, slot banks and packed expert records (reference
 * :83-143) are the same arithmetic with weight codes restricted to [-8, 7];
 * see the second half of this header.
 */
#ifndef RK_NPU_MOE_W8_H
#define RK_NPU_MOE_W8_H

#define RK_NPU_MOE_QUANT_BLOB_VERSION 3u
#include "rk_npu_common.h"

#ifdef __cplusplus
extern "C" {
#endif

/* reference :12-25.  Only RK_NPU_MOE_MIDDLE_CPU (the exact fp32 middle) is
 * accepted here; the approximate LUT middle is rejected at workspace_create. */
typedef enum rk_npu_moe_middle {
    RK_NPU_MOE_MIDDLE_CPU = 0,
    RK_NPU_MOE_MIDDLE_NPU_LUT = 1
} rk_npu_moe_middle;

/* reference :27-32 */
typedef struct rk_npu_moe_w8_weight_config {
    int hidden;         /* >= 64, multiple of 32        */
    int intermediate;   /* 32..8192, multiple of 32     */
    int routed_experts; /* 1..4096                      */
    int shared_expert;  /* 0 or 1; its index is routed_experts */
} rk_npu_moe_w8_weight_config;

/* reference :34-44 */
typedef struct rk_npu_moe_w8_config {
    uint32_t struct_size;
    rk_npu_moe_w8_weight_config weights;
    int max_rows;     /* 1..256 */
    int top_k;        /* 1..min(routed_experts, 8) */
    int npu_cores;    /* 1..3 */
    int cpu_threads;  /* 1..4 */
    int native_input; /* 0 or 1 */
    rk_npu_moe_middle middle;
    uint32_t timeout_ms; /* 1..60000 */
} rk_npu_moe_w8_config;

/* One expert's host tensors; copied by weights_create (reference :46-53). */
typedef struct rk_npu_moe_w8_expert {
    const int8_t* gate_up;       /* [hidden, 2*intermediate], gate columns then up columns */
    const float* gate_up_scales; /* [2*intermediate], finite > 0 */
    const int8_t* down;          /* [intermediate, hidden] */
    const float* down_scales;    /* [hidden], finite > 0 */
} rk_npu_moe_w8_expert;

/* reference :55-62.  input_us = token quantize + scatter, schedule_us =
 * device-side sort by expert, gate_us / down_us = grouped GEMMs,
 * middle_cpu_us = the re-quantize kernel, combine_us = weighted sum,
 * sync_us = host<->device copies. */
typedef struct rk_npu_moe_w8_timings {
    double input_us, schedule_us, build_us, sync_us, gather_us;
    double gate_us, middle_npu_us, middle_cpu_us, down_us, combine_us;
    double lut_load_us;
    double total_us;
    uint32_t gather_tasks, middle_tasks, gemm_tasks;
} rk_npu_moe_w8_timings;

typedef struct rk_npu_moe_w8_weights rk_npu_moe_w8_weights;
typedef struct rk_npu_moe_w8_workspace rk_npu_moe_w8_workspace;

/* {sizeof, {hidden, intermediate, routed_experts, shared_expert}, max_rows,
 *  top_k, npu_cores 3, cpu_threads 4, native_input 0, MIDDLE_CPU, 1000 ms}
 * (reference :69-71) */
void rk_npu_moe_w8_config_init(rk_npu_moe_w8_config* config, int hidden, int intermediate,
                               int routed_experts, int shared_expert, int top_k, int max_rows);

/* experts[routed_experts + shared_expert]; NULL on invalid configuration,
 * scale or allocation failure (reference :76-78). */
rk_npu_moe_w8_weights* rk_npu_moe_w8_weights_create(rk_npu_iommu_domain* domain,
                                                    const rk_npu_moe_w8_weight_config* config,
                                                    const rk_npu_moe_w8_expert* experts);
void rk_npu_moe_w8_weights_free(rk_npu_moe_w8_weights* weights);
rk_npu_moe_w8_workspace* rk_npu_moe_w8_workspace_create(rk_npu_iommu_domain* domain,
                                                        const rk_npu_moe_w8_config* config);
void rk_npu_moe_w8_workspace_free(rk_npu_moe_w8_workspace* workspace);

/* Device bytes held (reference :148-149). */
uint64_t rk_npu_moe_w8_weights_device_bytes(const rk_npu_moe_w8_weights* weights);
uint64_t rk_npu_moe_w8_workspace_device_bytes(const rk_npu_moe_w8_workspace* workspace);

/* expert_ids / route_weights are [rows, top_k]; ids in [0, routed_experts),
 * coefficients finite and >= 0; output is fp32 [rows, hidden]; input, ids and
 * coefficients must not overlap output; 1 <= rows <= max_rows.
 * (reference :166-173) */
int rk_npu_moe_w8_run_quantized(rk_npu_moe_w8_workspace* workspace,
                                const rk_npu_moe_w8_weights* weights, int rows,
                                const int8_t* input, const float* row_scales,
                                const int32_t* expert_ids, const float* route_weights,
                                float* output, rk_npu_moe_w8_timings* timings);
int rk_npu_moe_w8_run_f32(rk_npu_moe_w8_workspace* workspace,
                          const rk_npu_moe_w8_weights* weights, int rows, const float* input,
                          const int32_t* expert_ids, const float* route_weights,
                          float* output, rk_npu_moe_w8_timings* timings);

/* ---- INT4 experts, mixed banks, slot banks, packed records (reference :83-143) ----
 *
 * Expert tensors are passed exactly as for the W8 factories (one int8_t per
 * weight, the same scale vectors); an INT4 expert's codes must lie in [-8, 7].
 * On the RK3588 these formats select the NPU's int4 mode, K-sliced INT16
 * partials and their certificates; here INT4 experts are held and streamed as
 * packed nibbles (half the bytes of a W8 expert, as
 * rk_npu_moe_w8_weights_device_bytes reports), unpacked in registers to int8
 * MFMA operands and accumulated in int32 without any intermediate narrowing,
 * so results are bit-identical to the W8 path given the same codes.  What is
 * kept from the reference is the contract: geometry (hidden and intermediate
 * multiples of 64, hidden <= 8128), code range validation, native_input = 0,
 * and that weights only bind to a workspace made by the factory of the same
 * format (RK_NPU_ERR_PARAM otherwise).  All handles use the run / free / byte
 * query functions above.
 *
 *   quant_*      every expert INT4, the shared one included (reference :83-94).
 *                _full_k is the same here: there is no K slicing to certify.
 *   w4_*         routed experts INT4, the shared expert full-range int8
 *                (reference :96-106).
 *   *_slots_create  a bank whose routed slots start empty (zero weights, zero
 *                scales) and are filled by import; quant_slots needs
 *                shared_expert = 0, w4_slots needs shared_expert = 1 and packs
 *                `shared` at creation (reference :101-119).  The caller owns
 *                the logical expert -> slot map and passes slot numbers as
 *                expert_ids.
 *
 * Packed record of one INT4 expert, rk_npu_moe_quant_expert_blob_bytes() bytes
 * (0 for W8 handles): a 40-byte header {u32 magic "RKH4", u32
 * RK_NPU_MOE_QUANT_BLOB_VERSION, u32 hidden, u32 intermediate, u32 layout revision (2), u32 0,
 * u64 gate/up image bytes, u64 down image bytes}, the gate/up image (align256(2*intermediate) *
 * align256(hidden) / 2 bytes) and the down image (align256(hidden) *
 * align256(intermediate) / 2 bytes) in this library's execution layout -- 1 KiB
 * tiles of 32 columns x 64 k, two codes per byte, gate/up column blocks
 * interleaved --, 2*intermediate gate/up scales, hidden down scales (fp32,
 * little endian).  Records are native to this library (not interchangeable with the
 * RK3588 build's) and identical between the all-INT4 and the mixed bank of one
 * geometry.  export / import accept a larger buffer than the record, reject a
 * shorter one, a W8 handle, the shared int8 expert, an out-of-range slot, a
 * foreign header (another magic, blob version, geometry, layout revision or image size: records
 * written by an earlier build of this library, which held the codes as int8 tiles under the
 * magic "RKHM", are rejected) and non-finite or non-positive scales with RK_NPU_ERR_PARAM;
 * a rejected import leaves the slot unchanged.  Import only between blocking
 * runs that use the bank.  The timed import reports validate_us (header and
 * scale checks), copy_us (scales), gate_sync_us / down_sync_us (the two weight
 * images) and total_us.
 *
 * swap_slots exchanges the contents of two slots of all-INT4 banks of equal
 * geometry in the same context and domain (device-side copy; the reference
 * exchanges buffer ownership, the observable result is the same). */
typedef struct rk_npu_moe_import_timings {
    double copy_us, validate_us, gate_sync_us, down_sync_us, total_us;
} rk_npu_moe_import_timings;

rk_npu_moe_w8_weights* rk_npu_moe_quant_weights_create(rk_npu_iommu_domain* domain,
                                                       const rk_npu_moe_w8_weight_config* config,
                                                       const rk_npu_moe_w8_expert* experts);
rk_npu_moe_w8_weights* rk_npu_moe_quant_weights_create_full_k(rk_npu_iommu_domain* domain,
                                                              const rk_npu_moe_w8_weight_config* config,
                                                              const rk_npu_moe_w8_expert* experts);
rk_npu_moe_w8_workspace* rk_npu_moe_quant_workspace_create(rk_npu_iommu_domain* domain,
                                                           const rk_npu_moe_w8_config* config);
rk_npu_moe_w8_weights* rk_npu_moe_w4_weights_create(rk_npu_iommu_domain* domain,
                                                    const rk_npu_moe_w8_weight_config* config,
                                                    const rk_npu_moe_w8_expert* experts);
rk_npu_moe_w8_workspace* rk_npu_moe_w4_workspace_create(rk_npu_iommu_domain* domain,
                                                        const rk_npu_moe_w8_config* config);
rk_npu_moe_w8_weights* rk_npu_moe_w4_slots_create(rk_npu_iommu_domain* domain,
                                                  const rk_npu_moe_w8_weight_config* config,
                                                  const rk_npu_moe_w8_expert* shared);
rk_npu_moe_w8_weights* rk_npu_moe_quant_slots_create(rk_npu_iommu_domain* domain,
                                                     const rk_npu_moe_w8_weight_config* config);
uint64_t rk_npu_moe_quant_expert_blob_bytes(const rk_npu_moe_w8_weights* weights);
int rk_npu_moe_quant_export_expert(const rk_npu_moe_w8_weights* weights, int expert, void* data,
                                   uint64_t bytes);
int rk_npu_moe_quant_import_expert(rk_npu_moe_w8_weights* weights, int slot, const void* data,
                                   uint64_t bytes);
int rk_npu_moe_quant_import_expert_timed(rk_npu_moe_w8_weights* weights, int slot, const void* data,
                                         uint64_t bytes, rk_npu_moe_import_timings* timings);
int rk_npu_moe_quant_swap_slots(rk_npu_moe_w8_weights* first, int first_slot,
                                rk_npu_moe_w8_weights* second, int second_slot);

#ifdef __cplusplus
}
#endif
#endif /* RK_NPU_MOE_W8_H */
