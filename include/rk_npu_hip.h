/*
 * rk_npu_hip.h -- MI355X-only additions to the rk_npu_* C API.
 *
 * None of these entry points has a counterpart in the reference.  They exist
 * because the reference API hands over host buffers and blocks, which on a
 * discrete GPU puts a PCIe copy on both sides of every call.  Callers that
 * keep activations in HBM between layers (and the benchmark, which must time
 * the device path with inputs already resident) use the *_device variants:
 * same validation, same kernels, device pointers in and out, work enqueued on
 * the context's stream without waiting for it.
 *
 * Rules for the *_device calls:
 *   - pointers are device pointers valid on the context's device;
 *   - the call returns after enqueueing; rk_npu_hip_sync() (or any blocking
 *     reference call on the same context) waits for completion;
 *   - input rejection that needs a look at the data (NaN / Inf activations,
 *     non-finite SwiGLU middle) is reported by rk_npu_hip_sync() as
 *     RK_NPU_ERR_PARAM for the work enqueued since the previous sync;
 *   - the workspace stays BUSY only while the call enqueues, so the caller
 *     must not reuse a workspace from another thread before syncing.
 */
#ifndef RK_NPU_HIP_H
#define RK_NPU_HIP_H

#include "rk_npu_moe_w8.h"
#include "rk_npu_quant_matmul.h"
#include "rk_npu_w4a8.h"

#ifdef __cplusplus
extern "C" {
#endif

/* The context's hipStream_t (as void*), its device ordinal, and hardware facts
 * used to print rooflines. */
void* rk_npu_hip_stream(rk_npu_ctx* ctx);
int rk_npu_hip_device(const rk_npu_ctx* ctx);
int rk_npu_hip_device_info(const rk_npu_ctx* ctx, char* arch, int arch_len, int* cu_count,
                           int* clock_khz);
/* Wait for the context's stream; returns RK_NPU_ERR_PARAM if a kernel since the
 * last sync flagged rejected input, RK_NPU_ERR_SUBMIT on a runtime failure. */
int rk_npu_hip_sync(rk_npu_ctx* ctx);

/* Plain device memory helpers so that non-HIP callers can stage buffers. */
void* rk_npu_hip_malloc(rk_npu_ctx* ctx, size_t bytes);
void rk_npu_hip_free(rk_npu_ctx* ctx, void* ptr);
int rk_npu_hip_upload(rk_npu_ctx* ctx, void* dst_device, const void* src_host, size_t bytes);
int rk_npu_hip_download(rk_npu_ctx* ctx, void* dst_host, const void* src_device, size_t bytes);
/* Device-to-device copy enqueued on the context's stream (not waited for). */
int rk_npu_hip_copy(rk_npu_ctx* ctx, void* dst_device, const void* src_device, size_t bytes);

/* Stream timing (HIP events on the context's stream). */
typedef struct rk_npu_hip_event rk_npu_hip_event;
rk_npu_hip_event* rk_npu_hip_event_create(void);
void rk_npu_hip_event_free(rk_npu_hip_event* event);
int rk_npu_hip_event_record(rk_npu_ctx* ctx, rk_npu_hip_event* event);
/* Waits for `stop`; microseconds between the two records. */
int rk_npu_hip_event_elapsed_us(rk_npu_hip_event* start, rk_npu_hip_event* stop, double* us);

/* Device-resident variants of the blocking run calls. */
int rk_npu_i8i8i32_run_device(rk_npu_matmul_workspace* workspace,
                              const rk_npu_i8i8i32_weights* weights, const int8_t* A_device,
                              int32_t* C_device);
int rk_npu_f16i8f16_run_dynamic_device(rk_npu_matmul_workspace* workspace,
                                       const rk_npu_f16i8f16_weights* weights,
                                       const uint16_t* A_device, uint16_t* C_device);
int rk_npu_f32i8f32_run_dynamic_device(rk_npu_matmul_workspace* workspace,
                                       const rk_npu_f32i8f32_weights* weights,
                                       const float* A_device, float* C_device);
int rk_npu_w4a8_run_f16_device(rk_npu_w4a8_workspace* workspace,
                               const rk_npu_w4a8_weights* weights, const uint16_t* A_device,
                               uint16_t* C_device);
int rk_npu_w4a8_run_f32_device(rk_npu_w4a8_workspace* workspace,
                               const rk_npu_w4a8_weights* weights, const float* A_device,
                               float* C_device);
int rk_npu_w4a8_run_ffn_f32_device(rk_npu_w4a8_workspace* gate_up,
                                   const rk_npu_w4a8_weights* gate_up_weights,
                                   rk_npu_w4a8_workspace* down,
                                   const rk_npu_w4a8_weights* down_weights, const float* A_device,
                                   float* middle_device, float* C_device);
/* (The MoE layer: up to twelve tokens per call take two launches of dot-product kernels, more tokens the
 * five launches of the routed, grouped path; same results bit for bit.) */
int rk_npu_moe_w8_run_f32_device(rk_npu_moe_w8_workspace* workspace,
                                 const rk_npu_moe_w8_weights* weights, int rows,
                                 const float* input_device, const int32_t* expert_ids_device,
                                 const float* route_weights_device, float* output_device);

/* No counterpart in the reference.  rk_npu_f16i8f16_run_dynamic_device without a workspace
 * and without any allocation, for callers that cannot allocate: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  The scratch the kernels need (the
 * quantized rows, their scales, K-split partial tiles) lies in a static device array of
 * 12 MiB that each GPU the library runs on holds until the process ends; a shape whose rows
 * and scales need more (roughly align128(M) * align256(K) + 4 * align128(M), e.g. M = 2048
 * with K = 4096 fits, M = 4096 with K = 4096 does not) is rejected with RK_NPU_ERR_NOMEM
 * before any device work, and a shape whose partial tiles would not fit beside them runs
 * without the K split.  Device pointers in and out, work enqueued on the stream of the
 * context the weights belong to, nothing waited for; results are bit-identical to
 * rk_npu_f16i8f16_run_dynamic_device.  All calls on one GPU share the one array: calls
 * through the same context are ordered on its stream, calls that overlap on one GPU through
 * different contexts race. */
int rk_npu_f16i8f16_run_dynamic_noalloc_device(const rk_npu_f16i8f16_weights* weights, int M,
                                               const uint16_t* A_device, uint16_t* C_device);

/* Profiling hooks: launch only the GEMV / GEMM stage of an operator on the
 * activations its workspace quantized during the previous run, so that the
 * dominant kernel can be timed by itself with stream events.  `weights` is a
 * rk_npu_{i8i8i32,f16i8f16,f32i8f32}_weights handle matching the workspace's
 * op kind; the output element type is the workspace's (W8A8) or fp16 / fp32
 * as selected by `half` (W4A8). */
int rk_npu_matmul_workspace_rerun_gemm_device(rk_npu_matmul_workspace* workspace,
                                              const void* weights, void* C_device);
int rk_npu_w4a8_workspace_rerun_gemm_device(rk_npu_w4a8_workspace* workspace,
                                            const rk_npu_w4a8_weights* weights, void* C_device,
                                            int half);

/* Parity probes: the exact intermediates of the most recent run on a
 * workspace, copied to host.  q is the int8 activation matrix [M, K] in
 * row-major order, a_scale the per-row scales [M].  Blocking. */
int rk_npu_matmul_workspace_read_quantized(rk_npu_matmul_workspace* workspace, int8_t* q,
                                           float* a_scale);
int rk_npu_w4a8_workspace_read_quantized(rk_npu_w4a8_workspace* workspace, int8_t* q,
                                         float* a_scale);
/* int32 accumulators sum_k q[m,k] * B[k,n] of a W4A8 weight for host
 * activations A (fp32), through the same quantize + GEMM kernels.  Blocking. */
int rk_npu_w4a8_run_i32(rk_npu_w4a8_workspace* workspace, const rk_npu_w4a8_weights* weights,
                        const float* A, int32_t* acc);

/* Measurement probes: what the memory system and the matrix pipes of the box at hand give,
 * to put beside the datasheet peaks.  Each call enqueues ONE kernel on the context's stream
 * (time it with the events above):
 *   - a read-only pass over [src_device, src_device + bytes) in the decode GEMV's access
 *     order: one workgroup of eight waves per `span` bytes (a multiple of 1024; 131072 is the
 *     column block of a K = 4096 int8 matrix), 1 KiB pieces interleaved over the waves, 16
 *     bytes per lane, eight loads per wave in flight;
 *   - a pure int8 MFMA loop (v_mfma_i32_32x32x32_i8, eight waves per compute unit, four
 *     independent accumulators per wave, operands in registers, no memory traffic) on the
 *     32 KiB at operands_device -- the clock the chip sustains depends on the operands' bit
 *     patterns, so pass data like the workload's; *ops receives the operation count
 *     (2 * 32 * 32 * 32 per MFMA). */
int rk_npu_hip_probe_stream_read(rk_npu_ctx* ctx, const void* src_device, size_t bytes, size_t span);
int rk_npu_hip_probe_mfma_i8(rk_npu_ctx* ctx, const void* operands_device, int iterations, double* ops);

/* Per-kernel profile of the *_device calls: between profile_begin and profile_end a stream
 * event is recorded in front of every kernel the library launches on this context's stream.
 * profile_end waits for the stream and returns the number of kernels seen (or a negative
 * RK_NPU_ERR_*): us[i] is the time from the event in front of kernel i to the event in front
 * of kernel i + 1 (the last one: to the end of the work), i.e. the kernel plus the launch
 * gap behind it; names receives the kernels' names, one per line, as many as fit.  One
 * context at a time (RK_NPU_ERR_BUSY otherwise).  The events between the kernels cost a
 * little themselves: time whole steps without the profile. */
int rk_npu_hip_profile_begin(rk_npu_ctx* ctx);
int rk_npu_hip_profile_end(rk_npu_ctx* ctx, char* names, size_t names_bytes, double* us, int capacity);

/* Stream capture: the *_device calls made between capture_begin and capture_end on this
 * context (from the calling thread) are recorded instead of executed -- they only launch
 * kernels, no copy or memset node is ever recorded -- and graph_launch replays the recorded
 * sequence with one submission.  For decode loops, whose kernels are short enough that the
 * per-launch submission cost shows.  Run the sequence once eagerly before capturing it (first
 * use of a kernel may set function attributes); do not call rk_npu_hip_sync, blocking
 * reference calls or allocation calls on the context while capturing.  Rejected input (NaN /
 * Inf rows, expert ids out of range, negative coefficients) is reported by the next
 * rk_npu_hip_sync after a replay exactly as after the eager calls: the graph remembers the
 * workspaces it recorded and every launch registers their flags again.  A graph is launched on
 * the context it was captured on; free the workspaces it uses only when it is no longer
 * launched. */
typedef struct rk_npu_hip_graph rk_npu_hip_graph;
int rk_npu_hip_capture_begin(rk_npu_ctx* ctx);
rk_npu_hip_graph* rk_npu_hip_capture_end(rk_npu_ctx* ctx);
int rk_npu_hip_graph_launch(rk_npu_ctx* ctx, rk_npu_hip_graph* graph);
void rk_npu_hip_graph_free(rk_npu_hip_graph* graph);

/* Test hook: make the n-th next device allocation fail (1 = the next one,
 * 0 = off), to exercise RK_NPU_ERR_NOMEM / NULL-return paths from the host. */
void rk_npu_hip_fail_alloc_after(int n);

#ifdef __cplusplus
}
#endif
#endif /* RK_NPU_HIP_H */
