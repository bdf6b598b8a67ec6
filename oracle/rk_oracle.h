/*
 * rk_oracle.h -- CPU restatement of the reference's quantized-linear hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this code; it exists so that tests, the smoke check and the CPU
 * baseline leg of the benchmark have an independent statement of what the
 * reference computes.  Each function cites the reference file:line it
 * follows (paths relative to the reference checkout).
 *
 * Parity status of each group is stated in rk_oracle.c's header.
 */
#ifndef RK_ORACLE_H
#define RK_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_OK 0
#define ORC_ERR_PARAM (-3)

/* SwiGLU exponential flavour. */
#define ORC_EXP_POLY 0 /* degree-7 fp32 polynomial (the AArch64 production path) */
#define ORC_EXP_LIBM 1 /* expf, the reference's scalar fallback off AArch64      */

int orc_num_threads(void);

/* binary16 <-> binary32 */
float orc_half_to_float(uint16_t h);
uint16_t orc_float_to_half(float f);
void orc_half_to_float_n(const uint16_t* src, float* dst, int64_t n);
void orc_float_to_half_n(const float* src, uint16_t* dst, int64_t n);

/* W8A8 activation quantization (ties away from zero, no finite check). */
void orc_w8_scales_f16(int M, int K, const uint16_t* A, float* scale);
void orc_w8_scales_f32(int M, int K, const float* A, float* scale);
void orc_w8_quant_f16(int M, int K, const uint16_t* A, const float* scale, int8_t* q);
void orc_w8_quant_f32(int M, int K, const float* A, const float* scale, int8_t* q);

/* W4A8 activation quantization (FLT_MIN floor, finite check, ties away). */
int orc_w4a8_scales_f16(int M, int K, const uint16_t* A, float* scale, float* inverse);
int orc_w4a8_scales_f32(int M, int K, const float* A, float* scale, float* inverse);
void orc_w4a8_quant_f16(int M, int K, const uint16_t* A, const float* inverse, int8_t* q);
void orc_w4a8_quant_f32(int M, int K, const float* A, const float* inverse, int8_t* q);
/* The reference's INT8 -> two INT4 split and its inverse identity. */
void orc_w4a8_msd_split(int8_t q, int* high, int* low);

/* MoE row quantization (ties to even).  Returns the scale, or 0 when
 * validate != 0 and the row holds NaN/Inf. */
float orc_moe_quant_row(const float* x, int n, int validate, int8_t* q);

/* Exact integer GEMM: C[M,N] = A[M,K] * B[K,N], int32 wrap-around. */
void orc_gemm_i8(int M, int N, int K, const int8_t* A, const int8_t* B, int32_t* C);

/* y = ((float)acc * a_scale[m]) * w_scale[n] */
void orc_dequant_f32(int M, int N, const int32_t* acc, const float* a_scale,
                     const float* w_scale, float* C);
void orc_dequant_f16(int M, int N, const int32_t* acc, const float* a_scale,
                     const float* w_scale, uint16_t* C);

/* SwiGLU pieces. */
float orc_silu_mul(float g, float u, int flavour);
void orc_swiglu(int M, int F, const int32_t* acc /* [M,2F] */, const float* a_scale,
                const float* w_scale /* [2F] */, int flavour, float* middle /* [M,F] */,
                uint32_t* row_max_bits /* [M] or NULL */);
int orc_finish_scales(int M, const uint32_t* row_max_bits, float* scale, float* inverse);

/* Whole operators.  Optional outputs (may be NULL) expose the intermediates
 * that parity tests compare bit-exactly: q = int8 activations, acc = int32
 * accumulators. */
void orc_w8a8_f16(int M, int N, int K, const uint16_t* A, const int8_t* B,
                  const float* w_scale, const float* a_scale_static /* or NULL */,
                  uint16_t* C, int8_t* q_out, float* a_scale_out, int32_t* acc_out);
void orc_w8a8_f32(int M, int N, int K, const float* A, const int8_t* B,
                  const float* w_scale, const float* a_scale_static /* or NULL */,
                  float* C, int8_t* q_out, float* a_scale_out, int32_t* acc_out);
int orc_w4a8_f16(int M, int N, int K, const uint16_t* A, const int8_t* B,
                 const float* w_scale, uint16_t* C, int8_t* q_out, float* a_scale_out,
                 int32_t* acc_out);
int orc_w4a8_f32(int M, int N, int K, const float* A, const int8_t* B,
                 const float* w_scale, float* C, int8_t* q_out, float* a_scale_out,
                 int32_t* acc_out);
int orc_w4a8_swiglu_f32(int M, int N, int K, const float* A, const int8_t* B,
                        const float* w_scale, int flavour, float* middle,
                        uint32_t* row_max_bits, int32_t* acc_out);
int orc_w4a8_ffn_f32(int M, int H, int I, int Nout, const float* A,
                     const int8_t* B_gate_up /* [H,2I] */, const float* s_gate_up,
                     const int8_t* B_down /* [I,Nout] */, const float* s_down, int flavour,
                     float* middle /* [M,I] */, float* C /* [M,Nout] */,
                     int8_t* q_down_out /* [M,I] or NULL */,
                     float* down_scale_out /* [M] or NULL */,
                     int32_t* acc_down_out /* [M,Nout] or NULL */);

/* One expert's tensors, as rk_npu_moe_w8_expert. */
typedef struct orc_moe_expert {
    const int8_t* gate_up;       /* [H, 2I] */
    const float* gate_up_scales; /* [2I]    */
    const int8_t* down;          /* [I, H]  */
    const float* down_scales;    /* [H]     */
} orc_moe_expert;

/* input_f32 != NULL: quantize each token (ties even); else use input_q +
 * row_scales.  experts has E + shared entries.  fused_combine != 0 sums with
 * fmaf (AArch64 path and the reference test oracle), 0 uses mul + add. */
int orc_moe_w8(int rows, int H, int I, int E, int shared, int top_k,
               const orc_moe_expert* experts, const float* input_f32, const int8_t* input_q,
               const float* row_scales, const int32_t* ids, const float* routes, int flavour,
               int fused_combine, float* out /* [rows,H] */);

#ifdef __cplusplus
}
#endif
#endif
