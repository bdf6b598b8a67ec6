/*
 * rk_oracle.c -- CPU restatement of the reference's quantized-linear hot path.
 *
 * TEST INFRASTRUCTURE ONLY: used by tests, the smoke check and the CPU
 * baseline leg of the benchmark.  The shipped library never links or calls it.
 *
 * Build: gcc -O3 -march=x86-64-v3 -ffp-contract=off -fopenmp -shared -fPIC
 * (-ffp-contract=off matters: every place the reference fuses a multiply-add
 * is written as an explicit fmaf below; nothing else may be contracted.)
 *
 * What pins each group (checked by the CPU tests):
 *   half conversions   exhaustive 65536-pattern round trip + numpy float16
 *   W8A8 / W4A8 quant  tie / FLT_MIN / zero-row / NaN known answers of the
 *                      reference's own unit tests, and the compiled reference
 *                      translation units where they build
 *   MoE quant          ties-to-even anchors of the reference's MoE test
 *   integer GEMM       int64 brute force, split-K linearity, permutations
 *   dequant            known answers with sums above 2^24
 *   SwiGLU, libm       the compiled reference translation units (x86 build)
 *   SwiGLU, poly       restated from the NEON source text; pinned by the
 *                      reference's own bound |poly - expf| <= 7e-7 relative,
 *                      by exact special cases (g=0, g<-80, saturation) and by
 *                      an independent float64 evaluation of the same steps.
 *                      The NEON kernel itself cannot be compiled on x86.
 *   FFN / MoE          composition of the above + the reference test oracle's
 *                      formula on its own test inputs
 */
#include "rk_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------ half */

/* reference src/rk_npu_half_bits.h:8-28 and src/rk_npu_cpu_kernels.cpp:74-96 */
float orc_half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 31u;
    uint32_t m = h & 1023u;
    uint32_t bits;
    if (e == 0) {
        if (m == 0) {
            bits = sign;
        } else {
            int shift = 0;
            while (!(m & 1024u)) {
                m <<= 1;
                ++shift;
            }
            bits = sign | ((uint32_t)(113 - shift) << 23) | ((m & 1023u) << 13);
        }
    } else if (e == 31) {
        bits = sign | 0x7f800000u | (m << 13);
    } else {
        bits = sign | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* Round to nearest even, subnormals kept, overflow to Inf, NaN stays NaN.
 * reference src/rk_npu_half_bits.h:29-51 */
uint16_t orc_float_to_half(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t raw = (x >> 23) & 255u;
    uint32_t man = x & 0x7fffffu;
    const int e = (int)raw - 112;
    if (raw == 255u) return (uint16_t)(sign | 0x7c00u | (man ? ((man >> 13) | 0x200u) : 0u));
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        const int shift = 14 - e;
        uint32_t hm = man >> shift;
        const uint32_t rb = 1u << (shift - 1);
        if ((man & rb) && ((man & (rb - 1u)) || (hm & 1u))) ++hm;
        return (uint16_t)(sign | hm);
    }
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    uint32_t h = sign | ((uint32_t)e << 10) | (man >> 13);
    if ((man & 0x1000u) && ((man & 0xfffu) || (h & 1u))) ++h;
    return (uint16_t)h;
}

void orc_half_to_float_n(const uint16_t* src, float* dst, int64_t n) {
#pragma omp parallel for schedule(static) if (n >= (1 << 16))
    for (int64_t i = 0; i < n; ++i) dst[i] = orc_half_to_float(src[i]);
}
void orc_float_to_half_n(const float* src, uint16_t* dst, int64_t n) {
#pragma omp parallel for schedule(static) if (n >= (1 << 16))
    for (int64_t i = 0; i < n; ++i) dst[i] = orc_float_to_half(src[i]);
}

/* ------------------------------------------------------------ W8A8 quant */

/* reference src/rk_npu_cpu_kernels.cpp:628-646 (f16) and :853-871 (f32):
 * scale = maxabs > 0 ? maxabs / 127 : 1 */
void orc_w8_scales_f32(int M, int K, const float* A, float* scale) {
#pragma omp parallel for schedule(static) if ((int64_t)M * K >= (1 << 14))
    for (int m = 0; m < M; ++m) {
        const float* row = A + (size_t)m * K;
        float mx = 0.0f;
        for (int k = 0; k < K; ++k) {
            const float a = fabsf(row[k]);
            mx = a > mx ? a : mx; /* std::max(mx, a): NaN never replaces mx */
        }
        scale[m] = mx > 0.0f ? mx / 127.0f : 1.0f;
    }
}
void orc_w8_scales_f16(int M, int K, const uint16_t* A, float* scale) {
#pragma omp parallel for schedule(static) if ((int64_t)M * K >= (1 << 14))
    for (int m = 0; m < M; ++m) {
        const uint16_t* row = A + (size_t)m * K;
        float mx = 0.0f;
        for (int k = 0; k < K; ++k) {
            const float a = fabsf(orc_half_to_float(row[k]));
            mx = a > mx ? a : mx;
        }
        scale[m] = mx > 0.0f ? mx / 127.0f : 1.0f;
    }
}

/* reference src/rk_npu_cpu_kernels.cpp:127-132: multiply by the reciprocal,
 * round half away from zero, clamp the rounded float. */
static inline int8_t w8_quant_one(float x, float scale) {
    if (!(scale > 0.0f)) return 0;
    float q = roundf(x * (1.0f / scale));
    q = q < 127.0f ? q : 127.0f;   /* std::min(127, q) */
    q = q > -127.0f ? q : -127.0f; /* std::max(-127, .) */
    return (int8_t)q;
}
void orc_w8_quant_f32(int M, int K, const float* A, const float* scale, int8_t* q) {
#pragma omp parallel for schedule(static) if ((int64_t)M * K >= (1 << 14))
    for (int m = 0; m < M; ++m)
        for (int k = 0; k < K; ++k)
            q[(size_t)m * K + k] = w8_quant_one(A[(size_t)m * K + k], scale[m]);
}
void orc_w8_quant_f16(int M, int K, const uint16_t* A, const float* scale, int8_t* q) {
#pragma omp parallel for schedule(static) if ((int64_t)M * K >= (1 << 14))
    for (int m = 0; m < M; ++m)
        for (int k = 0; k < K; ++k)
            q[(size_t)m * K + k] = w8_quant_one(orc_half_to_float(A[(size_t)m * K + k]), scale[m]);
}

/* ------------------------------------------------------------ W4A8 quant */

/* reference src/rk_npu_w4a8_quant.cpp:52-85 */
static int w4a8_scale_row(const float* row32, const uint16_t* row16, int K, float* scale,
                          float* inverse) {
    int bad = 0;
    float mx = 0.0f;
    for (int k = 0; k < K; ++k) {
        const float x = row32 ? row32[k] : orc_half_to_float(row16[k]);
        if (!isfinite(x)) bad = 1;
        const float a = fabsf(x);
        mx = a > mx ? a : mx;
    }
    float s = 1.0f;
    if (mx != 0.0f) {
        s = mx / 127.0f;
        if (!(s > FLT_MIN)) s = FLT_MIN; /* std::max(mx/127, FLT_MIN) */
    }
    *scale = s;
    *inverse = 1.0f / s;
    return bad;
}
int orc_w4a8_scales_f32(int M, int K, const float* A, float* scale, float* inverse) {
    int bad = 0;
#pragma omp parallel for schedule(static) reduction(| : bad) if ((int64_t)M * K >= 8192)
    for (int m = 0; m < M; ++m)
        bad |= w4a8_scale_row(A + (size_t)m * K, NULL, K, scale + m, inverse + m);
    return bad ? ORC_ERR_PARAM : ORC_OK;
}
int orc_w4a8_scales_f16(int M, int K, const uint16_t* A, float* scale, float* inverse) {
    int bad = 0;
#pragma omp parallel for schedule(static) reduction(| : bad) if ((int64_t)M * K >= 8192)
    for (int m = 0; m < M; ++m)
        bad |= w4a8_scale_row(NULL, A + (size_t)m * K, K, scale + m, inverse + m);
    return bad ? ORC_ERR_PARAM : ORC_OK;
}

/* reference src/rk_npu_w4a8_quant.cpp:119-121 */
static inline int8_t w4a8_quant_one(float x, float inverse) {
    float q = roundf(x * inverse);
    q = q < 127.0f ? q : 127.0f;
    q = q > -127.0f ? q : -127.0f;
    return (int8_t)(int)q;
}
void orc_w4a8_quant_f32(int M, int K, const float* A, const float* inverse, int8_t* q) {
#pragma omp parallel for schedule(static) if ((int64_t)M * K >= 8192)
    for (int m = 0; m < M; ++m)
        for (int k = 0; k < K; ++k)
            q[(size_t)m * K + k] = w4a8_quant_one(A[(size_t)m * K + k], inverse[m]);
}
void orc_w4a8_quant_f16(int M, int K, const uint16_t* A, const float* inverse, int8_t* q) {
#pragma omp parallel for schedule(static) if ((int64_t)M * K >= 8192)
    for (int m = 0; m < M; ++m)
        for (int k = 0; k < K; ++k)
            q[(size_t)m * K + k] =
                w4a8_quant_one(orc_half_to_float(A[(size_t)m * K + k]), inverse[m]);
}

/* reference src/rk_npu_w4a8_quant.cpp:122 : h = q >> 4 (arithmetic),
 * l = (q & 15) - 8, so that q == 16*h + l + 8. */
void orc_w4a8_msd_split(int8_t q, int* high, int* low) {
    const uint8_t u = (uint8_t)q;
    const int h4 = u >> 4;              /* 0..15, two's-complement nibble */
    const int l4 = (u & 15) ^ 8;        /* nibble of (q & 15) - 8          */
    *high = h4 >= 8 ? h4 - 16 : h4;
    *low = l4 >= 8 ? l4 - 16 : l4;
}

/* ------------------------------------------------------------- MoE quant */

/* reference src/rk_npu_moe_w8.cpp:317-344 (token rows, validate) and
 * src/rk_npu_moe_cpu.cpp:78-97 (hidden rows): scale = max ? max/127 : 1,
 * clamp first, then round to nearest even. */
float orc_moe_quant_row(const float* x, int n, int validate, int8_t* q) {
    float mx = 0.0f;
    for (int i = 0; i < n; ++i) {
        if (validate && !isfinite(x[i])) return 0.0f;
        const float a = fabsf(x[i]);
        mx = a > mx ? a : mx;
    }
    const float scale = mx != 0.0f ? mx / 127.0f : 1.0f;
    const float inv = 1.0f / scale;
    if (validate && (!(scale > 0.0f) || !isfinite(inv))) return 0.0f;
    for (int i = 0; i < n; ++i) {
        float v = x[i] * inv;
        v = v < 127.0f ? v : 127.0f;
        v = v > -127.0f ? v : -127.0f;
        const float base = floorf(v);
        const float fraction = v - base;
        int code = (int)base;
        if (fraction > 0.5f || (fraction == 0.5f && (code & 1))) ++code;
        q[i] = (int8_t)code;
    }
    return scale;
}

/* ------------------------------------------------------------------ GEMM */

/* The reference has no CPU GEMM (its NPU does the MACs); every reference test
 * asserts the textbook exact product, e.g. tests/test_quant_matmul.cpp:93-104.
 * Accumulation is in uint32 so overflow wraps mod 2^32 as the API documents
 * (include/rk_npu_quant_matmul.h:333-334). */
void orc_gemm_i8(int M, int N, int K, const int8_t* A, const int8_t* B, int32_t* C) {
    enum { MB = 4, NB = 512 };
    const int mblocks = (M + MB - 1) / MB, nblocks = (N + NB - 1) / NB;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int nb = 0; nb < nblocks; ++nb) {
        for (int mb = 0; mb < mblocks; ++mb) {
            const int n0 = nb * NB, nn = N - n0 < NB ? N - n0 : NB;
            const int m0 = mb * MB, mm = M - m0 < MB ? M - m0 : MB;
            int32_t acc[MB][NB];
            memset(acc, 0, sizeof(acc));
            for (int k = 0; k < K; ++k) {
                const int8_t* brow = B + (size_t)k * N + n0;
                for (int r = 0; r < mm; ++r) {
                    const int32_t a = A[(size_t)(m0 + r) * K + k];
                    int32_t* dst = acc[r];
                    for (int n = 0; n < nn; ++n)
                        dst[n] = (int32_t)((uint32_t)dst[n] + (uint32_t)(a * (int32_t)brow[n]));
                }
            }
            for (int r = 0; r < mm; ++r)
                memcpy(C + (size_t)(m0 + r) * N + n0, acc[r], (size_t)nn * sizeof(int32_t));
        }
    }
}

/* --------------------------------------------------------------- dequant */

/* reference src/rk_npu_cpu_kernels.cpp:1393-1474 and
 * src/rk_npu_w4a8_output.cpp:68-80 : (float(acc) * a_scale) * w_scale */
void orc_dequant_f32(int M, int N, const int32_t* acc, const float* a_scale,
                     const float* w_scale, float* C) {
#pragma omp parallel for schedule(static) if ((int64_t)M * N >= (1 << 14))
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n)
            C[(size_t)m * N + n] = ((float)acc[(size_t)m * N + n] * a_scale[m]) * w_scale[n];
}
void orc_dequant_f16(int M, int N, const int32_t* acc, const float* a_scale,
                     const float* w_scale, uint16_t* C) {
#pragma omp parallel for schedule(static) if ((int64_t)M * N >= (1 << 14))
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n)
            C[(size_t)m * N + n] =
                orc_float_to_half(((float)acc[(size_t)m * N + n] * a_scale[m]) * w_scale[n]);
}

/* ---------------------------------------------------------------- SwiGLU */

/* Degree-7 fp32 exponential of reference src/rk_npu_swiglu_fp32_neon.h:13-51,
 * step for step: every vfmaq / vfmsq there is one fmaf here, min/max/floor/
 * divide are single IEEE operations.  d = 1 + p * 2^n: the product is exact
 * (power of two, no under/overflow for |n| <= 116), so it does not matter
 * whether the compiler fuses it. */
static inline float silu_poly(float g) {
    float x = -g;
    x = x < 80.0f ? x : 80.0f;
    x = x > -80.0f ? x : -80.0f;
    const float n = floorf(fmaf(x, 1.4426950408889634f, 0.5f));
    float r = fmaf(-n, 0.693145751953125f, x);
    r = fmaf(-n, 1.428606765330187e-6f, r);
    float p = 1.0f / 5040.0f;
    p = fmaf(p, r, 1.0f / 720.0f);
    p = fmaf(p, r, 1.0f / 120.0f);
    p = fmaf(p, r, 1.0f / 24.0f);
    p = fmaf(p, r, 1.0f / 6.0f);
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    const int32_t ni = (int32_t)n; /* NaN cannot reach here through a finite clamp */
    const uint32_t pbits = (uint32_t)(ni + 127) << 23;
    float power;
    memcpy(&power, &pbits, 4);
    const float d = 1.0f + p * power;
    return g < -80.0f ? -0.0f : g / d;
}

/* reference src/rk_npu_w4a8_swiglu.cpp:71 (libm flavour) / :82-87 (poly). */
float orc_silu_mul(float g, float u, int flavour) {
    if (flavour == ORC_EXP_LIBM) return (g / (1.0f + expf(-g))) * u;
    return silu_poly(g) * u;
}

/* reference src/rk_npu_w4a8_swiglu.cpp:61-78: gate column n, up column F+n;
 * row maximum is taken over the raw bit patterns with the sign cleared. */
void orc_swiglu(int M, int F, const int32_t* acc, const float* a_scale, const float* w_scale,
                int flavour, float* middle, uint32_t* row_max_bits) {
#pragma omp parallel for schedule(static) if ((int64_t)M * F >= (1 << 12))
    for (int m = 0; m < M; ++m) {
        uint32_t mx = 0;
        for (int n = 0; n < F; ++n) {
            const float g = ((float)acc[(size_t)m * 2 * F + n] * a_scale[m]) * w_scale[n];
            const float u = ((float)acc[(size_t)m * 2 * F + F + n] * a_scale[m]) * w_scale[F + n];
            const float y = orc_silu_mul(g, u, flavour);
            middle[(size_t)m * F + n] = y;
            uint32_t bits;
            memcpy(&bits, &y, 4);
            bits &= 0x7fffffffu;
            mx = bits > mx ? bits : mx;
        }
        if (row_max_bits) row_max_bits[m] = mx;
    }
}

/* reference src/rk_npu_w4a8_quant.cpp:145-161 */
int orc_finish_scales(int M, const uint32_t* row_max_bits, float* scale, float* inverse) {
    for (int m = 0; m < M; ++m) {
        const uint32_t bits = row_max_bits[m];
        if (bits >= 0x7f800000u) return ORC_ERR_PARAM;
        float mx;
        memcpy(&mx, &bits, 4);
        float s = 1.0f;
        if (mx != 0.0f) {
            s = mx / 127.0f;
            if (!(s > FLT_MIN)) s = FLT_MIN;
        }
        scale[m] = s;
        inverse[m] = 1.0f / s;
    }
    return ORC_OK;
}

/* ------------------------------------------------------- whole operators */

/* reference src/rk_npu_quant_matmul.cpp:799-878 (scale -> quantize -> exact
 * GEMM -> dequant) with the dynamic / static scale choice of :1855-1906. */
void orc_w8a8_f16(int M, int N, int K, const uint16_t* A, const int8_t* B,
                  const float* w_scale, const float* a_scale_static, uint16_t* C,
                  int8_t* q_out, float* a_scale_out, int32_t* acc_out) {
    float* s = (float*)malloc((size_t)M * sizeof(float));
    int8_t* q = q_out ? q_out : (int8_t*)malloc((size_t)M * K);
    int32_t* acc = acc_out ? acc_out : (int32_t*)malloc((size_t)M * N * sizeof(int32_t));
    if (a_scale_static) memcpy(s, a_scale_static, (size_t)M * sizeof(float));
    else orc_w8_scales_f16(M, K, A, s);
    orc_w8_quant_f16(M, K, A, s, q);
    orc_gemm_i8(M, N, K, q, B, acc);
    if (C) orc_dequant_f16(M, N, acc, s, w_scale, C);
    if (a_scale_out) memcpy(a_scale_out, s, (size_t)M * sizeof(float));
    free(s);
    if (!q_out) free(q);
    if (!acc_out) free(acc);
}
void orc_w8a8_f32(int M, int N, int K, const float* A, const int8_t* B, const float* w_scale,
                  const float* a_scale_static, float* C, int8_t* q_out, float* a_scale_out,
                  int32_t* acc_out) {
    float* s = (float*)malloc((size_t)M * sizeof(float));
    int8_t* q = q_out ? q_out : (int8_t*)malloc((size_t)M * K);
    int32_t* acc = acc_out ? acc_out : (int32_t*)malloc((size_t)M * N * sizeof(int32_t));
    if (a_scale_static) memcpy(s, a_scale_static, (size_t)M * sizeof(float));
    else orc_w8_scales_f32(M, K, A, s);
    orc_w8_quant_f32(M, K, A, s, q);
    orc_gemm_i8(M, N, K, q, B, acc);
    if (C) orc_dequant_f32(M, N, acc, s, w_scale, C);
    if (a_scale_out) memcpy(a_scale_out, s, (size_t)M * sizeof(float));
    free(s);
    if (!q_out) free(q);
    if (!acc_out) free(acc);
}

/* reference src/rk_npu_w4a8.cpp:98-151: scales (finite check) -> quantize ->
 * exact product (corr + 16*hi + lo reconstructs sum_k q*B exactly,
 * src/rk_npu_w4a8_output.cpp:36-81) -> dequant. */
static int w4a8_front(int M, int K, const float* A32, const uint16_t* A16, float* s, float* inv,
                      int8_t* q) {
    const int rc = A32 ? orc_w4a8_scales_f32(M, K, A32, s, inv) : orc_w4a8_scales_f16(M, K, A16, s, inv);
    if (rc) return rc;
    if (A32) orc_w4a8_quant_f32(M, K, A32, inv, q);
    else orc_w4a8_quant_f16(M, K, A16, inv, q);
    return ORC_OK;
}
int orc_w4a8_f16(int M, int N, int K, const uint16_t* A, const int8_t* B, const float* w_scale,
                 uint16_t* C, int8_t* q_out, float* a_scale_out, int32_t* acc_out) {
    float* s = (float*)malloc((size_t)M * 2 * sizeof(float));
    int8_t* q = q_out ? q_out : (int8_t*)malloc((size_t)M * K);
    int rc = w4a8_front(M, K, NULL, A, s, s + M, q);
    if (!rc) {
        int32_t* acc = acc_out ? acc_out : (int32_t*)malloc((size_t)M * N * sizeof(int32_t));
        orc_gemm_i8(M, N, K, q, B, acc);
        if (C) orc_dequant_f16(M, N, acc, s, w_scale, C);
        if (a_scale_out) memcpy(a_scale_out, s, (size_t)M * sizeof(float));
        if (!acc_out) free(acc);
    }
    free(s);
    if (!q_out) free(q);
    return rc;
}
int orc_w4a8_f32(int M, int N, int K, const float* A, const int8_t* B, const float* w_scale,
                 float* C, int8_t* q_out, float* a_scale_out, int32_t* acc_out) {
    float* s = (float*)malloc((size_t)M * 2 * sizeof(float));
    int8_t* q = q_out ? q_out : (int8_t*)malloc((size_t)M * K);
    int rc = w4a8_front(M, K, A, NULL, s, s + M, q);
    if (!rc) {
        int32_t* acc = acc_out ? acc_out : (int32_t*)malloc((size_t)M * N * sizeof(int32_t));
        orc_gemm_i8(M, N, K, q, B, acc);
        if (C) orc_dequant_f32(M, N, acc, s, w_scale, C);
        if (a_scale_out) memcpy(a_scale_out, s, (size_t)M * sizeof(float));
        if (!acc_out) free(acc);
    }
    free(s);
    if (!q_out) free(q);
    return rc;
}

/* reference src/rk_npu_w4a8.cpp:349-352 -> run(..., swiglu=true) */
int orc_w4a8_swiglu_f32(int M, int N, int K, const float* A, const int8_t* B,
                        const float* w_scale, int flavour, float* middle,
                        uint32_t* row_max_bits, int32_t* acc_out) {
    if (N % 2) return ORC_ERR_PARAM;
    float* s = (float*)malloc((size_t)M * 2 * sizeof(float));
    int8_t* q = (int8_t*)malloc((size_t)M * K);
    int rc = w4a8_front(M, K, A, NULL, s, s + M, q);
    if (!rc) {
        int32_t* acc = acc_out ? acc_out : (int32_t*)malloc((size_t)M * N * sizeof(int32_t));
        orc_gemm_i8(M, N, K, q, B, acc);
        orc_swiglu(M, N / 2, acc, s, w_scale, flavour, middle, row_max_bits);
        if (!acc_out) free(acc);
    }
    free(s);
    free(q);
    return rc;
}

/* reference src/rk_npu_w4a8.cpp:354-380: gate/up + SwiGLU collecting row
 * maxima, finish_scales (rejects a non-finite middle), Down quantizes middle
 * with the reused scale (no second scan), exact product, dequant to fp32. */
int orc_w4a8_ffn_f32(int M, int H, int I, int Nout, const float* A, const int8_t* B_gate_up,
                     const float* s_gate_up, const int8_t* B_down, const float* s_down,
                     int flavour, float* middle, float* C, int8_t* q_down_out,
                     float* down_scale_out, int32_t* acc_down_out) {
    uint32_t* bits = (uint32_t*)malloc((size_t)M * sizeof(uint32_t));
    int rc = orc_w4a8_swiglu_f32(M, 2 * I, H, A, B_gate_up, s_gate_up, flavour, middle, bits, NULL);
    if (!rc) {
        float* s = (float*)malloc((size_t)M * 2 * sizeof(float));
        rc = orc_finish_scales(M, bits, s, s + M);
        if (!rc) {
            int8_t* q = q_down_out ? q_down_out : (int8_t*)malloc((size_t)M * I);
            int32_t* acc =
                acc_down_out ? acc_down_out : (int32_t*)malloc((size_t)M * Nout * sizeof(int32_t));
            orc_w4a8_quant_f32(M, I, middle, s + M, q);
            orc_gemm_i8(M, Nout, I, q, B_down, acc);
            orc_dequant_f32(M, Nout, acc, s, s_down, C);
            if (down_scale_out) memcpy(down_scale_out, s, (size_t)M * sizeof(float));
            if (!q_down_out) free(q);
            if (!acc_down_out) free(acc);
        }
        free(s);
    }
    free(bits);
    return rc;
}

/* reference src/rk_npu_moe_w8.cpp:574-818 (validate, quantize, group, gate/up,
 * middle, down, combine) and the test oracle tests/test_moe_w8.cpp:24-44.
 * Rows are independent, so the grouping by expert only changes the order of
 * work, never a result; the combine order per token is the slot order. */
int orc_moe_w8(int rows, int H, int I, int E, int shared, int top_k,
               const orc_moe_expert* experts, const float* input_f32, const int8_t* input_q,
               const float* row_scales, const int32_t* ids, const float* routes, int flavour,
               int fused_combine, float* out) {
    for (int i = 0; i < rows * top_k; ++i)
        if (ids[i] < 0 || ids[i] >= E || !isfinite(routes[i]) || routes[i] < 0.0f)
            return ORC_ERR_PARAM;
    int8_t* q = (int8_t*)malloc((size_t)rows * H);
    float* s = (float*)malloc((size_t)rows * sizeof(float));
    int rc = ORC_OK;
    if (input_f32) {
        for (int r = 0; r < rows; ++r)
            s[r] = orc_moe_quant_row(input_f32 + (size_t)r * H, H, 1, q + (size_t)r * H);
    } else {
        memcpy(q, input_q, (size_t)rows * H);
        memcpy(s, row_scales, (size_t)rows * sizeof(float));
    }
    for (int r = 0; r < rows; ++r)
        if (!(s[r] > 0.0f) || !isfinite(s[r])) rc = ORC_ERR_PARAM;
    if (!rc) {
        const int slots = top_k + (shared ? 1 : 0);
#pragma omp parallel
        {
            int32_t* acc1 = (int32_t*)malloc((size_t)2 * I * sizeof(int32_t));
            int32_t* acc2 = (int32_t*)malloc((size_t)H * sizeof(int32_t));
            float* hid = (float*)malloc((size_t)I * sizeof(float));
            int8_t* q2 = (int8_t*)malloc((size_t)I);
#pragma omp for schedule(dynamic, 1)
            for (int r = 0; r < rows; ++r) {
                float* o = out + (size_t)r * H;
                for (int n = 0; n < H; ++n) o[n] = 0.0f;
                for (int slot = 0; slot < slots; ++slot) {
                    float w = 1.0f;
                    int e = E;
                    if (slot < top_k) {
                        w = routes[r * top_k + slot];
                        e = ids[r * top_k + slot];
                        if (w == 0.0f) continue;
                    }
                    const orc_moe_expert* x = experts + e;
                    memset(acc1, 0, (size_t)2 * I * sizeof(int32_t));
                    for (int k = 0; k < H; ++k) {
                        const int32_t a = q[(size_t)r * H + k];
                        const int8_t* b = x->gate_up + (size_t)k * 2 * I;
                        for (int n = 0; n < 2 * I; ++n) acc1[n] += a * (int32_t)b[n];
                    }
                    for (int n = 0; n < I; ++n) {
                        const float g = ((float)acc1[n] * s[r]) * x->gate_up_scales[n];
                        const float u = ((float)acc1[I + n] * s[r]) * x->gate_up_scales[I + n];
                        hid[n] = orc_silu_mul(g, u, flavour);
                    }
                    const float s2 = orc_moe_quant_row(hid, I, 0, q2);
                    memset(acc2, 0, (size_t)H * sizeof(int32_t));
                    for (int k = 0; k < I; ++k) {
                        const int32_t a = q2[k];
                        const int8_t* b = x->down + (size_t)k * H;
                        for (int n = 0; n < H; ++n) acc2[n] += a * (int32_t)b[n];
                    }
                    for (int n = 0; n < H; ++n) {
                        const float v = ((float)acc2[n] * s2) * x->down_scales[n];
                        o[n] = fused_combine ? fmaf(v, w, o[n]) : o[n] + v * w;
                    }
                }
            }
            free(acc1);
            free(acc2);
            free(hid);
            free(q2);
        }
    }
    free(q);
    free(s);
    return rc;
}
