// Device helpers shared by the kernel translation units of librk_npu_matmul.so
// (rk_kernels.hip, rk_kernels_gemv.hip, rk_kernels_gemm.hip, rk_kernels_stream.hip):
// row loaders, the quantization arithmetic, the dequantizing epilogue arithmetic,
// the int4 digit split of the dot-product kernels, the leading-scalar-argument
// macros, and the declarations of the launchers each unit gives the others.
// Everything that is defined here has internal linkage (one copy per unit).
#ifndef RK_KERNELS_COMMON_H
#define RK_KERNELS_COMMON_H

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <float.h>
#include <stdio.h>
#include <stdlib.h>
#include <atomic>
#include <mutex>
#include <type_traits>

#include "rk_hip_shim.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));

// ---- what the units give each other (defined in the unit named) ----
namespace rkk {
// rk_kernels.hip: tells the profiling marker, if one is set, which kernel is launched next
void mark(hipStream_t stream, const char* kernel);
// rk_kernels.hip: compute units of the current device (0 if the query fails)
int compute_units();
// rk_kernels_gemv.hip
bool gemv_swiglu_applies(const rkh_gemm_args& g);
int dispatch_gemv_swiglu(hipStream_t st, const rkh_gemm_args& g, const rkh_quant_args* fuse);
int dispatch_gemv(hipStream_t st, const rkh_gemm_args& g, const rkh_quant_args* fuse);
bool dense_stream_fits(const rkh_gemm_args& g);
int gemv_max_rows(const rkh_gemm_args& g);
bool gemv_can_fuse(const rkh_quant_args& q, const rkh_gemm_args& g, bool swiglu = false);
// rk_kernels_gemm.hip: tile_rows = 128 / 64 / 32
size_t wk_scratch_bytes(long tiles, int bm, int ksplit);
int launch_gemm_wk(hipStream_t st, const rkh_gemm_args& g, int tile_rows, int ksplit);
// rk_kernels_stream.hip
int launch_gemm_grouped(hipStream_t st, const rkh_gemm_args& g);
int launch_gemm_wk_narrow(hipStream_t st, const rkh_gemm_args& g, int tile_rows);
#ifdef RK_DEBUG_TS
void set_ts_gemv(unsigned long long* p);
void set_ts_gemm(unsigned long long* p);
void set_ts_stream(unsigned long long* p);
#endif
} // namespace rkk

namespace {

using rkk::mark;
using rkk::compute_units;

#define RKH_CHECK(expr)                                                        \
    do {                                                                       \
        hipError_t e_ = (expr);                                                \
        if (e_ != hipSuccess) return e_ == hipErrorOutOfMemory ? RKH_ERR_NOMEM \
                                                               : RKH_ERR_RUNTIME; \
    } while (0)

// Build with -DRK_DEBUG_TS for in-kernel wall-clock stamps (tuning aid, never in the product
// build): RK_TS(i) stores the 100 MHz real-time counter seen by a workgroup's first wave into slot i
// of its record (8 slots per workgroup) of the buffer set with rkh_debug_set_ts.
#ifdef RK_DEBUG_TS
static __device__ unsigned long long* rk_dbg_ts = nullptr;
#define RK_TS(i)                                                                                  \
    do {                                                                                          \
        /* (a wave-uniform branch: every lane of the first wave stores the same word) */         \
        if (rk_dbg_ts && __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) == 0)                   \
            rk_dbg_ts[(size_t)blockIdx.x * 8 + (i)] = wall_clock64();                             \
    } while (0)
#else
#define RK_TS(i) do {} while (0)
#endif

// Compile-time loop: f(std::integral_constant<int, 0>{}) ... f(<N-1>{}).
template <int N, int I = 0, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(f);
    }
}

// Compile-time chain: f(<0>) and, while it returns true, f(<1>) ... f(<N-1>).  Unlike N
// independent `if`s the generated control flow has no path that skips a step and runs a later
// one, which is what a sequence "the first n of N steps" means.
template <int N, int I = 0, class F>
__device__ __forceinline__ void static_while(F&& f) {
    if constexpr (I < N) {
        if (f(std::integral_constant<int, I>{})) static_while<N, I + 1>(f);
    }
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
__device__ __forceinline__ int wave_id() { return threadIdx.x >> 6; }

// Logical first column of physical 32-column block p.
__device__ __forceinline__ int block_first_col(int p, int interleave_F) {
    if (!interleave_F) return p * 32;
    return (p & 1) ? interleave_F + (p >> 1) * 32 : (p >> 1) * 32;
}

// ------------------------------------------------------------- quant_rows
__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
    return __half2float(__ushort_as_half(h));
}

template <typename T> struct RowLoader;
template <> struct RowLoader<uint16_t> {
    // The 16 elements as they lie in memory (elements beyond K read as zero), so
    // that a caller can put other loads between fetching and converting them.
    struct Raw { uint32_t w[8]; };
    static __device__ __forceinline__ Raw load16_raw(const uint16_t* row, int k0, int K, bool vec) {
        Raw r;
        if (vec && k0 + 16 <= K) {
            const uint4 a = *reinterpret_cast<const uint4*>(row + k0);
            const uint4 b = *reinterpret_cast<const uint4*>(row + k0 + 8);
            r.w[0] = a.x; r.w[1] = a.y; r.w[2] = a.z; r.w[3] = a.w;
            r.w[4] = b.x; r.w[5] = b.y; r.w[6] = b.z; r.w[7] = b.w;
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t lo = k0 + 2 * j < K ? row[k0 + 2 * j] : 0u;
                const uint32_t hi = k0 + 2 * j + 1 < K ? row[k0 + 2 * j + 1] : 0u;
                r.w[j] = lo | (hi << 16);
            }
        }
        return r;
    }
    static __device__ __forceinline__ void unpack(const Raw& r, float* out) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            out[2 * j] = half_bits_to_float((uint16_t)(r.w[j] & 0xffffu));
            out[2 * j + 1] = half_bits_to_float((uint16_t)(r.w[j] >> 16));
        }
    }
    static __device__ __forceinline__ void load16(const uint16_t* row, int k0, int K, bool vec,
                                                  float* out) {
        if (vec && k0 + 16 <= K) {
            const uint4 a = *reinterpret_cast<const uint4*>(row + k0);
            const uint4 b = *reinterpret_cast<const uint4*>(row + k0 + 8);
            const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                out[2 * j] = half_bits_to_float((uint16_t)(w[j] & 0xffffu));
                out[2 * j + 1] = half_bits_to_float((uint16_t)(w[j] >> 16));
            }
        } else {
#pragma unroll
            for (int j = 0; j < 16; ++j) out[j] = k0 + j < K ? half_bits_to_float(row[k0 + j]) : 0.0f;
        }
    }
};
template <> struct RowLoader<float> {
    struct Raw { float v[16]; };
    static __device__ __forceinline__ Raw load16_raw(const float* row, int k0, int K, bool vec) {
        Raw r;
        load16(row, k0, K, vec, r.v);
        return r;
    }
    static __device__ __forceinline__ void unpack(const Raw& r, float* out) {
#pragma unroll
        for (int j = 0; j < 16; ++j) out[j] = r.v[j];
    }
    static __device__ __forceinline__ void load16(const float* row, int k0, int K, bool vec,
                                                  float* out) {
        if (vec && k0 + 16 <= K) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float4 v = *reinterpret_cast<const float4*>(row + k0 + 4 * j);
                out[4 * j] = v.x; out[4 * j + 1] = v.y; out[4 * j + 2] = v.z; out[4 * j + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int j = 0; j < 16; ++j) out[j] = k0 + j < K ? row[k0 + j] : 0.0f;
        }
    }
};
template <> struct RowLoader<int8_t> {
    static __device__ __forceinline__ void load16(const int8_t* row, int k0, int K, bool vec,
                                                  float* out) {
        (void)vec;
#pragma unroll
        for (int j = 0; j < 16; ++j) out[j] = k0 + j < K ? (float)row[k0 + j] : 0.0f;
    }
};

// The largest magnitude bit pattern among the 16 elements of a chunk as fetched (sign bits
// cleared).  Magnitudes of finite values order like their patterns, and a pattern of 0x7c00
// (fp16) / 0x7f800000 (fp32) or more says that the chunk holds an Inf or a NaN.
typedef unsigned short rk_us2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t chunk_top_magnitude(const RowLoader<uint16_t>::Raw& r) {
    rk_us2 top = {0, 0};
#pragma unroll
    for (int j = 0; j < 8; ++j)
        top = __builtin_elementwise_max(top, __builtin_bit_cast(rk_us2, r.w[j] & 0x7fff7fffu));
    return top.x > top.y ? top.x : top.y;
}
__device__ __forceinline__ uint32_t chunk_top_magnitude(const RowLoader<float>::Raw& r) {
    uint32_t top = 0;
#pragma unroll
    for (int j = 0; j < 16; ++j) top = max(top, __float_as_uint(r.v[j]) & 0x7fffffffu);
    return top;
}

__device__ __forceinline__ bool not_finite(float x) {
    return (__float_as_uint(x) & 0x7f800000u) == 0x7f800000u;
}

// Running largest magnitude of 16 values and a watch for an Inf or a NaN among them: x * 0 is NaN
// for an Inf or a NaN and a zero otherwise, so one fma per element leaves `taint` (started at 0)
// NaN iff one was seen -- a comparison of the exponent bits costs three instructions per element,
// and the quantizers are bound by their vector instructions as much as by memory.
__device__ __forceinline__ void absmax16(const float* v, float& mx, float& taint) {
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        mx = fmaxf(mx, fabsf(v[j]));
        taint = fmaf(v[j], 0.0f, taint);
    }
}
__device__ __forceinline__ bool tainted(float taint) { return taint != taint; }

// Byte offset of the 16-byte chunk (row, chunk c = k/16) in a tiled int8 matrix.
__device__ __forceinline__ size_t tiled_chunk_offset(int row, int c, int KB) {
    const int kb = c >> 1, half = c & 1;
    return ((size_t)(row >> 5) * KB + kb) * 1024 + (size_t)((row & 31) + 32 * half) * 16;
}

// 16 quantized codes into the tiled matrix, as a write-through store (system scope, but not
// streaming).  The next kernel reads these tiles.  A plain store leaves the line dirty in this
// die's L2 until the write-back at the end of the kernel, which the launch then waits for
// (2048 x 4096 codes: 8.8 us with plain stores, 8.0 us written through); a streaming
// (non-temporal) store also bypasses the memory-side cache, and the GEMM behind it then
// fetches the tiles from HBM (the quantization got 1 us shorter and the GEMM 1.5 us longer).
// (The instruction is inline assembly because the cache policy cannot be spelled otherwise;
// the compiler therefore does not know that it is a 16-byte store, after which a vector
// instruction may not overwrite the data registers for two wait states -- the s_nop keeps
// that distance, without it the next instruction occasionally changed the first dword.)
__device__ __forceinline__ void store_codes(uint8_t* dst, uint4 codes) {
    const v4i v = {(int)codes.x, (int)codes.y, (int)codes.z, (int)codes.w};
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"(dst), "v"(v) : "memory");
}

// int8 code of v * inv as the low byte of the result.
//   EVEN:  rint(clamp(q, -127, 127))            (ties to even)
//   else:  clamp(roundf(q), -127, 127)          (ties away from zero; NaN -> 127, as the chain of
//          comparisons in the reference gives).  v_cvt_rpi_i32_f32 is floor(x + 0.5) computed
//          exactly, i.e. round-half-away on |q|; checked against roundf over all 2^32 bit patterns.
template <bool EVEN>
__device__ __forceinline__ int quantize_code(float v, float inv) {
    const float q = v * inv;
    if (EVEN) {
        return (int)rintf(fmaxf(fminf(q, 127.0f), -127.0f));
    } else {
        const float a = fminf(fabsf(q), 127.0f); // NaN -> 127
        int r;
        asm("v_cvt_rpi_i32_f32 %0, %1" : "=v"(r) : "v"(a));
        return q < 0.0f ? -r : r;
    }
}

// The low bytes of four dwords as one dword (c0 lowest).
__device__ __forceinline__ uint32_t pack_low_bytes(int c0, int c1, int c2, int c3) {
    const uint32_t lo = __builtin_amdgcn_perm((uint32_t)c1, (uint32_t)c0, 0x0c0c0400u);
    const uint32_t hi = __builtin_amdgcn_perm((uint32_t)c3, (uint32_t)c2, 0x0c0c0400u);
    return __builtin_amdgcn_perm(hi, lo, 0x05040100u);
}

template <bool EVEN>
__device__ __forceinline__ uint4 quantize16(const float* v, float inv) {
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
        w[j] = pack_low_bytes(quantize_code<EVEN>(v[4 * j], inv), quantize_code<EVEN>(v[4 * j + 1], inv),
                              quantize_code<EVEN>(v[4 * j + 2], inv), quantize_code<EVEN>(v[4 * j + 3], inv));
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// Workgroups of the streaming kernel's 32-row x 256-column grid below which a dense launch splits K
// over the waves of narrower tiles instead.  (256 or 512 instead, int8, 128 rows, K = 4096: 11008
// columns 25.6 -> 23.4 us, 14336 columns 27.3 -> 30.4 us.)
constexpr long DENSE_KS4_BELOW = 128;

// ---- leading scalar arguments
// The first 14 dwords of a kernel's scalar arguments arrive in registers when a wave starts
// (kernel-argument preload, switched on by the build's -amdgpu-kernarg-preload-count);
// a structure passed by value is fetched from memory by every wave, one more round trip ahead
// of its first data load.  The hot kernels therefore repeat, ahead of their argument
// structure, the fields their first loads depend on, and copy them back over the structure.
#define RK_QUANT_HEAD_PARAMS                                                                          \
    const void* h_src, const int* h_active, const uint32_t* h_row_max, int h_M, int h_K, int h_mode, int h_parts
#define RK_QUANT_HEAD(a) (a).src, (a).active_blocks, (a).row_max_bits, (a).M, (a).K, (a).mode, (a).row_max_parts
#define RK_QUANT_HEAD_APPLY(a)                                                                        \
    do {                                                                                              \
        (a).src = h_src; (a).active_blocks = h_active; (a).row_max_bits = h_row_max;                  \
        (a).M = h_M; (a).K = h_K; (a).mode = h_mode; (a).row_max_parts = h_parts;                     \
    } while (0)
#define RK_GEMM_HEAD_PARAMS                                                                           \
    const uint8_t* h_A, const uint8_t* h_W, const uint8_t* h_W4, const int* h_blk_expert, const int* h_num_blocks, \
        int h_M, int h_K, int h_int4_experts
#define RK_GEMM_HEAD(g) (g).A, (g).W, (g).W4, (g).blk_expert, (g).num_blocks, (g).M, (g).K, (g).int4_experts
#define RK_GEMM_HEAD_APPLY(g)                                                                         \
    do {                                                                                              \
        (g).A = h_A; (g).W = h_W; (g).W4 = h_W4; (g).blk_expert = h_blk_expert;                       \
        (g).num_blocks = h_num_blocks; (g).M = h_M; (g).K = h_K; (g).int4_experts = h_int4_experts;   \
    } while (0)
#define RK_SCATTER_HEAD(a) (a).ids, (a).routes, (a).src, (a).rows, (a).top_k, (a).experts, (a).shared, (a).K
#define RK_GEMV_HEAD_PARAMS const uint8_t* h_W, const void* h_src, int h_M, int h_K
#define RK_GEMV_HEAD(g, q) (g).W, (q).src, (g).M, (g).K
#define RK_GEMV_HEAD_APPLY(g, q)                                                                      \
    do { (g).W = h_W; (q).src = h_src; (g).M = h_M; (g).K = h_K; } while (0)

// ------------------------------------------------------------- epilogues
// Degree-7 fp32 exponential SiLU, step for step the sequence of the reference
// (src/rk_npu_swiglu_fp32_neon.h:13-51): every fused step is an explicit fmaf.
__device__ __forceinline__ float silu_poly(float g) {
    float x = -g;
    x = fminf(x, 80.0f);
    x = fmaxf(x, -80.0f);
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
    const float power = __uint_as_float((uint32_t)((int)n + 127) << 23);
    const float d = 1.0f + p * power;
    return g < -80.0f ? -0.0f : g / d;
}

// y = (float(acc) * as) * ws with both products rounded to fp32.  The empty asm
// makes the value opaque so the compiler cannot merge the second multiply with a
// following fp16 conversion into one mixed-precision instruction (which would
// round once instead of twice and differ from the reference on ties).
__device__ __forceinline__ float dequant(int acc, float as, float ws) {
    float y = __fmul_rn(__fmul_rn((float)acc, as), ws);
    asm volatile("" : "+v"(y));
    return y;
}

__device__ __forceinline__ void store_out(void* C, int epi, size_t index, int acc, float as,
                                          float ws) {
    if (epi == RKH_EPI_I32) {
        static_cast<int32_t*>(C)[index] = acc;
    } else if (epi == RKH_EPI_F16) {
        static_cast<__half*>(C)[index] = __float2half_rn(dequant(acc, as, ws));
    } else {
        static_cast<float*>(C)[index] = dequant(acc, as, ws);
    }
}

// ---- int4 weights in the GEMV kernels: no unpacking --------------------------------
// An int8 activation code q is split into two signed int4 digits, q = 16 * h + l + 8 with
// h = q >> 4 and l = (q & 15) - 8 (both in [-8, 7]), so that
//     sum_k q * w  =  16 * sum_k h * w  +  sum_k l * w  +  8 * sum_k w,
// and the two digit sums are v_dot8_i32_i4 products against the packed weight words as they
// lie in memory; the last term is a per-column constant computed at upload.  The staged
// activations hold, for every 8 consecutive k, one word of h digits and one of l digits in
// the nibble order of the weight words (byte j: k0 + j low, k0 + 4 + j high).  Unpacking the
// weights to int8 operands instead took 12 vector instructions per 1 KiB tile and lane on top
// of 8 dot products, and with every tile of a short K in flight at once that arithmetic, not
// the stream, was the tail of the kernel.
__device__ __forceinline__ void split_digits(uint32_t a, uint32_t b, uint32_t& hi, uint32_t& lo) {
    hi = ((a >> 4) & 0x0F0F0F0Fu) | (b & 0xF0F0F0F0u);
    lo = ((a & 0x0F0F0F0Fu) | ((b & 0x0F0F0F0Fu) << 4)) ^ 0x88888888u;
}
// 16 consecutive int8 codes -> {h, l, h, l} of their two groups of 8
__device__ __forceinline__ uint4 digits16(uint4 codes) {
    uint4 r;
    split_digits(codes.x, codes.y, r.x, r.y);
    split_digits(codes.z, codes.w, r.z, r.w);
    return r;
}
// Both digit sums of the 16 k a lane holds of one 32-deep half of an int4 super-tile: av = the
// staged digits {h, l, h, l}, w0 / w1 = the two weight words.
__device__ __forceinline__ void dot_digits(const v4i& av, int w0, int w1, int& acc_h, int& acc_l) {
    acc_h = __builtin_amdgcn_sdot8(av.x, w0, acc_h, false);
    acc_l = __builtin_amdgcn_sdot8(av.y, w0, acc_l, false);
    acc_h = __builtin_amdgcn_sdot8(av.z, w1, acc_h, false);
    acc_l = __builtin_amdgcn_sdot8(av.w, w1, acc_l, false);
}


// ---- ROWS consecutive rows quantized by the THREADS threads of the calling workgroup ----
// For a fixed 16-element chunk, consecutive rows are consecutive 16-byte slots of a tile of the
// int8 matrix, so with 8 rows every store instruction writes whole 128-byte lines (64-byte
// halves with 4).  Lane = (row r = lane % ROWS, chunk column lane / ROWS + (64 / ROWS) * wave).
// Rows of up to (THREADS / ROWS) * CACHE chunks are held in registers between the maximum and
// the quantization; longer rows are read twice, the second time from L2.  Modes: dynamic W8 /
// W4A8 maxima or a given static scale.  Every thread of the workgroup must call it (it contains
// a workgroup barrier); part_max / part_bad: THREADS / 64 * ROWS floats and THREADS / 64 ints of LDS.
template <typename T, int ROWS, int THREADS, int CACHE>
__device__ __forceinline__ void quant_rows_group(const rkh_quant_args& a, int first_row, float* part_max, int* part_bad) {
    static_assert(ROWS == 8 || ROWS == 4, "rows per group");
    constexpr int WAVES = THREADS / 64;
    constexpr int CPW = 64 / ROWS;        // chunk columns per wave instruction
    constexpr int CSTEP = WAVES * CPW;    // chunk columns per workgroup pass
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int r = lane % ROWS, cl = lane / ROWS + CPW * wave;
    const int m = first_row + r;
    const bool live = m < a.M;
    const int K = a.K, KB = (int)(rkh_align_up(K, RKH_K_ALIGN) / 32);
    const int nchunks = (K + 15) >> 4;
    const T* row = static_cast<const T*>(a.src) + (size_t)(live ? m : a.M - 1) * K;
    const bool vec = ((reinterpret_cast<uintptr_t>(row) & 15) == 0);
    const int mode = a.mode;
    const bool need_max = mode != RKH_Q_W8_STATIC;
    const bool check = mode == RKH_Q_W4A8;
    const bool cached = nchunks <= CSTEP * CACHE;

    float v[CACHE][16];
    float mx = 0.0f;
    float taint = 0.0f; // (NaN once an Inf or a NaN was seen, see absmax16)
    if (cached) {
#pragma unroll
        for (int i = 0; i < CACHE; ++i) {
            const int c = cl + CSTEP * i;
            if (c < nchunks) RowLoader<T>::load16(row, c * 16, K, vec, v[i]);
        }
        if (need_max) {
#pragma unroll
            for (int i = 0; i < CACHE; ++i) {
                if (cl + CSTEP * i < nchunks) {
                    absmax16(v[i], mx, taint);
                }
            }
        }
    } else if (need_max) {
        for (int c = cl; c < nchunks; c += CSTEP) {
            float tmp[16];
            RowLoader<T>::load16(row, c * 16, K, vec, tmp);
            absmax16(tmp, mx, taint);
        }
    }
    float scale = 1.0f;
    if (need_max) {
#pragma unroll
        for (int off = ROWS; off < 64; off <<= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
        const unsigned long long bad_mask = __ballot(tainted(taint) && check && live);
        if (lane < ROWS) part_max[wave * ROWS + lane] = mx;
        if (lane == 0) part_bad[wave] = bad_mask != 0ull;
        __syncthreads();
        int any_bad = 0;
        mx = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            mx = fmaxf(mx, part_max[w * ROWS + r]);
            any_bad |= part_bad[w];
        }
        if (t == 0 && a.bad_flag && any_bad) atomicOr(a.bad_flag, 1);
        if (mode == RKH_Q_W4A8) scale = mx == 0.0f ? 1.0f : fmaxf(mx / 127.0f, FLT_MIN);
        else scale = mx > 0.0f ? mx / 127.0f : 1.0f;
        if (t < ROWS && live && a.scale) a.scale[m] = scale;
    } else {
        scale = a.scale[live ? m : a.M - 1];
    }
    if (live) {
        const float inv = 1.0f / scale;
        if (cached) {
#pragma unroll
            for (int i = 0; i < CACHE; ++i) {
                const int c = cl + CSTEP * i;
                if (c < nchunks) store_codes(a.dst + tiled_chunk_offset(m, c, KB), quantize16<false>(v[i], inv));
            }
        } else {
            for (int c = cl; c < nchunks; c += CSTEP) {
                float tmp[16];
                RowLoader<T>::load16(row, c * 16, K, vec, tmp);
                store_codes(a.dst + tiled_chunk_offset(m, c, KB), quantize16<false>(tmp, inv));
            }
        }
    }
}

} // namespace

#endif // RK_KERNELS_COMMON_H
