// HIP kernels of the quantized-linear path for gfx950 (MI355X), and the C-ABI
// launchers declared in rk_hip_shim.h.  Data layouts are described there.
//
// Kernel inventory (what bounds each one):
//   pack_w8_kernel / pack_w4_kernel     weight re-tiling at upload                      (one-time)
//   quant_rows_kernel                   per-token absmax + int8 codes, workgroup per row (HBM, small)
//   quant_rows8_kernel                  the same for many rows, 8 / 4 rows per workgroup (HBM)
//   requant_rows_wave_kernel            re-quantize short fp32 rows, wave per row        (HBM, small)
//   gemv_kernel                         M <= 8 decode path: dot4, no MFMA, optional fused
//                                       per-token quantization                           (HBM)
//   gemv_swiglu_kernel                  gate/up + SwiGLU of one or two rows              (HBM)
//   gemm_wk_kernel                      int8 MFMA 32x32x32, (32..128) x 256 tiles, activations
//                                       through an LDS ring, waves split K               (MFMA)
//   gemm_wk_reduce_kernel               sum of K-split partial tiles + epilogue          (L2, small)
//   gemm_stream_kernel                  32 x 256 tiles, operands straight to registers: MoE
//                                       (grouped by expert) and dense GEMMs of 9..128 rows (HBM)
//   moe_scatter_kernel                  route by expert + quantize tokens into sorted rows (latency)
//   moe_combine_kernel                  weighted sum of expert outputs in slot order     (HBM, small)
//   moe_decode_gate_kernel / moe_decode_down_kernel   the MoE layer for up to eight tokens in two
//                                       launches: dot products, no routing tables          (latency, HBM)
//   stream_read_probe_kernel / mfma_i8_probe_kernel   measurement probes (practical ceilings)
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <float.h>
#include <stdio.h>
#include <stdlib.h>
#include <atomic>
#include <mutex>
#include <shared_mutex>
#include <type_traits>

#include "rk_hip_shim.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace {

#define RKH_CHECK(expr)                                                        \
    do {                                                                       \
        hipError_t e_ = (expr);                                                \
        if (e_ != hipSuccess) return e_ == hipErrorOutOfMemory ? RKH_ERR_NOMEM \
                                                               : RKH_ERR_RUNTIME; \
    } while (0)

// Stage marker (see rkh_set_marker): told the name of every kernel launched through this
// file just before the launch, so that a caller can put stream events between the kernels
// of a multi-kernel step.  Null unless a caller is profiling.
// Launches come from any thread: the pair is read under a shared lock, which rkh_set_marker
// takes exclusively -- so once it has returned, no thread is inside the old marker or about
// to call it with the old user pointer.  `g_marker_on` keeps the lock off the path of every
// launch while nobody profiles.
std::shared_mutex g_marker_mutex;
std::atomic<bool> g_marker_on{false};
rkh_marker_fn g_marker = nullptr;
void* g_marker_user = nullptr;
inline void mark(hipStream_t stream, const char* kernel) {
    if (!g_marker_on.load(std::memory_order_acquire)) return;
    std::shared_lock<std::shared_mutex> lock(g_marker_mutex);
    if (g_marker) g_marker(g_marker_user, stream, kernel);
}

// Build with -DRK_DEBUG_TS for in-kernel wall-clock stamps (tuning aid, never in the product
// build): RK_TS(i) stores the 100 MHz real-time counter seen by a workgroup's first wave into slot i
// of its record (8 slots per workgroup) of the buffer set with rkh_debug_set_ts.
#ifdef RK_DEBUG_TS
__device__ unsigned long long* rk_dbg_ts = nullptr;
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

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
__device__ __forceinline__ int wave_id() { return threadIdx.x >> 6; }

// Logical first column of physical 32-column block p.
__device__ __forceinline__ int block_first_col(int p, int interleave_F) {
    if (!interleave_F) return p * 32;
    return (p & 1) ? interleave_F + (p >> 1) * 32 : (p >> 1) * 32;
}

// ------------------------------------------------------------------ fill
__global__ void fill32_kernel(uint32_t* dst, uint32_t value, size_t words) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < words; i += stride) dst[i] = value;
}

// Exchanges two disjoint arrays of 32-bit words in place.
__global__ void exchange32_kernel(uint32_t* x, uint32_t* y, size_t words) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < words; i += stride) {
        const uint32_t a = x[i], b = y[i];
        x[i] = b;
        y[i] = a;
    }
}

// ------------------------------------------------------------ weight pack
// One thread produces one lane's 16 bytes of one tile.
__global__ __launch_bounds__(256) void pack_w8_kernel(const int8_t* __restrict__ src, int K, int N,
                                                      int KB, int interleave_F,
                                                      uint8_t* __restrict__ dst, size_t total_chunks) {
    const size_t chunk = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (chunk >= total_chunks) return;
    const int lane = (int)(chunk & 63);
    const size_t tile = chunk >> 6;
    const int kb = (int)(tile % KB);
    const int p = (int)(tile / KB);
    const int n = block_first_col(p, interleave_F) + (lane & 31);
    const int k0 = kb * 32 + (lane >> 5) * 16;
    uint32_t w[4] = {0, 0, 0, 0};
    const bool col_ok = interleave_F ? (p < N / 32) : (n < N);
    if (col_ok) {
        for (int j = 0; j < 16; ++j) {
            const int k = k0 + j;
            const uint32_t v = k < K ? (uint8_t)src[(size_t)k * N + n] : 0u;
            w[j >> 2] |= v << ((j & 3) * 8);
        }
    }
    reinterpret_cast<uint4*>(dst)[chunk] = make_uint4(w[0], w[1], w[2], w[3]);
}

__global__ __launch_bounds__(256) void pack_w4_kernel(const int8_t* __restrict__ src, int K, int N,
                                                      int KB2, int interleave_F,
                                                      uint8_t* __restrict__ dst, size_t total_chunks,
                                                      int* bad_flag, int32_t* colsum) {
    const size_t chunk = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (chunk >= total_chunks) return;
    const int lane = (int)(chunk & 63);
    const size_t tile = chunk >> 6;
    const int kb2 = (int)(tile % KB2);
    const int p = (int)(tile / KB2);
    const int n = block_first_col(p, interleave_F) + (lane & 31);
    const bool col_ok = interleave_F ? (p < N / 32) : (n < N);
    uint32_t w[4] = {0, 0, 0, 0};
    bool bad = false;
    int sum = 0; // of this lane's 32 codes: a share of the column sum the GEMV kernels need
    if (col_ok) {
        for (int t = 0; t < 2; ++t) {            // the two 32-k halves of the super-tile
            const int k0 = kb2 * 64 + t * 32 + (lane >> 5) * 16;
            for (int j = 0; j < 16; ++j) {
                const int k = k0 + j;
                int code = 0;
                if (k < K) {
                    code = src[(size_t)k * N + n];
                    if (code < -8 || code > 7) bad = true;
                    sum += code;
                }
                // word = t*2 + j/8 ; within the word: byte (j%8)%4, high nibble when (j%8) >= 4
                const int k8 = j & 7;
                const int shift = (k8 & 3) * 8 + (k8 >> 2) * 4;
                w[t * 2 + (j >> 3)] |= (uint32_t)(code & 15) << shift;
            }
        }
    }
    if (bad && bad_flag) atomicOr(bad_flag, 1);
    if (colsum && col_ok && sum) atomicAdd(&colsum[n], sum);
    reinterpret_cast<uint4*>(dst)[chunk] = make_uint4(w[0], w[1], w[2], w[3]);
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

__device__ __forceinline__ bool not_finite(float x) {
    return (__float_as_uint(x) & 0x7f800000u) == 0x7f800000u;
}

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

constexpr int QR_CACHE = 4; // 16-element chunks kept in registers per thread

// `split` workgroups share a row (blockIdx.x = row * split + part), each taking a
// contiguous range of its 16-element chunks.  Only the modes that do not scan the
// row for its maximum are launched with split > 1: re-quantization finds the
// maximum in the partial maxima the GEMM left behind, which every part reads.
template <typename T>
__global__ __launch_bounds__(256) void quant_rows_kernel(RK_QUANT_HEAD_PARAMS, int split, rkh_quant_args a) {
    RK_QUANT_HEAD_APPLY(a);
    __shared__ float wave_max[4];
    __shared__ int wave_bad[4];
    const int m = blockIdx.x / split, part = blockIdx.x - m * split, t = threadIdx.x;
    if (a.active_blocks && m >= a.active_blocks[0] * 32) return;
    const int K = a.K, KB = (int)(rkh_align_up(K, RKH_K_ALIGN) / 32);
    const int row_chunks = (K + 15) >> 4;
    const int per_part = (row_chunks + split - 1) / split;
    const int chunk0 = part * per_part;                         // this workgroup's chunks: chunk0 .. nchunks - 1
    const int nchunks = min(row_chunks, chunk0 + per_part);
    const T* row = static_cast<const T*>(a.src) + (size_t)m * K;
    const bool vec = ((reinterpret_cast<uintptr_t>(row) & 15) == 0);
    const bool cached = nchunks - chunk0 <= 256 * QR_CACHE;
    const int mode = a.mode;
    if constexpr (sizeof(T) == 1) {
        // int8 input is re-tiled byte for byte (the full range -128..127 is legal
        // for the raw integer operator)
        const int8_t* brow = reinterpret_cast<const int8_t*>(row);
        for (int c = chunk0 + t; c < nchunks; c += 256) {
            uint32_t w[4] = {0, 0, 0, 0};
            if (vec && c * 16 + 16 <= K) {
                const uint4 v4 = *reinterpret_cast<const uint4*>(brow + c * 16);
                w[0] = v4.x; w[1] = v4.y; w[2] = v4.z; w[3] = v4.w;
            } else {
                for (int j = 0; j < 16; ++j)
                    if (c * 16 + j < K) w[j >> 2] |= (uint32_t)(uint8_t)brow[c * 16 + j] << ((j & 3) * 8);
            }
            store_codes(a.dst + tiled_chunk_offset(m, c, KB), make_uint4(w[0], w[1], w[2], w[3]));
        }
        return;
    }
    const bool need_max = mode == RKH_Q_W8_DYNAMIC || mode == RKH_Q_W4A8;
    const bool check = mode == RKH_Q_W4A8;

    float v[QR_CACHE][16];
    float mx = 0.0f;
    bool bad = false;
    if (cached) {
#pragma unroll
        for (int i = 0; i < QR_CACHE; ++i) {
            const int c = chunk0 + t + i * 256;
            if (c < nchunks) {
                RowLoader<T>::load16(row, c * 16, K, vec, v[i]);
                if (need_max) {
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        mx = fmaxf(mx, fabsf(v[i][j]));
                        bad |= not_finite(v[i][j]);
                    }
                }
            }
        }
    } else if (need_max) {
        for (int c = chunk0 + t; c < nchunks; c += 256) {
            float tmp[16];
            RowLoader<T>::load16(row, c * 16, K, vec, tmp);
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                mx = fmaxf(mx, fabsf(tmp[j]));
                bad |= not_finite(tmp[j]);
            }
        }
    }

    float scale = 1.0f;
    if (need_max) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
        const unsigned long long bad_mask = __ballot(bad && check);
        if (lane_id() == 0) {
            wave_max[wave_id()] = mx;
            wave_bad[wave_id()] = bad_mask != 0ull;
        }
        __syncthreads();
        mx = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
        const int any_bad = wave_bad[0] | wave_bad[1] | wave_bad[2] | wave_bad[3];
        if (any_bad && t == 0 && a.bad_flag) atomicOr(a.bad_flag, 1);
        if (mode == RKH_Q_W4A8) scale = mx == 0.0f ? 1.0f : fmaxf(mx / 127.0f, FLT_MIN);
        else scale = mx > 0.0f ? mx / 127.0f : 1.0f;
    } else if (mode == RKH_Q_W8_STATIC || (mode == RKH_Q_COPY_I8 && a.scale)) {
        scale = a.scale[m];
    } else if (mode == RKH_Q_REUSE_BITS || mode == RKH_Q_REUSE_BITS_MOE) {
        // row maximum = max over the per-32-column partial maxima the SwiGLU
        // epilogue left behind (unsigned compare of |x| bit patterns)
        uint32_t bits = 0;
        for (int i = t; i < a.row_max_parts; i += 256)
            bits = max(bits, a.row_max_bits[(size_t)m * a.row_max_parts + i]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) bits = max(bits, (uint32_t)__shfl_xor((int)bits, off));
        if (lane_id() == 0) wave_bad[wave_id()] = (int)bits;
        __syncthreads();
        bits = max(max((uint32_t)wave_bad[0], (uint32_t)wave_bad[1]),
                   max((uint32_t)wave_bad[2], (uint32_t)wave_bad[3]));
        const float mxv = __uint_as_float(bits);
        if (mode == RKH_Q_REUSE_BITS) {
            if (bits >= 0x7f800000u) {
                if (t == 0 && a.bad_flag) atomicOr(a.bad_flag, 1);
                scale = 1.0f;
            } else {
                scale = mxv == 0.0f ? 1.0f : fmaxf(mxv / 127.0f, FLT_MIN);
            }
        } else {
            scale = mxv != 0.0f ? mxv / 127.0f : 1.0f;
        }
    }
    const float inv = mode == RKH_Q_COPY_I8 ? 1.0f : 1.0f / scale;
    const bool even = mode == RKH_Q_REUSE_BITS_MOE;

    if (t == 0 && part == 0 && a.scale && mode != RKH_Q_W8_STATIC && mode != RKH_Q_COPY_I8) a.scale[m] = scale;

    auto emit = [&](int c, const float* vals) {
        const uint4 packed = even ? quantize16<true>(vals, inv) : quantize16<false>(vals, inv);
        store_codes(a.dst + tiled_chunk_offset(m, c, KB), packed);
    };
    if (cached) {
#pragma unroll
        for (int i = 0; i < QR_CACHE; ++i) {
            const int c = chunk0 + t + i * 256;
            if (c < nchunks) emit(c, v[i]);
        }
    } else {
        for (int c = chunk0 + t; c < nchunks; c += 256) {
            float tmp[16];
            RowLoader<T>::load16(row, c * 16, K, vec, tmp);
            emit(c, tmp);
        }
    }
}

// Re-quantization of many short fp32 rows (the MoE middle: a thousand-odd rows of
// 1024): one wave per row, four rows per workgroup.  The row maximum comes from
// the partial maxima the SwiGLU epilogue left behind, so a row needs no
// workgroup-wide reduction; with a workgroup per row three of its four waves
// had nothing to do.  Rows of up to 64 * QR_CACHE chunks.
__global__ __launch_bounds__(256) void requant_rows_wave_kernel(RK_QUANT_HEAD_PARAMS, rkh_quant_args a) {
    RK_QUANT_HEAD_APPLY(a);
    const int lane = lane_id(), m = blockIdx.x * 4 + wave_id();
    if (m >= a.M || (a.active_blocks && m >= a.active_blocks[0] * 32)) return;
    const int K = a.K, KB = (int)(rkh_align_up(K, RKH_K_ALIGN) / 32);
    const int nchunks = (K + 15) >> 4;
    const float* row = static_cast<const float*>(a.src) + (size_t)m * K;
    const bool vec = ((reinterpret_cast<uintptr_t>(row) & 15) == 0);
    float v[QR_CACHE][16];
#pragma unroll
    for (int i = 0; i < QR_CACHE; ++i)
        if (lane + 64 * i < nchunks) RowLoader<float>::load16(row, (lane + 64 * i) * 16, K, vec, v[i]);
    uint32_t bits = 0; // unsigned compare of |x| bit patterns
    for (int i = lane; i < a.row_max_parts; i += 64) bits = max(bits, a.row_max_bits[(size_t)m * a.row_max_parts + i]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) bits = max(bits, (uint32_t)__shfl_xor((int)bits, off));
    const float mx = __uint_as_float(bits);
    float scale;
    if (a.mode == RKH_Q_REUSE_BITS) {
        if (bits >= 0x7f800000u) {
            if (lane == 0 && a.bad_flag) atomicOr(a.bad_flag, 1);
            scale = 1.0f;
        } else {
            scale = mx == 0.0f ? 1.0f : fmaxf(mx / 127.0f, FLT_MIN);
        }
    } else {
        scale = mx != 0.0f ? mx / 127.0f : 1.0f;
    }
    if (lane == 0 && a.scale) a.scale[m] = scale;
    const float inv = 1.0f / scale;
    const bool even = a.mode == RKH_Q_REUSE_BITS_MOE;
#pragma unroll
    for (int i = 0; i < QR_CACHE; ++i)
        if (lane + 64 * i < nchunks)
            store_codes(a.dst + tiled_chunk_offset(m, lane + 64 * i, KB),
                        even ? quantize16<true>(v[i], inv) : quantize16<false>(v[i], inv));
}

// Dense quantization of many rows: one workgroup per ROWS (8 or 4) consecutive
// rows.  For a fixed 16-element chunk, consecutive rows are consecutive 16-byte
// slots of a tile of the int8 matrix, so with 8 rows every store instruction
// writes whole 128-byte lines (64-byte halves with 4).  Lane = (row r = lane %
// ROWS, chunk column lane / ROWS + (64 / ROWS) * wave): a row's loads are 64 /
// ROWS consecutive chunks per wave instruction.  Rows of up to (256 / ROWS) *
// Q8_CACHE chunks are held in registers between the maximum and the
// quantization (all loads of a thread in flight at once); longer rows are read
// twice, the second time from L2.  The kernel is one load phase, one reduction
// and one store phase, so a compute unit only overlaps loads with stores when
// it holds several workgroups: 4 rows are used while 8 would leave fewer than
// two workgroups per compute unit.
// Modes: dynamic W8 / W4A8 maxima or a given static scale; rows written in place.
constexpr int Q8_CACHE = 8;

template <typename T, int ROWS>
__global__ __launch_bounds__(256) void quant_rows8_kernel(RK_QUANT_HEAD_PARAMS, rkh_quant_args a) {
    RK_QUANT_HEAD_APPLY(a);
    static_assert(ROWS == 8 || ROWS == 4, "rows per workgroup");
    constexpr int CPW = 64 / ROWS;    // chunk columns per wave instruction
    constexpr int CSTEP = 4 * CPW;    // chunk columns per workgroup pass
    __shared__ float part_max[4][ROWS];
    __shared__ int part_bad[4];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int r = lane % ROWS, cl = lane / ROWS + CPW * wave;
    const int m = blockIdx.x * ROWS + r;
    const bool live = m < a.M;
    const int K = a.K, KB = (int)(rkh_align_up(K, RKH_K_ALIGN) / 32);
    const int nchunks = (K + 15) >> 4;
    const T* row = static_cast<const T*>(a.src) + (size_t)(live ? m : a.M - 1) * K;
    const bool vec = ((reinterpret_cast<uintptr_t>(row) & 15) == 0);
    const int mode = a.mode;
    const bool need_max = mode != RKH_Q_W8_STATIC;
    const bool check = mode == RKH_Q_W4A8;
    const bool cached = nchunks <= CSTEP * Q8_CACHE;

    float v[Q8_CACHE][16];
    float mx = 0.0f;
    bool bad = false;
    if (cached) {
#pragma unroll
        for (int i = 0; i < Q8_CACHE; ++i) {
            const int c = cl + CSTEP * i;
            if (c < nchunks) RowLoader<T>::load16(row, c * 16, K, vec, v[i]);
        }
        if (need_max) {
#pragma unroll
            for (int i = 0; i < Q8_CACHE; ++i) {
                if (cl + CSTEP * i < nchunks) {
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        mx = fmaxf(mx, fabsf(v[i][j]));
                        bad |= not_finite(v[i][j]);
                    }
                }
            }
        }
    } else if (need_max) {
        for (int c = cl; c < nchunks; c += CSTEP) {
            float tmp[16];
            RowLoader<T>::load16(row, c * 16, K, vec, tmp);
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                mx = fmaxf(mx, fabsf(tmp[j]));
                bad |= not_finite(tmp[j]);
            }
        }
    }
    float scale = 1.0f;
    if (need_max) {
#pragma unroll
        for (int off = ROWS; off < 64; off <<= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
        const unsigned long long bad_mask = __ballot(bad && check && live);
        if (lane < ROWS) part_max[wave][lane] = mx;
        if (lane == 0) part_bad[wave] = bad_mask != 0ull;
        __syncthreads();
        mx = fmaxf(fmaxf(part_max[0][r], part_max[1][r]), fmaxf(part_max[2][r], part_max[3][r]));
        if (t == 0 && a.bad_flag && (part_bad[0] | part_bad[1] | part_bad[2] | part_bad[3])) atomicOr(a.bad_flag, 1);
        if (mode == RKH_Q_W4A8) scale = mx == 0.0f ? 1.0f : fmaxf(mx / 127.0f, FLT_MIN);
        else scale = mx > 0.0f ? mx / 127.0f : 1.0f;
        if (t < ROWS && live && a.scale) a.scale[m] = scale;
    } else {
        scale = a.scale[live ? m : a.M - 1];
    }
    if (!live) return;
    const float inv = 1.0f / scale;
    if (cached) {
#pragma unroll
        for (int i = 0; i < Q8_CACHE; ++i) {
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

// ------------------------------------------------------------------ GEMV
// One workgroup per physical 32-column block; the waves of the group split K
// (k-tiles interleaved across waves so that neighbouring loads are adjacent in
// memory); activations sit in LDS; lanes l and l+32 hold the two 16-byte
// halves of a k-tile for column l%32, so the cross-lane reduction is one xor
// shuffle, followed by a small LDS reduction across waves.
#ifndef RK_GEMV_WAVES
#define RK_GEMV_WAVES 8
#endif
#ifndef RK_GEMV_UNROLL
#define RK_GEMV_UNROLL 8
#endif
constexpr int GEMV_WAVES = RK_GEMV_WAVES;
constexpr int GEMV_UNROLL = RK_GEMV_UNROLL;
constexpr int GEMV_LDS_BYTES = 32768; // activation bytes staged per K chunk

constexpr int GEMV_QCHUNKS = 4; // 16-element activation chunks a thread may quantize in the fused path

// QT: 0 = activations come quantized from the tiled buffer g.A;
//     3 = int8 rows as the caller holds them (row-major q.src): staged from there, no launch of
//     the re-tiling kernel in front;
//     1 / 2 = fused per-token quantization of fp16 / fp32 rows q.src (every
//     workgroup quantizes the few rows itself -- they are L2 hits after the first
//     -- which saves a kernel launch per decode step; workgroup 0 also writes the
//     scales and the tiled int8 copy that the two-kernel path would have left).
// Two workgroups must fit a compute unit (a grid of a few hundred workgroups
// otherwise runs in two rounds), i.e. four waves per SIMD and at most 128
// vector registers: stated as a requirement, because the int4 variants with the
// fused quantization would otherwise be allocated more.
// CW < 32 (narrow matrices, where one workgroup per 32-column block leaves compute
// units without work -- 128 workgroups for a 4096-column projection): 32 / CW
// workgroups share a column block, CW = 16 or 8 columns each.  A load instruction
// then covers the workgroup's part of 32 / CW consecutive k-tiles (pieces of
// 16 * CW bytes): lane = column % CW + CW * k-half + 2 * CW * (tile of the group),
// and the cross-lane reduction takes two or three xor-shuffles instead of one.
//
// BURST (one int8 row of a wide matrix, more than 256 column blocks -- the decode shape of the
// benchmark): the loads past the end of K are skipped by branches instead of being sent through
// the bounds-checked descriptor.  With the branches the compiler no longer counts the
// outstanding loads exactly and waits for ALL of a wave's loads wherever it needs one of them --
// so every wave of a workgroup has its whole group of tiles before the quantization prologue
// starts, passes the prologue's barriers with nothing outstanding, uses the group at once and
// asks for the next group in one burst together with the other seven waves.  For a matrix that
// is bound by memory throughput that is the faster order, measured on one box for 4096 x 14336:
// 11.05 us against 11.5 us with exact waits (11.4 with an explicit wait for the whole group in
// front of the prologue or of the K loop).  Int4 matrices of the same shape are faster with
// exact waits (7.8 against 8.3 us).  Since the prologue waits for everything anyway, the weight
// tiles are requested ahead of the activation rows, a dozen instructions from the kernel's
// entry instead of behind the row loader's code (in-kernel time stamps: 2.4 us from a wave's
// start until its weight requests were out; 10.9 -> 10.6 us).  Tried on this variant and slower,
// same box, against 10.6 us: a second group of tiles requested before the prologue (11.0 us; all
// 16 loads of a wave requested at the start: 12.2), the wave index read into a scalar register
// (10.85: the branches around the loads become scalar and the compiler counts the loads exactly
// again), the column scales of the epilogue fetched with the first loads (10.7), a first group
// of 4 / 6 / 10 / 12 tiles per wave with the rest in one group behind the prologue (11.8 / 11.1 /
// 11.0 / 11.6), four tiles per group throughout (11.4), the exact-wait kernel with four loads
// per wave in flight (10.7), 28 instead of 32 columns per workgroup (512 workgroups, two for
// every compute unit, instead of 448 -- 11.85 us; the per-lane addresses this needs cost 0.4 us
// already with 32 columns).
template <int MR, bool W4, int QT, int CW, bool BURST = false>
__global__ __launch_bounds__(GEMV_WAVES * 64) __attribute__((amdgpu_waves_per_eu(GEMV_WAVES / 2)))
void gemv_kernel(RK_GEMV_HEAD_PARAMS, rkh_gemm_args g, rkh_quant_args q) {
    RK_GEMV_HEAD_APPLY(g, q);
    RK_TS(0);
    static_assert(CW == 32 || CW == 16 || CW == 8, "columns per workgroup");
    constexpr bool FUSEQ = QT == 1 || QT == 2; // the kernel quantizes the rows itself
    static_assert(QT != 3 || !W4, "int8 rows as given: the exact int8 x int8 product only");
    // Load instructions of a wave in flight.  One row, exact waits: four -- the quantization
    // prologue and the first dot products start after half as many bytes, and nothing is gained
    // by queueing more in front of the memory system (4096 x 14336 int4: 7.25 -> 6.8 us; int4
    // 4096 x 4096 4.9 -> 4.1, 4096 x 11008 7.0 -> 6.6, 8192 x 1024 5.1 -> 4.5; int8 2048 x 2048
    // 4.2 -> 3.6, 14336 x 4096 12.8 -> 12.5, the other int8 shapes within 1 %).  Several rows
    // and the burst variant are faster with eight (two rows lose 2 - 9 % with four on most
    // shapes; the burst variant 10.6 -> 11.4 us).
    constexpr int UNR = (MR == 1 && !BURST) ? 4 : GEMV_UNROLL;
    static_assert(!BURST || (MR == 1 && !W4 && CW == 32), "the burst variant serves one int8 row, whole column blocks");
    constexpr int TPL = 32 / CW;            // k-tiles (int4: super-tiles) covered by one load instruction
    // (padding for the single-row variants of narrow matrices: their look-ahead of UNR loads per wave, and
    // one more step for the activations, runs up to that many load instructions past the end
    // of a chunk, 32 / CW tiles of 32 -- int4: 64 -- staged bytes each)
    constexpr bool ROLLING = MR == 1 && CW < 32; // see the K loop
    constexpr int A_PAD = ROLLING ? GEMV_WAVES * (UNR + 1) * TPL * (W4 ? 64 : 32) : 0;
    __shared__ __attribute__((aligned(16))) uint8_t a_lds[GEMV_LDS_BYTES + A_PAD];
    __shared__ int red[GEMV_WAVES][MR][CW];
    __shared__ uint32_t row_max[MR];
    __shared__ float row_scale[MR];
    const int lane = lane_id(), wave = wave_id();
    const int half = (lane / CW) & 1;                       // which 16 k of a 32-k tile
    const int sub = lane / (2 * CW);                        // which tile of the group one load covers
    const int Kp = (int)rkh_align_up(g.K, RKH_K_ALIGN);
    const int KB = Kp / 32;
    const int p = (int)blockIdx.x / TPL;
    const int col0 = ((int)blockIdx.x % TPL) * CW;          // first column of the block this workgroup owns
    const bool first_wg = blockIdx.x == 0;
    // byte of this lane inside a 1 KiB tile
    const unsigned lane_byte = (unsigned)((col0 + lane % CW) + 32 * half) * 16u;
    // chunk of K staged in LDS at a time (multiple of 64)
    const int kc_max = (GEMV_LDS_BYTES / MR) & ~63;
    int acc[MR], acc_lo[MR]; // (int4 weights: the sums of the high and of the low activation digits)
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[m] = acc_lo[m] = 0;

    const size_t block_bytes = (size_t)(W4 ? Kp / 64 : KB) * 1024; // one column block over all of K
    const uint8_t* wbase = g.W + (size_t)p * block_bytes;
    // Weight loads go through a buffer descriptor over this column block: a load whose offset
    // lies beyond it returns zeros without touching memory, so the loop below needs no branch
    // around the loads past the end of K -- and without branches the compiler counts the
    // outstanding loads exactly (it waits for the one it needs, not for all of them).
    const __amdgpu_buffer_rsrc_t wrsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(wbase), 0, (int)block_bytes, 0x00020000);
    auto load_tile = [&](int unit, int units, int first_tile) -> v4i { // `unit` counts this wave's load instructions
        if constexpr (BURST) {
            return unit < units ? __builtin_nontemporal_load(reinterpret_cast<const v4i*>(
                                      wbase + (size_t)(first_tile + unit) * 1024 + lane * 16))
                                : v4i{0, 0, 0, 0};
        } else {
            const unsigned off = unit < units ? (unsigned)(first_tile + unit * TPL + sub) * 1024u + lane_byte : 0xFFFFFFF0u;
            return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, (int)off, 0, 2 /* streaming */));
        }
    };

    // Fused path: put the first batch of weight loads in flight before the
    // quantization prologue so that its latency hides behind them.
    // The activation rows are requested FIRST: loads return in issue order, so
    // behind the weight loads they would arrive with the last of those, and the
    // prologue (and with it the second batch of weight loads) would start only
    // then.  Fetched first they are back after one L2 round trip and the whole
    // quantization runs under the weight loads' latency.  (BURST: the other way round, see above.)
    v4i wpre[UNR];
    using QT_T = typename std::conditional<QT == 2, float, uint16_t>::type;
    typename RowLoader<QT_T>::Raw araw[FUSEQ ? GEMV_QCHUNKS : 1];
    if constexpr (FUSEQ) {
        const int tiles = (W4 ? Kp >> 6 : Kp >> 5) / TPL;
        if constexpr (BURST) {
#pragma unroll
            for (int u = 0; u < UNR; ++u) wpre[u] = load_tile(wave + u * GEMV_WAVES, tiles, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        const int K = g.K, nchunks = (K + 15) >> 4, total = g.M * nchunks;
#pragma unroll
        for (int i = 0; i < GEMV_QCHUNKS; ++i) {
            const int pidx = (int)threadIdx.x + i * GEMV_WAVES * 64;
            if (pidx < total) {
                const int m = pidx / nchunks, c = pidx - m * nchunks;
                const QT_T* row = static_cast<const QT_T*>(q.src) + (size_t)m * K;
                araw[i] = RowLoader<QT_T>::load16_raw(row, c * 16, K, (reinterpret_cast<uintptr_t>(row) & 15) == 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!BURST) {
#pragma unroll
            for (int u = 0; u < UNR; ++u) wpre[u] = load_tile(wave + u * GEMV_WAVES, tiles, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        RK_TS(4);
    }
    if constexpr (FUSEQ) {
        using T = QT_T;
        const int t = threadIdx.x;
        const int K = g.K, nchunks = (K + 15) >> 4, total = g.M * nchunks;
        if (t < MR) row_max[t] = 0u;
        __syncthreads();
        RK_TS(5);
        // (the rows stay in registers as fetched and are converted once per pass:
        // holding them as floats across the barriers costs the int4 variants their
        // second workgroup per compute unit)
        bool bad = false;
#pragma unroll
        for (int i = 0; i < GEMV_QCHUNKS; ++i) {
            const int pidx = t + i * GEMV_WAVES * 64;
            if (pidx < total) {
                const int m = pidx / nchunks;
                float v[16];
                RowLoader<T>::unpack(araw[i], v);
                float mx = 0.0f;
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    mx = fmaxf(mx, fabsf(v[j]));
                    bad |= not_finite(v[j]);
                }
                // (non-negative floats order like their bits.  For one row, a shuffle reduction per wave
                // and one atomic per wave instead of 64 on the same address measured slower: 4096 x 14336
                // int8 10.65 -> 10.7 us, int4 6.8 -> 7.2 us)
                atomicMax(&row_max[m], __float_as_uint(mx));
            }
        }
        __syncthreads();
        if (t < g.M) {
            const float mx = __uint_as_float(row_max[t]);
            const float sc = q.mode == RKH_Q_W4A8 ? (mx == 0.0f ? 1.0f : fmaxf(mx / 127.0f, FLT_MIN))
                                                  : (mx > 0.0f ? mx / 127.0f : 1.0f);
            row_scale[t] = sc;
            if (first_wg && q.scale) q.scale[t] = sc;
        }
        if (first_wg && bad && q.mode == RKH_Q_W4A8 && q.bad_flag) atomicOr(q.bad_flag, 1);
        // zero the K padding of the staged rows
        for (int idx = t; idx < g.M * ((Kp >> 4) - nchunks); idx += GEMV_WAVES * 64) {
            const int m = idx / ((Kp >> 4) - nchunks), c = nchunks + idx % ((Kp >> 4) - nchunks);
            *reinterpret_cast<uint4*>(a_lds + (size_t)m * Kp + (size_t)c * 16) = make_uint4(0, 0, 0, 0);
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < GEMV_QCHUNKS; ++i) {
            const int pidx = t + i * GEMV_WAVES * 64;
            if (pidx < total) {
                const int m = pidx / nchunks, c = pidx - m * nchunks;
                float v[16];
                RowLoader<T>::unpack(araw[i], v);
                const uint4 packed = quantize16<false>(v, 1.0f / row_scale[m]);
                *reinterpret_cast<uint4*>(a_lds + (size_t)m * Kp + (size_t)c * 16) = W4 ? digits16(packed) : packed;
                if (first_wg && q.dst) *reinterpret_cast<uint4*>(q.dst + tiled_chunk_offset(m, c, KB)) = packed;
            }
        }
        // a_scale of the epilogue comes from LDS in this path
        RK_TS(1);
    }

    for (int kc0 = 0; kc0 < Kp; kc0 += kc_max) {
        const int kc = min(kc_max, Kp - kc0);
        // stage activations: row-major [MR][kc] in LDS from the tiled buffer
        const int chunks = kc >> 4;
        if (kc0) __syncthreads();
        if constexpr (QT == 0) {
            for (int idx = threadIdx.x; idx < MR * chunks; idx += GEMV_WAVES * 64) {
                const int m = idx / chunks, c = idx - m * chunks;
                const uint4 v = *reinterpret_cast<const uint4*>(g.A + tiled_chunk_offset(m, (kc0 >> 4) + c, KB));
                *reinterpret_cast<uint4*>(a_lds + (size_t)m * kc + (size_t)c * 16) = W4 ? digits16(v) : v;
            }
        } else if constexpr (QT == 3) {
            // int8 rows as the caller holds them (row-major, any alignment, K not padded); the first
            // workgroup also leaves the tiled copy a launch of the re-tiling kernel would have left
            for (int idx = threadIdx.x; idx < MR * chunks; idx += GEMV_WAVES * 64) {
                const int m = idx / chunks, c = idx - m * chunks, gc = (kc0 >> 4) + c;
                uint4 v = make_uint4(0, 0, 0, 0);
                if (m < g.M) {
                    const int8_t* src = static_cast<const int8_t*>(q.src) + (size_t)m * g.K + (size_t)gc * 16;
                    if (gc * 16 + 16 <= g.K && (reinterpret_cast<uintptr_t>(src) & 15) == 0) {
                        v = *reinterpret_cast<const uint4*>(src);
                    } else {
                        uint32_t w[4] = {0, 0, 0, 0};
                        for (int j = 0; j < 16; ++j)
                            if (gc * 16 + j < g.K) w[j >> 2] |= (uint32_t)(uint8_t)src[j] << ((j & 3) * 8);
                        v = make_uint4(w[0], w[1], w[2], w[3]);
                    }
                    if (first_wg && q.dst) store_codes(q.dst + tiled_chunk_offset(m, gc, KB), v);
                }
                *reinterpret_cast<uint4*>(a_lds + (size_t)m * kc + (size_t)c * 16) = v;
            }
        }
        __syncthreads();

        // One group = UNR tiles per wave.  Int4: a tile is a 64-deep super-tile.
        // (counted in load instructions: one of them spans 32 / CW tiles; K is padded to 256 and a
        // chunk but the last holds a multiple of 4096 k, so the tile count is a multiple of that)
        const int tiles = (W4 ? kc >> 6 : kc >> 5) / TPL, tile0 = W4 ? kc0 >> 6 : kc0 >> 5;
        auto load_unit = [&](int unit) -> v4i { return load_tile(unit, tiles, tile0); };
        auto consume_unit = [&](const v4i& wu, int unit) {
            {
                // This lane's tile within the chunk.  Past the end of the chunk the weights are
                // zeros, so whatever the activation read returns does not matter: it lands in the
                // next row or in the padding behind the last one.
                const int tt = unit * TPL + sub;
                if constexpr (!W4) {
#pragma unroll
                    for (int m = 0; m < MR; ++m) {
                        const v4i av = *reinterpret_cast<const v4i*>(a_lds + (size_t)m * kc + (size_t)(tt * 2 + half) * 16);
                        acc[m] = __builtin_amdgcn_sdot4(av.x, wu.x, acc[m], false);
                        acc[m] = __builtin_amdgcn_sdot4(av.y, wu.y, acc[m], false);
                        acc[m] = __builtin_amdgcn_sdot4(av.z, wu.z, acc[m], false);
                        acc[m] = __builtin_amdgcn_sdot4(av.w, wu.w, acc[m], false);
                    }
                } else {
                    // (the staged activations of the lane's 16 k of each 32-deep half: digits, see above)
#pragma unroll
                    for (int s = 0; s < 2; ++s) {
                        const int w0 = s ? wu.z : wu.x, w1 = s ? wu.w : wu.y;
#pragma unroll
                        for (int m = 0; m < MR; ++m) {
                            const v4i av = *reinterpret_cast<const v4i*>(
                                a_lds + (size_t)m * kc + (size_t)((tt * 2 + s) * 2 + half) * 16);
                            dot_digits(av, w0, w1, acc[m], acc_lo[m]);
                        }
                    }
                }
            }
        };
        if constexpr (ROLLING) {
            // A rolling window of UNR loads per wave: as soon as a tile is used, the
            // register it sat in takes the load of the tile UNR places further on, so the
            // number of loads in flight does not drain between groups (a workgroup of a narrow
            // matrix walks a long K alone on its compute unit).  The fused path starts from the
            // group fetched ahead of the prologue (it has a single K chunk).
            // The staged activations of a tile are read one step ahead of its use, so that
            // their LDS latency does not sit between the arrival of a tile and the next load.
            struct ActTile { v4i a[W4 ? 2 : 1]; };
            auto read_act = [&](int unit) {
                const int tt = unit * TPL + sub; // (past the end of the chunk: the next row or the padding)
                ActTile r;
                if constexpr (!W4) {
                    r.a[0] = *reinterpret_cast<const v4i*>(a_lds + (size_t)(tt * 2 + half) * 16);
                } else {
#pragma unroll
                    for (int s = 0; s < 2; ++s)
                        r.a[s] = *reinterpret_cast<const v4i*>(a_lds + (size_t)((tt * 2 + s) * 2 + half) * 16);
                }
                return r;
            };
            auto dot_tile = [&](const v4i& wu, const ActTile& t) {
                if constexpr (!W4) {
                    acc[0] = __builtin_amdgcn_sdot4(t.a[0].x, wu.x, acc[0], false);
                    acc[0] = __builtin_amdgcn_sdot4(t.a[0].y, wu.y, acc[0], false);
                    acc[0] = __builtin_amdgcn_sdot4(t.a[0].z, wu.z, acc[0], false);
                    acc[0] = __builtin_amdgcn_sdot4(t.a[0].w, wu.w, acc[0], false);
                } else {
                    dot_digits(t.a[0], wu.x, wu.y, acc[0], acc_lo[0]);
                    dot_digits(t.a[1], wu.z, wu.w, acc[0], acc_lo[0]);
                }
            };
            v4i w[UNR];
#pragma unroll
            for (int u = 0; u < UNR; ++u) {
                if constexpr (FUSEQ) w[u] = wpre[u];
                else w[u] = load_unit(wave + u * GEMV_WAVES);
            }
            ActTile cur = read_act(wave);
            for (int tb = wave; tb < tiles; tb += GEMV_WAVES * UNR) {
#pragma unroll
                for (int u = 0; u < UNR; ++u) {
                    const ActTile nxt = read_act(tb + (u + 1) * GEMV_WAVES);
                    dot_tile(w[u], cur);
                    w[u] = load_unit(tb + (UNR + u) * GEMV_WAVES);
                    // (each load stays behind the use of its register; gathered at the end of the
                    // iteration, as the scheduler would have them, the window drains every time)
                    __builtin_amdgcn_sched_barrier(0);
                    cur = nxt;
                }
            }
        } else {
            // A group of UNR loads at a time.  Several rows: the rolling window above costs
            // those variants more registers than two workgroups per compute unit leave.  Wide
            // matrices: they are bound by memory throughput, not by a workgroup's own latency, and
            // a workgroup that asks for its next 64 KiB in one go is served faster than one that
            // trickles the requests out a tile at a time (4096 x 14336, int8: 11.5 against 11.9 us).
            int tb = wave;
            if constexpr (FUSEQ) {
#pragma unroll
                for (int u = 0; u < UNR; ++u)
                    if (tb + u * GEMV_WAVES < tiles) consume_unit(wpre[u], tb + u * GEMV_WAVES);
                tb += GEMV_WAVES * UNR;
            }
            for (; tb < tiles; tb += GEMV_WAVES * UNR) {
                v4i w[UNR];
#pragma unroll
                for (int u = 0; u < UNR; ++u) w[u] = load_unit(tb + u * GEMV_WAVES);
#pragma unroll
                for (int u = 0; u < UNR; ++u)
                    if (tb + u * GEMV_WAVES < tiles) consume_unit(w[u], tb + u * GEMV_WAVES);
            }
        }
    }

    RK_TS(2);
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        int v = W4 ? 16 * acc[m] + acc_lo[m] : acc[m];
        v += __shfl_xor(v, 32);
        if (CW <= 16) v += __shfl_xor(v, 16);
        if (CW <= 8) v += __shfl_xor(v, 8);
        if (lane < CW) red[wave][m][lane] = v;
    }
    __syncthreads();
    static_assert(MR * 32 <= GEMV_WAVES * 64, "one output element per thread");
    if ((int)threadIdx.x < MR * CW) {
        const int m = (int)threadIdx.x / CW, j = (int)threadIdx.x % CW;
        if (m >= g.M) return;
        RK_TS(3);
        int sum = 0;
#pragma unroll
        for (int w = 0; w < GEMV_WAVES; ++w) sum += red[w][m][j];
        const int n = block_first_col(p, g.interleave_F) + col0 + j;
        if (W4 && n < g.N) sum += 8 * g.w_colsum[n]; // (the constant term of the digit split)
        if (n < g.N)
            store_out(g.C, g.epilogue, (size_t)m * g.ldc + n, sum,
                      FUSEQ ? row_scale[m] : (g.a_scale ? g.a_scale[m] : 1.0f),
                      g.w_scale ? g.w_scale[n] : 1.0f);
    }
}


// ---- gate/up GEMV with the SwiGLU epilogue (one or two rows, quantized rows in g.A) ----
// One workgroup per 32 columns of the middle: its gate block (physical block 2j)
// and its up block (2j + 1) are neighbours in the weight buffer, so the eight
// waves stream both over their interleaved k-tiles exactly as gemv_kernel streams
// one, with two accumulators per row.  The epilogue is the one of the GEMM
// kernels: middle = silu_poly(gate) * up per element, one partial row maximum
// per (row, 32 columns).  With few rows the SwiGLU GEMM is a weight stream like
// any decode GEMV; on the MFMA kernel (one 32-row tile, 31 of them padding) the
// gate/up projection of a 4096 -> 14336 FFN took 14.9 us.
constexpr int GEMV_SWIGLU_UNROLL = 4; // load instructions per wave and block in flight (two blocks)

// QT as in gemv_kernel: 0 = quantized rows in g.A, 1 / 2 = the kernel quantizes the fp16 / fp32
// rows q.src itself (same prologue: rows requested first, then the first group of weights).
template <int MR, bool W4, int QT>
__global__ __launch_bounds__(GEMV_WAVES * 64) __attribute__((amdgpu_waves_per_eu(GEMV_WAVES / 2)))
void gemv_swiglu_kernel(RK_GEMV_HEAD_PARAMS, rkh_gemm_args g, rkh_quant_args q) {
    RK_GEMV_HEAD_APPLY(g, q);
    __shared__ __attribute__((aligned(16))) uint8_t a_lds[GEMV_LDS_BYTES];
    __shared__ int red[2][GEMV_WAVES][MR][32];
    __shared__ uint32_t row_max[MR];
    __shared__ float row_scale[MR];
    const int lane = lane_id(), wave = wave_id();
    const int half = lane >> 5;
    const int Kp = (int)rkh_align_up(g.K, RKH_K_ALIGN);
    const int KB = Kp / 32;
    const int F = g.interleave_F;
    const int j = blockIdx.x; // 32-column block of the middle
    const int kc_max = (GEMV_LDS_BYTES / MR) & ~63;
    int acc[2][MR], acc_lo[2][MR]; // (int4 weights: sums of the high / low activation digits, see split_digits)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int m = 0; m < MR; ++m) acc[b][m] = acc_lo[b][m] = 0;

    const size_t block_bytes = (size_t)(W4 ? Kp / 64 : KB) * 1024; // one column block over all of K
    const uint8_t* wbase = g.W + (size_t)(2 * j) * block_bytes;    // gate block, the up block right behind it
    // (bounds-checked descriptor over the two blocks: see gemv_kernel)
    const __amdgpu_buffer_rsrc_t wrsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(wbase), 0, (int)(2 * block_bytes), 0x00020000);
    v4i w[2][GEMV_SWIGLU_UNROLL];
    auto load_group = [&](int tb, int tiles, int tile0) {
#pragma unroll
        for (int u = 0; u < GEMV_SWIGLU_UNROLL; ++u)
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const int tt = tb + u * GEMV_WAVES;
                const unsigned off = tt < tiles ? (unsigned)(b * block_bytes) + (unsigned)(tile0 + tt) * 1024u + (unsigned)lane * 16u
                                                : 0xFFFFFFF0u;
                w[b][u] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, (int)off, 0, 2 /* streaming */));
            }
    };

    if constexpr (QT != 0) { // (the fused path has a single K chunk: rows fit the staging area)
        using T = typename std::conditional<QT == 2, float, uint16_t>::type;
        const int t = threadIdx.x;
        const bool first_wg = blockIdx.x == 0;
        const int K = g.K, nchunks = (K + 15) >> 4, total = g.M * nchunks;
        typename RowLoader<T>::Raw araw[GEMV_QCHUNKS];
#pragma unroll
        for (int i = 0; i < GEMV_QCHUNKS; ++i) {
            const int pidx = t + i * GEMV_WAVES * 64;
            if (pidx < total) {
                const int m = pidx / nchunks, c = pidx - m * nchunks;
                const T* row = static_cast<const T*>(q.src) + (size_t)m * K;
                araw[i] = RowLoader<T>::load16_raw(row, c * 16, K, (reinterpret_cast<uintptr_t>(row) & 15) == 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        load_group(wave, W4 ? Kp >> 6 : Kp >> 5, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (t < MR) row_max[t] = 0u;
        __syncthreads();
        bool bad = false;
#pragma unroll
        for (int i = 0; i < GEMV_QCHUNKS; ++i) {
            const int pidx = t + i * GEMV_WAVES * 64;
            if (pidx < total) {
                const int m = pidx / nchunks;
                float v[16];
                RowLoader<T>::unpack(araw[i], v);
                float mx = 0.0f;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    mx = fmaxf(mx, fabsf(v[e]));
                    bad |= not_finite(v[e]);
                }
                atomicMax(&row_max[m], __float_as_uint(mx)); // non-negative floats order like their bits
            }
        }
        __syncthreads();
        if (t < g.M) {
            const float mx = __uint_as_float(row_max[t]);
            const float sc = q.mode == RKH_Q_W4A8 ? (mx == 0.0f ? 1.0f : fmaxf(mx / 127.0f, FLT_MIN))
                                                  : (mx > 0.0f ? mx / 127.0f : 1.0f);
            row_scale[t] = sc;
            if (first_wg && q.scale) q.scale[t] = sc;
        }
        if (first_wg && bad && q.mode == RKH_Q_W4A8 && q.bad_flag) atomicOr(q.bad_flag, 1);
        for (int idx = t; idx < g.M * ((Kp >> 4) - nchunks); idx += GEMV_WAVES * 64) { // zero the K padding
            const int m = idx / ((Kp >> 4) - nchunks), c = nchunks + idx % ((Kp >> 4) - nchunks);
            *reinterpret_cast<uint4*>(a_lds + (size_t)m * Kp + (size_t)c * 16) = make_uint4(0, 0, 0, 0);
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < GEMV_QCHUNKS; ++i) {
            const int pidx = t + i * GEMV_WAVES * 64;
            if (pidx < total) {
                const int m = pidx / nchunks, c = pidx - m * nchunks;
                float v[16];
                RowLoader<T>::unpack(araw[i], v);
                const uint4 packed = quantize16<false>(v, 1.0f / row_scale[m]);
                *reinterpret_cast<uint4*>(a_lds + (size_t)m * Kp + (size_t)c * 16) = W4 ? digits16(packed) : packed;
                if (first_wg && q.dst) *reinterpret_cast<uint4*>(q.dst + tiled_chunk_offset(m, c, KB)) = packed;
            }
        }
    }

    for (int kc0 = 0; kc0 < Kp; kc0 += kc_max) {
        const int kc = min(kc_max, Kp - kc0);
        const int chunks = kc >> 4;
        if (kc0) __syncthreads();
        if constexpr (QT == 0) {
            for (int idx = threadIdx.x; idx < MR * chunks; idx += GEMV_WAVES * 64) {
                const int m = idx / chunks, c = idx - m * chunks;
                const uint4 v = *reinterpret_cast<const uint4*>(g.A + tiled_chunk_offset(m, (kc0 >> 4) + c, KB));
                *reinterpret_cast<uint4*>(a_lds + (size_t)m * kc + (size_t)c * 16) = W4 ? digits16(v) : v;
            }
        }
        __syncthreads();

        const int tiles = W4 ? kc >> 6 : kc >> 5, tile0 = W4 ? kc0 >> 6 : kc0 >> 5;
        for (int tb = wave; tb < tiles; tb += GEMV_WAVES * GEMV_SWIGLU_UNROLL) {
            if (QT == 0 || tb != wave) load_group(tb, tiles, tile0); // (fused: the first group is on its way)
#pragma unroll
            for (int u = 0; u < GEMV_SWIGLU_UNROLL; ++u) {
                const int tt = tb + u * GEMV_WAVES;
                if (tt >= tiles) continue;
#pragma unroll
                for (int b = 0; b < 2; ++b) {
                    if constexpr (!W4) {
#pragma unroll
                        for (int m = 0; m < MR; ++m) {
                            const v4i av = *reinterpret_cast<const v4i*>(a_lds + (size_t)m * kc + (size_t)(tt * 2 + half) * 16);
                            acc[b][m] = __builtin_amdgcn_sdot4(av.x, w[b][u].x, acc[b][m], false);
                            acc[b][m] = __builtin_amdgcn_sdot4(av.y, w[b][u].y, acc[b][m], false);
                            acc[b][m] = __builtin_amdgcn_sdot4(av.z, w[b][u].z, acc[b][m], false);
                            acc[b][m] = __builtin_amdgcn_sdot4(av.w, w[b][u].w, acc[b][m], false);
                        }
                    } else {
#pragma unroll
                        for (int s = 0; s < 2; ++s) {
                            const int w0 = s ? w[b][u].z : w[b][u].x, w1 = s ? w[b][u].w : w[b][u].y;
#pragma unroll
                            for (int m = 0; m < MR; ++m) {
                                const v4i av = *reinterpret_cast<const v4i*>(
                                    a_lds + (size_t)m * kc + (size_t)((tt * 2 + s) * 2 + half) * 16);
                                dot_digits(av, w0, w1, acc[b][m], acc_lo[b][m]);
                            }
                        }
                    }
                }
            }
        }
    }

#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            int v = W4 ? 16 * acc[b][m] + acc_lo[b][m] : acc[b][m];
            v += __shfl_xor(v, 32);
            if (lane < 32) red[b][wave][m][lane] = v;
        }
    __syncthreads();
    static_assert(MR * 32 <= GEMV_WAVES * 64, "one output element per thread");
    if ((int)threadIdx.x < MR * 32) { // a row of 32 columns per half wave
        const int m = (int)threadIdx.x >> 5, c = (int)threadIdx.x & 31;
        const int n = j * 32 + c;
        const bool live = m < g.M && n < F;
        int gate = 0, up = 0;
#pragma unroll
        for (int w = 0; w < GEMV_WAVES; ++w) {
            gate += red[0][w][m][c];
            up += red[1][w][m][c];
        }
        uint32_t bits = 0;
        if (live) {
            if (W4) { // (the constant term of the digit split)
                gate += 8 * g.w_colsum[n];
                up += 8 * g.w_colsum[F + n];
            }
            const float as = QT != 0 ? row_scale[m] : (g.a_scale ? g.a_scale[m] : 1.0f);
            const float gf = dequant(gate, as, g.w_scale ? g.w_scale[n] : 1.0f);
            const float uf = dequant(up, as, g.w_scale ? g.w_scale[F + n] : 1.0f);
            const float y = __fmul_rn(silu_poly(gf), uf);
            static_cast<float*>(g.C)[(size_t)m * g.ldc + n] = y;
            bits = __float_as_uint(y) & 0x7fffffffu;
        }
#pragma unroll
        for (int d = 16; d > 0; d >>= 1) bits = max(bits, (uint32_t)__shfl_xor((int)bits, d));
        if (g.row_max_bits && c == 0 && m < g.M) g.row_max_bits[(size_t)m * (F / 32) + j] = bits;
    }
}

// ------------------------------------------------------------------ GEMM
__device__ __forceinline__ int xcd_remap(int bid, int total) {
    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD one
    // contiguous range of logical tiles so neighbours share its L2.
    const int q = total >> 3, r = total & 7;
    const int xcd = bid & 7, idx = bid >> 3;
    return xcd * q + min(xcd, r) + idx;
}

// LDS-only workgroup barrier: waits for this wave's LDS traffic and joins the
// barrier, but leaves global loads in flight (the K loop keeps prefetches
// outstanding across it).  The "memory" clobber stops the compiler from moving
// LDS accesses across it.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ---- accumulator tile layout ------------------------------------------------
// The weights are the FIRST MFMA operand and the activations the second, so a
// 32x32 accumulator tile holds D[n_local][m_local]: lane l owns activation row
// m_local = l % 32 and the 16 weight columns
//     n_local(r) = 8 * (r / 4) + 4 * (l / 32) + (r % 4),  r = 0..15,
// i.e. four runs of four consecutive output columns of ONE output row.  That
// makes the per-row quantities (a_scale, SwiGLU row maximum) lane-local and the
// stores row-contiguous.
__device__ __forceinline__ int tile_col(int r, int lane) {
    return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
}

// Write one finished 32x32 tile of output elements to C[m0.., n0..] through a
// wave-private LDS staging area so that global stores are 16 bytes per lane and
// row-contiguous.  vals[r] is the element for (m0 + lane%32, n0 + tile_col(r)).
template <typename T>
__device__ __forceinline__ void store_tile(T* C, int ldc, int m0, int n0, int m_limit, int n_limit,
                                           const T* vals, uint8_t* stage_lds, int lane) {
    constexpr int ES = sizeof(T);
    constexpr int ROW = 32 * ES + 8;            // padded row pitch: conflict-free for b64 / b128
    constexpr int CHUNKS_PER_ROW = 32 * ES / 16; // 16-byte pieces per row
    const bool aligned = ((reinterpret_cast<uintptr_t>(C) | ((size_t)ldc * ES) | ((size_t)n0 * ES)) & 15) == 0;
    if (aligned && n0 + 32 <= n_limit) {
        const int ml = lane & 31;
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
            const int col = 8 * gq + 4 * (lane >> 5);
            T* dst = reinterpret_cast<T*>(stage_lds + ml * ROW + col * ES);
#pragma unroll
            for (int q = 0; q < 4; ++q) dst[q] = vals[gq * 4 + q];
        }
        __builtin_amdgcn_wave_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int t = 0; t < CHUNKS_PER_ROW * 32 / 64; ++t) {
            const int c = lane + 64 * t;
            const int row = c / CHUNKS_PER_ROW, part = c % CHUNKS_PER_ROW;
            // rows are 8 bytes past a 16-byte boundary apart, so read as two 8-byte halves
            const uint2 lo = *reinterpret_cast<const uint2*>(stage_lds + row * ROW + part * 16);
            const uint2 hi = *reinterpret_cast<const uint2*>(stage_lds + row * ROW + part * 16 + 8);
            if (m0 + row < m_limit) // the output is not read again by this kernel: streaming store
                __builtin_nontemporal_store(v4i{(int)lo.x, (int)lo.y, (int)hi.x, (int)hi.y},
                                            reinterpret_cast<v4i*>(reinterpret_cast<uint8_t*>(C) +
                                                                   ((size_t)(m0 + row) * ldc + n0) * ES + part * 16));
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
    } else {
        const int m = m0 + (lane & 31);
        if (m < m_limit) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int n = n0 + tile_col(r, lane);
                if (n < n_limit) C[(size_t)m * ldc + n] = vals[r];
            }
        }
    }
}

// Weight scales of the 16 columns a lane owns in the tile whose first logical
// column is n0 (zero beyond the matrix).
__device__ __forceinline__ void load_col_scales(float* ws, const float* w_scale, int n0, int n_limit,
                                                int lane) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int n = n0 + tile_col(r, lane);
        ws[r] = n < n_limit ? w_scale[n] : 0.0f;
    }
}

// Dequantize and store one accumulator tile whose physical column block is p;
// as / ws are the lane's row scale and its 16 column scales.
template <int EPI>
__device__ __forceinline__ void epilogue_tile_scaled(const rkh_gemm_args& g, const v16i& acc, int m0,
                                                     int p, int lane, float as, const float* ws,
                                                     int m_limit, uint8_t* stage_lds) {
    // padding blocks beyond the matrix hold zeros; with interleaved columns their
    // logical index would alias a real column, so test the block itself
    if (g.interleave_F ? p >= g.N / 32 : p * 32 >= g.N) return;
    const int n0 = block_first_col(p, g.interleave_F);
    if constexpr (EPI == RKH_EPI_I32) {
        int vals[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) vals[r] = acc[r];
        store_tile<int>(static_cast<int*>(g.C), g.ldc, m0, n0, m_limit, g.N, vals, stage_lds, lane);
    } else {
        float y[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) y[r] = dequant(acc[r], as, ws[r]);
        if constexpr (EPI == RKH_EPI_F16) {
            __half h[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) h[r] = __float2half_rn(y[r]);
            store_tile<__half>(static_cast<__half*>(g.C), g.ldc, m0, n0, m_limit, g.N, h, stage_lds, lane);
        } else {
            store_tile<float>(static_cast<float*>(g.C), g.ldc, m0, n0, m_limit, g.N, y, stage_lds, lane);
        }
    }
}

template <int EPI>
__device__ __forceinline__ void epilogue_tile(const rkh_gemm_args& g, const v16i& acc, int m0, int p,
                                              int lane, const float* a_scale, const float* w_scale,
                                              int m_limit, uint8_t* stage_lds) {
    if (g.interleave_F ? p >= g.N / 32 : p * 32 >= g.N) return;
    float as = 0.0f, ws[16];
    if constexpr (EPI != RKH_EPI_I32) {
        const int m = m0 + (lane & 31);
        as = m < m_limit ? a_scale[m] : 0.0f;
        load_col_scales(ws, w_scale, block_first_col(p, g.interleave_F), g.N, lane);
    }
    epilogue_tile_scaled<EPI>(g, acc, m0, p, lane, as, ws, m_limit, stage_lds);
}

// gate tile (physical block p, even) + up tile (p + 1) -> 32 columns of the
// middle and one partial row maximum per (row, 32-column block).  wsg / wsu are
// the lane's gate and up column scales.
__device__ __forceinline__ void epilogue_swiglu_scaled(const rkh_gemm_args& g, const v16i& gate,
                                                       const v16i& up, int m0, int p, int lane,
                                                       float as, const float* wsg, const float* wsu,
                                                       int m_limit, uint8_t* stage_lds) {
    const int F = g.interleave_F;
    const int n0 = (p >> 1) * 32;
    if (n0 >= F) return;
    const int m = m0 + (lane & 31);
    float y[16];
    uint32_t bits = 0;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const float gf = dequant(gate[r], as, wsg[r]);
        const float uf = dequant(up[r], as, wsu[r]);
        y[r] = __fmul_rn(silu_poly(gf), uf);
        bits = max(bits, __float_as_uint(y[r]) & 0x7fffffffu);
    }
    store_tile<float>(static_cast<float*>(g.C), g.ldc, m0, n0, m_limit, F, y, stage_lds, lane);
    if (g.row_max_bits) {
        bits = max(bits, (uint32_t)__shfl_xor((int)bits, 32));
        if (lane < 32 && m < m_limit) g.row_max_bits[(size_t)m * (F / 32) + (p >> 1)] = bits;
    }
}

__device__ __forceinline__ void epilogue_swiglu(const rkh_gemm_args& g, const v16i& gate,
                                                const v16i& up, int m0, int p, int lane,
                                                const float* a_scale, const float* w_scale,
                                                int m_limit, uint8_t* stage_lds) {
    const int F = g.interleave_F;
    const int n0 = (p >> 1) * 32;
    if (n0 >= F) return;
    const int m = m0 + (lane & 31);
    const float as = m < m_limit ? a_scale[m] : 0.0f;
    float wsg[16], wsu[16];
    load_col_scales(wsg, w_scale, n0, F, lane);
    load_col_scales(wsu, w_scale + F, n0, F, lane);
    epilogue_swiglu_scaled(g, gate, up, m0, p, lane, as, wsg, wsu, m_limit, stage_lds);
}

// ---- tiles of (32 * TM) rows x 256 columns, waves split K --------------------
// Eight waves = 4 column groups (wn) x 2 k-halves (wk): wave (wn, wk)
// accumulates the whole (32*TM) x 64 strip of column group wn, but only over
// every second 32-deep k-tile (k-tile % 2 == wk); the two halves are summed
// once, through LDS, before the epilogue.  Compared with splitting the rows
// between the two waves that share a SIMD, no weight byte is loaded (or
// unpacked) by two waves, which takes a third off the traffic through the
// vector memory path and halves the int4 unpack work.
//
// A sub-step always covers 8 KiB of activations = (32*TM) rows x (8/TM)
// k-tiles, i.e. 64 / 128 / 256 k for TM = 4 / 2 / 1, so that whatever the tile
// height a wave issues per sub-step one 1 KiB activation copy, four 16-byte
// fragment reads and eight MFMAs.
//
// Activations: every wave copies its 1 KiB share of a sub-step global -> LDS
// directly (no registers), D sub-steps ahead (WK_D; 8 for the 128-row tile), into
// a ring of WK_NBUF buffers.  Weights: global -> registers, NSW-1 sub-steps ahead (8 bytes per
// lane and k-tile pair for int4, 16 per k-tile for int8).  The fragments of
// the NEXT sub-step are read and, for int4, its operands unpacked in the
// shadow of this sub-step's MFMAs.
//
// A workgroup barrier costs a good part of a sub-step's MFMA time (the matrix
// pipes drain while the waves meet), so there is only one every WK_G
// sub-steps.
//
// All loads of the loop are inline assembly and every wait is explicit.  (The
// compiler's own bookkeeping orders each LDS read and each register load after
// ALL outstanding global -> LDS copies, which would undo the prefetch.)  The
// waits rely on vector memory loads completing in issue order and on every
// sub-step issuing exactly LPS loads -- copy first, then weights -- also
// beyond the end of K, where the source pointers simply stop advancing (those
// loads hit the L1 and their results are never used).  With that:
//  * weights of sub-step s+1 were issued at s+1-(NSW-1); (NSW-2) * LPS loads
//    have been issued since, hence vmcnt((NSW-2) * LPS);
//  * publication: the fragments read during sub-steps B+1..B+G (B = last
//    sub-step before a barrier) belong to sub-steps <= B+G+1; their copies
//    were issued at sub-steps <= B+G+1-D, before the weights a wave waits for
//    during sub-step B, so they have landed when it reaches the barrier
//    (needs D >= NSW + G - 1);
//  * reuse: the copy issued at sub-step s overwrites the buffer that held
//    sub-step s+D-NBUF, last read at sub-step s+D-NBUF-1 <= s-G-1, which is
//    before the latest barrier (needs NBUF >= D + G).
//
// Split K over workgroups (ksplit > 1, small M): every part stores its int32
// tile in accumulator order to scratch and gemm_wk_reduce_kernel, launched
// behind it, adds the parts and runs the epilogue.  (Summing inside this
// kernel, in the part that arrives last, needs a device-scope release per
// workgroup; on this multi-die part each one walks the die's L2, and 32
// workgroups per die queueing for that cost more than the second launch.)
constexpr int WK_NBUF = 16, WK_G = 4, WK_D = 12, WK_BUF = 8 * 1024;
constexpr int WK_SCALES_OFF = WK_NBUF * WK_BUF;                   // fp32 scales of the tile: 128 rows, then 256 columns
constexpr int WK_LDS_BYTES = WK_SCALES_OFF + (128 + 256) * 4;

typedef __attribute__((address_space(3))) uint8_t* lds_ptr_t;

// Row / column block of logical dense tile `tile`: column sweeps over groups of
// 4 row blocks, so that concurrently running tiles share weight columns in L2.
__device__ __forceinline__ void wk_tile_coords(int tile, int mblocks, int nblocks, int& mblk, int& nblk) {
    constexpr int GM = 4;
    const int per_group = GM * nblocks;
    const int group = tile / per_group;
    const int first_m = group * GM;
    const int gm = min(mblocks - first_m, GM);
    const int in_group = tile - group * per_group;
    mblk = first_m + in_group % gm;
    nblk = in_group / gm;
}

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm" // m0 is set and clobbered on purpose below
template <int TM, bool W4, int EPI>
__global__ __launch_bounds__(512) void gemm_wk_kernel(const uint8_t* h_A, const uint8_t* h_W, int h_M, int h_K,
                                                      int mblocks, int nblocks, int ksplit, int ksteps_per_part,
                                                      rkh_gemm_args g) {
    // (leading scalar arguments, see RK_GEMM_HEAD_PARAMS: everything the tile coordinates and the
    // prologue's loads depend on, ten dwords, arrives in registers)
    g.A = h_A; g.W = h_W; g.M = h_M; g.K = h_K;
    RK_TS(0);
    constexpr int TN = 2, KTS = 8 / TM, KTW = KTS / 2; // k-tiles per sub-step: all / this wave's
    // Look-ahead: weights NSW - 1 sub-steps, activation copies D sub-steps.  The 128-row tile runs
    // one tile per compute unit, all of them at once, so what the prologue requests before the first
    // MFMA (D copies + NSW - 1 weight groups per wave, 152 KB per compute unit with 8 / 12) is
    // issue-bound in the vector memory path: in-kernel time stamps showed 1.9 us until the requests
    // were out and 3.1 us until the first MFMA.  4 / 8 is enough to cover the latency (a sub-step
    // is ~570 cycles) and starts the loop sooner: 2048 x 4096 x 4096, same box, int8 weights
    // 30.8 -> 30.25 us, int4 32.55 -> 32.15 us.  (The 64-row int4 tile measured the same with
    // either depth and keeps the deeper one.)
    constexpr int NSW = TM == 4 ? 4 : (TM == 2 && W4) ? 8 : 4;
    constexpr int NBUF = WK_NBUF, G = WK_G, D = TM == 4 ? 8 : WK_D, BM = 32 * TM, BUF = WK_BUF;
    constexpr int UNR = 16;            // sub-steps per unrolled trip: multiple of NSW, NBUF, G and 2
    // int4 weights come in 1 KiB super-tiles of two k-tiles (16 bytes per lane).  When a
    // wave has two or more k-tiles per sub-step it takes WHOLE super-tiles (k-tiles
    // 4v + 2*wk, 4v + 2*wk + 1), one 16-byte load each; taking every second k-tile
    // instead would make both k-halves fetch every cache line for half of its bytes,
    // which doubles the weight traffic through the L1 and makes that the limit of the
    // 64- and 32-row tiles.  (With one k-tile per wave and sub-step, TM = 4, the two
    // halves of a super-tile necessarily go to the two waves, 8 bytes per lane each.)
    constexpr bool PAIRED = W4 && KTW >= 2;
    constexpr int NWOP = KTW * TN;                              // weight operands (k-tile x column block) per sub-step
    constexpr int NWREG = PAIRED ? (KTW / 2) * TN : KTW * TN;   // weight loads (registers of the ring) per sub-step
    constexpr int LPS = 1 + NWREG;                              // loads per sub-step and wave
    static_assert(UNR % NSW == 0 && UNR % NBUF == 0 && UNR % G == 0, "slot arithmetic must be compile-time");
    static_assert(D >= NSW + G - 1 && NBUF >= D + G, "see the ordering rules above");
    static_assert((NSW - 2) * LPS <= 63, "vmcnt field");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[]; // WK_LDS_BYTES

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    const int wn = wave & 3, wk = wave >> 2;
    const int Kp = (int)rkh_align_up(g.K, RKH_K_ALIGN);
    const int KB = Kp / 32;
    const int ksteps_total = KB / KTS;

    // ---- tile assignment: XCD-contiguous ranges, 4 row blocks per column sweep
    const int tiles = mblocks * nblocks;
    const int logical = xcd_remap(blockIdx.x, tiles * ksplit);
    const int kpart = logical / tiles;
    const int tile = logical - kpart * tiles;
    int mblk, nblk;
    wk_tile_coords(tile, mblocks, nblocks, mblk, nblk);
    const int kstep0 = kpart * ksteps_per_part;
    const int ksteps = min(ksteps_per_part, ksteps_total - kstep0); // >= 1 by construction of the launch

    const uint8_t* Wb = g.W;
    const float* w_scale = g.w_scale;
    const int m_limit = g.M;

    // ---- sources: wave-uniform base pointers (scalar registers) + a constant lane offset.
    // activation chunk of this wave: row block wave / KTS, k-tile wave % KTS of the sub-step
    const uint8_t* asrc = g.A + ((size_t)(mblk * TM + wave / KTS) * KB + (size_t)kstep0 * KTS + wave % KTS) * 1024;
    // int8 weights of a wave with four k-tiles per sub-step span 6 KiB; the base
    // sits in the middle so that the 13-bit signed instruction offset reaches all
    constexpr int W_BIAS = (!W4 && KTW > 2) ? 4096 : 0;
    const uint8_t* wsrc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int pb = nblk * 8 + wn * TN + j;
        wsrc[j] = W4 ? Wb + ((size_t)pb * (KB / 2) + (size_t)kstep0 * KTW) * 1024 + (PAIRED ? wk * 1024 : wk * 8)
                     : Wb + ((size_t)pb * KB + (size_t)kstep0 * KTS + wk) * 1024 + W_BIAS;
    }
    const unsigned lane_off = lane * 16;
    constexpr int A_STEP = KTS * 1024, W_STEP = W4 ? KTW * 1024 : KTS * 1024;
    using wraw_t = typename std::conditional<W4 && !PAIRED, v2i, v4i>::type;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds_raw;
    const uint32_t copy_dst = lds_base + wave * 1024; // this wave's chunk inside buffer 0
    // LDS byte addresses of this lane's fragment (row block 0, this wave's first k-tile) in buffers 0 and 8
    uint32_t frag_lo = lds_base + wk * (PAIRED ? 2048 : 1024) + lane * 16;
    uint32_t frag_hi = frag_lo + 8 * BUF;
    int a_left = ksteps - 1, w_left = ksteps - 1; // how often the sources may still advance

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    wraw_t wring[NSW][NWREG]; // weight prefetch ring, index u * TN + j
    v4i afr[2][4];            // activation fragments (index u * TM + i), this sub-step / next
    v4i wop[2][NWOP];         // int4 only: unpacked operands (index u * TN + j), this sub-step / next

    auto copy_a = [&](int buf) { // global -> LDS, 16 bytes per lane, lane-contiguous
        asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(asrc),
                     "s"(copy_dst + buf * BUF)
                     : "memory", "m0");
        asrc += a_left > 0 ? A_STEP : 0;
        --a_left;
    };
    auto load_w = [&](wraw_t* regs) {
        static_for<NWREG>([&](auto e_tag) {
            constexpr int E = decltype(e_tag)::value, U = E / TN, J = E % TN;
            const unsigned off = lane_off; // (locals: asm operands cannot name captures of an enclosing lambda)
            const uint8_t* base = wsrc[J];
            wraw_t r;
            if constexpr (PAIRED) // U counts this wave's super-tiles: every second one of the sub-step
                asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(r) : "v"(off), "s"(base), "n"(U * 2048));
            else if constexpr (W4)
                asm volatile("global_load_dwordx2 %0, %1, %2 offset:%3" : "=v"(r) : "v"(off), "s"(base), "n"(U * 1024));
            else
                asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(r) : "v"(off), "s"(base), "n"(U * 2048 - W_BIAS));
            regs[E] = r;
        });
#pragma unroll
        for (int j = 0; j < TN; ++j) wsrc[j] += w_left > 0 ? W_STEP : 0;
        --w_left;
    };
    // wait until at most (NSW-2)*LPS of this wave's loads are outstanding; regs become valid
    auto w_wait = [&](wraw_t* regs) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NSW - 2) * LPS) : "memory");
#pragma unroll
        for (int e = 0; e < NWREG; ++e) asm volatile("" : "+v"(regs[e]));
    };
    // fragment f = u * TM + i of buffer buf; completion is awaited by frags_wait()
    auto read_frag = [&](v4i& dst, auto buf_tag, auto f_tag) {
        constexpr int BUFI = decltype(buf_tag)::value, FI = decltype(f_tag)::value;
        constexpr int U = FI / TM, I = FI % TM;
        constexpr int KT = PAIRED ? (U / 2) * 4 + U % 2 : 2 * U; // this wave's u-th k-tile, relative to its first
        constexpr int OFF = (BUFI % 8) * BUF + (I * KTS + KT) * 1024;
        static_assert(OFF < 65536, "ds_read offset field");
        const uint32_t addr = BUFI < 8 ? frag_lo : frag_hi;
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
    };
    auto frags_wait = [&](v4i* f) {
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3])::"memory");
    };
    // ring register e of a sub-step -> its operand(s) in dst[NWOP]
    auto unpack_item = [&](v4i* dst, const wraw_t* ring_regs, auto e_tag) {
        constexpr int E = decltype(e_tag)::value;
        if constexpr (PAIRED) {
            constexpr int V = E / TN, J = E % TN; // super-tile V of this wave = its k-tiles 2V, 2V + 1
            const wraw_t raw = ring_regs[E];
            dst[(2 * V) * TN + J] = v4i{(raw.x << 4) & (int)0xF0F0F0F0, raw.x & (int)0xF0F0F0F0,
                                        (raw.y << 4) & (int)0xF0F0F0F0, raw.y & (int)0xF0F0F0F0};
            dst[(2 * V + 1) * TN + J] = v4i{(raw.z << 4) & (int)0xF0F0F0F0, raw.z & (int)0xF0F0F0F0,
                                            (raw.w << 4) & (int)0xF0F0F0F0, raw.w & (int)0xF0F0F0F0};
        } else if constexpr (W4) {
            const wraw_t raw = ring_regs[E];
            dst[E] = v4i{(raw.x << 4) & (int)0xF0F0F0F0, raw.x & (int)0xF0F0F0F0, (raw.y << 4) & (int)0xF0F0F0F0,
                         raw.y & (int)0xF0F0F0F0};
        }
    };

    // Sub-step s; SLOT = s % UNR.
    auto k_step = [&](auto slot_tag) {
        constexpr int SLOT = decltype(slot_tag)::value;
        constexpr int F = SLOT & 1;
        using NextBuf = std::integral_constant<int, (SLOT + 1) % NBUF>;
        constexpr int UPS = (NWREG + 3) / 4; // unpack items per MFMA slot (slots 2..5)
        // The two waves of a SIMD drift apart between barriers (the older one wins
        // every issue conflict) and the one left behind cannot keep the matrix pipe
        // busy alone; the wave that is further into the barrier interval yields.
        __builtin_amdgcn_s_setprio(G - 1 - SLOT % G);
        copy_a((SLOT + D) % NBUF);
        load_w(wring[(SLOT + NSW - 1) % NSW]);
        __builtin_amdgcn_sched_barrier(0);
        static_for<8>([&](auto q_tag) {
            constexpr int Q = decltype(q_tag)::value;
            constexpr int U = Q / (TN * TM), J = Q % (TN * TM) / TM, I = Q % TM;
            if constexpr (W4)
                acc[I][J] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wop[F][U * TN + J], afr[F][U * TM + I], acc[I][J], 0, 0, 0);
            else
                acc[I][J] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wring[SLOT % NSW][U * TN + J], afr[F][U * TM + I],
                                                                  acc[I][J], 0, 0, 0);
            // in the MFMA's shadow: one fragment read of the next sub-step, part of its unpack
            if constexpr (Q < 4) read_frag(afr[F ^ 1][Q], NextBuf{}, std::integral_constant<int, Q>{});
            if constexpr (Q == 1) w_wait(wring[(SLOT + 1) % NSW]);
            if constexpr (W4 && Q >= 2 && Q < 6) {
                static_for<UPS>([&](auto t_tag) {
                    constexpr int E = (Q - 2) * UPS + decltype(t_tag)::value;
                    if constexpr (E < NWREG)
                        unpack_item(wop[F ^ 1], wring[(SLOT + 1) % NSW], std::integral_constant<int, E>{});
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        frags_wait(afr[F ^ 1]);
        if constexpr ((SLOT + 1) % G == 0) asm volatile("s_barrier" ::: "memory");
    };

    // prologue: the same issue order as if the loop had run for sub-steps -D..-1
#pragma unroll
    for (int t = -D; t < 0; ++t) {
        copy_a(t + D);
        if (t + NSW - 1 >= 0) load_w(wring[t + NSW - 1]);
    }
    RK_TS(1);
    // The tile's scales are fetched now, behind the prologue's loads, and handed
    // to the epilogue through LDS after the loop, so the epilogue does not start
    // with a round trip to memory: thread t holds the row scale of row t
    // (t < BM) and the column scale of physical column t (t < 256).  (Two more
    // loads in the queue only make the first sub-steps' waits stricter.)
    float my_as = 0.0f, my_ws = 0.0f;
    bool as_valid = false, ws_valid = false;
    if constexpr (EPI != RKH_EPI_I32) {
        const int t = threadIdx.x;
        const int m = mblk * BM + (t & (BM - 1));
        const int pb = nblk * 8 + ((t & 255) >> 5);
        int n;
        if constexpr (EPI == RKH_EPI_SWIGLU) {
            // pb even = gate, odd = up block of middle columns (pb / 2) * 32
            const int F = g.interleave_F;
            const int nl = (pb >> 1) * 32 + (t & 31);
            n = (pb & 1 ? F : 0) + nl;
            ws_valid = nl < F;
        } else {
            const bool live = g.interleave_F ? pb < g.N / 32 : pb * 32 < g.N;
            n = block_first_col(pb, g.interleave_F) + (t & 31);
            ws_valid = live && n < g.N;
        }
        as_valid = m < m_limit;
        const float* pa = g.a_scale + (as_valid ? m : 0);
        const float* pw = w_scale + (ws_valid ? n : 0);
        asm volatile("global_load_dword %0, %1, off" : "=v"(my_as) : "v"(pa));
        asm volatile("global_load_dword %0, %1, off" : "=v"(my_ws) : "v"(pw));
    }
    w_wait(wring[0]); // weights of sub-step 0 and the copies of sub-steps 0..D-NSW+1 have landed
    asm volatile("s_barrier" ::: "memory");
    static_for<4>([&](auto f_tag) { read_frag(afr[0][decltype(f_tag)::value], std::integral_constant<int, 0>{}, f_tag); });
    static_for<NWREG>([&](auto e_tag) { unpack_item(wop[0], wring[0], e_tag); });
    frags_wait(afr[0]);
    RK_TS(2);

    int s = 0;
    for (; s + UNR <= ksteps; s += UNR) static_for<UNR>([&](auto slot) { k_step(slot); });
    if (s < ksteps)
        static_for<UNR>([&](auto slot) {
            if (s + decltype(slot)::value < ksteps) k_step(slot);
        });
    __builtin_amdgcn_s_setprio(0);
    RK_TS(3);

    // ---- epilogue.  Drain the look-ahead copies (they write LDS) and the scale
    // loads; then every wave is past its last fragment read and LDS is reused.
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(my_as), "+v"(my_ws)::"memory");
    // The weight loads issued for sub-steps beyond K were in flight until this
    // wait, while the compiler regards their destination registers as dead: the
    // uses below keep it from giving one of them to an epilogue value ahead of
    // the wait (the load would then land on top of that value).
#pragma unroll
    for (int t = 0; t < NSW; ++t)
#pragma unroll
        for (int e = 0; e < NWREG; ++e) asm volatile("" : "+v"(wring[t][e]));
    if constexpr (EPI != RKH_EPI_I32) {
        float* sc = reinterpret_cast<float*>(lds_raw + WK_SCALES_OFF);
        const int t = threadIdx.x;
        if (t < BM) sc[t] = as_valid ? my_as : 0.0f;
        if (t < 256) sc[128 + t] = ws_valid ? my_ws : 0.0f;
    }
    lds_barrier();

    // The k-half index is a template tag so that accumulator registers are
    // indexed with constants.  After the exchange a wave owns KEEP row blocks
    // of its strip: TM = 4: blocks 2*wk, 2*wk+1; TM = 2: block wk; TM = 1: the
    // wk = 0 wave owns the block and its partner only hands over.
    auto finish = [&](auto wk_tag) {
        constexpr int WK = decltype(wk_tag)::value;
        constexpr int KEEP = TM == 1 ? (WK == 0 ? 1 : 0) : TM / 2;  // row blocks kept
        constexpr int GIVE = TM == 1 ? (WK == 1 ? 1 : 0) : TM / 2;  // row blocks handed over
        constexpr int KEEP0 = TM == 1 ? 0 : WK * (TM / 2);          // first kept row block
        constexpr int GIVE0 = TM == 1 ? 0 : (WK ^ 1) * (TM / 2);    // first handed-over row block
        constexpr int XT = (TM == 1 ? 1 : TM / 2) * TN;             // tiles per exchange slot of a wave
        int* xch = reinterpret_cast<int*>(lds_raw);
        const int partner = wave ^ 4;
        static_assert(8 * XT * 16 * 64 * 4 <= WK_SCALES_OFF, "exchange area");
#pragma unroll
        for (int t = 0; t < GIVE * TN; ++t) {
            const v16i& give = acc[GIVE0 + t / TN][t % TN];
#pragma unroll
            for (int q = 0; q < 4; ++q)
                *reinterpret_cast<v4i*>(xch + (((wave * XT + t) * 4 + q) * 64 + lane) * 4) =
                    v4i{give[q * 4], give[q * 4 + 1], give[q * 4 + 2], give[q * 4 + 3]};
        }
        lds_barrier();
#pragma unroll
        for (int t = 0; t < KEEP * TN; ++t) {
            v16i& keep = acc[KEEP0 + t / TN][t % TN];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const v4i got = *reinterpret_cast<const v4i*>(xch + (((partner * XT + t) * 4 + q) * 64 + lane) * 4);
                keep[q * 4] += got.x;
                keep[q * 4 + 1] += got.y;
                keep[q * 4 + 2] += got.z;
                keep[q * 4 + 3] += got.w;
            }
        }
        lds_barrier();
        RK_TS(4);

        if (ksplit > 1) {
            // partial tile in accumulator order: [tile][part][owning wave][kept tile][q][lane] x 4 ints
            constexpr int OWNERS = TM == 1 ? 4 : 8;
            constexpr int PER_WAVE = (TM == 1 ? 1 : TM / 2) * TN * 1024;
            const int owner = TM == 1 ? wn : wave;
            int* dst0 = g.splitk_acc + ((size_t)tile * ksplit + kpart) * (OWNERS * PER_WAVE) + owner * PER_WAVE;
#pragma unroll
            for (int t = 0; t < KEEP * TN; ++t) {
                const v16i& mine = acc[KEEP0 + t / TN][t % TN];
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    *reinterpret_cast<v4i*>(dst0 + t * 1024 + (q * 64 + lane) * 4) =
                        v4i{mine[q * 4], mine[q * 4 + 1], mine[q * 4 + 2], mine[q * 4 + 3]};
            }
            return;
        }

        if constexpr (KEEP > 0) {
            float as[KEEP], ws[TN][16];
            if constexpr (EPI != RKH_EPI_I32) {
                const float* sc = reinterpret_cast<const float*>(lds_raw + WK_SCALES_OFF);
#pragma unroll
                for (int ii = 0; ii < KEEP; ++ii) as[ii] = sc[(KEEP0 + ii) * 32 + (lane & 31)];
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) ws[j][r] = sc[128 + (wn * TN + j) * 32 + tile_col(r, lane)];
            } else {
#pragma unroll
                for (int ii = 0; ii < KEEP; ++ii) as[ii] = 0.0f;
            }
            uint8_t* stage_lds = lds_raw + wave * (32 * (32 * 4 + 8));
#pragma unroll
            for (int ii = 0; ii < KEEP; ++ii) {
                constexpr int i0 = KEEP0;
                const int m0 = mblk * BM + (i0 + ii) * 32;
                if constexpr (W4) {
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int r = 0; r < 16; ++r) acc[i0 + ii][j][r] >>= 4;
                }
                const int pb0 = nblk * 8 + wn * TN;
                if constexpr (EPI == RKH_EPI_SWIGLU) {
                    epilogue_swiglu_scaled(g, acc[i0 + ii][0], acc[i0 + ii][1], m0, pb0, lane, as[ii], ws[0], ws[1],
                                           m_limit, stage_lds);
                } else {
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        epilogue_tile_scaled<EPI>(g, acc[i0 + ii][j], m0, pb0 + j, lane, as[ii], ws[j], m_limit,
                                                  stage_lds);
                }
            }
        }
    };
    if (wk == 0) finish(std::integral_constant<int, 0>{});
    else finish(std::integral_constant<int, 1>{});
    RK_TS(5);
}
#pragma clang diagnostic pop

// Second half of a K-split launch.  Workgroup = one wave = one owner of kept
// tiles of an output tile (the wave -> tile ownership gemm_wk_kernel has after
// its k-half exchange): blockIdx.x = tile * OWNERS + owner.  Adds the ksplit
// partial tiles and runs the epilogue.
template <int TM, bool W4, int EPI>
__global__ __launch_bounds__(64) void gemm_wk_reduce_kernel(rkh_gemm_args g, int mblocks, int nblocks, int ksplit) {
    constexpr int TN = 2, BM = 32 * TM;
    constexpr int OWNERS = TM == 1 ? 4 : 8;
    constexpr int KEEP = TM == 1 ? 1 : TM / 2;             // row blocks per owner
    constexpr int PER_WAVE = KEEP * TN * 1024;
    __shared__ __attribute__((aligned(16))) uint8_t stage_lds[32 * (32 * 4 + 8)];
    const int lane = lane_id();
    const int tile = blockIdx.x / OWNERS, owner = blockIdx.x % OWNERS;
    const int wn = owner & 3, wk = owner >> 2;             // TM == 1: owners are the wk == 0 waves
    int mblk, nblk;
    wk_tile_coords(tile, mblocks, nblocks, mblk, nblk);
    const int keep0 = TM == 1 ? 0 : wk * (TM / 2);
    const int* src0 = g.splitk_acc + (size_t)tile * ksplit * (OWNERS * PER_WAVE) + owner * PER_WAVE;
    const int pb0 = nblk * 8 + wn * TN;
#pragma unroll
    for (int ii = 0; ii < KEEP; ++ii) {
        v16i sum[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) sum[j][r] = 0;
        for (int p = 0; p < ksplit; ++p) {
            const int* src = src0 + (size_t)p * (OWNERS * PER_WAVE) + ii * TN * 1024;
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    // int4 weights ride as 16 * code: a part's sum is an exact multiple of 16 that fits
                    // int32 (a part spans at most 2^17 k), but the sum of the parts times 16 need not --
                    // so the factor comes off each part before it is added
                    constexpr int SH = W4 ? 4 : 0;
                    const v4i got = *reinterpret_cast<const v4i*>(src + j * 1024 + (q * 64 + lane) * 4);
                    sum[j][q * 4] += got.x >> SH;
                    sum[j][q * 4 + 1] += got.y >> SH;
                    sum[j][q * 4 + 2] += got.z >> SH;
                    sum[j][q * 4 + 3] += got.w >> SH;
                }
        }
        const int m0 = mblk * BM + (keep0 + ii) * 32;
        if constexpr (EPI == RKH_EPI_SWIGLU) {
            epilogue_swiglu(g, sum[0], sum[1], m0, pb0, lane, g.a_scale, g.w_scale, g.M, stage_lds);
        } else {
#pragma unroll
            for (int j = 0; j < TN; ++j)
                epilogue_tile<EPI>(g, sum[j], m0, pb0 + j, lane, g.a_scale, g.w_scale, g.M, stage_lds);
        }
    }
}

// ---- grouped (MoE) GEMM: 32 sorted rows x 256 columns, weights streamed -----
// With a few dozen rows per expert this GEMM is a weight stream: there are two
// MFMAs per KiB of expert weights.  So there is no LDS staging and no workgroup
// barrier: each of the four waves owns two 32-column blocks of the tile over
// the whole K and runs its own ring of RING k-tiles of loads -- the activation
// tile (1 KiB, shared with the other waves through the L1) and its two weight
// tiles, 16 bytes per lane each -- waiting with an explicit counter (loads
// complete in issue order; every step issues exactly three of them, also
// beyond the end of K, where the sources stop advancing).  Several workgroups
// share a compute unit.  An expert with more than 32 rows has one workgroup per
// row block and column tile; they run side by side and the second one finds
// the weights in L2 (taking all row blocks of an expert into one workgroup was
// measured slower: fewer workgroups than compute units remain; units of two row
// blocks that request the weights once measured the same: the loop waits for the
// first pass from HBM, not for the second one from L2).
// KS = 4 (decode-sized calls, whose handful of row blocks would leave most
// compute units without a workgroup): the tile shrinks to 256 / KS columns and
// KS waves share a column pair, taking 1/KS of K each; their accumulators are
// added through LDS before the first of them runs the epilogue -- KS times as
// many workgroups.
// W4 (int4 weights, dense or an expert bank's int4 images): a step is one
// 64-deep super-tile -- two activation tiles and 1 KiB of packed weights per
// column block, unpacked in registers into the two operands (every code times
// 16, undone by one shift of the accumulators, so K may not exceed 2^17).  A
// bank may hold int4 and int8 experts (routed INT4, shared int8): each format
// has its launch over the same grid, and a workgroup whose row block belongs to
// an expert of the other format exits at once.
template <int EPI, int KS, bool W4, bool BAL = false>
__global__ __launch_bounds__(BAL ? 512 : 256) void gemm_stream_kernel(RK_GEMM_HEAD_PARAMS, int mblocks, int nblocks,
                                                                      rkh_gemm_args g) {
    RK_GEMM_HEAD_APPLY(g);
    constexpr int TN = 2, WAVES = BAL ? 8 : 4;
    constexpr bool KSPLIT = KS > 1;
    static_assert(!BAL || !KSPLIT, "the balanced variant does not split K");
    constexpr int CG = WAVES / KS; // column pairs per workgroup
    // Steps of a wave in flight.  Shallow is faster here: every compute unit holds eight (four)
    // waves that stream, and what a deeper ring adds is queueing in front of the memory system,
    // not throughput.  Measured on one box, the MoE layer of 256 tokens (balanced launch):
    // 74.7 us with 8 steps, 74.4 with 4, 70.5 with 2; the same layer with a workgroup per tile:
    // 77.6 / 76.9 / 74.8; a dense 128-row int4 FFN and a 64-row int8 GEMM (K split over the
    // waves): 51.8 / 51.1 / 53.8 and 9.15 / 8.8 / 9.6 us.  (12 and 16 steps were slower still.)
    // A workgroup per tile without a K split (dense GEMMs of 65..128 rows on wide matrices, mid-sized
    // grouped calls): four -- a wave walks the whole K alone, 128 steps for K = 4096, and with two
    // it waits out a full memory latency per step: int8 128 x 4096 x 11008 took 37.9 us with 2,
    // 25.5 with 4, 25.9 with 8 (x 14336: 39.1 / 27.2 / 28.3).
    constexpr int RING = KSPLIT ? 4 : BAL ? 2 : 4;
    constexpr int AT = W4 ? 2 : 1;   // activation tiles per step
    constexpr int LPS = AT + TN;
    static_assert((RING - 1) * LPS <= 63, "vmcnt field");
    constexpr int STAGE_BYTES = WAVES * 32 * (32 * 4 + 8);
    constexpr int XCH_BYTES = KSPLIT ? CG * (KS - 1) * TN * 16 * 64 * 4 : 0;
    __shared__ __attribute__((aligned(16))) uint8_t stage_raw[STAGE_BYTES + XCH_BYTES];

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    // steps over K: k-tiles (a multiple of 8) or, for int4 weights, super-tiles (a multiple of 4): RING divides both
    const int KB = (int)rkh_align_up(g.K, RKH_K_ALIGN) / (32 * AT);

    [[maybe_unused]] constexpr int TSB = EPI == RKH_EPI_SWIGLU ? 4 : 0; // (debug stamps: the SwiGLU launch keeps its own slots)
    RK_TS(TSB + 0);
    // dense use (no block -> expert table): one weight matrix, every row block live
    const int live_blocks = g.blk_expert ? g.num_blocks[0] : mblocks;

    // One unit of work of a wave: row block mblk x the column pair that starts at column block
    // pair_pb0 (BAL) or the wave's pair of column tile nblk (otherwise).
    auto run_unit = [&](int mblk, int nblk, int pair_pb0) {
    if (mblk >= live_blocks) return;
    const int e = g.blk_expert ? g.blk_expert[mblk] : 0;
    // grouped: this launch serves the experts held in its own format (int4 images come first in a bank)
    if (g.blk_expert && (e < g.int4_experts) != W4) return;
    const uint8_t* Wb = !g.blk_expert ? g.W
                        : W4          ? g.W4 + (size_t)e * g.w4_expert_stride
                                      : g.W + (size_t)(e - g.int4_experts) * g.w_expert_stride;
    const float* w_scale = g.w_scale ? g.w_scale + (size_t)e * g.ws_expert_stride : nullptr;

    // this wave's column blocks and k-tiles [kt0, kt0 + kts)
    const int cg = wave / KS, kq = wave % KS; // column pair, part of K
    const int pb0 = BAL ? pair_pb0 : (nblk * CG + cg) * TN;
    // K split over waves: wave kq takes the steps kq, kq + KS, ... -- interleaved, so that the
    // KS waves of a column pair read KS adjacent KiB of each column block at a time (waves that
    // each walk a private range of memory reached 5.2 TB/s in a read-only test, waves that
    // interleave 6.4)
    const int kts = KB > kq ? (KB - kq + KS - 1) / KS : 0;
    const int kt0 = min(kq, KB - 1); // (a wave without a share still loads in bounds)
    const uint8_t* asrc = g.A + ((size_t)mblk * KB + kt0) * (1024 * AT);
    const uint8_t* wsrc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) wsrc[j] = Wb + ((size_t)(pb0 + j) * KB + kt0) * 1024;
    const unsigned lane_off = lane * 16;
    int left = max(kts, 1) - 1; // how often the sources may still advance

    // The scales of this wave's tile pair are requested now, ahead of every load of the ring
    // (loads return in issue order, so they are back with the first step), and handed to the
    // epilogue through the wave's staging area: fetched at the start of the epilogue they cost
    // it a round trip to memory (an epilogue of 2.8 us instead of 1.4, of a kernel whose loop
    // takes 7).  Lane l holds the row scale of row l % 32 and the column scale of column l % 32
    // of column block l / 32 of the pair.
    const int m0 = mblk * 32;
    const int m_limit = g.blk_expert ? live_blocks * 32 : g.M;
    float my_as = 0.0f, my_ws = 0.0f;
    bool as_ok = false, ws_ok = false;
    if constexpr (EPI != RKH_EPI_I32) {
        const int m = m0 + (lane & 31);
        const int pb = pb0 + (lane >> 5);
        int n;
        if constexpr (EPI == RKH_EPI_SWIGLU) { // pb0 is even: the gate block, its up block right behind it
            const int nl = (pb0 >> 1) * 32 + (lane & 31);
            n = (lane >> 5 ? g.interleave_F : 0) + nl;
            ws_ok = nl < g.interleave_F;
        } else {
            const bool live = g.interleave_F ? pb < g.N / 32 : pb * 32 < g.N;
            n = block_first_col(pb, g.interleave_F) + (lane & 31);
            ws_ok = live && n < g.N;
        }
        as_ok = m < m_limit;
        const float* pa = g.a_scale + (as_ok ? m : 0);
        const float* pw = w_scale + (ws_ok ? n : 0);
        asm volatile("global_load_dword %0, %1, off" : "=v"(my_as) : "v"(pa));
        asm volatile("global_load_dword %0, %1, off" : "=v"(my_ws) : "v"(pw));
    }

    v16i acc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0;
    v4i ring[RING][LPS]; // [0 .. AT) = activation tiles, [AT + j] = weights of column block j

    auto issue = [&](v4i* regs) {
        static_for<LPS>([&](auto l_tag) {
            constexpr int L = decltype(l_tag)::value;
            const unsigned off = lane_off; // (locals: asm operands cannot name captures of an enclosing lambda)
            const uint8_t* base = L < AT ? asrc + L * 1024 : wsrc[L < AT ? 0 : L - AT];
            v4i r;
            asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(r) : "v"(off), "s"(base));
            regs[L] = r;
        });
        const int step = left > 0 ? 1024 * KS : 0;
        asrc += step * AT;
#pragma unroll
        for (int j = 0; j < TN; ++j) wsrc[j] += step;
        --left;
    };
    auto wait = [&](v4i* regs) { // all but the latest (RING-1) steps' loads have landed
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((RING - 1) * LPS) : "memory");
#pragma unroll
        for (int l = 0; l < LPS; ++l) asm volatile("" : "+v"(regs[l]));
    };

#pragma unroll
    for (int t = 0; t < RING - 1; ++t) issue(ring[t]);
    for (int s = 0; s < kts; s += RING)
        static_for<RING>([&](auto slot_tag) {
            constexpr int SLOT = decltype(slot_tag)::value;
            issue(ring[(SLOT + RING - 1) % RING]);
            wait(ring[SLOT]);
            if (SLOT == 0 && s == 0) RK_TS(TSB + 1);
            // (a K share need not be a multiple of RING: the steps past its end reload the last tile and are skipped)
            if ((!KSPLIT && !W4) || s + SLOT < kts) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    if constexpr (W4) {
                        const v4i raw = ring[SLOT][AT + j];
                        const v4i lo = v4i{(raw.x << 4) & (int)0xF0F0F0F0, raw.x & (int)0xF0F0F0F0,
                                           (raw.y << 4) & (int)0xF0F0F0F0, raw.y & (int)0xF0F0F0F0};
                        const v4i hi = v4i{(raw.z << 4) & (int)0xF0F0F0F0, raw.z & (int)0xF0F0F0F0,
                                           (raw.w << 4) & (int)0xF0F0F0F0, raw.w & (int)0xF0F0F0F0};
                        acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(lo, ring[SLOT][0], acc[j], 0, 0, 0);
                        acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(hi, ring[SLOT][AT - 1], acc[j], 0, 0, 0);
                    } else {
                        acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ring[SLOT][AT + j], ring[SLOT][0], acc[j], 0, 0, 0);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    // The look-ahead loads beyond K are still in flight here and the compiler
    // regards their destination registers as dead: without the uses below it may
    // give one of them to an epilogue value ahead of the wait, and the load then
    // lands on top of that value.
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(my_as), "+v"(my_ws)::"memory");
#pragma unroll
    for (int t = 0; t < RING; ++t)
#pragma unroll
        for (int l = 0; l < LPS; ++l) asm volatile("" : "+v"(ring[t][l]));
    RK_TS(TSB + 2);

    if constexpr (KSPLIT) {
        // the other parts of K hand their accumulators to part 0: [column pair][part - 1][tile][q][lane] x 4 ints
        int* xch = reinterpret_cast<int*>(stage_raw + STAGE_BYTES) + cg * (KS - 1) * TN * 16 * 64;
        if (kq > 0) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    *reinterpret_cast<v4i*>(xch + ((((kq - 1) * TN + j) * 4 + q) * 64 + lane) * 4) =
                        v4i{acc[j][q * 4], acc[j][q * 4 + 1], acc[j][q * 4 + 2], acc[j][q * 4 + 3]};
        }
        __syncthreads();
        if (kq > 0) return;
#pragma unroll
        for (int w = 0; w < KS - 1; ++w)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const v4i got = *reinterpret_cast<const v4i*>(xch + (((w * TN + j) * 4 + q) * 64 + lane) * 4);
                    acc[j][q * 4] += got.x;
                    acc[j][q * 4 + 1] += got.y;
                    acc[j][q * 4 + 2] += got.z;
                    acc[j][q * 4 + 3] += got.w;
                }
    }
    if constexpr (W4) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[j][r] >>= 4;
    }
    uint8_t* stage_lds = stage_raw + wave * (32 * (32 * 4 + 8));
    float as = 0.0f, ws[TN][16];
    if constexpr (EPI != RKH_EPI_I32) { // scales: lane-wise registers -> the wave's staging area -> per-lane order
        float* sc = reinterpret_cast<float*>(stage_lds);
        sc[lane] = ws_ok ? my_ws : 0.0f;
        if (lane < 32) sc[64 + lane] = as_ok ? my_as : 0.0f;
        __builtin_amdgcn_wave_barrier();
        as = sc[64 + (lane & 31)];
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) ws[j][r] = sc[j * 32 + tile_col(r, lane)];
        __builtin_amdgcn_wave_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // (read before the staging below overwrites the area)
    }
    // (The epilogue is bound by its vector ALU work -- some 800 instructions of a wave for the
    // SwiGLU pair, 4 cycles each, two waves per SIMD: 4.3 us measured at the end of a unit whose
    // loop takes 14 us, 1.9 us for the plain fp32 tile pair.  A dry pass through the same code
    // while the first loads were in flight, to have it in the instruction cache, changed nothing.)
    if constexpr (EPI == RKH_EPI_SWIGLU) {
        epilogue_swiglu_scaled(g, acc[0], acc[1], m0, pb0, lane, as, ws[0], ws[1], m_limit, stage_lds);
    } else {
#pragma unroll
        for (int j = 0; j < TN; ++j)
            epilogue_tile_scaled<EPI>(g, acc[j], m0, pb0 + j, lane, as, ws[j], m_limit, stage_lds);
    }
    RK_TS(TSB + 3);
    }; // run_unit

    if constexpr (!BAL) {
        const int logical = xcd_remap(blockIdx.x, mblocks * nblocks);
        run_unit(logical % mblocks, logical / mblocks, 0);
    } else {
        // Balanced launch: one workgroup of eight waves per compute unit, the units (live row
        // block, column pair) dealt out in equal contiguous shares -- first to the dies (a
        // workgroup's die is blockIdx % 8), then to the workgroups of a die -- and a share walked
        // by its workgroup's waves in turn.  Consecutive units are column pairs of one row block,
        // so the waves of a workgroup share the activation tiles through the L1, and the row
        // blocks of one expert meet in one die's L2.
        const int pairs = (g.N + 63) / 64;
        const long units = (long)live_blocks * pairs;
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = (int)(gridDim.x + 7 - xcd) >> 3;
        const long die0 = units * xcd / 8, die1 = units * (xcd + 1) / 8;
        const long first = die0 + (die1 - die0) * slot / slots, last = die0 + (die1 - die0) * (slot + 1) / slots;
        for (long u = first + wave; u < last; u += WAVES) run_unit((int)(u / pairs), 0, (int)(u % pairs) * TN);
    }
}

// ---------------------------------------------------- MoE route + scatter
// One workgroup per token.  Live assignments (row-major over [rows, top_k], non-
// zero coefficient) are bucketed by expert id, stably, each bucket padded to a
// multiple of 32 sorted rows; the shared expert (id == experts) gets every row.
// Instead of a routing pass of its own, every workgroup derives the sorted rows
// of its token's assignments from the whole table (a few KiB, served by L2)
// while its token row is on its way from memory:
//   sorted row of assignment i with expert e  =  start[e] + #{live i' < i with expert e},
//   start[e] = sum over e' < e of pad32(count[e']),
// then quantizes the token (or copies pre-quantized codes) into each of those
// rows.  Workgroup 0 also writes the row-block -> expert table and the totals.
// Counting uses wave ballots: each wave owns a contiguous range of assignments;
// lanes with equal keys find each other bit by bit of the key, one lane per
// distinct key adds the group's size to its wave's bins, and the lane that
// holds one of the token's own assignments notes how many equal keys came
// before it.  (LDS atomics on a few dozen hot counters serialize and took three
// times as long.)  The loop is kept rolled: each workgroup runs it once, from a
// cold instruction cache, so straight-line code costs more than it saves.
constexpr int ROUTE_MAX_EXPERTS = 2048;
constexpr int ROUTE_MAX_TOPK = 8;
constexpr int ROUTE_MAX_ASSIGNMENTS = 2048; // rows * top_k

template <typename T>
__global__ __launch_bounds__(256) void moe_scatter_kernel(const int32_t* h_ids, const float* h_routes, const void* h_src,
                                                          int h_rows, int h_top_k, int h_experts, int h_shared, int h_K,
                                                          rkh_moe_scatter_args a) {
    // (leading scalar arguments: see RK_GEMM_HEAD_PARAMS)
    a.ids = h_ids; a.routes = h_routes; a.src = h_src;
    a.rows = h_rows; a.top_k = h_top_k; a.experts = h_experts; a.shared = h_shared; a.K = h_K;
    __shared__ int bins[4][ROUTE_MAX_EXPERTS];   // live assignments per expert, per wave
    __shared__ int start[ROUTE_MAX_EXPERTS + 1]; // first sorted row of each bucket
    __shared__ int own_key[ROUTE_MAX_TOPK], own_rank[ROUTE_MAX_TOPK], own_wave[ROUTE_MAX_TOPK];
    __shared__ int dest[ROUTE_MAX_TOPK + 1];
    __shared__ int wave_total[4];
    __shared__ int wave_live[4];
    __shared__ float wave_max[4];
    __shared__ int wave_bad[4];
    const int m = blockIdx.x, t = threadIdx.x, lane = lane_id(), wave = wave_id();
    const int E = a.experts, top_k = a.top_k, slots = top_k + a.shared, n = a.rows * top_k;
    const int K = a.K, KB = (int)(rkh_align_up(K, RKH_K_ALIGN) / 32);
    const int nchunks = (K + 15) >> 4;
    const T* row = static_cast<const T*>(a.src) + (size_t)m * K;
    const bool vec = ((reinterpret_cast<uintptr_t>(row) & 15) == 0);
    const bool cached = nchunks <= 256 * QR_CACHE;

    // Loads: this wave's share of the routing table first, then the token's row
    // -- loads return in issue order, so the routing can start while the row is
    // still on its way.  Wave w owns assignments [w, w + 1) * per_wave * 64.
    constexpr int PER_WAVE = ROUTE_MAX_ASSIGNMENTS / 256; // 64-assignment groups per wave
    const int per_wave = ((n + 63) / 64 + 3) / 4;
    const int wave_first = wave * per_wave * 64;
    int keys[PER_WAVE]; // expert of a live assignment, -1 if dropped or beyond the table
    bool bad_route = false; // an id outside [0, E) or a coefficient that is negative or not finite
#pragma unroll
    for (int c = 0; c < PER_WAVE; ++c) {
        const int i = wave_first + c * 64 + lane;
        keys[c] = -1;
        if (c < per_wave && i < n) {
            const int id = a.ids[i];
            const float coeff = a.routes[i];
            const bool id_ok = (unsigned)id < (unsigned)E;
            bad_route |= !id_ok || not_finite(coeff) || coeff < 0.0f;
            keys[c] = (coeff != 0.0f && id_ok) ? id : -1;
        }
    }
    // (every workgroup sees the whole table: the first one reports for all)
    if (m == 0 && bad_route && a.bad_flag) atomicOr(a.bad_flag, 1);
    float v[QR_CACHE][16];
    if constexpr (sizeof(T) == 4) {
        if (cached) {
#pragma unroll
            for (int i = 0; i < QR_CACHE; ++i) {
                const int c = t + i * 256;
                if (c < nchunks) RowLoader<T>::load16(row, c * 16, K, vec, v[i]);
            }
        }
    }

    // ---- routing
    for (int e = lane; e < E; e += 64) bins[wave][e] = 0;
    __builtin_amdgcn_wave_barrier(); // a wave only touches its own bins until the workgroup barrier below
    int key_bits = 1;
    while ((1 << key_bits) < E) ++key_bits;
    const unsigned long long below = (1ull << lane) - 1ull;
    const int own0 = m * top_k;
    int live = 0;
#pragma unroll 1
    for (int c = 0; c < per_wave; ++c) {
        const int key = keys[0];
#pragma unroll
        for (int u = 0; u + 1 < PER_WAVE; ++u) keys[u] = keys[u + 1];
        unsigned long long same = __ballot(key >= 0);
        live += __popcll(same);
#pragma unroll 1
        for (int bit = 0; bit < key_bits; ++bit) {
            const unsigned long long set = __ballot((key >> bit) & 1);
            same &= ((key >> bit) & 1) ? set : ~set;
        }
        const int earlier = __popcll(same & below); // equal keys in lower lanes
        int seen = 0;                                // equal keys in this wave's earlier groups
        if (key >= 0) seen = bins[wave][key];
        __builtin_amdgcn_wave_barrier();
        if (key >= 0 && earlier == 0) bins[wave][key] = seen + __popcll(same);
        const int k = wave_first + c * 64 + lane - own0;
        if (k >= 0 && k < top_k) {
            own_key[k] = key;
            own_rank[k] = seen + earlier;
            own_wave[k] = wave;
        }
    }
    if (lane == 0) wave_live[wave] = live;
    __syncthreads();
    // bucket sizes -> padded exclusive scan: 8 experts per thread, a shuffle scan
    // inside each wave, the wave totals through LDS
    constexpr int PER = ROUTE_MAX_EXPERTS / 256;
    const int Etot = E + a.shared;
    int sizes[PER];
    int local = 0;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int e = t * PER + j;
        int cnt = 0;
        if (e < E) cnt = bins[0][e] + bins[1][e] + bins[2][e] + bins[3][e];
        else if (e == E && a.shared) cnt = a.rows;
        sizes[j] = (cnt + 31) & ~31;
        local += sizes[j];
    }
    int incl = local;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(incl, off);
        if (lane >= off) incl += up;
    }
    if (lane == 63) wave_total[wave] = incl;
    __syncthreads();
    int run = incl - local;
    for (int w = 0; w < wave; ++w) run += wave_total[w];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int e = t * PER + j;
        if (e <= Etot) start[e] = run;
        if (m == 0 && e < Etot)
            for (int blk = run / 32; blk < (run + sizes[j]) / 32; ++blk)
                if (blk < a.max_blocks) a.blk_expert[blk] = e;
        run += sizes[j];
    }
    if (m == 0 && t == 255) {
        a.num_blocks[0] = min(run / 32, a.max_blocks);
        a.num_blocks[1] = wave_live[0] + wave_live[1] + wave_live[2] + wave_live[3] + (a.shared ? a.rows : 0);
    }
    __syncthreads();
    if (t < top_k) {
        const int key = own_key[t];
        int d = -1;
        if (key >= 0) {
            d = start[key] + own_rank[t];
            for (int w = 0; w < own_wave[t]; ++w) d += bins[w][key];
        }
        dest[t] = d;
        a.dest_rows[(size_t)m * slots + t] = d;
    } else if (t == top_k && a.shared) {
        const int d = start[E] + m;
        dest[t] = d;
        a.dest_rows[(size_t)m * slots + t] = d;
    }

    // ---- the token into its sorted rows
    if constexpr (sizeof(T) == 1) {
        __syncthreads(); // dest[]
        if (t == 0 && a.bad_flag) { // given scales must be finite and positive (reference :595)
            const float given = a.token_scale[m];
            if (!(given > 0.0f) || not_finite(given)) atomicOr(a.bad_flag, 1);
        }
        if (t < slots && dest[t] >= 0) a.scale_rows[dest[t]] = a.token_scale[m];
        const int8_t* brow = reinterpret_cast<const int8_t*>(row);
        for (int c = t; c < nchunks; c += 256) {
            uint32_t w[4] = {0, 0, 0, 0};
            if (vec && c * 16 + 16 <= K) {
                const uint4 v4 = *reinterpret_cast<const uint4*>(brow + c * 16);
                w[0] = v4.x; w[1] = v4.y; w[2] = v4.z; w[3] = v4.w;
            } else {
                for (int j = 0; j < 16; ++j)
                    if (c * 16 + j < K) w[j >> 2] |= (uint32_t)(uint8_t)brow[c * 16 + j] << ((j & 3) * 8);
            }
            const uint4 packed = make_uint4(w[0], w[1], w[2], w[3]);
            for (int j = 0; j < slots; ++j) {
                const int d = dest[j];
                if (d >= 0) store_codes(a.dst + tiled_chunk_offset(d, c, KB), packed);
            }
        }
    } else {
        float mx = 0.0f;
        bool bad = false;
        if (cached) {
#pragma unroll
            for (int i = 0; i < QR_CACHE; ++i)
                if (t + i * 256 < nchunks) {
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        mx = fmaxf(mx, fabsf(v[i][j]));
                        bad |= not_finite(v[i][j]);
                    }
                }
        } else {
            for (int c = t; c < nchunks; c += 256) {
                float tmp[16];
                RowLoader<T>::load16(row, c * 16, K, vec, tmp);
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    mx = fmaxf(mx, fabsf(tmp[j]));
                    bad |= not_finite(tmp[j]);
                }
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
        const unsigned long long bad_mask = __ballot(bad);
        if (lane == 0) {
            wave_max[wave] = mx;
            wave_bad[wave] = bad_mask != 0ull;
        }
        __syncthreads(); // also dest[]
        mx = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
        if ((wave_bad[0] | wave_bad[1] | wave_bad[2] | wave_bad[3]) && t == 0 && a.bad_flag) atomicOr(a.bad_flag, 1);
        const float scale = mx > 0.0f ? mx / 127.0f : 1.0f;
        const float inv = 1.0f / scale;
        // a maximum so small that the scale underflows to zero or its inverse overflows is
        // rejected like a non-finite token (reference src/rk_npu_moe_w8.cpp:323-324)
        if (t == 0 && a.bad_flag && (!(scale > 0.0f) || not_finite(inv))) atomicOr(a.bad_flag, 1);
        if (t == 0) a.token_scale[m] = scale;
        if (t < slots && dest[t] >= 0) a.scale_rows[dest[t]] = scale;
        auto emit = [&](int c, const float* vals) {
            const uint4 packed = quantize16<true>(vals, inv);
            for (int j = 0; j < slots; ++j) {
                const int d = dest[j];
                if (d >= 0) store_codes(a.dst + tiled_chunk_offset(d, c, KB), packed);
            }
        };
        if (cached) {
#pragma unroll
            for (int i = 0; i < QR_CACHE; ++i)
                if (t + i * 256 < nchunks) emit(t + i * 256, v[i]);
        } else {
            for (int c = t; c < nchunks; c += 256) {
                float tmp[16];
                RowLoader<T>::load16(row, c * 16, K, vec, tmp);
                emit(c, tmp);
            }
        }
    }
}

// out[t, n] = sum over slots, in slot order, of fma(Y[dest, n], w, out); the
// shared expert is the last slot with coefficient 1.
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* h_Y, const int* h_dest_rows, const float* h_routes,
                                                          float* h_out, int h_rows, int h_top_k, int h_shared, int h_H) {
    // (every field as a leading scalar argument: see RK_GEMM_HEAD_PARAMS)
    const rkh_moe_combine_args a = {h_Y, h_dest_rows, h_routes, h_rows, h_top_k, h_shared, h_H, h_out};
    const int tkn = blockIdx.y;
    const int n = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (n >= a.H) return;
    const int slots = a.top_k + a.shared;
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s = 0; s < slots; ++s) {
        const int d = a.dest_rows[(size_t)tkn * slots + s];
        if (d < 0) continue;
        const float w = s < a.top_k ? a.routes[(size_t)tkn * a.top_k + s] : 1.0f;
        const float4 y = *reinterpret_cast<const float4*>(a.Y + (size_t)d * a.H + n);
        sum.x = fmaf(y.x, w, sum.x);
        sum.y = fmaf(y.y, w, sum.y);
        sum.z = fmaf(y.z, w, sum.z);
        sum.w = fmaf(y.w, w, sum.w);
    }
    *reinterpret_cast<float4*>(a.out + (size_t)tkn * a.H + n) = sum;
}


// ------------------------------------------------ MoE layer for a handful of tokens
// With a few tokens the five launches of the layer (route + scatter, grouped gate/up, middle
// re-quantization, grouped down, combine) are almost all latency, and the grouped MFMA kernel
// works on 32-row blocks with one live row.  These two kernels do the same arithmetic with dot
// products, one workgroup of eight waves per (assignment, 32 columns):
//   gate:  token -> int8 (every workgroup quantizes its token itself, the row is an L2 hit after
//          the first), gate and up blocks of the assignment's expert streamed like a decode GEMV,
//          SwiGLU, the fp32 middle and its partial maximum per 32 columns;
//   down:  per token and 32 output columns, the live slots in slot order: the slot's middle row
//          re-quantized from the partial maxima, the expert's down block, dequantization and the
//          fma into the token's sum -- the combine's order and rounding.
// No routing tables: an assignment is live iff its coefficient is non-zero and its id in range
// (the shared expert: always), which both kernels read from the caller's arrays.
constexpr int MOE_DECODE_MAX_K = 32768; // int8 codes of a token / a middle row staged in LDS

struct MoeSlot { int expert; float coeff; bool live, bad; };
__device__ __forceinline__ MoeSlot moe_slot(const rkh_moe_decode_args& a, int t, int s) {
    if (s >= a.top_k) return {a.experts, 1.0f, true, false};
    const int id = a.ids[(size_t)t * a.top_k + s];
    const float c = a.routes[(size_t)t * a.top_k + s];
    const bool id_ok = (unsigned)id < (unsigned)a.experts;
    return {id, c, c != 0.0f && id_ok, !id_ok || not_finite(c) || c < 0.0f};
}

// One 1 KiB tile of a tiled expert image against the staged int8 row: a k-tile of int8 codes, or
// an int4 super-tile of two k-tiles, multiplied as 16 * code (the sum is shifted back at the end).
// `idx` counts tiles of the column block, `w` is the lane's 16 bytes of the tile.
__device__ __forceinline__ void moe_dot_tile(bool int4, const uint8_t* a_lds, int idx, int half, const v4i& w, int& acc) {
    if (!int4) {
        const v4i av = *reinterpret_cast<const v4i*>(a_lds + (size_t)(idx * 2 + half) * 16);
        acc = __builtin_amdgcn_sdot4(av.x, w.x, acc, false);
        acc = __builtin_amdgcn_sdot4(av.y, w.y, acc, false);
        acc = __builtin_amdgcn_sdot4(av.z, w.z, acc, false);
        acc = __builtin_amdgcn_sdot4(av.w, w.w, acc, false);
    } else {
        const v4i a0 = *reinterpret_cast<const v4i*>(a_lds + (size_t)(idx * 4 + half) * 16);
        const v4i a1 = *reinterpret_cast<const v4i*>(a_lds + (size_t)(idx * 4 + 2 + half) * 16);
        // a word holds eight codes: byte j = k + j (low nibble) and k + 4 + j (high nibble)
        acc = __builtin_amdgcn_sdot4(a0.x, (w.x << 4) & (int)0xF0F0F0F0, acc, false);
        acc = __builtin_amdgcn_sdot4(a0.y, w.x & (int)0xF0F0F0F0, acc, false);
        acc = __builtin_amdgcn_sdot4(a0.z, (w.y << 4) & (int)0xF0F0F0F0, acc, false);
        acc = __builtin_amdgcn_sdot4(a0.w, w.y & (int)0xF0F0F0F0, acc, false);
        acc = __builtin_amdgcn_sdot4(a1.x, (w.z << 4) & (int)0xF0F0F0F0, acc, false);
        acc = __builtin_amdgcn_sdot4(a1.y, w.z & (int)0xF0F0F0F0, acc, false);
        acc = __builtin_amdgcn_sdot4(a1.z, (w.w << 4) & (int)0xF0F0F0F0, acc, false);
        acc = __builtin_amdgcn_sdot4(a1.w, w.w & (int)0xF0F0F0F0, acc, false);
    }
}
__device__ __forceinline__ v4i moe_load_tile(const uint8_t* block, int idx, int tiles, int lane) {
    return idx < tiles ? __builtin_nontemporal_load(reinterpret_cast<const v4i*>(block + (size_t)idx * 1024 + lane * 16))
                       : v4i{0, 0, 0, 0};
}

constexpr int MOE_DECODE_PREFETCH = 4; // tiles per wave and column block requested ahead of the quantization

__global__ __launch_bounds__(512) void moe_decode_gate_kernel(rkh_moe_decode_args a) {
    __shared__ __attribute__((aligned(16))) uint8_t a_lds[MOE_DECODE_MAX_K];
    __shared__ int red[2][8][32];
    __shared__ float wave_max[8];
    __shared__ int wave_bad[8];
    const int slots = a.top_k + a.shared;
    const int j = blockIdx.x, asg = blockIdx.y, t = asg / slots, s = asg - t * slots;
    const int tid = threadIdx.x, lane = lane_id(), wave = wave_id(), half = lane >> 5;
    const MoeSlot slot = moe_slot(a, t, s);
    const bool reporter = j == 0 && tid == 0;
    if (slot.bad && reporter && a.bad_flag) atomicOr(a.bad_flag, 1);
    if (!slot.live) return;

    // ---- gate block 2j and up block 2j + 1 of the expert: the first tiles are requested now
    const int H = a.H, Hp = (int)rkh_align_up(H, RKH_K_ALIGN), nchunks = (H + 15) >> 4;
    const int e = slot.expert;
    const bool int4 = e < a.int4_experts;
    const int tiles = int4 ? Hp / 64 : Hp / 32; // per column block
    const size_t block_bytes = (size_t)tiles * 1024;
    const uint8_t* wb = (int4 ? a.gate_W4 + (size_t)e * a.gate_stride4
                              : a.gate_W + (size_t)(e - a.int4_experts) * a.gate_stride) + (size_t)(2 * j) * block_bytes;
    v4i pre[2][MOE_DECODE_PREFETCH];
#pragma unroll
    for (int u = 0; u < MOE_DECODE_PREFETCH; ++u)
#pragma unroll
        for (int b = 0; b < 2; ++b) pre[b][u] = moe_load_tile(wb + b * block_bytes, wave + 8 * u, tiles, lane);

    // ---- the token as int8 codes in LDS (s = max > 0 ? max / 127 : 1, ties to even)
    const float* row = a.x + (size_t)t * H;
    const bool vec = (reinterpret_cast<uintptr_t>(row) & 15) == 0;
    constexpr int CACHE = MOE_DECODE_MAX_K / 16 / 512; // chunks per thread
    float v[CACHE][16];
    float mx = 0.0f;
    bool bad = false;
#pragma unroll
    for (int i = 0; i < CACHE; ++i) {
        const int c = tid + i * 512;
        if (c < nchunks) {
            RowLoader<float>::load16(row, c * 16, H, vec, v[i]);
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                mx = fmaxf(mx, fabsf(v[i][q]));
                bad |= not_finite(v[i][q]);
            }
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    const unsigned long long bad_mask = __ballot(bad);
    if (lane == 0) {
        wave_max[wave] = mx;
        wave_bad[wave] = bad_mask != 0ull;
    }
    __syncthreads();
    mx = 0.0f;
    int any_bad = 0;
#pragma unroll
    for (int w = 0; w < 8; ++w) {
        mx = fmaxf(mx, wave_max[w]);
        any_bad |= wave_bad[w];
    }
    const float scale = mx > 0.0f ? mx / 127.0f : 1.0f;
    const float inv = 1.0f / scale;
    // (a non-finite token, or a maximum so small that the scale or its inverse leaves the fp32 range)
    if (reporter && a.bad_flag && (any_bad || !(scale > 0.0f) || not_finite(inv))) atomicOr(a.bad_flag, 1);
#pragma unroll
    for (int i = 0; i < CACHE; ++i) {
        const int c = tid + i * 512;
        if (c < nchunks) *reinterpret_cast<uint4*>(a_lds + (size_t)c * 16) = quantize16<true>(v[i], inv);
    }
    for (int c = nchunks + tid; c < Hp / 16; c += 512) *reinterpret_cast<uint4*>(a_lds + (size_t)c * 16) = make_uint4(0, 0, 0, 0);
    __syncthreads();

    // ---- dot products: the waves take the tiles of both blocks in turn
    int acc[2] = {0, 0};
#pragma unroll
    for (int u = 0; u < MOE_DECODE_PREFETCH; ++u)
#pragma unroll
        for (int b = 0; b < 2; ++b)
            if (wave + 8 * u < tiles) moe_dot_tile(int4, a_lds, wave + 8 * u, half, pre[b][u], acc[b]);
#pragma unroll 2
    for (int idx = wave + 8 * MOE_DECODE_PREFETCH; idx < tiles; idx += 8) {
        const v4i w0 = moe_load_tile(wb, idx, tiles, lane), w1 = moe_load_tile(wb + block_bytes, idx, tiles, lane);
        moe_dot_tile(int4, a_lds, idx, half, w0, acc[0]);
        moe_dot_tile(int4, a_lds, idx, half, w1, acc[1]);
    }
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        int p = acc[b];
        p += __shfl_xor(p, 32);
        if (lane < 32) red[b][wave][lane] = p;
    }
    __syncthreads();
    if (tid < 32) {
        int gate = 0, up = 0;
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            gate += red[0][w][tid];
            up += red[1][w][tid];
        }
        if (int4) {
            gate >>= 4;
            up >>= 4;
        }
        const int n = j * 32 + tid; // (I is a multiple of 32)
        // (fetched here, not with the first tiles: requested early the two scales made the kernel a
        // third slower for four and eight tokens)
        const float* ws = a.gate_scales + (size_t)e * 2 * a.I;
        const float gf = dequant(gate, scale, ws[n]);
        const float uf = dequant(up, scale, ws[a.I + n]);
        const float y = __fmul_rn(silu_poly(gf), uf);
        a.hidden[(size_t)asg * a.I + n] = y;
        uint32_t bits = __float_as_uint(y) & 0x7fffffffu;
#pragma unroll
        for (int d = 16; d > 0; d >>= 1) bits = max(bits, (uint32_t)__shfl_xor((int)bits, d));
        if (tid == 0) a.row_max_bits[(size_t)asg * (a.I / 32) + j] = bits;
    }
}

// One workgroup per (token, 32 output columns).  The live slots' middle rows are re-quantized side
// by side in LDS first (a wave per slot; row and partial maxima requested together), then the eight
// waves walk the slots' down blocks in one sequence of groups of tiles with the next group's loads
// always in flight -- also across the boundary between two slots, and the first group ahead of the
// re-quantization -- and the first 32 threads add the slots' dequantized values in slot order.
constexpr int MOE_DECODE_SLOTS = ROUTE_MAX_TOPK + 1;
constexpr int MOE_DECODE_DOWN_K = 3584; // longest middle row (padded): nine of them fit the staging area
static_assert(MOE_DECODE_SLOTS * MOE_DECODE_DOWN_K <= MOE_DECODE_MAX_K, "staging area");
__global__ __launch_bounds__(512) void moe_decode_down_kernel(rkh_moe_decode_args a) {
    __shared__ __attribute__((aligned(16))) uint8_t a_lds[MOE_DECODE_MAX_K]; // live slot i at i * Ip
    __shared__ int red[MOE_DECODE_SLOTS][8][32];
    __shared__ float live_scale[MOE_DECODE_SLOTS], live_coeff[MOE_DECODE_SLOTS];
    __shared__ int live_expert[MOE_DECODE_SLOTS], live_slot[MOE_DECODE_SLOTS];
    __shared__ int live_count;
    const int slots = a.top_k + a.shared;
    const int pb = blockIdx.x, t = blockIdx.y;
    const int tid = threadIdx.x, lane = lane_id(), wave = wave_id(), half = lane >> 5;
    const int I = a.I, Ip = (int)rkh_align_up(I, RKH_K_ALIGN), nchunks = I >> 4, parts = I / 32;
    if (tid == 0) { // the live slots in slot order
        int n = 0;
        for (int s = 0; s < slots; ++s) {
            const MoeSlot slot = moe_slot(a, t, s);
            if (slot.live) {
                live_expert[n] = slot.expert;
                live_coeff[n] = slot.coeff;
                live_slot[n] = s;
                ++n;
            }
        }
        live_count = n;
    }
    __syncthreads();
    const int nlive = live_count;
    // a slot's tiles are walked in groups of 8 waves x PF tiles
    constexpr int PF = MOE_DECODE_PREFETCH;
    auto block_of = [&](int li, bool& int4, int& tiles) -> const uint8_t* {
        const int e = live_expert[li];
        int4 = e < a.int4_experts;
        tiles = int4 ? Ip / 64 : Ip / 32;
        return (int4 ? a.down_W4 + (size_t)e * a.down_stride4
                     : a.down_W + (size_t)(e - a.int4_experts) * a.down_stride) + (size_t)pb * tiles * 1024;
    };
    auto load_group = [&](int li, int grp, v4i* regs) {
        bool int4;
        int tiles;
        const uint8_t* wb = block_of(li, int4, tiles);
#pragma unroll
        for (int u = 0; u < PF; ++u) regs[u] = moe_load_tile(wb, (grp * PF + u) * 8 + wave, tiles, lane);
    };
    v4i cur[PF], nxt[PF];
    if (nlive > 0) load_group(0, 0, cur);

    // ---- the middle rows (max != 0 ? max / 127 : 1, ties to even)
    for (int li = wave; li < nlive; li += 8) {
        const int asg = t * slots + live_slot[li];
        const float* hrow = a.hidden + (size_t)asg * I;
        constexpr int CACHE = (MOE_DECODE_DOWN_K / 16 + 63) / 64; // chunks per lane
        float v[CACHE][16];
#pragma unroll
        for (int i = 0; i < CACHE; ++i) {
            const int c = lane + 64 * i;
            if (c < nchunks) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 f = *reinterpret_cast<const float4*>(hrow + c * 16 + q * 4);
                    v[i][q * 4] = f.x; v[i][q * 4 + 1] = f.y; v[i][q * 4 + 2] = f.z; v[i][q * 4 + 3] = f.w;
                }
            }
        }
        uint32_t bits = 0;
        for (int i = lane; i < parts; i += 64) bits = max(bits, a.row_max_bits[(size_t)asg * parts + i]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) bits = max(bits, (uint32_t)__shfl_xor((int)bits, off));
        const float mx = __uint_as_float(bits);
        const float scale = mx != 0.0f ? mx / 127.0f : 1.0f;
        const float inv = 1.0f / scale;
        if (lane == 0) live_scale[li] = scale;
#pragma unroll
        for (int i = 0; i < CACHE; ++i) {
            const int c = lane + 64 * i;
            if (c < Ip / 16)
                *reinterpret_cast<uint4*>(a_lds + (size_t)li * Ip + (size_t)c * 16) =
                    c < nchunks ? quantize16<true>(v[i], inv) : make_uint4(0, 0, 0, 0);
        }
    }
    __syncthreads();

    // ---- the down blocks
    for (int li = 0; li < nlive; ++li) {
        bool int4;
        int tiles;
        block_of(li, int4, tiles);
        const int groups = (tiles + 8 * PF - 1) / (8 * PF);
        const uint8_t* codes = a_lds + (size_t)li * Ip;
        int acc = 0;
        for (int grp = 0; grp < groups; ++grp) {
            const bool last = grp + 1 == groups;
            if (!last) load_group(li, grp + 1, nxt);
            else if (li + 1 < nlive) load_group(li + 1, 0, nxt);
#pragma unroll
            for (int u = 0; u < PF; ++u) {
                const int idx = (grp * PF + u) * 8 + wave;
                if (idx < tiles) moe_dot_tile(int4, codes, idx, half, cur[u], acc);
            }
#pragma unroll
            for (int u = 0; u < PF; ++u) cur[u] = nxt[u];
        }
        acc += __shfl_xor(acc, 32);
        if (lane < 32) red[li][wave][lane] = acc;
    }
    __syncthreads();
    if (tid < 32) {
        const int n = pb * 32 + tid; // (H is a multiple of 32)
        float sum = 0.0f;
        for (int li = 0; li < nlive; ++li) {
            int acc = 0;
#pragma unroll
            for (int w = 0; w < 8; ++w) acc += red[li][w][tid];
            const int e = live_expert[li];
            if (e < a.int4_experts) acc >>= 4;
            const float y = dequant(acc, live_scale[li], a.down_scales[(size_t)e * a.H + n]);
            sum = fmaf(y, live_coeff[li], sum);
        }
        a.out[(size_t)t * a.H + n] = sum;
    }
}

// ------------------------------------------------------ measurement probes
// What the memory system and the matrix pipes give on the box the benchmark runs
// on, to put beside the datasheet peaks: a read-only stream over a footprint and
// a pure-MFMA loop with operands in registers.
//
// Read-only stream in the access order of the decode GEMV: every workgroup (eight waves)
// owns one contiguous span, its waves take the span's 1 KiB pieces in turn (16 bytes per
// lane), eight loads per wave in flight.  The xor of everything read is written only if it
// equals a value it is most unlikely to take, which keeps the loads alive.
__global__ __launch_bounds__(512) void stream_read_probe_kernel(const uint8_t* __restrict__ src, size_t span,
                                                                size_t bytes, uint32_t* sink) {
    const size_t begin = (size_t)blockIdx.x * span;
    const size_t end = begin + span < bytes ? begin + span : bytes;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t x = 0;
    for (size_t at = begin + (size_t)wave * 1024; at < end; at += 8 * 8 * 1024) {
        v4i got[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const size_t off = at + (size_t)u * 8 * 1024 + (size_t)lane * 16;
            got[u] = off + 16 <= end ? __builtin_nontemporal_load(reinterpret_cast<const v4i*>(src + off)) : v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) x ^= (uint32_t)(got[u].x ^ got[u].y ^ got[u].z ^ got[u].w);
    }
    if (x == 0x9e3779b9u && sink) atomicAdd(sink, 1u);
}

// Pure int8 MFMA: every wave keeps four independent 32x32 accumulators busy with
// v_mfma_i32_32x32x32_i8 on operands it loaded once (so their bit patterns -- and
// the switching activity in the multipliers, which sets the clock the chip
// sustains -- are those of the caller's data), `iterations` times.  Eight waves
// per workgroup, as in the GEMM kernels.  2 * 32 * 32 * 32 operations per MFMA.
__global__ __launch_bounds__(512) void mfma_i8_probe_kernel(const v4i* __restrict__ operands, int iterations,
                                                            int* sink) {
    const int t = threadIdx.x;
    v4i a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        a[i] = operands[(size_t)(2 * i) * 512 + t];
        b[i] = operands[(size_t)(2 * i + 1) * 512 + t];
    }
    v16i acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0;
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[j & 1], b[j >> 1], acc[j], 0, 0, 0);
    }
    int x = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) x ^= acc[j][r];
    if (x == 0x5bd1e995 && sink) atomicAdd(sink, 1);
}

// ------------------------------------------------- static device scratch
// Scratch memory for the entry point that allocates nothing: one array per
// device, held from the moment the code object is loaded until the process
// ends.  Host code never uses the array's name as an address: the per-device
// address is looked up once with hipGetSymbolAddress and kept.
constexpr size_t STATIC_SCRATCH_BYTES = size_t(12) << 20;
static __device__ __align__(256) uint8_t scratch[STATIC_SCRATCH_BYTES];

// ------------------------------------------------------------- launchers
// Workgroups of the 256-column grid below which the K-split variant is used.  Measured on a 32-expert
// top-4 layer (H 2048, I 1024): 1 / 2 tokens 32.9 -> 27.1 / 37.7 -> 35.7 us; from 4 tokens (16 possible
// row blocks) on the wide tile is faster again (41.4 vs 44.6 us).
// (Splitting K two ways over 128-column tiles for 4 .. 64 tokens was measured too: 1 - 3 us slower than
// the wide tile at every size.)
constexpr long GROUPED_KS4_BELOW = 96;
constexpr long GROUPED_BALANCED_UNITS_PER_CU = 4; // (row block, column pair) units per compute unit from which the balanced launch is used

// Compute units of the current device (0 if the query fails), looked up once per device.
int compute_units() {
    static int cached[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (!cached[dev]) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        cached[dev] = n;
    }
    return cached[dev];
}
// dense use of the same kernel: every row block is live.  (256 or 512 instead, int8, 128 rows, K = 4096:
// 11008 columns 25.6 -> 23.4 us, 14336 columns 27.3 -> 30.4 us.)
constexpr long DENSE_KS4_BELOW = 128;
// Grouped (MoE) launches: one workgroup per (32-row block of the sorted rows,
// 256-column tile); blocks beyond the live count exit at once.  When that grid
// would leave compute units idle (max_blocks is the caller's bound for this
// call, a handful for a decode step) the tile shrinks to 64 columns and the
// waves split K instead.
int launch_gemm_grouped(hipStream_t st, const rkh_gemm_args& g) {
    const bool grouped = g.blk_expert != nullptr;
    const bool any_int4 = grouped ? g.int4_experts > 0 : g.w_int4 != 0;
    const bool any_int8 = grouped ? g.W != nullptr : !g.w_int4;
    if (any_int4 && g.K > 131072) return RKH_ERR_RUNTIME; // (int4 codes ride as 16 * code in an int32 sum)
    if (grouped && any_int4 && !g.W4) return RKH_ERR_RUNTIME;
    const int mblocks = grouped ? g.max_blocks : (g.M + 31) / 32;
    const long wide = (long)mblocks * ((g.N + 255) / 256);
    const int ks = wide < (grouped ? GROUPED_KS4_BELOW : DENSE_KS4_BELOW) ? 4 : 1;
    const int cols = 256 / ks;
    const int nblocks = (g.N + cols - 1) / cols;
    // Many row blocks (a prefill-sized MoE call): the balanced launch, one workgroup per compute
    // unit.  With a workgroup per (row block, column tile) the 392 workgroups of a 256-token,
    // 32-expert, top-4 layer left 136 compute units with two of them and 120 with one, and a
    // compute unit draws at most 40 - 55 GB/s however many workgroups it holds: the launch
    // lasted as long as the compute units with two (down projection: last workgroup done after
    // 17.8 us, 15.4 balanced).  RK_NPU_HIP_GROUPED=balanced|tiles forces the choice (tuning aid).
    const int cus = compute_units();
    const bool moe_epilogue = g.epilogue == RKH_EPI_F32 || g.epilogue == RKH_EPI_SWIGLU;
    bool balanced = grouped && moe_epilogue && cus > 0 &&
                    (long)mblocks * ((g.N + 63) / 64) >= GROUPED_BALANCED_UNITS_PER_CU * (long)cus;
    static const char* forced = getenv("RK_NPU_HIP_GROUPED");
    if (forced && forced[0] == 'b') balanced = grouped && moe_epilogue && cus > 0;
    if (forced && forced[0] == 't') balanced = false;
    if (balanced) {
        mark(st, "gemm_stream_kernel<balanced>");
        const dim3 grid(cus), block(512);
#define RK_LAUNCH_BAL(EPI)                                                                                          \
    do {                                                                                                            \
        if (any_int4) hipLaunchKernelGGL((gemm_stream_kernel<EPI, 1, true, true>), grid, block, 0, st, RK_GEMM_HEAD(g), mblocks, nblocks, g);  \
        if (any_int8) hipLaunchKernelGGL((gemm_stream_kernel<EPI, 1, false, true>), grid, block, 0, st, RK_GEMM_HEAD(g), mblocks, nblocks, g); \
    } while (0)
        switch (g.epilogue) { // (grouped GEMMs are the MoE layer's: gate/up + SwiGLU and the fp32 down projection)
        case RKH_EPI_F32: RK_LAUNCH_BAL(RKH_EPI_F32); break;
        case RKH_EPI_SWIGLU: RK_LAUNCH_BAL(RKH_EPI_SWIGLU); break;
        default: return RKH_ERR_RUNTIME;
        }
#undef RK_LAUNCH_BAL
        RKH_CHECK(hipGetLastError());
        return RKH_OK;
    }
    const dim3 grid(mblocks * nblocks), block(256);
    mark(st, ks == 4 ? "gemm_stream_kernel<KS=4>" : "gemm_stream_kernel");
#define RK_LAUNCH(EPI)                                                                                         \
    do {                                                                                                       \
        if (any_int4 && ks == 4)                                                                               \
            hipLaunchKernelGGL((gemm_stream_kernel<EPI, 4, true>), grid, block, 0, st, RK_GEMM_HEAD(g), mblocks, nblocks, g);   \
        else if (any_int4)                                                                                     \
            hipLaunchKernelGGL((gemm_stream_kernel<EPI, 1, true>), grid, block, 0, st, RK_GEMM_HEAD(g), mblocks, nblocks, g);   \
        if (any_int8 && ks == 4)                                                                               \
            hipLaunchKernelGGL((gemm_stream_kernel<EPI, 4, false>), grid, block, 0, st, RK_GEMM_HEAD(g), mblocks, nblocks, g);  \
        else if (any_int8)                                                                                     \
            hipLaunchKernelGGL((gemm_stream_kernel<EPI, 1, false>), grid, block, 0, st, RK_GEMM_HEAD(g), mblocks, nblocks, g);  \
    } while (0)
    switch (g.epilogue) {
    case RKH_EPI_I32: RK_LAUNCH(RKH_EPI_I32); break;
    case RKH_EPI_F16: RK_LAUNCH(RKH_EPI_F16); break;
    case RKH_EPI_F32: RK_LAUNCH(RKH_EPI_F32); break;
    case RKH_EPI_SWIGLU: RK_LAUNCH(RKH_EPI_SWIGLU); break;
    default: return RKH_ERR_RUNTIME;
    }
#undef RK_LAUNCH
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}

// Bytes of split-K scratch for `tiles` output tiles of bm rows split into
// ksplit parts: the int32 partial tiles.
static size_t wk_scratch_bytes(long tiles, int bm, int ksplit) {
    return ksplit > 1 ? (size_t)tiles * ksplit * bm * 256 * 4 : 0;
}

template <int TM>
int launch_gemm_wk(hipStream_t st, const rkh_gemm_args& g, int ksplit) {
    constexpr int BM = 32 * TM, KTS = 8 / TM;
    const int mblocks = (g.M + BM - 1) / BM;
    const int nblocks = (g.N + 255) / 256;
    const int ksteps_total = (int)(rkh_align_up(g.K, RKH_K_ALIGN) / 32 / KTS);
    if (ksplit > ksteps_total) ksplit = ksteps_total;
    if (ksplit < 1) ksplit = 1;
    const int per = (ksteps_total + ksplit - 1) / ksplit;
    ksplit = (ksteps_total + per - 1) / per; // no empty part
    const dim3 grid(mblocks * nblocks * ksplit), block(512);
    mark(st, "gemm_wk_kernel");
#define RK_WK(W4, EPI)                                                                              \
    do {                                                                                            \
        /* the LDS opt-in is per function and per device: once for each device this process uses */ \
        /* (several threads may get here together: setting the attribute twice is harmless, and the  \
           flag is only set once a call has succeeded) */                                           \
        static std::atomic<bool> opted_in[64] = {};                                                 \
        int dev = 0;                                                                                \
        RKH_CHECK(hipGetDevice(&dev));                                                              \
        if (dev < 0 || dev >= 64) return RKH_ERR_RUNTIME;                                           \
        if (!opted_in[dev].load(std::memory_order_acquire)) {                                       \
            RKH_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_wk_kernel<TM, W4, EPI>), \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, WK_LDS_BYTES)); \
            opted_in[dev].store(true, std::memory_order_release);                                   \
        }                                                                                           \
        hipLaunchKernelGGL((gemm_wk_kernel<TM, W4, EPI>), grid, block, WK_LDS_BYTES, st,           \
                           g.A, g.W, g.M, g.K, mblocks, nblocks, ksplit, per, g);                   \
        if (ksplit > 1) mark(st, "gemm_wk_reduce_kernel");                                          \
        if (ksplit > 1)                                                                             \
            hipLaunchKernelGGL((gemm_wk_reduce_kernel<TM, W4, EPI>),                                \
                               dim3(mblocks * nblocks * (TM == 1 ? 4 : 8)), dim3(64), 0, st, g,     \
                               mblocks, nblocks, ksplit);                                           \
    } while (0)
    // (a dense SwiGLU GEMM exists for int4 weights only: the w4a8 FFN; the MoE layer's is grouped)
    switch (g.epilogue) {
    case RKH_EPI_I32: if (g.w_int4) RK_WK(true, RKH_EPI_I32); else RK_WK(false, RKH_EPI_I32); break;
    case RKH_EPI_F16: if (g.w_int4) RK_WK(true, RKH_EPI_F16); else RK_WK(false, RKH_EPI_F16); break;
    case RKH_EPI_F32: if (g.w_int4) RK_WK(true, RKH_EPI_F32); else RK_WK(false, RKH_EPI_F32); break;
    case RKH_EPI_SWIGLU: if (g.w_int4) RK_WK(true, RKH_EPI_SWIGLU); else return RKH_ERR_RUNTIME; break;
    default: return RKH_ERR_RUNTIME;
    }
#undef RK_WK
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}

template <int MR>
int launch_gemv(hipStream_t st, const rkh_gemm_args& g, const rkh_quant_args* fuse) {
    const int pblocks = (int)(rkh_align_up(g.N, 32) / 32);
    // Narrow matrices: several workgroups per column block (16 columns each up to 256 blocks =
    // 8192 columns, 8 columns each up to 64 blocks), so that a 4096-column projection has a
    // workgroup for every compute unit; all of them still run at once.  (Measured per shape on
    // one box, M = 1, int8 / int4 us: 4096 x 4096: 7.7 / 6.1 with 32 columns, 6.6 / 5.5 with 16,
    // 6.9 / 6.0 with 8; 14336 x 4096: 16.6 / 12.3, 14.5 / 10.5, 13.7 / 11.3; 8192 x 1024:
    // 10.6 / 8.1, 7.9 / 6.4, 6.4 / 5.7; a 14336-column matrix loses a quarter with 16.)
    // (RK_NPU_HIP_GEMV_COLS = 8 / 16 / 32 forces the choice: tuning aid)
    static const char* forced = getenv("RK_NPU_HIP_GEMV_COLS");
    const int want = forced ? atoi(forced) : 0;
    // Beyond 256 blocks: whole blocks -- unless the rows come as int8 (no quantization prologue that every
    // workgroup repeats) and halves leave the fullest compute unit with fewer columns: 344 blocks, an
    // 11008-column projection, 2 x 32 against 3 x 16 columns, one row 10.1 -> 9.3 us, four rows
    // 12.3 -> 10.9.  (448 blocks: 2 x 32 = 4 x 16, and whole blocks are a quarter faster.  With the
    // quantization fused, halves cost the same 344-block matrix 6 % to 18 % for 2 to 8 rows.)
    const int cus = compute_units() > 0 ? compute_units() : 256;
    const bool halves = fuse && fuse->in_dtype == RKH_I8 &&
                        ((2 * pblocks + cus - 1) / cus) * 16 < ((pblocks + cus - 1) / cus) * 32;
    const int cw = want == 8 || want == 16 || want == 32 ? want : pblocks <= 64 ? 8 : pblocks <= 256 || halves ? 16 : 32;
    const dim3 grid(pblocks * (32 / cw)), block(GEMV_WAVES * 64);
    const rkh_quant_args q = fuse ? *fuse : rkh_quant_args{};
    const int qt = !fuse ? 0 : fuse->in_dtype == RKH_F16 ? 1 : fuse->in_dtype == RKH_F32 ? 2 : 3;
    if (qt == 3 && g.w_int4) return RKH_ERR_RUNTIME; // (gemv_can_fuse lets int8 rows through for int8 weights only)
    // the instantiation that reads rows must have rows to read, the other one quantized rows
    if (qt ? !q.src : !g.A) return RKH_ERR_RUNTIME;
    if (!g.W || !g.C) return RKH_ERR_RUNTIME;
    const char* label = qt == 3 ? "gemv_kernel (int8 rows)" : qt ? "gemv_kernel (fused quantize)" : "gemv_kernel";
    if (MR == 1 && !g.w_int4 && cw == 32) { // (the burst variant, see gemv_kernel)
        mark(st, qt == 3 ? "gemv_kernel<burst> (int8 rows)" : qt ? "gemv_kernel<burst> (fused quantize)" : "gemv_kernel<burst>");
        if (qt == 0) hipLaunchKernelGGL((gemv_kernel<1, false, 0, 32, true>), grid, block, 0, st, RK_GEMV_HEAD(g, q), g, q);
        else if (qt == 1) hipLaunchKernelGGL((gemv_kernel<1, false, 1, 32, true>), grid, block, 0, st, RK_GEMV_HEAD(g, q), g, q);
        else if (qt == 2) hipLaunchKernelGGL((gemv_kernel<1, false, 2, 32, true>), grid, block, 0, st, RK_GEMV_HEAD(g, q), g, q);
        else hipLaunchKernelGGL((gemv_kernel<1, false, 3, 32, true>), grid, block, 0, st, RK_GEMV_HEAD(g, q), g, q);
        RKH_CHECK(hipGetLastError());
        return RKH_OK;
    }
    mark(st, label);
#define RK_GEMV(W4, QT)                                                                        \
    do {                                                                                       \
        if (cw == 8) hipLaunchKernelGGL((gemv_kernel<MR, W4, QT, 8>), grid, block, 0, st, RK_GEMV_HEAD(g, q), g, q);        \
        else if (cw == 16) hipLaunchKernelGGL((gemv_kernel<MR, W4, QT, 16>), grid, block, 0, st, RK_GEMV_HEAD(g, q), g, q); \
        else if constexpr (!(MR == 1 && !W4)) /* (one int8 row, 32 columns: the burst variant above) */   \
            hipLaunchKernelGGL((gemv_kernel<MR, W4, QT, 32>), grid, block, 0, st, RK_GEMV_HEAD(g, q), g, q);               \
    } while (0)
    if (g.w_int4) {
        if (qt == 0) RK_GEMV(true, 0); else if (qt == 1) RK_GEMV(true, 1); else RK_GEMV(true, 2);
    } else {
        if (qt == 0) RK_GEMV(false, 0); else if (qt == 1) RK_GEMV(false, 1); else if (qt == 2) RK_GEMV(false, 2);
        else RK_GEMV(false, 3);
    }
#undef RK_GEMV
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}

template <int MR>
int launch_gemv_swiglu(hipStream_t st, const rkh_gemm_args& g, const rkh_quant_args* fuse) {
    const dim3 grid(g.interleave_F / 32), block(GEMV_WAVES * 64);
    const rkh_quant_args q = fuse ? *fuse : rkh_quant_args{};
    const int qt = !fuse ? 0 : fuse->in_dtype == RKH_F16 ? 1 : 2;
    if (qt ? !q.src : !g.A) return RKH_ERR_RUNTIME; // (rows to read for the instantiation that is launched)
    if (!g.W || !g.C) return RKH_ERR_RUNTIME;
    mark(st, qt ? "gemv_swiglu_kernel (fused quantize)" : "gemv_swiglu_kernel");
#define RK_SWI(W4, QT) hipLaunchKernelGGL((gemv_swiglu_kernel<MR, W4, QT>), grid, block, 0, st, RK_GEMV_HEAD(g, q), g, q)
    // (dense SwiGLU exists for int4 weights only, with rows as fp32 or already quantized:
    // the w4a8 interface has no other call, and gemv_swiglu_applies lets nothing else through)
    if (!g.w_int4 || qt == 1) return RKH_ERR_RUNTIME;
    if (qt == 0) RK_SWI(true, 0); else RK_SWI(true, 2);
#undef RK_SWI
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}

// gate/up + SwiGLU of one or two rows as a GEMV (columns gate/up interleaved in blocks of 32,
// F a multiple of 32, both blocks of a workgroup within the 4 GiB reach of its descriptor).
// Measured for 4096 -> 2 x 14336 int4 against 14.9 us on the MFMA kernel: 12.8 us for one row,
// 13.8 for two, 15.1 for four, 20.1 for eight -- so from three rows on the MFMA kernel keeps it
// (also when the GEMV could quantize the rows itself and save that launch: a whole 4096 -> 14336
// -> 4096 FFN of three / four rows took 33.6 / 34.8 us that way against 34.6 / 34.5).
bool gemv_swiglu_applies(const rkh_gemm_args& g) {
    return !g.blk_expert && g.w_int4 && g.M <= 2 && g.epilogue == RKH_EPI_SWIGLU && g.interleave_F >= 32 &&
           g.interleave_F % 32 == 0 && g.N == 2 * g.interleave_F && g.K <= (1 << 24);
}

int dispatch_gemv_swiglu(hipStream_t st, const rkh_gemm_args& g, const rkh_quant_args* fuse) {
    if (g.M == 1) return launch_gemv_swiglu<1>(st, g, fuse);
    return launch_gemv_swiglu<2>(st, g, fuse);
}

int dispatch_gemv(hipStream_t st, const rkh_gemm_args& g, const rkh_quant_args* fuse) {
    if (g.M == 1) return launch_gemv<1>(st, g, fuse);
    if (g.M == 2) return launch_gemv<2>(st, g, fuse);
    if (g.M <= 4) return launch_gemv<4>(st, g, fuse);
    return launch_gemv<8>(st, g, fuse);
}

// The decode path can quantize inside the GEMV when the rows fit the kernel's
// LDS staging and per-thread register cache.
// Whether the streaming MFMA kernel can take this dense GEMM at all (int4 codes ride as 16 * code).
bool dense_stream_fits(const rkh_gemm_args& g) { return !g.w_int4 || g.K <= 131072; }

// Most rows the dot-product kernels take for this matrix: eight, but four on a matrix of more than
// 256 column blocks, where five to eight rows are faster as one 32-row block of the streaming MFMA
// kernel behind a quantization launch (fp16 rows, every step from HBM, dot products against
// stream, us: 4096 x 11008 int8 17.2 - 20.5 against 15.3 - 15.5, int4 15.5 - 18.9 against 12.3 - 12.5;
// 4096 x 14336 18.8 - 21.9 against 16.2 - 16.5, int4 16.1 - 19.3 against 12.8 - 12.9; on narrower
// matrices the dot products win: 4096 x 4096 9.5 - 11.6 against 13.6, 11008 x 4096 22.6 against 27.3;
// up to four rows they win everywhere).  RK_NPU_HIP_GEMV_MAX_ROWS = 1..8 lowers the limit (tuning aid).
int gemv_max_rows(const rkh_gemm_args& g) {
    static const int rows = [] {
        const char* e = getenv("RK_NPU_HIP_GEMV_MAX_ROWS");
        const int v = e ? atoi(e) : 8;
        return v >= 1 && v <= 8 ? v : 8;
    }();
    const bool wide = (g.N + 31) / 32 > 256;
    return wide && g.epilogue != RKH_EPI_SWIGLU && dense_stream_fits(g) ? min(rows, 4) : rows;
}

bool gemv_can_fuse(const rkh_quant_args& q, const rkh_gemm_args& g, bool swiglu = false) {
    if (g.w_int4 && !g.w_colsum) return false;
    if (g.blk_expert || g.M > gemv_max_rows(g) || (g.epilogue == RKH_EPI_SWIGLU) != swiglu || q.src_is_host) return false;
    // int8 rows as given (the exact int8 x int8 product): staged by the kernel in K chunks, any K
    if (q.in_dtype == RKH_I8) return q.mode == RKH_Q_COPY_I8 && !g.w_int4 && !swiglu;
    if (q.mode != RKH_Q_W8_DYNAMIC && q.mode != RKH_Q_W4A8) return false;
    if (q.in_dtype != RKH_F16 && q.in_dtype != RKH_F32) return false;
    const int mr = g.M == 1 ? 1 : g.M == 2 ? 2 : g.M <= 4 ? 4 : 8;
    const long kp = (long)rkh_align_up(g.K, RKH_K_ALIGN);
    if (kp * mr > GEMV_LDS_BYTES) return false;
    const long chunks = (long)g.M * ((g.K + 15) / 16);
    return chunks <= (long)GEMV_QCHUNKS * GEMV_WAVES * 64;
}

int g_fail_malloc_after = 0;

} // namespace

// =================================================================== C ABI
extern "C" {

int rkh_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int rkh_open(int device, void** stream_out, char* name_out, int name_len, int* cu_count,
             int* clock_khz) {
    RKH_CHECK(hipSetDevice(device));
    hipDeviceProp_t prop;
    RKH_CHECK(hipGetDeviceProperties(&prop, device));
    if (name_out && name_len > 0) {
        int i = 0;
        for (; i < name_len - 1 && prop.gcnArchName[i]; ++i) name_out[i] = prop.gcnArchName[i];
        name_out[i] = 0;
    }
    if (cu_count) *cu_count = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    hipStream_t st;
    RKH_CHECK(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    *stream_out = st;
    return RKH_OK;
}

void rkh_close(int device, void* stream) {
    if (hipSetDevice(device) != hipSuccess) return;
    if (stream) {
        (void)hipStreamSynchronize((hipStream_t)stream);
        (void)hipStreamDestroy((hipStream_t)stream);
    }
}

void rkh_fail_malloc_after(int n) { g_fail_malloc_after = n; }

#ifdef RK_DEBUG_TS
int rkh_debug_set_ts(void* device_buffer) {
    unsigned long long* p = static_cast<unsigned long long*>(device_buffer);
    RKH_CHECK(hipMemcpyToSymbol(HIP_SYMBOL(rk_dbg_ts), &p, sizeof(p)));
    return RKH_OK;
}
#endif

void rkh_set_marker(rkh_marker_fn fn, void* user) {
    std::unique_lock<std::shared_mutex> lock(g_marker_mutex);
    g_marker = fn;
    g_marker_user = fn ? user : nullptr;
    g_marker_on.store(fn != nullptr, std::memory_order_release);
}

int rkh_malloc(int device, void** ptr, size_t bytes) {
    *ptr = nullptr;
    if (g_fail_malloc_after > 0 && --g_fail_malloc_after == 0) return RKH_ERR_NOMEM;
    RKH_CHECK(hipSetDevice(device));
    if (bytes == 0) bytes = 16;
    RKH_CHECK(hipMalloc(ptr, bytes));
    return RKH_OK;
}

void rkh_free(int device, void* ptr) {
    if (!ptr) return;
    if (hipSetDevice(device) != hipSuccess) return;
    (void)hipFree(ptr);
}

int rkh_host_alloc(void** ptr, size_t bytes) {
    *ptr = nullptr;
    RKH_CHECK(hipHostMalloc(ptr, bytes ? bytes : 16, hipHostMallocDefault));
    return RKH_OK;
}
void rkh_host_free(void* ptr) {
    if (ptr) (void)hipHostFree(ptr);
}

int rkh_h2d(void* stream, void* dst, const void* src, size_t bytes) {
    if (!bytes) return RKH_OK;
    RKH_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
    return RKH_OK;
}
int rkh_d2h(void* stream, void* dst, const void* src, size_t bytes) {
    if (!bytes) return RKH_OK;
    RKH_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
    return RKH_OK;
}
int rkh_d2d(void* stream, void* dst, const void* src, size_t bytes) {
    if (!bytes) return RKH_OK;
    RKH_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
    return RKH_OK;
}
int rkh_fill32(void* stream, void* dst, uint32_t value, size_t words) {
    if (!words) return RKH_OK;
    mark((hipStream_t)stream, "fill32_kernel");
    const int blocks = (int)((words + 255) / 256 < 4096 ? (words + 255) / 256 : 4096);
    hipLaunchKernelGGL(fill32_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                       static_cast<uint32_t*>(dst), value, words);
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}
int rkh_exchange32(void* stream, void* x, void* y, size_t words) {
    if (!words) return RKH_OK;
    const int blocks = (int)((words + 255) / 256 < 4096 ? (words + 255) / 256 : 4096);
    hipLaunchKernelGGL(exchange32_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                       static_cast<uint32_t*>(x), static_cast<uint32_t*>(y), words);
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}
int rkh_sync(void* stream) {
    RKH_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return RKH_OK;
}

int rkh_event_create(void** event) {
    hipEvent_t e;
    RKH_CHECK(hipEventCreate(&e));
    *event = e;
    return RKH_OK;
}
void rkh_event_destroy(void* event) {
    if (event) (void)hipEventDestroy((hipEvent_t)event);
}
int rkh_event_record(void* event, void* stream) {
    RKH_CHECK(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
    return RKH_OK;
}
int rkh_event_sync(void* event) {
    RKH_CHECK(hipEventSynchronize((hipEvent_t)event));
    return RKH_OK;
}
int rkh_event_elapsed_us(void* start, void* stop, double* us) {
    RKH_CHECK(hipEventSynchronize((hipEvent_t)stop));
    float ms = 0.0f;
    RKH_CHECK(hipEventElapsedTime(&ms, (hipEvent_t)start, (hipEvent_t)stop));
    *us = (double)ms * 1000.0;
    return RKH_OK;
}

int rkh_pack_w8(void* stream, const int8_t* src, int K, int N, int interleave_F, uint8_t* dst) {
    const int KB = (int)(rkh_align_up(K, RKH_K_ALIGN) / 32);
    const size_t pblocks = (size_t)(rkh_align_up(N, RKH_COL_ALIGN) / 32);
    const size_t chunks = pblocks * KB * 64;
    hipLaunchKernelGGL(pack_w8_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, src, K, N, KB, interleave_F, dst, chunks);
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}

int rkh_pack_w4(void* stream, const int8_t* src, int K, int N, int interleave_F, uint8_t* dst,
                int* bad_flag, int32_t* colsum) {
    const int KB2 = (int)(rkh_align_up(K, RKH_K_ALIGN) / 64);
    const size_t pblocks = (size_t)(rkh_align_up(N, RKH_COL_ALIGN) / 32);
    const size_t chunks = pblocks * KB2 * 64;
    hipLaunchKernelGGL(pack_w4_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, src, K, N, KB2, interleave_F, dst, chunks, bad_flag, colsum);
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}

int rkh_quant_rows(void* stream, const rkh_quant_args* args) {
    if (args->M <= 0) return RKH_OK;
    const dim3 block(256);
    const int mode = args->mode;
    if (args->M >= 256 && !args->active_blocks && args->in_dtype != RKH_I8 &&
        (mode == RKH_Q_W8_DYNAMIC || mode == RKH_Q_W4A8 || mode == RKH_Q_W8_STATIC)) {
        const bool rows4 = args->M < 8 * 2 * 256; // 8 rows would give fewer than two workgroups per compute unit
        const dim3 grid(rows4 ? (args->M + 3) / 4 : (args->M + 7) / 8);
        const hipStream_t st = (hipStream_t)stream;
        mark(st, "quant_rows8_kernel");
        if (args->in_dtype == RKH_F16) {
            if (rows4) hipLaunchKernelGGL((quant_rows8_kernel<uint16_t, 4>), grid, block, 0, st, RK_QUANT_HEAD(*args), *args);
            else hipLaunchKernelGGL((quant_rows8_kernel<uint16_t, 8>), grid, block, 0, st, RK_QUANT_HEAD(*args), *args);
        } else {
            if (rows4) hipLaunchKernelGGL((quant_rows8_kernel<float, 4>), grid, block, 0, st, RK_QUANT_HEAD(*args), *args);
            else hipLaunchKernelGGL((quant_rows8_kernel<float, 8>), grid, block, 0, st, RK_QUANT_HEAD(*args), *args);
        }
        RKH_CHECK(hipGetLastError());
        return RKH_OK;
    }
    const bool reuse = mode == RKH_Q_REUSE_BITS || mode == RKH_Q_REUSE_BITS_MOE;
    if (reuse && args->in_dtype == RKH_F32 && args->M >= 64 && (args->K + 15) / 16 <= 64 * QR_CACHE) {
        mark((hipStream_t)stream, "requant_rows_wave_kernel");
        hipLaunchKernelGGL(requant_rows_wave_kernel, dim3((args->M + 3) / 4), block, 0, (hipStream_t)stream,
                           RK_QUANT_HEAD(*args), *args);
        RKH_CHECK(hipGetLastError());
        return RKH_OK;
    }
    // Re-quantization of a few long rows: several workgroups per row, about 256 chunks
    // each, until the grid has a few hundred workgroups.
    int split = 1;
    if (reuse) {
        const int row_chunks = (args->K + 15) / 16;
        while (split < 8 && args->M * split < 512 && row_chunks / (split * 2) >= 128) split *= 2;
    }
    const dim3 grid(args->M * split);
    mark((hipStream_t)stream, "quant_rows_kernel");
    switch (args->in_dtype) {
    case RKH_F16: hipLaunchKernelGGL(quant_rows_kernel<uint16_t>, grid, block, 0, (hipStream_t)stream, RK_QUANT_HEAD(*args), split, *args); break;
    case RKH_F32: hipLaunchKernelGGL(quant_rows_kernel<float>, grid, block, 0, (hipStream_t)stream, RK_QUANT_HEAD(*args), split, *args); break;
    case RKH_I8: hipLaunchKernelGGL(quant_rows_kernel<int8_t>, grid, block, 0, (hipStream_t)stream, RK_QUANT_HEAD(*args), split, *args); break;
    default: return RKH_ERR_RUNTIME;
    }
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}

// Dense launch plan: rows per workgroup follow M, shrinking while the output
// grid cannot fill the 256 compute units; what is still missing is made up by
// splitting K over workgroups (exact: integer partial tiles are added by the
// last part to arrive).  int4 operands ride as 16 * code, so one K part may
// span at most 2^17 k before the int32 sum could wrap.
struct DensePlan { int bm, ksplit; };
static int min_ksplit(int K, int w_int4) {
    return w_int4 ? (int)((rkh_align_up(K, RKH_K_ALIGN) + 131071) / 131072) : 1;
}
static long dense_tiles(int M, int N, int bm) { return (long)((M + bm - 1) / bm) * ((N + 255) / 256); }
// Tile rows (128 / 64 / 32) and K split of a dense launch of the large-tile kernel: the candidate
// with the smallest estimated time.  The estimate is linear in what a workgroup pulls through its
// compute unit (K / split x (tile rows + 256 weight columns) bytes -- a compute unit moves about
// 100 GB/s from L2, which is what bounds tiles this small) or its MFMA count, the rounds the grid takes
// on the device, and, for a split, the second launch and the int32 partial tiles written and read
// back; the coefficients are a least-squares fit to measured times (int8, fp16 in / out, 4096 x 4096,
// 4096 x 11008, 11008 x 4096, 4096 x 14336 at 192 to 1024 rows, nine forced plans each: the fit
// picks the fastest or second-fastest plan for all of them).  Against the earlier rule (shrink
// the tile until 160 tiles exist, then split): K = 11008, N = 4096 at 192 / 256 / 512 / 1024 rows
// 50.0 -> 33.5, 53.9 -> 44.9, 71.7 -> 55.0, 82.6 -> 78.4 us; 4096 x 11008 at 192 rows 36.6 -> 31.0.
static DensePlan dense_plan(int M, int N, int K, int w_int4) {
    const int kp = (int)rkh_align_up(K, RKH_K_ALIGN);
    const int need = min_ksplit(K, w_int4);
    constexpr int cus = 256; // (a constant: the plan also sizes the workspace's scratch, before any launch)
    const int max_bm = M > 64 ? 128 : M > 32 ? 64 : 32;
    DensePlan best{max_bm, need};
    double best_cost = 1e30;
    for (int bm = max_bm; bm >= 32; bm >>= 1) {
        const long tiles = dense_tiles(M, N, bm);
        for (int ks = need; ks <= (need > 16 ? need : 16); ks *= 2) {
            if (ks != need && kp / ks < 1024) break; // at least 1024 k per part
            const double kpart = (double)kp / ks;
            const double rounds = (double)((tiles * ks + cus - 1) / cus);
            const double mem_kb = kpart * (bm + (w_int4 ? 128 : 256)) / 1e3;
            const double kmfma = (bm / 32) * 8 * (kpart / 32) / 1e3;
            const double part_mb = ks > 1 ? (double)tiles * ks * bm * 256 * 4 / 1e6 : 0.0;
            if (ks != need && part_mb > 512.0) break; // (scratch the workspace would have to hold)
            // (4.4 us per 1000 MFMAs of a workgroup: 250 per SIMD, 32 cycles each, at the 1.8 GHz the matrix
            // pipes sustain -- the bound of the 128-row tile with int4 weights, whose bytes are few)
            const double loop_us = 0.0156 * mem_kb > 4.4 * kmfma ? 0.0156 * mem_kb : 4.4 * kmfma;
            const double cost = rounds * (loop_us + 0.54) + (ks > 1 ? 2.9 + 0.41 * part_mb : 0.0);
            if (cost < best_cost) {
                best_cost = cost;
                best = {bm, ks};
            }
        }
    }
    return best;
}
// RK_NPU_HIP_GEMM_PLAN="rows:ksplit" forces the workgroup tile rows (32 / 64 /
// 128) and the K split of dense launches (tuning aid).
static DensePlan effective_plan(int M, int N, int K, int w_int4) {
    DensePlan plan = dense_plan(M, N, K, w_int4);
    static const char* forced = getenv("RK_NPU_HIP_GEMM_PLAN");
    if (forced) {
        int rows = 0, split = 0;
        if (sscanf(forced, "%d:%d", &rows, &split) == 2 && (rows == 32 || rows == 64 || rows == 128) && split >= 1) {
            plan.bm = rows;
            plan.ksplit = split > min_ksplit(K, w_int4) ? split : min_ksplit(K, w_int4);
        }
    }
    return plan;
}

// A dense GEMM of up to four row blocks is a weight stream like a MoE expert's:
// it runs on the grouped kernel (one "expert"; for few column tiles K is split
// over the waves of a workgroup and summed through LDS) instead of splitting K
// over workgroups and finishing in a second launch.  Measured against the
// large-tile kernel, fp16 in / out, quantization included (us):
//   int8  M 64, 2048 x 2048: 10.2 vs 15.3   M 128, 4096 x 4096: 12.6 vs 20.2   M 128, K 14336, N 4096: 25.5 vs 28.9
//         M 128, K 4096, N 14336: 20.9 vs 20.9
//   int4  M 64, 2048 x 2048:  9.9 vs 14.1   M 128, 4096 x 4096: 11.9 vs 19.4   M 128, K 14336, N 4096: 22.2 vs 25.7
//         M 32, K 4096, N 14336: 11.4 vs 18.4
// From about 160 rows on the large tile wins for wide N (each row block streams
// the weights again).  The same holds earlier for the gate/up + SwiGLU GEMM of
// an FFN, whose N is twice as wide: the whole FFN (4096 -> 14336 -> 4096, weights
// from HBM) takes 47.4 vs 53.9 us at 16 rows, 49.4 vs 47.0 at 64, 63.0 vs 56.3 at 128.
constexpr int DENSE_STREAM_MAX_M = 128, DENSE_STREAM_SWIGLU_MAX_M = 32;
static bool dense_streams(const rkh_gemm_args& g) {
    static const char* forced = getenv("RK_NPU_HIP_STREAM_MAX_ROWS"); // (tuning aid)
    const int max_rows = forced ? atoi(forced) : DENSE_STREAM_MAX_M;
    if (g.blk_expert || g.M <= gemv_max_rows(g) || g.M > max_rows) return false;
    if (g.epilogue == RKH_EPI_SWIGLU) return g.w_int4 && g.K <= 131072 && g.M <= DENSE_STREAM_SWIGLU_MAX_M;
    return !g.w_int4 || g.K <= 131072;
}

size_t rkh_gemm_scratch_bytes(int M, int N, int K, int w_int4) {
    if (M <= 8) return 0;
    const DensePlan plan = effective_plan(M, N, K, w_int4);
    return wk_scratch_bytes(dense_tiles(M, N, plan.bm), plan.bm, plan.ksplit);
}

int rkh_gemm(void* stream, const rkh_gemm_args* args) {
    const rkh_gemm_args& g = *args;
    hipStream_t st = (hipStream_t)stream;
    const bool grouped = g.blk_expert != nullptr;
    const bool gemv_ok = !g.w_int4 || g.w_colsum; // (the int4 GEMV kernels need the column sums)
    if (!grouped && g.M <= gemv_max_rows(g) && g.epilogue != RKH_EPI_SWIGLU && gemv_ok) return dispatch_gemv(st, g, nullptr);
    if (gemv_swiglu_applies(g) && gemv_ok) return dispatch_gemv_swiglu(st, g, nullptr);
    if (grouped) return launch_gemm_grouped(st, g);
    if (dense_streams(g)) return launch_gemm_grouped(st, g);
    const DensePlan plan = effective_plan(g.M, g.N, g.K, g.w_int4);
    int ksplit = plan.ksplit;
    if (ksplit > 1 && !g.splitk_acc) {
        if (min_ksplit(g.K, g.w_int4) > 1) return RKH_ERR_RUNTIME;
        ksplit = 1;
    }
    if (plan.bm == 128) return launch_gemm_wk<4>(st, g, ksplit);
    if (plan.bm == 64) return launch_gemm_wk<2>(st, g, ksplit);
    return launch_gemm_wk<1>(st, g, ksplit);
}

int rkh_quant_gemm(void* stream, const rkh_quant_args* qargs, const rkh_gemm_args* gargs) {
    if (gemv_can_fuse(*qargs, *gargs)) return dispatch_gemv((hipStream_t)stream, *gargs, qargs);
    if (gemv_swiglu_applies(*gargs) && gemv_can_fuse(*qargs, *gargs, true))
        return dispatch_gemv_swiglu((hipStream_t)stream, *gargs, qargs);
    if (qargs->mode == RKH_Q_REUSE_BITS) {
        // A decode-sized re-quantization (the down projection of an FFN with a few rows) is
        // folded into the GEMV as well: the kernel scans its rows itself instead of reading the
        // partial maxima the SwiGLU epilogue left.  Same result -- the maximum of the partial
        // maxima IS the row maximum, the scale rule and the rejection of non-finite rows are
        // those of RKH_Q_W4A8 -- and one launch less.
        rkh_quant_args scan = *qargs;
        scan.mode = RKH_Q_W4A8;
        scan.row_max_bits = nullptr;
        scan.row_max_parts = 0;
        if (gemv_can_fuse(scan, *gargs)) return dispatch_gemv((hipStream_t)stream, *gargs, &scan);
    }
    // (int8 rows of 9..128-row calls: letting the streaming kernel read them from their row-major source
    // instead of a tiled copy saves the re-tiling launch but was slower -- a lane's 16 bytes then come from
    // 32 different cache lines per load: 128 x 4096 x 11008 26.8 -> 35.7 us, 128 x 11008 x 4096 25.3 -> 29.7.)
    const int rc = rkh_quant_rows(stream, qargs);
    return rc ? rc : rkh_gemm(stream, gargs);
}

int rkh_moe_scatter(void* stream, const rkh_moe_scatter_args* args) {
    if (args->rows <= 0) return RKH_OK;
    if (args->experts + args->shared > ROUTE_MAX_EXPERTS || args->top_k > ROUTE_MAX_TOPK ||
        (long)args->rows * args->top_k > ROUTE_MAX_ASSIGNMENTS)
        return RKH_ERR_RUNTIME;
    const dim3 grid(args->rows), block(256);
    mark((hipStream_t)stream, "moe_scatter_kernel");
    if (args->in_dtype == RKH_F32)
        hipLaunchKernelGGL(moe_scatter_kernel<float>, grid, block, 0, (hipStream_t)stream, RK_SCATTER_HEAD(*args), *args);
    else if (args->in_dtype == RKH_I8)
        hipLaunchKernelGGL(moe_scatter_kernel<int8_t>, grid, block, 0, (hipStream_t)stream, RK_SCATTER_HEAD(*args), *args);
    else
        return RKH_ERR_RUNTIME;
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}

int rkh_moe_combine(void* stream, const rkh_moe_combine_args* args) {
    const dim3 grid((args->H / 4 + 255) / 256, args->rows);
    mark((hipStream_t)stream, "moe_combine_kernel");
    hipLaunchKernelGGL(moe_combine_kernel, grid, dim3(256), 0, (hipStream_t)stream, args->Y, args->dest_rows,
                       args->routes, args->out, args->rows, args->top_k, args->shared, args->H);
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}

int rkh_moe_decode_applies(int rows, int H, int I) {
    static const char* forced = getenv("RK_NPU_HIP_MOE_DECODE_ROWS"); // (tuning aid: 0 switches the path off)
    const int max_rows = forced ? atoi(forced) : 8;
    return rows >= 1 && rows <= max_rows && H >= 32 && H % 32 == 0 && H <= MOE_DECODE_MAX_K && I >= 32 && I % 32 == 0 &&
           rkh_align_up(I, RKH_K_ALIGN) <= (size_t)MOE_DECODE_DOWN_K; // (nine middle rows side by side in LDS)
}

int rkh_moe_decode(void* stream, const rkh_moe_decode_args* args) {
    const rkh_moe_decode_args& a = *args;
    if (!rkh_moe_decode_applies(a.rows, a.H, a.I) || a.top_k < 1) return RKH_ERR_RUNTIME;
    const int slots = a.top_k + (a.shared ? 1 : 0);
    mark((hipStream_t)stream, "moe_decode_gate_kernel");
    hipLaunchKernelGGL(moe_decode_gate_kernel, dim3(a.I / 32, a.rows * slots), dim3(512), 0, (hipStream_t)stream, a);
    mark((hipStream_t)stream, "moe_decode_down_kernel");
    hipLaunchKernelGGL(moe_decode_down_kernel, dim3(a.H / 32, a.rows), dim3(512), 0, (hipStream_t)stream, a);
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}

int rkh_probe_stream_read(void* stream, const void* src, size_t bytes, size_t span, void* sink) {
    if (!src || bytes < 16 || span < 1024 || span % 1024) return RKH_ERR_RUNTIME;
    const size_t workgroups = (bytes + span - 1) / span;
    if (workgroups > 0x7fffffffu) return RKH_ERR_RUNTIME;
    hipLaunchKernelGGL(stream_read_probe_kernel, dim3((unsigned)workgroups), dim3(512), 0, (hipStream_t)stream,
                       static_cast<const uint8_t*>(src), span, bytes, static_cast<uint32_t*>(sink));
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}

int rkh_probe_mfma_i8(void* stream, const void* operands, int workgroups, int iterations, void* sink) {
    if (!operands || workgroups < 1 || iterations < 1) return RKH_ERR_RUNTIME;
    hipLaunchKernelGGL(mfma_i8_probe_kernel, dim3(workgroups), dim3(512), 0, (hipStream_t)stream,
                       static_cast<const v4i*>(operands), iterations, static_cast<int*>(sink));
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}

// ---- stream capture: a sequence of launches recorded once and replayed ----
int rkh_capture_begin(void* stream) {
    RKH_CHECK(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
    return RKH_OK;
}
int rkh_capture_end(void* stream, void** graph_exec) {
    *graph_exec = nullptr;
    hipGraph_t graph = nullptr;
    RKH_CHECK(hipStreamEndCapture((hipStream_t)stream, &graph));
    hipGraphExec_t exec = nullptr;
    const hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return e == hipErrorOutOfMemory ? RKH_ERR_NOMEM : RKH_ERR_RUNTIME;
    *graph_exec = exec;
    return RKH_OK;
}
int rkh_graph_launch(void* graph_exec, void* stream) {
    RKH_CHECK(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream));
    return RKH_OK;
}
void rkh_graph_destroy(void* graph_exec) {
    if (graph_exec) (void)hipGraphExecDestroy((hipGraphExec_t)graph_exec);
}

// ---- the static scratch array of `device` ----
int rkh_static_scratch(int device, void** ptr, size_t* bytes) {
    static void* address[64] = {};
    static std::mutex guard;
    *ptr = nullptr;
    *bytes = 0;
    if (device < 0 || device >= 64) return RKH_ERR_RUNTIME;
    std::lock_guard<std::mutex> lock(guard);
    if (!address[device]) {
        RKH_CHECK(hipSetDevice(device));
        void* p = nullptr;
        RKH_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return RKH_ERR_RUNTIME;
        address[device] = p;
    }
    *ptr = address[device];
    *bytes = STATIC_SCRATCH_BYTES;
    return RKH_OK;
}

} // extern "C"
