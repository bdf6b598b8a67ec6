// The 32 x 32 accumulator tile of v_mfma_i32_32x32x32_i8 as the MFMA kernels hold it, and the
// epilogues that turn it into output: shared by rk_kernels_gemm.hip and rk_kernels_stream.hip.
#ifndef RK_KERNELS_TILE_H
#define RK_KERNELS_TILE_H

#include "rk_kernels_common.h"

namespace {

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

} // namespace

#endif // RK_KERNELS_TILE_H
