// C-ABI wrappers around the reference's own CPU translation units, compiled in
// place from the reference checkout into oracle/_ref/libref_cpu.so (see the
// Makefile).  TEST INFRASTRUCTURE ONLY: it exists to cross-check the CPU oracle
// (rk_oracle.c) against what the reference actually computes, in the build
// container where the checkout is present.  Nothing here is shipped, and no
// reference source is copied: this file only calls into it.
//
// The reference has no CPU GEMM (its NPU does the integer products), so the
// wrappers cover what surrounds it: scales, quantization, native-layout
// de-tiling + dequantization, row-scale reuse, the MoE middle, and the INT16
// partial-sum certificate that resolves k_tile.
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <vector>

#include "rk_npu_cpu_kernels.h"
#include "rk_npu_i4_bounds.h"
#include "rk_npu_moe_cpu.h"
#include "rk_npu_w4a8_cpu.h"

using namespace rknpu2_matmul_open;

extern "C" {

void ref_w8_scales_f16(int M, int K, const uint16_t* A, float* scale) {
    cpu::i8_compute_dynamic_per_token_scale_f16(M, K, A, K, scale);
}
void ref_w8_scales_f32(int M, int K, const float* A, float* scale) {
    cpu::i8_compute_dynamic_per_token_scale_f32(M, K, A, K, scale);
}

// Quantize with given per-token scales into the reference's "normal" A layout
// [M, align32(K)], then compact to [M, K].
void ref_w8_quant_f16(int M, int K, const uint16_t* A, const float* scale, int8_t* q) {
    const int ak = (K + 31) / 32 * 32;
    std::vector<int8_t> packed((size_t)M * ak, 0);
    cpu::i8_pack_a_f16_quant_normal_strided(M, K, ak, A, K, scale, packed.data());
    for (int m = 0; m < M; ++m) std::memcpy(q + (size_t)m * K, packed.data() + (size_t)m * ak, (size_t)K);
}
void ref_w8_quant_f32(int M, int K, const float* A, const float* scale, int8_t* q) {
    const int ak = (K + 31) / 32 * 32;
    std::vector<int8_t> packed((size_t)M * ak, 0);
    cpu::i8_pack_a_f32_quant_normal_strided(M, K, ak, A, K, scale, packed.data());
    for (int m = 0; m < M; ++m) std::memcpy(q + (size_t)m * K, packed.data() + (size_t)m * ak, (size_t)K);
}

// Row-major int32 accumulators -> the reference's native C layout
// (ceil(N/4), M, 4) -> its fused de-tile + dequant (+ fp16 cast).
static std::vector<int32_t> to_native_c(int M, int N, const int32_t* acc) {
    const int nb = (N + 3) / 4;
    std::vector<int32_t> native((size_t)nb * M * 4, 0);
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n)
            native[cpu::i8_c_block_offset(M, N, m, n / 4, 0) + n % 4] = acc[(size_t)m * N + n];
    return native;
}
void ref_w8_dequant_f16(int M, int N, const int32_t* acc, const float* a_scale,
                        const float* w_scale, uint16_t* out) {
    const auto native = to_native_c(M, N, acc);
    const int32_t* parts[1] = {native.data()};
    cpu::i8_reduce_c_native_i32_dequant_f16(M, N, 1, parts, a_scale, w_scale, nullptr,
                                            cpu::ActivationOp::None, out);
}
void ref_w8_dequant_f32(int M, int N, const int32_t* acc, const float* a_scale,
                        const float* w_scale, float* out) {
    const auto native = to_native_c(M, N, acc);
    const int32_t* parts[1] = {native.data()};
    cpu::i8_reduce_c_native_i32_dequant_f32(M, N, 1, parts, a_scale, w_scale, nullptr,
                                            cpu::ActivationOp::None, out);
}
// Split-K: two native partials summed modulo 2^32, then de-tiled.
void ref_w8_reduce_two_i32(int M, int N, const int32_t* acc0, const int32_t* acc1, int32_t* out) {
    const auto n0 = to_native_c(M, N, acc0), n1 = to_native_c(M, N, acc1);
    const int32_t* parts[2] = {n0.data(), n1.data()};
    cpu::i8_reduce_c_native_i32_to_rowmajor(M, N, 2, parts, out);
}

int ref_w4a8_scales(const void* A, int half, int M, int K, float* scales, float* inverse) {
    return detail::w4a8_scales(A, half != 0, M, K, 1, scales, inverse);
}

// Quantize through the reference's INT4 high/low row packer and reassemble the
// INT8 code q = 16*h + l + 8 from the native K32 layout.
int ref_w4a8_quant(const void* A, int half, int M, int K, const float* scales,
                   const float* inverse, int8_t* q) {
    detail::W4A8Input input{A, half != 0, M, K, scales, inverse, 1, detail::I4InputLayout::Native};
    auto nibble = [](const uint8_t* p, size_t i) {
        const int x = (p[i / 2] >> ((i & 1) ? 0 : 4)) & 15;
        return x >= 8 ? x - 16 : x;
    };
    for (int m0 = 0; m0 < M; m0 += 64) {
        const int tokens = std::min(64, M - m0), rows = tokens * 2;
        for (int k0 = 0; k0 < K; k0 += 2048) {
            const int k = std::min(2048, K - k0), pk = (k + 31) / 32 * 32;
            std::vector<uint8_t> packed((size_t)rows * pk / 2, 0);
            rk_npu_i4_input_tile t{m0 * 2, rows, k0, k, pk, packed.data(), (uint64_t)packed.size()};
            const int rc = detail::w4a8_pack(&input, &t);
            if (rc) return rc;
            for (int m = 0; m < tokens; ++m)
                for (int j = 0; j < k; ++j) {
                    const size_t hi = ((size_t)(j / 32) * rows + 2 * m) * 32 + j % 32;
                    q[(size_t)(m0 + m) * K + k0 + j] =
                        (int8_t)(16 * nibble(packed.data(), hi) + nibble(packed.data(), hi + 32) + 8);
                }
        }
    }
    return 0;
}

void ref_w4a8_dequant(int M, int N, const int32_t* acc, const float* a_scale,
                      const float* w_scale, int half, void* out) {
    detail::w4a8_dequant(M, N, acc, a_scale, w_scale, half != 0, out, 1);
}

int ref_w4a8_finish_scales(int M, const uint32_t* bits, float* scales, float* inverse) {
    return detail::w4a8_finish_scales(M, 1, bits, M, scales, inverse);
}

// MoE middle of one assignment row: acc[2 * channels] (gate then up) ->
// SwiGLU (libm exp off AArch64) -> row scale -> nearest-even int8.
float ref_moe_middle_row(const int32_t* acc, int channels, const float* weight_scales,
                         float input_scale, int8_t* out_q) {
    moe::MiddleRow r{};
    r.partial = acc; // rows == 1: native (N/4, rows, 4) collapses to plain order
    r.correction = nullptr;
    r.weight_scales = weight_scales;
    r.input_scale = input_scale;
    r.rows = 1;
    r.row = 0;
    r.channels = channels;
    r.waves = 1;
    r.wave_stride = 0;
    r.output = out_q;
    r.layout = moe::MiddleLayout::I8Normal;
    return moe::swiglu_quantize_row(r);
}

// Largest certified fixed K partition (requested == 0) or certification of one
// requested tile.  Returns the tile, or a negative error code.
int ref_bound_i4(int K, int N, const int8_t* B, int requested) {
    detail::I4WeightBound bound;
    const int rc = detail::bound_i4_weights(K, N, B, requested, bound);
    return rc ? rc : bound.k_tile;
}

} // extern "C"
