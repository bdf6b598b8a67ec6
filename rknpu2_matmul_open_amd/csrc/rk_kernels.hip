// HIP kernels of the quantized-linear path for gfx950 (MI355X), and the C-ABI
// launchers declared in rk_hip_shim.h.  Data layouts are described there.
// This unit holds the C ABI and the small kernels; the three large kernel families are units
// of their own: rk_kernels_gemv.hip (gemv_kernel, gemv_swiglu_kernel), rk_kernels_gemm.hip
// (gemm_wk_kernel, gemm_wk_reduce_kernel), rk_kernels_stream.hip (gemm_stream_kernel).
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
//   moe_decode_gate_kernel / moe_decode_down_kernel   the MoE layer for up to twelve tokens in two
//                                       launches: dot products, no routing tables          (latency, HBM)
//   stream_read_probe_kernel / mfma_i8_probe_kernel   measurement probes (practical ceilings)
#include <shared_mutex>

#include "rk_kernels_common.h"

namespace {

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
} // namespace

namespace rkk {
void mark(hipStream_t stream, const char* kernel) {
    if (!g_marker_on.load(std::memory_order_acquire)) return;
    std::shared_lock<std::shared_mutex> lock(g_marker_mutex);
    if (g_marker) g_marker(g_marker_user, stream, kernel);
}

// Compute units of the current device (0 if the query fails), looked up once per device.
int compute_units() {
    static std::atomic<int> cached[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (!n) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}
} // namespace rkk

namespace {

// the other units' launchers and predicates, as the C ABI below uses them
using rkk::dense_stream_fits;
using rkk::dispatch_gemv;
using rkk::dispatch_gemv_swiglu;
using rkk::gemv_can_fuse;
using rkk::gemv_max_rows;
using rkk::gemv_swiglu_applies;
using rkk::launch_gemm_grouped;
using rkk::launch_gemm_wk_narrow;
using rkk::wk_scratch_bytes;

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
        // (four chunks are fetched before the first is stored: the store is an asm statement the
        // compiler keeps every load behind, and a thread that alternates load and store pays one
        // memory latency per chunk)
        for (int c0 = chunk0 + t; c0 < nchunks; c0 += 4 * 256) {
            uint4 v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int c = c0 + i * 256;
                uint32_t w[4] = {0, 0, 0, 0};
                if (c < nchunks) {
                    if (vec && c * 16 + 16 <= K) {
                        const uint4 v4 = *reinterpret_cast<const uint4*>(brow + c * 16);
                        w[0] = v4.x; w[1] = v4.y; w[2] = v4.z; w[3] = v4.w;
                    } else {
                        for (int j = 0; j < 16; ++j)
                            if (c * 16 + j < K) w[j >> 2] |= (uint32_t)(uint8_t)brow[c * 16 + j] << ((j & 3) * 8);
                    }
                }
                v[i] = make_uint4(w[0], w[1], w[2], w[3]);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int c = c0 + i * 256;
                if (c < nchunks) store_codes(a.dst + tiled_chunk_offset(m, c, KB), v[i]);
            }
        }
        return;
    }
    const bool need_max = mode == RKH_Q_W8_DYNAMIC || mode == RKH_Q_W4A8;
    const bool check = mode == RKH_Q_W4A8;

    float v[QR_CACHE][16];
    float mx = 0.0f;
    float taint = 0.0f; // (NaN once an Inf or a NaN was seen, see absmax16)
    if (cached) {
#pragma unroll
        for (int i = 0; i < QR_CACHE; ++i) {
            const int c = chunk0 + t + i * 256;
            if (c < nchunks) {
                RowLoader<T>::load16(row, c * 16, K, vec, v[i]);
                if (need_max) {
                    absmax16(v[i], mx, taint);
                }
            }
        }
    } else if (need_max) {
        for (int c = chunk0 + t; c < nchunks; c += 256) {
            float tmp[16];
            RowLoader<T>::load16(row, c * 16, K, vec, tmp);
            absmax16(tmp, mx, taint);
        }
    }

    float scale = 1.0f;
    if (need_max) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
        const unsigned long long bad_mask = __ballot(tainted(taint) && check);
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
    if (m >= a.M) return;
    // (The count of live row blocks is requested with the row, not ahead of it: rows beyond the
    // live blocks exist -- the buffers are sized for the most blocks a call can have -- so reading
    // one is harmless, and the wave leaves before it writes anything.  Asked for first, the count
    // cost every wave a round trip before its first row load.)
    const int live_rows = a.active_blocks ? a.active_blocks[0] * 32 : a.M;
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
    if (m >= live_rows) return;
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
// (Holding fp16 rows as fetched -- 8 registers a chunk, twice the reach -- with the maxima taken
// from the bit patterns was built and measured: rows of 11008 at 1024 rows 19.7 -> 15.7 us, but at
// 256 / 512 rows slower than a workgroup per row, 12.7 / 15.1 against 9.9 / 13.3 us, and the
// 2048 x 4096 case 0.5 us slower, so rows are held as floats.)
constexpr int Q8_CACHE = 8;

template <typename T, int ROWS>
__global__ __launch_bounds__(256) void quant_rows8_kernel(RK_QUANT_HEAD_PARAMS, rkh_quant_args a) {
    RK_QUANT_HEAD_APPLY(a);
    __shared__ float part_max[4 * ROWS];
    __shared__ int part_bad[4];
    quant_rows_group<T, ROWS, 256, Q8_CACHE>(a, blockIdx.x * ROWS, part_max, part_bad);
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
        float taint = 0.0f; // (NaN once an Inf or a NaN was seen, see absmax16)
        if (cached) {
#pragma unroll
            for (int i = 0; i < QR_CACHE; ++i)
                if (t + i * 256 < nchunks) {
                    absmax16(v[i], mx, taint);
                }
        } else {
            for (int c = t; c < nchunks; c += 256) {
                float tmp[16];
                RowLoader<T>::load16(row, c * 16, K, vec, tmp);
                absmax16(tmp, mx, taint);
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
        const unsigned long long bad_mask = __ballot(tainted(taint));
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
    // Eight slots at a time: their destination rows and coefficients first, then the rows they name,
    // then the sums in slot order.  Slot by slot the loop was a chain of two dependent round trips
    // per slot (row index, then the row), 2.7 us for the four slots of a top-4 layer in a kernel
    // that moves a few MB.
    constexpr int B = 8;
    for (int s0 = 0; s0 < slots; s0 += B) {
        int d[B];
        float w[B];
        float4 y[B];
#pragma unroll
        for (int j = 0; j < B; ++j) {
            const int s = s0 + j;
            d[j] = s < slots ? a.dest_rows[(size_t)tkn * slots + s] : -1;
            w[j] = s < a.top_k ? a.routes[(size_t)tkn * a.top_k + s] : 1.0f;
        }
#pragma unroll
        for (int j = 0; j < B; ++j) {
            y[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (d[j] >= 0) y[j] = *reinterpret_cast<const float4*>(a.Y + (size_t)d[j] * a.H + n);
        }
#pragma unroll
        for (int j = 0; j < B; ++j) {
            if (d[j] < 0) continue;
            sum.x = fmaf(y[j].x, w[j], sum.x);
            sum.y = fmaf(y[j].y, w[j], sum.y);
            sum.z = fmaf(y[j].z, w[j], sum.z);
            sum.w = fmaf(y[j].w, w[j], sum.w);
        }
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

// (Leading scalar arguments, in registers when a wave starts: what the first loads of both kernels
// depend on -- the routing arrays, the token rows, the middle rows.  Read from the argument
// structure they cost every wave a round trip to memory ahead of the routing entries.)
#define RK_MOE_DECODE_HEAD_PARAMS                                                                       \
    const float* h_x, const int32_t* h_ids, const float* h_routes, int h_top_k, int h_experts, int h_shared, int h_H, \
        int h_I, float* h_hidden, uint32_t* h_row_max_bits
#define RK_MOE_DECODE_HEAD(a) (a).x, (a).ids, (a).routes, (a).top_k, (a).experts, (a).shared, (a).H, (a).I, (a).hidden, (a).row_max_bits
#define RK_MOE_DECODE_HEAD_APPLY(a)                                                                     \
    do {                                                                                                \
        (a).x = h_x; (a).ids = h_ids; (a).routes = h_routes; (a).top_k = h_top_k; (a).experts = h_experts; \
        (a).shared = h_shared; (a).H = h_H; (a).I = h_I; (a).hidden = h_hidden; (a).row_max_bits = h_row_max_bits; \
    } while (0)

__global__ __launch_bounds__(512) void moe_decode_gate_kernel(RK_MOE_DECODE_HEAD_PARAMS, rkh_moe_decode_args a) {
    RK_MOE_DECODE_HEAD_APPLY(a);
    __shared__ __attribute__((aligned(16))) uint8_t a_lds[MOE_DECODE_MAX_K];
    __shared__ int red[2][8][32];
    __shared__ float wave_max[8];
    __shared__ int wave_bad[8];
    const int slots = a.top_k + a.shared;
    const int j = blockIdx.x, asg = blockIdx.y, t = asg / slots, s = asg - t * slots;
    const int tid = threadIdx.x, lane = lane_id(), wave = wave_id(), half = lane >> 5;
    const int H = a.H, Hp = (int)rkh_align_up(H, RKH_K_ALIGN), nchunks = (H + 15) >> 4;

    // ---- the token row is requested first: its address depends on nothing but the block index,
    // so it travels together with the routing entry instead of behind the first weight tiles
    // (loads return in issue order)
    const float* row = a.x + (size_t)t * H;
    const bool vec = (reinterpret_cast<uintptr_t>(row) & 15) == 0;
    constexpr int CACHE = MOE_DECODE_MAX_K / 16 / 512; // chunks per thread
    float v[CACHE][16];
#pragma unroll
    for (int i = 0; i < CACHE; ++i) {
        const int c = tid + i * 512;
        if (c < nchunks) RowLoader<float>::load16(row, c * 16, H, vec, v[i]);
    }
    const MoeSlot slot = moe_slot(a, t, s);
    const bool reporter = j == 0 && tid == 0;
    if (slot.bad && reporter && a.bad_flag) atomicOr(a.bad_flag, 1);
    if (!slot.live) return;

    // ---- gate block 2j and up block 2j + 1 of the expert.  Two groups of PF tiles per wave and
    // block are in flight: the first is requested now, the second when the token is quantized (one
    // token per call gained 0.3 us with the second group requested between the barriers of the
    // quantization, four and eight tokens lost 1.5 and 3.5 us).  The loads are unconditional -- past
    // the end of the block a wave reads its last tile again and does not use it -- so that the
    // compiler counts them and the quantization waits for the row only, not for the tiles.
    // Against the first group requested ahead of the row, behind branches, and the rest in the
    // loop: 17.8 -> 15.7 / 24.1 -> 23.8 / 37.3 -> 35.9 us for one / four / eight tokens (both launches).
    const int e = slot.expert;
    const bool int4 = e < a.int4_experts;
    const int tiles = int4 ? Hp / 64 : Hp / 32; // per column block
    const size_t block_bytes = (size_t)tiles * 1024;
    const uint8_t* wb = (int4 ? a.gate_W4 + (size_t)e * a.gate_stride4
                              : a.gate_W + (size_t)(e - a.int4_experts) * a.gate_stride) + (size_t)(2 * j) * block_bytes;
    constexpr int PF = MOE_DECODE_PREFETCH;
    v4i cur[2][PF], nxt[2][PF];
    auto load_group = [&](v4i (*regs)[PF], int grp) {
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            const int idx = min(wave + 8 * (grp * PF + u), tiles - 1);
#pragma unroll
            for (int b = 0; b < 2; ++b)
                regs[b][u] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wb + b * block_bytes + (size_t)idx * 1024 + lane * 16));
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    load_group(cur, 0);
    // (the two column scales of the epilogue ride behind the first group)
    const float* ws = a.gate_scales + (size_t)e * 2 * a.I;
    const int n = j * 32 + (tid & 31); // (I is a multiple of 32)
    const float ws_gate = ws[n], ws_up = ws[a.I + n];
    __builtin_amdgcn_sched_barrier(0);

    // ---- the token as int8 codes in LDS (s = max > 0 ? max / 127 : 1, ties to even)
    float mx = 0.0f;
    float taint = 0.0f; // (NaN once an Inf or a NaN was seen, see absmax16)
#pragma unroll
    for (int i = 0; i < CACHE; ++i) {
        const int c = tid + i * 512;
        if (c < nchunks) absmax16(v[i], mx, taint);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    const unsigned long long bad_mask = __ballot(tainted(taint));
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
    load_group(nxt, 1);

    // ---- dot products: the waves take the tiles of both blocks in turn
    int acc[2] = {0, 0};
    const int groups = (tiles + 8 * PF - 1) / (8 * PF);
    for (int grp = 0; grp < groups; ++grp) {
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            const int idx = wave + 8 * (grp * PF + u);
            if (idx < tiles) {
                moe_dot_tile(int4, a_lds, idx, half, cur[0][u], acc[0]);
                moe_dot_tile(int4, a_lds, idx, half, cur[1][u], acc[1]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            cur[0][u] = nxt[0][u];
            cur[1][u] = nxt[1][u];
        }
        if (grp + 2 < groups) load_group(nxt, grp + 2); // (uniform)
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
        const float gf = dequant(gate, scale, ws_gate);
        const float uf = dequant(up, scale, ws_up);
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
// CW = output columns per workgroup: 32, or 16 / 8 while that many workgroups still leave compute
// units without one (one token of a 2048-wide layer: 64 workgroups of 32 columns) -- a load then
// covers the workgroup's part of 32 / CW consecutive tiles, as in the decode GEMV.
template <int CW>
__global__ __launch_bounds__(512) void moe_decode_down_kernel(RK_MOE_DECODE_HEAD_PARAMS, rkh_moe_decode_args a) {
    RK_MOE_DECODE_HEAD_APPLY(a);
    constexpr int TPL = 32 / CW; // tiles covered by one load instruction
    __shared__ __attribute__((aligned(16))) uint8_t a_lds[MOE_DECODE_MAX_K]; // live slot i at i * Ip
    __shared__ int red[MOE_DECODE_SLOTS][8][CW];
    __shared__ float live_scale[MOE_DECODE_SLOTS], live_coeff[MOE_DECODE_SLOTS];
    __shared__ int live_expert[MOE_DECODE_SLOTS], live_slot[MOE_DECODE_SLOTS];
    __shared__ int live_count;
    const int slots = a.top_k + a.shared;
    const int pb = blockIdx.x / TPL, col0 = ((int)blockIdx.x % TPL) * CW, t = blockIdx.y;
    const int tid = threadIdx.x, lane = lane_id(), wave = wave_id();
    const int half = (lane / CW) & 1, sub = lane / (2 * CW); // k-half of a tile, tile of the load
    const unsigned lane_byte = (unsigned)((col0 + lane % CW) + 32 * half) * 16u;
    const int I = a.I, Ip = (int)rkh_align_up(I, RKH_K_ALIGN), nchunks = I >> 4, parts = I / 32;
    if (wave == 0) { // the live slots in slot order: lane s reads slot s, a live slot's place is its rank among them
        // (one thread walking the slots was a chain of as many round trips to the routing arrays)
        MoeSlot slot = {0, 0.0f, false, false};
        if (lane < slots) slot = moe_slot(a, t, lane);
        const unsigned long long live_mask = __ballot(slot.live);
        if (slot.live) {
            const int n = __popcll(live_mask & ((1ull << lane) - 1ull));
            live_expert[n] = slot.expert;
            live_coeff[n] = slot.coeff;
            live_slot[n] = lane;
        }
        if (lane == 0) live_count = __popcll(live_mask);
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
    // (unconditional loads -- past the end of a block a lane reads the block's last tile again and does
    // not use it -- so that the compiler counts them: a wait for older data then leaves them in flight)
    auto load_group = [&](int li, int grp, v4i* regs) {
        bool int4;
        int tiles;
        const uint8_t* wb = block_of(li, int4, tiles);
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            const int tile = min(((grp * PF + u) * 8 + wave) * TPL + sub, tiles - 1);
            regs[u] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wb + (size_t)tile * 1024 + lane_byte));
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    if (nlive == 0) { // (nothing routed to this token)
        if (tid < CW) a.out[(size_t)t * a.H + pb * 32 + col0 + tid] = 0.0f;
        return;
    }

    // ---- the middle rows (max != 0 ? max / 127 : 1, ties to even): wave li quantizes live slot li.
    // Its row and partial maxima are requested first, the first group of down tiles behind them.
    constexpr int CACHE = (MOE_DECODE_DOWN_K / 16 + 63) / 64; // chunks per lane
    auto fetch_row = [&](int li, float (*v)[16], uint32_t& bits) {
        const int asg = t * slots + live_slot[li];
        const float* hrow = a.hidden + (size_t)asg * I;
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
        bits = 0;
        for (int i = lane; i < parts; i += 64) bits = max(bits, a.row_max_bits[(size_t)asg * parts + i]);
    };
    auto quantize_row = [&](int li, float (*v)[16], uint32_t bits) {
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
    };
    v4i cur[PF], nxt[PF];
    {
        float v[CACHE][16];
        uint32_t bits = 0;
        if (wave < nlive) fetch_row(wave, v, bits);
        __builtin_amdgcn_sched_barrier(0);
        load_group(0, 0, cur);
        if (wave < nlive) quantize_row(wave, v, bits);
    }
    for (int li = wave + 8; li < nlive; li += 8) { // (more than eight live slots: top-8 and a shared expert)
        float v[CACHE][16];
        uint32_t bits = 0;
        fetch_row(li, v, bits);
        quantize_row(li, v, bits);
    }
    // the slots' column scales of the epilogue, requested now instead of one after the other at the end
    float dsc[MOE_DECODE_SLOTS];
#pragma unroll
    for (int li = 0; li < MOE_DECODE_SLOTS; ++li)
        dsc[li] = a.down_scales[(size_t)live_expert[li < nlive ? li : 0] * a.H + pb * 32 + col0 + tid % CW];
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();

    // ---- the down blocks
    for (int li = 0; li < nlive; ++li) {
        bool int4;
        int tiles;
        block_of(li, int4, tiles);
        const int groups = ((tiles + TPL - 1) / TPL + 8 * PF - 1) / (8 * PF);
        const uint8_t* codes = a_lds + (size_t)li * Ip;
        int acc = 0;
        for (int grp = 0; grp < groups; ++grp) {
            // the next group: of this slot, else the first of the next slot, else (nothing left) this one again
            const bool last = grp + 1 == groups, more = li + 1 < nlive;
            load_group(last && more ? li + 1 : li, last ? (more ? 0 : grp) : grp + 1, nxt);
#pragma unroll
            for (int u = 0; u < PF; ++u) {
                const int tile = ((grp * PF + u) * 8 + wave) * TPL + sub;
                if (tile < tiles) moe_dot_tile(int4, codes, tile, half, cur[u], acc);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < PF; ++u) cur[u] = nxt[u];
        }
        acc += __shfl_xor(acc, 32);
        if (CW <= 16) acc += __shfl_xor(acc, 16);
        if (CW <= 8) acc += __shfl_xor(acc, 8);
        if (lane < CW) red[li][wave][lane] = acc;
    }
    __syncthreads();
    if (tid < CW) {
        const int n = pb * 32 + col0 + tid; // (H is a multiple of 32)
        float sum = 0.0f;
#pragma unroll
        for (int li = 0; li < MOE_DECODE_SLOTS; ++li) {
            if (li < nlive) {
                int acc = 0;
#pragma unroll
                for (int w = 0; w < 8; ++w) acc += red[li][w][tid];
                const int e = live_expert[li];
                if (e < a.int4_experts) acc >>= 4;
                const float y = dequant(acc, live_scale[li], dsc[li]);
                sum = fmaf(y, live_coeff[li], sum);
            }
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
    rkk::set_ts_gemv(p); // (every unit has its own copy of the pointer)
    rkk::set_ts_gemm(p);
    rkk::set_ts_stream(p);
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
    // Several rows per workgroup only while a row fits the registers its threads hold it in (8 rows:
    // 4096 elements, 4 rows: 8192): longer rows are read twice in a loop, and 256 rows of 11008 then
    // took 15 us where a workgroup per row takes 6.5.
    const int row_chunks = (args->K + 15) / 16;
    const bool fits8 = row_chunks <= (256 / 8) * Q8_CACHE, fits4 = row_chunks <= (256 / 4) * Q8_CACHE;
    if (args->M >= 256 && !args->active_blocks && args->in_dtype != RKH_I8 && fits4 &&
        (mode == RKH_Q_W8_DYNAMIC || mode == RKH_Q_W4A8 || mode == RKH_Q_W8_STATIC)) {
        const bool rows4 = !fits8 || args->M < 8 * 2 * 256; // 8 rows would give fewer than two workgroups per compute unit
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
    if (g.blk_expert) return false;
    if (g.M > max_rows) {
        // 129 .. 256 rows on a narrow matrix, while the grid is small enough that K is split over the
        // waves (64-column tiles): up to eight row blocks x N / 64 workgroups of this kernel against a few
        // dozen tiles of the LDS-ring kernel.  fp16 in / out, quantization included, us, 136 / 256 rows:
        // int8 2048 x 2048 12.9 / 13.4 -> 10.0 / 10.5, 4096 x 2048 18.1 / 18.9 -> 13.1 / 14.1, 8192 x 2048
        // 27.4 / 29.2 -> 20.5 / 23.1, 4096 x 1024 20.2 / 19.1 -> 11.9 / 12.0, 4096 x 4096 at 136 / 224 rows
        // 20.2 / 20.5 -> 18.5 / 19.3, 6144 x 4096 26.8 / 27.3 -> 24.3 / 26.1; int4 2048 x 2048 10.7 -> 9.5,
        // 4096 x 2048 15.8 / 16.1 -> 12.3 / 13.1, 8192 x 2048 21.9 / 26.1 -> 17.4 / 18.8, 14336 x 2048
        // 29.8 / 32.3 -> 25.3 / 26.1.  Where it stops: a longer K (int8 11008 x 4096 32.5 -> 37.8, 14336 x 2048
        // 30.0 -> 31.3, 8192 x 4096 a tie), int4 weights from 4096 columns on (a tie), 256-column tiles
        // (4096 x 4096 at 256 rows 20.9 -> 27.1), more rows (4096 x 2048 at 384 rows a tie).
        static const char* plan = getenv("RK_NPU_HIP_GEMM_PLAN"); // (a forced plan is a plan of the large-tile kernel)
        // (a matrix of up to 1024 columns: up to 512 rows -- 4096 x 1024 at 384 rows 19.9 -> 14.6, int4 14.1 -> 12.7)
        if (forced || (plan && plan[0]) || g.epilogue == RKH_EPI_SWIGLU || g.M > (g.N <= 1024 ? 4 : 2) * DENSE_STREAM_MAX_M) return false;
        if ((long)((g.M + 31) / 32) * ((g.N + 255) / 256) >= DENSE_KS4_BELOW) return false;
        if (g.N <= 2048) return g.K <= (g.w_int4 ? 16384 : 8192);
        return !g.w_int4 && g.N <= 4096 && g.K <= 6144;
    }
    // (the SwiGLU decode kernel has taken its calls by now -- up to four rows -- whatever the row limit of
    // the plain decode kernels is: five to eight rows of a gate/up GEMM stream too)
    if (g.epilogue == RKH_EPI_SWIGLU) return g.w_int4 && g.K <= 131072 && g.M <= DENSE_STREAM_SWIGLU_MAX_M;
    if (g.M <= gemv_max_rows(g)) return false;
    // 65 .. 128 rows on an int8 matrix so wide that the tiles of 32 rows x 256 columns walk K without a
    // split: three or four row blocks stream every weight byte three or four times through the compute
    // units' memory paths, and the LDS-ring kernel's tiles of 64 rows x 128 columns (dense_narrow) or its
    // 128-row tiles do better.  fp16 in / out, quantization included, us, K = 4096 at 128 rows:
    // N = 11008 28.4 -> 24.1, 14336 28.5 -> 24.3, 28672 36 -> 26; K = 6144, N = 11008 36.4 -> 30.2; K = 2048,
    // N = 11008 17.0 -> 15.7.  (Narrower matrices split K over the waves of 64- or 32-column tiles and
    // stay: 4096 x 6144 19.9 against 22.8, 4096 x 8192 at 96 rows 18.1 against 21.7.)
    if (!forced && !g.w_int4 && g.M > 64 && g.K <= 6144 &&
        (long)((g.M + 31) / 32) * ((g.N + 255) / 256) >= DENSE_KS4_BELOW) return false;
    // (int4 weights: the two kernels measure the same there -- until the 32 x 256 tiles outnumber the compute
    // units and run in two rounds: 4096 x 28672 at 72 / 128 rows 33.5 / 34.8 -> 23.5 / 25.5 us on the large tiles)
    if (!forced && g.w_int4 && g.M > 64 && g.K <= 6144 &&
        (long)((g.M + 31) / 32) * ((g.N + 255) / 256) > (compute_units() > 0 ? compute_units() : 256)) return false;
    return !g.w_int4 || g.K <= 131072;
}

// A few hundred rows, while tiles of 64 rows x 128 columns still give every compute unit at most one: the
// LDS-ring kernel with one column block per wave (launch_gemm_wk_narrow) instead of its 256-column tiles
// with K split over workgroups and a reduce launch behind them.  A tile pulls K x (64 + 128) bytes through
// its compute unit (int4 weights: K x (64 + 64)) and every compute unit has one.  fp16 in / out,
// quantization included, weights from HBM, us: int8 4096 x 4096 at 160 / 256 / 512 rows 22.6 / 23.1 / 24.5 ->
// 20.5 / 20.9 / 22.1, 4096 x 11008 at 192 rows 27.2 -> 26.3, at 128 rows 23.9 -> 20.6, 4096 x 14336 at 128 rows
// 24.6 -> 22.1, 6144 x 11008 at 128 rows 30.1 -> 27.0; int4 4096 x 4096 at 160 / 256 / 512 rows 19.8 / 18.0 / 20.6 ->
// 16.1 / 15.5 / 17.8, 2048 x 8192 at 192 rows 13.7 -> 12.0.  (The int8 shapes ran on the streaming kernel with two
// row blocks per wave before, which pulled 1 MB per tile where this one pulls 768 KB and which lost to the
// other plans with int4 weights; those instantiations are gone.)  It loses where the tiles outnumber
// the compute units (int8 4096 x 4096 at 768 rows 30.8 -> 31.9, 4096 x 14336 at 512 rows 41 -> 68; int4
// 4096 x 11008 at 160 rows, 258 tiles: 20.6 -> 23.2) and for a long K (11008 x 4096 at 192 rows 33.2 -> 42:
// there the K split pays), which is where the rule stops.  RK_NPU_HIP_NARROW_TILES = 0 switches it off,
// 1 forces it (2: the 128-row tiles below) for every dense GEMM beyond the streaming kernel's rows that
// needs no K split (tuning aid).
static int dense_narrow(const rkh_gemm_args& g) { // rows of the tile, or 0: another plan
    if (g.blk_expert || g.epilogue == RKH_EPI_SWIGLU || min_ksplit(g.K, g.w_int4) > 1) return 0;
    static const char* forced = getenv("RK_NPU_HIP_NARROW_TILES");
    if (forced && forced[0]) return forced[0] == '1' ? 64 : forced[0] == '2' ? (g.w_int4 ? 64 : 128) : 0;
    static const char* plan = getenv("RK_NPU_HIP_GEMM_PLAN"); // (a forced plan is a plan of the 256-column tiles)
    if (plan && plan[0]) return 0;
    const int cus = compute_units() > 0 ? compute_units() : 256;
    const long nblocks = (g.N + 127) / 128;
    if (g.K <= 6144 && (long)((g.M + 63) / 64) * nblocks <= (g.w_int4 ? cus : cus + cus / 50)) return 64;
    // Beyond that, int8 weights: tiles of 128 rows x 128 columns of the same kernel while THEY give every
    // compute unit at most one and at least five in eight of them have one.  A tile pulls K x (128 + 128)
    // bytes for twice the products, and no K split means no reduce launch; a long K is no obstacle here.
    // us as above, against the 256-column tiles' plan: 4096 x 4096 at 520 / 640 / 768 / 1024 rows 31.0 / 31.7 /
    // 30.8 / 32.6 -> 27.3 / 27.8 / 27.8 / 28.8, 11008 x 4096 at 640 / 768 / 1024 rows 65.3 / 68.6 / 78.0 -> 62.5 / 65.4 /
    // 70.6, 4096 x 8192 at 260 / 384 / 512 rows 31.9 / 33.2 / 34.7 -> 26.6 / 27.2 / 30.9, 8192 x 8192 at 260 / 480 rows
    // 51.8 / 61.3 -> 46.3 / 49.8, 4096 x 11008 at 136 / 256 rows 29.4 / 32.7 -> 25.4 / 28.0, 11008 x 11008 at 136 / 256
    // rows 59.3 / 62.3 -> 41.9 / 46.2.  A last row block that is mostly padding costs little (4096 x 4096 at
    // 520 rows above).  No allowance beyond the compute units here: 258 tiles (three row blocks of an
    // 11008-wide matrix) run two of them in a second round and lose with a partly filled last block
    // (6144 x 11008 at 288 / 320 rows 46.5 / 46.3 -> 48.9 / 50.2, 11008 x 11008 68.9 / 69.7 -> 78.6 / 81.8); with a full
    // one, 384 rows, they won on one box (4096 x 11008 39.5 -> 35.8) and lost on another (39.2 -> 41.3).  With
    // more tiles it loses (4096 x 4096 at 1536 rows 39.5 -> 44.8, 4096 x 11008 at 640 rows 44.3 -> 49.5), and so
    // it does with int4 weights at every size measured (4096 x 4096 at 640 rows 23.5 -> 25.5, 4096 x 8192
    // 34.8 -> 42.3), whose tiles pull half the weight bytes to begin with.
    const long tiles128 = (long)((g.M + 127) / 128) * nblocks;
    if (!g.w_int4 && tiles128 >= cus * 5L / 8 && tiles128 <= cus) return 128;
    return 0;
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
    if (const int tile_rows = dense_narrow(g)) return launch_gemm_wk_narrow(st, g, tile_rows);
    const DensePlan plan = effective_plan(g.M, g.N, g.K, g.w_int4);
    int ksplit = plan.ksplit;
    if (ksplit > 1 && !g.splitk_acc) {
        if (min_ksplit(g.K, g.w_int4) > 1) return RKH_ERR_RUNTIME;
        ksplit = 1;
    }
    return rkk::launch_gemm_wk(st, g, plan.bm, ksplit);
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
    // (the 256-token layer of the benchmark, 32 experts, top-4, us, two launches against the grouped path:
    // 8 tokens 32.7 / 47.8, 10 43.4 / 50.2, 12 50.1 / 53.7, 16 62.2 / 55.3, 24 91.5 / 58.2)
    const int max_rows = forced ? atoi(forced) : 12;
    return rows >= 1 && rows <= max_rows && H >= 32 && H % 32 == 0 && H <= MOE_DECODE_MAX_K && I >= 32 && I % 32 == 0 &&
           rkh_align_up(I, RKH_K_ALIGN) <= (size_t)MOE_DECODE_DOWN_K; // (nine middle rows side by side in LDS)
}

int rkh_moe_decode(void* stream, const rkh_moe_decode_args* args) {
    const rkh_moe_decode_args& a = *args;
    if (!rkh_moe_decode_applies(a.rows, a.H, a.I) || a.top_k < 1) return RKH_ERR_RUNTIME;
    const int slots = a.top_k + (a.shared ? 1 : 0);
    mark((hipStream_t)stream, "moe_decode_gate_kernel");
    hipLaunchKernelGGL(moe_decode_gate_kernel, dim3(a.I / 32, a.rows * slots), dim3(512), 0, (hipStream_t)stream,
                       RK_MOE_DECODE_HEAD(a), a);
    mark((hipStream_t)stream, "moe_decode_down_kernel");
    const int cus = compute_units() > 0 ? compute_units() : 256;
    const long down_wgs = (long)(a.H / 32) * a.rows; // (with 32 columns each)
    if (down_wgs * 4 <= cus)
        hipLaunchKernelGGL(moe_decode_down_kernel<8>, dim3(a.H / 8, a.rows), dim3(512), 0, (hipStream_t)stream, RK_MOE_DECODE_HEAD(a), a);
    else if (down_wgs * 2 <= cus)
        hipLaunchKernelGGL(moe_decode_down_kernel<16>, dim3(a.H / 16, a.rows), dim3(512), 0, (hipStream_t)stream, RK_MOE_DECODE_HEAD(a), a);
    else
        hipLaunchKernelGGL(moe_decode_down_kernel<32>, dim3(a.H / 32, a.rows), dim3(512), 0, (hipStream_t)stream, RK_MOE_DECODE_HEAD(a), a);
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

