// Decode-sized rows (M <= 8): dot-product kernels, no MFMA.  gemv_kernel (optionally with the
// per-token quantization in its prologue), gemv_swiglu_kernel (gate/up + SwiGLU of one or two
// rows) and their launchers.  Bound by HBM.
#include "rk_kernels_common.h"

namespace {

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
// Activation bytes staged per K chunk: 32 KiB; 64 KiB in the BIG variants (two workgroups of 64 KiB +
// their reduction area still fit a compute unit's 160 KiB), which take four to eight rows of a long
// K on int8 weights, so that four rows of a 14336-deep projection are one chunk -- and can be
// quantized by the kernel itself instead of a launch in front (21.6 -> 18.0 us).  Shapes that fit
// the small area keep the small kernel: with room for eight chunks a thread, four rows of
// 4096 x 4096 took 7.1 instead of 6.65 us.  (The int4 variants have no registers to spare for it.)
constexpr int GEMV_LDS_BYTES = 32768;
__host__ __device__ constexpr int gemv_lds_bytes(bool big) { return big ? 2 * GEMV_LDS_BYTES : GEMV_LDS_BYTES; }
__host__ __device__ constexpr bool gemv_big_applies(int mr, bool w4, long padded_k) {
    return mr >= 4 && !w4 && padded_k * mr > GEMV_LDS_BYTES;
}

#ifndef RK_GEMV_MFMA_ROWS
#define RK_GEMV_MFMA_ROWS 4
#endif
constexpr int GEMV_MFMA_ROWS = RK_GEMV_MFMA_ROWS; // from this many rows on the products go through the matrix cores
#ifndef RK_GEMV_MFMA_ROWS_I8
#define RK_GEMV_MFMA_ROWS_I8 2
#endif
// (the same for int8 weights: two rows already -- 4096 x 4096 6.2 -> 5.85 us, 14336 x 4096 14.3 -> 13.9; int4
// weights pay for the unpacking, two rows 5.3 -> 6.4 us)
constexpr int GEMV_MFMA_ROWS_I8 = RK_GEMV_MFMA_ROWS_I8;
// 16-element activation chunks a thread may quantize in the fused path: four; eight for fp16 rows
// (8 registers a chunk as fetched) in the BIG variants, which fills their staging area
constexpr int GEMV_QCHUNKS = 4;
__host__ __device__ constexpr int gemv_qchunks(bool big, int elem_bytes) { return big && elem_bytes == 2 ? 2 * GEMV_QCHUNKS : GEMV_QCHUNKS; }

// The per-token quantization that both dot-product kernels can run in their prologue: every
// workgroup quantizes the few rows itself into its LDS staging area (they are L2 hits after the
// first workgroup), which saves a launch per decode step.  Every instruction here is executed by
// every workgroup, ahead of its first dot product -- for several rows this prologue, not the
// weight stream, is what a 4096 x 4096 call waits for (in-kernel time stamps, eight rows: 3.8 of
// 9.4 us) -- so it is kept lean:
//   * chunk i of 16 elements of thread t is number t + i * (threads) of the rows laid end to end;
//     its row and its place in the row are stepped from chunk to chunk (one division per thread,
//     none for a single row), and each pass steps again from the first chunk's place, which is all
//     that stays in registers between the passes (the empty asm keeps the compiler from holding
//     all eight indices instead);
//   * the largest magnitude of a chunk is taken from the bit patterns as fetched: magnitudes of
//     finite values order like their patterns, so no element is converted for this pass (fp16: two
//     per instruction), and a chunk that holds an Inf or a NaN -- its largest pattern says so --
//     takes the float comparisons, which skip NaNs;
//   * 1 / scale is divided once per row, not once per chunk.
// The rows stay in registers as fetched and are converted once, for the codes: holding them as
// floats across the barriers costs the int4 variants their second workgroup per compute unit.
// (One fp16 row in pieces of 8 elements, so that a row of 4096 gives every one of the 512 threads a
// piece instead of half of them a chunk, was built and measured: 10.9 against 10.75 us for
// 4096 x 14336, 5.35 against 5.15 for 4096 x 4096 -- twice the lanes on the one LDS maximum and
// twice the slots of straight-line code cost more than the idle waves.  Note for anyone who tries
// again: an LDS atomic whose address the compiler can prove uniform is replaced by a scalar loop
// over the 64 lanes, 1.5 us per use here; keep the index in a vector register.)
template <typename T, int MR, bool BIG>
struct FusedRows {
    static constexpr int THREADS = GEMV_WAVES * 64;
    static constexpr int QCH = gemv_qchunks(BIG, (int)sizeof(T));
    typename RowLoader<T>::Raw raw[QCH];
    int m0, c0; // row and place in the row of this thread's first chunk

    __device__ __forceinline__ void index(int nchunks, int (&m)[QCH], int (&c)[QCH]) {
        if constexpr (MR == 1) {
#pragma unroll
            for (int i = 0; i < QCH; ++i) {
                c[i] = (int)threadIdx.x + i * THREADS;
                m[i] = c[i] < nchunks ? 0 : 1;
            }
        } else {
            const int step_m = THREADS / nchunks, step_c = THREADS - step_m * nchunks; // (uniform)
            asm volatile("" : "+v"(m0), "+v"(c0));
            m[0] = m0;
            c[0] = c0;
#pragma unroll
            for (int i = 1; i < QCH; ++i) {
                const int cc = c[i - 1] + step_c;
                const bool wrap = cc >= nchunks;
                c[i] = wrap ? cc - nchunks : cc;
                m[i] = m[i - 1] + step_m + (wrap ? 1 : 0);
            }
        }
    }
    // requests this thread's chunks of the M rows of K elements at src
    // (Whole chunks with vector loads, whatever the row's alignment: this target reads under-aligned
    // vectors, the compiler itself emits them for a 16-byte copy from a 2-byte-aligned address.  The
    // ragged last chunk of a row -- one per row -- is read element by element in a loop of its own
    // and placed into its owner's slot: inlined into every slot, that path tripled the code between
    // the top of the kernel and the first dot product.)
    __device__ __forceinline__ void fetch(const void* src, int M, int K) {
        const int nchunks = (K + 15) >> 4, whole = K >> 4;
        m0 = MR == 1 ? 0 : (int)threadIdx.x / nchunks;
        c0 = (int)threadIdx.x - m0 * nchunks;
        int m[QCH], c[QCH];
        index(nchunks, m, c);
        // (zeros first, loads behind them: a register cleared after a load into it was issued makes
        // the compiler wait for every load in flight, the weight tiles requested ahead included)
#pragma unroll
        for (int i = 0; i < QCH; ++i) __builtin_memset(&raw[i], 0, sizeof(raw[i]));
#pragma unroll
        for (int i = 0; i < QCH; ++i) {
            if (m[i] < M && c[i] < whole)
                __builtin_memcpy(&raw[i], static_cast<const T*>(src) + (size_t)m[i] * K + (size_t)c[i] * 16, sizeof(raw[i]));
        }
        if (K & 15) {
#pragma nounroll
            for (int mm = 0; mm < M; ++mm) {
                const int pidx = mm * nchunks + whole; // (uniform: the tail chunk of row mm, its owner and slot)
                if ((int)threadIdx.x != pidx % THREADS) continue;
                const typename RowLoader<T>::Raw tail =
                    RowLoader<T>::load16_raw(static_cast<const T*>(src) + (size_t)mm * K, whole * 16, K, false);
#pragma unroll
                for (int i = 0; i < QCH; ++i)
                    if (i == pidx / THREADS) raw[i] = tail;
            }
        }
    }
    // row maxima (as float bits, into the zeroed row_max[] in LDS); true if a chunk of this thread
    // holds an Inf or a NaN
    __device__ __forceinline__ bool maxima(int M, int K, uint32_t* row_max) {
        const int nchunks = (K + 15) >> 4;
        int m[QCH], c[QCH];
        index(nchunks, m, c);
        bool bad = false;
#pragma unroll
        for (int i = 0; i < QCH; ++i) {
            if (m[i] < M) {
                uint32_t top = chunk_top_magnitude(raw[i]);
                if (top >= (sizeof(T) == 2 ? 0x7c00u : 0x7f800000u)) {
                    bad = true;
                    float v[16];
                    RowLoader<T>::unpack(raw[i], v);
                    float mx = 0.0f;
#pragma unroll
                    for (int j = 0; j < 16; ++j) mx = fmaxf(mx, fabsf(v[j]));
                    top = __float_as_uint(mx);
                } else if (sizeof(T) == 2) {
                    top = __float_as_uint(half_bits_to_float((uint16_t)top));
                }
                // (non-negative floats order like their bits.  For one row, a shuffle reduction per wave
                // and one atomic per wave instead of 64 on the same address measured slower: 4096 x 14336
                // int8 10.65 -> 10.7 us, int4 6.8 -> 7.2 us)
                atomicMax(&row_max[m[i]], top);
            }
        }
        return bad;
    }
    // scale and 1 / scale of row threadIdx.x (threads below M), by the rule of the mode
    static __device__ __forceinline__ void scales(int M, int mode, const uint32_t* row_max, float* row_scale,
                                                  float* row_inv, float* out_scale) {
        const int t = threadIdx.x;
        if (t < M) {
            const float mx = __uint_as_float(row_max[t]);
            const float sc = mode == RKH_Q_W4A8 ? (mx == 0.0f ? 1.0f : fmaxf(mx / 127.0f, FLT_MIN))
                                                : (mx > 0.0f ? mx / 127.0f : 1.0f);
            row_scale[t] = sc;
            row_inv[t] = 1.0f / sc;
            if (out_scale) out_scale[t] = sc;
        }
    }
    // zeroes the K padding of the staged rows (row-major [M][Kp] at a_lds)
    static __device__ __forceinline__ void zero_padding(int M, int K, int Kp, uint8_t* a_lds) {
        const int nchunks = (K + 15) >> 4, pad = (Kp >> 4) - nchunks;
        for (int idx = threadIdx.x; idx < M * pad; idx += THREADS) {
            const int m = idx / pad, c = nchunks + idx % pad;
            *reinterpret_cast<uint4*>(a_lds + (size_t)m * Kp + (size_t)c * 16) = make_uint4(0, 0, 0, 0);
        }
    }
    // codes into the staged rows (as their two signed digits if DIGITS) and, where dst is given,
    // into the tiled copy the separate quantization launch would have left
    template <bool DIGITS>
    __device__ __forceinline__ void quantize(int M, int K, int Kp, const float* row_inv, uint8_t* a_lds, uint8_t* dst) {
        const int nchunks = (K + 15) >> 4, KB = Kp / 32;
        int m[QCH], c[QCH];
        index(nchunks, m, c);
#pragma unroll
        for (int i = 0; i < QCH; ++i) {
            if (m[i] < M) {
                float v[16];
                RowLoader<T>::unpack(raw[i], v);
                const uint4 packed = quantize16<false>(v, row_inv[m[i]]);
                *reinterpret_cast<uint4*>(a_lds + (size_t)m[i] * Kp + (size_t)c[i] * 16) = DIGITS ? digits16(packed) : packed;
                if (dst) *reinterpret_cast<uint4*>(dst + tiled_chunk_offset(m[i], c[i], KB)) = packed;
            }
        }
    }
};

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
// per wave in flight (10.7), the exact-wait kernel with its first eight loads in four stages between
// the prologue's barriers, the first stage ahead of the row, as the int4 single-row kernel has them
// (10.6: the same, also with the epilogue's scales requested early; twelve / sixteen loads in stages
// 11.4 / spills), 28 instead of 32 columns per workgroup (512 workgroups, two for
// every compute unit, instead of 448 -- 11.85 us; the per-lane addresses this needs cost 0.4 us
// already with 32 columns).
template <int MR, bool W4, int QT, int CW, bool BURST = false, bool BIG = false>
__global__ __launch_bounds__(GEMV_WAVES * 64) __attribute__((amdgpu_waves_per_eu(GEMV_WAVES / 2)))
void gemv_kernel(RK_GEMV_HEAD_PARAMS, rkh_gemm_args g, rkh_quant_args q) {
    RK_GEMV_HEAD_APPLY(g, q);
    RK_TS(0);
    static_assert(CW == 32 || CW == 16 || CW == 8, "columns per workgroup");
    constexpr bool FUSEQ = QT == 1 || QT == 2; // the kernel quantizes the rows itself
    static_assert(QT != 3 || !W4, "int8 rows as given: the exact int8 x int8 product only");
    // Load instructions of a wave in flight.  One row, exact waits: four -- the quantization
    // prologue and the first dot products start after half as many bytes, and nothing is gained
    // by queueing more in front of the memory system (int4 4096 x 4096 4.9 -> 4.1, 4096 x 11008
    // 7.0 -> 6.6, 8192 x 1024 5.1 -> 4.5; int8 2048 x 2048 4.2 -> 3.6, 14336 x 4096 12.8 -> 12.5, the
    // other int8 shapes within 1 %).  Several rows and the burst variant are faster with eight (two
    // rows lose 2 - 9 % with four on most shapes; the burst variant 10.6 -> 11.4 us), and so is one
    // row on 32-column workgroups when it quantizes the row itself and requests the eight in
    // stages (see STAGES below).
    constexpr int UNR = (MR == 1 && !BURST && !(FUSEQ && CW == 32)) ? 4 : GEMV_UNROLL;
    static_assert(!BURST || (MR == 1 && !W4 && CW == 32), "the burst variant serves one int8 row, whole column blocks");
    static_assert(!BIG || (MR >= 4 && !W4), "the larger staging area: four to eight rows, int8 weights");
    constexpr int TPL = 32 / CW;            // k-tiles (int4: super-tiles) covered by one load instruction
    // (padding for the single-row variants of narrow matrices: their look-ahead of UNR loads per wave, and
    // one more step for the activations, runs up to that many load instructions past the end
    // of a chunk, 32 / CW tiles of 32 -- int4: 64 -- staged bytes each)
    constexpr bool ROLLING = MR == 1 && CW < 32; // see the K loop
    // Several rows, int8 weights: the group of loads is kept as two halves, see the K loop.  (Measured
    // per shape against the whole group at a time, fp16 rows, us: 4096 x 14336 two / four rows 11.85 ->
    // 11.7 / 13.85 -> 13.2; 14336 x 4096 16.1 -> 14.9 / 22.9 -> 21.4; 4096 x 4096 within 1 %; int4
    // weights lose with two rows, 8.5 -> 9.3 and 5.35 -> 5.6, and keep the whole group.)
    constexpr bool PINGPONG = MR > 1 && !W4;
    // Several rows on the matrix cores: with dot products every staged row costs a 16-byte LDS read
    // per lane and tile, and a compute unit's LDS serves one such read per 8 clocks while HBM
    // delivers it a tile every ~40 -- from four rows on the LDS, not the memory, sets the pace.
    // A weight tile as a lane holds it IS the first operand of v_mfma_i32_32x32x32_i8 (32 columns x
    // 32 k; the 16-column workgroups' piece of two consecutive tiles is the first operand of
    // v_mfma_i32_16x16x64_i8), and the staged rows are the second one: lane l reads the 16 bytes
    // of row l % CW at its k-half -- one LDS read and one MFMA per tile however many rows.  Rows
    // past MR read row MR - 1 again: column j of the product depends on column j of the second
    // operand only, and those columns are never stored.  (Int4 weights, 32 columns: the eight-row
    // instantiation only -- the four-row one spills with the unpacked operands, so it keeps the dot
    // products and the launcher sends three and four rows of a wide matrix to the eight-row kernel.)
    constexpr bool MATRIX = MR >= (W4 ? GEMV_MFMA_ROWS : GEMV_MFMA_ROWS_I8) && CW >= 16 && !(W4 && CW == 32 && MR < 8);
    constexpr int CREGS = CW == 32 ? 16 : 4;                // accumulator registers of the matrix path
    constexpr int A_PAD = ROLLING ? GEMV_WAVES * (UNR + 1) * TPL * (W4 ? 64 : 32) : 0;
    __shared__ __attribute__((aligned(16))) uint8_t a_lds[gemv_lds_bytes(BIG) + A_PAD];
    __shared__ int red[GEMV_WAVES][MR][CW];
    __shared__ uint32_t row_max[MR];
    __shared__ float row_scale[MR];
    __shared__ float row_inv[MR];
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
    const int kc_max = (gemv_lds_bytes(BIG) / MR) & ~63;
    int acc[MR], acc_lo[MR]; // (int4 weights: the sums of the high and of the low activation digits)
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[m] = acc_lo[m] = 0;
    // matrix path: the 32 x 32 (16 x 16) tile of sums, lane l = row l % CW; int4 weights ride as
    // 16 x code, taken off per K chunk into `ctot` so that no K can wrap the factor
    typename std::conditional<CW == 32, v16i, v4i>::type cacc, ctot;
#pragma unroll
    for (int r = 0; r < CREGS; ++r) cacc[r] = ctot[r] = 0;
    const int mrow = min(lane % (CW < 16 ? 16 : CW), MR - 1);

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
    // The activation rows are requested ahead of a whole batch: loads return in issue order, so
    // behind the weight loads they would arrive with the last of those, and the
    // prologue (and with it the second batch of weight loads) would start only
    // then.  Fetched first they are back after one L2 round trip and the whole
    // quantization runs under the weight loads' latency.  (BURST: the other way round, see above.)
    v4i wpre[UNR];
    using QT_T = typename std::conditional<QT == 2, float, uint16_t>::type;
    FusedRows<QT_T, MR, BIG> rows;
    // A batch of eight tiles is requested a quarter at a time, between the prologue's barriers.
    // Requested all at once the sixteen waves of a compute unit ask for 256 KB, more than its memory
    // path holds in flight: a wave's later requests wait at issue until earlier data has arrived, and
    // the prologue's first barrier, which every wave reaches only behind its last request, came 1.9 us
    // later than with four tiles (in-kernel time stamps, two rows, 4096 x 14336 int4: 4.8 against 3.0
    // us after the start).  In stages, fp16 rows, us: 4096 x 14336 int8 two / four / eight rows 12.0 ->
    // 11.05 / 12.1 -> 11.55 / 15.4 -> 14.0, int4 8.4 -> 7.55 / 10.8 -> 9.2 / 13.5 -> 12.5; 4096 x 4096 int8
    // 5.77 -> 5.25 / 6.8 -> 5.8 / 8.8 -> 7.4.  One row on 32-column int4 workgroups (eight tiles are all
    // of K = 4096 there): 6.75 -> 6.5 us, and 6.2 with the first quarter requested ahead of the row
    // (two tiles delay the row by little and are on their way a microsecond earlier; with several
    // rows that order loses 3 - 8 %).  Unequal stages (4-2-1-1, 3-3-1-1, 1-3-2-2, 4-4-0-0) measured
    // 6.3 - 6.7 against 6.2, and the single-row kernels of narrow matrices (four tiles in a rolling
    // window) lose 2 - 5 % with stages.
    constexpr int STAGES = (FUSEQ && !BURST && UNR == GEMV_UNROLL) ? 4 : 1;
    static_assert(UNR % STAGES == 0, "whole tiles per stage");
    const int pre_tiles = (W4 ? Kp >> 6 : Kp >> 5) / TPL;
    auto prefetch_stage = [&](int stage) {
#pragma unroll
        for (int u = 0; u < UNR / STAGES; ++u)
            wpre[stage * (UNR / STAGES) + u] = load_tile(wave + (stage * (UNR / STAGES) + u) * GEMV_WAVES, pre_tiles, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    (void)prefetch_stage;
    if constexpr (FUSEQ) {
        constexpr bool W_FIRST = BURST || (STAGES > 1 && MR == 1);
        if constexpr (W_FIRST) prefetch_stage(0);
        rows.fetch(q.src, g.M, g.K);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!W_FIRST) prefetch_stage(0);
        RK_TS(4);
    }
    // The epilogue's column scale (and, for the int4 dot products, the column sum) of the output
    // element this thread may write: requested now, unconditionally (counted by the compiler, so no
    // wait below covers more than it has to), instead of as a round trip at the end of the kernel.
    // 32-column workgroups only (4096 x 14336 int4, one row: 6.22 -> 6.12 us; int8, two / four rows
    // 11.1 -> 11.0 / 11.6 -> 11.4); the 16- and 8-column kernels of narrow matrices lose 3 - 6 % with it.
    constexpr bool EPI_EARLY = FUSEQ && !BURST && CW == 32;
    float early_ws = 1.0f;
    int early_colsum = 0;
    if constexpr (EPI_EARLY) {
        const int n_e = block_first_col(p, g.interleave_F) + col0 + (int)threadIdx.x % CW;
        const int n_c = n_e < g.N ? n_e : 0;
        if (g.w_scale) early_ws = g.w_scale[n_c];            // (uniform)
        if constexpr (W4 && !MATRIX) early_colsum = g.w_colsum[n_c];
        __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (FUSEQ) {
        if ((int)threadIdx.x < MR) row_max[threadIdx.x] = 0u;
        __syncthreads();
        RK_TS(5);
        if constexpr (STAGES >= 2) prefetch_stage(1);
        const bool bad = rows.maxima(g.M, g.K, row_max);
        __syncthreads();
        if constexpr (STAGES >= 4) prefetch_stage(2);
        rows.scales(g.M, q.mode, row_max, row_scale, row_inv, first_wg ? q.scale : nullptr);
        if (first_wg && bad && q.mode == RKH_Q_W4A8 && q.bad_flag) atomicOr(q.bad_flag, 1);
        rows.zero_padding(g.M, g.K, Kp, a_lds);
        __syncthreads();
        if constexpr (STAGES >= 4) prefetch_stage(3);
        rows.template quantize<W4 && !MATRIX>(g.M, g.K, Kp, row_inv, a_lds, first_wg ? q.dst : nullptr);
        // a_scale of the epilogue comes from LDS in this path
        RK_TS(1);
    }

    for (int kc0 = 0; kc0 < Kp; kc0 += kc_max) {
        const int kc = min(kc_max, Kp - kc0);
        // stage activations: row-major [MR][kc] in LDS from the tiled buffer
        const int chunks = kc >> 4;
        if (kc0) __syncthreads();
        if constexpr (QT == 0) {
            // (rows fastest: the MR rows of a chunk are MR adjacent 16-byte slots of a tile, so a wave's loads
            // cover whole lines; chunk by chunk along a row, every lane fetched a line of its own for 16 bytes)
            for (int idx = threadIdx.x; idx < MR * chunks; idx += GEMV_WAVES * 64) {
                const int c = idx / MR, m = idx - c * MR;
                const uint4 v = *reinterpret_cast<const uint4*>(g.A + tiled_chunk_offset(m, (kc0 >> 4) + c, KB));
                *reinterpret_cast<uint4*>(a_lds + (size_t)m * kc + (size_t)c * 16) = (W4 && !MATRIX) ? digits16(v) : v;
            }
        } else if constexpr (QT == 3) {
            // int8 rows as the caller holds them (row-major, any alignment, K not padded).  The tiled
            // copy a launch of the re-tiling kernel would have left is written on the side, every
            // workgroup storing an equal contiguous share of its chunks: when the first
            // workgroup wrote all of it (write-through stores between its loads), that workgroup
            // finished 2 - 4 us after the others and the launch with it -- four rows took 7.4 us
            // where one took 5.2 (4096 x 4096) and 15.1 where one took 10.0 (11008 x 4096).
            const unsigned copy_share = ((unsigned)g.M * (unsigned)(Kp >> 4) + gridDim.x - 1) / gridDim.x;
            const unsigned copy_lo = blockIdx.x * copy_share; // this workgroup's chunks of the tiled copy
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
                    if (q.dst && (unsigned)(m * (Kp >> 4) + gc) - copy_lo < copy_share)
                        *reinterpret_cast<uint4*>(q.dst + tiled_chunk_offset(m, gc, KB)) = v;
                }
                *reinterpret_cast<uint4*>(a_lds + (size_t)m * kc + (size_t)c * 16) = v;
            }
        }
        __syncthreads();
        RK_TS(6);

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
                if constexpr (MATRIX) {
                    auto mma = [&](const v4i& wop, const v4i& aop) {
                        if constexpr (CW == 32) cacc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wop, aop, cacc, 0, 0, 0);
                        else cacc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wop, aop, cacc, 0, 0, 0);
                    };
                    if constexpr (!W4) {
                        mma(wu, *reinterpret_cast<const v4i*>(a_lds + (size_t)mrow * kc + (size_t)(tt * 2 + half) * 16));
                    } else {
                        // (a super-tile: the lane's 8 bytes of each 32-deep half, unpacked as 16 x code)
                        const v4i lo = v4i{(wu.x << 4) & (int)0xF0F0F0F0, wu.x & (int)0xF0F0F0F0,
                                           (wu.y << 4) & (int)0xF0F0F0F0, wu.y & (int)0xF0F0F0F0};
                        const v4i hi = v4i{(wu.z << 4) & (int)0xF0F0F0F0, wu.z & (int)0xF0F0F0F0,
                                           (wu.w << 4) & (int)0xF0F0F0F0, wu.w & (int)0xF0F0F0F0};
                        mma(lo, *reinterpret_cast<const v4i*>(a_lds + (size_t)mrow * kc + (size_t)((tt * 2 + 0) * 2 + half) * 16));
                        mma(hi, *reinterpret_cast<const v4i*>(a_lds + (size_t)mrow * kc + (size_t)((tt * 2 + 1) * 2 + half) * 16));
                    }
                } else if constexpr (!W4) {
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
            if constexpr (PINGPONG) {
                // Several rows: the group is kept as two halves.  While one half is multiplied
                // with the rows (MR LDS reads and 4 * MR dot products per tile) the other half is
                // in flight, and a half's registers are asked for again as soon as it is used --
                // the loads of a wave never drain, in the registers the whole group took before.
                constexpr int H = UNR / 2;
                v4i wa[H], wb[H];
#pragma unroll
                for (int u = 0; u < H; ++u) {
                    if constexpr (FUSEQ) {
                        wa[u] = wpre[u];
                        wb[u] = wpre[H + u];
                    } else {
                        wa[u] = load_unit(tb + u * GEMV_WAVES);
                    }
                }
                if constexpr (!FUSEQ) {
#pragma unroll
                    for (int u = 0; u < H; ++u) wb[u] = load_unit(tb + (H + u) * GEMV_WAVES);
                }
                for (; tb < tiles; tb += GEMV_WAVES * UNR) {
#pragma unroll
                    for (int u = 0; u < H; ++u)
                        if (tb + u * GEMV_WAVES < tiles) consume_unit(wa[u], tb + u * GEMV_WAVES);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int u = 0; u < H; ++u) wa[u] = load_unit(tb + (UNR + u) * GEMV_WAVES); // (past the end: zeros, no access)
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int u = 0; u < H; ++u)
                        if (tb + (H + u) * GEMV_WAVES < tiles) consume_unit(wb[u], tb + (H + u) * GEMV_WAVES);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int u = 0; u < H; ++u) wb[u] = load_unit(tb + (UNR + H + u) * GEMV_WAVES);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
            // (int4 tiles on the matrix cores take two LDS reads and eight unpacked registers each: left
            // to itself the scheduler gathers the reads of a whole group up front and spills)
            constexpr bool FENCED = MATRIX && W4;
            if constexpr (FUSEQ) {
#pragma unroll
                for (int u = 0; u < UNR; ++u) {
                    if (tb + u * GEMV_WAVES < tiles) consume_unit(wpre[u], tb + u * GEMV_WAVES);
                    if constexpr (FENCED) __builtin_amdgcn_sched_barrier(0);
                }
                tb += GEMV_WAVES * UNR;
            }
            for (; tb < tiles; tb += GEMV_WAVES * UNR) {
                v4i w[UNR];
#pragma unroll
                for (int u = 0; u < UNR; ++u) w[u] = load_unit(tb + u * GEMV_WAVES);
                if constexpr (FENCED) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < UNR; ++u) {
                    if (tb + u * GEMV_WAVES < tiles) consume_unit(w[u], tb + u * GEMV_WAVES);
                    if constexpr (FENCED) __builtin_amdgcn_sched_barrier(0);
                }
            }
            }
        }
        if constexpr (MATRIX && W4 && !FUSEQ) {
            // (a wave's share of a chunk is at most 512 k per row: 16 x code sums stay far inside int32;
            // the fused path has a single chunk and shifts in the epilogue)
#pragma unroll
            for (int r = 0; r < CREGS; ++r) {
                ctot[r] += cacc[r] >> 4;
                cacc[r] = 0;
            }
        }
    }

    RK_TS(2);
    if constexpr (MATRIX) {
        // lane l holds row l % CW of the tile: 16 columns 8 * (r / 4) + 4 * (l / 32) + r % 4 of 32, or 4
        // columns 4 * (l / 16) + r of 16; the MFMA has already summed over the lanes' k-halves
        if (lane % CW < MR) {
#pragma unroll
            for (int r = 0; r < CREGS; ++r) {
                const int col = CW == 32 ? 8 * (r / 4) + 4 * (lane / 32) + r % 4 : 4 * (lane / 16) + r;
                red[wave][lane % CW][col] = !W4 ? cacc[r] : FUSEQ ? cacc[r] >> 4 : ctot[r];
            }
        }
    } else {
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        int v = W4 ? 16 * acc[m] + acc_lo[m] : acc[m];
        v += __shfl_xor(v, 32);
        if (CW <= 16) v += __shfl_xor(v, 16);
        if (CW <= 8) v += __shfl_xor(v, 8);
        if (lane < CW) red[wave][m][lane] = v;
    }
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
        if (W4 && !MATRIX && n < g.N) sum += 8 * (EPI_EARLY ? early_colsum : g.w_colsum[n]); // (the constant term of the digit split)
        if (n < g.N)
            store_out(g.C, g.epilogue, (size_t)m * g.ldc + n, sum,
                      FUSEQ ? row_scale[m] : (g.a_scale ? g.a_scale[m] : 1.0f),
                      EPI_EARLY ? early_ws : g.w_scale ? g.w_scale[n] : 1.0f);
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
    __shared__ float row_inv[MR];
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
    auto load_pair = [&](int u, int tb, int tiles, int tile0) { // tile u of the group: its gate and its up block
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const int tt = tb + u * GEMV_WAVES;
            const unsigned off = tt < tiles ? (unsigned)(b * block_bytes) + (unsigned)(tile0 + tt) * 1024u + (unsigned)lane * 16u
                                            : 0xFFFFFFF0u;
            w[b][u] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, (int)off, 0, 2 /* streaming */));
        }
    };
    auto load_group = [&](int tb, int tiles, int tile0) {
#pragma unroll
        for (int u = 0; u < GEMV_SWIGLU_UNROLL; ++u) load_pair(u, tb, tiles, tile0);
    };

    if constexpr (QT != 0) { // (the fused path has a single K chunk: rows fit the staging area)
        using T = typename std::conditional<QT == 2, float, uint16_t>::type;
        const bool first_wg = blockIdx.x == 0;
        FusedRows<T, MR, false> rows;
        // (the first group of weight tiles a quarter at a time between the barriers, as in gemv_kernel:
        // a whole 4096 -> 14336 -> 4096 FFN of one / two rows 20.55 -> 19.9 / 24.4 -> 23.3 us; the first
        // quarter ahead of the row changes nothing here)
        static_assert(GEMV_SWIGLU_UNROLL == 4, "one tile pair per stage");
        const int pre_tiles = W4 ? Kp >> 6 : Kp >> 5;
        rows.fetch(q.src, g.M, g.K);
        __builtin_amdgcn_sched_barrier(0);
        load_pair(0, wave, pre_tiles, 0);
        __builtin_amdgcn_sched_barrier(0);
        if ((int)threadIdx.x < MR) row_max[threadIdx.x] = 0u;
        __syncthreads();
        load_pair(1, wave, pre_tiles, 0);
        __builtin_amdgcn_sched_barrier(0);
        const bool bad = rows.maxima(g.M, g.K, row_max);
        __syncthreads();
        load_pair(2, wave, pre_tiles, 0);
        __builtin_amdgcn_sched_barrier(0);
        rows.scales(g.M, q.mode, row_max, row_scale, row_inv, first_wg ? q.scale : nullptr);
        if (first_wg && bad && q.mode == RKH_Q_W4A8 && q.bad_flag) atomicOr(q.bad_flag, 1);
        rows.zero_padding(g.M, g.K, Kp, a_lds);
        __syncthreads();
        load_pair(3, wave, pre_tiles, 0);
        __builtin_amdgcn_sched_barrier(0);
        rows.template quantize<W4>(g.M, g.K, Kp, row_inv, a_lds, first_wg ? q.dst : nullptr);
    }

    for (int kc0 = 0; kc0 < Kp; kc0 += kc_max) {
        const int kc = min(kc_max, Kp - kc0);
        const int chunks = kc >> 4;
        if (kc0) __syncthreads();
        if constexpr (QT == 0) {
            // (rows fastest: the MR rows of a chunk are MR adjacent 16-byte slots of a tile, so a wave's loads
            // cover whole lines; chunk by chunk along a row, every lane fetched a line of its own for 16 bytes)
            for (int idx = threadIdx.x; idx < MR * chunks; idx += GEMV_WAVES * 64) {
                const int c = idx / MR, m = idx - c * MR;
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
    // Beyond 128 blocks the 16-column workgroups outnumber the compute units, and several rows take whole
    // blocks as well.  Every workgroup stages (and, fused, quantizes) all the rows, so with eight of them the
    // prologues of 16-column workgroups move as many bytes as the weights: fp16 rows, us, five / eight rows,
    // int8 5120 x 5120 11.0 / 14.3 -> 10.2 / 11.8, 6144 x 8192 13.6 / 17.45 -> 13.0 / 14.9, 8192 x 8192 16.5 / 21.55 ->
    // 16.6 / 19.5, 4096 x 8192 8.9 / 10.95 -> 8.8 / 10.2, 4096 x 4160 8.3 / 10.45 -> 7.8 / 9.2, 13824 x 5120 (rows
    // in chunks behind a quantization launch) 27.8 -> 23.1; int4 4096 x 8192 8.4 / 10.7 -> 6.8 / 8.3, 4096 x 4160
    // 7.8 / 10.3 -> 6.4 / 7.8, 2048 x 8192 6.2 / 7.2 -> 5.5 / 6.0.  (128 blocks: half the compute units would
    // idle, int8 8192 x 4096 eight rows 14.6 -> 16.2.)
    // While K <= 5120 the same holds for two to four rows on int8 weights (4096 x 8192 two / three / four rows
    // 8.05 / 8.3 / 8.6 -> 7.6 / 7.8 / 8.3, 4096 x 5120 7.1 / 7.5 / 8.2 -> 6.7 / 7.0 / 7.5, 4096 x 4160 6.85 / 8.1 (two /
    // four) -> 6.5 / 7.3, 5120 x 5120 8.5 / 9.2 / 9.85 -> 7.8 / 8.35 / 8.75; K = 8192: 12.3 -> 13.4) and for one and
    // two rows on int4 weights, whose 32-column instantiations request their first weights in stages and
    // their scales early (one row 4096 x 8192 5.4 -> 4.65, 4096 x 5120 5.1 -> 4.2, 4096 x 4160 4.7 -> 4.1,
    // 5120 x 5120 6.15 -> 5.9, two rows 4096 x 4608 6.6 -> 5.1, 4096 x 8192 7.1 -> 5.4; K = 8192: one row
    // 7.3 -> 8.1).  One int8 row keeps 16 columns (4096 x 8192 7.4 -> 8.5, 4096 x 4160 6.0 -> 7.0).
    const bool short_k = rkh_align_up(g.K, RKH_K_ALIGN) <= 5120;
    // int8 rows as given (no quantization, but every workgroup still stages all the rows): the same from two
    // rows on while K <= 5120 -- 4096 x 8192 two / four / eight rows 8.3 / 8.4 / 9.3 -> 7.5 / 7.9 / 8.3, 4096 x 5120
    // 7.05 / 7.4 / 8.35 -> 6.2 / 6.4 / 6.95; 8192 x 8192 12.75 / 13.1 / 14.6 -> 13.4 / 13.8 / 14.8 -- and up to 64 blocks
    // from four rows on, from two while K <= 5120: 4096 x 2048 two / four / eight rows 4.8 / 5.35 / 6.35 ->
    // 4.45 / 4.7 / 5.6, 8192 x 2048 four / eight rows 7.1 / 9.1 -> 6.7 / 7.7.
    const bool raw_rows = fuse && fuse->in_dtype == RKH_I8;
    const bool several_wide = pblocks > 128 && (raw_rows ? MR >= 2 && short_k
                                                         : MR == 8 || (short_k && (g.w_int4 ? MR <= 2 : MR >= 2)));
    // Up to 64 blocks the same trade is between 8 and 16 columns: five to eight rows take 16 (fp16 rows, us,
    // five / eight rows, both weight formats alike: 4096 x 2048 7.0 / 8.5 -> 5.7 / 7.2, 4096 x 1024 6.9 / 8.3 ->
    // 5.65 / 7.2, int8 8192 x 2048 11.1 / 14.2 -> 10.5 / 13.4, 14336 x 2048 20.0 -> 18.0), four rows on int4 weights
    // (4096 x 2048 5.85 -> 5.5, 8192 x 2048 8.5 -> 7.5, 14336 x 2048 15.9 -> 13.3) and, while K <= 5120, four and
    // two rows on int8 weights (4096 x 2048 5.95 / 5.05 -> 5.55 / 4.7; K = 8192: 8.4 / 6.4 -> 9.0 / 7.1).  One row
    // keeps 8 (4096 x 2048 int8 3.9 -> 4.6), and so do two int4 rows (4.65 -> 4.85).
    const bool several_narrow = raw_rows ? MR >= 4 || (MR == 2 && short_k)
                                         : MR == 8 || (MR == 4 && (g.w_int4 || short_k)) || (MR == 2 && !g.w_int4 && short_k);
    const int cw = want == 8 || want == 16 || want == 32 ? want
                   : pblocks <= 64 && !several_narrow    ? 8
                   : (pblocks <= 256 && !several_wide) || halves ? 16
                                                         : 32;
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
#define RK_GEMV_CW(W4, QT, BIG)                                                                \
    do {                                                                                       \
        if (cw == 8) hipLaunchKernelGGL((gemv_kernel<MR, W4, QT, 8, false, BIG>), grid, block, 0, st, RK_GEMV_HEAD(g, q), g, q);        \
        else if (cw == 16) hipLaunchKernelGGL((gemv_kernel<MR, W4, QT, 16, false, BIG>), grid, block, 0, st, RK_GEMV_HEAD(g, q), g, q); \
        else if constexpr (!(MR == 1 && !W4)) /* (one int8 row, 32 columns: the burst variant above) */   \
            hipLaunchKernelGGL((gemv_kernel<MR, W4, QT, 32, false, BIG>), grid, block, 0, st, RK_GEMV_HEAD(g, q), g, q);               \
    } while (0)
    // (the larger staging area where the rows do not fit the small one, see gemv_lds_bytes)
    const bool big = gemv_big_applies(MR, g.w_int4 != 0, (long)rkh_align_up(g.K, RKH_K_ALIGN));
#define RK_GEMV(W4, QT)                                                                        \
    do {                                                                                       \
        if constexpr (MR >= 4 && !W4) {                                                        \
            if (big) { RK_GEMV_CW(W4, QT, true); break; }                                      \
        }                                                                                      \
        RK_GEMV_CW(W4, QT, false);                                                             \
    } while (0)
    if (g.w_int4) {
        if (qt == 0) RK_GEMV(true, 0); else if (qt == 1) RK_GEMV(true, 1); else RK_GEMV(true, 2);
    } else {
        if (qt == 0) RK_GEMV(false, 0); else if (qt == 1) RK_GEMV(false, 1); else if (qt == 2) RK_GEMV(false, 2);
        else RK_GEMV(false, 3);
    }
#undef RK_GEMV
#undef RK_GEMV_CW
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

// gate/up + SwiGLU of up to four rows as a GEMV (columns gate/up interleaved in blocks of 32,
// F a multiple of 32, both blocks of a workgroup within the 4 GiB reach of its descriptor).
// Measured for 4096 -> 2 x 14336 int4 against 14.9 us on the MFMA kernel: 12.8 us for one row,
// 13.8 for two, 15.1 for four, 20.1 for eight.  Three and four rows: the kernel as such is no
// faster than the MFMA kernel, but it quantizes the rows itself and saves that launch -- a whole
// 4096 -> 14336 -> 4096 FFN of three / four rows 31.9 / 32.0 -> 28.9 / 30.35 us (33.6 / 34.8 against
// 34.6 / 34.5 before its first weight tiles were requested in stages).
bool gemv_swiglu_applies(const rkh_gemm_args& g) {
    return !g.blk_expert && g.w_int4 && g.M <= 4 && g.epilogue == RKH_EPI_SWIGLU && g.interleave_F >= 32 &&
           g.interleave_F % 32 == 0 && g.N == 2 * g.interleave_F && g.K <= (1 << 24);
}

int dispatch_gemv_swiglu(hipStream_t st, const rkh_gemm_args& g, const rkh_quant_args* fuse) {
    if (g.M == 1) return launch_gemv_swiglu<1>(st, g, fuse);
    if (g.M == 2) return launch_gemv_swiglu<2>(st, g, fuse);
    return launch_gemv_swiglu<4>(st, g, fuse);
}

// An int4 matrix of more than 256 column blocks whose rows fit the staging area eight at a time: from
// three rows on the eight-row instantiation, the only 32-column int4 one whose products go through the
// matrix cores (the four-row one would spill).  4096 x 14336, fp16 rows, us, four-row dot products /
// streaming MFMA kernel -> eight-row kernel: three rows 9.5 -> 8.65, four 10.3 -> 9.3, five 11.3 -> 9.95,
// six 11.3 -> 10.85; eight rows stay on the streaming kernel (11.5 against 12.3), two on the dot products
// (7.7 against 8.0).
constexpr int GEMV_W4_WIDE_ROWS = 7; // (seven: a tie)
static bool w4_wide_eight(const rkh_gemm_args& g) {
    return (g.N + 31) / 32 > 256 && g.w_int4 && g.epilogue != RKH_EPI_SWIGLU &&
           rkh_align_up(g.K, RKH_K_ALIGN) * 8 <= (size_t)GEMV_LDS_BYTES;
}
// Rows of the kernel instantiation that takes the M rows of g.
int gemv_mr(const rkh_gemm_args& g) {
    if (g.M >= 3 && w4_wide_eight(g)) return 8;
    // The same beyond 128 column blocks, where the eight-row kernel takes whole blocks per workgroup (see
    // launch_gemv): 4096 x 8192 three / four rows 7.55 / 8.3 -> 5.95 / 6.45 us, 4096 x 5120 7.3 / 7.9 -> 5.8 / 6.3,
    // 4096 x 4608 four rows 7.8 -> 6.3, 2048 x 8192 6.3 / 6.4 -> 5.25 / 5.4.  (Two rows: the two-row dot products
    // on whole blocks are ahead of it there, 4096 x 4608 5.1 against 5.35, 4096 x 8192 5.4 against 5.6 -- and
    // behind it on a matrix of more than 256 blocks it would be: 4096 x 14336 7.7 against 8.0 for the eight-row
    // kernel, so two rows stay on the dot products everywhere.)
    if (g.M >= 3 && (g.N + 31) / 32 > 128 && g.w_int4 && g.epilogue != RKH_EPI_SWIGLU &&
        rkh_align_up(g.K, RKH_K_ALIGN) * 8 <= (size_t)GEMV_LDS_BYTES)
        return 8;
    return g.M == 1 ? 1 : g.M == 2 ? 2 : g.M <= 4 ? 4 : 8;
}

int dispatch_gemv(hipStream_t st, const rkh_gemm_args& g, const rkh_quant_args* fuse) {
    const int mr = gemv_mr(g);
    if (mr == 1) return launch_gemv<1>(st, g, fuse);
    if (mr == 2) return launch_gemv<2>(st, g, fuse);
    if (mr == 4) return launch_gemv<4>(st, g, fuse);
    return launch_gemv<8>(st, g, fuse);
}

// The decode path can quantize inside the GEMV when the rows fit the kernel's
// LDS staging and per-thread register cache.
// Whether the streaming MFMA kernel can take this dense GEMM at all (int4 codes ride as 16 * code).
bool dense_stream_fits(const rkh_gemm_args& g) { return !g.w_int4 || g.K <= 131072; }

// Most rows the decode kernels take for this matrix; the rows beyond go to the streaming MFMA kernel as
// one 32-row block behind a quantization launch.  Eight on int8 weights: with the products of five to
// eight rows on the matrix cores the decode kernel is ahead (4096 x 14336 12.6 - 14.7 us against 16.3,
// 4096 x 11008 12.2 - 14.1 against 15.3).  On int4 weights: seven on a wide matrix (more than 256 column
// blocks) whose rows fit the staging area eight at a time (the eight-row kernel, see gemv_mr); eight on
// a narrower one with such rows; otherwise four or two, see below.  (The four-row dot products on a wide
// matrix took 15.5 - 19.3 us for five to eight rows of 4096 x 11008 / 14336 against 12.3 - 12.9 streamed.)
// RK_NPU_HIP_GEMV_MAX_ROWS = 1..8 lowers the limit (tuning aid).
int gemv_max_rows(const rkh_gemm_args& g) {
    static const int rows = [] {
        const char* e = getenv("RK_NPU_HIP_GEMV_MAX_ROWS");
        const int v = e ? atoi(e) : 8;
        return v >= 1 && v <= 8 ? v : 8;
    }();
    const bool wide = (g.N + 31) / 32 > 256;
    if (w4_wide_eight(g)) return min(rows, GEMV_W4_WIDE_ROWS);
    if (g.w_int4 && g.epilogue != RKH_EPI_SWIGLU && dense_stream_fits(g)) {
        // int4 rows that do not fit the staging area at once (the kernel then walks K in chunks behind a
        // quantization launch): the streaming kernel behind the same launch is faster from five rows on --
        // K > 4096, eight-row instantiation (fp16 rows, weights from HBM, us: 14336 x 4096 18.1 -> 15.5,
        // 11008 x 4096 15.2 -> 13.0, 8192 x 8192 15.7 -> 12.05, 6144 x 8192 13.5 -> 10.6, 5120 x 5120 12.5 -> 9.7,
        // 20000 x 2048 28.0 -> 20.1, 28672 x 8192 42.4 -> 30.1) -- and from three rows on for K > 16384
        // (20000 x 2048 22.2 -> 20.2, 28672 x 8192 33.5 -> 29.8; between 8192 and 16384 the four-row kernel
        // with its chunks keeps up: 14336 x 4096 14.7 against 15.4, 11008 x 4096 12.95 both).  A wide matrix
        // whose K is beyond the eight-row instantiation's reach (K > 4096) does the same from three rows on,
        // although four rows would fit: 5120 x 11008 three / four rows 12.3 / 13.1 -> 11.7 / 11.8, 8192 x 14336
        // 16.8 / 18.6 -> 16.3, 8192 x 28672 30.3 / 33.0 -> 23.9, 11008 x 11008 23.4 -> 17.2.  Two rows stay on
        // the dot products (8192 x 14336 12.5 against 16.3) unless K > 16384 on a matrix of more than 4096
        // columns (20000 x 8192 28.3 -> 23.1, 28672 x 8192 37.3 -> 29.8, 17000 x 14336 34.9 -> 30.4; a tie at
        // 4096 columns, and at 2048 the streaming kernel has too few workgroups: 20000 x 2048 18.1 against
        // 20.0), and three and four rows on a narrower matrix that fits (6144 x 4096 6.1 / 6.6 against 10.1,
        // 8192 x 8192 10.3 / 12.0 against 12.0).  On int8 weights the decode kernel stays ahead or within
        // 6 % (14336 x 4096 five to eight rows 21.4 against 25.9 us, 13824 x 5120 27.8 against 26.2, 28672 x 8192
        // 55.4 against 54.5; int8 rows as given 19.6 against 23.0).
        const size_t kp = rkh_align_up(g.K, RKH_K_ALIGN);
        if (kp * 2 > (size_t)GEMV_LDS_BYTES && g.N > 4096) return 1;
        if (kp * 4 > 2 * (size_t)GEMV_LDS_BYTES || wide) return min(rows, 2);
        if (kp * 8 > (size_t)GEMV_LDS_BYTES) return min(rows, 4);
    }
    return rows;
}

bool gemv_can_fuse(const rkh_quant_args& q, const rkh_gemm_args& g, bool swiglu = false) {
    if (g.w_int4 && !g.w_colsum) return false;
    if (g.blk_expert || g.M > gemv_max_rows(g) || (g.epilogue == RKH_EPI_SWIGLU) != swiglu || q.src_is_host) return false;
    // int8 rows as given (the exact int8 x int8 product): staged by the kernel in K chunks, any K
    if (q.in_dtype == RKH_I8) return q.mode == RKH_Q_COPY_I8 && !g.w_int4 && !swiglu;
    if (q.mode != RKH_Q_W8_DYNAMIC && q.mode != RKH_Q_W4A8) return false;
    if (q.in_dtype != RKH_F16 && q.in_dtype != RKH_F32) return false;
    const int mr = gemv_mr(g);
    const long kp = (long)rkh_align_up(g.K, RKH_K_ALIGN);
    const bool big = !swiglu && gemv_big_applies(mr, g.w_int4 != 0, kp); // (the SwiGLU kernel keeps the small area)
    if (kp * mr > gemv_lds_bytes(big)) return false;
    const long chunks = (long)g.M * ((g.K + 15) / 16);
    return chunks <= (long)gemv_qchunks(big, q.in_dtype == RKH_F16 ? 2 : 4) * GEMV_WAVES * 64;
}

} // namespace

namespace rkk {
bool gemv_swiglu_applies(const rkh_gemm_args& g) { return ::gemv_swiglu_applies(g); }
int dispatch_gemv_swiglu(hipStream_t st, const rkh_gemm_args& g, const rkh_quant_args* fuse) { return ::dispatch_gemv_swiglu(st, g, fuse); }
int dispatch_gemv(hipStream_t st, const rkh_gemm_args& g, const rkh_quant_args* fuse) { return ::dispatch_gemv(st, g, fuse); }
bool dense_stream_fits(const rkh_gemm_args& g) { return ::dense_stream_fits(g); }
int gemv_max_rows(const rkh_gemm_args& g) { return ::gemv_max_rows(g); }
bool gemv_can_fuse(const rkh_quant_args& q, const rkh_gemm_args& g, bool swiglu) { return ::gemv_can_fuse(q, g, swiglu); }
#ifdef RK_DEBUG_TS
void set_ts_gemv(unsigned long long* p) { (void)hipMemcpyToSymbol(HIP_SYMBOL(rk_dbg_ts), &p, sizeof(p)); }
#endif
} // namespace rkk
