// gemm_stream_kernel: 32 (sorted) rows x 256 columns, operands straight to registers -- the
// grouped GEMMs of the MoE layer and dense GEMMs of 9..128 rows -- and its launcher.  Bound by HBM.
#include "rk_kernels_tile.h"

namespace {

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
template <int EPI, int KS, bool W4, bool BAL = false, int TN = 2, int TM = 1>
__global__ __launch_bounds__(BAL ? 512 : 256) void gemm_stream_kernel(RK_GEMM_HEAD_PARAMS, int mblocks, int nblocks,
                                                                      rkh_gemm_args g) {
    RK_GEMM_HEAD_APPLY(g);
    constexpr int WAVES = BAL ? 8 : 4;
    // TM: 32-row blocks per wave (`mblocks` counts units of TM row blocks).  One in every launch of this
    // library.  Two -- a weight tile in registers multiplied with both blocks' activation tiles, tiles
    // of 64 x 128 with K split over two waves -- served dense int8 GEMMs of a few hundred rows until
    // the LDS-ring kernel got tiles of that shape: four waves that each fetch their own operands pull
    // 1 MB per tile through the compute unit, the ring's eight waves 768 KB, and 4096 x 4096 at 512 rows
    // took 24.5 us here against 22.1 there.
    static_assert(TM == 1 || (TM == 2 && !BAL && TN == 2 && EPI != RKH_EPI_SWIGLU), "two row blocks per wave: dense launches");
    // TN: 32-column blocks per wave.  Two; one for small launches whose K is split over the waves
    // (32-column tiles: twice the workgroups where 64-column tiles leave most compute units idle).
    static_assert(TN == 2 || (TN == 1 && KS > 1 && !BAL && EPI != RKH_EPI_SWIGLU), "one column block per wave: small K-split launches");
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
    // (two row blocks per wave: four as well -- six and eight steps measured the same or slower)
    constexpr int RING = KSPLIT ? 4 : BAL ? 2 : 4;
    constexpr int AT = W4 ? 2 : 1;   // activation tiles per step
    constexpr int LPS = AT * TM + TN; // loads per step: TM activation tiles (int4: pairs), TN weight tiles
    static_assert((RING - 1) * LPS <= 63, "vmcnt field");
    constexpr int STAGE_BYTES = WAVES * 32 * (32 * 4 + 8);
    constexpr int XCH_BYTES = KSPLIT ? CG * (KS - 1) * TM * TN * 16 * 64 * 4 : 0;
    __shared__ __attribute__((aligned(16))) uint8_t stage_raw[STAGE_BYTES + XCH_BYTES];

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(wave_id());
    // steps over K: k-tiles (a multiple of 8) or, for int4 weights, super-tiles (a multiple of 4): RING divides both
    const int KB = (int)rkh_align_up(g.K, RKH_K_ALIGN) / (32 * AT);

    [[maybe_unused]] constexpr int TSB = EPI == RKH_EPI_SWIGLU ? 4 : 0; // (debug stamps: the SwiGLU launch keeps its own slots)
    RK_TS(TSB + 0);
    // Grouped: the block -> expert table (up to 64 row blocks, one entry per lane) is requested
    // together with the number of live blocks, so that a wave knows its unit's expert one round trip
    // after its start: read entry by entry, the expert waited for the block count and the first
    // weight tile for the expert -- three dependent round trips ahead of the first data (3.7 us from
    // a wave's start in the MoE layer of 256 tokens, against 2.6 us in a dense launch).  Entries of
    // blocks that are not live hold whatever the last call left; they are never used.
    int expert_of_lane = 0;
    const bool table_in_lanes = g.blk_expert && mblocks <= 64;
    if (table_in_lanes) expert_of_lane = g.blk_expert[min(lane, mblocks - 1)];
    // dense use (no block -> expert table): one weight matrix, every row block live
    const int live_blocks = g.blk_expert ? g.num_blocks[0] : mblocks;

    // One unit of work of a wave: row block mblk x the column pair that starts at column block
    // pair_pb0 (BAL) or the wave's pair of column tile nblk (otherwise).
    auto run_unit = [&](int mblk, int nblk, int pair_pb0) {
    if (mblk >= live_blocks) return;
    const int e = !g.blk_expert ? 0 : table_in_lanes ? __builtin_amdgcn_readlane(expert_of_lane, mblk) : g.blk_expert[mblk];
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
    const size_t rb_stride = (size_t)KB * (1024 * AT); // bytes from a row block of the activations to the next
    const uint8_t* asrc = g.A + ((size_t)mblk * TM * KB + kt0) * (1024 * AT);
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
    const int m0 = mblk * TM * 32;
    const int m_limit = g.blk_expert ? live_blocks * 32 : g.M;
    float my_as = 0.0f, my_ws = 0.0f;
    bool as_ok = false, ws_ok = false;
    if constexpr (EPI != RKH_EPI_I32) {
        const int m = m0 + (TM == 2 ? lane : (lane & 31)); // (two row blocks: lanes 32.. hold the second one's)
        const int pb = pb0 + (lane >> 5);
        int n;
        if constexpr (EPI == RKH_EPI_SWIGLU) { // pb0 is even: the gate block, its up block right behind it
            const int nl = (pb0 >> 1) * 32 + (lane & 31);
            n = (lane >> 5 ? g.interleave_F : 0) + nl;
            ws_ok = nl < g.interleave_F;
        } else {
            const bool live = g.interleave_F ? pb < g.N / 32 : pb * 32 < g.N;
            n = block_first_col(pb, g.interleave_F) + (lane & 31);
            ws_ok = live && n < g.N && (lane >> 5) < TN;
        }
        as_ok = m < m_limit;
        const float* pa = g.a_scale + (as_ok ? m : 0);
        const float* pw = w_scale + (ws_ok ? n : 0);
        asm volatile("global_load_dword %0, %1, off" : "=v"(my_as) : "v"(pa));
        asm volatile("global_load_dword %0, %1, off" : "=v"(my_ws) : "v"(pw));
    }

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    v4i ring[RING][LPS]; // [i * AT .. (i + 1) * AT) = activation tiles of row block i, [AT * TM + j] = weights of column block j

    auto issue = [&](v4i* regs) {
        static_for<LPS>([&](auto l_tag) {
            constexpr int L = decltype(l_tag)::value;
            const unsigned off = lane_off; // (locals: asm operands cannot name captures of an enclosing lambda)
            const uint8_t* base = L < AT * TM ? asrc + (L / AT) * rb_stride + (L % AT) * 1024 : wsrc[L < AT * TM ? 0 : L - AT * TM];
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
        // (the scale loads are older than every load of the ring: landed too.  From here on the
        // two values are, for the compiler, defined behind a wait -- a copy or a spill of them
        // moves data that has arrived)
        asm volatile("" : "+v"(my_as), "+v"(my_ws));
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
                        const v4i raw = ring[SLOT][AT * TM + j];
                        const v4i lo = v4i{(raw.x << 4) & (int)0xF0F0F0F0, raw.x & (int)0xF0F0F0F0,
                                           (raw.y << 4) & (int)0xF0F0F0F0, raw.y & (int)0xF0F0F0F0};
                        const v4i hi = v4i{(raw.z << 4) & (int)0xF0F0F0F0, raw.z & (int)0xF0F0F0F0,
                                           (raw.w << 4) & (int)0xF0F0F0F0, raw.w & (int)0xF0F0F0F0};
#pragma unroll
                        for (int i = 0; i < TM; ++i) {
                            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(lo, ring[SLOT][i * AT], acc[i][j], 0, 0, 0);
                            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(hi, ring[SLOT][i * AT + AT - 1], acc[i][j], 0, 0, 0);
                        }
                    } else {
#pragma unroll
                        for (int i = 0; i < TM; ++i)
                            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ring[SLOT][AT * TM + j], ring[SLOT][i * AT], acc[i][j], 0, 0, 0);
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
        // (tiles of a wave counted i * TN + j)
        int* xch = reinterpret_cast<int*>(stage_raw + STAGE_BYTES) + cg * (KS - 1) * TM * TN * 16 * 64;
        if (kq > 0) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        *reinterpret_cast<v4i*>(xch + ((((kq - 1) * TM * TN + i * TN + j) * 4 + q) * 64 + lane) * 4) =
                            v4i{acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]};
        }
        __syncthreads();
        if (kq > 0) return;
#pragma unroll
        for (int w = 0; w < KS - 1; ++w)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const v4i got = *reinterpret_cast<const v4i*>(xch + (((w * TM * TN + i * TN + j) * 4 + q) * 64 + lane) * 4);
                        acc[i][j][q * 4] += got.x;
                        acc[i][j][q * 4 + 1] += got.y;
                        acc[i][j][q * 4 + 2] += got.z;
                        acc[i][j][q * 4 + 3] += got.w;
                    }
    }
    if constexpr (W4) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] >>= 4;
    }
    uint8_t* stage_lds = stage_raw + wave * (32 * (32 * 4 + 8));
    float as[TM], ws[TN][16];
#pragma unroll
    for (int i = 0; i < TM; ++i) as[i] = 0.0f;
    if constexpr (EPI != RKH_EPI_I32) { // scales: lane-wise registers -> the wave's staging area -> per-lane order
        float* sc = reinterpret_cast<float*>(stage_lds);
        sc[lane] = ws_ok ? my_ws : 0.0f;
        if (lane < 32 * TM) sc[64 + lane] = as_ok ? my_as : 0.0f;
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < TM; ++i) as[i] = sc[64 + i * 32 + (lane & 31)];
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
        epilogue_swiglu_scaled(g, acc[0][0], acc[0][TN - 1], m0, pb0, lane, as[0], ws[0], ws[TN - 1], m_limit, stage_lds);
    } else {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                epilogue_tile_scaled<EPI>(g, acc[i][j], m0 + i * 32, pb0 + j, lane, as[i], ws[j], m_limit, stage_lds);
    }
    RK_TS(TSB + 3);
    }; // run_unit

    if constexpr (!BAL) {
        const unsigned logical = (unsigned)xcd_remap(blockIdx.x, mblocks * nblocks);
        const unsigned col_tile = logical / (unsigned)mblocks; // (one unsigned division ahead of the first load)
        run_unit((int)(logical - col_tile * (unsigned)mblocks), (int)col_tile, 0);
    } else {
        // Balanced launch: one workgroup of eight waves per compute unit, the units (live row
        // block, column pair) dealt out in equal contiguous shares -- first to the dies (a
        // workgroup's die is blockIdx % 8), then to the workgroups of a die -- and a share walked
        // by its workgroup's waves in turn.  Consecutive units are column pairs of one row block,
        // so the waves of a workgroup share the activation tiles through the L1, and the row
        // blocks of one expert meet in one die's L2.
        // (32-bit arithmetic: the launcher uses this variant only while 8 x the units fit; 64-bit
        // divisions are a few hundred instructions between a wave's start and its first load)
        const unsigned pairs = (unsigned)(g.N + 63) / 64;
        const unsigned units = (unsigned)live_blocks * pairs;
        const unsigned xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = (gridDim.x + 7 - xcd) >> 3;
        const unsigned die0 = units * xcd / 8, die1 = units * (xcd + 1) / 8;
        const unsigned first = die0 + (die1 - die0) * slot / slots, last = die0 + (die1 - die0) * (slot + 1) / slots;
        for (unsigned u = first + wave; u < last; u += WAVES) run_unit((int)(u / pairs), 0, (int)(u % pairs) * TN);
    }
}


// Workgroups of the 256-column grid below which the K-split variant is used.  Measured on a 32-expert
// top-4 layer (H 2048, I 1024): 1 / 2 tokens 32.9 -> 27.1 / 37.7 -> 35.7 us; from 4 tokens (16 possible
// row blocks) on the wide tile is faster again (41.4 vs 44.6 us).
// (Splitting K two ways over 128-column tiles for 4 .. 64 tokens was measured too: 1 - 3 us slower than
// the wide tile at every size.)
constexpr long GROUPED_KS4_BELOW = 96;
constexpr long GROUPED_BALANCED_UNITS_PER_CU = 4; // (row block, column pair) units per compute unit from which the balanced launch is used

// (dense use of the same kernel, every row block live: DENSE_KS4_BELOW in rk_kernels_common.h)
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
    // 64-column tiles with K split over the waves; 32-column tiles while even twice as many workgroups
    // leave compute units without one (a compute unit draws 55 GB/s however few of them work: 64 rows of
    // 2048 x 2048 are 64 workgroups of 192 KB or 128 of 128 KB).  RK_NPU_HIP_STREAM_NARROW=0 switches it off
    // (tuning aid).
    static const char* narrow_env = getenv("RK_NPU_HIP_STREAM_NARROW");
    const bool narrow = ks == 4 && g.epilogue != RKH_EPI_SWIGLU && !(narrow_env && narrow_env[0] == '0') &&
                        compute_units() > 0 && 2L * mblocks * ((g.N + 63) / 64) <= compute_units();
    const int cols = narrow ? 32 : 256 / ks;
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
    if ((long)mblocks * ((g.N + 63) / 64) > 0x0fffffffL) balanced = false; // (the kernel deals the units in 32-bit arithmetic)
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
    mark(st, narrow ? "gemm_stream_kernel<KS=4, 32 columns>" : ks == 4 ? "gemm_stream_kernel<KS=4>" : "gemm_stream_kernel");
#define RK_LAUNCH(EPI)                                                                                         \
    do {                                                                                                       \
        if constexpr (EPI != RKH_EPI_SWIGLU) {                                                                 \
            if (narrow) {                                                                                      \
                if (any_int4) hipLaunchKernelGGL((gemm_stream_kernel<EPI, 4, true, false, 1>), grid, block, 0, st, RK_GEMM_HEAD(g), mblocks, nblocks, g);  \
                if (any_int8) hipLaunchKernelGGL((gemm_stream_kernel<EPI, 4, false, false, 1>), grid, block, 0, st, RK_GEMM_HEAD(g), mblocks, nblocks, g); \
                break;                                                                                         \
            }                                                                                                  \
        }                                                                                                      \
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

} // namespace

namespace rkk {
int launch_gemm_grouped(hipStream_t st, const rkh_gemm_args& g) { return ::launch_gemm_grouped(st, g); }
#ifdef RK_DEBUG_TS
void set_ts_stream(unsigned long long* p) { (void)hipMemcpyToSymbol(HIP_SYMBOL(rk_dbg_ts), &p, sizeof(p)); }
#endif
} // namespace rkk
