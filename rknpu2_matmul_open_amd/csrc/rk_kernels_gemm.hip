// int8 MFMA GEMM for prefill-sized M: gemm_wk_kernel (tiles of 32..128 rows x 256 columns,
// activations through an LDS ring, waves split K), gemm_wk_reduce_kernel (sum of K-split
// partial tiles + epilogue) and their launcher.  Bound by the matrix pipes.
#include "rk_kernels_tile.h"

namespace {

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
// (unsigned arithmetic: these divisions stand between a wave's start and its first load, and a
// signed division by a run-time value is half as long again)
__device__ __forceinline__ void wk_tile_coords(unsigned tile, unsigned mblocks, unsigned nblocks, int& mblk, int& nblk) {
    constexpr unsigned GM = 4;
    const unsigned per_group = GM * nblocks;
    const unsigned group = tile / per_group;
    const unsigned first_m = group * GM;
    const unsigned gm = min(mblocks - first_m, GM);
    const unsigned in_group = tile - group * per_group;
    const unsigned col = in_group / gm;
    mblk = (int)(first_m + in_group - col * gm);
    nblk = (int)col;
}

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm" // m0 is set and clobbered on purpose below
// TN: 32-column blocks per wave.  Two -- tiles of 256 columns; one -- tiles of 128 columns, for a few
// hundred rows whose 256-column tiles would leave compute units without one (launch_gemm_wk_narrow).
template <int TM, bool W4, int EPI, int TN = 2>
__global__ __launch_bounds__(512) void gemm_wk_kernel(const uint8_t* h_A, const uint8_t* h_W, int h_M, int h_K,
                                                      int mblocks, int nblocks, int ksplit, int ksteps_per_part,
                                                      rkh_gemm_args g) {
    // (leading scalar arguments, see RK_GEMM_HEAD_PARAMS: everything the tile coordinates and the
    // prologue's loads depend on, ten dwords, arrives in registers)
    g.A = h_A; g.W = h_W; g.M = h_M; g.K = h_K;
    RK_TS(0);
    constexpr int KTS = 8 / TM, KTW = KTS / 2; // k-tiles per sub-step: all / this wave's
    constexpr int NMF = TM * KTW * TN;         // MFMAs of a wave per sub-step
    static_assert(TN == 2 || (TN == 1 && EPI != RKH_EPI_SWIGLU), "gate / up pairs need two column blocks per wave");
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
    const int kpart = ksplit > 1 ? (int)((unsigned)logical / (unsigned)tiles) : 0;
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
        const int pb = nblk * (4 * TN) + wn * TN + j;
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
        static_assert(NMF >= 4 && NWREG <= ((NWREG + 3) / 4) * (NMF - 2), "the slots below: four fragment reads, the wait, the unpack items");
        static_for<NMF>([&](auto q_tag) {
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
    // loads in the queue only make the first sub-steps' waits stricter.  Ahead of
    // the prologue's loads they cost the 128-row tile 0.2 us: the first copies
    // leave later.)  They are in flight until the wait of the loop's third
    // sub-step, or the closing wait; like every register an asm load writes they
    // must not be touched before -- which the build verifies in the compiled code
    // (audit_waits.py) rather than trusting the allocator.
    float my_as = 0.0f, my_ws = 0.0f;
    bool as_valid = false, ws_valid = false;
    if constexpr (EPI != RKH_EPI_I32) {
        const int t = threadIdx.x;
        const int m = mblk * BM + (t & (BM - 1));
        const int pb = nblk * (4 * TN) + ((t & (128 * TN - 1)) >> 5);
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
    // (the remaining sub-steps as a chain that ends at the first one beyond K: the control flow
    // then only holds the sequences of sub-steps that can happen, which is what the static check
    // of the waits, audit_waits.py, walks)
    static_while<UNR>([&](auto slot) {
        if (s + decltype(slot)::value >= ksteps) return false;
        k_step(slot);
        return true;
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
        if (t < 128 * TN) sc[128 + t] = ws_valid ? my_ws : 0.0f;
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
                const int pb0 = nblk * (4 * TN) + wn * TN;
                if constexpr (EPI == RKH_EPI_SWIGLU) {
                    epilogue_swiglu_scaled(g, acc[i0 + ii][0], acc[i0 + ii][TN - 1], m0, pb0, lane, as[ii], ws[0], ws[TN - 1],
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


// Bytes of split-K scratch for `tiles` output tiles of bm rows split into
// ksplit parts: the int32 partial tiles.
static size_t wk_scratch_bytes(long tiles, int bm, int ksplit) {
    return ksplit > 1 ? (size_t)tiles * ksplit * bm * 256 * 4 : 0;
}

// Workgroups of a launch with this tile height and K split (what launch_gemm_wk makes of `ksplit`).
static int wk_grid(const rkh_gemm_args& g, int tile_rows, int& ksplit) {
    const int kts = 8 / (tile_rows / 32);
    const int mblocks = (g.M + tile_rows - 1) / tile_rows, nblocks = (g.N + 255) / 256;
    const int ksteps_total = (int)(rkh_align_up(g.K, RKH_K_ALIGN) / 32 / kts);
    if (ksplit > ksteps_total) ksplit = ksteps_total;
    if (ksplit < 1) ksplit = 1;
    const int per = (ksteps_total + ksplit - 1) / ksplit;
    ksplit = (ksteps_total + per - 1) / per; // no empty part
    return mblocks * nblocks * ksplit;
}

template <int TM>
int launch_gemm_wk(hipStream_t st, const rkh_gemm_args& g, int ksplit) {
    constexpr int BM = 32 * TM, KTS = 8 / TM;
    const int mblocks = (g.M + BM - 1) / BM;
    const int nblocks = (g.N + 255) / 256;
    const int ksteps_total = (int)(rkh_align_up(g.K, RKH_K_ALIGN) / 32 / KTS);
    const dim3 grid(wk_grid(g, BM, ksplit)), block(512);
    const int per = (ksteps_total + ksplit - 1) / ksplit;
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

// Tiles of 64 or 128 rows x 128 columns (one column block per wave), K not split over workgroups: a few
// hundred rows whose 256-column tiles would leave compute units without one.  The activation rows of a tile
// go through LDS once for the eight waves, so a tile pulls K x (rows + 128) bytes through its compute unit.
template <int TM>
int launch_gemm_wk_narrow(hipStream_t st, const rkh_gemm_args& g) {
    constexpr int TN = 1, KTS = 8 / TM;
    const int mblocks = (g.M + 32 * TM - 1) / (32 * TM), nblocks = (g.N + 127) / 128;
    const int ksteps_total = (int)(rkh_align_up(g.K, RKH_K_ALIGN) / 32 / KTS);
    const dim3 grid(mblocks * nblocks), block(512);
    mark(st, TM == 2 ? "gemm_wk_kernel<64 x 128>" : "gemm_wk_kernel<128 x 128>");
#define RK_WKN(W4, EPI)                                                                             \
    do {                                                                                            \
        static std::atomic<bool> opted_in[64] = {};                                                 \
        int dev = 0;                                                                                \
        RKH_CHECK(hipGetDevice(&dev));                                                              \
        if (dev < 0 || dev >= 64) return RKH_ERR_RUNTIME;                                           \
        if (!opted_in[dev].load(std::memory_order_acquire)) {                                       \
            RKH_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_wk_kernel<TM, W4, EPI, TN>), \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, WK_LDS_BYTES)); \
            opted_in[dev].store(true, std::memory_order_release);                                   \
        }                                                                                           \
        hipLaunchKernelGGL((gemm_wk_kernel<TM, W4, EPI, TN>), grid, block, WK_LDS_BYTES, st,       \
                           g.A, g.W, g.M, g.K, mblocks, nblocks, 1, ksteps_total, g);               \
    } while (0)
    // (int4 weights: the 64-row tiles only -- the 128-row ones measured slower than the other plans everywhere)
#define RK_WKN_W(EPI)                                                                               \
    do {                                                                                            \
        if (!g.w_int4) RK_WKN(false, EPI);                                                          \
        else if constexpr (TM == 2) RK_WKN(true, EPI);                                              \
        else return RKH_ERR_RUNTIME;                                                                \
    } while (0)
    switch (g.epilogue) {
    case RKH_EPI_I32: RK_WKN_W(RKH_EPI_I32); break;
    case RKH_EPI_F16: RK_WKN_W(RKH_EPI_F16); break;
    case RKH_EPI_F32: RK_WKN_W(RKH_EPI_F32); break;
    default: return RKH_ERR_RUNTIME;
    }
#undef RK_WKN_W
#undef RK_WKN
    RKH_CHECK(hipGetLastError());
    return RKH_OK;
}

} // namespace

namespace rkk {
int launch_gemm_wk_narrow(hipStream_t st, const rkh_gemm_args& g, int tile_rows) {
    return tile_rows == 128 ? ::launch_gemm_wk_narrow<4>(st, g) : ::launch_gemm_wk_narrow<2>(st, g);
}
size_t wk_scratch_bytes(long tiles, int bm, int ksplit) { return ::wk_scratch_bytes(tiles, bm, ksplit); }
int launch_gemm_wk(hipStream_t st, const rkh_gemm_args& g, int tile_rows, int ksplit) {
    if (tile_rows == 128) return ::launch_gemm_wk<4>(st, g, ksplit);
    if (tile_rows == 64) return ::launch_gemm_wk<2>(st, g, ksplit);
    return ::launch_gemm_wk<1>(st, g, ksplit);
}
#ifdef RK_DEBUG_TS
void set_ts_gemm(unsigned long long* p) { (void)hipMemcpyToSymbol(HIP_SYMBOL(rk_dbg_ts), &p, sizeof(p)); }
#endif
} // namespace rkk
