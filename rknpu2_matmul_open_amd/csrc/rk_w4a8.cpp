// W4A8 linear, fused gate/up + SwiGLU, and the FFN block.
//
// Replaces src/rk_npu_w4a8.cpp of the reference: there an INT8 activation is
// split into two INT4 rows and a W4A4 NPU backend produces INT16 partials that
// the CPU reduces; here int8 x int4 runs on MFMA into int32 directly, so the
// whole call is  quantize rows -> GEMM (dequant or SwiGLU epilogue)
// [-> re-quantize middle with the collected row maxima -> GEMM].
// Validation, argument order of checks and byte accounting follow
// src/rk_npu_w4a8.cpp:47-68,83-94,162-207,249-380 and src/rk_npu_i4_plan.cpp:14-89.
#include <algorithm>
#include <cerrno>
#include <climits>
#include <cstdlib>
#include <new>
#include <thread>

#include "rk_host.h"
#include "rk_npu_hip.h"
#include "rk_npu_w4a8.h"
#include "rk_w4a8_internal.h"

using namespace rkhost;

namespace {

constexpr int kKTileMax = 2048;       // reference src/rk_npu_i4_bounds.h:5
constexpr int kKTileUniversal = 480;  // reference src/rk_npu_i4_bounds.h:6
constexpr int kNTileMax = 8128;

int64_t align_up64(int64_t v, int64_t a) { return (v + a - 1) / a * a; }
bool valid_shape(int K, int N) { return K > 0 && K <= INT32_MAX / 1024 && N > 0; }
bool weight_key_valid(int K, int N, int k_tile) {
    return K > 0 && K <= INT32_MAX / 64 && N > 0 && N <= INT_MAX - 63 && k_tile >= 32 &&
           k_tile <= kKTileMax && k_tile % 32 == 0;
}

struct Policy {
    bool panel8 = false;
    bool npu_reduce = false; // effective (requested and M > 16)
};

// reference src/rk_npu_w4a8.cpp:48-58
int read_options(const rk_npu_w4a8_options* opt, int M, Policy& p) {
    p = Policy{};
    if (!opt) return RK_NPU_OK;
    if (opt->struct_size != sizeof(*opt) ||
        (opt->input_layout != RK_NPU_W4A8_INPUT_NATIVE && opt->input_layout != RK_NPU_W4A8_INPUT_PANEL8) ||
        (opt->reduce_backend != RK_NPU_W4A8_REDUCE_CPU && opt->reduce_backend != RK_NPU_W4A8_REDUCE_NPU))
        return RK_NPU_ERR_PARAM;
    p.panel8 = opt->input_layout == RK_NPU_W4A8_INPUT_PANEL8;
    p.npu_reduce = opt->reduce_backend == RK_NPU_W4A8_REDUCE_NPU && M > 16;
    return RK_NPU_OK;
}

// Range validation of a workspace configuration.  The reference checks these
// through its W4A4 backend with physical rows = 2*M and m_tile doubled
// (src/rk_npu_w4a8.cpp:59-68, src/rk_npu_i4_plan.cpp:18-31).
bool config_valid(const rk_npu_w4a8_config& c, const Policy& p) {
    if (!valid_shape(c.K, c.N) || c.M < 1 || c.M > INT_MAX / 2 || c.m_tile < 1 ||
        c.m_tile > (p.panel8 ? 256 : 64) || c.pipeline < RK_NPU_W4A8_SERIAL ||
        c.pipeline > RK_NPU_W4A8_CHAIN)
        return false;
    if (!weight_key_valid(c.K, c.N, c.k_tile)) return false;
    if (p.panel8) {
        const int mt = c.m_tile * 2; // physical rows per tile
        if (mt % 8 || mt > 512 || mt < 8) return false;
    }
    const int cores = __builtin_popcount(c.npu_core_mask);
    const uint32_t m = c.npu_core_mask;
    if (!(m == 1 || m == 2 || m == 4 || m == 3 || m == 7)) return false;
    if (c.n_tile < 64 || c.n_tile > kNTileMax || c.n_tile % 64) return false;
    if (align_up64(c.N, 64) / 64 < cores) return false;
    if (c.timeout_ms == 0 || c.cpu_threads < 1 || c.cpu_threads > 4) return false;
    return true;
}

// The reference's INT16-partial certificate for one fixed K partition
// (src/rk_npu_i4_bounds.cpp:9-69): with activations split into int4 halves in
// [-8,7], the partial sum of a tile is bounded by P = sum(7w for w>=0, -8w for
// w<0) on the positive side and Q = sum(8w for w>=0, -7w for w<0) in
// magnitude on the negative side; the tile is safe when every 32-aligned
// group of `t` blocks has P <= 32767 and Q <= 32768.  It does not affect
// results here (accumulation is int32) but decides which k_tile a weight
// reports and whether an explicit k_tile > 480 is accepted.
struct BoundScan {
    int K, N, blocks;
    std::vector<int32_t> pos, neg; // [blocks + 1][N] prefix sums over 32-row blocks
    bool scan(const int8_t* B) {
        pos.assign((size_t)(blocks + 1) * N, 0);
        neg.assign((size_t)(blocks + 1) * N, 0);
        for (int b = 0; b < blocks; ++b) {
            int32_t* p = pos.data() + (size_t)(b + 1) * N;
            int32_t* q = neg.data() + (size_t)(b + 1) * N;
            std::memcpy(p, p - N, (size_t)N * sizeof(int32_t));
            std::memcpy(q, q - N, (size_t)N * sizeof(int32_t));
            const int kend = std::min(K, (b + 1) * 32);
            for (int k = b * 32; k < kend; ++k) {
                const int8_t* row = B + (size_t)k * N;
                for (int n = 0; n < N; ++n) {
                    const int w = row[n];
                    if (w < -8 || w > 7) return false;
                    p[n] += w >= 0 ? 7 * w : -8 * w;
                    q[n] += w >= 0 ? 8 * w : -7 * w;
                }
            }
        }
        return true;
    }
    bool certifies(int t) const {
        for (int b = 0; b < blocks; b += t) {
            const int e = std::min(blocks, b + t);
            const int32_t* p0 = pos.data() + (size_t)b * N;
            const int32_t* p1 = pos.data() + (size_t)e * N;
            const int32_t* q0 = neg.data() + (size_t)b * N;
            const int32_t* q1 = neg.data() + (size_t)e * N;
            for (int n = 0; n < N; ++n)
                if (p1[n] - p0[n] > 32767 || q1[n] - q0[n] > 32768) return false;
        }
        return true;
    }
};

// K is bounded by INT32_MAX/1024, so 8*K*... prefix sums fit int32: max per
// element contribution is 64, 64 * 2^21 = 2^27.
//
// Largest certified tile (or -1: an out-of-range code, or nothing certified).
// `requested` = 0 searches all tile sizes up to 2048, else only that one is
// tested.  `mask` (optional) receives one bit per certified size, bit t-1 for
// 32*t.  Column slabs keep the prefix tables small and are independent, so
// they are spread over a few host threads.
int largest_certified_tile(const int8_t* B, int K, int N, int requested /*0 = search*/, uint64_t* mask = nullptr) {
    const int blocks = (K + 31) / 32;
    constexpr int kSlab = 256;
    const int limit = requested ? requested / 32 : std::min(kKTileMax / 32, blocks);
    const int slabs = (N + kSlab - 1) / kSlab;
    const int workers = std::max(1, std::min({slabs, 8, (int)std::thread::hardware_concurrency()}));
    std::vector<std::vector<char>> safe_of((size_t)workers, std::vector<char>((size_t)limit + 1, 1));
    std::vector<char> failed((size_t)workers, 0);
    auto work = [&](int id) {
        std::vector<int8_t> slab;
        std::vector<char>& safe = safe_of[(size_t)id];
        for (int t = 1; t <= limit; ++t) safe[(size_t)t] = !requested || t == limit;
        for (int si = id; si < slabs; si += workers) {
            const int n0 = si * kSlab, width = std::min(kSlab, N - n0);
            slab.resize((size_t)K * width);
            for (int k = 0; k < K; ++k)
                std::memcpy(slab.data() + (size_t)k * width, B + (size_t)k * N + n0, (size_t)width);
            BoundScan part{K, width, blocks, {}, {}};
            if (!part.scan(slab.data())) {
                failed[(size_t)id] = 1;
                return;
            }
            for (int t = 1; t <= limit; ++t)
                if (safe[(size_t)t] && !part.certifies(t)) safe[(size_t)t] = 0;
        }
    };
    if (workers == 1) {
        work(0);
    } else {
        std::vector<std::thread> pool;
        for (int id = 0; id < workers; ++id) pool.emplace_back(work, id);
        for (auto& t : pool) t.join();
    }
    for (char f : failed)
        if (f) return -1;
    uint64_t bits = 0;
    int best = -1;
    for (int t = 1; t <= limit; ++t) {
        bool ok = true;
        for (int id = 0; id < workers; ++id) ok = ok && safe_of[(size_t)id][(size_t)t];
        if (ok) {
            bits |= uint64_t(1) << (t - 1);
            best = t * 32;
        }
    }
    if (mask) *mask = bits;
    return best;
}

// Identity of a weight matrix (codes and scales), not a security hash: FNV-1a
// per 1 MiB piece, the piece digests folded in order, so that the pieces can be
// hashed side by side.
uint64_t fingerprint_of(int K, int N, const int8_t* B, const float* w_scale) {
    auto fnv = [](uint64_t h, const void* data, size_t bytes) {
        const uint8_t* p = static_cast<const uint8_t*>(data);
        for (size_t i = 0; i < bytes; ++i) {
            h ^= p[i];
            h *= 0x100000001b3ull;
        }
        return h;
    };
    constexpr uint64_t kBasis = 0xcbf29ce484222325ull;
    constexpr size_t kPiece = 1u << 20;
    const size_t total = (size_t)K * N, pieces = (total + kPiece - 1) / kPiece;
    std::vector<uint64_t> digest(pieces);
    const int workers = std::max(1, std::min({(int)pieces, 8, (int)std::thread::hardware_concurrency()}));
    auto work = [&](int id) {
        for (size_t i = (size_t)id; i < pieces; i += (size_t)workers)
            digest[i] = fnv(kBasis, B + i * kPiece, std::min(kPiece, total - i * kPiece));
    };
    if (workers == 1) {
        work(0);
    } else {
        std::vector<std::thread> pool;
        for (int id = 0; id < workers; ++id) pool.emplace_back(work, id);
        for (auto& t : pool) t.join();
    }
    uint64_t h = kBasis;
    const int64_t shape[2] = {K, N};
    h = fnv(h, shape, sizeof(shape));
    h = fnv(h, digest.data(), digest.size() * sizeof(uint64_t));
    return fnv(h, w_scale, (size_t)N * sizeof(float));
}

} // namespace

struct rk_npu_w4a8_weights {
    Owner owner;
    rk_npu_w4a8_weight_info info{};
    rkhost::W4Profile profile;
    int interleave_F = 0;  // N/2 when N % 64 == 0 (gate/up column blocks interleaved)
    DeviceBuffer tiled;    // tiled int4
    DeviceBuffer w_scale;  // [N]
    DeviceBuffer colsum;   // [N] int32: sum over k of the codes of a column (decode GEMV constant)
};

struct rk_npu_w4a8_workspace {
    Owner owner;
    rk_npu_w4a8_config config{};
    Policy policy;
    DeviceBuffer a_raw;     // uploaded A (fp32 sized; fp16 uses half of it)
    DeviceBuffer a_tiled;   // quantized activations
    DeviceBuffer a_scale;   // [align128(M)]
    DeviceBuffer c_out;     // [M, N] fp32-sized result staging
    DeviceBuffer row_max;   // [align128(M)][N/64] partial row maxima of the SwiGLU middle
    DeviceBuffer splitk;
    HostStage stage_a, stage_c; // pinned mirrors of a small A / C that the kernels read / write in place
    BadFlag flag;
    std::atomic_flag busy = ATOMIC_FLAG_INIT;
    ~rk_npu_w4a8_workspace() {
        if (owner.ctx) rkhost::forget_pending_flag(owner.ctx, flag.device());
    }
};

namespace {

// reference src/rk_npu_w4a8.cpp:83-94
int validate(const rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w, const void* A,
             const void* C, bool swiglu) {
    if (!ws || !w || !A || !C || A == C || (swiglu && (ws->policy.npu_reduce || ws->config.N % 64)))
        return RK_NPU_ERR_PARAM;
    if (!w->owner.same(ws->owner)) return RK_NPU_ERR_DOMAIN;
    const auto& wc = w->info.config;
    if (wc.K != ws->config.K || wc.N != ws->config.N || wc.k_tile != ws->config.k_tile)
        return RK_NPU_ERR_PARAM;
    return RK_NPU_OK;
}

enum class Out { F32, F16, I32, SwiGLU };
int enqueue_gemm(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w, void* dC, Out out,
                 bool collect);
rkh_gemm_args gemm_args(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w, void* dC, Out out,
                        bool collect);

// quantize (or re-quantize with reused row maxima) + GEMM.  `scale_source`
// non-null: A is the fp32 middle of that workspace's SwiGLU run and its
// row_max feeds the scale (reference run_locked(scale_source), :98-151).
int enqueue(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w, const void* dA, bool half,
            void* dC, Out out, bool collect, rk_npu_w4a8_workspace* scale_source,
            StageTimer* timer, bool a_is_host = false) {
    const auto& c = ws->config;
    void* stream = ws->owner.ctx->stream;
    rkh_quant_args q{};
    q.src = dA;
    q.src_is_host = a_is_host ? 1 : 0;
    q.in_dtype = half ? RKH_F16 : RKH_F32;
    q.M = c.M;
    q.K = c.K;
    q.scale = ws->a_scale.as<float>();
    q.dst = ws->a_tiled.as<>();
    q.bad_flag = ws->flag.device();
    if (scale_source) {
        q.mode = RKH_Q_REUSE_BITS;
        q.row_max_bits = scale_source->row_max.as<uint32_t>();
        q.row_max_parts = scale_source->config.N / 64; // one partial per 32 middle columns
    } else {
        q.mode = RKH_Q_W4A8;
    }
    const rkh_gemm_args g = gemm_args(ws, w, dC, out, collect);
    int rc;
    if (timer) {
        // separate launches so the stage timer can tell the two apart
        rc = rkh_quant_rows(stream, &q);
        timer->mark();
        if (!rc) rc = rkh_gemm(stream, &g);
        timer->mark();
    } else {
        rc = rkh_quant_gemm(stream, &q, &g);
    }
    return map_error(rc);
}

rkh_gemm_args gemm_args(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w, void* dC, Out out,
                        bool collect) {
    const auto& c = ws->config;
    rkh_gemm_args g{};
    g.A = ws->a_tiled.as<>();
    g.W = w->tiled.as<>();
    g.w_int4 = 1;
    g.M = c.M;
    g.N = c.N;
    g.K = c.K;
    g.interleave_F = w->interleave_F;
    g.a_scale = ws->a_scale.as<float>();
    g.w_scale = w->w_scale.as<float>();
    g.w_colsum = w->colsum.as<int32_t>();
    g.C = dC;
    g.splitk_acc = ws->splitk ? ws->splitk.as<int32_t>() : nullptr;
    switch (out) {
    case Out::F32: g.epilogue = RKH_EPI_F32; g.ldc = c.N; break;
    case Out::F16: g.epilogue = RKH_EPI_F16; g.ldc = c.N; break;
    case Out::I32: g.epilogue = RKH_EPI_I32; g.ldc = c.N; break;
    case Out::SwiGLU:
        g.epilogue = RKH_EPI_SWIGLU;
        g.ldc = c.N / 2;
        g.row_max_bits = collect ? ws->row_max.as<uint32_t>() : nullptr;
        break;
    }
    return g;
}

// GEMV / GEMM stage on the activations already quantized into the workspace.
int enqueue_gemm(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w, void* dC, Out out,
                 bool collect) {
    const rkh_gemm_args g = gemm_args(ws, w, dC, out, collect);
    return map_error(rkh_gemm(ws->owner.ctx->stream, &g));
}

void fill_timings(rk_npu_w4a8_timings* t, StageTimer& timer, int first_mark, bool scanned,
                  double copy_us, double total_us) {
    if (!t) return;
    *t = rk_npu_w4a8_timings{};
    const double quant = timer.span_us(first_mark, first_mark + 1);
    if (scanned) {
        t->activation_scan_us = quant * 0.5; // one fused kernel: scan and pack halves
        t->quant_pack_us = quant * 0.5;
    } else {
        t->quant_pack_us = quant;
    }
    t->submit_us = timer.span_us(first_mark + 1, first_mark + 2);
    t->sync_us = copy_us;
    t->total_us = total_us;
}

int run_host(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w, const void* A, void* C,
             bool half, Out out, rk_npu_w4a8_timings* timings) {
    const bool swiglu = out == Out::SwiGLU;
    int rc = validate(ws, w, A, C, swiglu);
    if (rc) return rc;
    BusyLock lock(ws->busy);
    if (!lock) return RK_NPU_ERR_BUSY;
    const auto t0 = Clock::now();
    const auto& c = ws->config;
    rk_npu_ctx* ctx = ws->owner.ctx;
    const size_t a_bytes = (size_t)c.M * c.K * (half ? 2 : 4);
    const size_t out_cols = swiglu ? (size_t)c.N / 2 : (size_t)c.N;
    const size_t c_bytes = (size_t)c.M * out_cols * (out == Out::F16 ? 2 : 4);
    StageTimer timer(ctx->stream, timings != nullptr);
    // Small operands skip the copies: the kernels read A from / write the result
    // into the pinned mirrors (the caller's C is only written after the checks).
    const bool direct_in = ws->stage_a.direct(a_bytes), direct_out = ws->stage_c.direct(c_bytes);
    const void* src = direct_in ? ws->stage_a.fill(A, a_bytes) : ws->a_raw.as<>(); // before the submission lock
    {
        std::lock_guard<std::mutex> submit(ctx->submit_mutex);
        if (!direct_in) rc = map_error(ws->stage_a.upload(ctx->stream, ws->a_raw.as<>(), A, a_bytes));
        timer.mark();
        if (!rc)
            rc = enqueue(ws, w, src, half, direct_out ? ws->stage_c.data() : ws->c_out.as<>(), out, false, nullptr,
                         &timer, direct_in);
        if (!rc) rc = ws->flag.enqueue_readback(ctx->stream);
    }
    int wait = map_error(rkh_sync(ctx->stream));
    if (rc || wait) return rc ? rc : wait;
    if (ws->flag.consume(ctx->stream)) {
        if (timings) {
            *timings = rk_npu_w4a8_timings{};
            timings->activation_scan_us = timer.span_us(0, 1);
            timings->total_us = elapsed_us(t0);
        }
        return RK_NPU_ERR_PARAM; // NaN / Inf activation: C is not written
    }
    const auto t1 = Clock::now();
    if (direct_out) {
        ws->stage_c.finish(C, c_bytes);
    } else {
        rc = map_error(ws->stage_c.download(ctx->stream, C, ws->c_out.as<>(), c_bytes));
        if (!rc) rc = map_error(ws->stage_c.finish_download(ctx->stream, C, c_bytes));
    }
    fill_timings(timings, timer, 0, true, elapsed_us(t1), elapsed_us(t0));
    return rc;
}

int run_device(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w, const void* dA, void* dC,
               bool half, Out out) {
    int rc = validate(ws, w, dA, dC, out == Out::SwiGLU);
    if (rc) return rc;
    BusyLock lock(ws->busy);
    if (!lock) return RK_NPU_ERR_BUSY;
    std::lock_guard<std::mutex> submit(ws->owner.ctx->submit_mutex);
    note_pending_flag(ws->owner.ctx, ws->flag.device());
    return enqueue(ws, w, dA, half, dC, out, false, nullptr, nullptr);
}

// Shared checks of the FFN entry points (reference src/rk_npu_w4a8.cpp:358-368).
int validate_ffn(rk_npu_w4a8_workspace* gu, const rk_npu_w4a8_weights* guw,
                 rk_npu_w4a8_workspace* dn, const rk_npu_w4a8_weights* dnw, const void* A,
                 const void* middle, const void* C) {
    if (gu == dn || middle == C || A == C) return RK_NPU_ERR_PARAM;
    int rc = validate(gu, guw, A, middle, true);
    if (rc) return rc;
    rc = validate(dn, dnw, middle, C, false);
    if (rc) return rc;
    if (gu->config.M != dn->config.M || gu->config.N / 2 != dn->config.K) return RK_NPU_ERR_PARAM;
    if (!gu->owner.same(dn->owner)) return RK_NPU_ERR_DOMAIN;
    return RK_NPU_OK;
}

} // namespace

namespace rkhost {

double w4a8_env_multiplier() {
    const char* text = std::getenv("RK_NPU_W4A8_K_TILE_MULTIPLIER");
    if (!text) return 1.0;
    errno = 0;
    char* end = nullptr;
    const double factor = std::strtod(text, &end);
    if (errno || end == text || *end || !std::isfinite(factor) || factor < 1) return -1.0;
    return factor;
}

// reference src/rk_npu_w4a8_tune_policy.cpp:46-70 (the weight-dependent part)
int w4a8_make_profile(int K, int N, double multiplier, const int8_t* B, const float* w_scale, W4Profile* out) {
    if (!out || !B || !w_scale || !valid_shape(K, N) || N > INT_MAX - 63 || !std::isfinite(multiplier) ||
        multiplier < 1)
        return RK_NPU_ERR_PARAM;
    if (!finite_positive(w_scale, (size_t)N)) return RK_NPU_ERR_PARAM;
    W4Profile p;
    p.K = K;
    p.N = N;
    p.multiplier = multiplier;
    p.safe = largest_certified_tile(B, K, N, 0, &p.safe_tiles);
    if (p.safe < 32) return RK_NPU_ERR_PARAM;
    const int cap = std::min(kKTileMax, (int)align_up64(K, 32));
    p.limit = (int)(std::min((double)cap, p.safe * multiplier) / 32) * 32;
    p.fingerprint = fingerprint_of(K, N, B, w_scale);
    *out = p;
    return RK_NPU_OK;
}

// reference src/rk_npu_w4a8.cpp:208-247
rk_npu_w4a8_weights* w4a8_create_weights(rk_npu_iommu_domain* domain, const rk_npu_w4a8_weight_info& info,
                                         const int8_t* B, const float* w_scale, const W4Profile* profile) {
    const rk_npu_i4_weight_config& cfg = info.config;
    if (!domain || !domain->ctx || !B || !w_scale || !valid_shape(cfg.K, cfg.N) ||
        !weight_key_valid(cfg.K, cfg.N, cfg.k_tile))
        return nullptr;
    if (!finite_positive(w_scale, (size_t)cfg.N)) return nullptr;
    std::unique_ptr<rk_npu_w4a8_weights> w(new (std::nothrow) rk_npu_w4a8_weights());
    if (!w) return nullptr;
    if (profile) {
        w->profile = *profile;
    } else if (w4a8_make_profile(cfg.K, cfg.N, info.multiplier, B, w_scale, &w->profile)) {
        // the full proof is captured independently of the requested partition
        // (an explicit k_tile may be wider than K)
        return nullptr;
    }
    w->owner.bind(domain);
    w->info = info;
    w->interleave_F = cfg.N % 64 == 0 ? cfg.N / 2 : 0;
    rk_npu_ctx* ctx = domain->ctx;
    std::lock_guard<std::mutex> lock(ctx->submit_mutex);
    DeviceBuffer raw, bad;
    if (upload(w->owner, raw, B, (size_t)cfg.K * cfg.N)) return nullptr;
    if (bad.alloc(w->owner, sizeof(int), true)) return nullptr;
    if (w->tiled.alloc(w->owner, rkh_tiled_i4_bytes(cfg.N, cfg.K, RKH_COL_ALIGN), false)) return nullptr;
    if (w->colsum.alloc(w->owner, (size_t)cfg.N * sizeof(int32_t), true)) return nullptr;
    if (rkh_pack_w4(ctx->stream, raw.as<int8_t>(), cfg.K, cfg.N, w->interleave_F, w->tiled.as<>(),
                    bad.as<int>(), w->colsum.as<int32_t>()))
        return nullptr;
    if (upload(w->owner, w->w_scale, w_scale, (size_t)cfg.N * sizeof(float))) return nullptr;
    int bad_host = 0;
    if (rkh_d2h(ctx->stream, &bad_host, bad.as<>(), sizeof(int)) || rkh_sync(ctx->stream)) return nullptr;
    if (bad_host) return nullptr; // a code outside [-8, 7]
    return w.release();
}

const W4Profile& w4a8_profile_of(const rk_npu_w4a8_weights* weights) { return weights->profile; }

bool i4_tile_certified(const int8_t* B, int K, int N, int k_tile) {
    return largest_certified_tile(B, K, N, k_tile) == k_tile;
}

} // namespace rkhost

extern "C" {

void rk_npu_w4a8_config_init(rk_npu_w4a8_config* cfg, int M, int N, int K) {
    if (!cfg) return;
    cfg->M = M;
    cfg->N = N;
    cfg->K = K;
    cfg->m_tile = 64;
    cfg->k_tile = 480;
    cfg->n_tile = 1024;
    cfg->npu_core_mask = 1;
    cfg->timeout_ms = 500;
    cfg->pipeline = RK_NPU_W4A8_PIPELINED;
    cfg->cpu_threads = 1;
}

void rk_npu_w4a8_options_init(rk_npu_w4a8_options* options) {
    if (!options) return;
    options->struct_size = sizeof(*options);
    options->input_layout = RK_NPU_W4A8_INPUT_NATIVE;
    options->reduce_backend = RK_NPU_W4A8_REDUCE_CPU;
}

// Logical RK3588 byte accounting (reference src/rk_npu_w4a8.cpp:169-207 and
// src/rk_npu_i4_plan.cpp:57-89), physical rows = 2*M.  control_bytes and
// tasks_per_wave describe NPU command buffers and are reported as 0; the NPU
// reduce backend's own buffers are likewise 0.
int rk_npu_w4a8_memory_query_ex(const rk_npu_w4a8_config* cfg, const rk_npu_w4a8_options* options,
                                rk_npu_w4a8_memory_info_ex* out) {
    if (!cfg || !out) return RK_NPU_ERR_PARAM;
    Policy p;
    int rc = read_options(options, cfg->M, p);
    if (rc) return rc;
    if (!config_valid(*cfg, p)) return RK_NPU_ERR_PARAM;
    if (cfg->pipeline == RK_NPU_W4A8_CHAIN && p.npu_reduce) return RK_NPU_ERR_PARAM;
    rk_npu_w4a8_memory_info_ex info{};
    info.effective_reduce_backend = p.npu_reduce ? RK_NPU_W4A8_REDUCE_NPU : RK_NPU_W4A8_REDUCE_CPU;
    auto& b = info.base.backend;
    const uint64_t M2 = (uint64_t)cfg->M * 2;
    b.packed_weight_bytes = (uint64_t)align_up64(cfg->K, 32) * align_up64(cfg->N, 64) / 2;
    if (b.packed_weight_bytes > UINT32_MAX) return RK_NPU_ERR_NOMEM;
    b.wave_count = (uint32_t)((cfg->K + cfg->k_tile - 1) / cfg->k_tile);
    const uint64_t slots = cfg->pipeline == RK_NPU_W4A8_CHAIN ? b.wave_count
                                                                : std::min<uint32_t>(b.wave_count, 2u);
    b.input_bytes = slots * M2 * align_up64(std::min(cfg->K, cfg->k_tile), 32) / 2;
    b.partial_bytes = slots * M2 * align_up64(cfg->N, 64) * 2;
    b.control_bytes = 0;
    b.tasks_per_wave = 0;
    info.base.weight_metadata_bytes = (uint64_t)cfg->N * (sizeof(float) + sizeof(int32_t));
    info.base.cpu_scratch_bytes = (uint64_t)cfg->M * sizeof(float) * 2;
    if (!p.npu_reduce) {
        info.base.cpu_scratch_bytes += (uint64_t)cfg->M * align_up64(cfg->N, 64) * sizeof(int32_t);
        if (cfg->N % 64 == 0)
            info.base.cpu_scratch_bytes += ((uint64_t)cfg->M + 16) * cfg->cpu_threads * sizeof(uint32_t);
    }
    info.workspace_bytes = b.input_bytes + b.partial_bytes + b.control_bytes +
                           info.base.cpu_scratch_bytes + info.reduction_output_bytes +
                           info.reduction_weight_bytes + info.reduction_control_bytes;
    *out = info;
    return RK_NPU_OK;
}

int rk_npu_w4a8_memory_query(const rk_npu_w4a8_config* cfg, rk_npu_w4a8_memory_info* out) {
    if (!out) return RK_NPU_ERR_PARAM;
    rk_npu_w4a8_memory_info_ex info{};
    const int rc = rk_npu_w4a8_memory_query_ex(cfg, nullptr, &info);
    if (!rc) *out = info.base;
    return rc;
}

// reference src/rk_npu_w4a8.cpp:208-285
rk_npu_w4a8_weights* rk_npu_w4a8_weights_create(rk_npu_iommu_domain* domain,
                                                const rk_npu_i4_weight_config* cfg,
                                                const int8_t* B, const float* w_scale) {
    if (!domain || !domain->ctx || !cfg || !B || !w_scale || !valid_shape(cfg->K, cfg->N))
        return nullptr;
    if (cfg->N > INT_MAX - 63) return nullptr;
    rk_npu_w4a8_weight_info info{};
    info.config = *cfg;
    info.safe_k_tile = cfg->k_tile;
    info.multiplier = 1.0;
    if (cfg->k_tile == 0) {
        const double factor = rkhost::w4a8_env_multiplier();
        if (factor < 1) return nullptr;
        rkhost::W4Profile profile;
        if (rkhost::w4a8_make_profile(cfg->K, cfg->N, factor, B, w_scale, &profile)) return nullptr;
        return rkhost::w4a8_create_weights(domain, profile.info(profile.limit), B, w_scale, &profile);
    }
    if (!weight_key_valid(cfg->K, cfg->N, cfg->k_tile)) return nullptr;
    if (cfg->k_tile > kKTileUniversal &&
        largest_certified_tile(B, cfg->K, cfg->N, cfg->k_tile) != cfg->k_tile)
        return nullptr;
    return rkhost::w4a8_create_weights(domain, info, B, w_scale, nullptr);
}

void rk_npu_w4a8_weights_free(rk_npu_w4a8_weights* weights) { delete weights; }

int rk_npu_w4a8_weights_query(const rk_npu_w4a8_weights* weights, rk_npu_w4a8_weight_info* info) {
    if (!weights || !info) return RK_NPU_ERR_PARAM;
    *info = weights->info;
    return RK_NPU_OK;
}

rk_npu_w4a8_workspace* rk_npu_w4a8_workspace_create_ex(rk_npu_iommu_domain* domain,
                                                       const rk_npu_w4a8_config* cfg,
                                                       const rk_npu_w4a8_options* options) {
    if (!domain || !domain->ctx || !cfg) return nullptr;
    rk_npu_w4a8_memory_info_ex info{};
    if (rk_npu_w4a8_memory_query_ex(cfg, options, &info)) return nullptr;
    std::unique_ptr<rk_npu_w4a8_workspace> ws(new (std::nothrow) rk_npu_w4a8_workspace());
    if (!ws) return nullptr;
    if (read_options(options, cfg->M, ws->policy)) return nullptr;
    ws->owner.bind(domain);
    ws->config = *cfg;
    const int M = cfg->M, N = cfg->N, K = cfg->K;
    std::lock_guard<std::mutex> lock(domain->ctx->submit_mutex);
    const size_t rows = (size_t)rkh_align_up(M, RKH_ROW_ALIGN);
    if (ws->a_raw.alloc(ws->owner, (size_t)M * K * 4, false) ||
        ws->a_tiled.alloc(ws->owner, rkh_tiled_i8_bytes(M, K, RKH_ROW_ALIGN)) ||
        ws->a_scale.alloc(ws->owner, rows * sizeof(float)) ||
        ws->c_out.alloc(ws->owner, (size_t)M * N * 4, false) ||
        ws->row_max.alloc(ws->owner, rows * (size_t)(N / 64 + 1) * sizeof(uint32_t)) ||
        ws->flag.init(ws->owner))
        return nullptr;
    const size_t scratch = splitk_scratch_bytes(M, N, K, true);
    if (scratch && ws->splitk.alloc(ws->owner, scratch)) return nullptr;
    ws->stage_a.init((size_t)M * K * 4);
    ws->stage_c.init((size_t)M * N * 4);
    if (rkh_sync(domain->ctx->stream)) return nullptr;
    return ws.release();
}

rk_npu_w4a8_workspace* rk_npu_w4a8_workspace_create(rk_npu_iommu_domain* domain,
                                                    const rk_npu_w4a8_config* cfg) {
    return rk_npu_w4a8_workspace_create_ex(domain, cfg, nullptr);
}

void rk_npu_w4a8_workspace_free(rk_npu_w4a8_workspace* workspace) { delete workspace; }

int rk_npu_w4a8_run_f32(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w, const float* A,
                        float* C, rk_npu_w4a8_timings* t) {
    return run_host(ws, w, A, C, false, Out::F32, t);
}
int rk_npu_w4a8_run_f16(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w, const uint16_t* A,
                        uint16_t* C, rk_npu_w4a8_timings* t) {
    return run_host(ws, w, A, C, true, Out::F16, t);
}
int rk_npu_w4a8_run_swiglu_f32(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w,
                               const float* A, float* middle, rk_npu_w4a8_timings* t) {
    return run_host(ws, w, A, middle, false, Out::SwiGLU, t);
}
int rk_npu_w4a8_run_i32(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w, const float* A,
                        int32_t* acc) {
    return run_host(ws, w, A, acc, false, Out::I32, nullptr);
}
int rk_npu_w4a8_run_f32_device(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w,
                               const float* A, float* C) {
    return run_device(ws, w, A, C, false, Out::F32);
}
int rk_npu_w4a8_run_f16_device(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w,
                               const uint16_t* A, uint16_t* C) {
    return run_device(ws, w, A, C, true, Out::F16);
}

// reference src/rk_npu_w4a8.cpp:354-380
int rk_npu_w4a8_run_ffn_f32(rk_npu_w4a8_workspace* gu, const rk_npu_w4a8_weights* guw,
                            rk_npu_w4a8_workspace* dn, const rk_npu_w4a8_weights* dnw,
                            const float* A, float* middle, float* C,
                            rk_npu_w4a8_ffn_timings* metrics) {
    if (metrics) *metrics = rk_npu_w4a8_ffn_timings{};
    int rc = validate_ffn(gu, guw, dn, dnw, A, middle, C);
    if (rc) return rc;
    BusyLock gate_lock(gu->busy);
    if (!gate_lock) return RK_NPU_ERR_BUSY;
    BusyLock down_lock(dn->busy);
    if (!down_lock) return RK_NPU_ERR_BUSY;
    const auto t0 = Clock::now();
    rk_npu_ctx* ctx = gu->owner.ctx;
    const int M = gu->config.M, F = gu->config.N / 2;
    const size_t a_bytes = (size_t)M * gu->config.K * 4, c_bytes = (size_t)M * dn->config.N * 4;
    const size_t mid_bytes = (size_t)M * F * 4;
    const bool direct_in = gu->stage_a.direct(a_bytes), direct_out = dn->stage_c.direct(c_bytes);
    StageTimer timer(ctx->stream, metrics != nullptr);
    const void* src = direct_in ? gu->stage_a.fill(A, a_bytes) : gu->a_raw.as<>(); // before the submission lock
    {
        std::lock_guard<std::mutex> submit(ctx->submit_mutex);
        if (!direct_in) rc = map_error(gu->stage_a.upload(ctx->stream, gu->a_raw.as<>(), A, a_bytes));
        timer.mark();                                                                        // 0
        // middle lives in the gate/up workspace's result buffer (on the device: the
        // re-quantization reads it back)
        if (!rc) rc = enqueue(gu, guw, src, false, gu->c_out.as<>(), Out::SwiGLU, true, nullptr, &timer, direct_in); // 1,2
        if (!rc)
            rc = enqueue(dn, dnw, gu->c_out.as<>(), false, direct_out ? dn->stage_c.data() : dn->c_out.as<>(), Out::F32,
                         false, gu, &timer);                                                                         // 3,4
        if (!rc) rc = gu->flag.enqueue_readback(ctx->stream);
        if (!rc) rc = dn->flag.enqueue_readback(ctx->stream);
    }
    int wait = map_error(rkh_sync(ctx->stream));
    if (rc || wait) return rc ? rc : wait;
    const bool bad_in = gu->flag.consume(ctx->stream);
    const bool bad_mid = dn->flag.consume(ctx->stream);
    if (bad_in || bad_mid) return RK_NPU_ERR_PARAM; // NaN/Inf input or non-finite middle
    const auto t1 = Clock::now();
    // the middle goes through the gate/up workspace's output mirror (unused by the kernels in this call)
    rc = map_error(gu->stage_c.download(ctx->stream, middle, gu->c_out.as<>(), mid_bytes));
    if (!rc && !direct_out) rc = map_error(dn->stage_c.download(ctx->stream, C, dn->c_out.as<>(), c_bytes));
    if (!rc) rc = map_error(gu->stage_c.finish_download(ctx->stream, middle, mid_bytes));
    if (!rc && !direct_out) rc = map_error(dn->stage_c.finish_download(ctx->stream, C, c_bytes));
    if (!rc && direct_out) dn->stage_c.finish(C, c_bytes);
    if (metrics) {
        const double copy = elapsed_us(t1);
        fill_timings(&metrics->gate_up, timer, 0, true, copy, 0.0);
        metrics->gate_up.reduce_us = 0.0;
        metrics->gate_up.total_us = timer.span_us(0, 2);
        fill_timings(&metrics->down, timer, 2, false, 0.0, 0.0);
        metrics->down.total_us = timer.span_us(2, 4);
        metrics->total_us = elapsed_us(t0);
    }
    return rc;
}

int rk_npu_w4a8_run_ffn_f32_device(rk_npu_w4a8_workspace* gu, const rk_npu_w4a8_weights* guw,
                                   rk_npu_w4a8_workspace* dn, const rk_npu_w4a8_weights* dnw,
                                   const float* A, float* middle, float* C) {
    int rc = validate_ffn(gu, guw, dn, dnw, A, middle, C);
    if (rc) return rc;
    BusyLock gate_lock(gu->busy);
    if (!gate_lock) return RK_NPU_ERR_BUSY;
    BusyLock down_lock(dn->busy);
    if (!down_lock) return RK_NPU_ERR_BUSY;
    rk_npu_ctx* ctx = gu->owner.ctx;
    std::lock_guard<std::mutex> submit(ctx->submit_mutex);
    note_pending_flag(ctx, gu->flag.device());
    note_pending_flag(ctx, dn->flag.device());
    rc = enqueue(gu, guw, A, false, middle, Out::SwiGLU, true, nullptr, nullptr);
    if (!rc) rc = enqueue(dn, dnw, middle, false, C, Out::F32, false, gu, nullptr);
    return rc;
}

// Profiling hook: only the GEMV / GEMM stage (fp16 or fp32 output), on the
// activations the previous run left in the workspace.
int rk_npu_w4a8_workspace_rerun_gemm_device(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w,
                                            void* C, int half) {
    int rc = validate(ws, w, C, ws, false);
    if (rc) return rc;
    BusyLock lock(ws->busy);
    if (!lock) return RK_NPU_ERR_BUSY;
    std::lock_guard<std::mutex> submit(ws->owner.ctx->submit_mutex);
    return enqueue_gemm(ws, w, C, half ? Out::F16 : Out::F32, false);
}

int rk_npu_w4a8_workspace_read_quantized(rk_npu_w4a8_workspace* ws, int8_t* q, float* a_scale) {
    if (!ws || !q) return RK_NPU_ERR_PARAM;
    BusyLock lock(ws->busy);
    if (!lock) return RK_NPU_ERR_BUSY;
    const int M = ws->config.M, K = ws->config.K;
    const int KB = (int)(rkh_align_up(K, RKH_K_ALIGN) / 32);
    std::vector<uint8_t> tiled(ws->a_tiled.bytes());
    rk_npu_ctx* ctx = ws->owner.ctx;
    int rc = rkh_d2h(ctx->stream, tiled.data(), ws->a_tiled.as<>(), tiled.size());
    if (!rc && a_scale) rc = rkh_d2h(ctx->stream, a_scale, ws->a_scale.as<>(), (size_t)M * sizeof(float));
    if (!rc) rc = rkh_sync(ctx->stream);
    if (rc) return map_error(rc);
    for (int m = 0; m < M; ++m)
        for (int k = 0; k < K; ++k) {
            const size_t off = ((size_t)(m >> 5) * KB + (k >> 5)) * 1024 +
                               (size_t)((m & 31) + 32 * ((k & 31) >> 4)) * 16 + (k & 15);
            q[(size_t)m * K + k] = (int8_t)tiled[off];
        }
    return RK_NPU_OK;
}

} // extern "C"
