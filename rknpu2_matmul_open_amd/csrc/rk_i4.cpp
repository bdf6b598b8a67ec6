// Exact W4A4 integer GEMM (include/rk_npu_matmul_i4.h).
//
// Replaces src/rk_npu_matmul_i4.cpp, rk_npu_i4_plan.cpp, rk_npu_i4_executor.cpp
// and rk_npu_i4_cpu.cpp of the reference.  There the NPU multiplies INT4 by
// INT4 into INT16 partials per K tile, which a CPU team widens and adds; here
// the activation codes are kept as int8 and go through the int4-weight MFMA
// GEMM with int32 accumulation, so a run is
//     [producer callbacks ->] code check -> upload -> re-tile -> GEMM -> download.
// Validation (ranges, order of checks, BUSY / DOMAIN / PARAM) and the logical
// byte accounting follow src/rk_npu_i4_plan.cpp:14-89 and
// src/rk_npu_i4_executor.cpp:65-75.
#include <algorithm>
#include <climits>
#include <cstring>
#include <new>
#include <vector>

#include "rk_host.h"
#include "rk_npu_matmul_i4.h"
#include "rk_w4a8_internal.h"

using namespace rkhost;

namespace {

constexpr int kKTileMax = 2048;      // reference src/rk_npu_i4_bounds.h:5
constexpr int kKTileUniversal = 480; // reference src/rk_npu_i4_bounds.h:6
constexpr int kNTileMax = 8128;      // reference src/rk_npu_i4_regs.h:10
constexpr int kCommandWords = 112;   // reference src/rk_npu_i4_regs.h:8 (only bounds the task count)

int64_t align_up64(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

// reference src/rk_npu_i4_plan.cpp:14-17
bool weight_valid(const rk_npu_i4_weight_config& c) {
    return c.K > 0 && c.K <= INT32_MAX / 64 && c.N > 0 && c.N <= INT_MAX - 63 && c.k_tile >= 32 &&
           c.k_tile <= kKTileMax && c.k_tile % 32 == 0;
}

// reference src/rk_npu_i4_plan.cpp:18-31 (native input layout)
bool config_valid(const rk_npu_i4_config& c) {
    if (!weight_valid({c.K, c.N, c.k_tile}) || c.M < 1 || c.m_tile < 1 || c.m_tile > 128) return false;
    const uint32_t m = c.npu_core_mask;
    if (!(m == 1 || m == 2 || m == 4 || m == 3 || m == 7)) return false;
    return c.n_tile >= 64 && c.n_tile <= kNTileMax && c.n_tile % 64 == 0 &&
           align_up64(c.N, 64) / 64 >= __builtin_popcount(m) && c.timeout_ms > 0 &&
           (c.pipeline == 0 || c.pipeline == 1) && c.cpu_threads >= 1 && c.cpu_threads <= 4;
}

// reference src/rk_npu_i4_plan.cpp:57-64
int weights_bytes(const rk_npu_i4_weight_config& c, uint64_t* bytes) {
    if (!weight_valid(c)) return RK_NPU_ERR_PARAM;
    *bytes = (uint64_t)align_up64(c.K, 32) * (uint64_t)align_up64(c.N, 64) / 2;
    return *bytes > UINT32_MAX ? RK_NPU_ERR_NOMEM : RK_NPU_OK; // one arena of the NPU's 32-bit address space
}

} // namespace

struct rk_npu_i4i4i32_weights {
    Owner owner;
    rk_npu_i4_weight_config config{};
    DeviceBuffer tiled;  // tiled int4
    DeviceBuffer colsum; // [N] int32 column sums of the codes (constant of the decode GEMV's digit split)
};

struct rk_npu_i4_workspace {
    Owner owner;
    rk_npu_i4_config config{};
    std::vector<int8_t> codes;    // [M, K] host copy assembled from producer tiles
    std::vector<uint8_t> tile;    // one producer tile
    DeviceBuffer a_raw;           // uploaded codes
    DeviceBuffer a_tiled;         // the same, MFMA-tiled
    DeviceBuffer c_out;           // [M, N] int32
    DeviceBuffer splitk;
    HostStage stage_a, stage_c;   // pinned mirrors of small codes / results, used in place by the kernels
    std::atomic_flag busy = ATOMIC_FLAG_INIT;
};

namespace {

bool codes_in_range(const int8_t* p, size_t n) {
    // (v + 8) as unsigned must be < 16; OR-reduce so the loop vectorises
    unsigned bad = 0;
    for (size_t i = 0; i < n; ++i) bad |= (unsigned)(uint8_t)(p[i] + 8) & 0xf0u;
    return bad == 0;
}

// Upload `codes`, re-tile, multiply, download.  The workspace is locked by the caller.
int execute(rk_npu_i4_workspace* ws, const rk_npu_i4i4i32_weights* w, const int8_t* codes, int32_t* C,
            rk_npu_i4_timings* t) {
    const rk_npu_i4_config& c = ws->config;
    rk_npu_ctx* ctx = ws->owner.ctx;
    const size_t c_bytes = (size_t)c.M * c.N * sizeof(int32_t);
    const bool direct_in = ws->stage_a.direct((size_t)c.M * c.K), direct_out = ws->stage_c.direct_out(c_bytes);
    int rc;
    auto start = Clock::now();
    {
        std::lock_guard<std::mutex> submit(ctx->submit_mutex);
        const size_t a_bytes = (size_t)c.M * c.K;
        rkh_quant_args q{};
        q.src = ws->a_raw.as<>();
        if (direct_in) {
            q.src = ws->stage_a.fill(codes, a_bytes);
            q.src_is_host = 1;
            rc = RK_NPU_OK;
        } else {
            rc = map_error(ws->stage_a.upload(ctx->stream, ws->a_raw.as<>(), codes, a_bytes));
        }
        q.in_dtype = RKH_I8;
        q.mode = RKH_Q_COPY_I8;
        q.M = c.M;
        q.K = c.K;
        q.dst = ws->a_tiled.as<>();
        rkh_gemm_args g{};
        g.A = ws->a_tiled.as<>();
        g.W = w->tiled.as<>();
        g.w_int4 = 1;
        g.w_colsum = w->colsum.as<int32_t>();
        g.M = c.M;
        g.N = c.N;
        g.K = c.K;
        g.epilogue = RKH_EPI_I32;
        g.C = direct_out ? ws->stage_c.data() : ws->c_out.as<>();
        g.ldc = c.N;
        g.splitk_acc = ws->splitk ? ws->splitk.as<int32_t>() : nullptr;
        if (!rc) rc = map_error(rkh_quant_gemm(ctx->stream, &q, &g));
        t->submit_us += elapsed_us(start);
        start = Clock::now();
        if (!rc) rc = map_error(rkh_sync(ctx->stream));
        t->sync_us += elapsed_us(start);
        start = Clock::now();
        if (!rc && direct_out) ws->stage_c.finish(C, c_bytes);
        else if (!rc) rc = map_error(ws->stage_c.download(ctx->stream, C, ws->c_out.as<>(), c_bytes));
    }
    const int wait = direct_out || rc ? RK_NPU_OK : map_error(ws->stage_c.finish_download(ctx->stream, C, c_bytes));
    t->reduce_us += elapsed_us(start);
    return rc ? rc : wait;
}

// reference src/rk_npu_i4_executor.cpp:65-75, src/rk_npu_i4_plan.cpp:172-176
int check_run(rk_npu_i4_workspace* ws, const rk_npu_i4i4i32_weights* w) {
    if (!w->owner.same(ws->owner)) return RK_NPU_ERR_DOMAIN;
    const rk_npu_i4_weight_config& wc = w->config;
    const rk_npu_i4_config& c = ws->config;
    return wc.K != c.K || wc.N != c.N || wc.k_tile != c.k_tile ? RK_NPU_ERR_PARAM : RK_NPU_OK;
}

} // namespace

extern "C" {

// reference src/rk_npu_matmul_i4.cpp:10-12
void rk_npu_i4_config_init(rk_npu_i4_config* cfg, int M, int N, int K) {
    if (cfg) *cfg = {M, N, K, 128, 480, 1024, 1, 500, 1, 1};
}

int rk_npu_i4_weights_memory_query(const rk_npu_i4_weight_config* cfg, uint64_t* bytes) {
    if (!cfg || !bytes) return RK_NPU_ERR_PARAM;
    return weights_bytes(*cfg, bytes);
}

// reference src/rk_npu_i4_plan.cpp:66-89.  tasks_per_wave is the number of
// (N tile, M panel) NPU tasks the configuration describes; control_bytes, the
// size of their command words and descriptors, is 0 here.
int rk_npu_i4_memory_query(const rk_npu_i4_config* cfg, rk_npu_i4_memory_info* out) {
    if (!cfg || !out || !config_valid(*cfg)) return RK_NPU_ERR_PARAM;
    rk_npu_i4_memory_info info{};
    const int rc = weights_bytes({cfg->K, cfg->N, cfg->k_tile}, &info.packed_weight_bytes);
    if (rc) return rc;
    info.wave_count = (uint32_t)((cfg->K + cfg->k_tile - 1) / cfg->k_tile);
    const uint64_t slots = std::min<uint32_t>(info.wave_count, 2u);
    info.input_bytes = slots * (uint64_t)cfg->M * (uint64_t)align_up64(std::min(cfg->K, cfg->k_tile), 32) / 2;
    info.partial_bytes = slots * (uint64_t)cfg->M * (uint64_t)align_up64(cfg->N, 64) * 2;
    const int cores = __builtin_popcount(cfg->npu_core_mask);
    const int blocks = (int)(align_up64(cfg->N, 64) / 64);
    uint64_t n_tiles = 0;
    for (int i = 0; i < cores; ++i) {
        const int64_t shard = (int64_t)(blocks / cores + (i < blocks % cores)) * 64;
        n_tiles += (uint64_t)((shard + cfg->n_tile - 1) / cfg->n_tile);
    }
    const uint64_t panels = ((uint64_t)cfg->M + cfg->m_tile - 1) / cfg->m_tile;
    const uint64_t tasks = n_tiles * panels;
    if (tasks > (uint64_t)(INT_MAX / kCommandWords) || info.input_bytes / slots > UINT32_MAX ||
        info.partial_bytes / slots > UINT32_MAX)
        return RK_NPU_ERR_NOMEM;
    info.tasks_per_wave = (uint32_t)tasks;
    info.control_bytes = 0;
    *out = info;
    return RK_NPU_OK;
}

// reference src/rk_npu_i4_plan.cpp:92-116
rk_npu_i4i4i32_weights* rk_npu_i4i4i32_weights_create(rk_npu_iommu_domain* domain,
                                                      const rk_npu_i4_weight_config* cfg, const int8_t* B) {
    uint64_t bytes = 0;
    if (!domain || !domain->ctx || !cfg || !B || weights_bytes(*cfg, &bytes)) return nullptr;
    if (cfg->k_tile > kKTileUniversal && !i4_tile_certified(B, cfg->K, cfg->N, cfg->k_tile)) return nullptr;
    std::unique_ptr<rk_npu_i4i4i32_weights> w(new (std::nothrow) rk_npu_i4i4i32_weights());
    if (!w) return nullptr;
    w->owner.bind(domain);
    w->config = *cfg;
    rk_npu_ctx* ctx = domain->ctx;
    std::lock_guard<std::mutex> lock(ctx->submit_mutex);
    DeviceBuffer raw, bad;
    if (upload(w->owner, raw, B, (size_t)cfg->K * cfg->N)) return nullptr;
    if (bad.alloc(w->owner, sizeof(int), true)) return nullptr;
    if (w->tiled.alloc(w->owner, rkh_tiled_i4_bytes(cfg->N, cfg->K, RKH_COL_ALIGN), false)) return nullptr;
    if (w->colsum.alloc(w->owner, (size_t)cfg->N * sizeof(int32_t), true)) return nullptr;
    if (rkh_pack_w4(ctx->stream, raw.as<int8_t>(), cfg->K, cfg->N, 0, w->tiled.as<>(), bad.as<int>(),
                    w->colsum.as<int32_t>()))
        return nullptr;
    int bad_host = 0;
    if (rkh_d2h(ctx->stream, &bad_host, bad.as<>(), sizeof(int)) || rkh_sync(ctx->stream)) return nullptr;
    if (bad_host) return nullptr; // a code outside [-8, 7]
    return w.release();
}

void rk_npu_i4i4i32_weights_free(rk_npu_i4i4i32_weights* weights) { delete weights; }

rk_npu_i4_workspace* rk_npu_i4_workspace_create(rk_npu_iommu_domain* domain, const rk_npu_i4_config* cfg) {
    rk_npu_i4_memory_info info{};
    if (!domain || !domain->ctx || !cfg || rk_npu_i4_memory_query(cfg, &info)) return nullptr;
    std::unique_ptr<rk_npu_i4_workspace> ws(new (std::nothrow) rk_npu_i4_workspace());
    if (!ws) return nullptr;
    ws->owner.bind(domain);
    ws->config = *cfg;
    const int M = cfg->M, N = cfg->N, K = cfg->K;
    std::lock_guard<std::mutex> lock(domain->ctx->submit_mutex);
    if (ws->a_raw.alloc(ws->owner, (size_t)M * K, false) ||
        ws->a_tiled.alloc(ws->owner, rkh_tiled_i8_bytes(M, K, RKH_ROW_ALIGN)) ||
        ws->c_out.alloc(ws->owner, (size_t)M * N * sizeof(int32_t), false))
        return nullptr;
    const size_t scratch = splitk_scratch_bytes(M, N, K, true);
    if (scratch && ws->splitk.alloc(ws->owner, scratch)) return nullptr;
    ws->stage_a.init((size_t)M * K);
    ws->stage_c.init((size_t)M * N * sizeof(int32_t));
    if (rkh_sync(domain->ctx->stream)) return nullptr;
    return ws.release();
}

void rk_npu_i4_workspace_free(rk_npu_i4_workspace* workspace) { delete workspace; }

// reference src/rk_npu_i4_cpu.cpp:33-51
int rk_npu_i4_pack_a_tile(const rk_npu_i4_input_tile* t, const int8_t* A, int lda) {
    if (!t || !A || !t->dst || t->m0 < 0 || t->rows <= 0 || t->rows > 128 || t->k0 < 0 || t->k <= 0 ||
        t->padded_k < t->k || t->padded_k > kKTileMax || t->padded_k % 32 || (int64_t)t->k0 + t->k > lda ||
        t->bytes < (uint64_t)t->rows * t->padded_k / 2)
        return RK_NPU_ERR_PARAM;
    std::memset(t->dst, 0, (size_t)t->rows * t->padded_k / 2);
    for (int m = 0; m < t->rows; ++m) {
        const int8_t* row = A + ((size_t)t->m0 + m) * lda + t->k0;
        for (int k = 0; k < t->k; ++k) {
            const int v = row[k];
            if (v < -8 || v > 7) return RK_NPU_ERR_PARAM;
            // element k of row m sits at code index (k/32 * rows + m) * 32 + k%32; even index = high nibble
            const size_t index = ((size_t)(k / 32) * t->rows + m) * 32 + k % 32;
            t->dst[index / 2] |= (uint8_t)((v & 15) << (index & 1 ? 0 : 4));
        }
    }
    return RK_NPU_OK;
}

int rk_npu_i4i4i32_run_with_producer(rk_npu_i4_workspace* ws, const rk_npu_i4i4i32_weights* w,
                                     rk_npu_i4_input_producer producer, void* user, int32_t* C,
                                     rk_npu_i4_timings* timings) {
    if (!ws || !w || !producer || !C) return RK_NPU_ERR_PARAM;
    BusyLock lock(ws->busy);
    if (!lock) return RK_NPU_ERR_BUSY;
    const auto t0 = Clock::now();
    rk_npu_i4_timings t{};
    int rc = check_run(ws, w);
    const rk_npu_i4_config& c = ws->config;
    if (!rc) {
        try {
            ws->codes.resize((size_t)c.M * c.K);
        } catch (const std::bad_alloc&) {
            rc = RK_NPU_ERR_NOMEM;
        }
    }
    const auto pack0 = Clock::now();
    for (int k0 = 0; !rc && k0 < c.K; k0 += c.k_tile) {
        const int k = std::min(c.k_tile, c.K - k0), padded = (int)align_up64(k, 32);
        for (int m0 = 0; !rc && m0 < c.M; m0 += c.m_tile) {
            const int rows = std::min(c.m_tile, c.M - m0);
            const size_t bytes = (size_t)rows * padded / 2;
            try {
                ws->tile.assign(bytes, 0);
            } catch (const std::bad_alloc&) {
                rc = RK_NPU_ERR_NOMEM;
                break;
            }
            const rk_npu_i4_input_tile tile{m0, rows, k0, k, padded, ws->tile.data(), (uint64_t)bytes};
            try {
                rc = producer(user, &tile);
            } catch (...) {
                rc = RK_NPU_ERR_PARAM;
            }
            if (rc) break;
            for (int m = 0; m < rows; ++m) {
                int8_t* row = ws->codes.data() + ((size_t)m0 + m) * c.K + k0;
                for (int j = 0; j < k; ++j) {
                    const size_t index = ((size_t)(j / 32) * rows + m) * 32 + j % 32;
                    const int q = (ws->tile[index / 2] >> (index & 1 ? 0 : 4)) & 15;
                    row[j] = (int8_t)(q >= 8 ? q - 16 : q);
                }
            }
        }
    }
    t.pack_us = elapsed_us(pack0);
    if (!rc) rc = execute(ws, w, ws->codes.data(), C, &t);
    t.total_us = elapsed_us(t0);
    if (timings) *timings = t;
    return rc;
}

// reference src/rk_npu_matmul_i4.cpp:46-60
int rk_npu_i4i4i32_run(rk_npu_i4_workspace* ws, const rk_npu_i4i4i32_weights* w, const int8_t* A, int32_t* C,
                       rk_npu_i4_timings* timings) {
    if (!ws || !A || !w || !C) return RK_NPU_ERR_PARAM;
    BusyLock lock(ws->busy);
    if (!lock) return RK_NPU_ERR_BUSY;
    const auto t0 = Clock::now();
    rk_npu_i4_timings t{};
    int rc = check_run(ws, w);
    const rk_npu_i4_config& c = ws->config;
    if (!rc) {
        const auto pack0 = Clock::now();
        if (!codes_in_range(A, (size_t)c.M * c.K)) rc = RK_NPU_ERR_PARAM;
        t.pack_us = elapsed_us(pack0);
    }
    if (!rc) rc = execute(ws, w, A, C, &t);
    t.total_us = elapsed_us(t0);
    if (timings) *timings = t;
    return rc;
}

} // extern "C"
