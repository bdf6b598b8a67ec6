// W8A8 typed GEMM operators: handles, validation, byte accounting and the
// kernel sequence  quantize rows -> GEMV / MFMA GEMM with fused dequant.
//
// Replaces the executor of the reference (src/rk_npu_quant_matmul.cpp:799-1020,
// a CPU pack / NPU submit / CPU reduce pipeline over K waves with two helper
// threads) by two kernel launches on one stream.  Entry points, argument
// checks and their order follow src/rk_npu_quant_matmul.cpp:1696-1960.
#include <sched.h>

#include <algorithm>
#include <new>

#include "rk_host.h"
#include "rk_npu_hip.h"
#include "rk_npu_quant_matmul.h"

using namespace rkhost;

namespace {

constexpr int kMinChannelTile = 32;   // reference N granularity of one NPU core
constexpr int kNTileSafeMax = 3072;   // reference src/rk_npu_quant_matmul.cpp: n_tile limit

int align_up_i(int v, int a) { return (v + a - 1) / a * a; }
int ceil_div_i(int a, int b) { return (a + b - 1) / b; }

bool supported_mask(uint32_t m) { return m == 1u || m == 2u || m == 4u || m == 3u || m == 7u; }

uint64_t process_cpu_mask() {
    cpu_set_t set;
    CPU_ZERO(&set);
    if (sched_getaffinity(0, sizeof(set), &set) != 0) return ~0ull;
    uint64_t mask = 0;
    for (int i = 0; i < 64; ++i)
        if (CPU_ISSET(i, &set)) mask |= 1ull << i;
    return mask;
}

struct Traits {
    int in_dtype;   // rkh_dtype of A
    int out_epi;    // rkh_epilogue
    int quant;      // 0 none, 1 dynamic, 2 static
    bool valid;
};
Traits traits(rk_npu_matmul_op_kind kind) {
    switch (kind) {
    case RK_NPU_MATMUL_I8I8I32: return {RKH_I8, RKH_EPI_I32, 0, true};
    case RK_NPU_MATMUL_F16I8F16_DYNAMIC: return {RKH_F16, RKH_EPI_F16, 1, true};
    case RK_NPU_MATMUL_F16I8F16_STATIC: return {RKH_F16, RKH_EPI_F16, 2, true};
    case RK_NPU_MATMUL_F32I8F32_DYNAMIC: return {RKH_F32, RKH_EPI_F32, 1, true};
    case RK_NPU_MATMUL_F32I8F32_STATIC: return {RKH_F32, RKH_EPI_F32, 2, true};
    }
    return {0, 0, 0, false};
}
size_t elem_bytes(int dtype) { return dtype == RKH_F32 || dtype == RKH_I32 ? 4 : dtype == RKH_F16 ? 2 : 1; }
int out_dtype(int epi) { return epi == RKH_EPI_I32 ? RKH_I32 : epi == RKH_EPI_F16 ? RKH_F16 : RKH_F32; }

bool valid_weight_config(const rk_npu_matmul_weight_config* c) {
    return c && c->K > 0 && c->N > 0 && c->k_tile > 0 && c->k_tile <= c->K;
}

// reference src/rk_npu_quant_matmul.cpp:153-181
bool valid_strategy(const rk_npu_matmul_strategy* s) {
    if (!s || !traits(s->op_kind).valid || s->M <= 0 || s->N <= 0 || s->K <= 0 ||
        s->k_tile <= 0 || s->k_tile > s->K || s->n_tile <= 0 || s->n_tile > kNTileSafeMax ||
        s->a_layout < RK_NPU_MATMUL_A_LAYOUT_NORMAL || s->a_layout > RK_NPU_MATMUL_A_LAYOUT_PANEL16 ||
        s->c_layout < RK_NPU_MATMUL_C_LAYOUT_NATIVE || s->c_layout > RK_NPU_MATMUL_C_LAYOUT_PANEL16 ||
        !supported_mask(s->npu_core_mask) || s->cpu_core_mask == 0 || s->cpu_threads <= 0 ||
        s->cpu_threads != __builtin_popcountll(s->cpu_core_mask))
        return false;
    if (s->cpu_core_mask & ~process_cpu_mask()) return false;
    const int align_n = std::max(kMinChannelTile, align_up_i(s->N, kMinChannelTile));
    const int nt = std::min(align_n, align_up_i(s->n_tile, kMinChannelTile));
    return ceil_div_i(align_n, nt) >= __builtin_popcount(s->npu_core_mask);
}

struct Weights {
    Owner owner;
    int K = 0, N = 0, k_tile = 0;
    DeviceBuffer tiled;   // tiled int8, align256(N) x align256(K)
    DeviceBuffer w_scale; // [N] fp32 (absent for i8i8i32)
};

// reference src/rk_npu_quant_matmul.cpp:1786-1834
Weights* create_weights(rk_npu_iommu_domain* domain, const rk_npu_matmul_weight_config* config,
                        const int8_t* B, const float* w_scale, bool scaled) {
    if (!domain || !domain->ctx || !valid_weight_config(config) || !B) return nullptr;
    if (scaled && !finite_positive(w_scale, (size_t)config->N)) return nullptr;
    std::unique_ptr<Weights> w(new (std::nothrow) Weights());
    if (!w) return nullptr;
    w->owner.bind(domain);
    w->K = config->K;
    w->N = config->N;
    w->k_tile = config->k_tile;
    rk_npu_ctx* ctx = domain->ctx;
    std::lock_guard<std::mutex> lock(ctx->submit_mutex);
    DeviceBuffer raw;
    if (upload(w->owner, raw, B, (size_t)w->K * w->N)) return nullptr;
    if (w->tiled.alloc(w->owner, rkh_tiled_i8_bytes(w->N, w->K, RKH_COL_ALIGN), false)) return nullptr;
    if (rkh_pack_w8(ctx->stream, raw.as<int8_t>(), w->K, w->N, 0, w->tiled.as<>())) return nullptr;
    if (scaled) {
        if (upload(w->owner, w->w_scale, w_scale, (size_t)w->N * sizeof(float))) return nullptr;
    }
    if (rkh_sync(ctx->stream)) return nullptr;
    return w.release();
}

} // namespace

// The three public weight handle types are opaque aliases of Weights.

struct rk_npu_matmul_workspace {
    Owner owner;
    rk_npu_matmul_strategy strategy{};
    Traits t{};
    DeviceBuffer a_raw;    // caller's A as uploaded
    DeviceBuffer a_tiled;  // quantized activations, tiled int8
    DeviceBuffer a_scale;  // [align128(M)] fp32
    DeviceBuffer c_out;    // [M, N] result before the copy back
    DeviceBuffer splitk;   // int32 scratch when the shape may split K
    HostStage stage_a, stage_scale, stage_c; // pinned mirrors of small A / static scales / C
    BadFlag flag;
    std::atomic_flag busy = ATOMIC_FLAG_INIT;
};

namespace {

rkh_gemm_args gemm_args(rk_npu_matmul_workspace* ws, const Weights& w, void* dC) {
    const auto& s = ws->strategy;
    rkh_gemm_args g{};
    g.A = ws->a_tiled.as<>();
    g.W = w.tiled.as<>();
    g.M = s.M;
    g.N = s.N;
    g.K = s.K;
    g.a_scale = ws->a_scale.as<float>();
    g.w_scale = w.w_scale.as<float>();
    g.epilogue = ws->t.out_epi;
    g.C = dC;
    g.ldc = s.N;
    g.splitk_acc = ws->splitk ? ws->splitk.as<int32_t>() : nullptr;
    return g;
}

// Enqueue quantize + GEMM on the context's stream (one fused kernel for
// decode-sized M, unless A is a pinned host mirror).  dA / dC are device-
// visible pointers; static scales are expected in the workspace's a_scale buffer.
int enqueue(rk_npu_matmul_workspace* ws, const Weights& w, const void* dA, void* dC, bool a_is_host = false) {
    const auto& s = ws->strategy;
    rkh_quant_args q{};
    q.src = dA;
    q.src_is_host = a_is_host ? 1 : 0;
    q.in_dtype = ws->t.in_dtype;
    q.mode = ws->t.quant == 0 ? RKH_Q_COPY_I8 : ws->t.quant == 1 ? RKH_Q_W8_DYNAMIC : RKH_Q_W8_STATIC;
    q.M = s.M;
    q.K = s.K;
    q.scale = ws->t.quant == 0 ? nullptr : ws->a_scale.as<float>();
    q.dst = ws->a_tiled.as<>();
    const rkh_gemm_args g = gemm_args(ws, w, dC);
    return map_error(rkh_quant_gemm(ws->owner.ctx->stream, &q, &g));
}

// GEMV / GEMM stage on the activations already quantized into the workspace.
int enqueue_gemm(rk_npu_matmul_workspace* ws, const Weights& w, void* dC) {
    const rkh_gemm_args g = gemm_args(ws, w, dC);
    return map_error(rkh_gemm(ws->owner.ctx->stream, &g));
}

int check_run(rk_npu_matmul_workspace* ws, const Weights* w, rk_npu_matmul_op_kind kind,
              const void* A, const void* C) {
    if (!ws || !w || !A || !C || ws->strategy.op_kind != kind) return RK_NPU_ERR_PARAM;
    if (!w->owner.same(ws->owner)) return RK_NPU_ERR_DOMAIN;
    if (w->K != ws->strategy.K || w->N != ws->strategy.N || w->k_tile != ws->strategy.k_tile)
        return RK_NPU_ERR_PARAM;
    return RK_NPU_OK;
}

// Blocking host-pointer run: upload A (and static scales), kernels, download C.
int run_host(rk_npu_matmul_workspace* ws, const Weights* w, rk_npu_matmul_op_kind kind,
             const void* A, const float* a_scale, void* C) {
    int rc = check_run(ws, w, kind, A, C);
    if (rc) return rc;
    BusyLock lock(ws->busy);
    if (!lock) return RK_NPU_ERR_BUSY;
    const auto& s = ws->strategy;
    rk_npu_ctx* ctx = ws->owner.ctx;
    const size_t a_bytes = (size_t)s.M * s.K * elem_bytes(ws->t.in_dtype);
    const size_t c_bytes = (size_t)s.M * s.N * elem_bytes(out_dtype(ws->t.out_epi));
    // Small operands skip the copies: the kernels read A from / write C into the
    // pinned mirrors.  Static scales are read by every workgroup of the GEMM, so
    // they are always uploaded (from their mirror when there is one).
    const bool direct_in = ws->stage_a.direct(a_bytes), direct_out = ws->stage_c.direct_out(c_bytes);
    const size_t scale_bytes = (size_t)s.M * sizeof(float);
    // the mirrors are filled before the context's submission lock is taken
    const void* src = direct_in ? ws->stage_a.fill(A, a_bytes) : ws->a_raw.as<>();
    const void* scale_src = a_scale;
    if (ws->t.quant == 2 && ws->stage_scale) scale_src = ws->stage_scale.fill(a_scale, scale_bytes);
    {
        std::lock_guard<std::mutex> submit(ctx->submit_mutex);
        if (!direct_in) rc = map_error(ws->stage_a.upload(ctx->stream, ws->a_raw.as<>(), A, a_bytes));
        if (!rc && ws->t.quant == 2)
            rc = map_error(rkh_h2d(ctx->stream, ws->a_scale.as<>(), scale_src, scale_bytes));
        if (!rc) rc = enqueue(ws, *w, src, direct_out ? ws->stage_c.data() : ws->c_out.as<>(), direct_in);
        if (!rc && !direct_out) rc = map_error(ws->stage_c.download(ctx->stream, C, ws->c_out.as<>(), c_bytes));
    }
    if (rc || direct_out) {
        const int wait = map_error(rkh_sync(ctx->stream));
        if (!rc && !wait) ws->stage_c.finish(C, c_bytes);
        return rc ? rc : wait;
    }
    return map_error(ws->stage_c.finish_download(ctx->stream, C, c_bytes));
}

int run_device(rk_npu_matmul_workspace* ws, const Weights* w, rk_npu_matmul_op_kind kind,
               const void* dA, void* dC) {
    int rc = check_run(ws, w, kind, dA, dC);
    if (rc) return rc;
    BusyLock lock(ws->busy);
    if (!lock) return RK_NPU_ERR_BUSY;
    std::lock_guard<std::mutex> submit(ws->owner.ctx->submit_mutex);
    return enqueue(ws, *w, dA, dC);
}

// reference src/rk_npu_kn_plan.cpp:43-116 (logical RK3588 payload sizes)
int weights_memory_query(const rk_npu_matmul_weight_config* c, bool scaled,
                         rk_npu_matmul_weight_requirements* out) {
    if (!valid_weight_config(c) || !out) return RK_NPU_ERR_PARAM;
    std::memset(out, 0, sizeof(*out));
    const uint64_t np = (uint64_t)std::max(kMinChannelTile, align_up_i(c->N, kMinChannelTile));
    for (int k0 = 0; k0 < c->K; k0 += c->k_tile) {
        const int kt = std::min(c->k_tile, c->K - k0);
        out->packed_b_bytes += (uint64_t)align_up_i(kt, 32) * np;
        ++out->wave_count;
    }
    out->scale_bytes = scaled ? (uint64_t)c->N * sizeof(float) : 0;
    out->bytes = out->packed_b_bytes + out->scale_bytes;
    out->buffer_count = 1;
    return RK_NPU_OK;
}

} // namespace

extern "C" {

void rk_npu_matmul_autotune_config_init(rk_npu_matmul_autotune_config* cfg, int M, int N, int K) {
    if (!cfg) return;
    std::memset(cfg, 0, sizeof(*cfg));
    cfg->M = M;
    cfg->N = N;
    cfg->K = K;
    cfg->allowed_npu_core_mask = 7;
    cfg->warmup = 2;
    cfg->loops = 8;
    cfg->repeats = 3;
    cfg->timeout_ms = 500;
}

// reference src/rk_npu_quant_matmul.cpp:1131-1142,1696-1700
int rk_npu_matmul_k_partition_query(int M, int K, int k_tile) {
    if (M < 1 || K < 1 || k_tile < 1 || k_tile > K) return RK_NPU_ERR_PARAM;
    if (M <= 4) return RK_NPU_OK;
    if (K > k_tile && k_tile > 2048 && align_up_i(k_tile, kMinChannelTile) % 1024)
        return RK_NPU_ERR_PARAM;
    for (int k0 = 0; k0 < K; k0 += k_tile) {
        const int k = align_up_i(std::min(k_tile, K - k0), kMinChannelTile);
        if (k > 3072 && k < 4096) return RK_NPU_ERR_PARAM;
    }
    return RK_NPU_OK;
}

// reference src/rk_npu_quant_matmul.cpp:1702-1719 with the payload formulas of
// src/rk_npu_kn_plan.cpp:43-95.  control_bytes (NPU register command and task
// descriptor bytes) is reported as 0: no such buffers exist here.
int rk_npu_matmul_workspace_memory_query(const rk_npu_matmul_strategy* s,
                                         rk_npu_matmul_workspace_requirements* out) {
    if (!s || !out || !valid_strategy(s)) return RK_NPU_ERR_PARAM;
    std::memset(out, 0, sizeof(*out));
    const uint32_t waves = (uint32_t)ceil_div_i(s->K, s->k_tile);
    const uint64_t np = (uint64_t)std::max(kMinChannelTile, align_up_i(s->N, kMinChannelTile));
    const uint32_t in_slots = std::min<uint32_t>(waves, 2), out_slots = std::min<uint32_t>(waves, 3);
    out->wave_count = waves;
    out->input_bytes = (uint64_t)in_slots * s->M * align_up_i(std::min(s->k_tile, s->K), 32);
    out->output_bytes = (uint64_t)out_slots * s->M * np * sizeof(int32_t);
    out->control_bytes = 0;
    out->buffer_count = 2 * waves + in_slots + out_slots;
    out->bytes = out->input_bytes + out->output_bytes + out->control_bytes +
                 (uint64_t)s->M * sizeof(float);
    return RK_NPU_OK;
}

int rk_npu_i8i8i32_weights_memory_query(const rk_npu_matmul_weight_config* c,
                                        rk_npu_matmul_weight_requirements* out) {
    return weights_memory_query(c, false, out);
}
int rk_npu_f16i8f16_weights_memory_query(const rk_npu_matmul_weight_config* c,
                                         rk_npu_matmul_weight_requirements* out) {
    return weights_memory_query(c, true, out);
}
int rk_npu_f32i8f32_weights_memory_query(const rk_npu_matmul_weight_config* c,
                                         rk_npu_matmul_weight_requirements* out) {
    return weights_memory_query(c, true, out);
}

rk_npu_matmul_workspace* rk_npu_matmul_workspace_create(rk_npu_iommu_domain* domain,
                                                        const rk_npu_matmul_strategy* strategy) {
    if (!domain || !domain->ctx || !strategy || !valid_strategy(strategy)) return nullptr;
    std::unique_ptr<rk_npu_matmul_workspace> ws(new (std::nothrow) rk_npu_matmul_workspace());
    if (!ws) return nullptr;
    ws->owner.bind(domain);
    ws->strategy = *strategy;
    ws->t = traits(strategy->op_kind);
    const int M = strategy->M, N = strategy->N, K = strategy->K;
    std::lock_guard<std::mutex> lock(domain->ctx->submit_mutex);
    if (ws->a_raw.alloc(ws->owner, (size_t)M * K * elem_bytes(ws->t.in_dtype), false) ||
        ws->a_tiled.alloc(ws->owner, rkh_tiled_i8_bytes(M, K, RKH_ROW_ALIGN)) ||
        ws->a_scale.alloc(ws->owner, (size_t)rkh_align_up(M, RKH_ROW_ALIGN) * sizeof(float)) ||
        ws->c_out.alloc(ws->owner, (size_t)M * N * elem_bytes(out_dtype(ws->t.out_epi)), false) ||
        ws->flag.init(ws->owner))
        return nullptr;
    const size_t scratch = splitk_scratch_bytes(M, N, K, false);
    if (scratch && ws->splitk.alloc(ws->owner, scratch)) return nullptr;
    ws->stage_a.init((size_t)M * K * elem_bytes(ws->t.in_dtype));
    if (ws->t.quant == 2) ws->stage_scale.init((size_t)M * sizeof(float));
    ws->stage_c.init((size_t)M * N * elem_bytes(out_dtype(ws->t.out_epi)));
    if (rkh_sync(domain->ctx->stream)) return nullptr;
    return ws.release();
}

void rk_npu_matmul_workspace_free(rk_npu_matmul_workspace* workspace) { delete workspace; }

/* ---- i8i8i32 ---- */
rk_npu_i8i8i32_weights* rk_npu_i8i8i32_weights_create(rk_npu_iommu_domain* domain,
                                                      const rk_npu_matmul_weight_config* config,
                                                      const int8_t* B) {
    Weights* w = create_weights(domain, config, B, nullptr, false);
    return reinterpret_cast<rk_npu_i8i8i32_weights*>(w);
}
rk_npu_i8i8i32_weights* rk_npu_i8i8i32_weights_create_compress(
    rk_npu_iommu_domain* domain, const rk_npu_matmul_weight_config* config, const int8_t* B) {
    return rk_npu_i8i8i32_weights_create(domain, config, B);
}
void rk_npu_i8i8i32_weights_free(rk_npu_i8i8i32_weights* weights) {
    delete reinterpret_cast<Weights*>(weights);
}
int rk_npu_i8i8i32_run(rk_npu_matmul_workspace* ws, const rk_npu_i8i8i32_weights* weights,
                       const int8_t* A, int32_t* C) {
    return run_host(ws, reinterpret_cast<const Weights*>(weights), RK_NPU_MATMUL_I8I8I32, A,
                    nullptr, C);
}
int rk_npu_i8i8i32_run_device(rk_npu_matmul_workspace* ws, const rk_npu_i8i8i32_weights* weights,
                              const int8_t* A, int32_t* C) {
    return run_device(ws, reinterpret_cast<const Weights*>(weights), RK_NPU_MATMUL_I8I8I32, A, C);
}

/* ---- f16i8f16 ---- */
rk_npu_f16i8f16_weights* rk_npu_f16i8f16_weights_create(rk_npu_iommu_domain* domain,
                                                        const rk_npu_matmul_weight_config* config,
                                                        const int8_t* B, const float* w_scale) {
    return reinterpret_cast<rk_npu_f16i8f16_weights*>(create_weights(domain, config, B, w_scale, true));
}
rk_npu_f16i8f16_weights* rk_npu_f16i8f16_weights_create_compress(
    rk_npu_iommu_domain* domain, const rk_npu_matmul_weight_config* config, const int8_t* B,
    const float* w_scale) {
    return rk_npu_f16i8f16_weights_create(domain, config, B, w_scale);
}
void rk_npu_f16i8f16_weights_free(rk_npu_f16i8f16_weights* weights) {
    delete reinterpret_cast<Weights*>(weights);
}
int rk_npu_f16i8f16_run_dynamic(rk_npu_matmul_workspace* ws, const rk_npu_f16i8f16_weights* weights,
                                const uint16_t* A, uint16_t* C) {
    return run_host(ws, reinterpret_cast<const Weights*>(weights), RK_NPU_MATMUL_F16I8F16_DYNAMIC,
                    A, nullptr, C);
}
int rk_npu_f16i8f16_run_static(rk_npu_matmul_workspace* ws, const rk_npu_f16i8f16_weights* weights,
                               const uint16_t* A, const float* a_scale, uint16_t* C) {
    if (!ws || ws->strategy.op_kind != RK_NPU_MATMUL_F16I8F16_STATIC ||
        !finite_positive(a_scale, (size_t)ws->strategy.M))
        return RK_NPU_ERR_PARAM;
    return run_host(ws, reinterpret_cast<const Weights*>(weights), RK_NPU_MATMUL_F16I8F16_STATIC, A,
                    a_scale, C);
}
int rk_npu_f16i8f16_run_dynamic_device(rk_npu_matmul_workspace* ws,
                                       const rk_npu_f16i8f16_weights* weights, const uint16_t* A,
                                       uint16_t* C) {
    return run_device(ws, reinterpret_cast<const Weights*>(weights), RK_NPU_MATMUL_F16I8F16_DYNAMIC,
                      A, C);
}

// The f16i8f16 dynamic run without a workspace and without any allocation: the
// quantized rows, their scales and the K-split partial tiles live in this
// device's copy of the library's static scratch array instead of workspace
// buffers (same kernels, same launch plan as rk_npu_f16i8f16_run_dynamic_device).
// Layout of the scratch for one call, every part on a 256-byte boundary:
//   [row scales: align128(M) floats][tiled int8 rows][K-split partial tiles]
// Every call on a device shares that array; calls through one context are
// ordered on its stream, calls through different contexts of the same device
// race.  The array keeps the previous call's contents: the padding rows / k of
// the tiled rows are cleared first (a kernel, not a memset: the call may be
// recorded by a stream capture) whenever this call's shape has padding.
int rk_npu_f16i8f16_run_dynamic_noalloc_device(const rk_npu_f16i8f16_weights* weights, int M,
                                               const uint16_t* A, uint16_t* C) {
    const Weights* w = reinterpret_cast<const Weights*>(weights);
    if (!w || !A || !C || M < 1 || !w->w_scale) return RK_NPU_ERR_PARAM;
    rk_npu_ctx* ctx = w->owner.ctx;
    if (!ctx->scratch) return RK_NPU_ERR_NOMEM;
    auto round256 = [](size_t v) { return (v + 255) / 256 * 256; };
    const size_t scale_bytes = round256((size_t)rkh_align_up(M, RKH_ROW_ALIGN) * sizeof(float));
    const size_t tiled_bytes = round256(rkh_tiled_i8_bytes(M, w->K, RKH_ROW_ALIGN));
    // The K split over workgroups is an optimisation, not a need: without room for its int32
    // partial tiles the GEMM runs unsplit (integer sums: the same bits either way), so only rows
    // that do not fit by themselves are refused.
    size_t split_bytes = round256(splitk_scratch_bytes(M, w->N, w->K, false));
    if (scale_bytes + tiled_bytes > ctx->scratch_bytes) return RK_NPU_ERR_NOMEM;
    if (scale_bytes + tiled_bytes + split_bytes > ctx->scratch_bytes) split_bytes = 0;
    uint8_t* base = static_cast<uint8_t*>(ctx->scratch);
    rkh_quant_args q{};
    q.src = A;
    q.in_dtype = RKH_F16;
    q.mode = RKH_Q_W8_DYNAMIC;
    q.M = M;
    q.K = w->K;
    q.scale = reinterpret_cast<float*>(base);
    q.dst = base + scale_bytes;
    rkh_gemm_args g{};
    g.A = q.dst;
    g.W = w->tiled.as<>();
    g.M = M;
    g.N = w->N;
    g.K = w->K;
    g.a_scale = q.scale;
    g.w_scale = w->w_scale.as<float>();
    g.epilogue = RKH_EPI_F16;
    g.C = C;
    g.ldc = w->N;
    g.splitk_acc = split_bytes ? reinterpret_cast<int32_t*>(base + scale_bytes + tiled_bytes) : nullptr;
    std::lock_guard<std::mutex> submit(ctx->submit_mutex);
    int rc = RKH_OK;
    if (M % RKH_ROW_ALIGN || w->K % RKH_K_ALIGN) rc = rkh_fill32(ctx->stream, q.dst, 0u, tiled_bytes / 4);
    if (!rc) rc = rkh_quant_gemm(ctx->stream, &q, &g);
    return map_error(rc);
}

/* ---- f32i8f32 ---- */
rk_npu_f32i8f32_weights* rk_npu_f32i8f32_weights_create(rk_npu_iommu_domain* domain,
                                                        const rk_npu_matmul_weight_config* config,
                                                        const int8_t* B, const float* w_scale) {
    return reinterpret_cast<rk_npu_f32i8f32_weights*>(create_weights(domain, config, B, w_scale, true));
}
rk_npu_f32i8f32_weights* rk_npu_f32i8f32_weights_create_compress(
    rk_npu_iommu_domain* domain, const rk_npu_matmul_weight_config* config, const int8_t* B,
    const float* w_scale) {
    return rk_npu_f32i8f32_weights_create(domain, config, B, w_scale);
}
uint64_t rk_npu_f32i8f32_weights_compressed_layout_generation(const rk_npu_f32i8f32_weights*) {
    return 0;
}
void rk_npu_f32i8f32_weights_free(rk_npu_f32i8f32_weights* weights) {
    delete reinterpret_cast<Weights*>(weights);
}
int rk_npu_f32i8f32_run_dynamic(rk_npu_matmul_workspace* ws, const rk_npu_f32i8f32_weights* weights,
                                const float* A, float* C) {
    return run_host(ws, reinterpret_cast<const Weights*>(weights), RK_NPU_MATMUL_F32I8F32_DYNAMIC,
                    A, nullptr, C);
}
int rk_npu_f32i8f32_run_static(rk_npu_matmul_workspace* ws, const rk_npu_f32i8f32_weights* weights,
                               const float* A, const float* a_scale, float* C) {
    if (!ws || ws->strategy.op_kind != RK_NPU_MATMUL_F32I8F32_STATIC ||
        !finite_positive(a_scale, (size_t)ws->strategy.M))
        return RK_NPU_ERR_PARAM;
    return run_host(ws, reinterpret_cast<const Weights*>(weights), RK_NPU_MATMUL_F32I8F32_STATIC, A,
                    a_scale, C);
}
int rk_npu_f32i8f32_run_dynamic_device(rk_npu_matmul_workspace* ws,
                                       const rk_npu_f32i8f32_weights* weights, const float* A,
                                       float* C) {
    return run_device(ws, reinterpret_cast<const Weights*>(weights), RK_NPU_MATMUL_F32I8F32_DYNAMIC,
                      A, C);
}

// Profiling hook: only the GEMV / GEMM stage, on the activations the previous
// run left in the workspace.
int rk_npu_matmul_workspace_rerun_gemm_device(rk_npu_matmul_workspace* ws, const void* weights,
                                              void* C) {
    const Weights* w = static_cast<const Weights*>(weights);
    if (!ws || !w) return RK_NPU_ERR_PARAM;
    int rc = check_run(ws, w, ws->strategy.op_kind, C, C);
    if (rc) return rc;
    BusyLock lock(ws->busy);
    if (!lock) return RK_NPU_ERR_BUSY;
    std::lock_guard<std::mutex> submit(ws->owner.ctx->submit_mutex);
    return enqueue_gemm(ws, *w, C);
}

// Parity probe: de-tile the int8 activations of the last run.
int rk_npu_matmul_workspace_read_quantized(rk_npu_matmul_workspace* ws, int8_t* q, float* a_scale) {
    if (!ws || !q) return RK_NPU_ERR_PARAM;
    BusyLock lock(ws->busy);
    if (!lock) return RK_NPU_ERR_BUSY;
    const int M = ws->strategy.M, K = ws->strategy.K;
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
