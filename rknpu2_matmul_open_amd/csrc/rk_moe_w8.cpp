// Routed W8A8 SwiGLU experts.
//
// Replaces src/rk_npu_moe_w8.cpp of the reference, where the CPU buckets
// (token, slot) pairs by expert, the NPU gathers rows and runs one GEMM job
// per <=128-row slice, and the CPU computes the SwiGLU middle row by row.
// Here one call is six kernels on one stream:
//   route (stable bucket by expert, 32-row padded) -> quantize tokens straight
//   into their sorted rows -> grouped gate/up GEMM with fused SwiGLU + row max
//   -> re-quantize (ties to even) -> grouped down GEMM -> weighted combine.
// Validation and its order follow src/rk_npu_moe_w8.cpp:293-310,574-608,846-875.
#include <algorithm>
#include <new>

#include <cerrno>
#include "rk_host.h"
#include "rk_npu_hip.h"
#include "rk_npu_moe_w8.h"

using namespace rkhost;

namespace {

constexpr int kMaxIntermediate = 8192; // the reference stops at 512 (fixed CPU row buffer)
constexpr int kMaxExperts = 2047;      // routed + shared must fit the route kernel's tables

bool valid(const rk_npu_moe_w8_weight_config& c) {
    return c.hidden >= 64 && c.hidden % 32 == 0 && c.intermediate >= 32 &&
           c.intermediate <= kMaxIntermediate && c.intermediate % 32 == 0 &&
           c.routed_experts >= 1 && c.routed_experts <= kMaxExperts &&
           (c.shared_expert == 0 || c.shared_expert == 1);
}
bool same(const rk_npu_moe_w8_weight_config& a, const rk_npu_moe_w8_weight_config& b) {
    return a.hidden == b.hidden && a.intermediate == b.intermediate &&
           a.routed_experts == b.routed_experts && a.shared_expert == b.shared_expert;
}
bool valid(const rk_npu_moe_w8_config& c) {
    return c.struct_size == sizeof(c) && valid(c.weights) && c.max_rows >= 1 && c.max_rows <= 256 &&
           c.top_k >= 1 && c.top_k <= std::min(c.weights.routed_experts, 8) && c.npu_cores >= 1 &&
           c.npu_cores <= 3 && c.cpu_threads >= 1 && c.cpu_threads <= 4 &&
           (c.native_input == 0 || c.native_input == 1) && c.timeout_ms >= 1 &&
           c.timeout_ms <= 60000 && c.middle == RK_NPU_MOE_MIDDLE_CPU;
}
// Expert formats (reference src/rk_npu_moe_w8.cpp:366-387).  W4 experts arrive as
// signed INT4 codes in the same int8 arrays; the arithmetic is that of the W8
// path with codes restricted to [-8, 7] (the reference's own test runs one body
// against both).  On the device they are packed two codes per byte (tiled int4,
// half the bytes to hold and to stream) and run on the int4 variant of the
// grouped kernel, whose integer sums equal the int8 path's exactly.
enum Mode { kW8 = 0, kW4 = 1, kRoutedW4SharedW8 = 2 };
bool expert_is_w4(int mode, int expert, int routed) {
    return mode == kW4 || (mode == kRoutedW4SharedW8 && expert < routed);
}
// reference :384-387 (8128 = widest INT4 task of the NPU)
bool valid_w4(const rk_npu_moe_w8_weight_config& c) {
    return valid(c) && c.hidden % 64 == 0 && c.intermediate % 64 == 0 && c.hidden <= 8128;
}
bool int4_codes(const int8_t* p, size_t n) {
    unsigned bad = 0;
    for (size_t i = 0; i < n; ++i) bad |= (unsigned)(uint8_t)(p[i] + 8) & 0xf0u;
    return bad == 0;
}
bool overlap(const void* a, size_t na, const void* b, size_t nb) {
    const auto x = reinterpret_cast<uintptr_t>(a), y = reinterpret_cast<uintptr_t>(b);
    return x <= y ? y - x < na : x - y < nb;
}

} // namespace

struct rk_npu_moe_w8_weights {
    Owner owner;
    rk_npu_moe_w8_weight_config config{};
    int mode = kW8;
    int count = 0;              // routed + shared
    int count4 = 0;             // leading experts held as int4 images (all of them, the routed ones, or none)
    size_t gate_stride = 0;     // bytes between int8 experts in gate_up
    size_t down_stride = 0;
    size_t gate_stride4 = 0;    // bytes between int4 experts in gate_up4
    size_t down_stride4 = 0;
    DeviceBuffer gate_up;       // (count - count4) x tiled int8 [align256(2I) x align256(H)], gate/up interleaved
    DeviceBuffer down;          // (count - count4) x tiled int8 [align256(H) x align256(I)]
    DeviceBuffer gate_up4;      // count4 x tiled int4, same geometry
    DeviceBuffer down4;
    DeviceBuffer gate_scales;   // count x [2I]
    DeviceBuffer down_scales;   // count x [H]
    uint64_t bytes() const {
        return gate_up.bytes() + down.bytes() + gate_up4.bytes() + down4.bytes() + gate_scales.bytes() +
               down_scales.bytes();
    }
};

struct rk_npu_moe_w8_workspace {
    Owner owner;
    rk_npu_moe_w8_config config{};
    int mode = kW8;
    int slots = 0, max_blocks = 0, sorted_rows = 0;
    DeviceBuffer input;        // [max_rows, H] fp32 (or int8) as uploaded
    DeviceBuffer token_scale;  // [max_rows]
    DeviceBuffer ids, routes;  // [max_rows, top_k]
    DeviceBuffer dest_rows;    // [max_rows, slots]
    DeviceBuffer blk_expert;   // [max_blocks]
    DeviceBuffer num_blocks;   // [2]
    DeviceBuffer a_tiled;      // sorted token rows, tiled int8 [sorted_rows x align256(H)]
    DeviceBuffer a_scale;      // [sorted_rows]
    DeviceBuffer hidden;       // [sorted_rows, I] fp32
    DeviceBuffer row_max;      // [sorted_rows][I/32] partial row maxima of hidden
    DeviceBuffer h_tiled;      // re-quantized hidden, tiled int8 [sorted_rows x align256(I)]
    DeviceBuffer h_scale;      // [sorted_rows]
    DeviceBuffer y;            // [sorted_rows, H] fp32 expert outputs
    DeviceBuffer out;          // [max_rows, H] fp32
    // pinned mirrors for the host-pointer entry points: tokens and result (read /
    // written in place by the kernels when a call's share fits), routing table
    // [ids | coefficients | token scales] for max_rows
    HostStage stage_in, stage_out, stage_route;
    BadFlag flag;
    std::atomic_flag busy = ATOMIC_FLAG_INIT;
    uint64_t bytes() const {
        return input.bytes() + token_scale.bytes() + ids.bytes() + routes.bytes() +
               dest_rows.bytes() + blk_expert.bytes() + num_blocks.bytes() + a_tiled.bytes() +
               a_scale.bytes() + hidden.bytes() + row_max.bytes() + h_tiled.bytes() +
               h_scale.bytes() + y.bytes() + out.bytes();
    }
    ~rk_npu_moe_w8_workspace() {
        if (owner.ctx) rkhost::forget_pending_flag(owner.ctx, flag.device());
    }
};

namespace {

// Kernel sequence on device-resident inputs.  d_input is fp32 [rows, H] when
// f32, else int8 [rows, H] with d_scales[rows].
int enqueue(rk_npu_moe_w8_workspace* ws, const rk_npu_moe_w8_weights* w, int rows,
            const void* d_input, bool f32, const float* d_scales, const int32_t* d_ids,
            const float* d_routes, float* d_out, StageTimer* timer, bool device_resident = false) {
    const auto& wc = ws->config.weights;
    const int H = wc.hidden, I = wc.intermediate;
    void* stream = ws->owner.ctx->stream;
    auto mark = [&] { if (timer) timer->mark(); };
    // A handful of fp32 tokens whose rows and routing table lie in device memory: two launches of
    // dot-product kernels instead of the five of the grouped path (every workgroup of a token reads
    // its row and its routing entries, which is why operands in the pinned host mirrors do not qualify).
    if (device_resident && f32 && rkh_moe_decode_applies(rows, H, I)) {
        rkh_moe_decode_args a{};
        a.x = static_cast<const float*>(d_input);
        a.ids = d_ids;
        a.routes = d_routes;
        a.rows = rows;
        a.top_k = ws->config.top_k;
        a.experts = wc.routed_experts;
        a.shared = wc.shared_expert ? 1 : 0;
        a.H = H;
        a.I = I;
        a.gate_W = w->gate_up ? w->gate_up.as<>() : nullptr;
        a.gate_W4 = w->gate_up4 ? w->gate_up4.as<>() : nullptr;
        a.down_W = w->down ? w->down.as<>() : nullptr;
        a.down_W4 = w->down4 ? w->down4.as<>() : nullptr;
        a.int4_experts = w->count4;
        a.gate_stride = w->gate_stride;
        a.gate_stride4 = w->gate_stride4;
        a.down_stride = w->down_stride;
        a.down_stride4 = w->down_stride4;
        a.gate_scales = w->gate_scales.as<float>();
        a.down_scales = w->down_scales.as<float>();
        a.hidden = ws->hidden.as<float>();
        a.row_max_bits = ws->row_max.as<uint32_t>();
        a.out = d_out;
        a.bad_flag = ws->flag.device();
        mark(); // 1: schedule
        mark(); // 2: input
        const int rc = rkh_moe_decode(stream, &a);
        mark(); // 3: gate
        mark(); // 4: middle
        mark(); // 5: down
        mark(); // 6: combine
        return map_error(rc);
    }
    // most row blocks this call can produce (the workspace's max_blocks is the same bound for max_rows)
    const int routed = rows * ws->config.top_k;
    const int call_blocks = std::min(ws->max_blocks, routed / 32 + std::min(wc.routed_experts, routed) +
                                                         (wc.shared_expert ? (rows + 31) / 32 : 0));

    rkh_moe_scatter_args r{};
    r.ids = d_ids;
    r.routes = d_routes;
    r.rows = rows;
    r.top_k = ws->config.top_k;
    r.experts = wc.routed_experts;
    r.shared = wc.shared_expert;
    r.dest_rows = ws->dest_rows.as<int>();
    r.blk_expert = ws->blk_expert.as<int>();
    r.num_blocks = ws->num_blocks.as<int>();
    r.max_blocks = ws->max_blocks;
    r.src = d_input;
    r.in_dtype = f32 ? RKH_F32 : RKH_I8;
    r.K = H;
    r.token_scale = f32 ? ws->token_scale.as<float>() : const_cast<float*>(d_scales);
    r.dst = ws->a_tiled.as<>();
    r.scale_rows = ws->a_scale.as<float>();
    r.bad_flag = ws->flag.device();
    mark(); // 1: schedule (routing is part of the scatter launch)
    int rc = rkh_moe_scatter(stream, &r);
    if (rc) return map_error(rc);
    mark(); // 2: input

    rkh_gemm_args g{};
    g.A = ws->a_tiled.as<>();
    g.W = w->gate_up ? w->gate_up.as<>() : nullptr;
    g.W4 = w->gate_up4 ? w->gate_up4.as<>() : nullptr;
    g.int4_experts = w->count4;
    g.w4_expert_stride = w->gate_stride4;
    g.M = ws->sorted_rows;
    g.N = 2 * I;
    g.K = H;
    g.interleave_F = I;
    g.a_scale = ws->a_scale.as<float>();
    g.w_scale = w->gate_scales.as<float>();
    g.epilogue = RKH_EPI_SWIGLU;
    g.C = ws->hidden.as<>();
    g.ldc = I;
    g.row_max_bits = ws->row_max.as<uint32_t>();
    g.blk_expert = ws->blk_expert.as<int>();
    g.num_blocks = ws->num_blocks.as<int>();
    g.max_blocks = call_blocks;
    g.w_expert_stride = w->gate_stride;
    g.ws_expert_stride = (size_t)2 * I;
    rc = rkh_gemm(stream, &g);
    if (rc) return map_error(rc);
    mark(); // 3: gate

    rkh_quant_args q2{};
    q2.src = ws->hidden.as<>();
    q2.in_dtype = RKH_F32;
    q2.mode = RKH_Q_REUSE_BITS_MOE;
    q2.M = ws->sorted_rows;
    q2.K = I;
    q2.scale = ws->h_scale.as<float>();
    q2.dst = ws->h_tiled.as<>();
    q2.row_max_bits = ws->row_max.as<uint32_t>();
    q2.row_max_parts = I / 32;
    q2.active_blocks = ws->num_blocks.as<int>();
    rc = rkh_quant_rows(stream, &q2);
    if (rc) return map_error(rc);
    mark(); // 4: middle

    rkh_gemm_args d{};
    d.A = ws->h_tiled.as<>();
    d.W = w->down ? w->down.as<>() : nullptr;
    d.W4 = w->down4 ? w->down4.as<>() : nullptr;
    d.int4_experts = w->count4;
    d.w4_expert_stride = w->down_stride4;
    d.M = ws->sorted_rows;
    d.N = H;
    d.K = I;
    d.a_scale = ws->h_scale.as<float>();
    d.w_scale = w->down_scales.as<float>();
    d.epilogue = RKH_EPI_F32;
    d.C = ws->y.as<>();
    d.ldc = H;
    d.blk_expert = ws->blk_expert.as<int>();
    d.num_blocks = ws->num_blocks.as<int>();
    d.max_blocks = call_blocks;
    d.w_expert_stride = w->down_stride;
    d.ws_expert_stride = (size_t)H;
    rc = rkh_gemm(stream, &d);
    if (rc) return map_error(rc);
    mark(); // 5: down

    rkh_moe_combine_args c{};
    c.Y = ws->y.as<float>();
    c.dest_rows = ws->dest_rows.as<int>();
    c.routes = d_routes;
    c.rows = rows;
    c.top_k = ws->config.top_k;
    c.shared = wc.shared_expert;
    c.H = H;
    c.out = d_out;
    rc = rkh_moe_combine(stream, &c);
    mark(); // 6: combine
    return map_error(rc);
}

int check_handles(const rk_npu_moe_w8_workspace* ws, const rk_npu_moe_w8_weights* w) {
    if (ws->mode != w->mode || !same(ws->config.weights, w->config)) return RK_NPU_ERR_PARAM;
    if (!w->owner.same(ws->owner)) return RK_NPU_ERR_DOMAIN;
    return RK_NPU_OK;
}

// reference src/rk_npu_moe_w8.cpp:846-875 (argument checks, BUSY) and :574-608
// (handle match, id / coefficient / scale validation before any device work).
int moe_run(rk_npu_moe_w8_workspace* ws, const rk_npu_moe_w8_weights* w, int rows,
            const void* input, bool f32, const float* scales, const int32_t* ids,
            const float* routes, float* output, rk_npu_moe_w8_timings* timings) {
    if (timings) *timings = rk_npu_moe_w8_timings{};
    if (!ws || !w || !input || !ids || !routes || !output || (!f32 && !scales) || rows < 1 ||
        rows > ws->config.max_rows)
        return RK_NPU_ERR_PARAM;
    const int H = ws->config.weights.hidden, top = ws->config.top_k;
    const size_t values = (size_t)rows * H, nslots = (size_t)rows * top;
    if (overlap(input, values * (f32 ? 4 : 1), output, values * 4) ||
        overlap(ids, nslots * 4, output, values * 4) || overlap(routes, nslots * 4, output, values * 4) ||
        (!f32 && overlap(scales, (size_t)rows * 4, output, values * 4)))
        return RK_NPU_ERR_PARAM;
    BusyLock lock(ws->busy);
    if (!lock) return RK_NPU_ERR_BUSY;
    const auto t0 = Clock::now();
    int rc = check_handles(ws, w);
    if (rc) return rc;
    const int E = ws->config.weights.routed_experts;
    size_t live = ws->config.weights.shared_expert ? (size_t)rows : 0;
    for (size_t i = 0; i < nslots; ++i) {
        if (ids[i] < 0 || ids[i] >= E || !std::isfinite(routes[i]) || routes[i] < 0)
            return RK_NPU_ERR_PARAM;
        if (routes[i] != 0) ++live;
    }
    if (!f32 && !finite_positive(scales, (size_t)rows)) return RK_NPU_ERR_PARAM;
    rk_npu_ctx* ctx = ws->owner.ctx;
    if (!live) {
        // every route dropped and no shared expert: the result is all zeros
        // and no device work is issued -- but fp32 input must still be finite
        if (f32) {
            const float* x = static_cast<const float*>(input);
            for (size_t i = 0; i < values; ++i)
                if (!std::isfinite(x[i])) return RK_NPU_ERR_PARAM;
        }
        std::fill_n(output, values, 0.0f);
        if (timings) timings->total_us = timings->combine_us = elapsed_us(t0);
        return RK_NPU_OK;
    }
    StageTimer timer(ctx->stream, timings != nullptr);
    // Where the copies go.  Tokens are read once each and the result is written
    // once, so when they fit their pinned mirrors the kernels use those in place.
    // The routing table is read by every token's workgroup: in place only for a
    // decode-sized call, otherwise uploaded (from its mirror, without a wait).
    const size_t in_bytes = values * (f32 ? 4 : 1), out_bytes = values * 4;
    const bool direct_in = ws->stage_in.direct(in_bytes), direct_out = ws->stage_out.direct_out(out_bytes);
    const bool direct_route = ws->stage_route && rows <= 16;
    const void* d_input = ws->input.as<>();
    const float* d_scales = ws->token_scale.as<float>();
    const int32_t* d_ids = ws->ids.as<int32_t>();
    const float* d_routes = ws->routes.as<float>();
    // the mirrors are filled before the context's submission lock is taken
    if (direct_in) d_input = ws->stage_in.fill(input, in_bytes);
    const void *h_ids = ids, *h_routes = routes, *h_scales = scales;
    if (ws->stage_route) {
        const size_t table = (size_t)ws->config.max_rows * top * 4;
        uint8_t* mirror = static_cast<uint8_t*>(ws->stage_route.data());
        std::memcpy(mirror, ids, nslots * 4);
        std::memcpy(mirror + table, routes, nslots * 4);
        if (!f32) std::memcpy(mirror + 2 * table, scales, (size_t)rows * 4);
        h_ids = mirror;
        h_routes = mirror + table;
        h_scales = mirror + 2 * table;
    }
    {
        std::lock_guard<std::mutex> submit(ctx->submit_mutex);
        if (!direct_in) rc = map_error(ws->stage_in.upload(ctx->stream, ws->input.as<>(), input, in_bytes));
        if (direct_route) {
            d_ids = static_cast<const int32_t*>(h_ids);
            d_routes = static_cast<const float*>(h_routes);
            if (!f32) d_scales = static_cast<const float*>(h_scales);
        } else {
            if (!rc && !f32) rc = map_error(rkh_h2d(ctx->stream, ws->token_scale.as<>(), h_scales, (size_t)rows * 4));
            if (!rc) rc = map_error(rkh_h2d(ctx->stream, ws->ids.as<>(), h_ids, nslots * 4));
            if (!rc) rc = map_error(rkh_h2d(ctx->stream, ws->routes.as<>(), h_routes, nslots * 4));
        }
        timer.mark(); // 0
        if (!rc)
            rc = enqueue(ws, w, rows, d_input, f32, d_scales, d_ids, d_routes,
                         direct_out ? static_cast<float*>(ws->stage_out.data()) : ws->out.as<float>(), &timer);
        if (!rc) rc = ws->flag.enqueue_readback(ctx->stream);
    }
    const int wait = map_error(rkh_sync(ctx->stream));
    if (rc || wait) return rc ? rc : wait;
    if (ws->flag.consume(ctx->stream)) return RK_NPU_ERR_PARAM; // NaN / Inf token
    const auto t1 = Clock::now();
    if (direct_out) {
        ws->stage_out.finish(output, out_bytes);
    } else {
        rc = map_error(ws->stage_out.download(ctx->stream, output, ws->out.as<>(), out_bytes));
        if (!rc) rc = map_error(ws->stage_out.finish_download(ctx->stream, output, out_bytes));
    }
    if (timings) {
        timings->schedule_us = timer.span_us(0, 1);
        timings->input_us = timer.span_us(1, 2);
        timings->gate_us = timer.span_us(2, 3);
        timings->middle_cpu_us = timer.span_us(3, 4);
        timings->down_us = timer.span_us(4, 5);
        timings->combine_us = timer.span_us(5, 6);
        timings->sync_us = elapsed_us(t1);
        timings->gemm_tasks = 2;
        timings->gather_tasks = 1;
        timings->middle_tasks = 1;
        timings->total_us = elapsed_us(t0);
    }
    return rc;
}

} // namespace

extern "C" {

void rk_npu_moe_w8_config_init(rk_npu_moe_w8_config* c, int hidden, int intermediate,
                               int routed_experts, int shared_expert, int top_k, int max_rows) {
    if (!c) return;
    std::memset(c, 0, sizeof(*c));
    c->struct_size = sizeof(*c);
    c->weights.hidden = hidden;
    c->weights.intermediate = intermediate;
    c->weights.routed_experts = routed_experts;
    c->weights.shared_expert = shared_expert;
    c->max_rows = max_rows;
    c->top_k = top_k;
    c->npu_cores = 3;
    c->cpu_threads = 4;
    c->native_input = 0;
    c->middle = RK_NPU_MOE_MIDDLE_CPU;
    c->timeout_ms = 1000;
}

} // extern "C"

namespace {

// Packs one expert into slot e of the bank (the context's submit mutex is held): slots below
// count4 take int4 images (the codes were range-checked on the host), the others int8 images.
int pack_expert(rk_npu_moe_w8_weights* w, DeviceBuffer& raw, int e, const rk_npu_moe_w8_expert& x) {
    const int H = w->config.hidden, I = w->config.intermediate;
    void* stream = w->owner.ctx->stream;
    const bool int4 = e < w->count4;
    const int e8 = e - w->count4;
    int rc = rkh_h2d(stream, raw.as<>(), x.gate_up, (size_t)H * 2 * I);
    if (!rc)
        rc = int4 ? rkh_pack_w4(stream, raw.as<int8_t>(), H, 2 * I, I, w->gate_up4.as<>() + w->gate_stride4 * e, nullptr, nullptr)
                  : rkh_pack_w8(stream, raw.as<int8_t>(), H, 2 * I, I, w->gate_up.as<>() + w->gate_stride * e8);
    if (!rc) rc = rkh_h2d(stream, raw.as<>(), x.down, (size_t)I * H);
    if (!rc)
        rc = int4 ? rkh_pack_w4(stream, raw.as<int8_t>(), I, H, 0, w->down4.as<>() + w->down_stride4 * e, nullptr, nullptr)
                  : rkh_pack_w8(stream, raw.as<int8_t>(), I, H, 0, w->down.as<>() + w->down_stride * e8);
    if (!rc) rc = rkh_h2d(stream, w->gate_scales.as<float>() + (size_t)e * 2 * I, x.gate_up_scales, (size_t)2 * I * sizeof(float));
    if (!rc) rc = rkh_h2d(stream, w->down_scales.as<float>() + (size_t)e * H, x.down_scales, (size_t)H * sizeof(float));
    // the staging buffer is reused: finish this expert before the next copy lands
    if (!rc) rc = rkh_sync(stream);
    return rc;
}

bool expert_ok(const rk_npu_moe_w8_expert& x, int H, int I, bool w4) {
    if (!x.gate_up || !x.down || !finite_positive(x.gate_up_scales, (size_t)2 * I) ||
        !finite_positive(x.down_scales, (size_t)H))
        return false;
    return !w4 || (int4_codes(x.gate_up, (size_t)H * 2 * I) && int4_codes(x.down, (size_t)I * H));
}

// experts: all routed + shared experts, or NULL for a bank of empty slots (then
// `shared`, if given, fills the shared expert's slot).  Empty slots hold zero
// weights and zero scales until a record is imported.
rk_npu_moe_w8_weights* create_weights(rk_npu_iommu_domain* domain, const rk_npu_moe_w8_weight_config* config,
                                      const rk_npu_moe_w8_expert* experts, int mode,
                                      const rk_npu_moe_w8_expert* shared) {
    if (!domain || !domain->ctx || !config || !(mode == kW8 ? valid(*config) : valid_w4(*config))) return nullptr;
    const int H = config->hidden, I = config->intermediate;
    const int count = config->routed_experts + config->shared_expert;
    if (experts)
        for (int e = 0; e < count; ++e)
            if (!expert_ok(experts[e], H, I, expert_is_w4(mode, e, config->routed_experts))) return nullptr;
    if (shared && !expert_ok(*shared, H, I, expert_is_w4(mode, config->routed_experts, config->routed_experts)))
        return nullptr;
    std::unique_ptr<rk_npu_moe_w8_weights> w(new (std::nothrow) rk_npu_moe_w8_weights());
    if (!w) return nullptr;
    w->owner.bind(domain);
    w->config = *config;
    w->mode = mode;
    w->count = count;
    w->count4 = mode == kW4 ? count : mode == kRoutedW4SharedW8 ? config->routed_experts : 0;
    w->gate_stride = rkh_tiled_i8_bytes(2 * I, H, RKH_COL_ALIGN);
    w->down_stride = rkh_tiled_i8_bytes(H, I, RKH_COL_ALIGN);
    w->gate_stride4 = rkh_tiled_i4_bytes(2 * I, H, RKH_COL_ALIGN);
    w->down_stride4 = rkh_tiled_i4_bytes(H, I, RKH_COL_ALIGN);
    rk_npu_ctx* ctx = domain->ctx;
    std::lock_guard<std::mutex> lock(ctx->submit_mutex);
    DeviceBuffer raw;
    const bool zero = experts == nullptr;
    const int count8 = count - w->count4;
    if ((count8 && (w->gate_up.alloc(w->owner, w->gate_stride * count8, zero) ||
                    w->down.alloc(w->owner, w->down_stride * count8, zero))) ||
        (w->count4 && (w->gate_up4.alloc(w->owner, w->gate_stride4 * w->count4, zero) ||
                       w->down4.alloc(w->owner, w->down_stride4 * w->count4, zero))) ||
        w->gate_scales.alloc(w->owner, (size_t)count * 2 * I * sizeof(float), zero) ||
        w->down_scales.alloc(w->owner, (size_t)count * H * sizeof(float), zero) ||
        raw.alloc(w->owner, (size_t)H * 2 * I, false))
        return nullptr;
    if (experts)
        for (int e = 0; e < count; ++e)
            if (pack_expert(w.get(), raw, e, experts[e])) return nullptr;
    if (shared && pack_expert(w.get(), raw, config->routed_experts, *shared)) return nullptr;
    if (rkh_sync(ctx->stream)) return nullptr;
    return w.release();
}

} // namespace

extern "C" {

rk_npu_moe_w8_weights* rk_npu_moe_w8_weights_create(rk_npu_iommu_domain* domain,
                                                    const rk_npu_moe_w8_weight_config* config,
                                                    const rk_npu_moe_w8_expert* experts) {
    return experts ? create_weights(domain, config, experts, kW8, nullptr) : nullptr;
}

void rk_npu_moe_w8_weights_free(rk_npu_moe_w8_weights* weights) { delete weights; }

} // extern "C"

namespace {
rk_npu_moe_w8_workspace* create_workspace(rk_npu_iommu_domain* domain, const rk_npu_moe_w8_config* config, int mode);
}

extern "C" {

rk_npu_moe_w8_workspace* rk_npu_moe_w8_workspace_create(rk_npu_iommu_domain* domain,
                                                        const rk_npu_moe_w8_config* config) {
    return create_workspace(domain, config, kW8);
}

} // extern "C"

namespace {

// reference src/rk_npu_moe_w8.cpp:892-896,910-914: the INT4 modes take fp32 or
// pre-quantized rows in the normal (not NPU-native) layout only
rk_npu_moe_w8_workspace* create_workspace(rk_npu_iommu_domain* domain, const rk_npu_moe_w8_config* config, int mode) {
    if (!domain || !domain->ctx || !config || !valid(*config)) return nullptr;
    if (mode != kW8 && (!valid_w4(config->weights) || config->native_input)) return nullptr;
    std::unique_ptr<rk_npu_moe_w8_workspace> ws(new (std::nothrow) rk_npu_moe_w8_workspace());
    if (!ws) return nullptr;
    ws->owner.bind(domain);
    ws->config = *config;
    ws->mode = mode;
    const auto& wc = config->weights;
    const int R = config->max_rows, H = wc.hidden, I = wc.intermediate, top = config->top_k;
    ws->slots = top + wc.shared_expert;
    const int routed = R * top;
    ws->max_blocks = routed / 32 + std::min(wc.routed_experts, routed) + (wc.shared_expert ? (R + 31) / 32 : 0);
    ws->sorted_rows = ws->max_blocks * 32;
    const size_t S = (size_t)ws->sorted_rows;
    std::lock_guard<std::mutex> lock(domain->ctx->submit_mutex);
    if (ws->input.alloc(ws->owner, (size_t)R * H * 4, false) ||
        ws->token_scale.alloc(ws->owner, (size_t)R * 4) || ws->ids.alloc(ws->owner, (size_t)routed * 4) ||
        ws->routes.alloc(ws->owner, (size_t)routed * 4) ||
        ws->dest_rows.alloc(ws->owner, (size_t)R * ws->slots * 4) ||
        ws->blk_expert.alloc(ws->owner, (size_t)ws->max_blocks * 4) ||
        ws->num_blocks.alloc(ws->owner, 16) ||
        ws->a_tiled.alloc(ws->owner, rkh_tiled_i8_bytes(ws->sorted_rows, H, 32)) ||
        ws->a_scale.alloc(ws->owner, S * 4) || ws->hidden.alloc(ws->owner, S * I * 4) ||
        ws->row_max.alloc(ws->owner, S * (size_t)(I / 32) * 4) ||
        ws->h_tiled.alloc(ws->owner, rkh_tiled_i8_bytes(ws->sorted_rows, I, 32)) ||
        ws->h_scale.alloc(ws->owner, S * 4) || ws->y.alloc(ws->owner, S * H * 4) ||
        ws->out.alloc(ws->owner, (size_t)R * H * 4, false) || ws->flag.init(ws->owner))
        return nullptr;
    ws->stage_in.init((size_t)R * H * 4);
    ws->stage_out.init((size_t)R * H * 4);
    ws->stage_route.init((size_t)routed * 8 + (size_t)R * 4);
    if (rkh_sync(domain->ctx->stream)) return nullptr;
    return ws.release();
}

} // namespace

extern "C" {

void rk_npu_moe_w8_workspace_free(rk_npu_moe_w8_workspace* workspace) { delete workspace; }

// ---- INT4 experts, mixed banks, slot banks and packed expert records ----------
// reference src/rk_npu_moe_w8.cpp:885-926
rk_npu_moe_w8_weights* rk_npu_moe_quant_weights_create(rk_npu_iommu_domain* domain,
                                                       const rk_npu_moe_w8_weight_config* config,
                                                       const rk_npu_moe_w8_expert* experts) {
    return experts ? create_weights(domain, config, experts, kW4, nullptr) : nullptr;
}
// The reference certifies a full-K gate/up tile here; accumulation is int32 in
// this build, so both factories produce the same weights.
rk_npu_moe_w8_weights* rk_npu_moe_quant_weights_create_full_k(rk_npu_iommu_domain* domain,
                                                              const rk_npu_moe_w8_weight_config* config,
                                                              const rk_npu_moe_w8_expert* experts) {
    return rk_npu_moe_quant_weights_create(domain, config, experts);
}
rk_npu_moe_w8_workspace* rk_npu_moe_quant_workspace_create(rk_npu_iommu_domain* domain,
                                                           const rk_npu_moe_w8_config* config) {
    return create_workspace(domain, config, kW4);
}
rk_npu_moe_w8_weights* rk_npu_moe_w4_weights_create(rk_npu_iommu_domain* domain,
                                                    const rk_npu_moe_w8_weight_config* config,
                                                    const rk_npu_moe_w8_expert* experts) {
    return experts ? create_weights(domain, config, experts, kRoutedW4SharedW8, nullptr) : nullptr;
}
rk_npu_moe_w8_workspace* rk_npu_moe_w4_workspace_create(rk_npu_iommu_domain* domain,
                                                        const rk_npu_moe_w8_config* config) {
    return create_workspace(domain, config, kRoutedW4SharedW8);
}
rk_npu_moe_w8_weights* rk_npu_moe_w4_slots_create(rk_npu_iommu_domain* domain,
                                                  const rk_npu_moe_w8_weight_config* config,
                                                  const rk_npu_moe_w8_expert* shared) {
    if (!config || !shared || config->shared_expert != 1) return nullptr;
    return create_weights(domain, config, nullptr, kRoutedW4SharedW8, shared);
}
rk_npu_moe_w8_weights* rk_npu_moe_quant_slots_create(rk_npu_iommu_domain* domain,
                                                     const rk_npu_moe_w8_weight_config* config) {
    if (!config || config->shared_expert) return nullptr;
    return create_weights(domain, config, nullptr, kW4, nullptr);
}

} // extern "C"

namespace {

// A packed INT4 expert record: header, then the expert's device images exactly as
// the kernels read them (gate/up and down int4 tiles, two codes per byte; gate/up
// and down scales).  Records are produced by rk_npu_moe_quant_export_expert of
// this library and are not interchangeable with the reference's (its records
// hold NPU tile images).  Every byte of an image is two valid codes, so a record
// cannot smuggle a value outside [-8, 7] into a slot.
// `layout` is this library's own revision of the image layout, beside the API's blob version:
// it changes whenever the bytes of an image mean something else (revision 1 held the codes as
// int8 tiles padded to 64 k, under the magic "RKHM" and a 16-byte header; revision 2 holds
// packed nibbles padded to 256 k).  Every byte of an image is valid codes in any layout, so
// nothing but the header can tell a record of another revision apart: import checks the magic,
// both versions and the two image sizes before it touches a slot.
struct RecordHeader {
    uint32_t magic, version, hidden, intermediate;
    uint32_t layout, reserved;
    uint64_t gate_bytes, down_bytes;
};
constexpr uint32_t kRecordMagic = 0x34484b52u; // "RKH4"
constexpr uint32_t kRecordLayout = 2;

uint64_t record_bytes(const rk_npu_moe_w8_weights* w) {
    return sizeof(RecordHeader) + w->gate_stride4 + w->down_stride4 +
           ((uint64_t)2 * w->config.intermediate + w->config.hidden) * sizeof(float);
}

} // namespace

extern "C" {

// reference :927-929: 0 for handles without INT4 experts
uint64_t rk_npu_moe_quant_expert_blob_bytes(const rk_npu_moe_w8_weights* w) {
    return w && w->mode != kW8 ? record_bytes(w) : 0;
}

// reference :931-947
int rk_npu_moe_quant_export_expert(const rk_npu_moe_w8_weights* w, int e, void* data, uint64_t bytes) {
    const uint64_t need = rk_npu_moe_quant_expert_blob_bytes(w);
    if (!need || !data || bytes < need || e < 0 || e >= w->count ||
        !expert_is_w4(w->mode, e, w->config.routed_experts))
        return RK_NPU_ERR_PARAM;
    const int H = w->config.hidden, I = w->config.intermediate;
    rk_npu_ctx* ctx = w->owner.ctx;
    uint8_t* p = static_cast<uint8_t*>(data);
    const RecordHeader header{kRecordMagic, RK_NPU_MOE_QUANT_BLOB_VERSION, (uint32_t)H, (uint32_t)I,
                              kRecordLayout, 0u, (uint64_t)w->gate_stride4, (uint64_t)w->down_stride4};
    std::memcpy(p, &header, sizeof(header));
    p += sizeof(header);
    std::lock_guard<std::mutex> lock(ctx->submit_mutex);
    int rc = rkh_d2h(ctx->stream, p, w->gate_up4.as<>() + w->gate_stride4 * e, w->gate_stride4);
    p += w->gate_stride4;
    if (!rc) rc = rkh_d2h(ctx->stream, p, w->down4.as<>() + w->down_stride4 * e, w->down_stride4);
    p += w->down_stride4;
    if (!rc) rc = rkh_d2h(ctx->stream, p, w->gate_scales.as<float>() + (size_t)e * 2 * I, (size_t)2 * I * sizeof(float));
    p += (size_t)2 * I * sizeof(float);
    if (!rc) rc = rkh_d2h(ctx->stream, p, w->down_scales.as<float>() + (size_t)e * H, (size_t)H * sizeof(float));
    const int wait = rkh_sync(ctx->stream);
    return map_error(rc ? rc : wait);
}

int rk_npu_moe_quant_import_expert(rk_npu_moe_w8_weights* w, int slot, const void* data, uint64_t bytes) {
    return rk_npu_moe_quant_import_expert_timed(w, slot, data, bytes, nullptr);
}

// reference :952-985.  The record is checked (header, scales) before anything is
// written, so a rejected record leaves the slot as it was.
int rk_npu_moe_quant_import_expert_timed(rk_npu_moe_w8_weights* w, int slot, const void* data, uint64_t bytes,
                                         rk_npu_moe_import_timings* timings) {
    const uint64_t need = rk_npu_moe_quant_expert_blob_bytes(w);
    if (!need || !data || bytes < need || slot < 0 || slot >= w->count ||
        !expert_is_w4(w->mode, slot, w->config.routed_experts))
        return RK_NPU_ERR_PARAM;
    if (timings) *timings = rk_npu_moe_import_timings{};
    const auto begin = Clock::now();
    const int H = w->config.hidden, I = w->config.intermediate;
    const uint8_t* p = static_cast<const uint8_t*>(data);
    RecordHeader header;
    std::memcpy(&header, p, sizeof(header));
    const uint8_t* gate = p + sizeof(header);
    const uint8_t* down = gate + w->gate_stride4;
    const uint8_t* gate_scales = down + w->down_stride4;
    const uint8_t* down_scales = gate_scales + (size_t)2 * I * sizeof(float);
    auto at = Clock::now();
    bool ok = header.magic == kRecordMagic && header.version == RK_NPU_MOE_QUANT_BLOB_VERSION &&
              header.hidden == (uint32_t)H && header.intermediate == (uint32_t)I &&
              header.layout == kRecordLayout && header.gate_bytes == (uint64_t)w->gate_stride4 &&
              header.down_bytes == (uint64_t)w->down_stride4;
    if (ok) {
        std::vector<float> scales((size_t)2 * I + H); // the record need not be aligned for float access
        std::memcpy(scales.data(), gate_scales, scales.size() * sizeof(float));
        ok = finite_positive(scales.data(), scales.size());
    }
    if (timings) timings->validate_us = elapsed_us(at);
    if (!ok) return RK_NPU_ERR_PARAM;
    rk_npu_ctx* ctx = w->owner.ctx;
    std::lock_guard<std::mutex> lock(ctx->submit_mutex);
    at = Clock::now();
    int rc = rkh_h2d(ctx->stream, w->gate_scales.as<float>() + (size_t)slot * 2 * I, gate_scales, (size_t)2 * I * sizeof(float));
    if (!rc) rc = rkh_h2d(ctx->stream, w->down_scales.as<float>() + (size_t)slot * H, down_scales, (size_t)H * sizeof(float));
    if (!rc) rc = rkh_sync(ctx->stream);
    if (timings) timings->copy_us = elapsed_us(at);
    at = Clock::now();
    if (!rc) rc = rkh_h2d(ctx->stream, w->gate_up4.as<>() + w->gate_stride4 * slot, gate, w->gate_stride4);
    if (!rc) rc = rkh_sync(ctx->stream);
    if (timings) timings->gate_sync_us = elapsed_us(at);
    at = Clock::now();
    if (!rc) rc = rkh_h2d(ctx->stream, w->down4.as<>() + w->down_stride4 * slot, down, w->down_stride4);
    if (!rc) rc = rkh_sync(ctx->stream);
    if (timings) {
        timings->down_sync_us = elapsed_us(at);
        timings->total_us = elapsed_us(begin);
    }
    return map_error(rc);
}

// reference :987-998.  The reference exchanges buffer ownership; a bank here is
// one allocation that the kernels index by slot, so the two slots' images are
// exchanged in place by a kernel enqueued on the context's stream.  Nothing
// waits on the host: runs, imports and exports of the same context are ordered
// behind it on that stream.
int rk_npu_moe_quant_swap_slots(rk_npu_moe_w8_weights* a, int ai, rk_npu_moe_w8_weights* b, int bi) {
    if (!a || !b || a->mode != kW4 || b->mode != kW4 || a->config.hidden != b->config.hidden ||
        a->config.intermediate != b->config.intermediate || !a->owner.same(b->owner) || ai < 0 || bi < 0 ||
        ai >= a->count || bi >= b->count)
        return RK_NPU_ERR_PARAM;
    if (a == b && ai == bi) return RK_NPU_OK;
    const size_t H = a->config.hidden, I = a->config.intermediate;
    rk_npu_ctx* ctx = a->owner.ctx;
    std::lock_guard<std::mutex> lock(ctx->submit_mutex);
    int rc = rkh_exchange32(ctx->stream, a->gate_up4.as<>() + a->gate_stride4 * ai, b->gate_up4.as<>() + b->gate_stride4 * bi,
                            a->gate_stride4 / 4);
    if (!rc) rc = rkh_exchange32(ctx->stream, a->down4.as<>() + a->down_stride4 * ai, b->down4.as<>() + b->down_stride4 * bi,
                                 a->down_stride4 / 4);
    if (!rc) rc = rkh_exchange32(ctx->stream, a->gate_scales.as<float>() + ai * 2 * I, b->gate_scales.as<float>() + bi * 2 * I, 2 * I);
    if (!rc) rc = rkh_exchange32(ctx->stream, a->down_scales.as<float>() + ai * H, b->down_scales.as<float>() + bi * H, H);
    return map_error(rc);
}

uint64_t rk_npu_moe_w8_weights_device_bytes(const rk_npu_moe_w8_weights* w) {
    return w ? w->bytes() : 0;
}
uint64_t rk_npu_moe_w8_workspace_device_bytes(const rk_npu_moe_w8_workspace* w) {
    return w ? w->bytes() : 0;
}

int rk_npu_moe_w8_run_quantized(rk_npu_moe_w8_workspace* ws, const rk_npu_moe_w8_weights* w,
                                int rows, const int8_t* input, const float* row_scales,
                                const int32_t* ids, const float* routes, float* out,
                                rk_npu_moe_w8_timings* t) {
    return moe_run(ws, w, rows, input, false, row_scales, ids, routes, out, t);
}
int rk_npu_moe_w8_run_f32(rk_npu_moe_w8_workspace* ws, const rk_npu_moe_w8_weights* w, int rows,
                          const float* input, const int32_t* ids, const float* routes, float* out,
                          rk_npu_moe_w8_timings* t) {
    return moe_run(ws, w, rows, input, true, nullptr, ids, routes, out, t);
}

// Device-resident variant: ids, coefficients and tokens cannot be inspected without a copy back,
// so the kernels look at them: an id out of range, a negative or non-finite coefficient and a
// non-finite token raise the context's flag, which the next rk_npu_hip_sync returns as ERR_PARAM.
// Up to twelve tokens take the two-launch path (see enqueue), more the routed, grouped one.
int rk_npu_moe_w8_run_f32_device(rk_npu_moe_w8_workspace* ws, const rk_npu_moe_w8_weights* w,
                                 int rows, const float* input, const int32_t* ids,
                                 const float* routes, float* out) {
    if (!ws || !w || !input || !ids || !routes || !out || rows < 1 || rows > ws->config.max_rows)
        return RK_NPU_ERR_PARAM;
    BusyLock lock(ws->busy);
    if (!lock) return RK_NPU_ERR_BUSY;
    int rc = check_handles(ws, w);
    if (rc) return rc;
    std::lock_guard<std::mutex> submit(ws->owner.ctx->submit_mutex);
    note_pending_flag(ws->owner.ctx, ws->flag.device());
    return enqueue(ws, w, rows, input, true, nullptr, ids, routes, out, nullptr, true);
}

} // extern "C"
