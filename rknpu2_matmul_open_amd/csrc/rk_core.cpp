// Context, domain tags, error strings, device buffers and the generic part of
// the MI355X extension API.  Replaces the device core of the reference
// (src/rk_npu_core.cpp:98-183: open / close / strerror / domain handles); the
// GEM / dmabuf half of that file has no equivalent because HBM allocations are
// private to this library.
#include <algorithm>
#include <cerrno>
#include <cstdlib>
#include <new>

#include <cstring>

#include "rk_host.h"
#include "rk_npu_hip.h"

// A recorded sequence of launches, and the rejected-input flags of the workspaces it uses.
struct rk_npu_hip_graph {
    void* exec = nullptr;
    rk_npu_ctx* ctx = nullptr;
    std::vector<int*> flags;
};

namespace {
std::atomic<uint64_t> g_next_ctx_id{1};
}

namespace rkhost {

int DeviceBuffer::alloc(const Owner& owner, size_t bytes, bool zero) {
    release();
    if (!owner.ctx) return RK_NPU_ERR_PARAM;
    void* p = nullptr;
    // round to whole 32-bit words so the fill kernel can clear it
    const size_t rounded = (bytes + 15) / 16 * 16;
    auto& domain = owner.ctx->memory[owner.domain_id];
    const uint64_t epoch = domain.reclaim_epoch.load(std::memory_order_relaxed);
    int rc = rkh_malloc(owner.ctx->device, &p, rounded);
    if (rc == RKH_ERR_NOMEM) {
        // Memory pressure: give the domain's reclaim hook one chance to free idle allocations
        // (reference src/rk_npu_core.cpp:195-240), then try once more.  The hook may free
        // handles of this library (their release takes no lock held here) but must not allocate.
        bool reclaimed = false;
        {
            std::lock_guard<std::mutex> lock(domain.reclaim_mutex);
            if (domain.reclaim_epoch.load(std::memory_order_relaxed) != epoch) {
                reclaimed = true; // another thread's failed allocation already ran the hook
            } else if (domain.reclaim) {
                domain.reclaim(domain.reclaim_cookie);
                domain.reclaim_epoch.fetch_add(1, std::memory_order_relaxed);
                reclaimed = true;
            }
        }
        if (reclaimed) rc = rkh_malloc(owner.ctx->device, &p, rounded);
    }
    if (rc) return map_error(rc);
    if (zero) {
        rc = rkh_fill32(owner.ctx->stream, p, 0u, rounded / 4);
        if (rc) {
            rkh_free(owner.ctx->device, p);
            return map_error(rc);
        }
    }
    ptr_ = p;
    bytes_ = rounded;
    owner_ = owner;
    auto& mem = owner.ctx->memory[owner.domain_id];
    const uint64_t live = mem.live_bytes.fetch_add(rounded) + rounded;
    uint64_t peak = mem.peak_bytes.load();
    while (live > peak && !mem.peak_bytes.compare_exchange_weak(peak, live)) {
    }
    mem.creates.fetch_add(1);
    return RK_NPU_OK;
}

void DeviceBuffer::release() {
    if (!ptr_) return;
    // Work that may still read the buffer is on the context's stream.
    rkh_sync(owner_.ctx->stream);
    rkh_free(owner_.ctx->device, ptr_);
    auto& mem = owner_.ctx->memory[owner_.domain_id];
    mem.live_bytes.fetch_sub(bytes_);
    mem.destroys.fetch_add(1);
    ptr_ = nullptr;
    bytes_ = 0;
}

StageTimer::StageTimer(void* stream, bool enabled) : stream_(stream), enabled_(enabled) {}
StageTimer::~StageTimer() {
    for (int i = 0; i < count_; ++i) rkh_event_destroy(events_[i]);
}
void StageTimer::mark() {
    if (!enabled_ || count_ >= 12) return;
    void* e = nullptr;
    if (rkh_event_create(&e)) return;
    rkh_event_record(e, stream_);
    events_[count_++] = e;
}
double StageTimer::span_us(int from, int to) {
    if (!enabled_ || from < 0 || to >= count_ || from >= to) return 0.0;
    double us = 0.0;
    if (rkh_event_elapsed_us(events_[from], events_[to], &us)) return 0.0;
    return us;
}

HostStage::~HostStage() {
    for (void* e : events_) rkh_event_destroy(e);
    rkh_host_free(ptr_);
}
void HostStage::init(size_t bytes) {
    if (!bytes || bytes > kPipeLimit) return;
    void* p = nullptr;
    if (rkh_host_alloc(&p, bytes) != RKH_OK) return;
    ptr_ = p;
    bytes_ = bytes;
    if (bytes > kLimit) { // (a mirror that may serve staged downloads)
        const size_t chunks = (bytes + kChunk - 1) / kChunk;
        for (size_t i = 0; i < chunks; ++i) {
            void* e = nullptr;
            if (rkh_event_create(&e) != RKH_OK) { // without its events the mirror only serves uploads
                for (void* made : events_) rkh_event_destroy(made);
                events_.clear();
                break;
            }
            events_.push_back(e);
        }
    }
}
const void* HostStage::fill(const void* user, size_t bytes) const {
    std::memcpy(ptr_, user, bytes <= bytes_ ? bytes : bytes_);
    return ptr_;
}
void HostStage::finish(void* user, size_t bytes) const {
    if (ptr_ && bytes <= bytes_) std::memcpy(user, ptr_, bytes);
}
int HostStage::upload(void* stream, void* device, const void* user, size_t bytes) const {
    if (!ptr_ || bytes > bytes_) return rkh_h2d(stream, device, user, bytes);
    for (size_t off = 0; off < bytes; off += kChunk) {
        const size_t n = bytes - off < kChunk ? bytes - off : kChunk;
        std::memcpy(static_cast<uint8_t*>(ptr_) + off, static_cast<const uint8_t*>(user) + off, n);
        const int rc = rkh_h2d(stream, static_cast<uint8_t*>(device) + off, static_cast<uint8_t*>(ptr_) + off, n);
        if (rc) return rc;
    }
    return RKH_OK;
}
int HostStage::download(void* stream, void* user, const void* device, size_t bytes) {
    staged_ = ptr_ && bytes <= bytes_ && events_.size() * kChunk >= bytes;
    if (!staged_) return rkh_d2h(stream, user, device, bytes);
    size_t i = 0;
    for (size_t off = 0; off < bytes; off += kChunk, ++i) {
        const size_t n = bytes - off < kChunk ? bytes - off : kChunk;
        int rc = rkh_d2h(stream, static_cast<uint8_t*>(ptr_) + off, static_cast<const uint8_t*>(device) + off, n);
        if (!rc) rc = rkh_event_record(events_[i], stream);
        if (rc) return rc;
    }
    return RKH_OK;
}
int HostStage::finish_download(void* stream, void* user, size_t bytes) {
    if (!staged_) return rkh_sync(stream);
    size_t i = 0;
    for (size_t off = 0; off < bytes; off += kChunk, ++i) {
        const size_t n = bytes - off < kChunk ? bytes - off : kChunk;
        const int rc = rkh_event_sync(events_[i]);
        if (rc) return rc;
        std::memcpy(static_cast<uint8_t*>(user) + off, static_cast<uint8_t*>(ptr_) + off, n);
    }
    return RKH_OK;
}

BadFlag::~BadFlag() { rkh_host_free(host_); }
int BadFlag::init(const Owner& owner) {
    int rc = dev_.alloc(owner, sizeof(int), true);
    if (rc) return rc;
    void* h = nullptr;
    rc = rkh_host_alloc(&h, sizeof(int));
    if (rc) return map_error(rc);
    host_ = static_cast<int*>(h);
    *host_ = 0;
    return RK_NPU_OK;
}
int BadFlag::enqueue_readback(void* stream) {
    return map_error(rkh_d2h(stream, host_, dev_.as<>(), sizeof(int)));
}
bool BadFlag::consume(void* stream) {
    if (!*host_) return false;
    *host_ = 0;
    rkh_fill32(stream, dev_.as<>(), 0u, 1);
    return true;
}
bool consume_device_flag(rk_npu_ctx* ctx, int* flag) {
    int v = 0;
    if (rkh_d2h(ctx->stream, &v, flag, sizeof(int)) || rkh_sync(ctx->stream)) return false;
    if (!v) return false;
    rkh_fill32(ctx->stream, flag, 0u, 1);
    return true;
}
void note_pending_flag(rk_npu_ctx* ctx, int* flag) {
    std::lock_guard<std::mutex> lock(ctx->pending_mutex);
    if (ctx->capturing && std::find(ctx->capture_flags.begin(), ctx->capture_flags.end(), flag) == ctx->capture_flags.end())
        ctx->capture_flags.push_back(flag);
    for (int* f : ctx->pending_flags)
        if (f == flag) return;
    ctx->pending_flags.push_back(flag);
}
void forget_pending_flag(rk_npu_ctx* ctx, int* flag) {
    std::lock_guard<std::mutex> lock(ctx->pending_mutex);
    auto drop = [flag](std::vector<int*>& v) { v.erase(std::remove(v.begin(), v.end(), flag), v.end()); };
    drop(ctx->pending_flags);
    drop(ctx->capture_flags);
    for (rk_npu_hip_graph* g : ctx->graphs) drop(g->flags);
}

int upload(const Owner& owner, DeviceBuffer& dst, const void* src, size_t bytes) {
    int rc = dst.alloc(owner, bytes, false);
    if (rc) return rc;
    rc = rkh_h2d(owner.ctx->stream, dst.as<>(), src, bytes);
    return map_error(rc);
}

} // namespace rkhost

static void abandon_profile(rk_npu_ctx* ctx); // (defined beside the profile entry points)

extern "C" {

rk_npu_ctx* rk_npu_open(const char* dev) {
    int device = 0;
    if (dev) {
        if (std::strncmp(dev, "hip:", 4) != 0 || !dev[4]) {
            errno = ENODEV;
            return nullptr;
        }
        char* end = nullptr;
        const long v = std::strtol(dev + 4, &end, 10);
        if (*end || v < 0 || v > 1023) {
            errno = ENODEV;
            return nullptr;
        }
        device = (int)v;
    }
    if (device >= rkh_device_count()) {
        errno = ENODEV;
        return nullptr;
    }
    rk_npu_ctx* ctx = new (std::nothrow) rk_npu_ctx();
    if (!ctx) {
        errno = ENOMEM;
        return nullptr;
    }
    ctx->device = device;
    if (rkh_open(device, &ctx->stream, ctx->arch, (int)sizeof(ctx->arch), &ctx->cu_count,
                 &ctx->clock_khz)) {
        delete ctx;
        errno = ENODEV;
        return nullptr;
    }
    ctx->id = g_next_ctx_id.fetch_add(1);
    // (rkh_open made `device` current; a failed lookup only disables the no-allocation entry point)
    if (rkh_static_scratch(device, &ctx->scratch, &ctx->scratch_bytes)) {
        ctx->scratch = nullptr;
        ctx->scratch_bytes = 0;
    }
    return ctx;
}

void rk_npu_close(rk_npu_ctx* ctx) {
    if (!ctx) return;
    abandon_profile(ctx); // (a context closed between profile_begin and profile_end)
    rkh_close(ctx->device, ctx->stream);
    {
        // graphs that outlive their context only keep their executable; graph_free releases it
        std::lock_guard<std::mutex> lock(ctx->pending_mutex);
        for (rk_npu_hip_graph* g : ctx->graphs) {
            g->ctx = nullptr;
            g->flags.clear();
        }
    }
    delete ctx;
}

const char* rk_npu_strerror(int code) {
    switch (code) {
    case RK_NPU_OK: return "ok";
    case RK_NPU_ERR_OPEN: return "could not open device";
    case RK_NPU_ERR_IOCTL: return "device runtime call failed";
    case RK_NPU_ERR_PARAM: return "bad argument";
    case RK_NPU_ERR_NOMEM: return "allocation failed or buffer too small";
    case RK_NPU_ERR_SUBMIT: return "device job failed/timed out";
    case RK_NPU_ERR_BUSY: return "workspace is already running";
    case RK_NPU_ERR_DOMAIN: return "domain mismatch or unavailable";
    case RK_NPU_ERR_IO: return "file I/O failed";
    case RK_NPU_ERR_CACHE_MISS: return "tuning cache miss";
    default: return "unknown error";
    }
}

rk_npu_iommu_domain* rk_npu_iommu_domain_create(rk_npu_ctx* ctx, uint32_t domain_id) {
    if (!ctx || domain_id >= RK_NPU_IOMMU_DOMAIN_COUNT) return nullptr;
    rk_npu_iommu_domain* d = new (std::nothrow) rk_npu_iommu_domain();
    if (!d) return nullptr;
    d->ctx = ctx;
    d->id = domain_id;
    return d;
}

void rk_npu_iommu_domain_free(rk_npu_iommu_domain* domain) { delete domain; }

uint32_t rk_npu_iommu_domain_id(const rk_npu_iommu_domain* domain) {
    return domain ? domain->id : UINT32_MAX;
}

void rk_npu_iommu_domain_set_reclaim(rk_npu_iommu_domain* domain, rk_npu_reclaim_idle_fn reclaim, void* cookie) {
    if (!domain || !domain->ctx) return;
    auto& m = domain->ctx->memory[domain->id];
    std::lock_guard<std::mutex> lock(m.reclaim_mutex);
    m.reclaim = reclaim;
    m.reclaim_cookie = reclaim ? cookie : nullptr;
}

int rk_npu_iommu_domain_memory_stats(const rk_npu_iommu_domain* domain,
                                     rk_npu_domain_memory_stats* stats) {
    if (!domain || !domain->ctx || !stats) return RK_NPU_ERR_PARAM;
    const auto& m = domain->ctx->memory[domain->id];
    stats->live_bytes = m.live_bytes.load();
    stats->peak_bytes = m.peak_bytes.load();
    stats->creates = m.creates.load();
    stats->destroys = m.destroys.load();
    return RK_NPU_OK;
}

/* ---- MI355X extension: generic part ---- */

void* rk_npu_hip_stream(rk_npu_ctx* ctx) { return ctx ? ctx->stream : nullptr; }
int rk_npu_hip_device(const rk_npu_ctx* ctx) { return ctx ? ctx->device : -1; }

int rk_npu_hip_device_info(const rk_npu_ctx* ctx, char* arch, int arch_len, int* cu_count,
                           int* clock_khz) {
    if (!ctx) return RK_NPU_ERR_PARAM;
    if (arch && arch_len > 0) {
        std::strncpy(arch, ctx->arch, (size_t)arch_len - 1);
        arch[arch_len - 1] = 0;
    }
    if (cu_count) *cu_count = ctx->cu_count;
    if (clock_khz) *clock_khz = ctx->clock_khz;
    return RK_NPU_OK;
}

int rk_npu_hip_sync(rk_npu_ctx* ctx) {
    if (!ctx) return RK_NPU_ERR_PARAM;
    if (rkh_sync(ctx->stream)) return RK_NPU_ERR_SUBMIT;
    std::vector<int*> flags;
    {
        std::lock_guard<std::mutex> lock(ctx->pending_mutex);
        flags.swap(ctx->pending_flags);
    }
    bool rejected = false;
    for (int* f : flags) rejected |= rkhost::consume_device_flag(ctx, f);
    return rejected ? RK_NPU_ERR_PARAM : RK_NPU_OK;
}

void* rk_npu_hip_malloc(rk_npu_ctx* ctx, size_t bytes) {
    if (!ctx) return nullptr;
    void* p = nullptr;
    if (rkh_malloc(ctx->device, &p, bytes)) return nullptr;
    return p;
}
void rk_npu_hip_free(rk_npu_ctx* ctx, void* ptr) {
    if (!ctx || !ptr) return;
    rkh_sync(ctx->stream);
    rkh_free(ctx->device, ptr);
}
int rk_npu_hip_upload(rk_npu_ctx* ctx, void* dst_device, const void* src_host, size_t bytes) {
    if (!ctx || !dst_device || !src_host) return RK_NPU_ERR_PARAM;
    int rc = rkh_h2d(ctx->stream, dst_device, src_host, bytes);
    if (!rc) rc = rkh_sync(ctx->stream);
    return rkhost::map_error(rc);
}
int rk_npu_hip_download(rk_npu_ctx* ctx, void* dst_host, const void* src_device, size_t bytes) {
    if (!ctx || !dst_host || !src_device) return RK_NPU_ERR_PARAM;
    int rc = rkh_d2h(ctx->stream, dst_host, src_device, bytes);
    if (!rc) rc = rkh_sync(ctx->stream);
    return rkhost::map_error(rc);
}

int rk_npu_hip_copy(rk_npu_ctx* ctx, void* dst_device, const void* src_device, size_t bytes) {
    if (!ctx || !dst_device || !src_device) return RK_NPU_ERR_PARAM;
    return rkhost::map_error(rkh_d2d(ctx->stream, dst_device, src_device, bytes));
}

struct rk_npu_hip_event {
    void* handle = nullptr;
};
rk_npu_hip_event* rk_npu_hip_event_create(void) {
    auto* e = new (std::nothrow) rk_npu_hip_event();
    if (!e) return nullptr;
    if (rkh_event_create(&e->handle)) {
        delete e;
        return nullptr;
    }
    return e;
}
void rk_npu_hip_event_free(rk_npu_hip_event* event) {
    if (!event) return;
    rkh_event_destroy(event->handle);
    delete event;
}
int rk_npu_hip_event_record(rk_npu_ctx* ctx, rk_npu_hip_event* event) {
    if (!ctx || !event) return RK_NPU_ERR_PARAM;
    return rkhost::map_error(rkh_event_record(event->handle, ctx->stream));
}
int rk_npu_hip_event_elapsed_us(rk_npu_hip_event* start, rk_npu_hip_event* stop, double* us) {
    if (!start || !stop || !us) return RK_NPU_ERR_PARAM;
    return rkhost::map_error(rkh_event_elapsed_us(start->handle, stop->handle, us));
}

void rk_npu_hip_fail_alloc_after(int n) { rkh_fail_malloc_after(n); }

/* ---- measurement probes ---- */
int rk_npu_hip_probe_stream_read(rk_npu_ctx* ctx, const void* src_device, size_t bytes, size_t span) {
    if (!ctx || !src_device || bytes < 16 || span < 1024 || span % 1024) return RK_NPU_ERR_PARAM;
    std::lock_guard<std::mutex> submit(ctx->submit_mutex);
    return rkhost::map_error(rkh_probe_stream_read(ctx->stream, src_device, bytes, span, nullptr));
}
int rk_npu_hip_probe_mfma_i8(rk_npu_ctx* ctx, const void* operands_device, int iterations, double* ops) {
    if (!ctx || !operands_device || iterations < 1) return RK_NPU_ERR_PARAM;
    const int workgroups = ctx->cu_count; // one workgroup of eight waves per compute unit, as the GEMM runs
    if (ops) *ops = (double)workgroups * 8.0 * iterations * 4.0 * 2.0 * 32 * 32 * 32;
    std::lock_guard<std::mutex> submit(ctx->submit_mutex);
    return rkhost::map_error(rkh_probe_mfma_i8(ctx->stream, operands_device, workgroups, iterations, nullptr));
}

/* ---- per-kernel profile ---- */
namespace {
std::mutex g_profile_owner_mutex;
rk_npu_ctx* g_profile_owner = nullptr; // the marker is process-wide: one context profiles at a time

void profile_marker(void* user, void* stream, const char* kernel) {
    rk_npu_ctx* ctx = static_cast<rk_npu_ctx*>(user);
    if (stream != ctx->stream) return;
    std::lock_guard<std::mutex> lock(ctx->profile_mutex);
    if (!ctx->profiling) return;
    void* event = nullptr;
    if (rkh_event_create(&event)) return;
    rkh_event_record(event, stream);
    ctx->profile_marks.push_back({kernel, event});
}
} // namespace

} // extern "C"

// Called by rk_npu_close: a context that is still the profile owner takes the marker down
// (rkh_set_marker returns once no launch is inside the marker any more), gives the ownership
// back and releases the events it recorded, so that nothing points at the context afterwards.
static void abandon_profile(rk_npu_ctx* ctx) {
    {
        std::lock_guard<std::mutex> owner(g_profile_owner_mutex);
        if (g_profile_owner != ctx) return;
        rkh_set_marker(nullptr, nullptr);
        g_profile_owner = nullptr;
    }
    std::lock_guard<std::mutex> lock(ctx->profile_mutex);
    ctx->profiling = false;
    for (auto& m : ctx->profile_marks) rkh_event_destroy(m.event);
    ctx->profile_marks.clear();
}

extern "C" {

int rk_npu_hip_profile_begin(rk_npu_ctx* ctx) {
    if (!ctx) return RK_NPU_ERR_PARAM;
    std::lock_guard<std::mutex> owner(g_profile_owner_mutex);
    if (g_profile_owner) return RK_NPU_ERR_BUSY;
    g_profile_owner = ctx;
    {
        std::lock_guard<std::mutex> lock(ctx->profile_mutex);
        ctx->profiling = true;
    }
    rkh_set_marker(profile_marker, ctx);
    return RK_NPU_OK;
}

int rk_npu_hip_profile_end(rk_npu_ctx* ctx, char* names, size_t names_bytes, double* us, int capacity) {
    if (!ctx || capacity < 0 || (capacity > 0 && !us)) return RK_NPU_ERR_PARAM;
    {
        std::lock_guard<std::mutex> owner(g_profile_owner_mutex);
        if (g_profile_owner != ctx) return RK_NPU_ERR_PARAM;
        rkh_set_marker(nullptr, nullptr);
        g_profile_owner = nullptr;
    }
    std::vector<rk_npu_ctx::ProfileMark> marks;
    {
        std::lock_guard<std::mutex> lock(ctx->profile_mutex);
        ctx->profiling = false;
        marks.swap(ctx->profile_marks);
    }
    void* last = nullptr;
    int rc = rkh_event_create(&last);
    if (!rc) rc = rkh_event_record(last, ctx->stream);
    if (!rc) rc = rkh_sync(ctx->stream);
    int count = 0;
    size_t used = 0;
    if (names && names_bytes) names[0] = 0;
    for (size_t i = 0; i < marks.size() && !rc; ++i) {
        if (count >= capacity) break;
        void* next = i + 1 < marks.size() ? marks[i + 1].event : last;
        double span = 0.0;
        rc = rkh_event_elapsed_us(marks[i].event, next, &span);
        us[count++] = span;
        if (names) { // newline-separated kernel names, as many as fit
            const size_t len = std::strlen(marks[i].kernel);
            if (used + len + 2 <= names_bytes) {
                std::memcpy(names + used, marks[i].kernel, len);
                names[used + len] = '\n';
                used += len + 1;
                names[used] = 0;
            }
        }
    }
    for (auto& m : marks) rkh_event_destroy(m.event);
    rkh_event_destroy(last);
    return rc ? RK_NPU_ERR_SUBMIT : count;
}

/* ---- stream capture ---- */
int rk_npu_hip_capture_begin(rk_npu_ctx* ctx) {
    if (!ctx) return RK_NPU_ERR_PARAM;
    std::lock_guard<std::mutex> submit(ctx->submit_mutex);
    const int rc = rkhost::map_error(rkh_capture_begin(ctx->stream));
    if (!rc) {
        std::lock_guard<std::mutex> lock(ctx->pending_mutex);
        ctx->capturing = true;
        ctx->capture_flags.clear();
    }
    return rc;
}
rk_npu_hip_graph* rk_npu_hip_capture_end(rk_npu_ctx* ctx) {
    if (!ctx) return nullptr;
    auto* g = new (std::nothrow) rk_npu_hip_graph();
    std::lock_guard<std::mutex> submit(ctx->submit_mutex);
    void* exec = nullptr;
    const int rc = rkh_capture_end(ctx->stream, &exec); // (always ends the capture, also when g is null)
    std::lock_guard<std::mutex> lock(ctx->pending_mutex);
    ctx->capturing = false;
    if (rc || !g) {
        ctx->capture_flags.clear();
        rkh_graph_destroy(exec);
        delete g;
        return nullptr;
    }
    g->exec = exec;
    g->ctx = ctx;
    g->flags.swap(ctx->capture_flags); // the workspaces whose kernels the graph replays
    ctx->graphs.push_back(g);
    return g;
}
int rk_npu_hip_graph_launch(rk_npu_ctx* ctx, rk_npu_hip_graph* graph) {
    if (!ctx || !graph || !graph->exec || graph->ctx != ctx) return RK_NPU_ERR_PARAM;
    std::lock_guard<std::mutex> submit(ctx->submit_mutex);
    {
        // A replay can reject input exactly like the eager calls it recorded: the next
        // rk_npu_hip_sync has to look at the same flags (the sync before took them off the list).
        std::lock_guard<std::mutex> lock(ctx->pending_mutex);
        for (int* f : graph->flags)
            if (std::find(ctx->pending_flags.begin(), ctx->pending_flags.end(), f) == ctx->pending_flags.end())
                ctx->pending_flags.push_back(f);
    }
    return rkhost::map_error(rkh_graph_launch(graph->exec, ctx->stream));
}
void rk_npu_hip_graph_free(rk_npu_hip_graph* graph) {
    if (!graph) return;
    if (graph->ctx) {
        std::lock_guard<std::mutex> lock(graph->ctx->pending_mutex);
        auto& v = graph->ctx->graphs;
        v.erase(std::remove(v.begin(), v.end(), graph), v.end());
    }
    rkh_graph_destroy(graph->exec);
    delete graph;
}

} // extern "C"
