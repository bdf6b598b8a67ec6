// Host-layer internals shared by the three operator translation units:
// context / domain objects, device buffers with per-domain accounting, the
// workspace busy flag, and small validation helpers.  Nothing here touches
// HIP types: the device is reached only through rk_hip_shim.h.
#ifndef RK_HOST_H
#define RK_HOST_H

#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <memory>
#include <mutex>
#include <vector>

#include "rk_hip_shim.h"
#include "rk_npu_common.h"

struct rk_npu_ctx {
    int device = 0;
    void* stream = nullptr;
    uint64_t id = 0;          // unique per open(), never reused
    int cu_count = 0;
    int clock_khz = 0;
    char arch[64] = {0};
    struct DomainMemory {
        std::atomic<uint64_t> live_bytes{0}, peak_bytes{0}, creates{0}, destroys{0};
    } memory[RK_NPU_IOMMU_DOMAIN_COUNT];
    // Device work of one context is issued on one stream; submissions from
    // different workspaces are serialised here so stream order == call order.
    std::mutex submit_mutex;
    // Rejected-input flags of workspaces used through the *_device entry
    // points since the last rk_npu_hip_sync().
    std::mutex pending_mutex;
    std::vector<int*> pending_flags;
};

struct rk_npu_iommu_domain {
    rk_npu_ctx* ctx = nullptr;
    uint32_t id = 0;
};

namespace rkhost {

inline int map_error(int rkh) {
    if (rkh == RKH_OK) return RK_NPU_OK;
    return rkh == RKH_ERR_NOMEM ? RK_NPU_ERR_NOMEM : RK_NPU_ERR_SUBMIT;
}

// (ctx, domain) tag remembered by every handle for the ERR_DOMAIN check.
struct Owner {
    rk_npu_ctx* ctx = nullptr;
    uint64_t ctx_id = 0;
    uint32_t domain_id = 0;
    void bind(const rk_npu_iommu_domain* d) {
        ctx = d->ctx;
        ctx_id = d->ctx->id;
        domain_id = d->id;
    }
    bool same(const Owner& o) const { return ctx_id == o.ctx_id && domain_id == o.domain_id; }
};

// Device allocation accounted against the owning domain tag.
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    ~DeviceBuffer() { release(); }
    // Allocates and zero-fills.  Returns an RK_NPU_* code.
    int alloc(const Owner& owner, size_t bytes, bool zero = true);
    void release();
    template <class T = uint8_t> T* as() const { return static_cast<T*>(ptr_); }
    size_t bytes() const { return bytes_; }
    explicit operator bool() const { return ptr_ != nullptr; }

private:
    void* ptr_ = nullptr;
    size_t bytes_ = 0;
    Owner owner_;
};

// Non-reentrancy guard of a workspace: try-lock semantics, BUSY on contention.
class BusyLock {
public:
    explicit BusyLock(std::atomic_flag& flag)
        : flag_(flag), held_(!flag.test_and_set(std::memory_order_acquire)) {}
    ~BusyLock() {
        if (held_) flag_.clear(std::memory_order_release);
    }
    BusyLock(const BusyLock&) = delete;
    BusyLock& operator=(const BusyLock&) = delete;
    explicit operator bool() const { return held_; }

private:
    std::atomic_flag& flag_;
    bool held_;
};

inline bool finite_positive(const float* v, size_t n) {
    if (!v) return false;
    for (size_t i = 0; i < n; ++i)
        if (!std::isfinite(v[i]) || !(v[i] > 0.0f)) return false;
    return true;
}

using Clock = std::chrono::steady_clock;
inline double elapsed_us(Clock::time_point t0) {
    return std::chrono::duration<double, std::micro>(Clock::now() - t0).count();
}

// Stream-side stage timer: records events only when the caller asked for
// timings, so the default path adds no event traffic.
class StageTimer {
public:
    StageTimer(void* stream, bool enabled);
    ~StageTimer();
    void mark();                      // record the next event
    double span_us(int from, int to); // elapsed between marks (after sync)
    int marks() const { return count_; }

private:
    void* stream_;
    bool enabled_;
    void* events_[12] = {nullptr};
    int count_ = 0;
};

// Device int that kernels OR a 1 into when they reject input (NaN / Inf
// activations, non-finite SwiGLU middle), with a pinned host mirror so the
// read-back rides the stream before the call's single wait.
class BadFlag {
public:
    ~BadFlag();
    int init(const Owner& owner);
    int* device() const { return dev_.as<int>(); }
    int enqueue_readback(void* stream);
    // After the stream wait: true when input was rejected; re-arms the flag.
    bool consume(void* stream);

private:
    DeviceBuffer dev_;
    int* host_ = nullptr;
};
// Pinned, device-visible mirror of a caller's host buffer for the blocking
// host-pointer entry points.  A copy between pageable memory and the device is
// staged and waited for inside the runtime, once per direction (~15-20 us
// each); a copy from pinned memory still costs a DMA round of ~8-12 us.  The
// kernels can instead read the mirror of a small input directly (each row is
// read once, by the quantization kernel) and write a small result straight into
// the mirror of the output, which adds ~1.5 us to a call.  Only for buffers up
// to kLimit: beyond that the bus transfer itself dominates and the DMA engines
// do it without occupying compute units.  A failed allocation leaves the stage
// off (the call then copies from / to the caller's buffer as before).
class HostStage {
public:
    static constexpr size_t kLimit = size_t(1) << 20;
    HostStage() = default;
    HostStage(const HostStage&) = delete;
    HostStage& operator=(const HostStage&) = delete;
    ~HostStage();
    void init(size_t bytes);        // stays off for 0 or more than kLimit bytes
    void init_capped(size_t bytes); // min(bytes, kLimit): for buffers whose use varies from call to call
    explicit operator bool() const { return ptr_ != nullptr; }
    bool fits(size_t bytes) const { return ptr_ && bytes <= bytes_; }
    // The mirror, filled with `bytes` from `user` (kernels read it in place).
    const void* fill(const void* user, size_t bytes) const;
    // The mirror as a kernel's output; finish() copies it on to `user` after the wait.
    void* data() const { return ptr_; }
    void finish(void* user, size_t bytes) const;

private:
    void* ptr_ = nullptr;
    size_t bytes_ = 0;
};

// Blocking check of one raw device flag (used by rk_npu_hip_sync).
bool consume_device_flag(rk_npu_ctx* ctx, int* flag);
void note_pending_flag(rk_npu_ctx* ctx, int* flag);

// Raw upload of a host array into a fresh device buffer (used at weights_create).
int upload(const Owner& owner, DeviceBuffer& dst, const void* src, size_t bytes);

// Bytes of split-K scratch a dense GEMM of this shape may use (0 = never splits).
inline size_t splitk_scratch_bytes(int M, int N, int K, bool w_int4) {
    return rkh_gemm_scratch_bytes(M, N, K, w_int4 ? 1 : 0);
}

} // namespace rkhost

#endif // RK_HOST_H
