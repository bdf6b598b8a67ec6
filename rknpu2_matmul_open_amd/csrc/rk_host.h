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
    // This device's copy of the library's static scratch array (looked up at open; null when
    // the lookup failed): memory for the entry point that allocates nothing.
    void* scratch = nullptr;
    size_t scratch_bytes = 0;
    struct DomainMemory {
        std::atomic<uint64_t> live_bytes{0}, peak_bytes{0}, creates{0}, destroys{0};
        // Reclaim hook of the domain tag (rk_npu_iommu_domain_set_reclaim): called once when a
        // device allocation for this tag reports out-of-memory, after which the allocation is
        // tried once more.  `reclaim_epoch` counts completed calls, so that of several
        // allocations failing together only the first one runs the hook.
        std::mutex reclaim_mutex;
        rk_npu_reclaim_idle_fn reclaim = nullptr;
        void* reclaim_cookie = nullptr;
        std::atomic<uint64_t> reclaim_epoch{0};
    } memory[RK_NPU_IOMMU_DOMAIN_COUNT];
    // Device work of one context is issued on one stream; submissions from
    // different workspaces are serialised here so stream order == call order.
    std::mutex submit_mutex;
    // Per-kernel profile (rk_npu_hip_profile_begin / _end): one stream event in front of every
    // kernel launched on this context's stream while it is on.
    struct ProfileMark {
        const char* kernel;
        void* event;
    };
    std::mutex profile_mutex;
    bool profiling = false;
    std::vector<ProfileMark> profile_marks;
    // Rejected-input flags of workspaces used through the *_device entry
    // points since the last rk_npu_hip_sync().
    std::mutex pending_mutex;
    std::vector<int*> pending_flags;
    // Stream capture (rk_npu_hip_capture_begin / _end): the flags noted while capturing are kept
    // with the graph, whose every launch registers them again -- a replay runs the same kernels
    // and can reject input like the eager call did.  `graphs` lists the live graphs of this
    // context so that a workspace being freed can take its flag out of them.
    bool capturing = false;
    std::vector<int*> capture_flags;
    std::vector<struct rk_npu_hip_graph*> graphs;
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
// host-pointer entry points.  Measured on this box: a copy between pageable
// memory and the device is staged and waited for inside the runtime (15-20 us
// per direction when small; 36 GB/s up, 17 GB/s down when large); a DMA from /
// to pinned memory costs 8-12 us when small and runs at 55 GB/s; a plain
// memcpy runs at 80 GB/s.
//  * Up to kLimit bytes ("direct"): no copy at all.  The quantization kernel
//    reads A from the mirror (each row once) and the GEMM writes its result
//    straight into the output's mirror, which adds ~1.5 us to a call.
//  * Up to kPipeLimit bytes: the mirror is a staging buffer.  Uploads memcpy a
//    chunk and enqueue its DMA while the next chunk is being copied; downloads
//    enqueue one DMA per chunk with an event behind it and memcpy each chunk to
//    the caller's buffer as soon as its event has passed.
// Beyond that, or when the pinned allocation fails, the calls copy from / to
// the caller's buffer as the runtime sees fit.
class HostStage {
public:
    static constexpr size_t kLimit = size_t(1) << 20;
    // Results of the W8A8 and MoE calls are written in place up to 4 MiB: the reference's bench_llm_i8 at 128
    // rows (2 MiB of int32) 158 -> 143 us (4096 x 4096), 201 -> 183 us (11008 x 4096), the MoE layer of 256
    // tokens 281 -> 262 us; 8 MiB and more lose (5.6 MiB of int32: 290 -> 340 - 390 us), and the W4A8 calls
    // keep the input's limit (the FFN's 2 MiB of fp32 written in place: 510 -> 560 us).
    static constexpr size_t kOutLimit = size_t(4) << 20;
    static constexpr size_t kPipeLimit = size_t(64) << 20;
    static constexpr size_t kChunk = size_t(2) << 20;
    HostStage() = default;
    HostStage(const HostStage&) = delete;
    HostStage& operator=(const HostStage&) = delete;
    ~HostStage();
    void init(size_t bytes);        // stays off for 0 or more than kPipeLimit bytes
    explicit operator bool() const { return ptr_ != nullptr; }
    bool direct(size_t bytes) const { return ptr_ && bytes <= bytes_ && bytes <= kLimit; }
    bool direct_out(size_t bytes) const { return ptr_ && bytes <= bytes_ && bytes <= kOutLimit; }
    // direct use: the mirror filled with `bytes` from `user` (kernels read it in place) ...
    const void* fill(const void* user, size_t bytes) const;
    // ... and the mirror as a kernel's output; finish() copies it on to `user` after the wait.
    void* data() const { return ptr_; }
    void finish(void* user, size_t bytes) const;
    // staged use: enqueue the upload of `bytes` from `user` to `device` (RKH_* code)
    int upload(void* stream, void* device, const void* user, size_t bytes) const;
    // enqueue the download of `bytes` from `device`, then wait for it and deliver it to `user`
    int download(void* stream, void* user, const void* device, size_t bytes);
    int finish_download(void* stream, void* user, size_t bytes);

private:
    void* ptr_ = nullptr;
    size_t bytes_ = 0;
    std::vector<void*> events_; // one per chunk of a staged download
    bool staged_ = false;       // the enqueued download went through the mirror
};

// Blocking check of one raw device flag (used by rk_npu_hip_sync).
bool consume_device_flag(rk_npu_ctx* ctx, int* flag);
void note_pending_flag(rk_npu_ctx* ctx, int* flag);
// A workspace that owns `flag` is going away: no later sync or graph launch may read it.
void forget_pending_flag(rk_npu_ctx* ctx, int* flag);

// Raw upload of a host array into a fresh device buffer (used at weights_create).
int upload(const Owner& owner, DeviceBuffer& dst, const void* src, size_t bytes);

// Bytes of split-K scratch a dense GEMM of this shape may use (0 = never splits).
inline size_t splitk_scratch_bytes(int M, int N, int K, bool w_int4) {
    return rkh_gemm_scratch_bytes(M, N, K, w_int4 ? 1 : 0);
}

} // namespace rkhost

#endif // RK_HOST_H
