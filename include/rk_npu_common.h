/*
 * rk_npu_common.h -- context, domain tags and error codes shared by the
 * quantized-linear operators of this library (MI355X / gfx950 build).
 *
 * This header keeps the caller-visible names and values of the reference's
 * include/rk_npu_common.h:28-37 (error codes), :76-77 (opaque ctx / domain),
 * :126-135 (open / close / domain create / free / id), :147-153 (reclaim hook) and :156
 * (strerror), so
 * code written against the reference links against this library unchanged.
 *
 * What is different underneath: a context owns one HIP device and one HIP
 * stream instead of a DRM file descriptor; an "IOMMU domain" is a small tag
 * object whose only job is the cross-domain check (RK_NPU_ERR_DOMAIN) that the
 * operator run functions perform.  The rknpu GEM / dmabuf memory helpers
 * (rk_npu_mem_*) of the reference are what the HIP runtime replaces and are
 * not part of this library.
 */
#ifndef RK_NPU_COMMON_H
#define RK_NPU_COMMON_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Return codes of every int-returning entry point. */
#define RK_NPU_OK               0
#define RK_NPU_ERR_OPEN       (-1)  /* no usable device                          */
#define RK_NPU_ERR_IOCTL      (-2)  /* a device runtime call failed               */
#define RK_NPU_ERR_PARAM      (-3)  /* invalid argument / rejected input          */
#define RK_NPU_ERR_NOMEM      (-4)  /* host or device allocation failed           */
#define RK_NPU_ERR_SUBMIT     (-5)  /* a kernel launch or stream wait failed      */
#define RK_NPU_ERR_BUSY       (-6)  /* workspace already running on another thread*/
#define RK_NPU_ERR_DOMAIN     (-7)  /* objects come from different ctx / domain   */
#define RK_NPU_ERR_IO         (-8)  /* file I/O failed                            */
#define RK_NPU_ERR_CACHE_MISS (-9)  /* tuning cache absent or stale               */

#define RK_NPU_IOMMU_DOMAIN_COUNT 16u

typedef struct rk_npu_ctx rk_npu_ctx;
typedef struct rk_npu_iommu_domain rk_npu_iommu_domain;

/*
 * Open a device context.  dev == NULL selects HIP device 0; "hip:N" selects
 * device N.  Any other string fails with errno = ENODEV.  Returns NULL (errno
 * set) when no gfx950-capable device can be initialised.  The context must
 * outlive every handle created from it.
 * Replaces rk_npu_open / rk_npu_close (reference include/rk_npu_common.h:126-127).
 */
rk_npu_ctx* rk_npu_open(const char* dev);
void rk_npu_close(rk_npu_ctx* ctx);

/*
 * Domain tags 0..15.  A handle remembers the (ctx, domain id) it was created
 * with; mixing handles of different tags in one run returns
 * RK_NPU_ERR_DOMAIN.  A domain object may be freed as soon as the handles
 * made from it exist.  (reference include/rk_npu_common.h:132-135)
 */
rk_npu_iommu_domain* rk_npu_iommu_domain_create(rk_npu_ctx* ctx, uint32_t domain_id);
void rk_npu_iommu_domain_free(rk_npu_iommu_domain* domain);
uint32_t rk_npu_iommu_domain_id(const rk_npu_iommu_domain* domain);

/* Device bytes currently / at most held by handles created from this domain
 * tag, and how many allocations were made and released
 * (reference include/rk_npu_common.h:141-145). */
typedef struct {
    uint64_t live_bytes, peak_bytes, creates, destroys;
} rk_npu_domain_memory_stats;
int rk_npu_iommu_domain_memory_stats(const rk_npu_iommu_domain* domain,
                                     rk_npu_domain_memory_stats* stats);

/*
 * Optional reclaim hook of a domain tag (reference include/rk_npu_common.h:147-153,
 * src/rk_npu_core.cpp:176-210).  When a device allocation made for this (context, domain id)
 * reports out-of-memory, the hook is called once and the allocation is tried once more; of
 * several allocations that fail together only the first runs the hook.  The hook may free
 * handles of this library but must not create any.  Install or clear it (reclaim == NULL)
 * while no thread is creating handles in the domain, and keep `cookie` alive while it is
 * installed.  The hook belongs to the (context, domain id) pair, not to the domain object it
 * was installed through: freeing that object does not clear it.
 */
typedef void (*rk_npu_reclaim_idle_fn)(void* cookie);
void rk_npu_iommu_domain_set_reclaim(rk_npu_iommu_domain* domain, rk_npu_reclaim_idle_fn reclaim, void* cookie);

/* Fixed English text for a return code (reference include/rk_npu_common.h:156). */
const char* rk_npu_strerror(int code);

#ifdef __cplusplus
}
#endif
#endif /* RK_NPU_COMMON_H */
