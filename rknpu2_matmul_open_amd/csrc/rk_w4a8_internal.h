// Shared between the W4A8 operator (rk_w4a8.cpp) and its tuning entry points
// (rk_w4a8_tune.cpp): the weight "profile" -- bounds and identity of a weight
// matrix captured when it is created -- and the factory that accepts an
// already resolved K partition.
#ifndef RK_W4A8_INTERNAL_H
#define RK_W4A8_INTERNAL_H

#include <cstdint>

#include "rk_host.h"
#include "rk_npu_w4a8.h"

namespace rkhost {

// What the reference keeps per weight matrix for tuning and cache identity
// (src/rk_npu_w4a8_tune_internal.h:27-35): the largest K tile its INT16-partial
// certificate proves safe, one bit per certified tile size (bit t-1 <=> 32*t),
// the widest tile the multiplier policy admits, and a fingerprint of the codes
// and scales.
struct W4Profile {
    int K = 0, N = 0, safe = 0, limit = 0;
    double multiplier = 1.0;
    uint64_t fingerprint = 0, safe_tiles = 0;
    bool certified(int k) const {
        return k >= 32 && k <= 2048 && k % 32 == 0 && (safe_tiles & (uint64_t(1) << (k / 32 - 1)));
    }
    bool permits(int k) const {
        return k >= 32 && k <= limit && k % 32 == 0 && (certified(k) || multiplier > 1);
    }
    rk_npu_w4a8_weight_info info(int k) const { return {{K, N, k}, safe, multiplier, !certified(k)}; }
};

// Scans B[K, N] (codes in [-8, 7]) and fills `out` for the given multiplier
// (>= 1).  RK_NPU_ERR_PARAM for an out-of-range code, non-finite or
// non-positive scales, or a shape outside the operator's limits.
int w4a8_make_profile(int K, int N, double multiplier, const int8_t* B, const float* w_scale, W4Profile* out);

// Creates weights for an already resolved K partition; `info.config.k_tile`
// beyond the certificate is accepted when info.bound_relaxed says so.  The
// profile is stored in the handle (computed here when `profile` is NULL).
rk_npu_w4a8_weights* w4a8_create_weights(rk_npu_iommu_domain* domain, const rk_npu_w4a8_weight_info& info,
                                         const int8_t* B, const float* w_scale, const W4Profile* profile);

const W4Profile& w4a8_profile_of(const rk_npu_w4a8_weights* weights);

// RK_NPU_W4A8_K_TILE_MULTIPLIER: 1 when unset, < 0 when set but invalid.
double w4a8_env_multiplier();

// True when the INT16-partial certificate holds for exactly this K tile
// (multiple of 32) on B[K, N]; false also for a code outside [-8, 7].
bool i4_tile_certified(const int8_t* B, int K, int N, int k_tile);

} // namespace rkhost

#endif
