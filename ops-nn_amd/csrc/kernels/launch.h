// Internal: kernel-variant ids shared by the launchers and the selector.
#pragma once
#include "opsnn_kernels.h"

#define OPSNN_NOT_TAKEN 0x7fff0001

enum {
    OPSNN_VARIANT_AUTO = 0,
    OPSNN_VARIANT_PLAIN = 1,      // strided one-thread-per-output kernels (any shape)
    OPSNN_VARIANT_I8_256 = 2,     // int8 MFMA, 256x256 tile
    OPSNN_VARIANT_I8_128 = 3,     // int8 MFMA, 128x128 tile
    OPSNN_VARIANT_I8_256x128_S3 = 4,  // int8 MFMA, 256x128 tile, BK 64, 3 stages, 2 workgroups per CU
    OPSNN_VARIANT_I8_256_W8 = 5,  // int8 MFMA, 256x256 tile, 8 waves, BK 64, 4 stages
    OPSNN_VARIANT_I8_256_S4 = 6,  // int8 MFMA, 256x256 tile, 4 waves, BK 64, 4 stages
    OPSNN_VARIANT_I8_256_W8_K128 = 7,  // int8 MFMA, 256x256 tile, 8 waves, BK 128, 2 stages
    OPSNN_VARIANT_I8_WIDE8 = 8,   // int8 MFMA, 4 waves with 128 x 16n sub-tiles, 256 x 32n tile, n = 8..11 (ids 8..11)
    OPSNN_VARIANT_I8_WIDE11 = 11,
    OPSNN_VARIANT_MX_128 = 16,    // MX MFMA, 128x128 tile
    OPSNN_VARIANT_MX_FP8_MFMA = 17,  // MXFP8 on the MFMA path (reduced accumulation precision, see qmm_mx.hip)
};

#ifdef __cplusplus
#ifdef __HIPCC__
#include <hip/hip_runtime.h>
#include <atomic>
namespace opsnn {
// hipFuncSetAttribute belongs to a (kernel, device) pair: launchers keep one of these masks per kernel instantiation,
// a bit per device ordinal (mod 64).  Two threads that both find the bit clear both set the attribute: harmless.
inline bool device_flag_test(const std::atomic<uint64_t>& mask)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    return (mask.load(std::memory_order_acquire) >> (dev & 63)) & 1u;
}
inline void device_flag_set(std::atomic<uint64_t>& mask)
{
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess) mask.fetch_or(1ull << (dev & 63), std::memory_order_release);
}
}  // namespace opsnn
#endif
namespace opsnn {
// K split over workgroups for tile-kernel calls whose tiles would leave most of the chip idle (few rows against a narrow N):
// `splits` workgroups per tile each take a contiguous range of K tiles and leave fp32 partial sums in `part`
// ([splits][batch][M][N], at the front of the call's workspace); a second kernel adds them in split order, adds the bias
// and rounds.  splits <= 1: one workgroup per tile, no partial sums.
struct SplitK {
    int splits = 1;
    float* part = nullptr;
};
// How many ways a call with `tiles` output tiles (at most max_tiles, else it is not split) and `ktiles` K tiles is split:
// enough to give every CU a workgroup, at least four K tiles per workgroup, at most sixteen ways.
inline int splitk_factor(int64_t tiles, int64_t ktiles, int64_t max_tiles = 128)
{
    if (tiles <= 0 || tiles > max_tiles) return 1;
    int64_t s = 256 / tiles;
    if (s > ktiles / 4) s = ktiles / 4;
    if (s > 16) s = 16;
    return s >= 2 ? (int)s : 1;
}
// Opened by every exported matmul entry point for the time it enqueues its launches (weight_cache.hip): copies that the
// weight cache hands out inside the scope cannot be evicted before it closes; bypass = true switches the cache off for
// this thread while the scope is open.  Scopes nest; the pins drop when the outermost one closes.
class WeightCacheScope {
public:
    explicit WeightCacheScope(bool bypass = false);
    ~WeightCacheScope();
    WeightCacheScope(const WeightCacheScope&) = delete;
    WeightCacheScope& operator=(const WeightCacheScope&) = delete;
private:
    bool saved_bypass_;
};
}  // namespace opsnn
#endif
