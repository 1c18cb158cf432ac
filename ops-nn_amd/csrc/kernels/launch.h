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
// How many ways a call with `tiles` output tiles, `ktiles` K tiles of `tile_us` microseconds each and `out_elems` outputs
// is split: at most one workgroup per CU, at least four K tiles per workgroup, at most sixteen ways -- and among those the
// count with the largest estimated gain, if that is at least 3 us: the loop time saved, ktiles * tile_us * (1 - 1/s), less
// a second launch (4 us) and the partial sums written and read back (2 s out_elems 4 bytes at `bytes_per_us`: fitted to
// measurements, 5e6 for the kernels that store 64-byte row pieces from 16 x 16 fragments, 2.4e6 for the 32 x 32-fragment
// kernel's 32-byte pieces).  (Measured without the traffic term: MXFP4 1024 x 4096 x 4096 in four splits 28 -> 65 us.)
inline int splitk_factor(int64_t tiles, int64_t ktiles, double tile_us, int64_t out_elems, double bytes_per_us)
{
    if (tiles <= 0 || tiles > 128) return 1;
    int64_t smax = 256 / tiles;
    if (smax > ktiles / 4) smax = ktiles / 4;
    if (smax > 16) smax = 16;
    int best = 1;
    double best_gain = 3.0;
    for (int64_t s = 2; s <= smax; s++) {
        const double gain = (double)ktiles * tile_us * (1.0 - 1.0 / (double)s) - 4.0 - 2.0 * (double)s * (double)out_elems * 4.0 / bytes_per_us;
        if (gain > best_gain) { best = (int)s; best_gain = gain; }
    }
    return best;
}
// How the x-in-registers kernel (weight-only, up to 16 rows of x) covers K.  A workgroup holds `nw` waves x `nch` chunks
// (of 64 weight bytes): 16 x 4, 8-bit weights also 16 x 8, or 8 x 4 / 8 x 8.  A K that is exactly one such shape runs on
// one workgroup per row block range; any other K of whole 128-element units goes in `splits` segments of 16 x 4 chunks
// (else of 8 x 4), one workgroup column per segment, the last one with idle chunks past the end of K (`exact` false) when
// that wastes at most a fifth of K's chunks; with more than one segment the columns leave fp32 partial sums
// [splits][M][N] at the front of the workspace.  False: the kernel does not take this K.
struct WqXregPlan {
    int nw, nch, splits;
    bool exact;
};
inline bool wq_xreg_plan(int wbits, int64_t M, int64_t K, WqXregPlan& pl)
{
    const int64_t kc = 4 * (128 / wbits);
    if (M < 1 || M > 16 || K < 128 || K % 128 != 0) return false;
    const int64_t nch = K / kc;
    if (nch == 64) { pl = {16, 4, 1, true}; return true; }
    if (wbits == 8 && nch == 128) { pl = {16, 8, 1, true}; return true; }
    if (nch == 32) { pl = {8, 4, 1, true}; return true; }
    const int64_t s64 = (nch + 63) / 64, w64 = s64 * 64 - nch, s32 = (nch + 31) / 32, w32 = s32 * 32 - nch;
    if (s64 == 1 && w64 * 5 <= nch) { pl = {16, 4, 1, false}; return true; }   // one workgroup, its last waves idle
    if (s32 <= 16 && w32 * 5 <= nch) { pl = {8, 4, (int)s32, w32 == 0}; return true; }
    if (s64 <= 16 && w64 * 5 <= nch) { pl = {16, 4, (int)s64, w64 == 0}; return true; }
    return false;
}
// the count of partial-sum slices that plan needs (0: none)
inline int wq_xreg_splits(int wbits, int64_t M, int64_t K)
{
    WqXregPlan pl;
    return (wq_xreg_plan(wbits, M, K, pl) && pl.splits > 1) ? pl.splits : 1;
}
// Row slabs of the many-rows weight-only kernel for a narrow N.  Its workgroups take 128 columns each, so one pass over a
// narrow weight leaves most CUs idle, and passes launched one after the other do not overlap (4096 x 4096 int4: 32
// workgroups, 256 rows 56 us, 1024 rows in four passes 219 us).  With at most 128 workgroups per pass and more than 64
// rows the rows are cut into equal slabs of 64 .. 256 rows, as many as give every CU a workgroup in one round, and all
// slabs go out in one launch (grid.y).  Returns the slab's rows, or 0 where the one-pass-at-a-time order stays.
inline int64_t wq_narrow_slab_rows(int64_t M, int64_t N, bool on)
{
    const int64_t wgs = (N + 127) / 128;
    if (M <= 64 || wgs > 128 || !on) return 0;
    int64_t n = 256 / wgs;
    if (n > (M + 63) / 64) n = (M + 63) / 64;
    if (n < (M + 255) / 256) n = (M + 255) / 256;
    if (n < 2) return 0;
    return ((M + n - 1) / n + 15) / 16 * 16;
}
// The same kernel, from 17 rows: a narrow N leaves CUs without a workgroup even with all row slabs in one
// launch (64 rows against 28672 x 8192: 64 workgroups of 128 columns), and a long K makes each of them slow.  Then K is
// cut into segments, one per blockIdx.z, whose fp32 partial sums a second kernel adds in segment order.  Segments are
// whole units (a slab of x of the 64-row instance -- two chunks of 128 bytes of a weight row -- or a group where that is
// longer), as equal as that allows, at least 2048 k each.  Returns the segment count (1: no split) and the unit.
// (Measured, int4 with groups of 128, 64 rows: 14336 x 4096 64 -> 22 us, 28672 x 8192 124 -> 66, 8192 x 8192 30 -> 24; a K
// of 4096 lost 2 to 6 us to the second kernel, and so did two segments of 128 workgroups at K = 8192; 64 x 7168 x 7168, where
// the 64-column workgroups cannot run, 42 -> 26.)
inline int wq_rows_ksplit(int wbits, int64_t M, int64_t N, int64_t K, int64_t group, bool on, int64_t* kunit = nullptr)
{
    if (!on || M < 17 || N % 32 != 0 || N < 256 || K < 4096 || K >= (1ll << 23)) return 1;
    const int64_t slab = wq_narrow_slab_rows(M, N, on);
    if (M > 64 && slab == 0) return 1;
    const int64_t slabs = slab ? (M + slab - 1) / slab : 1;
    const int64_t wgs = slabs * ((N + 127) / 128), kx = 2 * 4 * (128 / wbits);
    int64_t unit = kx;
    if (group < K) {
        if (group > kx) unit = group;
        if (unit % group != 0 || unit % kx != 0) return 1;
    }
    if (wgs > 128 || K % unit != 0) return 1;
    // (below 8192 only where the 64-column workgroups, which double the workgroups without a second kernel, cannot run: they
    // want K in whole slabs of four chunks; and from 33 rows: 17 x 5120 x 5120 int4 took 19 us on the streaming kernel, 22 here)
    if (K < 8192 && (K % (2 * kx) == 0 || wgs > 64 || M < 33)) return 1;
    int64_t s = 256 / wgs;
    if (s > 8) s = 8;
    if (s > K / 2048) s = K / 2048;
    if (s > K / unit) s = K / unit;
    if (s == 2 && wgs > 64 && K < 12288) return 1;
    if (kunit) *kunit = unit;
    return s < 2 ? 1 : (int)s;
}
// fp32 partial-sum slices [slices][M][N] at the front of a weight-only call's workspace (1: none)
inline int wq_part_slices(int wbits, int64_t M, int64_t N, int64_t K, int64_t group, bool narrow_on)
{
    if (M <= 16) return wq_xreg_splits(wbits, M, K);
    return wq_rows_ksplit(wbits, M, N, K, group, narrow_on);
}
// The fp8 / int8 decode kernel (qmm_fp8_decode.hip, up to 32 rows of x1): K in blocks of 128 that the NW = 16 or 8 waves
// of a workgroup share, NBLK each (a wave keeps its blocks of x1 in registers: 16 waves up to 4, not 3; 8 waves up to 7).
// A K that the waves of one workgroup share exactly runs as one segment; any other whole number of blocks in 1 .. 16
// segments of NW * NBLK blocks, the last one with idle waves (K a whole number of NBLK blocks): the layout with the fewest
// wave slots, then the fewest segments.  More than one segment needs room for fp32 partial sums (may_split).
// (w4: the fp8 x fp4 MX form of the kernel, which has no instance of 16 waves with one block each.)
struct QmmDecodePlan { int nw = 0, nblk = 0, splits = 1; };
inline bool qmm_decode_plan(int64_t K, bool may_split, QmmDecodePlan& pl, bool w4 = false)
{
    if (K <= 0 || K % 128 != 0) return false;
    const int64_t nb = K / 128;
    if (nb % 16 == 0 && nb / 16 <= 4 && nb / 16 != 3 && !(w4 && nb == 16)) { pl.nw = 16; pl.nblk = (int)(nb / 16); pl.splits = 1; return true; }
    if (nb % 8 == 0 && nb / 8 <= 7) { pl.nw = 8; pl.nblk = (int)(nb / 8); pl.splits = 1; return true; }
    static const int shapes[10][2] = {{16, 4}, {16, 2}, {16, 1}, {8, 7}, {8, 6}, {8, 5}, {8, 4}, {8, 3}, {8, 2}, {8, 1}};
    int64_t best_slots = 0;
    bool found = false;
    for (const auto& sh : shapes) {
        const int nw = sh[0], nblk = sh[1];
        if (nb % nblk != 0 || (w4 && nw == 16 && nblk == 1)) continue;
        const int64_t waves = nb / nblk, s = (waves + nw - 1) / nw;
        if (s > 16 || (s > 1 && !may_split)) continue;
        const int64_t slots = s * nw * nblk;
        if (!found || slots < best_slots || (slots == best_slots && s < pl.splits)) {
            found = true; best_slots = slots; pl.nw = nw; pl.nblk = nblk; pl.splits = (int)s;
        }
    }
    return found;
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
