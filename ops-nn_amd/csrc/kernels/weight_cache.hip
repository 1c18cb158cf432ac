// Opt-in cache of re-laid-out right operands.  The matrix-core kernels stream a K-contiguous right operand; a caller
// that keeps the reference's literal [K, N] storage pays one re-layout pass per call unless the copy is kept.  With the
// cache switched on (opsnnSetWeightCache(max_bytes) or OPSNN_WEIGHT_CACHE_MB) the launchers keep the K-contiguous
// copy in memory of the library's own, keyed by the operand's device address, shape, element width and batch count:
// the first call pays the pass, later calls with the same operand find the copy.  This is the runtime counterpart of
// the offline weight re-layout that the reference folds into its graphs
// (matmul/weight_quant_batch_matmul_v2/op_graph/fusion_pass/weight_quant_batch_matmul_v2_transpose_fusion_pass.cpp,
// matmul/quant_batch_matmul_v4/op_graph/fusion_pass/quant_batch_matmul_v4_transpose_fusion_pass.cpp).
//
// Contract: the cache cannot see a weight change.  A caller that overwrites, frees or re-uses the memory of a cached
// operand must call opsnnWeightCacheClear() first.  Off by default.
// A copy is written on the stream of the call that misses; an event recorded behind it orders every later use on
// any stream.  Nothing is cached (and the caller's workspace path runs) while the stream is being captured into a
// graph, when the copy does not fit the limit, or when the allocation fails.  Entries are evicted least recently
// used first; hipFree waits for the device, so no kernel can still be reading an evicted copy.
#include <cstdlib>
#include <list>
#include <mutex>

#include <hip/hip_runtime.h>

#include "launch.h"

namespace opsnn {
namespace {

struct Entry {
    const void* src; int64_t K, N, nb; int bits;
    void* copy; uint64_t bytes; hipEvent_t ready; int device;
};

std::mutex g_mu;
std::list<Entry> g_entries;   // most recently used first
uint64_t g_limit = [] { const char* e = getenv("OPSNN_WEIGHT_CACHE_MB"); return e ? (uint64_t)atoll(e) << 20 : (uint64_t)0; }();
uint64_t g_used = 0, g_hits = 0, g_misses = 0;

void drop(std::list<Entry>::iterator it)
{
    (void)hipEventDestroy(it->ready);
    (void)hipFree(it->copy);
    g_used -= it->bytes;
    g_entries.erase(it);
}

}  // namespace

// The K-contiguous copy of the [K, N] matrix (N contiguous, nb dense batches) of `bits`-wide elements at src, ready for
// use on `st`; nullptr when the cache does not serve this call (the caller then re-lays the operand out itself).
const void* weight_cache_get(const void* src, int64_t K, int64_t N, int bits, int64_t nb, hipStream_t st)
{
    if (!g_limit || !src || K <= 0 || N <= 0 || nb <= 0) return nullptr;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) return nullptr;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    const uint64_t bytes = (uint64_t)K * (uint64_t)N * (uint64_t)bits / 8 * (uint64_t)nb;
    std::lock_guard<std::mutex> lock(g_mu);
    for (auto it = g_entries.begin(); it != g_entries.end(); ++it) {
        if (it->src == src && it->K == K && it->N == N && it->bits == bits && it->nb == nb && it->device == dev) {
            if (hipStreamWaitEvent(st, it->ready, 0) != hipSuccess) return nullptr;
            g_entries.splice(g_entries.begin(), g_entries, it);
            g_hits++;
            return it->copy;
        }
    }
    if (bytes > g_limit) return nullptr;
    while (g_used + bytes > g_limit && !g_entries.empty()) drop(std::prev(g_entries.end()));
    Entry e{src, K, N, nb, bits, nullptr, bytes, nullptr, dev};
    if (hipMalloc(&e.copy, bytes) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    if (hipEventCreateWithFlags(&e.ready, hipEventDisableTiming) != hipSuccess) { (void)hipFree(e.copy); return nullptr; }
    const int rc = bits == 4 ? opsnnTranspose4(src, e.copy, K, N, nb, st) : opsnnTranspose8(src, e.copy, K, N, nb, st);
    if (rc != 0 || hipEventRecord(e.ready, st) != hipSuccess) {
        (void)hipEventDestroy(e.ready);
        (void)hipFree(e.copy);
        return nullptr;
    }
    g_used += bytes;
    g_misses++;
    g_entries.push_front(e);
    return e.copy;
}

}  // namespace opsnn

using namespace opsnn;

extern "C" void opsnnSetWeightCache(int64_t max_bytes)
{
    std::lock_guard<std::mutex> lock(g_mu);
    g_limit = max_bytes > 0 ? (uint64_t)max_bytes : 0;
    while (g_used > g_limit && !g_entries.empty()) drop(std::prev(g_entries.end()));
}

extern "C" void opsnnWeightCacheClear(void)
{
    std::lock_guard<std::mutex> lock(g_mu);
    while (!g_entries.empty()) drop(g_entries.begin());
}

extern "C" void opsnnWeightCacheStats(int64_t* entries, int64_t* bytes, int64_t* hits, int64_t* misses)
{
    std::lock_guard<std::mutex> lock(g_mu);
    if (entries) *entries = (int64_t)g_entries.size();
    if (bytes) *bytes = (int64_t)g_used;
    if (hits) *hits = (int64_t)g_hits;
    if (misses) *misses = (int64_t)g_misses;
}
