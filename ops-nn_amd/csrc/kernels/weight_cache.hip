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
// operand must call opsnnWeightCacheInvalidate(ptr, bytes) for that operand (or opsnnWeightCacheClear()) first.  Off by
// default.
// A copy is written on the stream of the call that misses; an event recorded behind it orders every later use on
// any stream.  Nothing is cached (and the caller's workspace path runs) while the stream is being captured into a
// graph, when the copy does not fit the limit, or when the allocation fails.  Entries are evicted least recently
// used first; hipFree waits for the device, so no kernel that is already enqueued can still be reading an evicted copy.
// A call that has been handed a copy but has not enqueued its kernels yet is protected by a pin: every exported matmul
// entry point opens a WeightCacheScope, each copy handed out inside it is pinned, and the pins drop when the scope
// closes (all launches enqueued).  Pinned entries are never evicted; clearing the cache or lowering the limit takes a
// pinned entry out of the table at once and frees it when its last pin drops.
// A scope can also switch the cache off for its thread (WeightCacheScope(true)): the FRACTAL_NZ entry points, which
// re-write the keyed memory -- the front of the caller's workspace -- on every call, and the entry point that promises to
// allocate nothing.
#include <cstdlib>
#include <list>
#include <mutex>

#include <hip/hip_runtime.h>

#include "launch.h"

namespace opsnn {
namespace {

struct Entry {
    const void* src; const void* src2; const void* src3; int64_t K, N, nb; int bits;
    void* copy; uint64_t bytes; hipEvent_t ready; int device;
    bool committed;   // filled and its event recorded; until then other callers do not use it
    int pins;         // calls that hold `copy` and may not have enqueued their kernels yet
};

std::mutex g_mu;
std::list<Entry> g_entries;   // most recently used first
std::list<Entry> g_zombies;   // taken out of the table while pinned: freed when the last pin drops
uint64_t g_limit = [] { const char* e = getenv("OPSNN_WEIGHT_CACHE_MB"); return e ? (uint64_t)atoll(e) << 20 : (uint64_t)0; }();
uint64_t g_used = 0, g_hits = 0, g_misses = 0;

struct ThreadScope {
    int depth = 0;
    bool bypass = false;
    void* pinned[8];
    int n = 0;
};
thread_local ThreadScope t_scope;

void release(const Entry& e)
{
    (void)hipEventDestroy(e.ready);
    (void)hipFree(e.copy);
}

// Takes the entry out of the table (g_mu held); its memory goes at once unless a call still holds it.  Returns the
// entry that followed it.
std::list<Entry>::iterator drop(std::list<Entry>::iterator it)
{
    g_used -= it->bytes;
    const auto next = std::next(it);
    if (it->pins > 0) g_zombies.splice(g_zombies.begin(), g_entries, it);
    else {
        release(*it);
        g_entries.erase(it);
    }
    return next;
}

// Pins the entry for the open scope of this thread (g_mu held).  False when no scope is open or it is full: the entry
// is then not handed out.
bool pin(Entry& e)
{
    ThreadScope& t = t_scope;
    if (t.depth <= 0 || t.n >= (int)(sizeof(t.pinned) / sizeof(t.pinned[0]))) return false;
    t.pinned[t.n++] = e.copy;
    e.pins++;
    return true;
}

void unpin_all()
{
    ThreadScope& t = t_scope;
    if (!t.n) return;
    std::lock_guard<std::mutex> lock(g_mu);
    for (int i = 0; i < t.n; i++) {
        bool found = false;
        for (auto it = g_entries.begin(); it != g_entries.end() && !found; ++it)
            if (it->copy == t.pinned[i]) { it->pins--; found = true; }
        for (auto it = g_zombies.begin(); it != g_zombies.end() && !found; ++it)
            if (it->copy == t.pinned[i]) {
                found = true;
                if (--it->pins <= 0) {
                    release(*it);
                    g_zombies.erase(it);
                }
            }
    }
    t.n = 0;
}

}  // namespace

WeightCacheScope::WeightCacheScope(bool bypass) : saved_bypass_(t_scope.bypass)
{
    t_scope.depth++;
    if (bypass) t_scope.bypass = true;
}
WeightCacheScope::~WeightCacheScope()
{
    t_scope.bypass = saved_bypass_;
    if (--t_scope.depth == 0) unpin_all();
}

// A buffer of `bytes` that belongs to the operand (src, src2, src3 -- e.g. data, scales and offsets --, shape, element width,
// batch count):
// on a hit (*fresh = false) it holds what an earlier call put there and is ordered behind that call's writes on `st`; on a
// miss (*fresh = true) it is new: the caller fills it with launches on `st` and then calls weight_cache_commit(buffer, st).
// nullptr when the cache does not serve this call (off, under graph capture, larger than the limit, allocation failure).
void* weight_cache_blob3(const void* src, const void* src2, const void* src3, int64_t K, int64_t N, int bits, int64_t nb, uint64_t bytes, hipStream_t st,
                         bool* fresh)
{
    *fresh = false;
    if (!g_limit || t_scope.bypass || t_scope.depth <= 0 || !src || K <= 0 || N <= 0 || nb <= 0 || !bytes) return nullptr;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) return nullptr;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lock(g_mu);
    for (auto it = g_entries.begin(); it != g_entries.end(); ++it) {
        if (it->src == src && it->src2 == src2 && it->src3 == src3 && it->K == K && it->N == N && it->bits == bits && it->nb == nb && it->bytes == bytes &&
            it->device == dev) {
            if (!it->committed) return nullptr;   // another call is still filling it: this one goes its own way
            if (hipStreamWaitEvent(st, it->ready, 0) != hipSuccess) return nullptr;
            if (!pin(*it)) return nullptr;
            g_entries.splice(g_entries.begin(), g_entries, it);
            g_hits++;
            return it->copy;
        }
    }
    if (bytes > g_limit) return nullptr;
    // make room: least recently used first, skipping what a call still holds or is still filling
    for (auto it = g_entries.end(); g_used + bytes > g_limit && it != g_entries.begin();) {
        --it;
        if (it->pins > 0 || !it->committed) continue;
        it = drop(it);
    }
    if (g_used + bytes > g_limit) return nullptr;   // everything else is in use
    Entry e{src, src2, src3, K, N, nb, bits, nullptr, bytes, nullptr, dev, false, 0};
    if (hipMalloc(&e.copy, bytes) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    if (hipEventCreateWithFlags(&e.ready, hipEventDisableTiming) != hipSuccess) { (void)hipFree(e.copy); return nullptr; }
    if (!pin(e)) { release(e); return nullptr; }
    // until the commit nobody else uses the entry; one whose filling call fails is removed by weight_cache_abandon
    g_used += bytes;
    g_misses++;
    g_entries.push_front(e);
    *fresh = true;
    return e.copy;
}

void* weight_cache_blob(const void* src, const void* src2, int64_t K, int64_t N, int bits, int64_t nb, uint64_t bytes, hipStream_t st, bool* fresh)
{
    return weight_cache_blob3(src, src2, nullptr, K, N, bits, nb, bytes, st, fresh);
}

// The fresh buffer has been filled by the launches already enqueued on st.
void weight_cache_commit(void* buffer, hipStream_t st)
{
    std::lock_guard<std::mutex> lock(g_mu);
    for (auto it = g_entries.begin(); it != g_entries.end(); ++it)
        if (it->copy == buffer) {
            if (hipEventRecord(it->ready, st) == hipSuccess) it->committed = true;
            else drop(it);
            return;
        }
}

// The fresh buffer could not be filled: forget it.
void weight_cache_abandon(void* buffer)
{
    std::lock_guard<std::mutex> lock(g_mu);
    for (auto it = g_entries.begin(); it != g_entries.end(); ++it)
        if (it->copy == buffer) { drop(it); return; }
}

// The K-contiguous copy of the [K, N] matrix (N contiguous, nb dense batches) of `bits`-wide elements at src, ready for
// use on `st`; nullptr when the cache does not serve this call (the caller then re-lays the operand out itself).
const void* weight_cache_get(const void* src, int64_t K, int64_t N, int bits, int64_t nb, hipStream_t st)
{
    const uint64_t bytes = (uint64_t)K * (uint64_t)N * (uint64_t)bits / 8 * (uint64_t)nb;
    bool fresh = false;
    void* copy = weight_cache_blob(src, nullptr, K, N, bits, nb, bytes, st, &fresh);
    if (!copy || !fresh) return copy;
    const int rc = bits == 4 ? opsnnTranspose4(src, copy, K, N, nb, st) : opsnnTranspose8(src, copy, K, N, nb, st);
    if (rc != 0) { weight_cache_abandon(copy); return nullptr; }
    weight_cache_commit(copy, st);
    return copy;
}

}  // namespace opsnn

using namespace opsnn;

extern "C" void opsnnSetWeightCache(int64_t max_bytes)
{
    std::lock_guard<std::mutex> lock(g_mu);
    g_limit = max_bytes > 0 ? (uint64_t)max_bytes : 0;
    while (g_used > g_limit && !g_entries.empty()) drop(std::prev(g_entries.end()));   // (pinned ones leave the table now and are freed by their holders)
}

extern "C" void opsnnWeightCacheClear(void)
{
    std::lock_guard<std::mutex> lock(g_mu);
    while (!g_entries.empty()) drop(g_entries.begin());
}

// Drops the entries made from one operand: every entry whose data, scale or offset address lies inside
// [ptr, ptr + bytes) (bytes = 0: equals ptr).  Returns how many.
extern "C" int opsnnWeightCacheInvalidate(const void* ptr, uint64_t bytes)
{
    if (!ptr) return 0;
    const uintptr_t lo = (uintptr_t)ptr, hi = lo + (bytes ? bytes : 1);
    auto inside = [&](const void* q) { return q && (uintptr_t)q >= lo && (uintptr_t)q < hi; };
    std::lock_guard<std::mutex> lock(g_mu);
    int n = 0;
    for (auto it = g_entries.begin(); it != g_entries.end();) {
        if (inside(it->src) || inside(it->src2) || inside(it->src3)) { it = drop(it); n++; }
        else ++it;
    }
    return n;
}

extern "C" void opsnnWeightCacheStats(int64_t* entries, int64_t* bytes, int64_t* hits, int64_t* misses)
{
    std::lock_guard<std::mutex> lock(g_mu);
    if (entries) *entries = (int64_t)g_entries.size();
    if (bytes) *bytes = (int64_t)g_used;
    if (hits) *hits = (int64_t)g_hits;
    if (misses) *misses = (int64_t)g_misses;
}
