// opsnnQmmInt8Static: opsnnQmmInt8 for callers that cannot allocate device memory (code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc).  opsnnQmmInt8 needs a workspace of N*K bytes when x2 is stored [K, N]
// with N contiguous (the operand is re-laid out K-contiguous before the matrix-core kernel); here that workspace is a
// fixed array in the library's own device image instead of a buffer the caller allocates.
#include <mutex>

#include "common.hip.h"
#include "launch.h"

namespace opsnn {
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));   // host/acl_min.cpp: text behind aclGetRecentErrMsg
}

// The re-laid-out right operand.  Every device that loads the library holds its own copy of this array until the
// process ends.  In host code the name is only a handle for hipGetSymbolAddress, never a device address.
static __device__ __align__(256) unsigned char scratch[OPSNN_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];   // device address of `scratch` on each device, looked up once per device
std::mutex g_scratch_mutex;

// Device address of this device's copy of `scratch` (the device must be current).
int scratch_address(void** out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return -1;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!ptr) return (int)hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}
}  // namespace

extern "C" __attribute__((visibility("hidden"))) uint64_t opsnn_qmm_workspace_base(const OpsnnQmmArgs* a, int mode);   // dispatch.hip
extern "C" __attribute__((visibility("hidden"))) int opsnn_qmm_int8_nosplit(const OpsnnQmmArgs* a, void* stream);       // qmm_int8.hip

extern "C" int opsnnQmmInt8Static(const OpsnnQmmArgs* a, void* stream)
{
    if (!a) return -1;
    // (the workspace of opsnnQmmInt8 without the partial sums of a K split: this entry point runs every call unsplit)
    const uint64_t need = opsnn_qmm_workspace_base(a, 0);
    if (need > (uint64_t)OPSNN_STATIC_SCRATCH_BYTES) {
        opsnn::set_error("opsnnQmmInt8Static: the re-laid-out x2 needs %llu bytes, the built-in scratch array holds %llu; "
                         "pass x2 K-contiguous or use opsnnQmmInt8 with a workspace",
                         (unsigned long long)need, (unsigned long long)OPSNN_STATIC_SCRATCH_BYTES);
        return OPSNN_ERR_SCRATCH_TOO_SMALL;
    }
    opsnn::WeightCacheScope no_cache(true);   // a miss in the weight cache allocates, an eviction frees: not from this entry point
    OpsnnQmmArgs b = *a;
    b.workspace = nullptr;
    if (need) {
        void* ptr = nullptr;
        const int rc = scratch_address(&ptr);
        if (rc != 0) {
            opsnn::set_error("opsnnQmmInt8Static: hipGetSymbolAddress of the scratch array failed (%d)", rc);
            return rc;
        }
        b.workspace = ptr;   // written in full by the re-layout before the matmul reads it: nothing to clear
    }
    return opsnn_qmm_int8_nosplit(&b, stream);
}
