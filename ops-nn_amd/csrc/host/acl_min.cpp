// Minimal ACL runtime over HIP: tensors, streams, events, memory.  See include/acl/acl.h.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include <mutex>
#include <unordered_set>

#include "tensor.h"

namespace opsnn {

namespace {
std::mutex g_exec_mutex;
std::unordered_set<const void*> g_live_executors;
}
void* executor_publish(void* ex)
{
    std::lock_guard<std::mutex> lock(g_exec_mutex);
    g_live_executors.insert(ex);
    return ex;
}
bool executor_claim(const void* ex)
{
    std::lock_guard<std::mutex> lock(g_exec_mutex);
    return g_live_executors.erase(ex) != 0;
}

static thread_local char g_err[1024] = "";

void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    if (log_enabled()) fprintf(stderr, "[opsnn] %s\n", g_err);
}
void clear_error() { g_err[0] = 0; }
bool log_enabled()
{
    static const bool on = [] { const char* e = getenv("OPSNN_LOG"); return e && *e && *e != '0'; }();
    return on;
}

const char* dtype_name(aclDataType d)
{
    switch (d) {
        case ACL_FLOAT: return "FLOAT";
        case ACL_FLOAT16: return "FLOAT16";
        case ACL_INT8: return "INT8";
        case ACL_INT32: return "INT32";
        case ACL_UINT8: return "UINT8";
        case ACL_INT64: return "INT64";
        case ACL_UINT64: return "UINT64";
        case ACL_BF16: return "BF16";
        case ACL_INT4: return "INT4";
        case ACL_HIFLOAT8: return "HIFLOAT8";
        case ACL_FLOAT8_E5M2: return "FLOAT8_E5M2";
        case ACL_FLOAT8_E4M3FN: return "FLOAT8_E4M3FN";
        case ACL_FLOAT8_E8M0: return "FLOAT8_E8M0";
        case ACL_FLOAT4_E2M1: return "FLOAT4_E2M1";
        case ACL_FLOAT4_E1M2: return "FLOAT4_E1M2";
        default: return "OTHER";
    }
}

std::string shape_str(const std::vector<int64_t>& s)
{
    std::string r = "[";
    for (size_t i = 0; i < s.size(); i++) { if (i) r += ","; r += std::to_string(s[i]); }
    return r + "]";
}

TView make_view(const aclTensor* t)
{
    TView v;
    if (!t) return v;
    v.present = true;
    v.shape = t->view; v.strides = t->strides; v.offset = t->offset; v.dtype = t->dtype;
    v.format = t->format; v.storage = t->storage; v.data = t->data;
    return v;
}

bool is_contiguous(const TView& v)
{
    int64_t expect = 1;
    for (int64_t i = v.rank() - 1; i >= 0; i--) {
        if (v.shape[(size_t)i] != 1 && v.strides[(size_t)i] != expect) return false;
        expect *= v.shape[(size_t)i];
    }
    return true;
}

// matmul/common/op_host/op_api/matmul_util.cpp:2040-2064
bool is_transposed_last2(const TView& v)
{
    int64_t r = v.rank();
    if (r < 2 || r > 6) return false;
    int64_t d1 = v.dim(-1), d2 = v.dim(-2);
    if (v.stride(-2) != 1 || v.stride(-1) != d2) return false;
    int64_t expect = d1 * d2;
    for (int64_t i = r - 3; i >= 0; i--) {
        if (v.strides[(size_t)i] != expect) return false;
        expect *= v.shape[(size_t)i];
    }
    if (d1 == 1 && d2 == 1) return false;
    return true;
}

void swap_last2(TView& v)
{
    size_t r = v.shape.size();
    std::swap(v.shape[r - 1], v.shape[r - 2]);
    std::swap(v.strides[r - 1], v.strides[r - 2]);
}

static aclError hip_rc(hipError_t e, const char* what)
{
    if (e == hipSuccess) return ACL_SUCCESS;
    set_error("%s failed: %s", what, hipGetErrorString(e));
    return ACL_ERROR_RT_FAILURE;
}

}  // namespace opsnn

using namespace opsnn;

extern "C" {

aclError aclInit(const char*) { clear_error(); return ACL_SUCCESS; }
aclError aclFinalize(void) { return ACL_SUCCESS; }
aclError aclrtSetDevice(int32_t deviceId) { return hip_rc(hipSetDevice(deviceId), "hipSetDevice"); }
aclError aclrtResetDevice(int32_t) { return hip_rc(hipDeviceSynchronize(), "hipDeviceSynchronize"); }
aclError aclrtGetDeviceCount(uint32_t* count)
{
    if (!count) return ACL_ERROR_INVALID_PARAM;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    *count = e == hipSuccess ? (uint32_t)n : 0u;
    return e == hipSuccess ? ACL_SUCCESS : ACL_ERROR_RT_FAILURE;
}
aclError aclrtSynchronizeDevice(void) { return hip_rc(hipDeviceSynchronize(), "hipDeviceSynchronize"); }
const char* aclGetRecentErrMsg(void) { return g_err; }

aclError aclrtCreateStream(aclrtStream* stream)
{
    if (!stream) return ACL_ERROR_INVALID_PARAM;
    hipStream_t s = nullptr;
    aclError rc = hip_rc(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreate");
    *stream = (aclrtStream)s;
    return rc;
}
aclError aclrtDestroyStream(aclrtStream stream) { return hip_rc(hipStreamDestroy((hipStream_t)stream), "hipStreamDestroy"); }
aclError aclrtSynchronizeStream(aclrtStream stream)
{
    return hip_rc(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
}
aclError aclrtCreateEvent(aclrtEvent* event)
{
    if (!event) return ACL_ERROR_INVALID_PARAM;
    hipEvent_t e = nullptr;
    aclError rc = hip_rc(hipEventCreate(&e), "hipEventCreate");
    *event = (aclrtEvent)e;
    return rc;
}
aclError aclrtDestroyEvent(aclrtEvent event) { return hip_rc(hipEventDestroy((hipEvent_t)event), "hipEventDestroy"); }
aclError aclrtRecordEvent(aclrtEvent event, aclrtStream stream)
{
    return hip_rc(hipEventRecord((hipEvent_t)event, (hipStream_t)stream), "hipEventRecord");
}
aclError aclrtSynchronizeEvent(aclrtEvent event) { return hip_rc(hipEventSynchronize((hipEvent_t)event), "hipEventSynchronize"); }
aclError aclrtEventElapsedTime(float* ms, aclrtEvent start, aclrtEvent end)
{
    if (!ms) return ACL_ERROR_INVALID_PARAM;
    return hip_rc(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)end), "hipEventElapsedTime");
}

aclError aclrtMalloc(void** devPtr, size_t size, aclrtMemMallocPolicy)
{
    if (!devPtr) return ACL_ERROR_INVALID_PARAM;
    *devPtr = nullptr;
    if (size == 0) return ACL_ERROR_INVALID_PARAM;
    hipError_t e = hipMalloc(devPtr, size);
    if (e != hipSuccess) { set_error("hipMalloc(%zu) failed: %s", size, hipGetErrorString(e)); return ACL_ERROR_BAD_ALLOC; }
    return ACL_SUCCESS;
}
aclError aclrtFree(void* devPtr) { return devPtr ? hip_rc(hipFree(devPtr), "hipFree") : ACL_SUCCESS; }
aclError aclrtMallocHost(void** hostPtr, size_t size)
{
    if (!hostPtr || size == 0) return ACL_ERROR_INVALID_PARAM;
    return hip_rc(hipHostMalloc(hostPtr, size, hipHostMallocDefault), "hipHostMalloc");
}
aclError aclrtFreeHost(void* hostPtr) { return hostPtr ? hip_rc(hipHostFree(hostPtr), "hipHostFree") : ACL_SUCCESS; }

static hipMemcpyKind to_kind(aclrtMemcpyKind k)
{
    switch (k) {
        case ACL_MEMCPY_HOST_TO_HOST: return hipMemcpyHostToHost;
        case ACL_MEMCPY_HOST_TO_DEVICE: return hipMemcpyHostToDevice;
        case ACL_MEMCPY_DEVICE_TO_HOST: return hipMemcpyDeviceToHost;
        default: return hipMemcpyDeviceToDevice;
    }
}
aclError aclrtMemcpy(void* dst, size_t destMax, const void* src, size_t count, aclrtMemcpyKind kind)
{
    if (!dst || !src || count > destMax) { set_error("aclrtMemcpy: bad arguments"); return ACL_ERROR_INVALID_PARAM; }
    if (count == 0) return ACL_SUCCESS;
    return hip_rc(hipMemcpy(dst, src, count, to_kind(kind)), "hipMemcpy");
}
aclError aclrtMemcpyAsync(void* dst, size_t destMax, const void* src, size_t count, aclrtMemcpyKind kind,
                          aclrtStream stream)
{
    if (!dst || !src || count > destMax) { set_error("aclrtMemcpyAsync: bad arguments"); return ACL_ERROR_INVALID_PARAM; }
    if (count == 0) return ACL_SUCCESS;
    return hip_rc(hipMemcpyAsync(dst, src, count, to_kind(kind), (hipStream_t)stream), "hipMemcpyAsync");
}
aclError aclrtMemset(void* devPtr, size_t maxCount, int32_t value, size_t count)
{
    if (!devPtr || count > maxCount) return ACL_ERROR_INVALID_PARAM;
    if (count == 0) return ACL_SUCCESS;
    return hip_rc(hipMemset(devPtr, value, count), "hipMemset");
}

aclTensor* aclCreateTensor(const int64_t* viewDims, uint64_t viewDimsNum, aclDataType dataType, const int64_t* stride,
                           int64_t offset, aclFormat format, const int64_t* storageDims, uint64_t storageDimsNum,
                           void* tensorData)
{
    if (viewDimsNum > 0 && !viewDims) { set_error("aclCreateTensor: viewDims is null"); return nullptr; }
    if (viewDimsNum > 8 || storageDimsNum > 8) { set_error("aclCreateTensor: more than 8 dims"); return nullptr; }
    aclTensor* t = new (std::nothrow) aclTensor();
    if (!t) return nullptr;
    t->view.assign(viewDims, viewDims + viewDimsNum);
    if (stride) {
        t->strides.assign(stride, stride + viewDimsNum);
    } else {
        t->strides.assign(viewDimsNum, 1);
        for (int64_t i = (int64_t)viewDimsNum - 2; i >= 0; i--) t->strides[(size_t)i] = t->strides[(size_t)i + 1] * t->view[(size_t)i + 1];
    }
    t->offset = offset;
    t->dtype = dataType;
    t->format = format;
    if (storageDims && storageDimsNum > 0) t->storage.assign(storageDims, storageDims + storageDimsNum);
    else t->storage = t->view;
    t->data = tensorData;
    return t;
}
aclnnStatus aclDestroyTensor(const aclTensor* tensor) { delete tensor; return ACLNN_SUCCESS; }
aclnnStatus aclGetViewShape(const aclTensor* tensor, int64_t** viewDims, uint64_t* viewDimsNum)
{
    if (!tensor || !viewDims || !viewDimsNum) return ACLNN_ERR_PARAM_NULLPTR;
    *viewDimsNum = tensor->view.size();
    *viewDims = new int64_t[tensor->view.size() ? tensor->view.size() : 1];
    for (size_t i = 0; i < tensor->view.size(); i++) (*viewDims)[i] = tensor->view[i];
    return ACLNN_SUCCESS;
}
aclnnStatus aclGetDataType(const aclTensor* tensor, aclDataType* dataType)
{
    if (!tensor || !dataType) return ACLNN_ERR_PARAM_NULLPTR;
    *dataType = tensor->dtype;
    return ACLNN_SUCCESS;
}
aclnnStatus aclGetFormat(const aclTensor* tensor, aclFormat* format)
{
    if (!tensor || !format) return ACLNN_ERR_PARAM_NULLPTR;
    *format = tensor->format;
    return ACLNN_SUCCESS;
}
aclnnStatus aclDestroyAclOpExecutor(aclOpExecutor* executor)
{
    if (executor && opsnn::executor_claim(executor)) delete executor;   // unknown, already run or already destroyed: nothing to do
    return ACLNN_SUCCESS;
}

}  // extern "C"
