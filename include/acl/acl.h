/*
 * Minimal ACL runtime surface for MI355X.
 *
 * The reference operator library links against an external runtime (headers
 * "acl/acl.h" and "aclnn/aclnn_base.h", included at
 * matmul/quant_batch_matmul_v4/op_host/op_api/aclnn_quant_matmul_v5.cpp:11-30)
 * that supplies the tensor, executor, stream and memory objects every aclnn
 * entry point takes.  That runtime is not part of the reference tree, so this
 * header defines the subset the quantized-matmul callers use
 * (matmul/quant_batch_matmul_v4/examples/test_aclnn_quant_matmul_v5_perblock.cpp:52-93),
 * implemented over HIP.  Names, argument order and meaning follow the public
 * ACL API so existing caller code compiles unchanged.
 *
 * Plain C ABI: opaque handles, plain pointers and sizes.
 */
#ifndef OPSNN_AMD_ACL_H_
#define OPSNN_AMD_ACL_H_

#include <stddef.h>
#include <stdint.h>
#ifndef __cplusplus
#include <stdbool.h>
#endif

#ifdef __cplusplus
extern "C" {
#endif

#define ACL_FUNC_VISIBILITY __attribute__((visibility("default")))
#define ACLNN_API ACL_FUNC_VISIBILITY

typedef int aclError;
typedef int32_t aclnnStatus;
typedef void* aclrtStream;
typedef void* aclrtEvent;
typedef struct aclTensor aclTensor;
typedef struct aclOpExecutor aclOpExecutor;

/* Status codes (docs/zh/context/aclnn_return_code.md:8-26). */
#define ACL_SUCCESS 0
#define ACL_ERROR_INVALID_PARAM 100000
#define ACL_ERROR_UNINITIALIZE 100001
#define ACL_ERROR_REPEAT_INITIALIZE 100002
#define ACL_ERROR_BAD_ALLOC 200000
#define ACL_ERROR_RT_FAILURE 500000
#define ACLNN_SUCCESS 0
#define ACLNN_ERR_PARAM_NULLPTR 161001
#define ACLNN_ERR_PARAM_INVALID 161002
#define ACLNN_ERR_RUNTIME_ERROR 361001
#define ACLNN_ERR_INNER 561000
#define ACLNN_ERR_INNER_TILING_ERROR 561002
#define ACLNN_ERR_INNER_CREATE_EXECUTOR 561101
#define ACLNN_ERR_INNER_NULLPTR 561103

/* Element types (names: docs/zh/context/data_type.md; values evidenced in the
 * reference at matmul/quant_batch_matmul_v3/op_api/quant_matmul_v3.cpp:26-31
 * for FLOAT/FLOAT16/INT32/BF16/HIFLOAT8/FLOAT8_E4M3FN, the rest follow the
 * public ACL enumeration). */
typedef enum {
    ACL_DT_UNDEFINED = -1,
    ACL_FLOAT = 0,
    ACL_FLOAT16 = 1,
    ACL_INT8 = 2,
    ACL_INT32 = 3,
    ACL_UINT8 = 4,
    ACL_INT16 = 6,
    ACL_UINT16 = 7,
    ACL_UINT32 = 8,
    ACL_INT64 = 9,
    ACL_UINT64 = 10,
    ACL_DOUBLE = 11,
    ACL_BOOL = 12,
    ACL_STRING = 13,
    ACL_COMPLEX64 = 16,
    ACL_COMPLEX128 = 17,
    ACL_BF16 = 27,
    ACL_INT4 = 29,
    ACL_UINT1 = 30,
    ACL_COMPLEX32 = 33,
    ACL_HIFLOAT8 = 34,
    ACL_FLOAT8_E5M2 = 35,
    ACL_FLOAT8_E4M3FN = 36,
    ACL_FLOAT8_E8M0 = 37,
    ACL_FLOAT6_E3M2 = 38,
    ACL_FLOAT6_E2M3 = 39,
    ACL_FLOAT4_E2M1 = 40,
    ACL_FLOAT4_E1M2 = 41
} aclDataType;

typedef enum {
    ACL_FORMAT_UNDEFINED = -1,
    ACL_FORMAT_NCHW = 0,
    ACL_FORMAT_NHWC = 1,
    ACL_FORMAT_ND = 2,
    ACL_FORMAT_NC1HWC0 = 3,
    ACL_FORMAT_FRACTAL_Z = 4,
    ACL_FORMAT_NC1HWC0_C04 = 12,
    ACL_FORMAT_HWCN = 16,
    ACL_FORMAT_NDHWC = 27,
    ACL_FORMAT_FRACTAL_NZ = 29,
    ACL_FORMAT_NCDHW = 30,
    ACL_FORMAT_NDC1HWC0 = 32,
    ACL_FRACTAL_Z_3D = 33,
    ACL_FORMAT_NC = 35,
    ACL_FORMAT_NCL = 47,
    ACL_FORMAT_FRACTAL_NZ_C0_16 = 50,
    ACL_FORMAT_FRACTAL_NZ_C0_32 = 51
} aclFormat;

typedef enum {
    ACL_MEM_MALLOC_HUGE_FIRST = 0,
    ACL_MEM_MALLOC_HUGE_ONLY = 1,
    ACL_MEM_MALLOC_NORMAL_ONLY = 2
} aclrtMemMallocPolicy;

typedef enum {
    ACL_MEMCPY_HOST_TO_HOST = 0,
    ACL_MEMCPY_HOST_TO_DEVICE = 1,
    ACL_MEMCPY_DEVICE_TO_HOST = 2,
    ACL_MEMCPY_DEVICE_TO_DEVICE = 3
} aclrtMemcpyKind;

/* ---- process / device ---------------------------------------------------- */
ACL_FUNC_VISIBILITY aclError aclInit(const char* configPath);
ACL_FUNC_VISIBILITY aclError aclFinalize(void);
ACL_FUNC_VISIBILITY aclError aclrtSetDevice(int32_t deviceId);
ACL_FUNC_VISIBILITY aclError aclrtResetDevice(int32_t deviceId);
ACL_FUNC_VISIBILITY aclError aclrtGetDeviceCount(uint32_t* count);
ACL_FUNC_VISIBILITY aclError aclrtSynchronizeDevice(void);
/* Thread-local text of the most recent failure on the calling thread
 * (docs/zh/context/aclnn_return_code.md:3-4). Never NULL. */
ACL_FUNC_VISIBILITY const char* aclGetRecentErrMsg(void);

/* ---- streams and events -------------------------------------------------- */
ACL_FUNC_VISIBILITY aclError aclrtCreateStream(aclrtStream* stream);
ACL_FUNC_VISIBILITY aclError aclrtDestroyStream(aclrtStream stream);
ACL_FUNC_VISIBILITY aclError aclrtSynchronizeStream(aclrtStream stream);
ACL_FUNC_VISIBILITY aclError aclrtCreateEvent(aclrtEvent* event);
ACL_FUNC_VISIBILITY aclError aclrtDestroyEvent(aclrtEvent event);
ACL_FUNC_VISIBILITY aclError aclrtRecordEvent(aclrtEvent event, aclrtStream stream);
ACL_FUNC_VISIBILITY aclError aclrtSynchronizeEvent(aclrtEvent event);
ACL_FUNC_VISIBILITY aclError aclrtEventElapsedTime(float* ms, aclrtEvent start, aclrtEvent end);

/* ---- memory -------------------------------------------------------------- */
ACL_FUNC_VISIBILITY aclError aclrtMalloc(void** devPtr, size_t size, aclrtMemMallocPolicy policy);
ACL_FUNC_VISIBILITY aclError aclrtFree(void* devPtr);
ACL_FUNC_VISIBILITY aclError aclrtMallocHost(void** hostPtr, size_t size);
ACL_FUNC_VISIBILITY aclError aclrtFreeHost(void* hostPtr);
ACL_FUNC_VISIBILITY aclError aclrtMemcpy(void* dst, size_t destMax, const void* src, size_t count,
                                         aclrtMemcpyKind kind);
ACL_FUNC_VISIBILITY aclError aclrtMemcpyAsync(void* dst, size_t destMax, const void* src, size_t count,
                                              aclrtMemcpyKind kind, aclrtStream stream);
ACL_FUNC_VISIBILITY aclError aclrtMemset(void* devPtr, size_t maxCount, int32_t value, size_t count);

/* ---- tensors ------------------------------------------------------------- */
/* viewDims/stride/offset are counted in ELEMENTS, also for 4-bit types
 * (docs/zh/context/non_contiguous_tensor.md:3-24).  stride may be NULL, which
 * means contiguous; tensorData may be NULL for shape-only use (the reference's
 * own API tests build such tensors, matmul/quant_batch_matmul_v4/tests/ut/
 * op_host/test_aclnn_quant_matmul_v5_api.cpp:187-270). */
ACL_FUNC_VISIBILITY aclTensor* aclCreateTensor(const int64_t* viewDims, uint64_t viewDimsNum, aclDataType dataType,
                                               const int64_t* stride, int64_t offset, aclFormat format,
                                               const int64_t* storageDims, uint64_t storageDimsNum,
                                               void* tensorData);
ACL_FUNC_VISIBILITY aclnnStatus aclDestroyTensor(const aclTensor* tensor);
ACL_FUNC_VISIBILITY aclnnStatus aclGetViewShape(const aclTensor* tensor, int64_t** viewDims, uint64_t* viewDimsNum);
ACL_FUNC_VISIBILITY aclnnStatus aclGetDataType(const aclTensor* tensor, aclDataType* dataType);
ACL_FUNC_VISIBILITY aclnnStatus aclGetFormat(const aclTensor* tensor, aclFormat* format);
ACL_FUNC_VISIBILITY aclnnStatus aclDestroyAclOpExecutor(aclOpExecutor* executor);

#ifdef __cplusplus
}
#endif
#endif /* OPSNN_AMD_ACL_H_ */
