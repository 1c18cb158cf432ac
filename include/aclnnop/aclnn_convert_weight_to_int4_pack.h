/*
 * aclnnConvertWeightToINT4Pack -- packs a weight given as one 4-bit value per 32-bit element (INT32: the value's low
 * four bits; FLOAT: the fp4 e2m1 code of the value) into two values per byte, the form aclnnWeightQuantBatchMatmulV2/V3
 * and aclnnQuantMatmulV5 take as INT4 / FLOAT4_E2M1 tensors or as INT32 / FLOAT carriers with a last dim of N / 8.
 *
 * Replaces matmul/convert_weight_to_int4_pack/op_host/op_api/aclnn_convert_weight_to_int4_pack.h:24-31.
 * As in the reference (aclnn_convert_weight_to_int4_pack.cpp:368-412) the conversion is complete when the first call
 * returns, workspaceSize and executor are not needed by the second call, and the second call does nothing.  Here the
 * first call runs one device kernel and waits for it instead of copying the weight to the host and back.
 * weight: INT32 or FLOAT, ND, contiguous, 2 or 3 dims.  weightInt4Pack: INT4 / FLOAT4_E2M1 with weight's shape (last dim
 * even), or INT32 / FLOAT with the last dim divided by 8; ND only -- a FRACTAL_NZ output is answered with
 * ACLNN_ERR_PARAM_INVALID, as the matmul entry points here do not take that layout.
 */
#ifndef OPSNN_AMD_ACLNN_CONVERT_WEIGHT_TO_INT4_PACK_H_
#define OPSNN_AMD_ACLNN_CONVERT_WEIGHT_TO_INT4_PACK_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnConvertWeightToINT4PackGetWorkspaceSize(const aclTensor* weight, aclTensor* weightInt4Pack,
                                                                   uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnConvertWeightToINT4Pack(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                   aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
