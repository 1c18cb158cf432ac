/*
 * aclnnDynamicQuantV2 -- aclnnDynamicQuant plus the asymmetric form: with offsetOut (FLOAT, scaleOut's shape)
 * scaleOut = (max - min) / (2 * typeMax + 1), offsetOut = typeMax - max / scaleOut, yOut = round(x / scaleOut + offsetOut);
 * without it the symmetric form.
 *
 * Replaces quant/dynamic_quant_v2/op_host/op_api/aclnn_dynamic_quant_v2.h:23-33 (implementation:
 * quant/dynamic_quant/op_host/op_api/aclnn_dynamic_quant.cpp:478-490).  dstType is carried as in the reference, which
 * takes the output type from yOut.  groupIndexOptional [experts] (INT32 / INT64, the row where each expert's rows end) selects the
 * row of smoothScalesOptional [experts, x.shape[-1]] that a row of x is multiplied with; rows past the last end are left untouched.
 */
#ifndef OPSNN_AMD_ACLNN_DYNAMIC_QUANT_V2_H_
#define OPSNN_AMD_ACLNN_DYNAMIC_QUANT_V2_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnDynamicQuantV2GetWorkspaceSize(const aclTensor* x, const aclTensor* smoothScalesOptional,
                                                          const aclTensor* groupIndexOptional, int64_t dstType,
                                                          const aclTensor* yOut, const aclTensor* scaleOut,
                                                          const aclTensor* offsetOut, uint64_t* workspaceSize,
                                                          aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnDynamicQuantV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
