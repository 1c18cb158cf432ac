/*
 * aclnnDynamicMxQuantV3 -- aclnnDynamicMxQuant with dstTypeMax and a lower clamp of the block maximum (maxLowBound).
 *
 * Generated entry point of the reference, documented in quant/dynamic_mx_quant/docs/aclnnDynamicMxQuantV3.md.  Run here with the
 * added arguments at 0 (the first version's arithmetic) and scaleAlg 0 or 1; other values are answered with
 * ACLNN_ERR_INNER_TILING_ERROR.  Everything else as aclnnDynamicMxQuant.
 */
#ifndef OPSNN_AMD_ACLNN_DYNAMIC_MX_QUANT_V3_H_
#define OPSNN_AMD_ACLNN_DYNAMIC_MX_QUANT_V3_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnDynamicMxQuantV3GetWorkspaceSize(const aclTensor* x, int64_t axis, char* roundModeOptional, int64_t dstType,
                                                            int64_t blocksize, int64_t scaleAlg, double dstTypeMax, double maxLowBound, const aclTensor* yOut,
                                                            const aclTensor* mxscaleOut, uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnDynamicMxQuantV3(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
