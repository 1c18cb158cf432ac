/*
 * aclnnDynamicBlockQuantV2 -- aclnnDynamicBlockQuant with a custom maximum of the target type (dstTypeMax).
 *
 * Generated entry point of the reference, documented in quant/dynamic_block_quant/docs/aclnnDynamicBlockQuantV2.md:51-72.  The
 * golden (quant/dynamic_block_quant/tests/assets/golden.py:95-222) does not use dstTypeMax for the FLOAT8 outputs that run here:
 * 0 is accepted, any other value is answered with ACLNN_ERR_INNER_TILING_ERROR.  Everything else as aclnnDynamicBlockQuant.
 */
#ifndef OPSNN_AMD_ACLNN_DYNAMIC_BLOCK_QUANT_V2_H_
#define OPSNN_AMD_ACLNN_DYNAMIC_BLOCK_QUANT_V2_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnDynamicBlockQuantV2GetWorkspaceSize(const aclTensor* x, double minScale, char* roundModeOptional,
                                                               int64_t dstType, int64_t rowBlockSize, int64_t colBlockSize,
                                                               double dstTypeMax, const aclTensor* yOut, const aclTensor* scaleOut,
                                                               uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnDynamicBlockQuantV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
