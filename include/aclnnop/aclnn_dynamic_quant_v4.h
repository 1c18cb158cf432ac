/*
 * aclnnDynamicQuantV4 -- aclnnDynamicQuantV2 with the symmetry flag and the quantisation mode as attributes and a custom
 * maximum of the target type.
 *
 * Replaces quant/dynamic_quant/op_host/op_api/aclnn_dynamic_quant_v4.h; attribute and shape rules of
 * aclnn_dynamic_quant.cpp:171-189, 191-291.  isSymmetrical must agree with offsetOut (null when true).  quantMode "pertoken",
 * "pertensor" (scaleOut [1]) and "perchannel" (scaleOut = x's shape without the second-to-last dim; smoothScales one factor per
 * row of that dim) run here; a dstTypeMax other than 0 is answered with ACLNN_ERR_INNER_TILING_ERROR.
 */
#ifndef OPSNN_AMD_ACLNN_DYNAMIC_QUANT_V4_H_
#define OPSNN_AMD_ACLNN_DYNAMIC_QUANT_V4_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnDynamicQuantV4GetWorkspaceSize(const aclTensor* x, const aclTensor* smoothScalesOptional,
                                                          const aclTensor* groupIndexOptional, int64_t dstType, bool isSymmetrical,
                                                          const char* quantMode, float dstTypeMax, const aclTensor* yOut, const aclTensor* scaleOut,
                                                          const aclTensor* offsetOut, uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnDynamicQuantV4(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
