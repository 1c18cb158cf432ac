/*
 * aclnnDynamicQuantV3 -- aclnnDynamicQuantV2 with the symmetry flag and the quantisation mode as attributes.
 *
 * Replaces quant/dynamic_quant/op_host/op_api/aclnn_dynamic_quant_v3.h; attribute and shape rules of
 * aclnn_dynamic_quant.cpp:171-189, 191-291.  isSymmetrical must agree with offsetOut (null when true).  quantMode "pertoken",
 * "pertensor" (scaleOut [1]) and "perchannel" (scaleOut = x's shape without the second-to-last dim; smoothScales one factor per
 * row of that dim) run here.
 */
#ifndef OPSNN_AMD_ACLNN_DYNAMIC_QUANT_V3_H_
#define OPSNN_AMD_ACLNN_DYNAMIC_QUANT_V3_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnDynamicQuantV3GetWorkspaceSize(const aclTensor* x, const aclTensor* smoothScalesOptional,
                                                          const aclTensor* groupIndexOptional, int64_t dstType, bool isSymmetrical,
                                                          const char* quantMode, const aclTensor* yOut, const aclTensor* scaleOut,
                                                          const aclTensor* offsetOut, uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnDynamicQuantV3(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
