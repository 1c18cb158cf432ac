/*
 * aclnnDynamicQuant -- symmetric per-token dynamic quantisation of an activation: per row of x (all dims but the last
 * flattened) scaleOut = max|x * smoothScales| / typeMax and yOut = round(x * smoothScales / scaleOut).
 *
 * Replaces quant/dynamic_quant/op_host/op_api/aclnn_dynamic_quant.h:23-32; checks in the order of
 * aclnn_dynamic_quant.cpp:320-328 (null, attributes, dtypes, shapes); arithmetic of
 * quant/dynamic_quant/tests/assets/golden.py:17-122.
 * x: FLOAT16 / BF16, 2 to 8 dims.  smoothScalesOptional: x's dtype, [x.shape[-1]].  yOut: INT8, INT4 (last dim even),
 * INT32 (eight INT4 per element, last dim / 8), FLOAT8_E4M3FN or FLOAT8_E5M2, x's shape.  scaleOut: FLOAT, x's shape
 * without the last dim.  Tensors must be contiguous here (the reference copies strided ones); HIFLOAT8 is answered
 * with ACLNN_ERR_INNER_TILING_ERROR.
 */
#ifndef OPSNN_AMD_ACLNN_DYNAMIC_QUANT_H_
#define OPSNN_AMD_ACLNN_DYNAMIC_QUANT_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnDynamicQuantGetWorkspaceSize(const aclTensor* x, const aclTensor* smoothScalesOptional,
                                                        const aclTensor* yOut, const aclTensor* scaleOut,
                                                        uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnDynamicQuant(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
