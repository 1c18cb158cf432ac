/*
 * aclnnDynamicBlockQuant -- quantises x in blocks of rowBlockSize x colBlockSize elements: per block
 * scaleOut = min(max|x| / typeMax, 1 / minScale) and yOut = cast(x / scaleOut).
 *
 * The reference generates this entry point from the operator definition (quant/dynamic_block_quant/op_host/
 * dynamic_block_quant_def.cpp); its signature and rules are the documented ones,
 * quant/dynamic_block_quant/docs/aclnnDynamicBlockQuant.md:51-70, 95-220, with the attribute checks of
 * op_host/dynamic_block_quant_tiling.cpp:135-230, 300-340; arithmetic of quant/dynamic_block_quant/tests/assets/golden.py:95-222.
 * x: FLOAT16 / BF16, 2 or 3 dims.  yOut: FLOAT8_E4M3FN or FLOAT8_E5M2 (dstType 36 / 35 and equal to yOut's dtype), x's
 * shape.  scaleOut: FLOAT, [.., ceil(M / rowBlockSize), ceil(N / colBlockSize)].  rowBlockSize 1, 64, 128, 256 or 512;
 * colBlockSize 64, 128, 192 or 256; roundModeOptional NULL or "rint"; minScale >= 0.  INT8 and HIFLOAT8 outputs (whose
 * arithmetic the golden does not define / whose format definition is absent) are answered with
 * ACLNN_ERR_INNER_TILING_ERROR; tensors must be contiguous here.
 */
#ifndef OPSNN_AMD_ACLNN_DYNAMIC_BLOCK_QUANT_H_
#define OPSNN_AMD_ACLNN_DYNAMIC_BLOCK_QUANT_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnDynamicBlockQuantGetWorkspaceSize(const aclTensor* x, double minScale, char* roundModeOptional,
                                                             int64_t dstType, int64_t rowBlockSize, int64_t colBlockSize,
                                                             const aclTensor* yOut, const aclTensor* scaleOut,
                                                             uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnDynamicBlockQuant(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
