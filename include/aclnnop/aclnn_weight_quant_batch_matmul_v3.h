/*
 * aclnnWeightQuantBatchMatmulV3 -- as V2 plus the innerPrecise attribute.
 *
 * Replaces matmul/weight_quant_batch_matmul_v2/op_host/op_api/aclnn_weight_quant_batch_matmul_v3.h:24-34.
 * innerPrecise must be 0 (high precision) or 1 (high performance)
 * (aclnn_weight_quant_batch_matmul_v2.cpp:283-291); both select the same fp32-accumulating kernels here.
 */
#ifndef OPSNN_AMD_ACLNN_WEIGHT_QUANT_BATCH_MATMUL_V3_H_
#define OPSNN_AMD_ACLNN_WEIGHT_QUANT_BATCH_MATMUL_V3_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnWeightQuantBatchMatmulV3GetWorkspaceSize(
    const aclTensor* x, const aclTensor* weight, const aclTensor* antiquantScale,
    const aclTensor* antiquantOffsetOptional, const aclTensor* quantScaleOptional, const aclTensor* quantOffsetOptional,
    const aclTensor* biasOptional, int antiquantGroupSize, int innerPrecise, const aclTensor* y,
    uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnWeightQuantBatchMatmulV3(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                    aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
