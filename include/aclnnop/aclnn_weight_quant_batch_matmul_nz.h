/*
 * aclnnWeightQuantBatchMatmulNz: aclnnWeightQuantBatchMatmulV2 with the weight in FRACTAL_NZ format.
 *
 * Replaces matmul/weight_quant_batch_matmul_v2/op_host/op_api/aclnn_weight_quant_batch_matmul_nz.h:38-54 (same two
 * entry points, same arguments).  The weight's view is the logical [k, n] matrix (INT8 also as the transposed view of an
 * [n, k] matrix); its storage is the 4-D fractal array [ceil(cols / c0), ceil(rows / 16), 16, c0] of the stored matrix,
 * c0 = 32 elements for INT8, 16 or 32 for INT4 / FLOAT4_E2M1, 2 or 4 for the INT32 / FLOAT carriers of eight 4-bit
 * values (aclnnWeightQuantBatchMatmulNz.md:326-338) -- what aclnnConvertWeightToINT4Pack writes when its output
 * tensor is FRACTAL_NZ.  On this device the fractal form buys nothing: phase 2 lays the weight out as the dense matrix
 * once (workspace) and runs the V2 kernels; callers that can should keep the weight in ND, K-contiguous.
 */
#ifndef OPSNN_ACLNN_WEIGHT_QUANT_BATCH_MATMUL_NZ_H_
#define OPSNN_ACLNN_WEIGHT_QUANT_BATCH_MATMUL_NZ_H_
#include "acl/acl.h"
#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnWeightQuantBatchMatmulNzGetWorkspaceSize(
    const aclTensor* x, const aclTensor* weight, const aclTensor* antiquantScale,
    const aclTensor* antiquantOffsetOptional, const aclTensor* quantScaleOptional, const aclTensor* quantOffsetOptional,
    const aclTensor* biasOptional, int antiquantGroupSize, const aclTensor* y, uint64_t* workspaceSize,
    aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnWeightQuantBatchMatmulNz(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                    aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
