/*
 * aclnnWeightQuantBatchMatmulV2 -- weight-only quantized matmul
 * (fp16/bf16 activations, int8/int4/fp8/mxfp4 weights), two-phase C entry points.
 *
 * Replaces, with the same names, argument order and meaning:
 *   matmul/weight_quant_batch_matmul_v2/op_host/op_api/aclnn_weight_quant_batch_matmul_v2.h:38-54
 * (implementation in the reference: aclnn_weight_quant_batch_matmul_v2.cpp:1719-1767, 1870-1875).
 *
 * y = x @ ((weight + antiquantOffset) * antiquantScale) + bias, where the two
 * dequantisation steps are each rounded to x's dtype before the fp32-accumulated
 * contraction.
 */
#ifndef OPSNN_AMD_ACLNN_WEIGHT_QUANT_BATCH_MATMUL_V2_H_
#define OPSNN_AMD_ACLNN_WEIGHT_QUANT_BATCH_MATMUL_V2_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 *  x                        fp16 / bf16 [m, k], contiguous
 *  weight                   int8 / int4 / fp8 e4m3fn / fp4 e2m1 [k, n]; int32 and fp32 tensors carry eight
 *                           4-bit values per element; a view with strides (1, k) means the storage is [n, k]
 *  antiquantScale           x's dtype: [1], [n], [1, n] or per-group [ceil(k/g), n]; or e8m0 [ceil(k/32), n]
 *  antiquantOffsetOptional  same dtype and shape as the scale, or NULL
 *  quantScaleOptional, quantOffsetOptional   must be NULL
 *  biasOptional             [n] or [1, n]
 *  antiquantGroupSize       0, or a multiple of 32 in [32, k-1]
 *  y                        [m, n], x's dtype
 */
ACLNN_API aclnnStatus aclnnWeightQuantBatchMatmulV2GetWorkspaceSize(
    const aclTensor* x, const aclTensor* weight, const aclTensor* antiquantScale,
    const aclTensor* antiquantOffsetOptional, const aclTensor* quantScaleOptional, const aclTensor* quantOffsetOptional,
    const aclTensor* biasOptional, int antiquantGroupSize, const aclTensor* y, uint64_t* workspaceSize,
    aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnWeightQuantBatchMatmulV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                    aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
