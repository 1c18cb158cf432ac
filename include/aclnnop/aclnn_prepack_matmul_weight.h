/*
 * aclnnPrepackMatmulWeight: one-time re-layout of a quantized right operand into the form the gfx950 kernels stream.
 *
 * It has no single counterpart in the reference; it stands where the reference prepares a weight offline for its cube
 * unit -- aclnnTransMatmulWeight / aclnnNpuFormatCast (ND -> FRACTAL_NZ; matmul/quant_batch_matmul_v3/docs/
 * aclnnQuantMatmulWeightNz.md:548, matmul/weight_quant_batch_matmul_v2/docs/aclnnWeightQuantBatchMatmulNz.md:328-333),
 * aclnnConvertWeightToINT4Pack (matmul/convert_weight_to_int4_pack/op_host/op_api/aclnn_convert_weight_to_int4_pack.h:24-31,
 * the model for this two-phase signature) and the graph passes that fold a caller's transpose into the operator
 * (matmul/quant_batch_matmul_v4/op_graph/fusion_pass/quant_batch_matmul_v4_transpose_fusion_pass.cpp,
 *  matmul/weight_quant_batch_matmul_v2/op_graph/fusion_pass/weight_quant_batch_matmul_v2_transpose_fusion_pass.cpp).
 *
 * The matrix-core kernels read both operands with K contiguous.  A right operand stored [k, n] (the literal layout of the
 * operators' x2 / weight) is re-laid out inside EVERY matmul call; this operator does it ONCE:
 *
 *   weight            [.., k, n], dense ND, or FRACTAL_NZ (storage [.., ceil(n/c0), ceil(k/16), 16, c0]);
 *                     INT8, FLOAT8_E4M3FN, FLOAT8_E5M2, INT4, FLOAT4_E2M1 (4-bit: k and n even)
 *   scaleOptional     NULL, or a scale that runs along k and must follow the weight:
 *                     FLOAT8_E8M0 [.., ceil(k/64), n, 2] (MX), or FLOAT16 / BF16 [ceil(k/group), n] (per group)
 *   weightPacked      [.., n, k], dense ND, same dtype: weightPacked[n][k] = weight[k][n]
 *   scalePackedOptional  [.., n, ceil(k/64), 2] resp. [n, ceil(k/group)], same dtype as scaleOptional
 *
 * Afterwards pass weightPacked to aclnnQuantMatmulV5 with transposeX2 = true (MX: x2Scale = scalePacked), or to
 * aclnnWeightQuantBatchMatmulV2/V3 as the transposed view (shape [k, n], strides (1, k); antiquantScale likewise a
 * transposed view of scalePacked): those calls then need no workspace and no re-layout.
 * Status codes as everywhere: 161001 null pointer, 161002 invalid argument.
 */
#ifndef OPSNN_ACLNN_PREPACK_MATMUL_WEIGHT_H_
#define OPSNN_ACLNN_PREPACK_MATMUL_WEIGHT_H_
#include "acl/acl.h"
#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnPrepackMatmulWeightGetWorkspaceSize(const aclTensor* weight, const aclTensor* scaleOptional,
                                                               aclTensor* weightPacked, aclTensor* scalePackedOptional,
                                                               uint64_t* workspaceSize, aclOpExecutor** executor);
ACLNN_API aclnnStatus aclnnPrepackMatmulWeight(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                               aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
