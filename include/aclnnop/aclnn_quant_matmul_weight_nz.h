/*
 * aclnnQuantMatmulWeightNz: aclnnQuantMatmulV5 with x2 in FRACTAL_NZ format.
 *
 * Replaces matmul/quant_batch_matmul_v3/op_api/aclnn_quant_matmul_weight_nz.h:41-71 (same two entry points, same
 * arguments as aclnnQuantMatmulV5).  x2's view is the logical [.., k, n] matrix ([.., n, k] with transposeX2); its storage
 * is the fractal array [.., ceil(cols / c0), ceil(rows / 16), 16, c0] of that matrix with zero padding, c0 = 32 elements
 * for 8-bit types and 32 (or 16) for FLOAT4_E2M1 (aclnnQuantMatmulWeightNz.md:544-550; layout
 * matmul/common/tests/st/arch35/matmul_golden_util.py:76-114).  Phase 2 lays x2 out as the dense matrix once
 * (workspace) and runs the V5 kernels; every quantisation mode of V5 is available.
 */
#ifndef OPSNN_ACLNN_QUANT_MATMUL_WEIGHT_NZ_H_
#define OPSNN_ACLNN_QUANT_MATMUL_WEIGHT_NZ_H_
#include "acl/acl.h"
#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnQuantMatmulWeightNzGetWorkspaceSize(const aclTensor* x1, const aclTensor* x2,
                                                               const aclTensor* x1Scale, const aclTensor* x2Scale,
                                                               const aclTensor* yScale, const aclTensor* x1Offset,
                                                               const aclTensor* x2Offset, const aclTensor* yOffset,
                                                               const aclTensor* bias, bool transposeX1,
                                                               bool transposeX2, int64_t groupSize, aclTensor* out,
                                                               uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnQuantMatmulWeightNz(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                               aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
