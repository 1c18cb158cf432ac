/*
 * aclnnQuantMatmulV5 -- quantized matmul, two-phase C entry points.
 *
 * Replaces, with the same names, argument order and meaning:
 *   matmul/quant_batch_matmul_v4/op_host/op_api/aclnn_quant_matmul_v5.h:43-60
 * (implementation in the reference: aclnn_quant_matmul_v5.cpp:1189-1227).
 *
 * out = dequant(x1 @ x2) with the quantization mode inferred from the scale
 * tensors: per-token x per-channel (K-C / K-T), per-tensor / per-channel (T-T /
 * T-C), 128-wide block scales (G-B / B-B) and MX e8m0 group scales.
 */
#ifndef OPSNN_AMD_ACLNN_QUANT_MATMUL_V5_H_
#define OPSNN_AMD_ACLNN_QUANT_MATMUL_V5_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Phase 1: validate, pick the kernel variant, report the device workspace size
 * and hand back an executor (only on ACLNN_SUCCESS; ownership passes to the
 * caller until phase 2 consumes it).  Never reads tensor data.
 *
 *  x1        int8 / int4 / fp8 e4m3fn / fp8 e5m2 / fp4 e2m1, [.., m, k] (or [.., k, m] if transposeX1)
 *  x2        same family as x1, [.., k, n] (or [.., n, k] if transposeX2)
 *  x1Scale   optional; fp32 per-token [m], fp32 block scale [m, ceil(k/128)] or e8m0 [m, ceil(k/64), 2]
 *  x2Scale   required; fp32/bf16 [1] or [n], uint64/int64 packed, fp32 block scale, or e8m0
 *  yScale    uint64 [1] or [n] output scale of the fp8 x fp4 group-scale mode (x2Scale bf16/fp16 [ceil(k/gsK), n]); NULL otherwise
 *  x1Offset, yOffset   must be NULL
 *  x2Offset  fp32 [1] or [n] with int8 inputs and int8 output; fp16 [ceil(k/256), n] in the int4 K-group mode
 *  bias      optional [n] (int32 / bf16 / fp16 / fp32 depending on the mode)
 *  groupSize gsK | gsN << 16 | gsM << 32; 0 outside block/MX modes
 */
ACLNN_API aclnnStatus aclnnQuantMatmulV5GetWorkspaceSize(const aclTensor* x1, const aclTensor* x2,
                                                         const aclTensor* x1Scale, const aclTensor* x2Scale,
                                                         const aclTensor* yScale, const aclTensor* x1Offset,
                                                         const aclTensor* x2Offset, const aclTensor* yOffset,
                                                         const aclTensor* bias, bool transposeX1, bool transposeX2,
                                                         int64_t groupSize, aclTensor* out, uint64_t* workspaceSize,
                                                         aclOpExecutor** executor);

/*
 * Phase 2: enqueue the computation on `stream` (asynchronous; the caller
 * synchronises).  Consumes the executor; running one executor twice is an
 * error (docs/zh/context/two_phase_api.md:17-24).
 */
ACLNN_API aclnnStatus aclnnQuantMatmulV5(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                         aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
