/*
 * aclnnTransQuantParamV3 -- packs an fp32 dequantisation scale and an optional fp32 offset into the UINT64 / INT64 tensor
 * that aclnnQuantMatmulV5 takes as x2Scale in its per-tensor / per-channel modes; roundMode 0 truncates the scale to
 * 19 bits, 1 rounds it to nearest even.
 *
 * Replaces quant/trans_quant_param_v2/op_host/op_api/aclnn_trans_quant_param_v3.h; checks of
 * aclnn_trans_quant_param_v2.cpp:36-127; arithmetic of the device kernel op_kernel/trans_quant_param_v2.h:224-300.
 * scale: FLOAT, [n] or [g, n] (any g, as on the reference's newest SoC).  offset: optional FLOAT, [n] or [1, n]; when both
 * have more than one element the counts must agree.  out: UINT64 or INT64 with max(count(scale), count(offset)) elements.
 */
#ifndef OPSNN_AMD_ACLNN_TRANS_QUANT_PARAM_V3_H_
#define OPSNN_AMD_ACLNN_TRANS_QUANT_PARAM_V3_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnTransQuantParamV3GetWorkspaceSize(const aclTensor* scale, const aclTensor* offset, int64_t roundMode,
                                                             const aclTensor* out, uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnTransQuantParamV3(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, const aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
