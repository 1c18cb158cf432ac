/*
 * aclnnDynamicMxQuant -- MX quantisation along one axis: per `blocksize` elements one FLOAT8_E8M0 scale
 * 2^(floor(log2 max|x|) - emax) and the elements x / scale rounded to the FLOAT4 / FLOAT8 target.
 *
 * The reference generates this entry point from the operator definition (quant/dynamic_mx_quant/op_host/
 * dynamic_mx_quant_def.cpp); signature and rules are the documented ones, quant/dynamic_mx_quant/docs/
 * aclnnDynamicMxQuant.md:76-95, 99-260, 312-320; arithmetic of quant/dynamic_mx_quant/tests/assets/golden.py:140-330.
 * x: FLOAT16 / BF16 / FLOAT (FLOAT: blocksize 32), 1 to 7 dims.  yOut: x's shape, FLOAT4_E2M1 or FLOAT4_E1M2 (last dim even),
 * FLOAT8_E4M3FN or FLOAT8_E5M2, equal to dstType (40 / 41 / 36 / 35).  mxscaleOut: FLOAT8_E8M0, x's shape with the axis dim
 * replaced by ceil(ceil(n / blocksize) / 2) and a trailing dim of 2 (the two blocks of a pair side by side).  Any axis, every
 * blocksize (a multiple of 32 up to 1024), roundMode NULL or "rint" (the 4-bit types also "floor" and "round"), scaleAlg 0 and
 * (FLOAT8 outputs) 1; the last axis of a 16-bit x with blocks of 32 and "rint" has the tuned kernel.  Tensors must be
 * contiguous.  The V2 / V3 arguments dstTypeMax / maxLowBound other than 0 and scaleAlg 2 are answered with
 * ACLNN_ERR_INNER_TILING_ERROR (the reference's golden does not define them).
 */
#ifndef OPSNN_AMD_ACLNN_DYNAMIC_MX_QUANT_H_
#define OPSNN_AMD_ACLNN_DYNAMIC_MX_QUANT_H_

#include "acl/acl.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnDynamicMxQuantGetWorkspaceSize(const aclTensor* x, int64_t axis, char* roundModeOptional, int64_t dstType,
                                                          int64_t blocksize, int64_t scaleAlg, const aclTensor* yOut,
                                                          const aclTensor* mxscaleOut, uint64_t* workspaceSize,
                                                          aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnDynamicMxQuant(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif
