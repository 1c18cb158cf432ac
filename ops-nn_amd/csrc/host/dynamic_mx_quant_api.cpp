// aclnnDynamicMxQuant: validation by the documented rules, then the MX quantisation kernel.
//
// The reference has no hand-written host file for this entry point (it is generated from the operator definition); the
// rules are those of quant/dynamic_mx_quant/docs/aclnnDynamicMxQuant.md:99-260 and :312-320.  Phase 1 never touches
// tensor data.
#include <algorithm>
#include <cstring>
#include <initializer_list>
#include <memory>

#include "aclnnop/aclnn_dynamic_mx_quant.h"
#include "aclnnop/aclnn_dynamic_mx_quant_v2.h"
#include "aclnnop/aclnn_dynamic_mx_quant_v3.h"
#include "tensor.h"

using namespace opsnn;

namespace {

constexpr const char* kApi = "aclnnDynamicMxQuant";

#define FAIL(code, ...)         \
    do {                        \
        set_error(__VA_ARGS__); \
        return (code);          \
    } while (0)
#define INVALID(...) FAIL(ACLNN_ERR_PARAM_INVALID, __VA_ARGS__)
#define NOT_RUN(...) FAIL(ACLNN_ERR_INNER_TILING_ERROR, __VA_ARGS__)

bool in_list(int64_t v, std::initializer_list<int64_t> l) { return std::find(l.begin(), l.end(), v) != l.end(); }

}  // namespace

extern "C" {

aclnnStatus aclnnDynamicMxQuantGetWorkspaceSize(const aclTensor* x_, int64_t axis, char* roundModeOptional, int64_t dstType,
                                                int64_t blocksize, int64_t scaleAlg, const aclTensor* y_, const aclTensor* scale_,
                                                uint64_t* workspaceSize, aclOpExecutor** executor)
{
    clear_error();
    if (!x_ || !y_ || !scale_) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: x, yOut and mxscaleOut must not be null", kApi);
    if (!workspaceSize || !executor) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: workspaceSize/executor is null", kApi);
    const TView x = make_view(x_), y = make_view(y_), sc = make_view(scale_);
    if (!in_list(x.dtype, {ACL_FLOAT16, ACL_BF16, ACL_FLOAT})) INVALID("%s: x must be FLOAT16, BF16 or FLOAT, got %s", kApi, dtype_name(x.dtype));
    if (!in_list(dstType, {ACL_FLOAT8_E5M2, ACL_FLOAT8_E4M3FN, ACL_FLOAT4_E2M1, ACL_FLOAT4_E1M2})) INVALID("%s: dstType %ld is not supported", kApi, (long)dstType);
    if ((int64_t)y.dtype != dstType) INVALID("%s: yOut is %s but dstType is %ld", kApi, dtype_name(y.dtype), (long)dstType);
    if (sc.dtype != ACL_FLOAT8_E8M0) INVALID("%s: mxscaleOut must be FLOAT8_E8M0, got %s", kApi, dtype_name(sc.dtype));
    const bool fp4 = is_4bit(y.dtype);
    const char* mode = roundModeOptional ? roundModeOptional : "rint";
    const bool mode_ok = fp4 ? (!std::strcmp(mode, "rint") || !std::strcmp(mode, "floor") || !std::strcmp(mode, "round")) : !std::strcmp(mode, "rint");
    if (!mode_ok) INVALID("%s: roundMode %s is not supported for this output type", kApi, mode);
    if (blocksize <= 0 || blocksize % 32 != 0 || blocksize > 1024) INVALID("%s: blocksize must be a multiple of 32 up to 1024, got %ld", kApi, (long)blocksize);
    if (x.dtype == ACL_FLOAT && blocksize != 32) INVALID("%s: blocksize must be 32 for a FLOAT x", kApi);
    if (scaleAlg != 0 && scaleAlg != 1) INVALID("%s: scaleAlg must be 0 or 1, got %ld", kApi, (long)scaleAlg);
    if (fp4 && scaleAlg != 0) INVALID("%s: scaleAlg must be 0 for a FLOAT4 output", kApi);
    if (x.rank() < 1 || x.rank() > 7) INVALID("%s: x must have 1 to 7 dims, got %ld", kApi, (long)x.rank());
    if (axis < -x.rank() || axis >= x.rank()) INVALID("%s: axis %ld is out of range for %ld dims", kApi, (long)axis, (long)x.rank());
    const int64_t ax = axis < 0 ? axis + x.rank() : axis;
    if (y.shape != x.shape) INVALID("%s: yOut %s must have x's shape %s", kApi, shape_str(y.shape).c_str(), shape_str(x.shape).c_str());
    if (fp4 && x.dim(-1) % 2 != 0) INVALID("%s: the last dim of x must be even for a FLOAT4 output, got %ld", kApi, (long)x.dim(-1));
    std::vector<int64_t> want = x.shape;
    want[(size_t)ax] = ((x.dim(ax) + blocksize - 1) / blocksize + 1) / 2;
    want.push_back(2);
    if (sc.shape != want) INVALID("%s: mxscaleOut %s must be %s", kApi, shape_str(sc.shape).c_str(), shape_str(want).c_str());
    if (!is_contiguous(x) || !is_contiguous(y) || !is_contiguous(sc)) INVALID("%s: tensors must be contiguous here", kApi);
    // the last axis of a 16-bit x, rounded to nearest even onto e2m1 / fp8: the tuned kernels; anything else the general one
    const int round_mode = !std::strcmp(mode, "rint") ? 0 : !std::strcmp(mode, "round") ? 1 : 2;
    const bool general = ax != x.rank() - 1 || x.dtype == ACL_FLOAT || y.dtype == ACL_FLOAT4_E1M2 || round_mode != 0;

    std::unique_ptr<aclOpExecutor> ex(new (std::nothrow) aclOpExecutor());
    if (!ex) FAIL(ACLNN_ERR_INNER_CREATE_EXECUTOR, "%s: cannot allocate executor", kApi);
    ex->api = kApi;
    *workspaceSize = 0;
    if (x.empty()) {
        ex->kind = OpKind::None;
        *executor = (aclOpExecutor*)executor_publish(ex.release());
        return ACLNN_SUCCESS;
    }
    ex->kind = OpKind::MxQuant;
    OpsnnMxQuantArgs& a = ex->mxq;
    a.x = x.ptr_at(0); a.x_dtype = x.dtype;
    a.y = const_cast<void*>(y.ptr_at(0)); a.y_dtype = y.dtype;
    a.scale = const_cast<void*>(sc.ptr_at(0));
    a.cols = x.dim(-1); a.rows = x.numel() / a.cols; a.force_variant = 0;
    a.block = blocksize; a.scale_alg = (int)scaleAlg;
    a.outer = a.axis_len = a.inner = 0; a.round_mode = 0;
    if (general) {
        a.axis_len = x.dim(ax); a.outer = 1; a.inner = 1; a.round_mode = round_mode;
        for (int64_t i = 0; i < ax; i++) a.outer *= x.dim(i);
        for (int64_t i = ax + 1; i < x.rank(); i++) a.inner *= x.dim(i);
    }
    *executor = (aclOpExecutor*)executor_publish(ex.release());
    return ACLNN_SUCCESS;
}

// V2 adds dstTypeMax, V3 maxLowBound (a lower clamp of the block maximum): both belong to scale algorithms and type maxima
// that have no kernel here; with both at 0 the call is the first version's.
static aclnnStatus mx_quant_later_version(const char* api, const aclTensor* x, int64_t axis, char* roundModeOptional, int64_t dstType,
                                          int64_t blocksize, int64_t scaleAlg, double dstTypeMax, double maxLowBound, const aclTensor* yOut,
                                          const aclTensor* mxscaleOut, uint64_t* workspaceSize, aclOpExecutor** executor)
{
    if (scaleAlg == 2 && x && yOut && mxscaleOut && workspaceSize && executor) NOT_RUN("%s: scaleAlg 2 has no kernel here", api);
    const aclnnStatus rc = aclnnDynamicMxQuantGetWorkspaceSize(x, axis, roundModeOptional, dstType, blocksize, scaleAlg, yOut, mxscaleOut,
                                                               workspaceSize, executor);
    if (rc != ACLNN_SUCCESS) return rc;
    if (dstTypeMax != 0.0 || maxLowBound != 0.0) {
        aclDestroyAclOpExecutor(*executor);
        *executor = nullptr;
        NOT_RUN("%s: dstTypeMax / maxLowBound other than 0 have no kernel here", api);
    }
    return ACLNN_SUCCESS;
}

aclnnStatus aclnnDynamicMxQuantV2GetWorkspaceSize(const aclTensor* x, int64_t axis, char* roundModeOptional, int64_t dstType, int64_t blocksize,
                                                  int64_t scaleAlg, double dstTypeMax, const aclTensor* yOut, const aclTensor* mxscaleOut,
                                                  uint64_t* workspaceSize, aclOpExecutor** executor)
{
    return mx_quant_later_version("aclnnDynamicMxQuantV2", x, axis, roundModeOptional, dstType, blocksize, scaleAlg, dstTypeMax, 0.0, yOut,
                                  mxscaleOut, workspaceSize, executor);
}
aclnnStatus aclnnDynamicMxQuantV3GetWorkspaceSize(const aclTensor* x, int64_t axis, char* roundModeOptional, int64_t dstType, int64_t blocksize,
                                                  int64_t scaleAlg, double dstTypeMax, double maxLowBound, const aclTensor* yOut,
                                                  const aclTensor* mxscaleOut, uint64_t* workspaceSize, aclOpExecutor** executor)
{
    return mx_quant_later_version("aclnnDynamicMxQuantV3", x, axis, roundModeOptional, dstType, blocksize, scaleAlg, dstTypeMax, maxLowBound, yOut,
                                  mxscaleOut, workspaceSize, executor);
}
aclnnStatus aclnnDynamicMxQuantV2(void* ws, uint64_t n, aclOpExecutor* executor, aclrtStream stream) { return aclnnDynamicMxQuant(ws, n, executor, stream); }
aclnnStatus aclnnDynamicMxQuantV3(void* ws, uint64_t n, aclOpExecutor* executor, aclrtStream stream) { return aclnnDynamicMxQuant(ws, n, executor, stream); }

aclnnStatus aclnnDynamicMxQuant(void*, uint64_t, aclOpExecutor* executor, aclrtStream stream)
{
    clear_error();
    if (!executor) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: executor is null", kApi);
    if (!executor_claim(executor)) INVALID("%s: executor is not valid (already run or destroyed)", kApi);
    std::unique_ptr<aclOpExecutor> ex(executor);
    ex->magic = 0;
    if (ex->kind == OpKind::None) return ACLNN_SUCCESS;
    if (ex->kind != OpKind::MxQuant) INVALID("%s: executor belongs to another operator", kApi);
    if (!ex->mxq.x || !ex->mxq.y || !ex->mxq.scale) INVALID("%s: a tensor has no device address", kApi);
    const int rc = opsnnDynamicMxQuant(&ex->mxq, stream);
    if (rc != 0) FAIL(rc < 0 ? ACLNN_ERR_INNER_TILING_ERROR : ACLNN_ERR_RUNTIME_ERROR, "%s: launch failed with code %d", kApi, rc);
    return ACLNN_SUCCESS;
}

}  // extern "C"
