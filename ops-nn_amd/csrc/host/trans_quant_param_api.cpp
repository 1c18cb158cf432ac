// aclnnTransQuantParamV2 / V3: validation in the reference's rule order, then the packing kernel.
//
// Behaviour follows quant/trans_quant_param_v2/op_host/op_api/aclnn_trans_quant_param_v2.cpp: CheckParams :113-127 (null,
// dtypes, formats, shapes and round mode), the newest-SoC shape rule :67-75.  Phase 1 never touches tensor data.
#include <memory>

#include "aclnnop/aclnn_trans_quant_param_v2.h"
#include "aclnnop/aclnn_trans_quant_param_v3.h"
#include "tensor.h"

using namespace opsnn;

namespace {

#define FAIL(code, ...)         \
    do {                        \
        set_error(__VA_ARGS__); \
        return (code);          \
    } while (0)
#define INVALID(...) FAIL(ACLNN_ERR_PARAM_INVALID, __VA_ARGS__)

aclnnStatus get_workspace(const char* api, const aclTensor* scale_, const aclTensor* offset_, int64_t roundMode, const aclTensor* out_,
                          uint64_t* workspaceSize, aclOpExecutor** executor)
{
    clear_error();
    if (!scale_ || !out_) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: scale and out must not be null", api);
    if (!workspaceSize || !executor) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: workspaceSize/executor is null", api);
    const TView sc = make_view(scale_), off = make_view(offset_), out = make_view(out_);
    if (sc.dtype != ACL_FLOAT) INVALID("%s: scale must be FLOAT, got %s", api, dtype_name(sc.dtype));
    if (off.present && off.dtype != ACL_FLOAT) INVALID("%s: offset must be FLOAT, got %s", api, dtype_name(off.dtype));
    if (out.dtype != ACL_UINT64 && out.dtype != ACL_INT64) INVALID("%s: out must be UINT64 or INT64, got %s", api, dtype_name(out.dtype));
    if (sc.format != ACL_FORMAT_ND || out.format != ACL_FORMAT_ND || (off.present && off.format != ACL_FORMAT_ND))
        INVALID("%s: tensors must be in ND format", api);
    const bool sc_ok = (sc.rank() == 1 && sc.dim(0) > 0) || (sc.rank() == 2 && sc.dim(0) > 0 && sc.dim(1) > 0);
    if (!sc_ok) INVALID("%s: scale must be [n] or [g, n] with positive dims, got %s", api, shape_str(sc.shape).c_str());
    if (off.present) {
        const bool off_ok = (off.rank() == 1 && off.dim(0) > 0) || (off.rank() == 2 && off.dim(0) == 1 && off.dim(1) > 0);
        if (!off_ok) INVALID("%s: offset must be [n] or [1, n], got %s", api, shape_str(off.shape).c_str());
        if (off.rank() == 1 && sc.dim(0) > 1 && off.dim(0) > 1 && sc.dim(0) != off.dim(0))
            INVALID("%s: scale and offset must have the same length when both are longer than 1 (%ld, %ld)", api, (long)sc.dim(0), (long)off.dim(0));
    }
    if (roundMode != 0 && roundMode != 1) INVALID("%s: roundMode must be 0 or 1, got %ld", api, (long)roundMode);
    // what the kernel needs beyond the reference's checks: dense tensors, broadcast only from one element, out large enough
    const int64_t ns = sc.numel(), no = off.present ? off.numel() : 0, n = ns > no ? ns : no;
    if ((ns != 1 && ns != n) || (off.present && no != 1 && no != n))
        INVALID("%s: scale (%ld elements) and offset (%ld) do not broadcast to one length", api, (long)ns, (long)no);
    if (out.numel() != n) INVALID("%s: out has %ld elements, %ld expected", api, (long)out.numel(), (long)n);
    if (!is_contiguous(sc) || !is_contiguous(out) || (off.present && !is_contiguous(off))) INVALID("%s: tensors must be contiguous here", api);

    std::unique_ptr<aclOpExecutor> ex(new (std::nothrow) aclOpExecutor());
    if (!ex) FAIL(ACLNN_ERR_INNER_CREATE_EXECUTOR, "%s: cannot allocate executor", api);
    ex->api = "aclnnTransQuantParam";
    ex->kind = OpKind::TransQuantParam;
    ex->tqp.scale = (const float*)sc.ptr_at(0); ex->tqp.scale_len = ns;
    ex->tqp.offset = off.present ? (const float*)off.ptr_at(0) : nullptr; ex->tqp.offset_len = no;
    ex->tqp.round_mode = (int)roundMode;
    ex->tqp.out = (uint64_t*)const_cast<void*>(out.ptr_at(0));
    *workspaceSize = 0;
    *executor = (aclOpExecutor*)executor_publish(ex.release());
    return ACLNN_SUCCESS;
}

aclnnStatus run(const char* api, aclOpExecutor* executor, aclrtStream stream)
{
    clear_error();
    if (!executor) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: executor is null", api);
    if (!executor_claim(executor)) INVALID("%s: executor is not valid (already run or destroyed)", api);
    std::unique_ptr<aclOpExecutor> ex(executor);
    ex->magic = 0;
    if (ex->kind != OpKind::TransQuantParam) INVALID("%s: executor belongs to another operator", api);
    if (!ex->tqp.scale || !ex->tqp.out) INVALID("%s: a tensor has no device address", api);
    const int rc = opsnnTransQuantParam(ex->tqp.scale, ex->tqp.scale_len, ex->tqp.offset, ex->tqp.offset_len, ex->tqp.round_mode, ex->tqp.out, stream);
    if (rc != 0) FAIL(rc < 0 ? ACLNN_ERR_INNER_TILING_ERROR : ACLNN_ERR_RUNTIME_ERROR, "%s: launch failed with code %d", api, rc);
    return ACLNN_SUCCESS;
}

}  // namespace

extern "C" {

aclnnStatus aclnnTransQuantParamV2GetWorkspaceSize(const aclTensor* scale, const aclTensor* offset, const aclTensor* out,
                                                   uint64_t* workspaceSize, aclOpExecutor** executor)
{
    return get_workspace("aclnnTransQuantParamV2GetWorkspaceSize", scale, offset, 0, out, workspaceSize, executor);
}
aclnnStatus aclnnTransQuantParamV3GetWorkspaceSize(const aclTensor* scale, const aclTensor* offset, int64_t roundMode, const aclTensor* out,
                                                   uint64_t* workspaceSize, aclOpExecutor** executor)
{
    return get_workspace("aclnnTransQuantParamV3GetWorkspaceSize", scale, offset, roundMode, out, workspaceSize, executor);
}
aclnnStatus aclnnTransQuantParamV2(void*, uint64_t, aclOpExecutor* executor, const aclrtStream stream) { return run("aclnnTransQuantParamV2", executor, stream); }
aclnnStatus aclnnTransQuantParamV3(void*, uint64_t, aclOpExecutor* executor, const aclrtStream stream) { return run("aclnnTransQuantParamV3", executor, stream); }

}  // extern "C"
