// aclnnDynamicQuant / aclnnDynamicQuantV2: validation in the reference's rule order, then the per-token quantisation kernel.
//
// Behaviour follows quant/dynamic_quant/op_host/op_api/aclnn_dynamic_quant.cpp (CheckParams :320-328 and the checks it
// calls, empty tensors :366-371, the INT32 carrier of INT4 :384-389) for the per-token mode on the reference's newest
// SoC generation.  Phase 1 never touches tensor data and never calls HIP.
#include <algorithm>
#include <cstring>
#include <initializer_list>
#include <memory>

#include "aclnnop/aclnn_dynamic_quant.h"
#include "aclnnop/aclnn_dynamic_quant_v2.h"
#include "aclnnop/aclnn_dynamic_quant_v3.h"
#include "aclnnop/aclnn_dynamic_quant_v4.h"
#include "tensor.h"

using namespace opsnn;

namespace {

#define FAIL(code, ...)         \
    do {                        \
        set_error(__VA_ARGS__); \
        return (code);          \
    } while (0)
#define INVALID(...) FAIL(ACLNN_ERR_PARAM_INVALID, __VA_ARGS__)

bool in_list(aclDataType d, std::initializer_list<aclDataType> l) { return std::find(l.begin(), l.end(), d) != l.end(); }

aclnnStatus get_workspace(const char* api, const aclTensor* x_, const aclTensor* smooth_, const aclTensor* group_, bool symmetrical,
                          const char* quantMode, float dstTypeMax, const aclTensor* y_, const aclTensor* scale_, const aclTensor* offset_,
                          uint64_t* workspaceSize, aclOpExecutor** executor)
{
    clear_error();
    if (!x_ || !y_ || !scale_) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: x, yOut and scaleOut must not be null", api);   // :136-142
    if (!workspaceSize || !executor) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: workspaceSize/executor is null", api);
    // attributes :171-189
    if (symmetrical && offset_) INVALID("%s: offsetOut must be null when isSymmetrical is true", api);
    if (!symmetrical && !offset_) INVALID("%s: offsetOut must not be null when isSymmetrical is false", api);
    if (!quantMode) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: quantMode is null", api);
    const bool pertensor = !std::strcmp(quantMode, "pertensor"), perchannel = !std::strcmp(quantMode, "perchannel");
    if (!pertensor && !perchannel && std::strcmp(quantMode, "pertoken") != 0) INVALID("%s: quantMode must be pertensor, pertoken or perchannel, got %s", api, quantMode);
    if (perchannel && group_) INVALID("%s: groupIndex must be null when quantMode is perchannel", api);
    const TView x = make_view(x_), sm = make_view(smooth_), gi = make_view(group_), y = make_view(y_), sc = make_view(scale_),
                off = make_view(offset_);
    // dtypes :293-317
    if (!in_list(x.dtype, {ACL_FLOAT16, ACL_BF16})) INVALID("%s: x must be FLOAT16 or BF16, got %s", api, dtype_name(x.dtype));
    if (sm.present) {
        if (!in_list(sm.dtype, {ACL_FLOAT16, ACL_BF16})) INVALID("%s: smoothScales must be FLOAT16 or BF16, got %s", api, dtype_name(sm.dtype));
        if (sm.dtype != x.dtype) INVALID("%s: the dtypes of x and smoothScales are not equal", api);
        if (gi.present && !in_list(gi.dtype, {ACL_INT32, ACL_INT64})) INVALID("%s: groupIndex must be INT32 or INT64", api);
    }
    if (!in_list(y.dtype, {ACL_INT4, ACL_INT8, ACL_INT32, ACL_HIFLOAT8, ACL_FLOAT8_E5M2, ACL_FLOAT8_E4M3FN}))
        INVALID("%s: yOut dtype %s is not supported", api, dtype_name(y.dtype));
    if (sc.dtype != ACL_FLOAT) INVALID("%s: scaleOut must be FLOAT, got %s", api, dtype_name(sc.dtype));
    if (off.present && off.dtype != ACL_FLOAT) INVALID("%s: offsetOut must be FLOAT, got %s", api, dtype_name(off.dtype));
    // shapes :191-291
    if (x.rank() <= 1 || x.rank() >= 9) INVALID("%s: x must have 2 to 8 dims, got %ld", api, (long)x.rank());
    const int64_t cols = x.dim(-1);
    if (sm.present) {
        if (gi.present) {
            if (gi.rank() != 1) INVALID("%s: groupIndex must have one dim", api);
            // documented (quant/dynamic_quant_v2/docs/aclnnDynamicQuantV2.md:156-166): smoothScales [experts <= 1024, x.shape[-1]]
            if (sm.rank() != 2 || sm.dim(1) != cols || sm.dim(0) != gi.dim(0) || sm.dim(0) > 1024)
                INVALID("%s: with groupIndex [%ld] smoothScales must be [%ld, %ld] (at most 1024 experts), got %s", api, (long)gi.dim(0),
                        (long)gi.dim(0), (long)cols, shape_str(sm.shape).c_str());
        } else {
            if (sm.rank() != 1) INVALID("%s: smoothScales must have one dim, got %ld", api, (long)sm.rank());
            const int64_t want_len = perchannel ? x.dim(-2) : cols;
            if (sm.dim(0) != want_len) INVALID("%s: smoothScales has %ld elements, %ld expected", api, (long)sm.dim(0), (long)want_len);
        }
    }
    if (y.dtype != ACL_INT32) {
        if (y.shape != x.shape) INVALID("%s: the shapes of x %s and yOut %s are inconsistent", api, shape_str(x.shape).c_str(), shape_str(y.shape).c_str());
    } else {
        if (y.rank() != x.rank() || cols != y.dim(-1) * 8)
            INVALID("%s: an INT32 yOut carries eight INT4: its last dim must be 1/8 of x's (%ld), got %ld", api, (long)cols,
                    y.rank() ? (long)y.dim(-1) : 0L);
        for (int64_t i = 0; i + 1 < x.rank(); i++)
            if (x.dim(i) != y.dim(i)) INVALID("%s: dim %ld of x (%ld) and yOut (%ld) differ", api, (long)i, (long)x.dim(i), (long)y.dim(i));
    }
    if (y.dtype == ACL_INT4 && cols % 2 != 0) INVALID("%s: the last dim of x must be even for an INT4 yOut, got %ld", api, (long)cols);
    if (pertensor) {
        if (sc.rank() != 1 || sc.dim(0) != 1) INVALID("%s: scaleOut must be [1] when quantMode is pertensor", api);
    } else if (perchannel) {
        std::vector<int64_t> want(x.shape.begin(), x.shape.end() - 2);
        want.push_back(cols);
        if (sc.shape != want) INVALID("%s: scaleOut %s must be %s when quantMode is perchannel", api, shape_str(sc.shape).c_str(), shape_str(want).c_str());
    } else if (sc.rank() != x.rank() - 1 || !std::equal(sc.shape.begin(), sc.shape.end(), x.shape.begin()))
        INVALID("%s: scaleOut %s must have x's shape %s without the last dim", api, shape_str(sc.shape).c_str(), shape_str(x.shape).c_str());
    if (off.present && off.shape != sc.shape) INVALID("%s: offsetOut %s and scaleOut %s differ in shape", api, shape_str(off.shape).c_str(), shape_str(sc.shape).c_str());

    std::unique_ptr<aclOpExecutor> ex(new (std::nothrow) aclOpExecutor());
    if (!ex) FAIL(ACLNN_ERR_INNER_CREATE_EXECUTOR, "%s: cannot allocate executor", api);
    ex->api = "aclnnDynamicQuant";
    *workspaceSize = 0;
    if (x.empty() || y.empty() || sc.empty()) {   // :366-371
        ex->kind = OpKind::None;
        *executor = (aclOpExecutor*)executor_publish(ex.release());
        return ACLNN_SUCCESS;
    }
    // what this build does not run
    if ((pertensor || perchannel) && gi.present) FAIL(ACLNN_ERR_INNER_TILING_ERROR, "%s: groupIndex with quantMode %s has no kernel here", api, quantMode);
    if (dstTypeMax != 0.0f) FAIL(ACLNN_ERR_INNER_TILING_ERROR, "%s: a dstTypeMax other than 0 has no kernel here", api);
    if (gi.present && !sm.present) INVALID("%s: groupIndex needs smoothScales", api);
    if (gi.present && (gi.empty() || !is_contiguous(gi))) INVALID("%s: groupIndex must be a non-empty contiguous tensor here", api);
    if (y.dtype == ACL_HIFLOAT8) FAIL(ACLNN_ERR_INNER_TILING_ERROR, "%s: HIFLOAT8 output has no kernel on this device", api);
    if (!is_contiguous(x) || !is_contiguous(y) || !is_contiguous(sc) || (sm.present && !is_contiguous(sm)) || (off.present && !is_contiguous(off)))
        INVALID("%s: tensors must be contiguous here", api);
    if (x.numel() / cols > 0x7fffffff) INVALID("%s: more than 2^31 - 1 rows", api);
    ex->kind = OpKind::DynQuant;
    OpsnnDynQuantArgs& a = ex->dynq;
    a.x = x.ptr_at(0); a.x_dtype = x.dtype;
    a.smooth = sm.present ? sm.ptr_at(0) : nullptr;
    a.y = const_cast<void*>(y.ptr_at(0)); a.y_dtype = y.dtype == ACL_INT32 ? ACL_INT4 : y.dtype;
    a.scale = (float*)const_cast<void*>(sc.ptr_at(0));
    a.offset = off.present ? (float*)const_cast<void*>(off.ptr_at(0)) : nullptr;
    a.rows = x.numel() / cols; a.cols = cols;
    a.force_variant = 0;
    if (gi.present) { a.group_index = gi.ptr_at(0); a.group_index_dtype = gi.dtype; a.groups = gi.dim(0); }
    a.quant_mode = pertensor ? 1 : perchannel ? 2 : 0;
    a.chan_rows = perchannel ? x.dim(-2) : 0;
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
    if (ex->kind == OpKind::None) return ACLNN_SUCCESS;
    if (ex->kind != OpKind::DynQuant) INVALID("%s: executor belongs to another operator", api);
    if (!ex->dynq.x || !ex->dynq.y || !ex->dynq.scale) INVALID("%s: a tensor has no device address", api);
    const int rc = opsnnDynamicQuant(&ex->dynq, stream);
    if (rc != 0) FAIL(rc < 0 ? ACLNN_ERR_INNER_TILING_ERROR : ACLNN_ERR_RUNTIME_ERROR, "%s: launch failed with code %d", api, rc);
    return ACLNN_SUCCESS;
}

}  // namespace

extern "C" {

aclnnStatus aclnnDynamicQuantGetWorkspaceSize(const aclTensor* x, const aclTensor* smoothScalesOptional, const aclTensor* yOut,
                                              const aclTensor* scaleOut, uint64_t* workspaceSize, aclOpExecutor** executor)
{
    return get_workspace("aclnnDynamicQuantGetWorkspaceSize", x, smoothScalesOptional, nullptr, true, "pertoken", 0.0f, yOut, scaleOut, nullptr,
                         workspaceSize, executor);
}

aclnnStatus aclnnDynamicQuant(void*, uint64_t, aclOpExecutor* executor, aclrtStream stream) { return run("aclnnDynamicQuant", executor, stream); }

aclnnStatus aclnnDynamicQuantV2GetWorkspaceSize(const aclTensor* x, const aclTensor* smoothScalesOptional,
                                                const aclTensor* groupIndexOptional, int64_t dstType, const aclTensor* yOut,
                                                const aclTensor* scaleOut, const aclTensor* offsetOut, uint64_t* workspaceSize,
                                                aclOpExecutor** executor)
{
    (void)dstType;   // the reference takes the output type from yOut (:384-389); dstType only reaches its log
    return get_workspace("aclnnDynamicQuantV2GetWorkspaceSize", x, smoothScalesOptional, groupIndexOptional, offsetOut == nullptr, "pertoken", 0.0f,
                         yOut, scaleOut, offsetOut, workspaceSize, executor);
}

aclnnStatus aclnnDynamicQuantV2(void*, uint64_t, aclOpExecutor* executor, aclrtStream stream) { return run("aclnnDynamicQuantV2", executor, stream); }

aclnnStatus aclnnDynamicQuantV3GetWorkspaceSize(const aclTensor* x, const aclTensor* smoothScalesOptional, const aclTensor* groupIndexOptional,
                                                int64_t dstType, bool isSymmetrical, const char* quantMode, const aclTensor* yOut,
                                                const aclTensor* scaleOut, const aclTensor* offsetOut, uint64_t* workspaceSize,
                                                aclOpExecutor** executor)
{
    (void)dstType;
    return get_workspace("aclnnDynamicQuantV3GetWorkspaceSize", x, smoothScalesOptional, groupIndexOptional, isSymmetrical, quantMode, 0.0f, yOut,
                         scaleOut, offsetOut, workspaceSize, executor);
}

aclnnStatus aclnnDynamicQuantV3(void*, uint64_t, aclOpExecutor* executor, aclrtStream stream) { return run("aclnnDynamicQuantV3", executor, stream); }

aclnnStatus aclnnDynamicQuantV4GetWorkspaceSize(const aclTensor* x, const aclTensor* smoothScalesOptional, const aclTensor* groupIndexOptional,
                                                int64_t dstType, bool isSymmetrical, const char* quantMode, float dstTypeMax,
                                                const aclTensor* yOut, const aclTensor* scaleOut, const aclTensor* offsetOut,
                                                uint64_t* workspaceSize, aclOpExecutor** executor)
{
    (void)dstType;
    return get_workspace("aclnnDynamicQuantV4GetWorkspaceSize", x, smoothScalesOptional, groupIndexOptional, isSymmetrical, quantMode, dstTypeMax,
                         yOut, scaleOut, offsetOut, workspaceSize, executor);
}

aclnnStatus aclnnDynamicQuantV4(void*, uint64_t, aclOpExecutor* executor, aclrtStream stream) { return run("aclnnDynamicQuantV4", executor, stream); }

}  // extern "C"
