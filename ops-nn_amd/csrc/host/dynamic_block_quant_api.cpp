// aclnnDynamicBlockQuant: validation by the documented rules, then the block quantisation kernel.
//
// The reference has no hand-written host file for this entry point (it is generated from the operator definition); the
// rules are those of quant/dynamic_block_quant/docs/aclnnDynamicBlockQuant.md:95-220 and of the operator's own attribute
// and shape checks (op_host/dynamic_block_quant_tiling.cpp:135-230, 300-340).  Phase 1 never touches tensor data.
#include <algorithm>
#include <cstring>
#include <initializer_list>
#include <memory>

#include "aclnnop/aclnn_dynamic_block_quant.h"
#include "aclnnop/aclnn_dynamic_block_quant_v2.h"
#include "tensor.h"

using namespace opsnn;

namespace {

constexpr const char* kApi = "aclnnDynamicBlockQuant";

#define FAIL(code, ...)         \
    do {                        \
        set_error(__VA_ARGS__); \
        return (code);          \
    } while (0)
#define INVALID(...) FAIL(ACLNN_ERR_PARAM_INVALID, __VA_ARGS__)

bool in_list(int64_t v, std::initializer_list<int64_t> l) { return std::find(l.begin(), l.end(), v) != l.end(); }

}  // namespace

extern "C" {

aclnnStatus aclnnDynamicBlockQuantGetWorkspaceSize(const aclTensor* x_, double minScale, char* roundModeOptional, int64_t dstType,
                                                   int64_t rowBlockSize, int64_t colBlockSize, const aclTensor* y_,
                                                   const aclTensor* scale_, uint64_t* workspaceSize, aclOpExecutor** executor)
{
    clear_error();
    if (!x_ || !y_ || !scale_) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: x, yOut and scaleOut must not be null", kApi);
    if (!workspaceSize || !executor) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: workspaceSize/executor is null", kApi);
    const TView x = make_view(x_), y = make_view(y_), sc = make_view(scale_);
    if (x.dtype != ACL_FLOAT16 && x.dtype != ACL_BF16) INVALID("%s: x must be FLOAT16 or BF16, got %s", kApi, dtype_name(x.dtype));
    if (!in_list(dstType, {ACL_INT8, ACL_HIFLOAT8, ACL_FLOAT8_E5M2, ACL_FLOAT8_E4M3FN})) INVALID("%s: dstType %ld is not supported", kApi, (long)dstType);
    if ((int64_t)y.dtype != dstType) INVALID("%s: yOut is %s but dstType is %ld", kApi, dtype_name(y.dtype), (long)dstType);
    if (sc.dtype != ACL_FLOAT) INVALID("%s: scaleOut must be FLOAT, got %s", kApi, dtype_name(sc.dtype));
    const bool hif8 = dstType == ACL_HIFLOAT8;
    if (roundModeOptional && std::strcmp(roundModeOptional, hif8 ? "round" : "rint") != 0)
        INVALID("%s: roundMode must be %s for this output type, got %s", kApi, hif8 ? "round" : "rint", roundModeOptional);
    if (!in_list(rowBlockSize, {1, 64, 128, 256, 512})) INVALID("%s: rowBlockSize must be 1, 64, 128, 256 or 512, got %ld", kApi, (long)rowBlockSize);
    if (!in_list(colBlockSize, {64, 128, 192, 256})) INVALID("%s: colBlockSize must be 64, 128, 192 or 256, got %ld", kApi, (long)colBlockSize);
    if (!(minScale >= 0)) INVALID("%s: minScale must not be negative", kApi);
    if (x.rank() != 2 && x.rank() != 3) INVALID("%s: x must have 2 or 3 dims, got %ld", kApi, (long)x.rank());
    if (y.shape != x.shape) INVALID("%s: yOut %s must have x's shape %s", kApi, shape_str(y.shape).c_str(), shape_str(x.shape).c_str());
    if (x.empty()) INVALID("%s: empty tensors are not supported", kApi);
    std::vector<int64_t> want = x.shape;
    want[want.size() - 2] = (x.dim(-2) + rowBlockSize - 1) / rowBlockSize;
    want[want.size() - 1] = (x.dim(-1) + colBlockSize - 1) / colBlockSize;
    if (sc.shape != want) INVALID("%s: scaleOut %s must be %s", kApi, shape_str(sc.shape).c_str(), shape_str(want).c_str());
    // what this build does not run
    if (dstType == ACL_INT8 || hif8) FAIL(ACLNN_ERR_INNER_TILING_ERROR, "%s: %s output has no kernel here", kApi, dtype_name(y.dtype));
    if (!is_contiguous(x) || !is_contiguous(y) || !is_contiguous(sc)) INVALID("%s: tensors must be contiguous here", kApi);

    std::unique_ptr<aclOpExecutor> ex(new (std::nothrow) aclOpExecutor());
    if (!ex) FAIL(ACLNN_ERR_INNER_CREATE_EXECUTOR, "%s: cannot allocate executor", kApi);
    ex->api = kApi;
    ex->kind = OpKind::BlockQuant;
    OpsnnBlockQuantArgs& a = ex->blkq;
    a.x = x.ptr_at(0); a.x_dtype = x.dtype;
    a.y = const_cast<void*>(y.ptr_at(0)); a.y_dtype = y.dtype;
    a.scale = (float*)const_cast<void*>(sc.ptr_at(0));
    a.batch = x.rank() == 3 ? x.dim(0) : 1; a.rows = x.dim(-2); a.cols = x.dim(-1);
    a.row_block = rowBlockSize; a.col_block = colBlockSize; a.min_scale = minScale; a.force_variant = 0;
    *workspaceSize = 0;
    *executor = (aclOpExecutor*)executor_publish(ex.release());
    return ACLNN_SUCCESS;
}

aclnnStatus aclnnDynamicBlockQuantV2GetWorkspaceSize(const aclTensor* x, double minScale, char* roundModeOptional, int64_t dstType,
                                                     int64_t rowBlockSize, int64_t colBlockSize, double dstTypeMax, const aclTensor* yOut,
                                                     const aclTensor* scaleOut, uint64_t* workspaceSize, aclOpExecutor** executor)
{
    const aclnnStatus rc = aclnnDynamicBlockQuantGetWorkspaceSize(x, minScale, roundModeOptional, dstType, rowBlockSize, colBlockSize, yOut,
                                                                  scaleOut, workspaceSize, executor);
    if (rc != ACLNN_SUCCESS) return rc;
    if (dstTypeMax != 0.0) {   // a custom maximum belongs to the HIFLOAT8 output of the reference; the fp8 formulas do not use it
        aclDestroyAclOpExecutor(*executor);
        *executor = nullptr;
        FAIL(ACLNN_ERR_INNER_TILING_ERROR, "aclnnDynamicBlockQuantV2: a dstTypeMax other than 0 has no kernel here");
    }
    return ACLNN_SUCCESS;
}

aclnnStatus aclnnDynamicBlockQuantV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream)
{
    return aclnnDynamicBlockQuant(workspace, workspaceSize, executor, stream);
}

aclnnStatus aclnnDynamicBlockQuant(void*, uint64_t, aclOpExecutor* executor, aclrtStream stream)
{
    clear_error();
    if (!executor) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: executor is null", kApi);
    if (!executor_claim(executor)) INVALID("%s: executor is not valid (already run or destroyed)", kApi);
    std::unique_ptr<aclOpExecutor> ex(executor);
    ex->magic = 0;
    if (ex->kind != OpKind::BlockQuant) INVALID("%s: executor belongs to another operator", kApi);
    if (!ex->blkq.x || !ex->blkq.y || !ex->blkq.scale) INVALID("%s: a tensor has no device address", kApi);
    const int rc = opsnnDynamicBlockQuant(&ex->blkq, stream);
    if (rc != 0) FAIL(rc < 0 ? ACLNN_ERR_INNER_TILING_ERROR : ACLNN_ERR_RUNTIME_ERROR, "%s: launch failed with code %d", kApi, rc);
    return ACLNN_SUCCESS;
}

}  // extern "C"
