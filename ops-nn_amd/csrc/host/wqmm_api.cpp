// aclnnWeightQuantBatchMatmulV2 / V3: validation and routing to the weight-only HIP launcher.
//
// Behaviour (status codes, rule order, carrier re-tagging, stride-derived transposition) follows
//   matmul/weight_quant_batch_matmul_v2/op_host/op_api/aclnn_weight_quant_batch_matmul_v2.cpp
// for the reference's newest SoC generation.  Phase 1 never touches tensor data and never calls HIP.
#include <algorithm>
#include <cstring>
#include <initializer_list>
#include <memory>

#include "aclnnop/aclnn_weight_quant_batch_matmul_v2.h"
#include "aclnnop/aclnn_weight_quant_batch_matmul_v3.h"
#include "aclnnop/aclnn_weight_quant_batch_matmul_nz.h"
#include "launch.h"
#include "tensor.h"

using namespace opsnn;

namespace {

bool in_list(aclDataType d, std::initializer_list<aclDataType> l) { return std::find(l.begin(), l.end(), d) != l.end(); }
int64_t ceil_div(int64_t a, int64_t b) { return b ? (a + b - 1) / b : 0; }

#define FAIL(code, ...)         \
    do {                        \
        set_error(__VA_ARGS__); \
        return (code);          \
    } while (0)
#define INVALID(...) FAIL(ACLNN_ERR_PARAM_INVALID, __VA_ARGS__)

bool is_nz(aclFormat f)
{
    return f == ACL_FORMAT_FRACTAL_NZ || f == ACL_FORMAT_FRACTAL_NZ_C0_16 || f == ACL_FORMAT_FRACTAL_NZ_C0_32;
}

// aclnn_weight_quant_batch_matmul_v2.cpp:1156-1169: exactly 2-D with strides (1, shape[-2]).
bool is_trans_2d(const TView& t) { return t.rank() == 2 && t.stride(-2) == 1 && t.stride(-1) == t.dim(-2); }

aclnnStatus get_workspace(const char* api, const aclTensor* x_, const aclTensor* w_, const aclTensor* scale_,
                          const aclTensor* offset_, const aclTensor* qscale_, const aclTensor* qoffset_,
                          const aclTensor* bias_, int group, int innerPrecise, const aclTensor* y_,
                          uint64_t* workspaceSize, aclOpExecutor** executor)
{
    clear_error();
    if (log_enabled()) fprintf(stderr, "[opsnn] %s group=%d innerPrecise=%d\n", api, group, innerPrecise);
    // :841-849, 863-873
    if (!x_ || !w_ || !scale_ || !y_) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: x, weight, antiquantScale and y must not be null", api);
    if (!workspaceSize || !executor) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: workspaceSize/executor is null", api);
    if (qscale_ || qoffset_) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: quantScaleOptional and quantOffsetOptional must be null", api);
    if (w_->format != ACL_FORMAT_ND) INVALID("%s: weight must be in ND format%s", api, is_nz(w_->format) ? " (FRACTAL_NZ is not supported here)" : "");
    if (innerPrecise != 0 && innerPrecise != 1) INVALID("%s: innerPrecise must be 0 or 1, got %d", api, innerPrecise);

    TView x = make_view(x_), w = make_view(w_), sc = make_view(scale_), off = make_view(offset_), bias = make_view(bias_),
          y = make_view(y_);

    // ContiguousCheck :1213-1262
    bool tX = is_transposed_last2(x);
    if (!tX && !is_contiguous(x)) INVALID("%s: x must be contiguous or a last-two-dims transposed view", api);
    bool tW = is_transposed_last2(w);
    if (!tW && !is_contiguous(w)) INVALID("%s: weight must be contiguous or a last-two-dims transposed view", api);
    auto consistent = [&](const TView& t) {
        if (!t.present || t.rank() != 2 || (t.dim(0) == 1 && t.dim(1) == 1)) return true;
        return (tW && is_trans_2d(t)) || (!tW && is_contiguous(t));
    };
    if (!consistent(sc)) INVALID("%s: antiquantScale layout is not consistent with weight (transposed=%d)", api, (int)tW);
    if (!consistent(off)) INVALID("%s: antiquantOffsetOptional layout is not consistent with weight (transposed=%d)", api, (int)tW);
    if (!is_contiguous(y)) INVALID("%s: y must be contiguous", api);
    if (bias.present && !is_contiguous(bias)) INVALID("%s: biasOptional must be contiguous", api);

    // carrier re-tagging :1482-1576
    if (w.dtype == ACL_INT32 || w.dtype == ACL_FLOAT) {
        if (w.rank() != 2) INVALID("%s: weight must be 2-D, got %ldD", api, (long)w.rank());
        bool fp = w.dtype == ACL_FLOAT;
        if (tW) { w.shape[0] *= 8; w.strides[1] *= 8; }
        else { w.shape[1] *= 8; w.strides[0] *= 8; }
        w.offset *= 8;
        w.dtype = fp ? ACL_FLOAT4_E2M1 : ACL_INT4;
        if (fp && sc.dtype == ACL_UINT8) sc.dtype = ACL_FLOAT8_E8M0;
    }

    // dtypes :79-86, 1039-1071
    if (!in_list(x.dtype, {ACL_FLOAT16, ACL_BF16})) INVALID("%s: x must be FLOAT16 or BF16, got %s", api, dtype_name(x.dtype));
    if (!in_list(w.dtype, {ACL_INT8, ACL_INT4, ACL_FLOAT8_E4M3FN, ACL_HIFLOAT8, ACL_FLOAT4_E2M1}))
        INVALID("%s: weight dtype %s not supported", api, dtype_name(w.dtype));
    if (!in_list(sc.dtype, {ACL_FLOAT16, ACL_BF16, ACL_FLOAT8_E8M0})) INVALID("%s: antiquantScale dtype %s not supported", api, dtype_name(sc.dtype));
    if (!in_list(y.dtype, {ACL_FLOAT16, ACL_BF16})) INVALID("%s: y dtype %s not supported", api, dtype_name(y.dtype));
    if (y.dtype != x.dtype) INVALID("%s: y dtype %s must equal x dtype %s", api, dtype_name(y.dtype), dtype_name(x.dtype));
    // ranks :1101-1113
    if (x.rank() != 2 || w.rank() != 2 || y.rank() != 2) INVALID("%s: x, weight and y must be 2-D", api);
    if (bias.present && (bias.rank() < 1 || bias.rank() > 2)) INVALID("%s: biasOptional must be 1-D or 2-D", api);
    if (sc.rank() < 1 || sc.rank() > 2) INVALID("%s: antiquantScale must be 1-D or 2-D", api);
    if (off.present && (off.rank() < 1 || off.rank() > 2)) INVALID("%s: antiquantOffsetOptional must be 1-D or 2-D", api);

    const bool w_f4 = w.dtype == ACL_FLOAT4_E2M1, w_f8 = in_list(w.dtype, {ACL_FLOAT8_E4M3FN, ACL_HIFLOAT8});
    const bool mx = sc.dtype == ACL_FLOAT8_E8M0;
    // offset / scale dtype rules :875-966
    if (off.present && off.dtype == ACL_INT32) INVALID("%s: INT32 antiquantOffsetOptional is not supported", api);
    if (!mx && sc.dtype != x.dtype) INVALID("%s: antiquantScale dtype %s must equal x dtype %s", api, dtype_name(sc.dtype), dtype_name(x.dtype));
    if ((w_f4 || w_f8) && off.present) INVALID("%s: antiquantOffsetOptional must be null for %s weights", api, dtype_name(w.dtype));
    if (off.present && off.dtype != sc.dtype) INVALID("%s: antiquantOffsetOptional dtype must equal antiquantScale dtype", api);
    // bias dtype :968-1020
    if (bias.present) {
        if (x.dtype == ACL_FLOAT16 && bias.dtype != ACL_FLOAT16) INVALID("%s: biasOptional must be FLOAT16 when x is FLOAT16", api);
        if (x.dtype == ACL_BF16) {
            if ((w_f4 || w_f8) && bias.dtype != ACL_BF16) INVALID("%s: biasOptional must be BF16 for %s weights", api, dtype_name(w.dtype));
            if (!in_list(bias.dtype, {ACL_BF16, ACL_FLOAT})) INVALID("%s: biasOptional must be BF16 or FLOAT when x is BF16", api);
        }
        if (bias.format != ACL_FORMAT_ND) INVALID("%s: biasOptional must be ND", api);
    }
    if (x.format != ACL_FORMAT_ND || sc.format != ACL_FORMAT_ND || (off.present && off.format != ACL_FORMAT_ND)) INVALID("%s: tensors must be ND", api);

    // shapes :461-576 (the view of weight is always logical [k, n])
    const int64_t M = tX ? x.dim(1) : x.dim(0), Kx = tX ? x.dim(0) : x.dim(1);
    const int64_t K = w.dim(0), N = w.dim(1);
    if (Kx != K) INVALID("%s: K of x (%ld) and weight (%ld) differ", api, (long)Kx, (long)K);
    if (M < 1 || K < 1 || N < 1) INVALID("%s: M, K and N must be at least 1", api);
    if (in_list(w.dtype, {ACL_INT4, ACL_FLOAT4_E2M1})) {
        if (tW && (K % 2)) INVALID("%s: K must be even for 4-bit transposed weight", api);
        if (!tW && (N % 2)) INVALID("%s: N must be even for 4-bit weight", api);
    }
    if (y.dim(0) != M || y.dim(1) != N) INVALID("%s: y shape must be [%ld, %ld]", api, (long)M, (long)N);

    // group size and scale shape :251-400, 735-791
    if (group != 0 && (group % 32 != 0 || group < 32 || group > K - 1)) INVALID("%s: antiquantGroupSize %d must be 0 or a multiple of 32 in [32, K-1]", api, group);
    if (w_f4 && mx) {
        if (group != 32) INVALID("%s: antiquantGroupSize must be 32 for mxfp4 weights", api);
    } else if (w_f4 && group <= 0) {
        INVALID("%s: FLOAT4 weights need a positive antiquantGroupSize", api);
    }
    if (w_f8) {
        if (mx) INVALID("%s: FLOAT8_E8M0 antiquantScale is not supported for fp8 weights", api);
        if (group != 0) INVALID("%s: fp8 weights support per-channel only (antiquantGroupSize 0)", api);
    }
    if (mx && !w_f4) INVALID("%s: FLOAT8_E8M0 antiquantScale needs FLOAT4_E2M1 weights", api);
    int64_t scale_n = N, G = 1;
    auto check_qshape = [&](const TView& t, const char* name) -> aclnnStatus {
        if (t.rank() == 1) {
            if (group != 0) INVALID("%s: %s must be 2-D in per-group mode", api, name);
            if (t.dim(0) != 1 && t.dim(0) != N) INVALID("%s: %s length %ld must be 1 or N %ld", api, name, (long)t.dim(0), (long)N);
            return ACLNN_SUCCESS;
        }
        int64_t g = t.dim(0), n = t.dim(1);  // logical [G, N] view (strides carry the transposition)
        if (group == 0) {
            if (!((g == 1 && n == N) || (g == 1 && n == 1))) INVALID("%s: %s shape must be [1, N] or [1, 1] without groups", api, name);
        } else if (g != ceil_div(K, group) || n != N) {
            INVALID("%s: %s shape must be [%ld, %ld] in per-group mode, got [%ld, %ld]", api, name, (long)ceil_div(K, group), (long)N, (long)g, (long)n);
        }
        return ACLNN_SUCCESS;
    };
    aclnnStatus rc;
    if ((rc = check_qshape(sc, "antiquantScale")) != ACLNN_SUCCESS) return rc;
    if (off.present) {
        if ((rc = check_qshape(off, "antiquantOffsetOptional")) != ACLNN_SUCCESS) return rc;
        if (off.shape != sc.shape) INVALID("%s: antiquantOffsetOptional shape must equal antiquantScale shape", api);
    }
    if (sc.numel() == 1) scale_n = 1;
    if (group > 0) G = ceil_div(K, group);
    if (w_f8 && scale_n == 1 && N != 1) INVALID("%s: fp8 weights do not support per-tensor scales", api);
    if (bias.present) {
        if (bias.rank() == 1 ? bias.dim(0) != N : (bias.dim(0) != 1 || bias.dim(1) != N)) INVALID("%s: biasOptional shape must be [N] or [1, N]", api);
    }
    // :1584-1590
    if (tX || !is_contiguous(x)) INVALID("%s: x must be contiguous and not transposed", api);
    if (w.dtype == ACL_HIFLOAT8) FAIL(ACLNN_ERR_INNER_TILING_ERROR, "%s: HIFLOAT8 weights have no kernel on this device", api);

    std::unique_ptr<aclOpExecutor> ex(new (std::nothrow) aclOpExecutor());
    if (!ex) FAIL(ACLNN_ERR_INNER_CREATE_EXECUTOR, "%s: cannot allocate executor", api);
    ex->api = "aclnnWeightQuantBatchMatmul";
    ex->kind = OpKind::Wqmm;
    OpsnnWqmmArgs& a = ex->wqmm;
    a.M = M; a.N = N; a.K = K;
    a.x = x.ptr_at(0); a.x_dtype = x.dtype;
    a.w.ptr = w.ptr_at(0); a.w.row_stride = w.stride(0); a.w.col_stride = w.stride(1); a.w_dtype = w.dtype;
    a.scale.ptr = sc.ptr_at(0); a.scale_dtype = sc.dtype; a.scale_n = scale_n;
    if (sc.rank() == 2) { a.scale.row_stride = sc.stride(0); a.scale.col_stride = sc.stride(1); }
    else { a.scale.row_stride = 0; a.scale.col_stride = 1; }
    if (scale_n == 1) { a.scale.row_stride = 0; a.scale.col_stride = 0; }
    if (G == 1) a.scale.row_stride = 0;
    a.offset = off.present ? off.ptr_at(0) : nullptr;
    a.group = mx ? 32 : group;
    a.bias = bias.present ? bias.ptr_at(0) : nullptr; a.bias_dtype = bias.dtype;
    a.y = const_cast<void*>(y.ptr_at(0));
    ex->workspace_size = opsnnWqmmWorkspace(&a);
    *workspaceSize = ex->workspace_size;
    *executor = (aclOpExecutor*)executor_publish(ex.release());
    return ACLNN_SUCCESS;
}

aclnnStatus run(const char* api, void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream)
{
    clear_error();
    if (!executor) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: executor is null", api);
    if (!executor_claim(executor)) INVALID("%s: executor is not valid (already run or destroyed)", api);
    std::unique_ptr<aclOpExecutor> ex(executor);
    ex->magic = 0;
    if (ex->kind == OpKind::None) return ACLNN_SUCCESS;
    if (ex->kind != OpKind::Wqmm) INVALID("%s: executor belongs to another operator", api);
    if (ex->workspace_size > 0 && (!workspace || workspaceSize < ex->workspace_size))
        INVALID("%s: workspace of %lu bytes required", api, (unsigned long)ex->workspace_size);
    ex->wqmm.workspace = ex->workspace_size ? workspace : nullptr;
    if (!ex->wqmm.x || !ex->wqmm.w.ptr || !ex->wqmm.y || !ex->wqmm.scale.ptr) INVALID("%s: a tensor has no device address", api);
    // a FRACTAL_NZ weight is re-written into the workspace on every call: an address the weight cache must not key on
    WeightCacheScope cache_scope(ex->nz.active);
    if (ex->nz.active) {   // weight arrived in FRACTAL_NZ (aclnnWeightQuantBatchMatmulNz): lay it out as ND in the front of the workspace
        const void* nd = nullptr;
        void* rest = nullptr;
        const int nrc = run_nz_step(*ex, workspace, stream, &nd, &rest);
        if (nrc != 0) FAIL(ACLNN_ERR_RUNTIME_ERROR, "%s: FRACTAL_NZ re-layout failed with code %d", api, nrc);
        ex->wqmm.w.ptr = nd;
        ex->wqmm.workspace = ex->workspace_size > nz_front_bytes(*ex) ? rest : nullptr;
    }
    int rc = opsnnWqmm(&ex->wqmm, stream);
    if (rc != 0) FAIL(rc < 0 ? ACLNN_ERR_INNER_TILING_ERROR : ACLNN_ERR_RUNTIME_ERROR, "%s: launch failed with code %d", api, rc);
    return ACLNN_SUCCESS;
}

}  // namespace

extern "C" {

aclnnStatus aclnnWeightQuantBatchMatmulV2GetWorkspaceSize(const aclTensor* x, const aclTensor* weight,
                                                          const aclTensor* antiquantScale,
                                                          const aclTensor* antiquantOffsetOptional,
                                                          const aclTensor* quantScaleOptional,
                                                          const aclTensor* quantOffsetOptional,
                                                          const aclTensor* biasOptional, int antiquantGroupSize,
                                                          const aclTensor* y, uint64_t* workspaceSize,
                                                          aclOpExecutor** executor)
{
    return get_workspace("aclnnWeightQuantBatchMatmulV2GetWorkspaceSize", x, weight, antiquantScale, antiquantOffsetOptional,
                         quantScaleOptional, quantOffsetOptional, biasOptional, antiquantGroupSize, 0, y, workspaceSize,
                         executor);
}

aclnnStatus aclnnWeightQuantBatchMatmulV2(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                          aclrtStream stream)
{
    return run("aclnnWeightQuantBatchMatmulV2", workspace, workspaceSize, executor, stream);
}

aclnnStatus aclnnWeightQuantBatchMatmulV3GetWorkspaceSize(const aclTensor* x, const aclTensor* weight,
                                                          const aclTensor* antiquantScale,
                                                          const aclTensor* antiquantOffsetOptional,
                                                          const aclTensor* quantScaleOptional,
                                                          const aclTensor* quantOffsetOptional,
                                                          const aclTensor* biasOptional, int antiquantGroupSize,
                                                          int innerPrecise, const aclTensor* y,
                                                          uint64_t* workspaceSize, aclOpExecutor** executor)
{
    return get_workspace("aclnnWeightQuantBatchMatmulV3GetWorkspaceSize", x, weight, antiquantScale, antiquantOffsetOptional,
                         quantScaleOptional, quantOffsetOptional, biasOptional, antiquantGroupSize, innerPrecise, y,
                         workspaceSize, executor);
}

aclnnStatus aclnnWeightQuantBatchMatmulV3(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                          aclrtStream stream)
{
    return run("aclnnWeightQuantBatchMatmulV3", workspace, workspaceSize, executor, stream);
}

// aclnnWeightQuantBatchMatmulNz (aclnn_weight_quant_batch_matmul_nz.h:38-54): the V2 operator with the weight handed over
// in FRACTAL_NZ, as aclnnConvertWeightToINT4Pack produces it for 4-bit weights ([ceil(n/16), ceil(k/16), 16, 16] elements,
// or 32 in the last dimension; INT32 / FLOAT carriers: 2 or 4) and the format cast produces it for INT8
// ([ceil(n/32), ceil(k/16), 16, 32]).  Everything else -- argument rules, quantisation modes, results -- is V2's.  The
// weight is laid out as the dense ND matrix once per call, into the front of the workspace.
aclnnStatus aclnnWeightQuantBatchMatmulNzGetWorkspaceSize(const aclTensor* x, const aclTensor* weight,
                                                          const aclTensor* antiquantScale,
                                                          const aclTensor* antiquantOffsetOptional,
                                                          const aclTensor* quantScaleOptional,
                                                          const aclTensor* quantOffsetOptional,
                                                          const aclTensor* biasOptional, int antiquantGroupSize,
                                                          const aclTensor* y, uint64_t* workspaceSize,
                                                          aclOpExecutor** executor)
{
    const char* api = "aclnnWeightQuantBatchMatmulNzGetWorkspaceSize";
    clear_error();
    if (!weight) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: weight is null", api);
    if (!workspaceSize || !executor) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: workspaceSize/executor is null", api);
    if (!is_nz(weight->format)) INVALID("%s: weight must be in FRACTAL_NZ format (aclnn_weight_quant_batch_matmul_v2.cpp:1836-1839)", api);
    aclOpExecutorImpl::NzStep step;
    if (!describe_nz_operand(api, "weight", weight, &step)) return ACLNN_ERR_PARAM_INVALID;
    aclTensor nd = *weight;   // the same view over the dense ND matrix the pre-step will write
    nd.format = ACL_FORMAT_ND;
    nd.storage = nd.view;
    uint64_t inner = 0;
    aclOpExecutor* ex = nullptr;
    const aclnnStatus rc = get_workspace(api, x, &nd, antiquantScale, antiquantOffsetOptional, quantScaleOptional, quantOffsetOptional,
                                         biasOptional, antiquantGroupSize, 0, y, &inner, &ex);
    if (rc != ACLNN_SUCCESS) return rc;
    if (ex->kind != OpKind::None) {
        ex->nz = step;
        ex->workspace_size = nz_front_bytes(*ex) + inner;
    }
    *workspaceSize = ex->workspace_size;
    *executor = ex;
    return ACLNN_SUCCESS;
}

aclnnStatus aclnnWeightQuantBatchMatmulNz(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream)
{
    return run("aclnnWeightQuantBatchMatmulNz", workspace, workspaceSize, executor, stream);
}

}  // extern "C"
