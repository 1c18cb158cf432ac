// aclnnPrepackMatmulWeight: [k, n] (ND or FRACTAL_NZ) -> K-contiguous [n, k], with the scales that run along k.
// See include/aclnnop/aclnn_prepack_matmul_weight.h for what it replaces in the reference.
#include <algorithm>
#include <initializer_list>
#include <memory>

#include "aclnnop/aclnn_prepack_matmul_weight.h"
#include "tensor.h"

using namespace opsnn;

namespace {
constexpr const char* kApi = "aclnnPrepackMatmulWeight";
#define FAIL(code, ...)         \
    do {                        \
        set_error(__VA_ARGS__); \
        return (code);          \
    } while (0)
#define INVALID(...) FAIL(ACLNN_ERR_PARAM_INVALID, __VA_ARGS__)
bool in_list(aclDataType d, std::initializer_list<aclDataType> l) { return std::find(l.begin(), l.end(), d) != l.end(); }
bool is_nz(aclFormat f) { return f == ACL_FORMAT_FRACTAL_NZ || f == ACL_FORMAT_FRACTAL_NZ_C0_16 || f == ACL_FORMAT_FRACTAL_NZ_C0_32; }
}  // namespace

extern "C" aclnnStatus aclnnPrepackMatmulWeightGetWorkspaceSize(const aclTensor* weight_, const aclTensor* scale_, aclTensor* packed_,
                                                                aclTensor* spacked_, uint64_t* workspaceSize, aclOpExecutor** executor)
{
    clear_error();
    if (!weight_ || !packed_) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: weight and weightPacked must not be null", kApi);
    if (!workspaceSize || !executor) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: workspaceSize/executor is null", kApi);
    if ((scale_ == nullptr) != (spacked_ == nullptr)) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: scaleOptional and scalePackedOptional go together", kApi);
    const TView w = make_view(weight_), p = make_view(packed_), s = make_view(scale_), sp = make_view(spacked_);
    if (!in_list(w.dtype, {ACL_INT8, ACL_FLOAT8_E4M3FN, ACL_FLOAT8_E5M2, ACL_INT4, ACL_FLOAT4_E2M1}))
        INVALID("%s: weight dtype %s not supported", kApi, dtype_name(w.dtype));
    if (p.dtype != w.dtype) INVALID("%s: weightPacked dtype %s must equal weight dtype %s", kApi, dtype_name(p.dtype), dtype_name(w.dtype));
    if (w.rank() < 2 || w.rank() > 6 || p.rank() != w.rank()) INVALID("%s: weight and weightPacked must have the same rank in 2..6", kApi);
    const bool nz = is_nz(w.format);
    if (!nz && w.format != ACL_FORMAT_ND) INVALID("%s: weight must be ND or FRACTAL_NZ", kApi);
    if (p.format != ACL_FORMAT_ND) INVALID("%s: weightPacked must be ND", kApi);
    if (!is_contiguous(w) || !is_contiguous(p)) INVALID("%s: weight and weightPacked must be dense", kApi);
    const int64_t k = w.dim(-2), n = w.dim(-1);
    if (p.dim(-2) != n || p.dim(-1) != k) INVALID("%s: weightPacked %s must be weight %s with the last two dims swapped", kApi, shape_str(p.shape).c_str(), shape_str(w.shape).c_str());
    int64_t batch = 1;
    for (int64_t i = 0; i + 2 < w.rank(); i++) {
        if (w.dim(i) != p.dim(i)) INVALID("%s: batch dims of weight and weightPacked differ", kApi);
        batch *= w.dim(i);
    }
    const int bits = dtype_bits(w.dtype);
    if (bits == 4 && ((k | n) & 1)) INVALID("%s: k and n must be even for 4-bit weights", kApi);
    if (batch > 65535) INVALID("%s: at most 65535 batches", kApi);

    std::unique_ptr<aclOpExecutor> ex(new (std::nothrow) aclOpExecutor());
    if (!ex) FAIL(ACLNN_ERR_INNER_CREATE_EXECUTOR, "%s: cannot allocate executor", kApi);
    ex->api = kApi;
    if (k == 0 || n == 0 || batch == 0) {   // nothing to move
        *workspaceSize = 0;
        *executor = (aclOpExecutor*)executor_publish(ex.release());
        return ACLNN_SUCCESS;
    }
    ex->kind = OpKind::Prepack;
    auto& pp = ex->prepack;
    pp.src = w.ptr_at(0); pp.dst = const_cast<void*>(p.ptr_at(0)); pp.k = k; pp.n = n; pp.batch = batch; pp.bits = bits;
    if (nz) {
        if (!describe_nz_operand(kApi, "weight", weight_, &ex->nz)) return ACLNN_ERR_PARAM_INVALID;
        ex->workspace_size = nz_front_bytes(*ex);   // the ND intermediate
    }
    if (scale_) {
        if (!is_contiguous(s) || !is_contiguous(sp)) INVALID("%s: the scales must be dense", kApi);
        if (sp.dtype != s.dtype) INVALID("%s: scalePackedOptional dtype must equal scaleOptional dtype", kApi);
        if (s.dtype == ACL_FLOAT8_E8M0) {   // [.., ceil(k/64), n, 2] -> [.., n, ceil(k/64), 2]
            const int64_t ks = (k + 63) / 64;
            if (s.rank() != w.rank() + 1 || sp.rank() != s.rank() || s.dim(-1) != 2 || sp.dim(-1) != 2 || s.dim(-3) != ks || s.dim(-2) != n ||
                sp.dim(-3) != n || sp.dim(-2) != ks)
                INVALID("%s: MX scales must be [.., %ld, %ld, 2] and [.., %ld, %ld, 2], got %s and %s", kApi, (long)ks, (long)n, (long)n, (long)ks,
                        shape_str(s.shape).c_str(), shape_str(sp.shape).c_str());
            int64_t sb = 1;
            for (int64_t i = 0; i + 3 < s.rank(); i++) sb *= s.dim(i);
            if (sb != batch) INVALID("%s: batch dims of the scale and the weight differ", kApi);
            pp.srows = ks; pp.scols = n; pp.sbatch = sb;
        } else if (s.dtype == ACL_FLOAT16 || s.dtype == ACL_BF16) {   // [G, n] -> [n, G]
            if (s.rank() != 2 || sp.rank() != 2 || s.dim(1) != n || sp.dim(0) != n || sp.dim(1) != s.dim(0) || batch != 1)
                INVALID("%s: group scales must be [G, %ld] and [%ld, G] with a 2-D weight, got %s and %s", kApi, (long)n, (long)n,
                        shape_str(s.shape).c_str(), shape_str(sp.shape).c_str());
            pp.srows = s.dim(0); pp.scols = n; pp.sbatch = 1;
        } else {
            INVALID("%s: scale dtype %s not supported (FLOAT8_E8M0, FLOAT16, BF16)", kApi, dtype_name(s.dtype));
        }
        pp.ssrc = s.ptr_at(0); pp.sdst = const_cast<void*>(sp.ptr_at(0));
    }
    *workspaceSize = ex->workspace_size;
    *executor = (aclOpExecutor*)executor_publish(ex.release());
    return ACLNN_SUCCESS;
}

extern "C" aclnnStatus aclnnPrepackMatmulWeight(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream)
{
    clear_error();
    if (!executor) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: executor is null", kApi);
    if (!executor_claim(executor)) INVALID("%s: executor is not valid (already run or destroyed)", kApi);
    std::unique_ptr<aclOpExecutor> ex(executor);
    ex->magic = 0;
    if (ex->kind == OpKind::None) return ACLNN_SUCCESS;
    if (ex->kind != OpKind::Prepack) INVALID("%s: executor belongs to another operator", kApi);
    if (ex->workspace_size > 0 && (!workspace || workspaceSize < ex->workspace_size)) INVALID("%s: workspace of %lu bytes required", kApi, (unsigned long)ex->workspace_size);
    auto& pp = ex->prepack;
    if (!pp.src || !pp.dst || (pp.ssrc && !pp.sdst)) INVALID("%s: a tensor has no device address", kApi);
    const void* src = pp.src;
    int rc = 0;
    if (ex->nz.active) {
        void* rest = nullptr;
        rc = run_nz_step(*ex, workspace, stream, &src, &rest);
        if (rc != 0) FAIL(ACLNN_ERR_RUNTIME_ERROR, "%s: FRACTAL_NZ re-layout failed with code %d", kApi, rc);
    }
    rc = pp.bits == 4 ? opsnnTranspose4(src, pp.dst, pp.k, pp.n, pp.batch, stream) : opsnnTranspose8(src, pp.dst, pp.k, pp.n, pp.batch, stream);
    if (rc == 0 && pp.ssrc) rc = opsnnTranspose16(pp.ssrc, pp.sdst, pp.srows, pp.scols, pp.sbatch, stream);
    if (rc != 0) FAIL(rc < 0 ? ACLNN_ERR_INNER_TILING_ERROR : ACLNN_ERR_RUNTIME_ERROR, "%s: launch failed with code %d", kApi, rc);
    return ACLNN_SUCCESS;
}
