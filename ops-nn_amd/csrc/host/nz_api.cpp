// FRACTAL_NZ right operands: the shared phase-1 shape check and phase-2 pre-step, and aclnnQuantMatmulWeightNz.
//
// The reference keeps the right operand of its cube unit in a fractal layout and has entry points that take it in that
// form (matmul/quant_batch_matmul_v3/op_api/aclnn_quant_matmul_weight_nz.h:41,
// matmul/weight_quant_batch_matmul_v2/op_host/op_api/aclnn_weight_quant_batch_matmul_nz.h:38-54).  Here the kernels
// stream K-contiguous rows, so an NZ operand is laid out as the dense ND matrix first (opsnnNzToNd) and the ND operator
// does the rest.
#include <cstdio>
#include <memory>

#include "aclnnop/aclnn_quant_matmul_v5.h"
#include "aclnnop/aclnn_quant_matmul_weight_nz.h"
#include "tensor.h"

namespace opsnn {

#define NZ_FAIL(...)            \
    do {                        \
        set_error(__VA_ARGS__); \
        return false;           \
    } while (0)

bool describe_nz_operand(const char* api, const char* name, const aclTensor* t, aclOpExecutorImpl::NzStep* step)
{
    const TView v = make_view(t);
    if (v.rank() < 2) NZ_FAIL("%s: %s must have at least two dimensions", api, name);
    if (v.offset != 0) NZ_FAIL("%s: a FRACTAL_NZ %s must start at its storage (view offset 0)", api, name);
    const int bits = dtype_bits(v.dtype);
    if (bits != 4 && bits != 8 && bits != 32) NZ_FAIL("%s: %s dtype %s has no FRACTAL_NZ form here", api, name, dtype_name(v.dtype));
    const bool transposed = is_transposed_last2(v);
    if (!transposed && !is_contiguous(v)) NZ_FAIL("%s: a FRACTAL_NZ %s must be a dense view or its last-two-dims transpose", api, name);
    const int64_t rows = transposed ? v.dim(-1) : v.dim(-2), cols = transposed ? v.dim(-2) : v.dim(-1);
    int64_t batch = 1;
    for (int64_t i = 0; i + 2 < v.rank(); i++) batch *= v.dim(i);
    const std::vector<int64_t>& st = t->storage;
    if (st.size() < 4) NZ_FAIL("%s: the storage shape of a FRACTAL_NZ %s must have at least four dimensions, got %s", api, name, shape_str(st).c_str());
    const size_t n = st.size();
    const int64_t x1 = st[n - 4], y1 = st[n - 3], m0 = st[n - 2], c0e = st[n - 1];
    int64_t sbatch = 1;
    for (size_t i = 0; i + 4 < n; i++) sbatch *= st[i];
    const int64_t c0_bytes = c0e * bits / 8;
    if (m0 != 16 || (c0_bytes != 8 && c0_bytes != 16 && c0_bytes != 32) || c0e * bits % 8 != 0)
        NZ_FAIL("%s: FRACTAL_NZ storage shape %s of %s: the last two dimensions must be 16 and 8, 16 or 32 bytes of elements", api, shape_str(st).c_str(), name);
    if (x1 != (cols + c0e - 1) / c0e || y1 != (rows + 15) / 16 || sbatch != batch)
        NZ_FAIL("%s: FRACTAL_NZ storage shape %s of %s does not match the stored matrix [%ld x %ld x %ld]: expected [.., %ld, %ld, 16, %ld]", api,
                shape_str(st).c_str(), name, (long)batch, (long)rows, (long)cols, (long)((cols + c0e - 1) / c0e), (long)((rows + 15) / 16), (long)c0e);
    if ((cols * bits) % 8 != 0) NZ_FAIL("%s: the rows of %s must be whole bytes", api, name);
    step->active = true;
    step->src = t->data;
    step->rows = rows;
    step->row_bytes = cols * bits / 8;
    step->batch = batch;
    step->c0 = (int)c0_bytes;
    step->nd_bytes = (uint64_t)batch * (uint64_t)rows * (uint64_t)step->row_bytes;
    return true;
}

int run_nz_step(const aclOpExecutorImpl& ex, void* workspace, void* stream, const void** nd_ptr, void** rest)
{
    if (!ex.nz.active || !workspace || !ex.nz.src) return -1;
    const int rc = opsnnNzToNd(ex.nz.src, workspace, ex.nz.rows, ex.nz.row_bytes, ex.nz.c0, ex.nz.batch, stream);
    *nd_ptr = workspace;
    *rest = (char*)workspace + nz_front_bytes(ex);
    return rc;
}

}  // namespace opsnn

using namespace opsnn;

extern "C" aclnnStatus aclnnQuantMatmulWeightNzGetWorkspaceSize(const aclTensor* x1, const aclTensor* x2, const aclTensor* x1Scale,
                                                                const aclTensor* x2Scale, const aclTensor* yScale,
                                                                const aclTensor* x1Offset, const aclTensor* x2Offset,
                                                                const aclTensor* yOffset, const aclTensor* bias, bool transposeX1,
                                                                bool transposeX2, int64_t groupSize, aclTensor* out,
                                                                uint64_t* workspaceSize, aclOpExecutor** executor)
{
    const char* api = "aclnnQuantMatmulWeightNzGetWorkspaceSize";
    clear_error();
    if (!workspaceSize || !executor) { set_error("%s: workspaceSize/executor is null", api); return ACLNN_ERR_PARAM_NULLPTR; }
    if (!x2) { set_error("%s: x2 is null", api); return ACLNN_ERR_PARAM_NULLPTR; }
    const aclFormat f = x2->format;
    if (f != ACL_FORMAT_FRACTAL_NZ && f != ACL_FORMAT_FRACTAL_NZ_C0_16 && f != ACL_FORMAT_FRACTAL_NZ_C0_32) {
        set_error("%s: x2 must be in FRACTAL_NZ format; for ND use aclnnQuantMatmulV5", api);
        return ACLNN_ERR_PARAM_INVALID;
    }
    // (the reference: an original ND matrix with a dimension of 1 has no NZ form, aclnnQuantMatmulWeightNz.md:550)
    aclOpExecutorImpl::NzStep step;
    if (!describe_nz_operand(api, "x2", x2, &step)) return ACLNN_ERR_PARAM_INVALID;
    if (step.rows == 1 || step.row_bytes == 0) { set_error("%s: an x2 with a dimension of 1 has no FRACTAL_NZ form", api); return ACLNN_ERR_PARAM_INVALID; }
    aclTensor nd = *x2;   // the same view over the dense ND matrix the pre-step will write
    nd.format = ACL_FORMAT_ND;
    nd.storage = nd.view;
    uint64_t inner = 0;
    aclOpExecutor* ex = nullptr;
    const aclnnStatus rc = aclnnQuantMatmulV5GetWorkspaceSize(x1, &nd, x1Scale, x2Scale, yScale, x1Offset, x2Offset, yOffset, bias, transposeX1,
                                                              transposeX2, groupSize, out, &inner, &ex);
    if (rc != ACLNN_SUCCESS) return rc;
    if (!ex->batch_runs.empty()) {   // several launches with their own operand addresses: not combined with the NZ pre-step
        aclDestroyAclOpExecutor(ex);
        set_error("%s: batch dims that broadcast partially are not supported with a FRACTAL_NZ x2", api);
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (ex->kind != OpKind::None) {
        ex->nz = step;
        ex->workspace_size = nz_front_bytes(*ex) + inner;
        ex->api = "aclnnQuantMatmulWeightNz";
    }
    *workspaceSize = ex->workspace_size;
    *executor = ex;
    return ACLNN_SUCCESS;
}

extern "C" aclnnStatus aclnnQuantMatmulWeightNz(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream)
{
    return aclnnQuantMatmulV5(workspace, workspaceSize, executor, stream);
}
