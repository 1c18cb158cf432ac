// aclnnConvertWeightToINT4Pack: validation in the reference's rule order, then the device pack kernel.
//
// Behaviour follows matmul/convert_weight_to_int4_pack/op_host/op_api/aclnn_convert_weight_to_int4_pack.cpp:
// ParamsCheck :305-314 (null, contiguous, dtype pair, format, dims, shape), conversion in the first call :368-405, an
// empty second call :407-411.  The reference copies the weight to the host, packs it there and copies it back; here
// the first call launches opsnnPackB4 on the null stream and waits, so the result is equally in place on return.
#include <algorithm>
#include <initializer_list>

#include <hip/hip_runtime_api.h>

#include "aclnnop/aclnn_convert_weight_to_int4_pack.h"
#include "tensor.h"

using namespace opsnn;

namespace {

constexpr const char* kApi = "aclnnConvertWeightToINT4Pack";

#define FAIL(code, ...)         \
    do {                        \
        set_error(__VA_ARGS__); \
        return (code);          \
    } while (0)
#define INVALID(...) FAIL(ACLNN_ERR_PARAM_INVALID, __VA_ARGS__)

bool in_list(aclDataType d, std::initializer_list<aclDataType> l) { return std::find(l.begin(), l.end(), d) != l.end(); }

}  // namespace

extern "C" {

aclnnStatus aclnnConvertWeightToINT4PackGetWorkspaceSize(const aclTensor* weight_, aclTensor* pack_, uint64_t* workspaceSize,
                                                         aclOpExecutor** executor)
{
    clear_error();
    if (!weight_ || !pack_) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: weight and weightInt4Pack must not be null", kApi);   // :148-153
    const TView w = make_view(weight_), p = make_view(pack_);
    if (!is_contiguous(w) || !is_contiguous(p)) INVALID("%s: weight and weightInt4Pack must be contiguous", kApi);   // :155-162
    // dtype pairs :164-182
    if (!in_list(w.dtype, {ACL_INT32, ACL_FLOAT})) INVALID("%s: weight must be INT32 or FLOAT, got %s", kApi, dtype_name(w.dtype));
    if (!in_list(p.dtype, {ACL_INT4, ACL_INT32, ACL_FLOAT4_E2M1, ACL_FLOAT}))
        INVALID("%s: weightInt4Pack must be INT4, INT32, FLOAT4_E2M1 or FLOAT, got %s", kApi, dtype_name(p.dtype));
    const bool fp = w.dtype == ACL_FLOAT;
    if ((!fp && !in_list(p.dtype, {ACL_INT32, ACL_INT4})) || (fp && !in_list(p.dtype, {ACL_FLOAT, ACL_FLOAT4_E2M1})))
        INVALID("%s: weight %s goes with weightInt4Pack %s, got %s", kApi, dtype_name(w.dtype), fp ? "FLOAT or FLOAT4_E2M1" : "INT32 or INT4",
                dtype_name(p.dtype));
    // formats :184-189
    if (w.format != ACL_FORMAT_ND) INVALID("%s: weight must be in ND format", kApi);
    const bool nz_out = p.format == ACL_FORMAT_FRACTAL_NZ || p.format == ACL_FORMAT_FRACTAL_NZ_C0_16 || p.format == ACL_FORMAT_FRACTAL_NZ_C0_32;
    if (p.format != ACL_FORMAT_ND && !nz_out) INVALID("%s: weightInt4Pack must be in ND or FRACTAL_NZ format", kApi);
    // dims :191-197
    if (w.rank() < 2 || w.rank() > 3) INVALID("%s: weight must have 2 or 3 dims, got %ld", kApi, (long)w.rank());
    if (p.rank() < 2 || p.rank() > 3) INVALID("%s: weightInt4Pack must have 2 or 3 dims, got %ld", kApi, (long)p.rank());
    // shapes :246-296 (the last two dims only, as there)
    const int64_t wf = w.dim(-2), wl = w.dim(-1), pf = p.dim(-2), pl = p.dim(-1);
    if (is_4bit(p.dtype)) {
        if (wl % 2 != 0) INVALID("%s: the last dim of weight must be even for a 4-bit weightInt4Pack, got %ld", kApi, (long)wl);
        if (wf != pf || wl != pl)
            INVALID("%s: weightInt4Pack %s must have weight's shape %s", kApi, shape_str(p.shape).c_str(), shape_str(w.shape).c_str());
    } else {
        if (wl % 8 != 0) INVALID("%s: the last dim of weight must be a multiple of 8 for a 32-bit weightInt4Pack, got %ld", kApi, (long)wl);
        if (wf != pf || wl / 8 != pl)
            INVALID("%s: weightInt4Pack %s must be weight's shape %s with the last dim divided by 8", kApi, shape_str(p.shape).c_str(),
                    shape_str(w.shape).c_str());
    }
    // The reference sizes its buffers from weight alone (:380-390); a leading dim that differs would overrun the output here.
    if (w.rank() != p.rank() || (w.rank() == 3 && w.dim(0) != p.dim(0)))
        INVALID("%s: weight %s and weightInt4Pack %s differ in their leading dim", kApi, shape_str(w.shape).c_str(), shape_str(p.shape).c_str());
    // FRACTAL_NZ output: storage [ceil(n / c0), ceil(k / 16), 16, c0] of the packed [k, n] matrix (:205-250, 318-366)
    aclOpExecutorImpl::NzStep nz;
    if (nz_out && !describe_nz_operand(kApi, "weightInt4Pack", pack_, &nz)) return ACLNN_ERR_PARAM_INVALID;
    if (workspaceSize) *workspaceSize = 0;
    if (executor) *executor = nullptr;
    const int64_t count = w.numel();
    if (count == 0) return ACLNN_SUCCESS;
    if (!w.data || !p.data) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: tensor without device memory", kApi);
    const void* src = w.ptr_at(0);
    void* dst = const_cast<void*>(p.ptr_at(0));
    if ((uintptr_t)src % 16 != 0 || (uintptr_t)dst % 8 != 0) INVALID("%s: weight must be 16-byte and weightInt4Pack 8-byte aligned", kApi);
    if (nz_out) {
        // pack into a temporary ND buffer, then write the fractals (zero padding included).  This operator is the offline
        // weight preparation (the reference does it on the host inside this very call), so it may allocate.
        void* tmp = nullptr;
        hipError_t e = hipMalloc(&tmp, (size_t)count / 2);
        if (e != hipSuccess) FAIL(ACLNN_ERR_RUNTIME_ERROR, "%s: cannot allocate %ld bytes for the ND intermediate: %s", kApi, (long)(count / 2), hipGetErrorString(e));
        int rc = opsnnPackB4(src, fp ? 1 : 0, tmp, count, nullptr);
        if (rc == 0) rc = opsnnNdToNz(tmp, dst, nz.rows, nz.row_bytes, nz.c0, nz.batch, nullptr);
        e = hipStreamSynchronize(nullptr);
        (void)hipFree(tmp);
        if (rc != 0) FAIL(ACLNN_ERR_RUNTIME_ERROR, "%s: kernel launch failed (%d)", kApi, rc);
        if (e != hipSuccess) FAIL(ACLNN_ERR_RUNTIME_ERROR, "%s: %s", kApi, hipGetErrorString(e));
        return ACLNN_SUCCESS;
    }
    const int rc = opsnnPackB4(src, fp ? 1 : 0, dst, count, nullptr);
    if (rc != 0) FAIL(ACLNN_ERR_RUNTIME_ERROR, "%s: kernel launch failed (%d)", kApi, rc);
    const hipError_t e = hipStreamSynchronize(nullptr);
    if (e != hipSuccess) FAIL(ACLNN_ERR_RUNTIME_ERROR, "%s: %s", kApi, hipGetErrorString(e));
    return ACLNN_SUCCESS;
}

aclnnStatus aclnnConvertWeightToINT4Pack(void*, uint64_t, aclOpExecutor*, aclrtStream) { return ACLNN_SUCCESS; }

}  // extern "C"
