// aclnnQuantMatmulV5: validation, quant-mode inference, routing to the HIP launchers.
//
// Behaviour (status codes, rule order, view normalisation) follows the reference for its newest
// SoC generation:
//   matmul/quant_batch_matmul_v4/op_host/op_api/aclnn_quant_matmul_v5.cpp      (entry, A8W4 checks, router)
//   matmul/quant_batch_matmul_v4/op_host/op_api/quant_matmul_common_check.cpp  (view normalisation)
//   matmul/quant_batch_matmul_v3/op_api/quant_matmul_checker.cpp               (dtype / shape tables)
// Phase 1 never touches tensor data and never calls HIP, so it runs without a GPU.
#include <algorithm>
#include <cstring>
#include <initializer_list>
#include <memory>

#include "aclnnop/aclnn_quant_matmul_v5.h"
#include "launch.h"
#include "tensor.h"

using namespace opsnn;

namespace {

constexpr const char* kApi = "aclnnQuantMatmulV5GetWorkspaceSize";
constexpr uint64_t kMask16 = 0xFFFF;

bool in_list(aclDataType d, std::initializer_list<aclDataType> l) { return std::find(l.begin(), l.end(), d) != l.end(); }
int64_t ceil_div(int64_t a, int64_t b) { return (a != 0 && b != 0) ? (a + b - 1) / b : a; }

#define FAIL(code, ...)                 \
    do {                                \
        set_error(__VA_ARGS__);         \
        return (code);                  \
    } while (0)
#define INVALID(...) FAIL(ACLNN_ERR_PARAM_INVALID, __VA_ARGS__)

bool is_nz(aclFormat f)
{
    return f == ACL_FORMAT_FRACTAL_NZ || f == ACL_FORMAT_FRACTAL_NZ_C0_16 || f == ACL_FORMAT_FRACTAL_NZ_C0_32;
}

struct Ctx {
    TView x1, x2, x1s, x2s, ys, x1o, x2o, yo, bias, out;
    bool tA = false, tB = false;
    int64_t groupSize = 0;
    int64_t M = 0, N = 0, K1 = 0, K2 = 0;

    bool int8_in() const { return x1.dtype == ACL_INT8 && x2.dtype == ACL_INT8; }
    bool int4_in() const { return x1.dtype == ACL_INT4 && x2.dtype == ACL_INT4; }
    bool hif8_in() const { return x1.dtype == ACL_HIFLOAT8 && x2.dtype == ACL_HIFLOAT8; }
    bool fp8_in() const
    {
        return in_list(x1.dtype, {ACL_FLOAT8_E4M3FN, ACL_FLOAT8_E5M2}) && in_list(x2.dtype, {ACL_FLOAT8_E4M3FN, ACL_FLOAT8_E5M2});
    }
    bool fp4_in() const { return x1.dtype == ACL_FLOAT4_E2M1 && x2.dtype == ACL_FLOAT4_E2M1; }
    bool mx() const { return x1s.present && x1s.dtype == ACL_FLOAT8_E8M0 && x2s.dtype == ACL_FLOAT8_E8M0; }
    bool a8w4f() const { return in_list(x1.dtype, {ACL_FLOAT8_E4M3FN, ACL_FLOAT8_E5M2}) && x2.dtype == ACL_FLOAT4_E2M1; }
    bool a8w4i_raw() const { return x1.dtype == ACL_INT8 && x2.dtype == ACL_INT32; }
    // quant_matmul_checker.cpp:293-303
    bool perblock() const
    {
        return x1s.present && (int8_in() || fp8_in() || hif8_in()) && x1s.dtype == ACL_FLOAT && x1s.rank() > 1 &&
               x2s.dtype == ACL_FLOAT && x2s.rank() > 1;
    }
    void refresh_dims()
    {
        if (x1.rank() >= 2 && x2.rank() >= 2) {
            K1 = tA ? x1.dim(-2) : x1.dim(-1);
            M = tA ? x1.dim(-1) : x1.dim(-2);
            K2 = tB ? x2.dim(-1) : x2.dim(-2);
            N = tB ? x2.dim(-2) : x2.dim(-1);
        }
    }
};

// A matrix operand whose view is neither dense nor a dense transpose, but regular: 8-bit elements, positive strides on
// the last two dims, and batch dims that collapse into one stride.  The reference makes such a view contiguous by a copy
// (quant_matmul_common_check.cpp:106-123); here the kernels take the strides of an 8-bit operand as they are (the
// matrix-core route gathers the operand into the workspace, the plain kernels index it directly), and a 4-bit operand is
// copied densely into the front of the workspace before anything else.
bool regular_strided_matrix(const TView& t)
{
    // 8-bit operands: the kernels take the strides; 4-bit operands (also in their INT32 carriers, whose eight elements per
    // word must stay together): gathered into a dense copy in front of the workspace by phase 2
    const int bits = dtype_bits(t.dtype);
    if (t.rank() < 2 || (bits != 8 && bits != 4 && t.dtype != ACL_INT32)) return false;
    if (t.dtype == ACL_INT32 && t.stride(-1) != 1) return false;
    if (bits == 4 && (t.dim(-1) % 2) != 0) return false;
    if (t.stride(-1) < 1 || t.stride(-2) < 1) return false;
    for (int64_t i = t.rank() - 4; i >= 0; i--)
        if (t.strides[(size_t)i] != t.strides[(size_t)i + 1] * t.shape[(size_t)i + 1]) return false;
    return t.rank() < 3 || t.stride(-3) >= 0;
}

// quant_matmul_common_check.cpp:106-123.  A last-two-dims-transposed view becomes a dense view of the
// swapped shape and flips the flag.  Other non-contiguous views are accepted for the two matrix operands when they are
// regular (see above) and rejected otherwise.
aclnnStatus contiguous_process(TView& t, bool& transpose, const char* name, bool matrix_operand = false)
{
    if (!t.present) return ACLNN_SUCCESS;
    if (t.rank() >= 2 && is_transposed_last2(t)) {
        swap_last2(t);
        transpose = !transpose;
        return ACLNN_SUCCESS;
    }
    if (is_contiguous(t)) return ACLNN_SUCCESS;
    if (matrix_operand && regular_strided_matrix(t)) return ACLNN_SUCCESS;
    INVALID("%s: %s has strides that are neither dense nor a last-two-dims transpose", kApi, name);
}

// aclnn_quant_matmul_v5.cpp:908-945: an MX scale [.., a, b, 2] whose strides describe [.., b, a, 2].
aclnnStatus mx_scale_process(TView& t, const char* name)
{
    if (!t.present || t.rank() < 3) return ACLNN_SUCCESS;
    int64_t r = t.rank();
    int64_t last = t.dim(-1), second = t.dim(-2), third = t.dim(-3);
    bool flag = false;
    if (t.stride(-3) == last && t.stride(-2) == last * third) {
        flag = true;
        int64_t expect = last * second * third;
        for (int64_t b = r - 4; b >= 0; b--) {
            if (t.strides[(size_t)b] != expect) { flag = false; break; }
            expect *= t.shape[(size_t)b];
        }
        if (second == 1 && third == 1) flag = false;
    }
    if (flag) {
        std::swap(t.shape[(size_t)r - 2], t.shape[(size_t)r - 3]);
        std::swap(t.strides[(size_t)r - 2], t.strides[(size_t)r - 3]);
        // now dense in the swapped order
        return ACLNN_SUCCESS;
    }
    if (!is_contiguous(t)) INVALID("%s: %s has unsupported strides", kApi, name);
    return ACLNN_SUCCESS;
}

void retag_int32_as_int4(TView& t)
{
    if (t.dtype != ACL_INT32) return;
    t.shape.back() *= 8;
    for (size_t i = 0; i + 1 < t.strides.size(); i++) t.strides[i] *= 8;
    t.offset *= 8;
    t.dtype = ACL_INT4;
}

// ---- group size inference: quant_matmul_checker.cpp:597-722 ----
bool recalc_group(int64_t in_size, int64_t scale_size, uint64_t& g, const char* dim)
{
    if (scale_size == 0) { set_error("%s: scale extent along %s is 0", kApi, dim); return false; }
    if (g == 0) {
        if (in_size % scale_size != 0) {
            set_error("%s: groupSize along %s cannot be inferred: %ld is not divisible by %ld", kApi, dim, (long)in_size, (long)scale_size);
            return false;
        }
        g = (uint64_t)(in_size / scale_size);
    }
    return true;
}

bool a4w4_pergroup_nonsym(const Ctx& c, uint64_t gsK);

bool infer_group_size(const Ctx& c, int64_t& groupSize)
{
    if (!c.x1s.present || c.x1s.rank() < 2 || c.x2s.rank() < 2) return true;
    uint64_t gk = (uint64_t)groupSize & kMask16, gn = ((uint64_t)groupSize >> 16) & kMask16, gm = ((uint64_t)groupSize >> 32) & kMask16;
    bool mx = c.mx();
    int64_t inM = c.tA ? c.x1.dim(-1) : c.x1.dim(-2);
    int64_t inK = c.tA ? c.x1.dim(-2) : c.x1.dim(-1);
    int64_t inN = c.tB ? c.x2.dim(-2) : c.x2.dim(-1);
    int64_t sM, sK, sN;
    if (mx) {
        if (c.x1s.rank() < 3 || c.x2s.rank() < 3) return true;  // rank errors are reported by the shape checks
        int64_t b1 = c.x1s.rank() - 3, b2 = c.x2s.rank() - 3;
        sM = c.x1s.dim(b1 + (c.tA ? 1 : 0));
        sK = c.x1s.dim(b1 + (c.tA ? 0 : 1)) * 2;
        sN = c.x2s.dim(b2 + (c.tB ? 0 : 1));
        int64_t d0 = c.x2s.dim(b2), d1 = c.x2s.dim(b2 + 1);
        if ((d0 == 1 && d1 == inN) || (d0 == inN && d1 == 1) || (inN == 1 && (d0 == 1 || d1 == 1))) sN = inN;
    } else {
        sM = c.tA ? c.x1s.dim(-1) : c.x1s.dim(-2);
        sK = c.tA ? c.x1s.dim(-2) : c.x1s.dim(-1);
        sN = 0;
    }
    if (!recalc_group(inM, sM, gm, "m")) return false;
    if (!recalc_group(inK, sK, gk, "k")) return false;
    if (!mx) {
        if (a4w4_pergroup_nonsym(c, gk)) sN = c.tB ? c.x2s.dim(-1) : c.x2s.dim(-2);
        else sN = c.tB ? c.x2s.dim(-2) : c.x2s.dim(-1);
    }
    if (!recalc_group(inN, sN, gn, "n")) return false;
    groupSize = (int64_t)((gm << 32) | (gn << 16) | gk);
    return true;
}

// quant_matmul_checker.cpp:386-424
bool a4w4_pergroup_nonsym(const Ctx& c, uint64_t gsK)
{
    if (!c.x1s.present || !c.x2s.present || !c.x2o.present) return false;
    if (c.x1s.dtype != ACL_FLOAT || c.x1s.rank() <= 1) return false;
    if (c.x2s.dtype != ACL_FLOAT || c.x2s.rank() <= 1) return false;
    if (c.x2o.dtype != ACL_FLOAT16 || c.x2o.rank() <= 1) return false;
    if (c.bias.present) return false;
    if (c.x1.rank() < 2 || c.x2.rank() < 2) return false;
    int64_t m = c.tA ? c.x1.dim(1) : c.x1.dim(0);
    int64_t k = c.tB ? c.x2.dim(1) : c.x2.dim(0);
    int64_t n = c.tB ? c.x2.dim(0) : c.x2.dim(1);
    if (k % 1024 != 0 || n % 256 != 0) return false;
    return c.int4_in() && c.x1s.dim(0) == m && c.x1s.dim(1) == 1 && c.x2s.dim(0) == ceil_div(k, (int64_t)gsK) &&
           c.x2s.dim(1) == n && c.x2o.dim(0) == ceil_div(k, (int64_t)gsK) && c.x2o.dim(1) == n;
}

// ---- dtype rules for this SoC generation: quant_matmul_checker.cpp:1574-1848 ----
aclnnStatus check_dtype(const Ctx& c)
{
    const aclDataType out = c.out.dtype, s2 = c.x2s.dtype;
    if (out == ACL_INT32 && c.x1s.present) INVALID("%s: out INT32 is not supported together with x1Scale", kApi);
    if (!c.x1s.present) {  // T-T / T-C
        if (out == ACL_INT32 && !c.int8_in()) INVALID("%s: out INT32 needs INT8 inputs", kApi);
        if (c.int8_in() || c.int4_in()) {
            if (out == ACL_BF16) {
                if (!in_list(s2, {ACL_UINT64, ACL_INT64, ACL_FLOAT, ACL_BF16})) INVALID("%s: x2Scale dtype %s not supported for BF16 out", kApi, dtype_name(s2));
            } else if (out == ACL_INT8 || out == ACL_FLOAT16) {
                if (!in_list(s2, {ACL_UINT64, ACL_INT64})) INVALID("%s: x2Scale must be UINT64/INT64 for %s out, got %s", kApi, dtype_name(out), dtype_name(s2));
            } else if (out == ACL_INT32) {
                if (!in_list(s2, {ACL_FLOAT, ACL_BF16})) INVALID("%s: x2Scale must be FLOAT/BF16 for INT32 out", kApi);
            }
            if (c.bias.present) {
                if (out == ACL_INT32 && c.bias.dtype != ACL_INT32) INVALID("%s: bias must be INT32 for INT32 out", kApi);
                if (out == ACL_BF16 && in_list(s2, {ACL_FLOAT, ACL_BF16}) && !in_list(c.bias.dtype, {ACL_INT32, ACL_BF16, ACL_FLOAT}))
                    INVALID("%s: bias dtype %s not supported", kApi, dtype_name(c.bias.dtype));
                if (in_list(out, {ACL_INT8, ACL_FLOAT16, ACL_BF16}) && in_list(s2, {ACL_UINT64, ACL_INT64}) && c.bias.dtype != ACL_INT32)
                    INVALID("%s: bias must be INT32 with a 64-bit x2Scale, got %s", kApi, dtype_name(c.bias.dtype));
            }
            if (c.x2o.present) {
                if (out != ACL_INT8) INVALID("%s: x2Offset is only supported with INT8 out", kApi);
                if (c.x2o.dtype != ACL_FLOAT) INVALID("%s: x2Offset must be FLOAT, got %s", kApi, dtype_name(c.x2o.dtype));
            }
            if (!in_list(out, {ACL_INT8, ACL_FLOAT16, ACL_BF16, ACL_INT32})) INVALID("%s: out dtype %s not supported", kApi, dtype_name(out));
        } else if (c.hif8_in() || c.fp8_in()) {
            if (!in_list(s2, {ACL_UINT64, ACL_INT64})) INVALID("%s: x2Scale must be UINT64/INT64 without x1Scale, got %s", kApi, dtype_name(s2));
            if (c.bias.present && c.bias.dtype != ACL_FLOAT) INVALID("%s: bias must be FLOAT for fp8 inputs", kApi);
            if (c.x2o.present) INVALID("%s: x2Offset must be null for fp8 inputs", kApi);
            if (!in_list(out, {ACL_FLOAT16, ACL_BF16, ACL_FLOAT})) INVALID("%s: out dtype %s not supported for fp8 inputs", kApi, dtype_name(out));
        } else {
            INVALID("%s: unsupported input dtypes x1 %s, x2 %s", kApi, dtype_name(c.x1.dtype), dtype_name(c.x2.dtype));
        }
        return ACLNN_SUCCESS;
    }
    if (c.mx()) {
        if (!c.fp4_in() && !c.fp8_in()) INVALID("%s: MX mode needs FLOAT4_E2M1 or FLOAT8 inputs, got %s, %s", kApi, dtype_name(c.x1.dtype), dtype_name(c.x2.dtype));
        if (c.bias.present && c.bias.dtype != ACL_FLOAT) INVALID("%s: bias must be FLOAT in MX mode", kApi);
        if (!in_list(out, {ACL_FLOAT16, ACL_BF16, ACL_FLOAT})) INVALID("%s: out dtype %s not supported in MX mode", kApi, dtype_name(out));
        if (c.x2o.present) INVALID("%s: x2Offset must be null in MX mode", kApi);
        return ACLNN_SUCCESS;
    }
    if (c.int4_in() && c.x2o.present) {  // K-G asymmetric
        if (!in_list(out, {ACL_FLOAT16, ACL_BF16})) INVALID("%s: out must be FLOAT16/BF16 in K-G mode", kApi);
        if (c.x1s.dtype != ACL_FLOAT || c.x2s.dtype != ACL_FLOAT) INVALID("%s: scales must be FLOAT in K-G mode", kApi);
        if (c.x2o.dtype != ACL_FLOAT16) INVALID("%s: x2Offset must be FLOAT16 in K-G mode", kApi);
        if (c.tA || !c.tB) INVALID("%s: K-G mode needs transposeX1=false, transposeX2=true", kApi);
        return ACLNN_SUCCESS;
    }
    if (c.int8_in() || c.int4_in()) {  // K-C / K-T (and int8 per-block)
        if (!in_list(out, {ACL_FLOAT16, ACL_BF16})) INVALID("%s: out must be FLOAT16/BF16 with x1Scale, got %s", kApi, dtype_name(out));
        if (c.x1s.dtype != ACL_FLOAT) INVALID("%s: x1Scale must be FLOAT, got %s", kApi, dtype_name(c.x1s.dtype));
        if (c.x2o.present) INVALID("%s: x2Offset must be null with x1Scale", kApi);
        if (out == ACL_BF16) {
            if (!in_list(s2, {ACL_BF16, ACL_FLOAT})) INVALID("%s: x2Scale must be BF16/FLOAT, got %s", kApi, dtype_name(s2));
            if (c.bias.present && !in_list(c.bias.dtype, {ACL_INT32, ACL_BF16, ACL_FLOAT})) INVALID("%s: bias dtype %s not supported", kApi, dtype_name(c.bias.dtype));
        } else {
            if (s2 != ACL_FLOAT) INVALID("%s: x2Scale must be FLOAT for FLOAT16 out, got %s", kApi, dtype_name(s2));
            if (c.bias.present && !in_list(c.bias.dtype, {ACL_INT32, ACL_FLOAT16, ACL_FLOAT})) INVALID("%s: bias dtype %s not supported", kApi, dtype_name(c.bias.dtype));
        }
        return ACLNN_SUCCESS;
    }
    if (c.hif8_in() || c.fp8_in()) {  // double scale, K-C, G-B, B-B
        if (c.x1s.dtype != ACL_FLOAT) INVALID("%s: x1Scale must be FLOAT, got %s", kApi, dtype_name(c.x1s.dtype));
        if (s2 != ACL_FLOAT) INVALID("%s: x2Scale must be FLOAT, got %s", kApi, dtype_name(s2));
        if (!in_list(out, {ACL_FLOAT16, ACL_BF16, ACL_FLOAT})) INVALID("%s: out dtype %s not supported", kApi, dtype_name(out));
        if (c.perblock() && c.bias.present) INVALID("%s: bias must be null in G-B / B-B mode", kApi);
        if (c.bias.present && c.bias.dtype != ACL_FLOAT) INVALID("%s: bias must be FLOAT", kApi);
        if (c.x2o.present) INVALID("%s: x2Offset must be null", kApi);
        return ACLNN_SUCCESS;
    }
    INVALID("%s: unsupported input dtypes x1 %s, x2 %s", kApi, dtype_name(c.x1.dtype), dtype_name(c.x2.dtype));
}

// ---- shape rules: quant_matmul_checker.cpp:453-1195 ----
aclnnStatus check_shape(const Ctx& c, std::vector<int64_t>& batch)
{
    const uint64_t gk = (uint64_t)c.groupSize & kMask16, gn = ((uint64_t)c.groupSize >> 16) & kMask16, gm = ((uint64_t)c.groupSize >> 32) & kMask16;
    // scale ranks
    if (!c.x1s.present) {
        if (c.x2s.rank() != 1) INVALID("%s: x2Scale must be 1-D without x1Scale, got %ldD", kApi, (long)c.x2s.rank());
    } else if (c.mx()) {
        if (c.x1s.rank() < 3 || c.x2s.rank() < 3) INVALID("%s: MX scales must be at least 3-D", kApi);
        int64_t b1 = c.x1s.rank() - 3, b2 = c.x2s.rank() - 3;
        if (b1 != std::max<int64_t>(c.x1.rank() - 2, 0) || b2 != std::max<int64_t>(c.x2.rank() - 2, 0)) INVALID("%s: MX scale batch rank does not match the input", kApi);
        for (int64_t i = 0; i < b1; i++) if (c.x1s.dim(i) != c.x1.dim(i)) INVALID("%s: x1Scale batch dim %ld mismatch", kApi, (long)i);
        for (int64_t i = 0; i < b2; i++) if (c.x2s.dim(i) != c.x2.dim(i)) INVALID("%s: x2Scale batch dim %ld mismatch", kApi, (long)i);
    } else if (!a4w4_pergroup_nonsym(c, gk)) {
        bool pb = c.perblock();
        if ((pb && c.x1s.rank() != c.x1.rank()) || (!pb && c.x1s.rank() != 1)) INVALID("%s: x1Scale rank %ld not valid", kApi, (long)c.x1s.rank());
        if ((pb && c.x2s.rank() != c.x2.rank()) || (!pb && c.x2s.rank() != 1)) INVALID("%s: x2Scale rank %ld not valid", kApi, (long)c.x2s.rank());
    }
    // group size
    if (a4w4_pergroup_nonsym(c, gk)) {
        if (gk != 256) INVALID("%s: groupSizeK must be 256 in K-G mode", kApi);
    } else if (c.mx()) {
        if (gk != 32 || gm != 1 || gn != 1) INVALID("%s: MX mode needs groupSize [1,1,32], got [%lu,%lu,%lu]", kApi, (unsigned long)gm, (unsigned long)gn, (unsigned long)gk);
    } else if (c.perblock()) {
        if (gk != 128) INVALID("%s: groupSizeK must be 128 in G-B / B-B mode, got %lu", kApi, (unsigned long)gk);
        if (gn != 128) INVALID("%s: groupSizeN must be 128 in G-B / B-B mode, got %lu", kApi, (unsigned long)gn);
        if (gm != 128 && gm != 1) INVALID("%s: groupSizeM must be 1 or 128 in G-B / B-B mode, got %lu", kApi, (unsigned long)gm);
    } else if (c.groupSize != 0) {
        INVALID("%s: groupSize must be 0 in this quant mode, got %ld", kApi, (long)c.groupSize);
    }
    if (c.int4_in()) {
        if (c.K1 <= 0 || c.K1 % 2) INVALID("%s: K must be even for INT4", kApi);
        if (c.tB && (c.K2 <= 0 || c.K2 % 2)) INVALID("%s: K must be even for INT4", kApi);
        if (!c.tB && (c.N <= 0 || c.N % 2)) INVALID("%s: N must be even for INT4", kApi);
        if (c.tA) INVALID("%s: transposeX1 must be false for INT4", kApi);
        if (c.x2.rank() != 2) INVALID("%s: x2 must be 2-D for INT4", kApi);
        if (c.bias.present && c.bias.rank() != 1) INVALID("%s: bias must be 1-D for INT4", kApi);
    }
    if (c.K1 != c.K2) INVALID("%s: K of x1 (%ld) and x2 (%ld) differ", kApi, (long)c.K1, (long)c.K2);
    // per-mode extent checks
    bool done = false;
    if (c.x1s.present) {
        if (c.mx()) {
            int64_t b1 = c.x1s.rank() - 3, b2 = c.x2s.rank() - 3;
            int64_t sM = c.x1s.dim(b1 + (c.tA ? 1 : 0)), sK1 = c.x1s.dim(b1 + (c.tA ? 0 : 1));
            int64_t sN = c.x2s.dim(b2 + (c.tB ? 0 : 1)), sK2 = c.x2s.dim(b2 + (c.tB ? 1 : 0));
            int64_t k64a = ceil_div(c.K1, 64), k64b = ceil_div(c.K2, 64);
            bool one1 = (sM == 1 && sK1 == c.M) || (sM == c.M && sK1 == 1) || (sM == 1 && sK1 == k64a) || (sM == k64a && sK1 == 1);
            bool one2 = (sN == 1 && sK2 == c.N) || (sN == c.N && sK2 == 1) || (sN == 1 && sK2 == k64b) || (sN == k64b && sK2 == 1);
            if ((!one1 && sM != c.M) || (!one2 && sN != c.N)) INVALID("%s: MX scale M/N extents must equal those of x1/x2", kApi);
            if ((!one1 && k64a != sK1) || (!one2 && k64b != sK2)) INVALID("%s: MX scale K extent must be ceil(K/64)", kApi);
            if (c.x1s.dim(-1) != 2 || c.x2s.dim(-1) != 2) INVALID("%s: the last dim of MX scales must be 2", kApi);
            if (c.fp4_in()) {
                if (c.x1.dim(-1) % 2 || c.x2.dim(-1) % 2) INVALID("%s: inner axes of FLOAT4 inputs must be even", kApi);
                if (c.K1 <= 2 || c.K2 <= 2) INVALID("%s: K must be greater than 2 for FLOAT4 inputs", kApi);
            }
            done = true;
        } else if (c.perblock()) {
            if (c.x1s.rank() != c.x1.rank() || c.x2s.rank() != c.x2.rank()) INVALID("%s: block scale rank must equal the input rank", kApi);
            for (int64_t i = c.x1.rank() - 3; i >= 0; i--) if (c.x1s.dim(i) != c.x1.dim(i)) INVALID("%s: x1Scale batch dims mismatch", kApi);
            for (int64_t i = c.x2.rank() - 3; i >= 0; i--) if (c.x2s.dim(i) != c.x2.dim(i)) INVALID("%s: x2Scale batch dims mismatch", kApi);
            int64_t gsm = std::max<uint64_t>(gm, 1);
            int64_t mi = c.tA ? -1 : -2, k1i = c.tA ? -2 : -1, ni = c.tB ? -2 : -1, k2i = c.tB ? -1 : -2;
            if (ceil_div(c.x1.dim(mi), gsm) != c.x1s.dim(mi)) INVALID("%s: x1Scale M extent must be ceil(M/groupSizeM)", kApi);
            if (ceil_div(c.x1.dim(k1i), 128) != c.x1s.dim(k1i)) INVALID("%s: x1Scale K extent must be ceil(K/128)", kApi);
            if (ceil_div(c.x2.dim(ni), 128) != c.x2s.dim(ni)) INVALID("%s: x2Scale N extent must be ceil(N/128)", kApi);
            if (ceil_div(c.x2.dim(k2i), 128) != c.x2s.dim(k2i)) INVALID("%s: x2Scale K extent must be ceil(K/128)", kApi);
            done = true;
        } else if (c.x1s.rank() >= 1) {
            int64_t s0 = c.x1s.dim(0);
            if (c.M == 1) {
                if (s0 != 1) INVALID("%s: x1Scale must have 1 element when M is 1", kApi);
            } else if (s0 == 1 && !c.int8_in()) {
                if (c.x2s.dim(0) != 1 && c.x2s.dim(0) != c.N) INVALID("%s: x2Scale length must be 1 or N", kApi);
            } else if (s0 != c.M) {
                INVALID("%s: x1Scale length %ld must equal M %ld", kApi, (long)s0, (long)c.M);
            }
        }
    }
    if (!done) {
        bool kg = a4w4_pergroup_nonsym(c, gk);
        if (!kg && c.x2s.dim(0) != c.N && c.x2s.dim(0) != 1) INVALID("%s: x2Scale length %ld must be 1 or N %ld", kApi, (long)c.x2s.dim(0), (long)c.N);
        if (c.x2o.present && !kg) {
            if (c.x2o.rank() != 1) INVALID("%s: x2Offset must be 1-D", kApi);
            if (c.x2o.dim(0) != c.N && c.x2o.dim(0) != 1) INVALID("%s: x2Offset length must be 1 or N", kApi);
        }
    }
    // broadcast batch dims
    int64_t r1 = c.x1.rank(), r2 = c.x2.rank();
    int64_t outr = std::max(r1, r2), off = outr - std::min(r1, r2);
    const TView& lg = r1 > r2 ? c.x1 : c.x2;
    const TView& sh = r1 > r2 ? c.x2 : c.x1;
    int64_t out_batch = 1;
    batch.clear();
    for (int64_t i = 0; i < outr - 2; i++) {
        int64_t l = lg.dim(i), s = i < off ? 1 : sh.dim(i - off);
        if (s > 1 && l > 1 && s != l) INVALID("%s: batch dims of x1 and x2 cannot be broadcast", kApi);
        int64_t b = std::max(l, s);
        out_batch *= b;
        batch.push_back(b);
    }
    if (c.bias.present) {
        int64_t br = c.bias.rank();
        if (br != 3 && br != 1) INVALID("%s: bias must be 1-D or 3-D, got %ldD", kApi, (long)br);
        if (br == 1) {
            if (c.bias.dim(0) != c.N) INVALID("%s: bias length %ld must equal N %ld", kApi, (long)c.bias.dim(0), (long)c.N);
        } else {
            if (batch.size() != 1) INVALID("%s: a 3-D bias needs exactly one batch dim", kApi);
            if (c.bias.dim(1) != 1) INVALID("%s: bias second dim must be 1", kApi);
            if (c.bias.dim(2) != c.N) INVALID("%s: bias last dim must equal N", kApi);
            if (c.bias.dim(0) != out_batch) INVALID("%s: bias first dim must equal the out batch", kApi);
        }
    }
    int64_t outd = c.out.rank();
    int64_t oM = c.out.dim(-2), oN = c.out.dim(-1);
    int64_t inferred = (int64_t)batch.size() + 2;
    if (oM == 1 && inferred == 2 && outd == 3 && r1 == 2 && r2 == 2) { outd -= 1; oM = c.out.dim(0); }
    if (inferred != outd) INVALID("%s: out must be %ldD, got %ldD", kApi, (long)inferred, (long)c.out.rank());
    if (oM != c.M) INVALID("%s: out M %ld must equal %ld", kApi, (long)oM, (long)c.M);
    if (oN != c.N) INVALID("%s: out N %ld must equal %ld", kApi, (long)oN, (long)c.N);
    for (int64_t i = 0; i < outd - 2; i++) if (c.out.dim(i) != batch[(size_t)i]) INVALID("%s: out batch dim %ld mismatch", kApi, (long)i);
    return ACLNN_SUCCESS;
}

aclnnStatus check_format(const Ctx& c)
{
    auto nd = [](const TView& t) { return !t.present || t.format == ACL_FORMAT_ND; };
    if (!nd(c.x1) || !nd(c.x1s) || !nd(c.x2s) || !nd(c.x2o) || !nd(c.bias)) INVALID("%s: x1, scales, offset and bias must be ND", kApi);
    if (c.x2.format != ACL_FORMAT_ND) INVALID("%s: x2 must be ND", kApi);
    return ACLNN_SUCCESS;
}

// fp8 x fp4 checks: aclnn_quant_matmul_v5.cpp:193-243, 327-504, 597-835
aclnnStatus check_a8w4_pre(const Ctx& c)
{
    bool mx = c.mx();
    bool tcg = !c.x1s.present && in_list(c.x2s.dtype, {ACL_BF16, ACL_FLOAT16});
    if (!mx && !tcg) INVALID("%s: fp8 x fp4 supports only MX (e8m0 scales) or T-CG (no x1Scale, b16 x2Scale)", kApi);
    if (c.tA) INVALID("%s: transposeX1 must be false for fp8 x fp4", kApi);
    if (!c.tB) INVALID("%s: transposeX2 must be true for fp8 x fp4 ND", kApi);
    if (((uint64_t)c.groupSize & kMask16) != 32) INVALID("%s: groupSizeK must be 32 for fp8 x fp4", kApi);
    if (c.x1.rank() != 2 || c.x2.rank() != 2) INVALID("%s: x1 and x2 must be 2-D for fp8 x fp4", kApi);
    if (c.bias.present && c.bias.rank() != 2) INVALID("%s: bias must be 2-D for fp8 x fp4", kApi);
    int64_t want = mx ? 3 : 2;
    if (c.x1s.present && c.x1s.rank() != want) INVALID("%s: x1Scale must be %ldD", kApi, (long)want);
    if (c.x2s.rank() != want) INVALID("%s: x2Scale must be %ldD", kApi, (long)want);
    if (c.ys.present && c.ys.rank() != 2) INVALID("%s: yScale must be 2-D", kApi);
    if (c.yo.present && c.yo.rank() != 1) INVALID("%s: yOffset must be 1-D", kApi);
    if (c.out.rank() != 2) INVALID("%s: out must be 2-D for fp8 x fp4", kApi);
    return ACLNN_SUCCESS;
}

aclnnStatus check_a8w4_params(const Ctx& c)
{
    if (!in_list(c.x1.dtype, {ACL_FLOAT8_E4M3FN, ACL_FLOAT8_E5M2})) INVALID("%s: x1 dtype not supported", kApi);
    if (c.x2.dtype != ACL_FLOAT4_E2M1) INVALID("%s: x2 must be FLOAT4_E2M1", kApi);
    if (!in_list(c.out.dtype, {ACL_BF16, ACL_FLOAT16})) INVALID("%s: out must be BF16/FLOAT16 for fp8 x fp4", kApi);
    bool mx = c.mx();
    if (!c.x1s.present) {
        if (c.bias.present) INVALID("%s: bias must be null in T-CG mode", kApi);
        if (!c.ys.present) INVALID("%s: yScale must not be null in T-CG mode", kApi);
        if (!in_list(c.x2s.dtype, {ACL_BF16, ACL_FLOAT16})) INVALID("%s: x2Scale must be BF16/FLOAT16 in T-CG mode", kApi);
        if (c.ys.dtype != ACL_UINT64) INVALID("%s: yScale must be UINT64/INT64", kApi);
    } else if (mx) {
        if (c.bias.present && c.bias.dtype != c.out.dtype) INVALID("%s: bias dtype must equal out dtype in MX fp8 x fp4 mode", kApi);
        if (c.ys.present) INVALID("%s: yScale must be null in MX fp8 x fp4 mode", kApi);
    } else {
        INVALID("%s: unexpected quant mode", kApi);
    }
    auto nd = [](const TView& t) { return !t.present || t.format == ACL_FORMAT_ND; };
    if (!nd(c.x1) || !nd(c.x2s) || !nd(c.ys) || !nd(c.bias) || !nd(c.x1s) || !nd(c.yo) || !nd(c.out)) INVALID("%s: tensors must be ND", kApi);
    if (c.M <= 0) INVALID("%s: M must be positive", kApi);
    if (c.K1 <= 0) INVALID("%s: K must be positive", kApi);
    if (c.N <= 0) INVALID("%s: N must be positive", kApi);
    if (c.K1 != c.K2) INVALID("%s: K of x1 and x2 differ", kApi);
    if (c.x1.dtype == ACL_FLOAT8_E4M3FN && !c.x1s.present) {
        if (c.K1 % 32 != 0 || c.K1 <= 32) INVALID("%s: K must be a multiple of 32 and greater than 32 in T-CG mode", kApi);
    } else if (c.x1.dtype == ACL_FLOAT8_E4M3FN && mx) {
        if (c.K1 % 8 != 0) INVALID("%s: K must be a multiple of 8 in MX fp8 x fp4 mode", kApi);
    } else if (c.K1 % 64 != 0) {
        INVALID("%s: K must be a multiple of 64", kApi);
    }
    int64_t gdim = (c.K2 + 31) / 32;
    if (mx) {
        if (c.x1s.dim(0) != c.M || c.x1s.dim(1) != ceil_div(gdim, 2) || c.x1s.dim(2) != 2) INVALID("%s: x1Scale shape must be [M, ceil(K/64), 2]", kApi);
    }
    int64_t sn = c.tB ? c.x2s.dim(0) : c.x2s.dim(1), sg = c.tB ? c.x2s.dim(1) : c.x2s.dim(0);
    if (mx) {
        if (sn != c.N || sg != ceil_div(gdim, 2) || c.x2s.dim(2) != 2) INVALID("%s: x2Scale shape must be [N, ceil(K/64), 2]", kApi);
    } else if (sn != c.N || sg != gdim) {
        INVALID("%s: x2Scale shape must be [N, ceil(K/32)]", kApi);
    }
    if (c.ys.present && (c.ys.dim(0) != 1 || c.ys.dim(1) != c.N)) INVALID("%s: yScale shape must be [1, N]", kApi);
    if (c.bias.present && (c.bias.dim(0) != 1 || c.bias.dim(1) != c.N)) INVALID("%s: bias shape must be [1, N]", kApi);
    if (c.out.dim(0) != c.M || c.out.dim(1) != c.N) INVALID("%s: out shape must be [M, N]", kApi);
    return ACLNN_SUCCESS;
}

OpsnnMat mat_of(const TView& t, bool transposed)
{
    // logical [R, C] over a dense view of [.., R, C] (or [.., C, R] when transposed)
    OpsnnMat m{};
    m.ptr = t.ptr_at(0);
    if (!is_contiguous(t)) {   // a regular strided view (contiguous_process admitted it): its own strides
        m.row_stride = transposed ? t.stride(-1) : t.stride(-2);
        m.col_stride = transposed ? t.stride(-2) : t.stride(-1);
        m.batch_stride = t.rank() > 2 ? t.stride(-3) : 0;
        return m;
    }
    int64_t d1 = t.dim(-1);
    if (transposed) { m.row_stride = 1; m.col_stride = d1; }
    else { m.row_stride = d1; m.col_stride = 1; }
    m.batch_stride = t.rank() > 2 ? t.dim(-1) * t.dim(-2) : 0;
    return m;
}

}  // namespace

extern "C" aclnnStatus aclnnQuantMatmulV5GetWorkspaceSize(const aclTensor* x1, const aclTensor* x2,
                                                          const aclTensor* x1Scale, const aclTensor* x2Scale,
                                                          const aclTensor* yScale, const aclTensor* x1Offset,
                                                          const aclTensor* x2Offset, const aclTensor* yOffset,
                                                          const aclTensor* bias, bool transposeX1, bool transposeX2,
                                                          int64_t groupSize, aclTensor* out, uint64_t* workspaceSize,
                                                          aclOpExecutor** executor)
{
    clear_error();
    if (log_enabled()) fprintf(stderr, "[opsnn] %s tA=%d tB=%d groupSize=%ld\n", kApi, (int)transposeX1, (int)transposeX2, (long)groupSize);
    if (!workspaceSize || !executor) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: workspaceSize/executor is null", kApi);
    if (!x2) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: x2 is null", kApi);
    if (is_nz(x2->format)) INVALID("%s: x2 in FRACTAL_NZ format is not supported, use ND", kApi);

    Ctx c;
    c.x1 = make_view(x1); c.x2 = make_view(x2); c.x1s = make_view(x1Scale); c.x2s = make_view(x2Scale);
    c.ys = make_view(yScale); c.x1o = make_view(x1Offset); c.x2o = make_view(x2Offset); c.yo = make_view(yOffset);
    c.bias = make_view(bias); c.out = make_view(out);
    c.tA = transposeX1; c.tB = transposeX2; c.groupSize = groupSize;

    // required / forbidden arguments (aclnn_quant_matmul_v5.cpp:245-283): all report NULLPTR
    if (!x1) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: x1 is null", kApi);
    if (!x2Scale) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: x2Scale is null", kApi);
    if (!out) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: out is null", kApi);
    const bool isA8W4F = c.a8w4f();
    const bool isA8W4 = isA8W4F || c.a8w4i_raw();
    if (!isA8W4 && c.ys.present && !c.ys.empty()) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: yScale must be null or empty", kApi);
    if (c.x1o.present && !c.x1o.empty()) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: x1Offset must be null or empty", kApi);
    if (isA8W4 && c.x2o.present) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: x2Offset must be null for 8-bit x 4-bit inputs", kApi);
    if (c.yo.present && !c.yo.empty() && !c.a8w4i_raw()) FAIL(ACLNN_ERR_PARAM_NULLPTR, "%s: yOffset must be null or empty", kApi);

    if (isA8W4F) {  // aclnn_quant_matmul_v5.cpp:1045-1061
        uint64_t gn = ((uint64_t)c.groupSize >> 16) & kMask16, gm = ((uint64_t)c.groupSize >> 32) & kMask16;
        if (!((gm == 0 && gn == 0) || (gm == 1 && gn == 1))) INVALID("%s: groupSizeM and groupSizeN must both be 0 or 1 for fp8 x fp4", kApi);
        c.groupSize = (int64_t)((uint64_t)c.groupSize & kMask16);
    }

    std::unique_ptr<aclOpExecutor> ex(new (std::nothrow) aclOpExecutor());
    if (!ex) FAIL(ACLNN_ERR_INNER_CREATE_EXECUTOR, "%s: cannot allocate executor", kApi);
    ex->api = "aclnnQuantMatmulV5";

    // empty output: success without a launch (aclnn_quant_matmul_v5.cpp:1088-1108)
    if (!isA8W4 && c.x1.rank() >= 2 && c.x2.rank() >= 2) {
        int64_t m = c.tA ? c.x1.dim(-1) : c.x1.dim(-2);
        int64_t n = c.tB ? c.x2.dim(-2) : c.x2.dim(-1);
        if (m == 0 || n == 0) {
            *workspaceSize = 0;
            *executor = (aclOpExecutor*)executor_publish(ex.release());
            return ACLNN_SUCCESS;
        }
    }

    // view normalisation (PreMatmulCalcProcess, aclnn_quant_matmul_v5.cpp:967-1016)
    aclnnStatus rc;
    bool tmp = false;
    if ((rc = contiguous_process(c.x1, c.tA, "x1", true)) != ACLNN_SUCCESS) return rc;
    const bool mx_like = c.mx() && (c.fp4_in() || c.fp8_in() || isA8W4F);
    if (c.x1s.present) {
        rc = mx_like ? mx_scale_process(c.x1s, "x1Scale") : contiguous_process(c.x1s, tmp, "x1Scale");
        if (rc != ACLNN_SUCCESS) return rc;
    }
    rc = mx_like ? mx_scale_process(c.x2s, "x2Scale") : contiguous_process(c.x2s, tmp, "x2Scale");
    if (rc != ACLNN_SUCCESS) return rc;
    if ((rc = contiguous_process(c.bias, tmp, "bias")) != ACLNN_SUCCESS) return rc;
    if ((rc = contiguous_process(c.x2o, tmp, "x2Offset")) != ACLNN_SUCCESS) return rc;
    if ((rc = contiguous_process(c.ys, tmp, "yScale")) != ACLNN_SUCCESS) return rc;
    if ((rc = contiguous_process(c.x2, c.tB, "x2", true)) != ACLNN_SUCCESS) return rc;

    if (isA8W4) {
        if (c.a8w4i_raw()) FAIL(ACLNN_ERR_RUNTIME_ERROR, "%s: int8 x int4 (A8W4 int) is not supported on this device generation", kApi);
        if ((rc = check_a8w4_pre(c)) != ACLNN_SUCCESS) return rc;
    } else {
        // CheckDimRange (aclnn_quant_matmul_v5.cpp:285-325)
        int64_t sr = (int64_t)c.x2.storage.size();
        if (sr < 2 || sr > 6) INVALID("%s: x2 storage rank %ld must be in [2, 6]", kApi, (long)sr);
        if (c.x1.rank() < 2) INVALID("%s: x1 must be at least 2-D", kApi);
        if (c.out.rank() < 2) INVALID("%s: out must be at least 2-D", kApi);
        if (c.x1.rank() > 6) INVALID("%s: x1 must be at most 6-D", kApi);
        if (c.out.rank() > 6) INVALID("%s: out must be at most 6-D", kApi);
        if (c.x2.rank() < 2) INVALID("%s: x2 must be at least 2-D", kApi);
    }
    retag_int32_as_int4(c.x2);
    retag_int32_as_int4(c.x1);

    int64_t gsReal = c.groupSize;
    if (!isA8W4) {
        if (!infer_group_size(c, gsReal)) return ACLNN_ERR_PARAM_INVALID;
    } else if (!c.x1s.present && c.ys.present && c.ys.dtype == ACL_INT64) {
        c.ys.dtype = ACL_UINT64;
    }
    if (c.x2s.dtype == ACL_INT64) c.x2s.dtype = ACL_UINT64;
    c.refresh_dims();

    if (isA8W4F) {
        if ((rc = check_a8w4_params(c)) != ACLNN_SUCCESS) return rc;
    } else {
        Ctx cc = c;
        cc.groupSize = gsReal;
        if ((rc = check_dtype(cc)) != ACLNN_SUCCESS) return rc;
        std::vector<int64_t> batch;
        if ((rc = check_shape(cc, batch)) != ACLNN_SUCCESS) return rc;
        if ((rc = check_format(cc)) != ACLNN_SUCCESS) return rc;
        if (cc.x1.empty() || cc.x2.empty()) INVALID("%s: x1 and x2 must not be empty", kApi);
        c.groupSize = gsReal;
    }
    if (!is_contiguous(c.out)) INVALID("%s: out must be contiguous", kApi);

    // ---- route (aclnn_quant_matmul_v5.cpp:1163-1174) and build the launch plan ----
    OpsnnQmmArgs& a = ex->qmm;
    a.M = c.M; a.N = c.N; a.K = c.K1;
    // a strided 4-bit operand (or 8-bit MX operand): phase 2 gathers it; from here on the view is the dense copy (its address is filled in then)
    auto plan_gather = [&](TView& t, int which) {
        const bool mx8 = dtype_bits(t.dtype) == 8 && c.mx();   // (the other 8-bit modes gather in their launchers)
        if ((!is_4bit(t.dtype) && !mx8) || is_contiguous(t)) return;
        auto& g = ex->gather[which];
        g.active = true; g.bits = mx8 ? 8 : 4; g.base = t.data; g.off = t.offset;
        g.rows = t.dim(-2); g.cols = t.dim(-1); g.rs = t.stride(-2); g.cs = t.stride(-1);
        g.nb = 1;
        for (int64_t i = 0; i < t.rank() - 2; i++) g.nb *= t.dim(i);
        g.bs = t.rank() > 2 ? t.stride(-3) : 0;
        g.bytes = (uint64_t)(g.nb * g.rows * g.cols * g.bits / 8);
        t.offset = 0;
        int64_t st = 1;
        for (int64_t i = t.rank() - 1; i >= 0; i--) { t.strides[(size_t)i] = st; st *= t.shape[(size_t)i]; }
        t.data = (void*)(uintptr_t)256;   // any aligned non-null address until phase 2 knows the workspace
    };
    plan_gather(c.x1, 0);
    plan_gather(c.x2, 1);
    a.x1 = mat_of(c.x1, c.tA);
    a.x2 = mat_of(c.x2, c.tB);
    a.x1_dtype = c.x1.dtype; a.x2_dtype = c.x2.dtype;
    a.out = const_cast<void*>(c.out.ptr_at(0)); a.out_dtype = c.out.dtype;
    int64_t b1 = 1, b2 = 1;
    for (int64_t i = 0; i < c.x1.rank() - 2; i++) b1 *= c.x1.dim(i);
    for (int64_t i = 0; i < c.x2.rank() - 2; i++) b2 *= c.x2.dim(i);
    int64_t ob = 1;
    for (int64_t i = 0; i < c.out.rank() - 2; i++) ob *= c.out.dim(i);
    if (c.x1.rank() == 2 && c.x2.rank() == 2) ob = 1;
    a.batch = ob;
    // one launch covers an operand with no batch dims (or all ones) or with the full out batch; any other broadcast
    // pattern (qbmmv3_kernel_golden.py:288-330 broadcasts any pair) is split into launches over the innermost batch dim below
    const bool general_broadcast = (b1 != 1 && b1 != ob) || (b2 != 1 && b2 != ob);
    if (b1 == 1) a.x1.batch_stride = 0;
    if (b2 == 1) a.x2.batch_stride = 0;
    if (c.bias.present) {
        a.bias = c.bias.ptr_at(0); a.bias_dtype = c.bias.dtype;
        a.bias_batch_stride = c.bias.rank() == 3 ? c.N : 0;
    }
    a.x2_scale = c.x2s.ptr_at(0); a.x2_scale_dtype = c.x2s.dtype;
    a.x1_scale = c.x1s.present ? c.x1s.ptr_at(0) : nullptr;
    a.gsK = (int64_t)((uint64_t)c.groupSize & kMask16);
    a.gsN = (int64_t)(((uint64_t)c.groupSize >> 16) & kMask16);
    a.gsM = (int64_t)(((uint64_t)c.groupSize >> 32) & kMask16);

    int mode = 0;
    if (isA8W4F && !c.mx()) {
        // fp8 x fp4 with a 16-bit scale per K group and a packed 64-bit output scale: qbmmv4_kernel_golden.py:189-255
        if (c.x1.dtype != ACL_FLOAT8_E4M3FN)
            FAIL(ACLNN_ERR_INNER_TILING_ERROR, "%s: fp8 x fp4 with group scales takes FLOAT8_E4M3FN x1 only on this device, got %s", kApi, dtype_name(c.x1.dtype));
        ex->kind = OpKind::QmmGroup; mode = 4;
        a.gsK = (int64_t)((uint64_t)c.groupSize & kMask16);
        const int64_t G = ceil_div(c.K1, std::max<int64_t>(a.gsK, 1));
        a.x2_scale_mat.ptr = c.x2s.ptr_at(0);
        if (c.tB) { a.x2_scale_mat.row_stride = 1; a.x2_scale_mat.col_stride = G; }    // stored [N, G]
        else { a.x2_scale_mat.row_stride = c.N; a.x2_scale_mat.col_stride = 1; }       // stored [G, N]
        if (c.ys.present) { a.y_scale = c.ys.ptr_at(0); a.y_scale_len = c.ys.numel(); }
    } else if (a4w4_pergroup_nonsym(c, (uint64_t)a.gsK)) {
        // int4 x int4 with per-group scales and offsets: qbmmv4_kernel_golden.py:328-395
        ex->kind = OpKind::QmmGroup; mode = 4;
        a.x2_scale_mat.ptr = c.x2s.ptr_at(0); a.x2_scale_mat.row_stride = c.N; a.x2_scale_mat.col_stride = 1;
        a.x2_offset_mat.ptr = c.x2o.ptr_at(0); a.x2_offset_mat.row_stride = c.N; a.x2_offset_mat.col_stride = 1;
    } else if (c.mx()) {
        ex->kind = OpKind::QmmMx; mode = 2;
        // scale byte of row r and 32-wide K block kb: ptr[r*row_stride + (kb/2)*col_stride + kb%2]
        int64_t ks = ceil_div(c.K1, 64);
        a.x1_scale_mat.ptr = c.x1s.ptr_at(0);
        if (c.tA) { a.x1_scale_mat.row_stride = 2; a.x1_scale_mat.col_stride = c.M * 2; }   // stored [ks, M, 2]
        else { a.x1_scale_mat.row_stride = ks * 2; a.x1_scale_mat.col_stride = 2; }         // stored [M, ks, 2]
        a.x1_scale_mat.batch_stride = b1 == 1 ? 0 : c.M * ks * 2;
        a.x2_scale_mat.ptr = c.x2s.ptr_at(0);
        if (c.tB) { a.x2_scale_mat.row_stride = ks * 2; a.x2_scale_mat.col_stride = 2; }    // stored [N, ks, 2]
        else { a.x2_scale_mat.row_stride = 2; a.x2_scale_mat.col_stride = c.N * 2; }        // stored [ks, N, 2]
        a.x2_scale_mat.batch_stride = b2 == 1 ? 0 : c.N * ks * 2;
    } else if (c.perblock()) {
        ex->kind = OpKind::QmmBlockScale; mode = 1;
        int64_t kb = ceil_div(c.K1, 128), mb = ceil_div(c.M, std::max<int64_t>(a.gsM, 1)), nb = ceil_div(c.N, 128);
        a.x1_scale_mat.ptr = c.x1s.ptr_at(0);
        if (c.tA) { a.x1_scale_mat.row_stride = 1; a.x1_scale_mat.col_stride = mb; }
        else { a.x1_scale_mat.row_stride = kb; a.x1_scale_mat.col_stride = 1; }
        a.x1_scale_mat.batch_stride = b1 == 1 ? 0 : mb * kb;
        a.x2_scale_mat.ptr = c.x2s.ptr_at(0);
        if (c.tB) { a.x2_scale_mat.row_stride = 1; a.x2_scale_mat.col_stride = kb; }
        else { a.x2_scale_mat.row_stride = nb; a.x2_scale_mat.col_stride = 1; }
        a.x2_scale_mat.batch_stride = b2 == 1 ? 0 : nb * kb;
    } else if (c.int8_in() && in_list(c.x2s.dtype, {ACL_FLOAT, ACL_BF16}) && in_list(c.out.dtype, {ACL_BF16, ACL_FLOAT16, ACL_INT32}) &&
               !(!c.x1s.present && c.x2s.dim(0) == 1 && c.out.dtype != ACL_INT32 &&
                 !(c.bias.present && in_list(c.bias.dtype, {ACL_BF16, ACL_FLOAT})))) {
        // (the excluded case is the per-tensor scale that the reference truncates to 19 bits: it goes to the T-C kernel)
        ex->kind = OpKind::QmmInt8; mode = 0;
        a.x2_scale_len = c.x2s.dim(0);
    } else if ((c.int8_in() && in_list(c.x2s.dtype, {ACL_FLOAT, ACL_BF16, ACL_UINT64}) &&
                in_list(c.out.dtype, {ACL_BF16, ACL_FLOAT16, ACL_INT8, ACL_INT32}) && !c.x1s.present) ||
               (c.fp8_in() && in_list(c.x2s.dtype, {ACL_FLOAT, ACL_BF16, ACL_UINT64}) && in_list(c.out.dtype, {ACL_BF16, ACL_FLOAT16, ACL_FLOAT}) &&
                (!c.x1s.present || (c.x1s.dtype == ACL_FLOAT && c.x1s.rank() == 1 && (c.x1s.dim(0) == 1 || c.x1s.dim(0) == c.M))))) {
        // per-tensor / per-channel family: qbmmv3_kernel_golden.py:390-513
        ex->kind = OpKind::QmmTc; mode = 3;
        a.x2_scale_len = c.x2s.dim(0);
        a.x1_scale_len = c.x1s.present ? c.x1s.dim(0) : 0;
        if (c.x2o.present) {
            a.x2_offset = (const float*)c.x2o.ptr_at(0);
            a.x2_offset_len = c.x2o.dim(0);
        }
    } else {
        FAIL(ACLNN_ERR_INNER_TILING_ERROR, "%s: no kernel for x1 %s, x2 %s, x2Scale %s, out %s on this device yet", kApi,
             dtype_name(c.x1.dtype), dtype_name(c.x2.dtype), dtype_name(c.x2s.dtype), dtype_name(c.out.dtype));
    }
    if (general_broadcast) {
        if (!is_contiguous(c.x1) || !is_contiguous(c.x2) || ex->gather[0].active || ex->gather[1].active)
            INVALID("%s: batch dims that broadcast partially need dense x1 and x2", kApi);
        if (c.bias.present && c.bias.rank() == 3) INVALID("%s: a 3-D bias cannot go with partially broadcast batch dims", kApi);
        const int64_t nb = c.out.rank() - 2, r1 = c.x1.rank() - 2, r2 = c.x2.rank() - 2;
        std::vector<int64_t> od((size_t)nb), d1((size_t)nb, 1), d2((size_t)nb, 1);
        for (int64_t i = 0; i < nb; i++) od[(size_t)i] = c.out.dim(i);
        for (int64_t i = 0; i < r1; i++) d1[(size_t)(nb - r1 + i)] = c.x1.dim(i);
        for (int64_t i = 0; i < r2; i++) d2[(size_t)(nb - r2 + i)] = c.x2.dim(i);
        const int64_t L = nb - 1, inner = od[(size_t)L];
        int64_t outer = 1;
        for (int64_t i = 0; i < L; i++) outer *= od[(size_t)i];
        auto bytes_of = [](int64_t elems, int dt) { return elems * dtype_bits((aclDataType)dt) / 8; };
        const int64_t x1_slice = a.x1.batch_stride, x2_slice = a.x2.batch_stride;   // elements per batch slice (dense operands)
        const int64_t s1_slice = a.x1_scale_mat.batch_stride, s2_slice = a.x2_scale_mat.batch_stride;
        // element size of the scale tables: fp32 in the block-scale modes, e8m0 bytes in the MX modes; no other mode gives
        // its scales batch dims
        const int64_t s_esize = mode == 2 ? 1 : 4;
        const int64_t out_slice_bytes = bytes_of(c.M * c.N, c.out.dtype);
        for (int64_t o = 0; o < outer; o++) {
            int64_t rem = o, f1 = 0, f2 = 0, st1 = d1[(size_t)L], st2 = d2[(size_t)L];   // flat slice index of the run's first slice
            for (int64_t i = L - 1; i >= 0; i--) {
                const int64_t idx = rem % od[(size_t)i];
                rem /= od[(size_t)i];
                if (d1[(size_t)i] > 1) f1 += idx * st1;
                if (d2[(size_t)i] > 1) f2 += idx * st2;
                st1 *= d1[(size_t)i];
                st2 *= d2[(size_t)i];
            }
            OpsnnQmmArgs q = a;
            q.batch = inner;
            q.x1.ptr = (const char*)a.x1.ptr + bytes_of(f1 * x1_slice, a.x1_dtype);
            q.x2.ptr = (const char*)a.x2.ptr + bytes_of(f2 * x2_slice, a.x2_dtype);
            q.x1.batch_stride = d1[(size_t)L] > 1 ? x1_slice : 0;
            q.x2.batch_stride = d2[(size_t)L] > 1 ? x2_slice : 0;
            if (a.x1_scale_mat.ptr) {
                q.x1_scale_mat.ptr = (const char*)a.x1_scale_mat.ptr + f1 * s1_slice * s_esize;
                q.x1_scale_mat.batch_stride = d1[(size_t)L] > 1 ? s1_slice : 0;
            }
            if (a.x2_scale_mat.ptr) {
                q.x2_scale_mat.ptr = (const char*)a.x2_scale_mat.ptr + f2 * s2_slice * s_esize;
                q.x2_scale_mat.batch_stride = d2[(size_t)L] > 1 ? s2_slice : 0;
            }
            q.out = (char*)a.out + o * inner * out_slice_bytes;
            ex->batch_runs.push_back(q);
        }
        a.batch = inner;   // the workspace one launch needs; the launches run one after the other on the stream and share it
        a.x1.batch_stride = ex->batch_runs[0].x1.batch_stride;
        a.x2.batch_stride = ex->batch_runs[0].x2.batch_stride;
    }
    ex->workspace_size = ex->gather_front() + opsnnQmmWorkspace(&a, mode);
    *workspaceSize = ex->workspace_size;
    *executor = (aclOpExecutor*)executor_publish(ex.release());
    return ACLNN_SUCCESS;
}

extern "C" aclnnStatus aclnnQuantMatmulV5(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                          aclrtStream stream)
{
    clear_error();
    if (!executor) FAIL(ACLNN_ERR_PARAM_NULLPTR, "aclnnQuantMatmulV5: executor is null");
    if (!executor_claim(executor)) INVALID("aclnnQuantMatmulV5: executor is not valid (already run or destroyed)");
    std::unique_ptr<aclOpExecutor> ex(executor);  // consumed by this call
    ex->magic = 0;
    if (ex->kind == OpKind::None) return ACLNN_SUCCESS;
    if (ex->workspace_size > 0 && (!workspace || workspaceSize < ex->workspace_size))
        INVALID("aclnnQuantMatmulV5: workspace of %lu bytes required", (unsigned long)ex->workspace_size);
    if (!ex->qmm.x1.ptr || !ex->qmm.x2.ptr || !ex->qmm.out) INVALID("aclnnQuantMatmulV5: a tensor has no device address");
    int rc = 0;
    // strided 4-bit (and 8-bit MX) operands first become dense copies at the front of the workspace
    char* w = (char*)workspace;
    for (int i = 0; i < 2; i++) {
        const auto& g = ex->gather[i];
        if (!g.active) continue;
        if (!g.base) INVALID("aclnnQuantMatmulV5: a tensor has no device address");
        rc = (g.bits == 4 ? opsnnGather4 : opsnnGather8)(g.base, g.off, g.nb, g.rows, g.cols, g.bs, g.rs, g.cs, w, stream);
        if (rc != 0) FAIL(ACLNN_ERR_RUNTIME_ERROR, "%s: gathering the strided %s failed with code %d", ex->api, i ? "x2" : "x1", rc);
        (i ? ex->qmm.x2 : ex->qmm.x1).ptr = w;
        w += (g.bytes + 255) / 256 * 256;
    }
    const uint64_t front = ex->gather_front();
    ex->qmm.workspace = ex->workspace_size > front ? w : nullptr;
    // a FRACTAL_NZ x2 is re-written into the workspace on every call, and so is a gathered one: addresses the weight cache
    // must not key on
    WeightCacheScope cache_scope(ex->nz.active || ex->gather[1].active);
    if (ex->nz.active) {   // x2 arrived in FRACTAL_NZ (aclnnQuantMatmulWeightNz): lay it out as ND in the front of the workspace
        const void* nd = nullptr;
        void* rest = nullptr;
        rc = run_nz_step(*ex, w, stream, &nd, &rest);
        if (rc != 0) FAIL(ACLNN_ERR_RUNTIME_ERROR, "%s: FRACTAL_NZ re-layout failed with code %d", ex->api, rc);
        ex->qmm.x2.ptr = nd;
        ex->qmm.workspace = ex->workspace_size > front + nz_front_bytes(*ex) ? rest : nullptr;
    }
    auto launch = [&](const OpsnnQmmArgs& q) -> int {
        switch (ex->kind) {
            case OpKind::QmmInt8: return opsnnQmmInt8(&q, stream);
            case OpKind::QmmBlockScale: return opsnnQmmBlockScale(&q, stream);
            case OpKind::QmmMx: return opsnnQmmMx(&q, stream);
            case OpKind::QmmTc: return opsnnQmmTc(&q, stream);
            case OpKind::QmmGroup: return opsnnQmmGroup(&q, stream);
            default: return -100;
        }
    };
    if (ex->batch_runs.empty()) {
        rc = launch(ex->qmm);
    } else {
        for (OpsnnQmmArgs& q : ex->batch_runs) {   // partially broadcast batch dims: one launch per outer combination
            q.workspace = ex->qmm.workspace;
            if ((rc = launch(q)) != 0) break;
        }
    }
    if (rc != 0) FAIL(rc < 0 ? ACLNN_ERR_INNER_TILING_ERROR : ACLNN_ERR_RUNTIME_ERROR, "aclnnQuantMatmulV5: launch failed with code %d", rc);
    return ACLNN_SUCCESS;
}
