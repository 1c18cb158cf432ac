// Two chains a user of the reference writes around the quantized matmuls, against the public headers only:
//   1. int32 weight carriers -> aclnnConvertWeightToINT4Pack -> aclnnWeightQuantBatchMatmulV2 (W4A16, per-channel scale)
//      (the sequence of the reference's matmul/convert_weight_to_int4_pack/examples/test_aclnn_convert_weight_to_int4_pack.cpp)
//   2. fp16 activation -> aclnnDynamicQuant -> aclnnQuantMatmulV5 (W8A8, the per-token scale as x1Scale)
// Both results are verified on the host with plain loops.
//
//   g++ -std=c++17 -I../../include w4_pack_and_dynamic_quant_chain.cpp -L../lib -lopsnn_amd -Wl,-rpath,'$ORIGIN/../lib' -o chain
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "acl/acl.h"
#include "aclnnop/aclnn_convert_weight_to_int4_pack.h"
#include "aclnnop/aclnn_dynamic_quant.h"
#include "aclnnop/aclnn_quant_matmul_v5.h"
#include "aclnnop/aclnn_weight_quant_batch_matmul_v2.h"

#define CHECK(expr)                                                                      \
    do {                                                                                 \
        int rc_ = (expr);                                                                \
        if (rc_ != 0) {                                                                  \
            std::printf("%s failed: %d (%s)\n", #expr, rc_, aclGetRecentErrMsg());       \
            return 1;                                                                    \
        }                                                                                \
    } while (0)

// IEEE binary16 <-> float for the values used here (normal numbers, no overflow)
static uint16_t float_to_half(float f)
{
    uint32_t u;
    std::memcpy(&u, &f, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const int32_t e = (int32_t)((u >> 23) & 0xFF) - 127 + 15;
    if (e <= 0) return (uint16_t)sign;
    uint32_t m = u & 0x7FFFFFu;
    uint32_t h = sign | ((uint32_t)e << 10) | (m >> 13);
    const uint32_t rest = m & 0x1FFFu;
    if (rest > 0x1000u || (rest == 0x1000u && (h & 1u))) h += 1;
    return (uint16_t)h;
}
static float half_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    uint32_t u = e == 0 ? sign : (sign | ((e - 15 + 127) << 23) | (m << 13));
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

template <class T>
static int make_tensor(const std::vector<T>& host, const std::vector<int64_t>& shape, aclDataType dt, void** dev, aclTensor** t)
{
    CHECK(aclrtMalloc(dev, host.size() * sizeof(T), ACL_MEM_MALLOC_HUGE_FIRST));
    CHECK(aclrtMemcpy(*dev, host.size() * sizeof(T), host.data(), host.size() * sizeof(T), ACL_MEMCPY_HOST_TO_DEVICE));
    std::vector<int64_t> strides(shape.size(), 1);
    for (int i = (int)shape.size() - 2; i >= 0; i--) strides[i] = strides[i + 1] * shape[i + 1];
    *t = aclCreateTensor(shape.data(), shape.size(), dt, strides.data(), 0, ACL_FORMAT_ND, shape.data(), shape.size(), *dev);
    return *t ? 0 : 1;
}

int main()
{
    CHECK(aclInit(nullptr));
    CHECK(aclrtSetDevice(0));
    aclrtStream stream;
    CHECK(aclrtCreateStream(&stream));
    uint32_t seed = 2024;
    auto next = [&] { seed = seed * 1664525u + 1013904223u; return seed >> 8; };
    uint64_t ws_size = 0;
    aclOpExecutor* exec = nullptr;
    double worst1 = 0.0, worst2 = 0.0;

    {   // ---- 1. W4A16: pack the weight on the device, then the weight-only matmul
        const int64_t M = 8, K = 256, N = 128;
        std::vector<uint16_t> x(M * K), scale(N), y(M * N, 0);
        std::vector<int32_t> w(K * N), packed(K * N / 8, 0);
        for (auto& v : x) v = float_to_half(((int)(next() % 2001) - 1000) * 1e-3f);
        for (auto& v : w) v = (int32_t)(next() % 16) - 8;
        for (auto& v : scale) v = float_to_half(0.01f + (next() % 100) * 1e-4f);
        void *d_x, *d_w, *d_p, *d_s, *d_y;
        aclTensor *t_x, *t_w, *t_p, *t_s, *t_y;
        CHECK(make_tensor(x, {M, K}, ACL_FLOAT16, &d_x, &t_x));
        CHECK(make_tensor(w, {K, N}, ACL_INT32, &d_w, &t_w));
        CHECK(make_tensor(packed, {K, N / 8}, ACL_INT32, &d_p, &t_p));
        CHECK(make_tensor(scale, {N}, ACL_FLOAT16, &d_s, &t_s));
        CHECK(make_tensor(y, {M, N}, ACL_FLOAT16, &d_y, &t_y));
        CHECK(aclnnConvertWeightToINT4PackGetWorkspaceSize(t_w, t_p, &ws_size, &exec));
        CHECK(aclnnConvertWeightToINT4Pack(nullptr, ws_size, exec, stream));
        CHECK(aclnnWeightQuantBatchMatmulV2GetWorkspaceSize(t_x, t_p, t_s, nullptr, nullptr, nullptr, nullptr, 0, t_y, &ws_size, &exec));
        void* ws = nullptr;
        if (ws_size > 0) CHECK(aclrtMalloc(&ws, ws_size, ACL_MEM_MALLOC_HUGE_FIRST));
        CHECK(aclnnWeightQuantBatchMatmulV2(ws, ws_size, exec, stream));
        CHECK(aclrtSynchronizeStream(stream));
        CHECK(aclrtMemcpy(y.data(), y.size() * 2, d_y, y.size() * 2, ACL_MEMCPY_DEVICE_TO_HOST));
        for (int64_t m = 0; m < M; m++)
            for (int64_t n = 0; n < N; n++) {
                double acc = 0.0;
                for (int64_t k = 0; k < K; k++)
                    acc += (double)half_to_float(x[m * K + k]) * (double)half_to_float(float_to_half((float)w[k * N + n] * half_to_float(scale[n])));
                const double rel = std::fabs(half_to_float(y[m * N + n]) - acc) / (std::fabs(acc) + 1e-2);
                if (rel > worst1) worst1 = rel;
            }
        std::printf("int32 carriers -> ConvertWeightToINT4Pack -> WeightQuantBatchMatmulV2 %ldx%ldx%ld: worst relative error %.3g\n",
                    (long)M, (long)K, (long)N, worst1);
        for (aclTensor* t : {t_x, t_w, t_p, t_s, t_y}) aclDestroyTensor(t);
        for (void* d : {d_x, d_w, d_p, d_s, d_y}) aclrtFree(d);
        if (ws) aclrtFree(ws);
    }
    {   // ---- 2. W8A8: quantise the activation per token on the device, then the int8 matmul with that scale as x1Scale
        const int64_t M = 64, K = 512, N = 96;
        std::vector<uint16_t> x(M * K), out(M * N, 0);
        std::vector<int8_t> q(M * K, 0), w(N * K);
        std::vector<float> s1(M, 0.0f), s2(N);
        for (auto& v : x) v = float_to_half(((int)(next() % 4001) - 2000) * 1e-3f);
        for (auto& v : w) v = (int8_t)((int)(next() % 255) - 127);
        for (auto& v : s2) v = 1e-3f + (next() % 1000) * 9e-6f;
        void *d_x, *d_q, *d_s1, *d_w, *d_s2, *d_out;
        aclTensor *t_x, *t_q, *t_s1, *t_w, *t_s2, *t_out;
        CHECK(make_tensor(x, {M, K}, ACL_FLOAT16, &d_x, &t_x));
        CHECK(make_tensor(q, {M, K}, ACL_INT8, &d_q, &t_q));
        CHECK(make_tensor(s1, {M}, ACL_FLOAT, &d_s1, &t_s1));
        CHECK(make_tensor(w, {N, K}, ACL_INT8, &d_w, &t_w));
        CHECK(make_tensor(s2, {N}, ACL_FLOAT, &d_s2, &t_s2));
        CHECK(make_tensor(out, {M, N}, ACL_FLOAT16, &d_out, &t_out));
        CHECK(aclnnDynamicQuantGetWorkspaceSize(t_x, nullptr, t_q, t_s1, &ws_size, &exec));
        CHECK(aclnnDynamicQuant(nullptr, ws_size, exec, stream));
        CHECK(aclnnQuantMatmulV5GetWorkspaceSize(t_q, t_w, t_s1, t_s2, nullptr, nullptr, nullptr, nullptr, nullptr, false, true, 0, t_out,
                                                 &ws_size, &exec));
        void* ws = nullptr;
        if (ws_size > 0) CHECK(aclrtMalloc(&ws, ws_size, ACL_MEM_MALLOC_HUGE_FIRST));
        CHECK(aclnnQuantMatmulV5(ws, ws_size, exec, stream));
        CHECK(aclrtSynchronizeStream(stream));
        CHECK(aclrtMemcpy(out.data(), out.size() * 2, d_out, out.size() * 2, ACL_MEMCPY_DEVICE_TO_HOST));
        // against the unquantised product: the error is the int8 quantisation's (half a step of 1/127 of a row's maximum per element)
        for (int64_t m = 0; m < M; m++)
            for (int64_t n = 0; n < N; n++) {
                double acc = 0.0, mag = 0.0;
                for (int64_t k = 0; k < K; k++) {
                    const double t = (double)half_to_float(x[m * K + k]) * (double)w[n * K + k] * (double)s2[n];
                    acc += t;
                    mag += std::fabs(t);
                }
                const double rel = std::fabs(half_to_float(out[m * N + n]) - acc) / (mag + 1e-6);
                if (rel > worst2) worst2 = rel;
            }
        std::printf("fp16 activation -> DynamicQuant -> QuantMatmulV5 %ldx%ldx%ld: worst error relative to sum|terms| %.3g\n", (long)M,
                    (long)K, (long)N, worst2);
        for (aclTensor* t : {t_x, t_q, t_s1, t_w, t_s2, t_out}) aclDestroyTensor(t);
        for (void* d : {d_x, d_q, d_s1, d_w, d_s2, d_out}) aclrtFree(d);
        if (ws) aclrtFree(ws);
    }
    aclrtDestroyStream(stream);
    aclFinalize();
    return (worst1 < 5e-3 && worst2 < 5e-3) ? 0 : 2;
}
