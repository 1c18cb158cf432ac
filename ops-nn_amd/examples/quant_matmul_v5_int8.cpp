// A caller of aclnnQuantMatmulV5 written the way users of the reference write theirs (two phases, ACL runtime
// objects), linked against libopsnn_amd.so.  int8 x int8 with per-token and per-channel fp32 scales, bf16 output;
// the result is verified on the host with a plain triple loop.
//
//   g++ -std=c++17 -I../../include quant_matmul_v5_int8.cpp -L../lib -lopsnn_amd -Wl,-rpath,'$ORIGIN/../lib' -o qmm_v5_int8
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "acl/acl.h"
#include "aclnnop/aclnn_quant_matmul_v5.h"

#define CHECK(expr)                                                                      \
    do {                                                                                 \
        int rc_ = (expr);                                                                \
        if (rc_ != 0) {                                                                  \
            std::printf("%s failed: %d (%s)\n", #expr, rc_, aclGetRecentErrMsg());       \
            return 1;                                                                    \
        }                                                                                \
    } while (0)

static float bf16_to_float(uint16_t b)
{
    uint32_t u = (uint32_t)b << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

template <class T>
static int upload(const std::vector<T>& host, const std::vector<int64_t>& shape, aclDataType dt, void** dev, aclTensor** t)
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
    const int64_t M = 96, K = 320, N = 160;
    CHECK(aclInit(nullptr));
    CHECK(aclrtSetDevice(0));
    aclrtStream stream;
    CHECK(aclrtCreateStream(&stream));

    std::vector<int8_t> x1(M * K), x2(N * K);   // x2 stored [N, K] and passed with transposeX2 = true
    std::vector<float> s1(M), s2(N);
    uint32_t seed = 12345;
    auto next = [&] { seed = seed * 1664525u + 1013904223u; return seed >> 8; };
    for (auto& v : x1) v = (int8_t)((int)(next() % 255) - 127);
    for (auto& v : x2) v = (int8_t)((int)(next() % 255) - 127);
    for (auto& v : s1) v = 1e-3f + (next() % 1000) * 9e-6f;
    for (auto& v : s2) v = 1e-3f + (next() % 1000) * 9e-6f;
    std::vector<uint16_t> out(M * N, 0);

    void *d_x1 = nullptr, *d_x2 = nullptr, *d_s1 = nullptr, *d_s2 = nullptr, *d_out = nullptr;
    aclTensor *t_x1 = nullptr, *t_x2 = nullptr, *t_s1 = nullptr, *t_s2 = nullptr, *t_out = nullptr;
    CHECK(upload(x1, {M, K}, ACL_INT8, &d_x1, &t_x1));
    CHECK(upload(x2, {N, K}, ACL_INT8, &d_x2, &t_x2));
    CHECK(upload(s1, {M}, ACL_FLOAT, &d_s1, &t_s1));
    CHECK(upload(s2, {N}, ACL_FLOAT, &d_s2, &t_s2));
    CHECK(upload(out, {M, N}, ACL_BF16, &d_out, &t_out));

    uint64_t ws_size = 0;
    aclOpExecutor* exec = nullptr;
    CHECK(aclnnQuantMatmulV5GetWorkspaceSize(t_x1, t_x2, t_s1, t_s2, nullptr, nullptr, nullptr, nullptr, nullptr,
                                             false, true, 0, t_out, &ws_size, &exec));
    void* ws = nullptr;
    if (ws_size > 0) CHECK(aclrtMalloc(&ws, ws_size, ACL_MEM_MALLOC_HUGE_FIRST));
    CHECK(aclnnQuantMatmulV5(ws, ws_size, exec, stream));
    CHECK(aclrtSynchronizeStream(stream));
    CHECK(aclrtMemcpy(out.data(), out.size() * 2, d_out, out.size() * 2, ACL_MEMCPY_DEVICE_TO_HOST));

    double worst = 0.0;
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            int32_t acc = 0;
            for (int64_t k = 0; k < K; k++) acc += (int32_t)x1[m * K + k] * (int32_t)x2[n * K + k];
            const float want = (float)acc * s2[n] * s1[m];
            const float got = bf16_to_float(out[m * N + n]);
            const double rel = std::fabs(got - want) / (std::fabs(want) + 1e-6);
            if (rel > worst) worst = rel;
        }
    std::printf("quant_matmul_v5 int8 %ldx%ldx%ld: workspace %lu B, worst relative error %.3g (bf16 rounding is 3.9e-3)\n",
                (long)M, (long)K, (long)N, (unsigned long)ws_size, worst);

    for (aclTensor* t : {t_x1, t_x2, t_s1, t_s2, t_out}) aclDestroyTensor(t);
    for (void* d : {d_x1, d_x2, d_s1, d_s2, d_out}) aclrtFree(d);
    if (ws) aclrtFree(ws);
    aclrtDestroyStream(stream);
    aclFinalize();
    return worst < 4e-3 ? 0 : 2;
}
