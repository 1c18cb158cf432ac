// What one decode-shaped call costs on the host: aclnnWeightQuantBatchMatmulV2, W8A16 per channel, bf16, 16 x 4096 x 4096
// with the weight stored [N, K], both phases per call as a serving loop issues them, 500 calls back to back on one
// stream.  Prints the host time per call (phase 1 + phase 2 enqueue) and the elapsed time per call with the GPU kept fed
// (wall clock around the whole loop including the final synchronisation): the larger of the two is what a step costs.
//
//   g++ -std=c++17 -I../../include decode_call_cost.cpp -L../lib -lopsnn_amd -Wl,-rpath,'$ORIGIN/../lib' -o decode_call_cost
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <vector>

#include "acl/acl.h"
#include "aclnnop/aclnn_weight_quant_batch_matmul_v2.h"

#define CHECK(expr)                                                                      \
    do {                                                                                 \
        int rc_ = (expr);                                                                \
        if (rc_ != 0) {                                                                  \
            std::printf("%s failed: %d (%s)\n", #expr, rc_, aclGetRecentErrMsg());       \
            return 1;                                                                    \
        }                                                                                \
    } while (0)

static aclTensor* tensor(void* dev, const std::vector<int64_t>& shape, const std::vector<int64_t>& strides, aclDataType dt)
{
    return aclCreateTensor(shape.data(), shape.size(), dt, strides.data(), 0, ACL_FORMAT_ND, shape.data(), shape.size(), dev);
}

int main()
{
    const int64_t M = 16, K = 4096, N = 4096;
    CHECK(aclInit(nullptr));
    CHECK(aclrtSetDevice(0));
    aclrtStream stream = nullptr;
    CHECK(aclrtCreateStream(&stream));
    void *dx, *dw, *ds, *dy;
    CHECK(aclrtMalloc(&dx, M * K * 2, ACL_MEM_MALLOC_HUGE_FIRST));
    CHECK(aclrtMalloc(&dw, N * K, ACL_MEM_MALLOC_HUGE_FIRST));
    CHECK(aclrtMalloc(&ds, N * 2, ACL_MEM_MALLOC_HUGE_FIRST));
    CHECK(aclrtMalloc(&dy, M * N * 2, ACL_MEM_MALLOC_HUGE_FIRST));
    {   // any finite contents will do: bf16 0.5 activations, weights 1, scales bf16 2^-7
        std::vector<uint16_t> hx(M * K, 0x3F00), hs(N, 0x3C00);
        std::vector<int8_t> hw(N * K, 1);
        CHECK(aclrtMemcpy(dx, hx.size() * 2, hx.data(), hx.size() * 2, ACL_MEMCPY_HOST_TO_DEVICE));
        CHECK(aclrtMemcpy(dw, hw.size(), hw.data(), hw.size(), ACL_MEMCPY_HOST_TO_DEVICE));
        CHECK(aclrtMemcpy(ds, hs.size() * 2, hs.data(), hs.size() * 2, ACL_MEMCPY_HOST_TO_DEVICE));
    }
    aclTensor* x = tensor(dx, {M, K}, {K, 1}, ACL_BF16);
    aclTensor* w = tensor(dw, {K, N}, {1, K}, ACL_INT8);   // logical [K, N] over [N, K] storage
    aclTensor* s = tensor(ds, {N}, {1}, ACL_BF16);
    aclTensor* y = tensor(dy, {M, N}, {N, 1}, ACL_BF16);
    if (!x || !w || !s || !y) { std::printf("aclCreateTensor failed\n"); return 1; }

    auto one_call = [&]() -> int {
        uint64_t ws = 0;
        aclOpExecutor* ex = nullptr;
        CHECK(aclnnWeightQuantBatchMatmulV2GetWorkspaceSize(x, w, s, nullptr, nullptr, nullptr, nullptr, 0, y, &ws, &ex));
        if (ws != 0) { std::printf("unexpected workspace %llu\n", (unsigned long long)ws); return 1; }
        CHECK(aclnnWeightQuantBatchMatmulV2(nullptr, 0, ex, stream));
        return 0;
    };
    for (int i = 0; i < 50; i++) if (one_call()) return 1;
    CHECK(aclrtSynchronizeStream(stream));

    const int calls = 500;
    using clk = std::chrono::steady_clock;
    const auto t0 = clk::now();
    for (int i = 0; i < calls; i++) if (one_call()) return 1;
    const auto t1 = clk::now();
    CHECK(aclrtSynchronizeStream(stream));
    const auto t2 = clk::now();
    const double host_us = std::chrono::duration<double, std::micro>(t1 - t0).count() / calls;
    const double total_us = std::chrono::duration<double, std::micro>(t2 - t0).count() / calls;
    std::printf("decode call cost, W8A16 %lld x %lld x %lld: host %.2f us per call (phase 1 + phase 2 enqueue), %.2f us per call end to end over %d calls\n",
                (long long)M, (long long)K, (long long)N, host_us, total_us, calls);
    aclDestroyTensor(x); aclDestroyTensor(w); aclDestroyTensor(s); aclDestroyTensor(y);
    aclrtFree(dx); aclrtFree(dw); aclrtFree(ds); aclrtFree(dy);
    aclrtDestroyStream(stream);
    aclFinalize();
    return 0;
}
