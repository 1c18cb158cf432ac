// Plain strided kernels: one thread per output element, any strides, any K, every supported dtype.
// They are the fallback for shapes and layouts the MFMA kernels do not take, and they evaluate the
// reference formulas operation by operation in ascending-k order (no fused multiply-add where the
// golden rounds twice), so on small cases they can be compared bit for bit with a sequential CPU
// evaluation.
//
// Formulas: matmul/quant_batch_matmul_v3/tests/assets/qbmmv3_kernel_golden.py:153-234 (MX), 237-358 (block scale);
//           matmul/weight_quant_batch_matmul_v2/tests/assets/wqbmmv2_kernel_golden.py:199-352 (weight-only).
#include "common.hip.h"
#include "launch.h"

namespace opsnn {

struct PlainQmmParams {
    OpsnnQmmArgs a;
};

// block scale: out = sum_kb (sum_{k in kb} x1*x2) * (s1[m/gsM, kb] * s2[kb, n/gsN])
__global__ void qmm_blockscale_plain(OpsnnQmmArgs a)
{
    const int64_t nchunks = (a.N + blockDim.x - 1) / blockDim.x;
    const int64_t m = blockIdx.x / nchunks;
    const int64_t n = (blockIdx.x % nchunks) * (int64_t)blockDim.x + threadIdx.x;
    const int64_t bz = blockIdx.y;
    if (n >= a.N) return;
    const int64_t gsM = a.gsM > 0 ? a.gsM : 1, gsN = a.gsN > 0 ? a.gsN : 1, gsK = a.gsK > 0 ? a.gsK : a.K;
    const float* s1 = (const float*)a.x1_scale_mat.ptr + bz * a.x1_scale_mat.batch_stride;
    const float* s2 = (const float*)a.x2_scale_mat.ptr + bz * a.x2_scale_mat.batch_stride;
    const int64_t abase = bz * a.x1.batch_stride + m * a.x1.row_stride;
    const int64_t bbase = bz * a.x2.batch_stride + n * a.x2.col_stride;
    float acc = 0.0f;
    for (int64_t k0 = 0, kb = 0; k0 < a.K; k0 += gsK, kb++) {
        const int64_t k1 = k0 + gsK < a.K ? k0 + gsK : a.K;
        float part = 0.0f;
        for (int64_t k = k0; k < k1; k++) {
            float x = load_q_as_f32(a.x1.ptr, a.x1_dtype, abase + k * a.x1.col_stride);
            float w = load_q_as_f32(a.x2.ptr, a.x2_dtype, bbase + k * a.x2.row_stride);
            part = __fadd_rn(part, __fmul_rn(x, w));
        }
        float sa = s1[(m / gsM) * a.x1_scale_mat.row_stride + kb * a.x1_scale_mat.col_stride];
        float sb = s2[kb * a.x2_scale_mat.row_stride + (n / gsN) * a.x2_scale_mat.col_stride];
        acc = __fadd_rn(acc, __fmul_rn(part, __fmul_rn(sa, sb)));
    }
    if (a.bias) acc = __fadd_rn(acc, load_scalar_as_f32(a.bias, a.bias_dtype, bz * a.bias_batch_stride + n));
    store_f32_as(a.out, a.out_dtype, (bz * a.M + m) * a.N + n, acc);
}

// MX: out = sum_k (x1 * 2^e1[m, k/32]) * (x2 * 2^e2[k/32, n]) + bias
__global__ void qmm_mx_plain(OpsnnQmmArgs a)
{
    const int64_t nchunks = (a.N + blockDim.x - 1) / blockDim.x;
    const int64_t m = blockIdx.x / nchunks;
    const int64_t n = (blockIdx.x % nchunks) * (int64_t)blockDim.x + threadIdx.x;
    const int64_t bz = blockIdx.y;
    if (n >= a.N) return;
    const uint8_t* s1 = (const uint8_t*)a.x1_scale_mat.ptr + bz * a.x1_scale_mat.batch_stride + m * a.x1_scale_mat.row_stride;
    const uint8_t* s2 = (const uint8_t*)a.x2_scale_mat.ptr + bz * a.x2_scale_mat.batch_stride + n * a.x2_scale_mat.row_stride;
    const int64_t abase = bz * a.x1.batch_stride + m * a.x1.row_stride;
    const int64_t bbase = bz * a.x2.batch_stride + n * a.x2.col_stride;
    float acc = 0.0f;
    for (int64_t k = 0; k < a.K; k++) {
        const int64_t kb = k >> 5;
        float sa = e8m0_to_f32(s1[(kb >> 1) * a.x1_scale_mat.col_stride + (kb & 1)]);
        float sb = e8m0_to_f32(s2[(kb >> 1) * a.x2_scale_mat.col_stride + (kb & 1)]);
        float x = __fmul_rn(load_q_as_f32(a.x1.ptr, a.x1_dtype, abase + k * a.x1.col_stride), sa);
        float w = __fmul_rn(load_q_as_f32(a.x2.ptr, a.x2_dtype, bbase + k * a.x2.row_stride), sb);
        acc = __fadd_rn(acc, __fmul_rn(x, w));
    }
    if (a.bias) acc = __fadd_rn(acc, load_scalar_as_f32(a.bias, a.bias_dtype, bz * a.bias_batch_stride + n));
    store_f32_as(a.out, a.out_dtype, (bz * a.M + m) * a.N + n, acc);
}

__device__ __forceinline__ float round_through(float v, int dt)
{
    if (dt == DT_F16) return f16_to_f32(f16_bits(v));
    if (dt == DT_BF16) return bf16_to_f32(bf16_bits(v));
    return v;
}

// weight-only: y = x @ T(T(w + off) * s) + bias;  T = rounding through x's dtype
__global__ void wqmm_plain(OpsnnWqmmArgs a)
{
    const int64_t nchunks = (a.N + blockDim.x - 1) / blockDim.x;
    const int64_t m = blockIdx.x / nchunks;
    const int64_t n = (blockIdx.x % nchunks) * (int64_t)blockDim.x + threadIdx.x;
    if (n >= a.N) return;
    const int T = a.x_dtype;
    const bool mx = a.scale_dtype == DT_E8M0;
    const int64_t g = a.group > 0 ? a.group : a.K;
    float acc = 0.0f;
    for (int64_t k = 0; k < a.K; k++) {
        const int64_t gi = k / g;
        const int64_t si = gi * a.scale.row_stride + (a.scale_n == 1 ? 0 : n) * a.scale.col_stride;
        float w = load_q_as_f32(a.w.ptr, a.w_dtype, k * a.w.row_stride + n * a.w.col_stride);
        if (mx) {
            float s = e8m0_to_f32(((const uint8_t*)a.scale.ptr)[si]);
            if (T == DT_F16) s = round_through(s, DT_F16);
            w = round_through(__fmul_rn(w, s), T);
        } else {
            float s = load_scalar_as_f32(a.scale.ptr, a.scale_dtype, si);
            if (a.offset) w = round_through(__fadd_rn(w, load_scalar_as_f32(a.offset, a.scale_dtype, si)), T);
            w = round_through(__fmul_rn(w, s), T);
        }
        float x = load_scalar_as_f32(a.x, T, m * a.K + k);
        acc = __fadd_rn(acc, __fmul_rn(x, w));
    }
    if (a.bias) acc = __fadd_rn(acc, load_scalar_as_f32(a.bias, a.bias_dtype, n));
    if (T == DT_BF16) acc = round_through(acc, DT_BF16);
    store_f32_as(a.y, T, m * a.N + n, acc);
}

int launch_blockscale_plain(const OpsnnQmmArgs& a, hipStream_t st)
{
    dim3 block(256), grid((unsigned)(((a.N + 255) / 256) * a.M), (unsigned)a.batch);
    hipLaunchKernelGGL(qmm_blockscale_plain, grid, block, 0, st, a);
    return (int)hipGetLastError();
}
int launch_mx_plain(const OpsnnQmmArgs& a, hipStream_t st)
{
    dim3 block(256), grid((unsigned)(((a.N + 255) / 256) * a.M), (unsigned)a.batch);
    hipLaunchKernelGGL(qmm_mx_plain, grid, block, 0, st, a);
    return (int)hipGetLastError();
}
int launch_wqmm_plain(const OpsnnWqmmArgs& a, hipStream_t st)
{
    dim3 block(256), grid((unsigned)(((a.N + 255) / 256) * a.M));
    hipLaunchKernelGGL(wqmm_plain, grid, block, 0, st, a);
    return (int)hipGetLastError();
}

}  // namespace opsnn
