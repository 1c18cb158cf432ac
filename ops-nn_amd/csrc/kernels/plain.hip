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

// per-tensor / per-channel family: see opsnnQmmTc in opsnn_kernels.h and qbmmv3_kernel_golden.py:390-513
__device__ __forceinline__ float trunc19(float s) { return u2f(f2u(s) & 0xFFFFE000u); }
__device__ __forceinline__ float s9f(float v)
{
    const float r = __builtin_rintf(v);   // round half to even
    return r < -256.0f ? -256.0f : (r > 255.0f ? 255.0f : r);
}
__global__ void qmm_tc_plain(OpsnnQmmArgs a)
{
    const int64_t nchunks = (a.N + blockDim.x - 1) / blockDim.x;
    const int64_t m = blockIdx.x / nchunks;
    const int64_t n = (blockIdx.x % nchunks) * (int64_t)blockDim.x + threadIdx.x;
    const int64_t bz = blockIdx.y;
    if (n >= a.N) return;
    const bool is_int = a.x1_dtype == DT_I8;
    const int64_t abase = bz * a.x1.batch_stride + m * a.x1.row_stride;
    const int64_t bbase = bz * a.x2.batch_stride + n * a.x2.col_stride;
    int32_t iacc = 0;
    float facc = 0.0f;
    if (is_int) {
        const int8_t* x1 = (const int8_t*)a.x1.ptr;
        const int8_t* x2 = (const int8_t*)a.x2.ptr;
        for (int64_t k = 0; k < a.K; k++) iacc += (int32_t)x1[abase + k * a.x1.col_stride] * (int32_t)x2[bbase + k * a.x2.row_stride];
    } else {
        for (int64_t k = 0; k < a.K; k++) {
            const float x = load_q_as_f32(a.x1.ptr, a.x1_dtype, abase + k * a.x1.col_stride);
            const float w = load_q_as_f32(a.x2.ptr, a.x2_dtype, bbase + k * a.x2.row_stride);
            facc = __fadd_rn(facc, __fmul_rn(x, w));
        }
    }
    const int64_t si = a.x2_scale_len == 1 ? 0 : n;
    const bool u64 = a.x2_scale_dtype == DT_U64;
    const uint64_t packed = u64 ? ((const uint64_t*)a.x2_scale)[si] : 0;
    const float s = u64 ? trunc19(u2f((uint32_t)packed)) : load_scalar_as_f32(a.x2_scale, a.x2_scale_dtype, si);
    const int64_t bi = bz * a.bias_batch_stride + n;
    const int64_t o_idx = (bz * a.M + m) * a.N + n;
    const bool bias_i32 = a.bias && a.bias_dtype == DT_I32, bias_float = a.bias && a.bias_dtype != DT_I32;
    if (a.out_dtype == DT_I8) {
        int32_t v = iacc;
        if (bias_i32) v += ((const int32_t*)a.bias)[bi];
        float o = s9f(__fmul_rn((float)v, s));
        bool has_off = a.x2_offset != nullptr || u64;
        if (has_off) {
            float off;
            if (a.x2_offset) off = a.x2_offset[a.x2_offset_len == 1 ? 0 : n];
            else {
                int64_t raw = (int64_t)((packed >> 37) & 0x1FF);
                if (raw & 0x100) raw -= 0x200;
                off = (float)raw;
            }
            o = __fadd_rn(s9f(o), s9f(off));
        }
        o = o < -128.0f ? -128.0f : (o > 127.0f ? 127.0f : o);
        ((int8_t*)a.out)[o_idx] = (int8_t)o;
        return;
    }
    if (a.out_dtype == DT_I32) {
        int32_t v = iacc;
        if (bias_i32) v += ((const int32_t*)a.bias)[bi];
        else if (bias_float) v = (int32_t)__fadd_rn((float)v, load_scalar_as_f32(a.bias, a.bias_dtype, bi));
        ((int32_t*)a.out)[o_idx] = v;
        return;
    }
    const bool pertoken = a.x1_scale != nullptr;
    const bool do_scale_gen = is_int && a.x2_scale_len == 1 && !(a.bias && (a.bias_dtype == DT_BF16 || a.bias_dtype == DT_F32));
    const bool is_bias_vec = bias_float && (is_int || pertoken);
    float o;
    if (is_int) {
        int32_t v = iacc;
        if (!is_bias_vec && bias_i32) v += ((const int32_t*)a.bias)[bi];
        o = (float)v;
    } else {
        o = facc;
    }
    if (!is_bias_vec && bias_float) o = __fadd_rn(o, load_scalar_as_f32(a.bias, a.bias_dtype, bi));
    if (pertoken) {
        // one-element x1Scale: the double-scale modes; one per row: K-C / K-T (compute_pertoken, no truncation)
        const float pt = ((const float*)a.x1_scale)[a.x1_scale_len == 1 ? 0 : m];
        if (a.x1_scale_len == 1 && a.x2_scale_len == 1 && !is_bias_vec) o = __fmul_rn(o, trunc19(__fmul_rn(s, pt)));
        else o = __fmul_rn(__fmul_rn(o, do_scale_gen ? trunc19(s) : s), pt);
    } else {
        o = __fmul_rn(o, do_scale_gen ? trunc19(s) : s);
    }
    if (is_bias_vec) o = __fadd_rn(o, load_scalar_as_f32(a.bias, a.bias_dtype, bi));
    store_f32_as(a.out, a.out_dtype, o_idx, o);
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

// K-group modes of quant_batch_matmul_v4: see opsnnQmmGroup in opsnn_kernels.h and qbmmv4_kernel_golden.py:189-255, 328-395
__global__ void qmm_tcg_plain(OpsnnQmmArgs a)
{
    const int64_t nchunks = (a.N + blockDim.x - 1) / blockDim.x;
    const int64_t m = blockIdx.x / nchunks;
    const int64_t n = (blockIdx.x % nchunks) * (int64_t)blockDim.x + threadIdx.x;
    if (n >= a.N) return;
    const int64_t abase = m * a.x1.row_stride, bbase = n * a.x2.col_stride;
    const int sdt = a.x2_scale_dtype;
    float acc = 0.0f;
    for (int64_t k = 0; k < a.K; k++) {
        const float x = load_q_as_f32(a.x1.ptr, a.x1_dtype, abase + k * a.x1.col_stride);
        const float w4 = load_q_as_f32(a.x2.ptr, a.x2_dtype, bbase + k * a.x2.row_stride);
        const float sc = load_scalar_as_f32(a.x2_scale_mat.ptr, sdt, (k / a.gsK) * a.x2_scale_mat.row_stride + n * a.x2_scale_mat.col_stride);
        const float mid = round_through(__fmul_rn(round_through(w4, sdt), sc), sdt);
        const float w = e4m3_to_f32(f32_to_e4m3_bits(mid));
        acc = __fadd_rn(acc, __fmul_rn(x, w));
    }
    if (a.y_scale) acc = __fmul_rn(acc, trunc19(u2f((uint32_t)((const uint64_t*)a.y_scale)[a.y_scale_len == 1 ? 0 : n])));
    if (a.bias) acc = __fadd_rn(acc, load_scalar_as_f32(a.bias, a.bias_dtype, n));
    store_f32_as(a.out, a.out_dtype, m * a.N + n, acc);
}
// Prologue of the matrix-core path of the same mode: the re-quantised weight once, as e4m3 bytes [N, K] K-contiguous
// (the per-element operation of the loop above, so the bytes are the oracle's), the decoded output scale per column
// (1.0 when absent) and a 1.0 for the row scale.  x2 is [N, K] with two fp4 per byte, low nibble first; thread t turns
// the 32 elements k0 .. k0+31 of row n (16 bytes in, 32 bytes out), t = n * K/32 + k0/32.  They share one scale
// (gsK % 32 == 0), and every step of the operation is odd in the weight, so the thread converts the 8 magnitudes once
// into a table of 8 bytes and each element is a table byte with the nibble's sign bit.
// Rows of w8 are Kp >= K bytes long (K rounded up to the matrix-core kernels' 128): the tail is written as zeros.
__global__ __launch_bounds__(256) void tcg_requant_kernel(OpsnnQmmArgs a, uint8_t* w8, float* cs, float* one, int64_t Kp)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t kq = Kp / 32;
    if (t == 0) one[0] = 1.0f;
    if (t < a.N) cs[t] = a.y_scale ? trunc19(u2f((uint32_t)((const uint64_t*)a.y_scale)[a.y_scale_len == 1 ? 0 : t])) : 1.0f;
    if (t >= a.N * kq) return;
    const int64_t n = t / kq, k0 = (t % kq) * 32;
    if (k0 >= a.K) {
        uint4* z = (uint4*)(w8 + n * Kp + k0);
        z[0] = z[1] = make_uint4(0, 0, 0, 0);
        return;
    }
    const int sdt = a.x2_scale_dtype;
    const float sc = load_scalar_as_f32(a.x2_scale_mat.ptr, sdt, (k0 / a.gsK) * a.x2_scale_mat.row_stride + n * a.x2_scale_mat.col_stride);
    uint64_t table = 0;
#pragma unroll
    for (uint32_t v = 0; v < 8; v++) {
        const float mid = round_through(__fmul_rn(round_through(e2m1_to_f32(v), sdt), sc), sdt);
        table |= (uint64_t)(f32_to_e4m3_bits(mid) & 0x7fu) << (8 * v);
    }
    if (sc < 0.0f || f2u(sc) == 0x80000000u) table |= 0x8080808080808080ull;   // a negative scale turns every sign
    const uint4 in = *(const uint4*)((const uint8_t*)a.x2.ptr + (n * a.K + k0) / 2);
    const uint32_t words[4] = {in.x, in.y, in.z, in.w};
    uint32_t o[8];
#pragma unroll
    for (int w = 0; w < 8; w++) {
        const uint32_t nib = (words[w >> 1] >> (16 * (w & 1))) & 0xffffu;
        uint32_t r = 0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t q = (nib >> (4 * e)) & 15u;
            const uint32_t b = (uint32_t)(table >> (8 * (q & 7u))) & 0xffu;
            r |= (b ^ ((q & 8u) << 4)) << (8 * e);
        }
        o[w] = r;
    }
    uint4* dst = (uint4*)(w8 + n * Kp + k0);
    dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
    dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
}
// x1 [M, K] (rows of 16-byte pieces) into rows of Kp bytes, the tail zero
__global__ __launch_bounds__(256) void tcg_pad_x1_kernel(const uint8_t* __restrict__ src, int64_t ld, uint8_t* __restrict__ dst, int64_t M, int64_t K, int64_t Kp)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x, pieces = Kp / 16;
    if (i >= M * pieces) return;
    const int64_t r = i / pieces, c = i - r * pieces;
    *(uint4*)(dst + r * Kp + c * 16) = c * 16 < K ? *(const uint4*)(src + r * ld + c * 16) : make_uint4(0, 0, 0, 0);
}
__global__ void qmm_i4_asym_plain(OpsnnQmmArgs a)
{
    const int64_t nchunks = (a.N + blockDim.x - 1) / blockDim.x;
    const int64_t m = blockIdx.x / nchunks;
    const int64_t n = (blockIdx.x % nchunks) * (int64_t)blockDim.x + threadIdx.x;
    if (n >= a.N) return;
    const int64_t abase = m * a.x1.row_stride, bbase = n * a.x2.col_stride;
    const int64_t G = (a.K + a.gsK - 1) / a.gsK;
    float out = 0.0f;
    for (int64_t g = 0; g < G; g++) {
        const int64_t k0 = g * a.gsK, k1 = (g + 1) * a.gsK < a.K ? (g + 1) * a.gsK : a.K;
        int32_t mm = 0, rs = 0;
        for (int64_t k = k0; k < k1; k++) {
            const int32_t xa = (int32_t)load_q_as_f32(a.x1.ptr, DT_I4, abase + k * a.x1.col_stride);
            const int32_t xb = (int32_t)load_q_as_f32(a.x2.ptr, DT_I4, bbase + k * a.x2.row_stride);
            mm += xa * xb;
            rs += xa;
        }
        const float off = __fmul_rn((float)rs, load_scalar_as_f32(a.x2_offset_mat.ptr, DT_F16, g * a.x2_offset_mat.row_stride + n * a.x2_offset_mat.col_stride));
        const float sc = ((const float*)a.x2_scale_mat.ptr)[g * a.x2_scale_mat.row_stride + n * a.x2_scale_mat.col_stride];
        out = __fadd_rn(out, __fmul_rn(__fsub_rn((float)mm, off), sc));
    }
    out = __fmul_rn(out, ((const float*)a.x1_scale)[m]);
    store_f32_as(a.out, a.out_dtype, m * a.N + n, out);
}
int launch_fp8_rowcol_mfma(const OpsnnQmmArgs& a, hipStream_t st, bool merged_scales_ok, SplitK sk = {});   // qmm_fp8_block.hip

int launch_rowcol_rows(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk);      // qmm_fp8_rows.hip
int launch_rowcol_decode(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk);    // qmm_fp8_decode.hip
void* weight_cache_blob3(const void* src, const void* src2, const void* src3, int64_t K, int64_t N, int bits, int64_t nb, uint64_t bytes, hipStream_t st,
                         bool* fresh);   // weight_cache.hip
void weight_cache_commit(void* buffer, hipStream_t st);

static inline uint64_t align256(uint64_t v) { return (v + 255) / 256 * 256; }
// The re-quantised weight with its side values: e4m3 bytes [N, K], the decoded output scale per column, a 1.0.
static inline int64_t tcg_kp(const OpsnnQmmArgs& a) { return (a.K + 127) / 128 * 128; }   // K as the matrix-core kernels walk it
static inline uint64_t tcg_blob_bytes(const OpsnnQmmArgs& a) { return align256((uint64_t)a.N * tcg_kp(a)) + align256((uint64_t)a.N * 4) + 256; }
// a K tail: x1 copied into rows of Kp bytes behind the blob
static inline uint64_t tcg_x1pad_bytes(const OpsnnQmmArgs& a) { return tcg_kp(a) != a.K ? align256((uint64_t)a.M * tcg_kp(a)) : 0; }
// 17 .. 128 rows go to the many-rows streaming kernel, which wants x1 widened to fp16 (M * Kp * 2 bytes behind those)
static inline uint64_t tcg_rows_bytes(const OpsnnQmmArgs& a) { return a.M > 16 && a.M <= 128 ? (uint64_t)a.M * tcg_kp(a) * 2 : 0; }
// Workspace of the matrix-core path of the fp8 x fp4 group-scale mode (0: the shape stays on the plain kernel).
uint64_t tcg_workspace_bytes(const OpsnnQmmArgs& a)
{
    if (a.x1_dtype != DT_E4M3 || a.x2_dtype != DT_E2M1 || a.batch != 1) return 0;
    if (a.K % 32 != 0 || a.K < 128 || a.gsK <= 0 || a.gsK % 32 != 0 || (uintptr_t)a.x2.ptr % 16 != 0 || a.M * a.N < 64 * 64) return 0;
    if (a.x1.col_stride != 1 || a.x2.row_stride != 1 || a.x2.col_stride != a.K) return 0;
    // x1 in 16-byte pieces: what the matrix-core kernels (and the padded copy of a K tail) move; checked here, before the
    // re-quantisation is launched or cached, so that no later step of launch_tcg_mfma can still decline the call
    if (((uintptr_t)a.x1.ptr | (uint64_t)a.x1.row_stride) % 16 != 0 || a.x1.row_stride < a.K) return 0;
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16) return 0;
    if (a.bias && a.bias_dtype != DT_F32) return 0;
    return tcg_blob_bytes(a) + tcg_x1pad_bytes(a) + tcg_rows_bytes(a);
}
// Re-quantise x2 into the workspace -- or, with the weight cache on and dense scales, once into a cached buffer that
// later calls with the same x2, scales and output scale find again -- then an fp8 kernel with a column scale (the
// decoded output scale) and a unit row scale: the streaming kernels with up to 128 rows of x1, else the tile kernel.
int launch_tcg_mfma(const OpsnnQmmArgs& a, hipStream_t st)
{
    const uint64_t need = tcg_workspace_bytes(a);
    if (!need || !a.workspace || (uintptr_t)a.workspace % 16 != 0) return OPSNN_NOT_TAKEN;
    const uint64_t blob = tcg_blob_bytes(a);
    uint8_t* w8 = (uint8_t*)a.workspace;
    // what the cache key has to tell apart beside the three pointers, K, N and the size: group size, scale type, which
    // way the dense scale matrix lies, one output scale or N
    const int64_t Kp = tcg_kp(a);
    const int64_t kg = (a.K + a.gsK - 1) / a.gsK;
    const bool s_nk = a.x2_scale_mat.row_stride == 1 && a.x2_scale_mat.col_stride == kg;
    const bool s_kn = a.x2_scale_mat.row_stride == a.N && a.x2_scale_mat.col_stride == 1;
    const bool dense = s_nk || s_kn;
    const int64_t key = (a.gsK << 8) | ((int64_t)(a.x2_scale_dtype & 31) << 3) | (s_nk ? 4 : 0) | (a.y_scale_len == 1 ? 2 : 0) | 1;
    bool fresh = false;
    void* cached = dense ? weight_cache_blob3(a.x2.ptr, a.x2_scale_mat.ptr, a.y_scale, a.K, a.N, 4, key, blob, st, &fresh) : nullptr;
    if (cached) w8 = (uint8_t*)cached;
    float* cs = (float*)(w8 + align256((uint64_t)a.N * Kp));
    float* one = (float*)((char*)cs + align256((uint64_t)a.N * 4));
    if (!cached || fresh) {
        const int64_t threads = a.N * (Kp / 32);   // >= N since Kp >= 128
        hipLaunchKernelGGL(tcg_requant_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, a, w8, cs, one, Kp);
        if (cached) weight_cache_commit(cached, st);
    }
    OpsnnQmmArgs b = a;
    if (Kp != a.K) {   // a K tail: x1 into rows of Kp bytes behind the blob's place in the workspace; zero products change no sum
        uint8_t* x1p = (uint8_t*)a.workspace + blob;
        const int64_t pieces = a.M * (Kp / 16);
        hipLaunchKernelGGL(tcg_pad_x1_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, st, (const uint8_t*)a.x1.ptr, a.x1.row_stride, x1p,
                           a.M, a.K, Kp);
        b.x1.ptr = x1p; b.x1.row_stride = Kp; b.K = Kp;
    }
    b.x2.ptr = w8; b.x2_dtype = DT_E4M3; b.x2.row_stride = 1; b.x2.col_stride = Kp; b.x2.batch_stride = 0;
    b.x1_scale = one; b.x1_scale_len = 1;
    b.x2_scale = cs; b.x2_scale_dtype = DT_F32; b.x2_scale_len = a.N;
    b.workspace = tcg_rows_bytes(a) ? (char*)a.workspace + blob + tcg_x1pad_bytes(a) : nullptr;
    if (a.force_variant == 0) {
        int rc = launch_rowcol_rows(b, st, SplitK{});
        if (rc != OPSNN_NOT_TAKEN) return rc;
        rc = launch_rowcol_decode(b, st, SplitK{});
        if (rc != OPSNN_NOT_TAKEN) return rc;
    }
    return launch_fp8_rowcol_mfma(b, st, true);
}
int launch_group_plain(const OpsnnQmmArgs& a, bool tcg, hipStream_t st)
{
    dim3 block(256), grid((unsigned)(((a.N + 255) / 256) * a.M));
    if (tcg) hipLaunchKernelGGL(qmm_tcg_plain, grid, block, 0, st, a);
    else hipLaunchKernelGGL(qmm_i4_asym_plain, grid, block, 0, st, a);
    return (int)hipGetLastError();
}
int launch_blockscale_plain(const OpsnnQmmArgs& a, hipStream_t st)
{
    dim3 block(256), grid((unsigned)(((a.N + 255) / 256) * a.M), (unsigned)a.batch);
    hipLaunchKernelGGL(qmm_blockscale_plain, grid, block, 0, st, a);
    return (int)hipGetLastError();
}
int launch_tc_plain(const OpsnnQmmArgs& a, hipStream_t st)
{
    dim3 block(256), grid((unsigned)(((a.N + 255) / 256) * a.M), (unsigned)a.batch);
    hipLaunchKernelGGL(qmm_tc_plain, grid, block, 0, st, a);
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
