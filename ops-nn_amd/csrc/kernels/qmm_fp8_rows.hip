// fp8 e4m3 block-scale matmul (G-B, B-B) with 17 .. 128 rows of x1: the many-rows streaming kernel of wqmm_stream.hip.h
// in its block-scale form (WF = 3).  A pre-step widens x1 to fp16 in the workspace (exact; M * K * 2 bytes), so that x
// travels global -> LDS by asynchronous copies like the activations of the weight-only path; x2 is streamed once and
// widened in registers.  Formula and arithmetic: see qmm_fp8_decode.hip (exact products, fp32 sums per half block, one
// fused multiply-add per half block and output).
#include <cstdlib>

#include "wqmm_stream.hip.h"

namespace opsnn {
namespace {

// 16 e4m3 bytes -> 16 fp16
__global__ __launch_bounds__(256) void widen_e4m3_f16_kernel(const uint8_t* __restrict__ src, int64_t ld, uint16_t* __restrict__ dst, int64_t rows, int64_t K)
{
    const int64_t pieces = K / 16;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * pieces) return;
    const int64_t r = i / pieces, c = i - r * pieces;
    const uint4 v = *(const uint4*)(src + r * ld + c * 16);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[8];
#pragma unroll
    for (int d = 0; d < 4; d++) {
        typedef _Float16 h2v __attribute__((ext_vector_type(2)));
        o[2 * d] = __builtin_bit_cast(uint32_t, (h2v)__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[d], 1.0f, false));
        o[2 * d + 1] = __builtin_bit_cast(uint32_t, (h2v)__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[d], 1.0f, true));
    }
    uint4* out = (uint4*)(dst + r * K + c * 16);
    out[0] = make_uint4(o[0], o[1], o[2], o[3]);
    out[1] = make_uint4(o[4], o[5], o[6], o[7]);
}

// rows of x1 per workgroup: all of them, or, against a narrow x2 (at most 128 workgroups of 128 columns), equal slabs of up
// to 64 rows that go out in one launch
int64_t rows_per_slab(const OpsnnQmmArgs& a)
{
    const int64_t slab = wq_narrow_slab_rows(a.M, a.N, true);
    return slab ? slab : a.M;
}
// K segments for a long K against few workgroups (wq_rows_ksplit; the unit is one scale block)
int rows_ksplit(const OpsnnQmmArgs& a, int64_t* kunit = nullptr)
{
    if (a.force_variant != 0 || rows_per_slab(a) > 64) return 1;
    return wq_rows_ksplit(8, a.M, a.N, a.K, a.K, true, kunit);
}

bool rows_eligible(const OpsnnQmmArgs& a)
{
    if (a.x1_dtype != DT_E4M3 || a.x2_dtype != DT_E4M3 || a.batch != 1 || a.bias) return false;
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16 && a.out_dtype != DT_F32) return false;
    if (a.M <= 16 || a.M > 128) return false;
    if (a.gsK != 128 || a.gsN != 128 || (a.gsM != 1 && a.gsM != 128)) return false;
    // the kernel's shape conditions: whole workgroups of 128 columns inside one scale block, K in slabs of 128, 16-byte
    // pieces, the products of the block scales of one workgroup's K (all of K, or its longest segment) in 64 KB of LDS
    if (a.N % 128 != 0 || a.N < 256 || a.K % 128 != 0) return false;
    {
        const int ks = rows_ksplit(a);
        const int64_t blocks = (a.K / 128 + ks - 1) / ks;
        if (blocks * 16 * (rows_per_slab(a) > 64 ? 8 : 4) * 4 > 65536) return false;
    }
    if (a.x1.col_stride != 1 || a.x2.row_stride != 1 || a.x1.row_stride < a.K || a.x2.col_stride < a.K) return false;
    if (((uintptr_t)a.x1.ptr | (uintptr_t)a.x2.ptr | (uint64_t)a.x1.row_stride | (uint64_t)a.x2.col_stride) % 16) return false;
    if (((uintptr_t)a.x1_scale_mat.ptr | (uintptr_t)a.x2_scale_mat.ptr) % 4 || (uintptr_t)a.out % 16) return false;
    if (a.K >= (1ll << 31) || a.N >= (1ll << 31)) return false;
    return true;
}

}  // namespace

uint64_t blockscale_rows_workspace(const OpsnnQmmArgs& a) { return rows_eligible(a) ? (uint64_t)a.M * (uint64_t)a.K * 2 : 0; }
// the K segments that kernel would run in (1: K in one piece, or another kernel's call): fp32 partial sums [segments][M][N]
int blockscale_rows_ksplit(const OpsnnQmmArgs& a) { return rows_eligible(a) ? rows_ksplit(a) : 1; }

int launch_blockscale_rows(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk)
{
    if (!rows_eligible(a) || !a.workspace || (uintptr_t)a.workspace % 16) return OPSNN_NOT_TAKEN;
    int64_t kunit = 0;
    const int ks = rows_ksplit(a, &kunit);
    if (ks > 1 && (!sk.part || sk.splits < ks)) return OPSNN_NOT_TAKEN;   // (eligibility counted on the segments' scale tables)
    uint16_t* x16 = (uint16_t*)a.workspace;
    const int64_t pieces = a.M * (a.K / 16);
    hipLaunchKernelGGL(widen_e4m3_f16_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, st, (const uint8_t*)a.x1.ptr, a.x1.row_stride, x16,
                       a.M, a.K);
    WqParams p{};
    p.x = x16; p.w = (const uint8_t*)a.x2.ptr; p.ldw = a.x2.col_stride;
    p.y = (uint16_t*)a.out; p.M = a.M; p.N = a.N; p.K = a.K;
    p.group = a.K; p.group_shift = -1; p.cpg_shift = 31;
    p.m_base = 0; p.m_rows = a.M;
    p.w_float = 1;
    p.bs1 = (const float*)a.x1_scale_mat.ptr; p.bs1_rs = a.x1_scale_mat.row_stride; p.bs1_cs = a.x1_scale_mat.col_stride;
    p.bs2 = (const float*)a.x2_scale_mat.ptr; p.bs2_rs = a.x2_scale_mat.row_stride; p.bs2_cs = a.x2_scale_mat.col_stride;
    p.bs_gsm = (int)a.gsM; p.bs_out_dt = a.out_dtype;
    if (ks > 1) { p.ksplit = ks; p.kunit = kunit; p.part = sk.part; }
    if (const int64_t slab = wq_narrow_slab_rows(a.M, a.N, true)) {   // narrow x2 (at most 128 workgroups): two slabs in one launch, twice the workgroups
        p.m_rows = slab; p.m_slab = slab; p.m_end = a.M;
        return launch_rows_one<DT_F16, 8, 4, 2, 4, 2, false, 3>(p, st);
    }
    return a.M > 64 ? launch_rows_one<DT_F16, 8, 8, 2, 4, 2, false, 3>(p, st) : launch_rows_one<DT_F16, 8, 4, 2, 4, 2, false, 3>(p, st);
}

// The row / column scale form, (sum * x2Scale[n]) * x1Scale[m] + bias[n] with fp32 scales (K-C, K-T), 17 .. 128 rows.
static bool rowcol_rows_eligible(const OpsnnQmmArgs& a)
{
    if (a.x1_dtype != DT_E4M3 || a.x2_dtype != DT_E4M3 || a.batch != 1) return false;
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16 && a.out_dtype != DT_F32) return false;
    if (!a.x1_scale || !a.x2_scale || a.x2_scale_dtype != DT_F32 || (a.bias && a.bias_dtype != DT_F32)) return false;
    if (a.x1_scale_len == 1 && a.x2_scale_len == 1 && !a.bias) return false;   // that case merges and truncates the scales
    if (a.M <= 16 || a.M > 128 || a.N % 32 != 0 || a.N < 256 || a.K % 128 != 0) return false;
    if (a.x1.col_stride != 1 || a.x2.row_stride != 1 || a.x1.row_stride < a.K || a.x2.col_stride < a.K) return false;
    if (((uintptr_t)a.x1.ptr | (uintptr_t)a.x2.ptr | (uint64_t)a.x1.row_stride | (uint64_t)a.x2.col_stride) % 16 || (uintptr_t)a.out % 16) return false;
    if (a.K >= (1ll << 31) || a.N >= (1ll << 31)) return false;
    return true;
}

uint64_t rowcol_rows_workspace(const OpsnnQmmArgs& a) { return rowcol_rows_eligible(a) ? (uint64_t)a.M * (uint64_t)a.K * 2 : 0; }
int rowcol_rows_ksplit(const OpsnnQmmArgs& a) { return rowcol_rows_eligible(a) ? rows_ksplit(a) : 1; }

int launch_rowcol_rows(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk)
{
    if (!rowcol_rows_eligible(a) || !a.workspace || (uintptr_t)a.workspace % 16) return OPSNN_NOT_TAKEN;
    int64_t kunit = 0;
    int ks = rows_ksplit(a, &kunit);
    if (ks > 1 && (!sk.part || sk.splits < ks)) ks = 1;   // (no room for partial sums: K in one piece)
    uint16_t* x16 = (uint16_t*)a.workspace;
    const int64_t pieces = a.M * (a.K / 16);
    hipLaunchKernelGGL(widen_e4m3_f16_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, st, (const uint8_t*)a.x1.ptr, a.x1.row_stride, x16,
                       a.M, a.K);
    WqParams p{};
    p.x = x16; p.w = (const uint8_t*)a.x2.ptr; p.ldw = a.x2.col_stride;
    p.y = (uint16_t*)a.out; p.M = a.M; p.N = a.N; p.K = a.K;
    p.group = a.K; p.group_shift = -1; p.cpg_shift = 31;
    p.m_base = 0; p.m_rows = a.M;
    p.w_float = 1;
    p.bias = a.bias; p.bias_dt = a.bias_dtype;
    p.bs1 = (const float*)a.x1_scale; p.bs1_rs = a.x1_scale_len == 1 ? 0 : 1;
    p.bs2 = (const float*)a.x2_scale; p.bs2_cs = a.x2_scale_len == 1 ? 0 : 1;
    p.bs_out_dt = a.out_dtype;
    if (ks > 1) { p.ksplit = ks; p.kunit = kunit; p.part = sk.part; }
    if (const int64_t slab = wq_narrow_slab_rows(a.M, a.N, true)) {   // narrow x2 (at most 128 workgroups): two slabs in one launch, twice the workgroups
        p.m_rows = slab; p.m_slab = slab; p.m_end = a.M;
        return launch_rows_one<DT_F16, 8, 4, 2, 4, 2, false, 4>(p, st);
    }
    return a.M > 64 ? launch_rows_one<DT_F16, 8, 8, 2, 4, 2, false, 4>(p, st) : launch_rows_one<DT_F16, 8, 4, 2, 4, 2, false, 4>(p, st);
}

// ---- MXFP8 (e8m0 scales per 32 elements of K on both operands) with 17 .. 256 rows of x1 ----
// The many-rows kernel in its weight-only form for e4m3 codes with e8m0 group scales and bf16 activations: a pre-step widens
// x1 to bf16 with its block scales folded in (an e4m3 value times a power of two is a bf16 value wherever fp32 would hold
// it: M * K * 2 bytes of workspace), the kernel widens x2's codes the same way (T(w * s) is exact) and
// v_mfma_f32_16x16x32_bf16 sums exact products in fp32 -- the arithmetic of mx8_decode_kernel (qmm_fp8_decode.hip).
int launch_wq_mx8_rows(const WqParams& p, hipStream_t st);   // wqmm.hip

namespace {
// 16 e4m3 bytes of one 32-element block (half of it) -> 16 bf16, times 2^(scale byte - 127)
__global__ __launch_bounds__(256) void widen_mx8_bf16_kernel(const uint8_t* __restrict__ src, int64_t ld, const uint8_t* __restrict__ sc, int64_t sc_rs,
                                                             uint16_t* __restrict__ dst, int64_t rows, int64_t K)
{
    const int64_t pieces = K / 16;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * pieces) return;
    const int64_t r = i / pieces, c = i - r * pieces;
    const uint4 v = *(const uint4*)(src + r * ld + c * 16);
    const float s = e8m0_to_f32(sc[r * sc_rs + c / 2]);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[8];
#pragma unroll
    for (int d = 0; d < 4; d++) {
        typedef __bf16 b2v __attribute__((ext_vector_type(2)));
        o[2 * d] = __builtin_bit_cast(uint32_t, (b2v)__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[d], s, false));
        o[2 * d + 1] = __builtin_bit_cast(uint32_t, (b2v)__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[d], s, true));
    }
    uint4* out = (uint4*)(dst + r * K + c * 16);
    out[0] = make_uint4(o[0], o[1], o[2], o[3]);
    out[1] = make_uint4(o[4], o[5], o[6], o[7]);
}

bool mx8_rows_eligible(const OpsnnQmmArgs& a)
{
    if (a.x1_dtype != DT_E4M3 || a.x2_dtype != DT_E4M3 || a.batch != 1 || a.out_dtype != DT_BF16) return false;
    if (a.force_variant != 0 || (a.bias && a.bias_dtype != DT_F32)) return false;
    if (a.M <= 16 || a.M > 256 || a.N % 32 != 0 || a.N < 256 || a.K % 128 != 0 || a.K >= (1ll << 23)) return false;
    if (a.x1.col_stride != 1 || a.x2.row_stride != 1 || a.x1.row_stride < a.K || a.x2.col_stride < a.K) return false;
    if (((uintptr_t)a.x1.ptr | (uintptr_t)a.x2.ptr | (uint64_t)a.x1.row_stride | (uint64_t)a.x2.col_stride) % 16 || (uintptr_t)a.out % 16) return false;
    if (a.x1_scale_mat.col_stride != 2 || a.x2_scale_mat.col_stride != 2) return false;   // [rows, K / 64, 2]: a row's bytes contiguous
    if (a.x1_scale_mat.row_stride < a.K / 32 || a.x2_scale_mat.row_stride < a.K / 32) return false;
    if (((uintptr_t)a.x2_scale_mat.ptr | (uint64_t)a.x2_scale_mat.row_stride) % 4) return false;
    // the 192- / 256-row instances want K in whole rounds of four x slabs of 128
    const int64_t slab = wq_narrow_slab_rows(a.M, a.N, true);
    if ((slab ? slab : a.M) > 128 && a.K % 512 != 0) return false;
    return true;
}
}  // namespace

uint64_t mxfp8_rows_workspace(const OpsnnQmmArgs& a) { return mx8_rows_eligible(a) ? (uint64_t)a.M * (uint64_t)a.K * 2 : 0; }
int mxfp8_rows_ksplit(const OpsnnQmmArgs& a) { return mx8_rows_eligible(a) ? wq_rows_ksplit(8, a.M, a.N, a.K, 32, true) : 1; }

// `region`: mxfp8_rows_workspace(a) bytes for the bf16 copy of x1.
int launch_mxfp8_rows(const OpsnnQmmArgs& a, void* region, hipStream_t st, SplitK sk)
{
    if (!mx8_rows_eligible(a) || !region || (uintptr_t)region % 16) return OPSNN_NOT_TAKEN;
    const int ks = wq_rows_ksplit(8, a.M, a.N, a.K, 32, true);
    uint16_t* x16 = (uint16_t*)region;
    const int64_t pieces = a.M * (a.K / 16);
    hipLaunchKernelGGL(widen_mx8_bf16_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, st, (const uint8_t*)a.x1.ptr, a.x1.row_stride,
                       (const uint8_t*)a.x1_scale_mat.ptr, a.x1_scale_mat.row_stride, x16, a.M, a.K);
    WqParams p{};
    p.x = x16; p.w = (const uint8_t*)a.x2.ptr; p.ldw = a.x2.col_stride;
    p.scale = (const uint16_t*)a.x2_scale_mat.ptr; p.s_cs = a.x2_scale_mat.row_stride;
    p.bias = a.bias; p.bias_dt = a.bias_dtype;
    p.y = (uint16_t*)a.out; p.M = a.M; p.N = a.N; p.K = a.K;
    p.part = (ks > 1 && sk.part && sk.splits >= ks) ? sk.part : nullptr;
    return launch_wq_mx8_rows(p, st);
}

}  // namespace opsnn
