// Dynamic block quantisation to fp8: the quantizer that produces the operands and the per-block scales of the block-scale
// matmul (aclnnDynamicBlockQuant; formula quant/dynamic_block_quant/tests/assets/golden.py:95-222).
//
// x [batch, rows, cols] (fp16 / bf16) is cut into blocks of rb x cb.  Per block, every step a separately rounded fp32
// operation:  amax = max|x| (infinities and NaN count as 0);  scale = amax / tmax, capped at 1 / min_scale;
// q = x / scale (x itself where x is infinite or NaN), clipped to +-tmax;  q = rint(q * 1e8) / 1e8;  NaN -> +0;  y = fp8(q).
// HBM-bound: 2 bytes read, 1 written per element.
//   rb == 1, cols % 8 == 0: a block is cb / 8 lanes of one wave (8 elements per lane, held in registers between the
//     reduction and the quantisation), a lane group of 8 / 16 / 32 lanes per block, reduced by lane exchange only.
//   any other shape: one workgroup per block, two sweeps over the block (the second one hits in cache: a block is at
//     most 512 x 256 x 2 bytes).
// The two divisions per element (by the block's scale, by 1e8) are done with the correctly rounded reciprocal and one
// exact residual step, which gives the correctly rounded quotient except for a divisor whose mantissa is all ones or
// operands near the ends of the exponent range; blocks where that could be keep the division instruction.
#include "common.hip.h"
#include "launch.h"

namespace opsnn {

struct BlockQuantParams {
    const uint16_t* x; uint8_t* y; float* scale;
    int64_t batch, rows, cols, rb, cb, nrb, ncb;
    float tmax, cap;   // cap = fp32(1 / min_scale), or +inf when min_scale == 0
};

template <int X_DT>
__device__ __forceinline__ float bq_x_to_f32(uint32_t h)
{
    if constexpr (X_DT == DT_BF16) return u2f(h << 16);
    else return f16_to_f32((uint16_t)h);
}

struct BlockScale { float scale, rcp; bool fast; };

__device__ __forceinline__ BlockScale block_scale(const BlockQuantParams& p, float amax)
{
    BlockScale b;
    b.scale = fminf(__fdiv_rn(amax, p.tmax), p.cap);
    b.rcp = __fdiv_rn(1.0f, b.scale);
    // the quotients stay far from overflow (a capped scale under a huge bf16 maximum would not)
    b.fast = (f2u(b.scale) & 0x7fffffu) != 0x7fffffu && b.scale > 0x1p-60f && b.scale < 0x1p60f && __fmul_rn(amax, b.rcp) < 0x1p100f;
    return b;
}

// the value that is cast: finite, within +-tmax, never NaN
__device__ __forceinline__ float block_quant_value(float v, const BlockScale& b, float tmax)
{
    const bool finite = fabsf(v) < __builtin_inff();   // false for NaN too
    float q;
    {
        const float q0 = __fmul_rn(v, b.rcp);
        q = __fmaf_rn(__fmaf_rn(-q0, b.scale, v), b.rcp, q0);
    }
    // with the scale in [2^-60, 2^60] and |v| above 2^-100 every intermediate is a normal number; a zero stays a zero
    if (!(b.fast && (fabsf(v) > 0x1p-100f || v == 0.0f))) q = __fdiv_rn(v, b.scale);
    if (!finite) q = v;
    // NaN (a NaN input, or 0 / 0 in a block of zeros) passes numpy's clip and rounding and becomes +0 at the end: done first
    // here, which leaves the clip a single median instruction
    q = (q == q) ? q : 0.0f;
    q = __builtin_amdgcn_fmed3f(q, -tmax, tmax);
    const float t = __builtin_rintf(__fmul_rn(q, 1e8f));
    const float d0 = __fmul_rn(t, 1e-8f);   // 1e-8f is the correctly rounded reciprocal of 1e8f
    return __fmaf_rn(__fmaf_rn(-d0, 1e8f, t), 1e-8f, d0);
}
template <int Y_DT>
__device__ __forceinline__ uint32_t block_quant_one(float v, const BlockScale& b, float tmax)
{
    return cvt2_fp8_in_range<Y_DT>(block_quant_value(v, b, tmax), 0.0f) & 0xffu;
}
// eight elements -> eight bytes
template <int Y_DT>
__device__ __forceinline__ uint2 block_quant_eight(const float* v, const BlockScale& b, float tmax)
{
    uint32_t h[4];
#pragma unroll
    for (int e = 0; e < 4; e++) h[e] = cvt2_fp8_in_range<Y_DT>(block_quant_value(v[2 * e], b, tmax), block_quant_value(v[2 * e + 1], b, tmax));
    return make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
}

// rb == 1: lane groups of G lanes, LPB = cb / 8 of them active.  A group takes NB (row, block) pairs, the pairs
// g, g + ngroups, g + 2 ngroups, ... so that neighbouring groups read neighbouring blocks; all NB loads are issued
// before the first is used.
template <int X_DT, int Y_DT, int G, int NB>
__global__ __launch_bounds__(256) void block_quant_rows_kernel(BlockQuantParams p, int lpb, int64_t ngroups)
{
    const int64_t group = ((int64_t)blockIdx.x * 256 + threadIdx.x) / G;
    const int lane = threadIdx.x % G;
    const int64_t total = p.batch * p.rows * p.ncb;
    // rows that are a whole number of blocks: pair number x block length is the element offset, and the 64-bit divisions by
    // the row's block count (more instructions than the quantisation of a piece) drop out
    const bool flat = p.cols == p.ncb * p.cb;
    uint4 buf[NB];
    int64_t at[NB];      // element offset of the lane's piece, -1 when there is none
    bool live_pair[NB];
#pragma unroll
    for (int i = 0; i < NB; i++) {
        const int64_t pair = (int64_t)i * ngroups + group;
        live_pair[i] = group < ngroups && pair < total;
        if (flat) {
            at[i] = (live_pair[i] && lane < lpb) ? pair * p.cb + (int64_t)lane * 8 : -1;
        } else {
            const int64_t row = live_pair[i] ? pair / p.ncb : 0, bc = live_pair[i] ? pair % p.ncb : 0;
            const int64_t col = bc * p.cb + (int64_t)lane * 8;
            // cols % 8 == 0: a piece is inside the row or outside
            at[i] = (live_pair[i] && lane < lpb && col < p.cols) ? row * p.cols + col : -1;
        }
        buf[i] = make_uint4(0, 0, 0, 0);
        if (at[i] >= 0) buf[i] = *(const uint4*)(p.x + at[i]);
    }
#pragma unroll
    for (int i = 0; i < NB; i++) {
        const uint32_t w[4] = {buf[i].x, buf[i].y, buf[i].z, buf[i].w};
        float v[8];
        float amax = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            v[e] = bq_x_to_f32<X_DT>((w[e >> 1] >> (16 * (e & 1))) & 0xffffu);
            const float a = fabsf(v[e]);
            amax = fmaxf(amax, a < __builtin_inff() ? a : 0.0f);
        }
#pragma unroll
        for (int o = G / 2; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
        const BlockScale b = block_scale(p, amax);
        if (live_pair[i] && lane == 0) p.scale[(int64_t)i * ngroups + group] = b.scale;
        if (at[i] >= 0) *(uint2*)(p.y + at[i]) = block_quant_eight<Y_DT>(v, b, p.tmax);
    }
}

// Any block shape: one workgroup per block, two sweeps.  VEC: cols % 8 == 0 (then every block row is a whole number of
// 16-byte pieces, since cb % 8 == 0); otherwise element by element.
template <int X_DT, int Y_DT, bool VEC>
__global__ __launch_bounds__(256) void block_quant_tile_kernel(BlockQuantParams p)
{
    __shared__ float red[4];
    const int64_t blk = blockIdx.x;
    const int64_t bc = blk % p.ncb, br = (blk / p.ncb) % p.nrb, bt = blk / (p.ncb * p.nrb);
    const int64_t r0 = br * p.rb, c0 = bc * p.cb;
    const int64_t nr = (r0 + p.rb < p.rows ? p.rb : p.rows - r0), nc = (c0 + p.cb < p.cols ? p.cb : p.cols - c0);
    const uint16_t* xb = p.x + (bt * p.rows + r0) * p.cols + c0;
    uint8_t* yb = p.y + (bt * p.rows + r0) * p.cols + c0;
    constexpr int W = VEC ? 8 : 1;
    // pieces per block row (at most 256) and rows: a thread's piece index advances by 256 = da rows + db pieces per
    // step, kept as (row, piece) so that the loops carry no division
    const int ppr = (int)(nc / W), rows_here = (int)nr;
    const int da = 256 / ppr, db = 256 % ppr;
    const int r_first = (int)threadIdx.x / ppr, c_first = (int)threadIdx.x % ppr;
    float amax = 0.0f;
    if constexpr (VEC) {
        // A block of at most 8 pieces per thread whose rows tile the 256 threads evenly (128 x 128 is 8 steps of 16 rows)
        // stays in registers between the two sweeps: all its loads are issued at once and nothing is read twice.
        constexpr int HELD = 8;
        if (db == 0 && rows_here <= HELD * da) {   // uniform over the workgroup
            uint4 held[HELD];
#pragma unroll
            for (int k = 0; k < HELD; k++) {
                const int r = r_first + k * da;
                held[k] = r < rows_here ? *(const uint4*)(xb + (int64_t)r * p.cols + c_first * 8) : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int k = 0; k < HELD; k++) {
                const uint32_t w[4] = {held[k].x, held[k].y, held[k].z, held[k].w};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const float a = fabsf(bq_x_to_f32<X_DT>((w[e >> 1] >> (16 * (e & 1))) & 0xffffu));
                    amax = fmaxf(amax, a < __builtin_inff() ? a : 0.0f);
                }
            }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
            if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
            __syncthreads();
            amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
            const BlockScale b = block_scale(p, amax);
            if (threadIdx.x == 0) p.scale[blk] = b.scale;
#pragma unroll
            for (int k = 0; k < HELD; k++) {
                const int r = r_first + k * da;
                const uint32_t w[4] = {held[k].x, held[k].y, held[k].z, held[k].w};
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; e++) v[e] = bq_x_to_f32<X_DT>((w[e >> 1] >> (16 * (e & 1))) & 0xffffu);
                const uint2 q = block_quant_eight<Y_DT>(v, b, p.tmax);
                if (r < rows_here) *(uint2*)(yb + (int64_t)r * p.cols + c_first * 8) = q;
            }
            return;
        }
    }
    for (int r = r_first, c = c_first; r < rows_here;) {
        const int64_t o = (int64_t)r * p.cols + c * W;
        if constexpr (VEC) {
            const uint4 b = *(const uint4*)(xb + o);
            const uint32_t w[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float a = fabsf(bq_x_to_f32<X_DT>((w[e >> 1] >> (16 * (e & 1))) & 0xffffu));
                amax = fmaxf(amax, a < __builtin_inff() ? a : 0.0f);
            }
        } else {
            const float a = fabsf(bq_x_to_f32<X_DT>(xb[o]));
            amax = fmaxf(amax, a < __builtin_inff() ? a : 0.0f);
        }
        r += da; c += db;
        if (c >= ppr) { c -= ppr; r++; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const BlockScale b = block_scale(p, amax);
    if (threadIdx.x == 0) p.scale[blk] = b.scale;
    for (int r = r_first, c = c_first; r < rows_here;) {
        const int64_t o = (int64_t)r * p.cols + c * W;
        if constexpr (VEC) {
            const uint4 xv = *(const uint4*)(xb + o);
            const uint32_t w[4] = {xv.x, xv.y, xv.z, xv.w};
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; e++) v[e] = bq_x_to_f32<X_DT>((w[e >> 1] >> (16 * (e & 1))) & 0xffffu);
            *(uint2*)(yb + o) = block_quant_eight<Y_DT>(v, b, p.tmax);
        } else {
            yb[o] = (uint8_t)block_quant_one<Y_DT>(bq_x_to_f32<X_DT>(xb[o]), b, p.tmax);
        }
        r += da; c += db;
        if (c >= ppr) { c -= ppr; r++; }
    }
}

template <int X_DT, int Y_DT>
static int launch_block_quant(const BlockQuantParams& p, int variant, hipStream_t st)
{
    const bool rows_ok = p.rb == 1 && p.cols % 8 == 0 && p.cb % 8 == 0 && p.cb <= 256 && (uintptr_t)p.x % 16 == 0 && (uintptr_t)p.y % 8 == 0;
    if (variant != 2 && rows_ok) {
        const int lpb = (int)(p.cb / 8);
        const int g = lpb <= 8 ? 8 : lpb <= 16 ? 16 : 32;
        const int64_t pairs = p.batch * p.rows * p.ncb;
        // four pairs per group once that still leaves every SIMD eight waves
        const int nb = pairs * g / 64 >= (int64_t)4 * 8 * 1024 ? 4 : 1;
        const int64_t groups = (pairs + nb - 1) / nb;
        const int64_t wgs = (groups * g + 255) / 256;
        if (wgs > 0x7fffffff) return -1;
        auto go = [&](auto kernel) { hipLaunchKernelGGL(kernel, dim3((unsigned)wgs), dim3(256), 0, st, p, lpb, groups); };
        if (nb == 4) {
            if (g == 8) go(block_quant_rows_kernel<X_DT, Y_DT, 8, 4>);
            else if (g == 16) go(block_quant_rows_kernel<X_DT, Y_DT, 16, 4>);
            else go(block_quant_rows_kernel<X_DT, Y_DT, 32, 4>);
        } else {
            if (g == 8) go(block_quant_rows_kernel<X_DT, Y_DT, 8, 1>);
            else if (g == 16) go(block_quant_rows_kernel<X_DT, Y_DT, 16, 1>);
            else go(block_quant_rows_kernel<X_DT, Y_DT, 32, 1>);
        }
    } else {
        if (variant == 1) return -4;
        const int64_t blocks = p.batch * p.nrb * p.ncb;
        if (blocks > 0x7fffffff) return -1;
        const bool vec = p.cols % 8 == 0 && p.cb % 8 == 0 && (uintptr_t)p.x % 16 == 0 && (uintptr_t)p.y % 8 == 0;
        if (vec) hipLaunchKernelGGL((block_quant_tile_kernel<X_DT, Y_DT, true>), dim3((unsigned)blocks), dim3(256), 0, st, p);
        else hipLaunchKernelGGL((block_quant_tile_kernel<X_DT, Y_DT, false>), dim3((unsigned)blocks), dim3(256), 0, st, p);
    }
    return (int)hipGetLastError();
}

}  // namespace opsnn

using namespace opsnn;

extern "C" int opsnnDynamicBlockQuant(const OpsnnBlockQuantArgs* a, void* stream)
{
    if (!a || !a->x || !a->y || !a->scale || a->batch <= 0 || a->rows <= 0 || a->cols <= 0 || a->row_block <= 0 || a->col_block <= 0) return -1;
    if ((a->x_dtype != DT_F16 && a->x_dtype != DT_BF16) || (a->y_dtype != DT_E4M3 && a->y_dtype != DT_E5M2) || !(a->min_scale >= 0)) return -2;
    BlockQuantParams p{};
    p.x = (const uint16_t*)a->x; p.y = (uint8_t*)a->y; p.scale = a->scale;
    p.batch = a->batch; p.rows = a->rows; p.cols = a->cols; p.rb = a->row_block; p.cb = a->col_block;
    p.nrb = (p.rows + p.rb - 1) / p.rb; p.ncb = (p.cols + p.cb - 1) / p.cb;
    p.tmax = a->y_dtype == DT_E4M3 ? 448.0f : 57344.0f;
    p.cap = a->min_scale != 0 ? (float)(1.0 / a->min_scale) : __builtin_inff();
    const hipStream_t st = (hipStream_t)stream;
    if (a->x_dtype == DT_BF16)
        return a->y_dtype == DT_E4M3 ? launch_block_quant<DT_BF16, DT_E4M3>(p, a->force_variant, st) : launch_block_quant<DT_BF16, DT_E5M2>(p, a->force_variant, st);
    return a->y_dtype == DT_E4M3 ? launch_block_quant<DT_F16, DT_E4M3>(p, a->force_variant, st) : launch_block_quant<DT_F16, DT_E5M2>(p, a->force_variant, st);
}
