// Dynamic MX quantisation along the last axis: 16-bit activations / weights -> fp4 e2m1 or fp8 elements with one e8m0
// scale per 32 elements, the operand format of the MX matmuls (aclnnDynamicMxQuant; formula
// quant/dynamic_mx_quant/tests/assets/golden.py:140-153, 196-218, 263-330 with round mode "rint", scale algorithm 0).
//
// Per block of 32:  share_exp = floor(log2 max|x|) - emax, at least -127;  q = x * 2^-share_exp (exact);  y = q rounded to
// nearest even on the element grid, saturated at the format's maximum;  scale byte = share_exp + 127.  A block that holds
// an infinity or a NaN gets scale 0xFF and zeros.  Scale rows are padded to an even number of bytes with 0.
// HBM-bound: 2 bytes read and 1 (fp8) or 1/2 (fp4) written per element.  A block is four lanes of a wave with 8 elements
// each (one 16-byte load per lane), reduced by two lane exchanges; rows whose length is not a multiple of 8 take the
// one-thread-per-block kernel.
#include "common.hip.h"
#include "launch.h"

namespace opsnn {

struct MxQuantParams {
    const uint16_t* x; uint8_t* y; uint8_t* scale;
    int64_t rows, cols, nblk, spitch;
    int block;       // elements per scale block (32 on the lane-group kernel)
    int scale_alg;   // 0: floor(log2 max) - emax;  1 (fp8 elements): exponent of max / tmax, rounded up when it has mantissa bits
};

template <int X_DT>
__device__ __forceinline__ float mx_x_to_f32(uint32_t h)
{
    if constexpr (X_DT == DT_BF16) return u2f(h << 16);
    else return f16_to_f32((uint16_t)h);
}

template <int Y_DT> struct MxFormat;
template <> struct MxFormat<DT_E2M1> { static constexpr int emax = 2; static constexpr float tmax = 6.0f; };
template <> struct MxFormat<DT_E4M3> { static constexpr int emax = 8; static constexpr float tmax = 448.0f; };
template <> struct MxFormat<DT_E5M2> { static constexpr int emax = 15; static constexpr float tmax = 57344.0f; };

// Shared exponent of a block from the bits of its largest magnitude (a finite, non-negative fp32).  floor(log2) of a
// normal fp32 is its exponent field; a zero or subnormal maximum lands below the floor of -127 in any case.
template <int Y_DT>
__device__ __forceinline__ int mx_share_exp(float amax, int alg = 0)
{
    if (alg == 1) {   // golden.py:156-176: the scale is max / tmax rounded up to a power of two
        if (amax == 0.0f) return -127;
        const uint32_t u = f2u(__fdiv_rn(amax, MxFormat<Y_DT>::tmax));
        int e = (int)(u >> 23);
        const uint32_t mant = u & 0x7fffffu;
        if ((e > 0 && e < 254 && mant > 0) || (e == 0 && mant > 0x400000u)) e += 1;
        return e - 127;
    }
    const int e = (int)(f2u(amax) >> 23);
    const int s = e - 127 - MxFormat<Y_DT>::emax;
    return (e == 0 || s < -127) ? -127 : s;
}

// |q| < 8 rounded to nearest even on {0, .5, 1, 1.5, 2, 3, 4, 6} by the binade of q and saturated at 6 -> code with sign
// bit.  The step is 2^(max(e, 0) - 1) for a in [2^e, 2^(e+1)); adding and subtracting 1.5 * 2^23 times the step rounds a to
// a multiple of the step, ties to even.  For r >= 1 the code is r's exponent and first mantissa bit, (bits >> 22) - 252.
__device__ __forceinline__ uint32_t mx_e2m1_code(float q)
{
    const uint32_t sign = (f2u(q) >> 28) & 8u;
    const float a = fminf(fabsf(q), 6.0f);
    const uint32_t e = f2u(a) >> 23;
    const float c = u2f((((e > 127u ? e : 127u) + 22u) << 23) | 0x400000u);
    const float r = __fsub_rn(__fadd_rn(a, c), c);
    const uint32_t code = r < 1.0f ? (uint32_t)__fmul_rn(r, 2.0f) : (f2u(r) >> 22) - 252u;
    return sign | code;
}

template <int Y_DT>
__device__ __forceinline__ float mx_scaled(float v, float inv_scale, bool bad)
{
    const float q = __fmul_rn(v, inv_scale);   // a power of two: exact
    return bad ? 0.0f : q;
}

// eight scaled elements -> their bytes (fp8: 8 bytes in lo/hi; fp4: 4 bytes in lo)
template <int Y_DT>
__device__ __forceinline__ uint2 mx_pack8(const float* q)
{
    if constexpr (Y_DT == DT_E2M1) {
        // The hardware conversion (two values -> one byte, low nibble first) returns mx_e2m1_code's nibble for every fp32 of
        // either sign up to 8 (compared exhaustively on the device, with a unit scale operand); |q| < 8 by construction.
        uint32_t r = 0;
        r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, q[0], q[1], 1.0f, 0);
        r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, q[2], q[3], 1.0f, 1);
        r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, q[4], q[5], 1.0f, 2);
        r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, q[6], q[7], 1.0f, 3);
        return make_uint2(r, 0);
    } else {
        constexpr float t = MxFormat<Y_DT>::tmax;
        uint32_t h[4];
#pragma unroll
        for (int e = 0; e < 4; e++)
            h[e] = cvt2_fp8_in_range<Y_DT>(fminf(fmaxf(q[2 * e], -t), t), fminf(fmaxf(q[2 * e + 1], -t), t));
        return make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
    }
}

// cols % 8 == 0: lane groups of four.  A group takes NB (row, block) pairs, the pairs g, g + ngroups, g + 2 ngroups, ...
// so that neighbouring groups read neighbouring blocks; all NB loads are issued before the first is used.
// FLAT: every row is a whole, even number of blocks, so pair number, element offset / 32 and scale index coincide and the
// 64-bit divisions by the row's block count (more instructions than the quantisation itself) drop out.
template <int X_DT, int Y_DT, int NB, bool FLAT>
__global__ __launch_bounds__(256) void mx_quant_kernel(MxQuantParams p, int64_t ngroups)
{
    const int64_t group = ((int64_t)blockIdx.x * 256 + threadIdx.x) / 4;
    const int lane = threadIdx.x & 3;
    const int64_t total = p.rows * p.nblk;
    uint4 buf[NB];
    int64_t at[NB];        // element offset of the lane's piece, -1 when it lies in the zero padding of a short last block
    int64_t sidx[NB];      // index of the pair's scale byte, -1 for a pair that does not exist
    bool pad_after[NB];    // the pair is the last block of a row with an odd number of blocks
#pragma unroll
    for (int i = 0; i < NB; i++) {
        const int64_t pair = (int64_t)i * ngroups + group;
        const bool live_pair = group < ngroups && pair < total;
        if constexpr (FLAT) {
            at[i] = live_pair ? pair * 32 + lane * 8 : -1;
            sidx[i] = live_pair ? pair : -1;
            pad_after[i] = false;
        } else {
            const int64_t row = live_pair ? pair / p.nblk : 0, blk = live_pair ? pair % p.nblk : 0;
            const int64_t col = blk * 32 + lane * 8;
            at[i] = (live_pair && col < p.cols) ? row * p.cols + col : -1;
            sidx[i] = live_pair ? row * p.spitch + blk : -1;
            pad_after[i] = blk == p.nblk - 1 && (p.nblk & 1);
        }
        buf[i] = make_uint4(0, 0, 0, 0);
        if (at[i] >= 0) buf[i] = *(const uint4*)(p.x + at[i]);
    }
#pragma unroll
    for (int i = 0; i < NB; i++) {
        const uint32_t w[4] = {buf[i].x, buf[i].y, buf[i].z, buf[i].w};
        float v[8];
        float amax = 0.0f;
        bool bad = false;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            v[e] = mx_x_to_f32<X_DT>((w[e >> 1] >> (16 * (e & 1))) & 0xffffu);
            const float a = fabsf(v[e]);
            bad |= !(a < __builtin_inff());   // infinity or NaN
            amax = fmaxf(amax, a);
        }
        amax = fmaxf(amax, __shfl_xor(amax, 1));
        amax = fmaxf(amax, __shfl_xor(amax, 2));
        bad |= (bool)__shfl_xor((int)bad, 1);
        bad |= (bool)__shfl_xor((int)bad, 2);
        const int share = bad ? 0 : mx_share_exp<Y_DT>(amax, p.scale_alg);
        if (sidx[i] >= 0 && lane == 0) {
            p.scale[sidx[i]] = bad ? 0xFFu : (uint8_t)(share + 127);
            if (pad_after[i]) p.scale[sidx[i] + 1] = 0;
        }
        if (at[i] < 0) continue;
        // 2^-share: share is in [-127, 125]; 2^127 and 2^-125 are both normal numbers
        const float inv_scale = u2f((uint32_t)(127 - share) << 23);
        float q[8];
#pragma unroll
        for (int e = 0; e < 8; e++) q[e] = mx_scaled<Y_DT>(v[e], inv_scale, bad);
        const uint2 out = mx_pack8<Y_DT>(q);
        if constexpr (Y_DT == DT_E2M1) *(uint32_t*)(p.y + at[i] / 2) = out.x;
        else *(uint2*)(p.y + at[i]) = out;
    }
}

// Blocks of 64, 128, 256, 512 or 1024 elements, cols % 8 == 0: a wave takes 512 * PPL consecutive elements of a row (a whole
// number of blocks), every lane PPL 16-byte pieces (1024: two, 512 elements apart; otherwise one), and the block maximum is
// an exchange over the 2^lg neighbouring lanes that share a block.  One pass, every access of a wave contiguous.
template <int X_DT, int Y_DT, int PPL>
__global__ __launch_bounds__(256) void mx_quant_wideblock_kernel(MxQuantParams p, int lg, int chunks_per_row)
{
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t row = wave / chunks_per_row;
    if (row >= p.rows) return;
    const int64_t col_base = (wave - row * chunks_per_row) * (512 * PPL);
    float v[PPL][8];
    bool live[PPL];
    float amax = 0.0f;
    bool bad = false;
#pragma unroll
    for (int k = 0; k < PPL; k++) {
        const int64_t col = col_base + (k * 64 + lane) * 8;
        live[k] = col < p.cols;
        uint4 b = make_uint4(0, 0, 0, 0);
        if (live[k]) b = *(const uint4*)(p.x + row * p.cols + col);
        const uint32_t w[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
        for (int e = 0; e < 8; e++) {
            v[k][e] = mx_x_to_f32<X_DT>((w[e >> 1] >> (16 * (e & 1))) & 0xffffu);
            const float a = fabsf(v[k][e]);
            bad |= !(a < __builtin_inff());
            amax = fmaxf(amax, a);
        }
    }
    int badi = bad;
    for (int d = 1; d < (1 << lg); d <<= 1) {
        amax = fmaxf(amax, __shfl_xor(amax, d));
        badi |= __shfl_xor(badi, d);
    }
    bad = badi != 0;
    const int share = bad ? 0 : mx_share_exp<Y_DT>(amax, p.scale_alg);
    const int64_t col0 = col_base + lane * 8;
    if ((lane & ((1 << lg) - 1)) == 0 && live[0]) {
        const int64_t blk = col0 / p.block;
        p.scale[row * p.spitch + blk] = bad ? 0xFFu : (uint8_t)(share + 127);
        if (blk == p.nblk - 1 && (p.nblk & 1)) p.scale[row * p.spitch + blk + 1] = 0;
    }
    const float inv_scale = u2f((uint32_t)(127 - share) << 23);
#pragma unroll
    for (int k = 0; k < PPL; k++) {
        if (!live[k]) continue;
        float q[8];
#pragma unroll
        for (int e = 0; e < 8; e++) q[e] = mx_scaled<Y_DT>(v[k][e], inv_scale, bad);
        const uint2 out = mx_pack8<Y_DT>(q);
        const int64_t at = row * p.cols + col_base + (k * 64 + lane) * 8;
        if constexpr (Y_DT == DT_E2M1) *(uint32_t*)(p.y + at / 2) = out.x;
        else *(uint2*)(p.y + at) = out;
    }
}

// any row length and block size: one thread per block
template <int X_DT, int Y_DT>
__global__ __launch_bounds__(256) void mx_quant_generic_kernel(MxQuantParams p)
{
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= p.rows * p.nblk) return;
    const int64_t row = g / p.nblk, blk = g % p.nblk;
    const int64_t c0 = blk * p.block, c1 = c0 + p.block < p.cols ? c0 + p.block : p.cols;
    const uint16_t* xr = p.x + row * p.cols;
    float amax = 0.0f;
    bool bad = false;
    for (int64_t c = c0; c < c1; c++) {
        const float a = fabsf(mx_x_to_f32<X_DT>(xr[c]));
        bad |= !(a < __builtin_inff());
        amax = fmaxf(amax, a);
    }
    const int share = bad ? 0 : mx_share_exp<Y_DT>(amax, p.scale_alg);
    p.scale[row * p.spitch + blk] = bad ? 0xFFu : (uint8_t)(share + 127);
    if (blk == p.nblk - 1 && (p.nblk & 1)) p.scale[row * p.spitch + blk + 1] = 0;
    const float inv_scale = u2f((uint32_t)(127 - share) << 23);
    constexpr float t = MxFormat<Y_DT>::tmax;
    for (int64_t c = c0; c < c1; c += 2) {   // pairs: an fp4 byte holds two columns (cols is even for fp4)
        const float q0 = mx_scaled<Y_DT>(mx_x_to_f32<X_DT>(xr[c]), inv_scale, bad);
        const float q1 = c + 1 < c1 ? mx_scaled<Y_DT>(mx_x_to_f32<X_DT>(xr[c + 1]), inv_scale, bad) : 0.0f;
        if constexpr (Y_DT == DT_E2M1) {
            p.y[(row * p.cols + c) / 2] = (uint8_t)(mx_e2m1_code(q0) | (mx_e2m1_code(q1) << 4));
        } else {
            const uint32_t h = cvt2_fp8_in_range<Y_DT>(fminf(fmaxf(q0, -t), t), fminf(fmaxf(q1, -t), t));
            p.y[row * p.cols + c] = (uint8_t)h;
            if (c + 1 < c1) p.y[row * p.cols + c + 1] = (uint8_t)(h >> 8);
        }
    }
}

// ---- general form: blocks along any axis of [outer, A, inner], fp32 input, e1m2 elements, every rounding mode ----
// (golden.py:181-218, 263-330).  One thread per block and inner column -- two neighbouring columns for the 4-bit types,
// whose bytes hold two elements of the last axis -- so that neighbouring threads read neighbouring addresses when
// inner > 1; not tuned beyond that.  floor(log2) of the block maximum and of every scaled element is the exponent field of
// the fp32 (the element's clamped from below at the format's smallest normal exponent), all scalings are by powers of two
// and exact, and the mantissa is rounded as an integer by the mode.
struct MxGeneralParams {
    const void* x; uint8_t* y; uint8_t* scale;
    int64_t outer, A, inner, nblk, np;
    int block, scale_alg, round_mode, x_dt, y_dt;
};

__device__ __forceinline__ float mxg_load(const void* x, int dt, int64_t i)
{
    if (dt == DT_F32) return ((const float*)x)[i];
    const uint32_t h = ((const uint16_t*)x)[i];
    return dt == DT_BF16 ? u2f(h << 16) : f16_to_f32((uint16_t)h);
}

// one scaled element -> its code (8-bit formats: the byte; 4-bit: the nibble)
__device__ __forceinline__ uint32_t mxg_element(float v, float inv_scale, bool bad, int emin, int mbits, float tmax, int mode, int y_dt)
{
    float q = 0.0f;
    if (!bad) {
        q = __fmul_rn(v, inv_scale);
        int e = (int)((f2u(q) >> 23) & 0xffu) - 127;
        e = e < emin ? emin : e;
        // q / 2^e * 2^mbits and back: exact scalings (|q| < 2 tmax, e >= emin >= -14)
        const float up = u2f((uint32_t)(127 + mbits - e) << 23), down = u2f((uint32_t)(127 - mbits + e) << 23);
        float r = __fmul_rn(q, up);
        switch (mode) {
            case 0: r = __builtin_rintf(r); break;
            case 1: { const float t = __builtin_floorf(__fadd_rn(fabsf(r), 0.5f)); r = (f2u(r) >> 31) ? -t : t; break; }
            case 2: r = __builtin_floorf(r); break;
            case 3: r = __builtin_ceilf(r); break;
            default: r = __builtin_truncf(r); break;
        }
        q = __fmul_rn(r, down);
        q = fminf(fmaxf(q, -tmax), tmax);
    }
    if (y_dt == DT_E4M3) return f32_to_e4m3_bits(q) & 0xffu;
    if (y_dt == DT_E5M2) return f32_to_e5m2_bits(q) & 0xffu;
    if (y_dt == DT_E2M1) return mx_e2m1_code(q);                     // q is on the grid: the code of q itself
    return (uint32_t)__fmul_rn(fabsf(q), 4.0f) | ((f2u(q) >> 28) & 8u);   // e1m2: the magnitudes are k / 4
}

__global__ __launch_bounds__(256) void mx_quant_general_kernel(MxGeneralParams p)
{
    const bool fp4 = p.y_dt == DT_E2M1 || p.y_dt == DT_E1M2;
    const bool pair_inner = fp4 && p.inner > 1;            // a thread takes the inner columns 2 iw, 2 iw + 1
    const int64_t iw = pair_inner ? p.inner / 2 : p.inner;
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= p.outer * p.nblk * iw) return;
    const int64_t o = g / (p.nblk * iw), rem = g - o * (p.nblk * iw), b = rem / iw, ic = rem - b * iw;
    int emax, emin, mbits; float tmax;
    switch (p.y_dt) {
        case DT_E2M1: emax = 2; emin = 0; mbits = 1; tmax = 6.0f; break;
        case DT_E1M2: emax = 0; emin = 0; mbits = 2; tmax = 1.75f; break;
        case DT_E4M3: emax = 8; emin = -6; mbits = 3; tmax = 448.0f; break;
        default: emax = 15; emin = -14; mbits = 2; tmax = 57344.0f; break;
    }
    const int64_t a0 = b * p.block, a1 = a0 + p.block < p.A ? a0 + p.block : p.A;
    const int ncol = pair_inner ? 2 : 1;
    float inv_scale[2]; bool bad[2];
    for (int c = 0; c < ncol; c++) {
        const int64_t in = pair_inner ? 2 * ic + c : ic;
        float amax = 0.0f; bool bd = false;
        for (int64_t a = a0; a < a1; a++) {
            const float v = fabsf(mxg_load(p.x, p.x_dt, (o * p.A + a) * p.inner + in));
            bd |= !(v < __builtin_inff());
            amax = fmaxf(amax, v);
        }
        int share = -127;
        if (!bd && amax != 0.0f) {
            if (p.scale_alg == 1) {
                const uint32_t u = f2u(__fdiv_rn(amax, tmax));
                int e = (int)(u >> 23);
                const uint32_t mant = u & 0x7fffffu;
                if ((e > 0 && e < 254 && mant > 0) || (e == 0 && mant > 0x400000u)) e += 1;
                share = e - 127;
            } else {
                const int e = (int)(f2u(amax) >> 23);
                share = (e == 0 || e - 127 - emax < -127) ? -127 : e - 127 - emax;
            }
        }
        p.scale[((o * p.np + b / 2) * p.inner + in) * 2 + (b & 1)] = bd ? 0xFFu : (uint8_t)(share + 127);
        if (b == p.nblk - 1 && (p.nblk & 1)) p.scale[((o * p.np + b / 2) * p.inner + in) * 2 + 1] = 0;
        inv_scale[c] = u2f((uint32_t)(127 - share) << 23);
        bad[c] = bd;
    }
    if (pair_inner) {
        for (int64_t a = a0; a < a1; a++) {
            const int64_t i = (o * p.A + a) * p.inner + 2 * ic;
            const uint32_t lo = mxg_element(mxg_load(p.x, p.x_dt, i), inv_scale[0], bad[0], emin, mbits, tmax, p.round_mode, p.y_dt);
            const uint32_t hi = mxg_element(mxg_load(p.x, p.x_dt, i + 1), inv_scale[1], bad[1], emin, mbits, tmax, p.round_mode, p.y_dt);
            p.y[i >> 1] = (uint8_t)(lo | (hi << 4));
        }
    } else if (fp4) {   // inner == 1: the block's own elements pair up (A is even, blocks are multiples of 32)
        for (int64_t a = a0; a < a1; a += 2) {
            const int64_t i = o * p.A + a;
            const uint32_t lo = mxg_element(mxg_load(p.x, p.x_dt, i), inv_scale[0], bad[0], emin, mbits, tmax, p.round_mode, p.y_dt);
            const uint32_t hi = a + 1 < a1 ? mxg_element(mxg_load(p.x, p.x_dt, i + 1), inv_scale[0], bad[0], emin, mbits, tmax, p.round_mode, p.y_dt) : 0u;
            p.y[i >> 1] = (uint8_t)(lo | (hi << 4));
        }
    } else {
        for (int64_t a = a0; a < a1; a++) {
            const int64_t i = (o * p.A + a) * p.inner + ic;
            p.y[i] = (uint8_t)mxg_element(mxg_load(p.x, p.x_dt, i), inv_scale[0], bad[0], emin, mbits, tmax, p.round_mode, p.y_dt);
        }
    }
}

// The same arithmetic for blocks along an axis that is not the last, 16-bit x and inner % 8 == 0: a thread takes 8
// neighbouring inner columns (16-byte loads, 8- or 4-byte stores) and one PAIR of blocks, so that it also owns the 16
// contiguous scale bytes of its columns ([.., pair, inner, 2]).  x is read twice (the second time from cache).
// YT: the element type when the rounding is to nearest even (the hardware conversions of the last-axis kernels), or 0:
// any type and rounding mode through mxg_element.
template <int YT>
__global__ __launch_bounds__(256) void mx_quant_inner8_kernel(MxGeneralParams p)
{
    const int64_t iw = p.inner / 8;
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= p.outer * p.np * iw) return;
    const int64_t o = g / (p.np * iw), rem = g - o * (p.np * iw), pb = rem / iw, ic = rem - pb * iw;
    int emax, emin, mbits; float tmax;
    switch (p.y_dt) {
        case DT_E2M1: emax = 2; emin = 0; mbits = 1; tmax = 6.0f; break;
        case DT_E1M2: emax = 0; emin = 0; mbits = 2; tmax = 1.75f; break;
        case DT_E4M3: emax = 8; emin = -6; mbits = 3; tmax = 448.0f; break;
        default: emax = 15; emin = -14; mbits = 2; tmax = 57344.0f; break;
    }
    const bool fp4 = p.y_dt == DT_E2M1 || p.y_dt == DT_E1M2;
    const uint16_t* xs = (const uint16_t*)p.x;
    // rows travel eight at a time (eight independent 16-byte loads in flight per thread); rows past the block repeat its last
    auto fetch8 = [&](int64_t a, int64_t a1, uint4 (&buf)[8]) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int64_t aj = a + j < a1 ? a + j : a1 - 1;
            buf[j] = *(const uint4*)(xs + (o * p.A + aj) * p.inner + ic * 8);
        }
    };
    auto widen = [&](const uint4& xv, float (&v)[8]) {
        const uint32_t w[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const uint32_t h = (w[e >> 1] >> (16 * (e & 1))) & 0xffffu;
            v[e] = p.x_dt == DT_BF16 ? u2f(h << 16) : f16_to_f32((uint16_t)h);
        }
    };
    uint32_t sb[8] = {0, 0, 0, 0, 0, 0, 0, 0};   // per column: the pair's two scale bytes (an absent second block: 0)
    for (int h = 0; h < 2; h++) {
        const int64_t b = 2 * pb + h;
        if (b >= p.nblk) break;
        const int64_t a0 = b * p.block, a1 = a0 + p.block < p.A ? a0 + p.block : p.A;
        float amax[8], inv_scale[8];
        uint32_t badm = 0;
#pragma unroll
        for (int e = 0; e < 8; e++) amax[e] = 0.0f;
        for (int64_t a = a0; a < a1; a += 8) {
            uint4 buf[8];
            fetch8(a, a1, buf);
#pragma unroll
            for (int j = 0; j < 8; j++) {   // (a repeated last row changes neither the maximum nor the flags)
                float v[8];
                widen(buf[j], v);
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const float t = fabsf(v[e]);
                    badm |= (t < __builtin_inff() ? 0u : 1u) << e;
                    amax[e] = fmaxf(amax[e], t);
                }
            }
        }
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const bool bd = (badm >> e) & 1u;
            int share = -127;
            if (!bd && amax[e] != 0.0f) {
                if (p.scale_alg == 1) {
                    const uint32_t u = f2u(__fdiv_rn(amax[e], tmax));
                    int ex = (int)(u >> 23);
                    const uint32_t mant = u & 0x7fffffu;
                    if ((ex > 0 && ex < 254 && mant > 0) || (ex == 0 && mant > 0x400000u)) ex += 1;
                    share = ex - 127;
                } else {
                    const int ex = (int)(f2u(amax[e]) >> 23);
                    share = (ex == 0 || ex - 127 - emax < -127) ? -127 : ex - 127 - emax;
                }
            }
            sb[e] |= (bd ? 0xFFu : (uint32_t)(share + 127)) << (8 * h);
            inv_scale[e] = u2f((uint32_t)(127 - share) << 23);
        }
        for (int64_t a = a0; a < a1; a += 8) {
            uint4 buf[8];
            fetch8(a, a1, buf);
#pragma unroll
            for (int j = 0; j < 8; j++) {
                if (a + j >= a1) break;
                float v[8];
                widen(buf[j], v);
                const int64_t i = (o * p.A + a + j) * p.inner + ic * 8;
                if constexpr (YT != 0) {
                    float qf[8];
#pragma unroll
                    for (int e = 0; e < 8; e++) qf[e] = mx_scaled<YT>(v[e], inv_scale[e], (badm >> e) & 1u);
                    const uint2 pk = mx_pack8<YT>(qf);
                    if constexpr (YT == DT_E2M1) *(uint32_t*)(p.y + (i >> 1)) = pk.x;
                    else *(uint2*)(p.y + i) = pk;
                    continue;
                }
                uint32_t q[8];
#pragma unroll
                for (int e = 0; e < 8; e++) q[e] = mxg_element(v[e], inv_scale[e], (badm >> e) & 1u, emin, mbits, tmax, p.round_mode, p.y_dt);
                if (fp4) {
                    uint32_t w = 0;
#pragma unroll
                    for (int e = 0; e < 8; e++) w |= q[e] << (4 * e);
                    *(uint32_t*)(p.y + (i >> 1)) = w;
                } else {
                    *(uint2*)(p.y + i) = make_uint2(q[0] | (q[1] << 8) | (q[2] << 16) | (q[3] << 24), q[4] | (q[5] << 8) | (q[6] << 16) | (q[7] << 24));
                }
            }
        }
    }
    *(uint4*)(p.scale + ((o * p.np + pb) * p.inner + ic * 8) * 2) =
        make_uint4(sb[0] | (sb[1] << 16), sb[2] | (sb[3] << 16), sb[4] | (sb[5] << 16), sb[6] | (sb[7] << 16));
}

static int launch_mx_quant_general(const OpsnnMxQuantArgs& a, hipStream_t st)
{
    MxGeneralParams p{};
    p.x = a.x; p.y = (uint8_t*)a.y; p.scale = (uint8_t*)a.scale;
    p.outer = a.outer; p.A = a.axis_len; p.inner = a.inner;
    p.block = a.block ? (int)a.block : 32; p.scale_alg = a.scale_alg; p.round_mode = a.round_mode;
    p.x_dt = a.x_dtype; p.y_dt = a.y_dtype;
    if (p.outer <= 0 || p.A <= 0 || p.inner <= 0 || p.block <= 0 || p.block % 32 != 0 || p.block > 1024) return -2;
    if (p.x_dt != DT_F16 && p.x_dt != DT_BF16 && p.x_dt != DT_F32) return -2;
    const bool fp4 = p.y_dt == DT_E2M1 || p.y_dt == DT_E1M2;
    if (!fp4 && p.y_dt != DT_E4M3 && p.y_dt != DT_E5M2) return -2;
    if (p.round_mode < 0 || p.round_mode > 4 || (p.scale_alg != 0 && (p.scale_alg != 1 || fp4))) return -2;
    if (fp4 && ((p.inner > 1 ? p.inner : p.A) & 1)) return -2;
    p.nblk = (p.A + p.block - 1) / p.block; p.np = (p.nblk + 1) / 2;
    if (p.x_dt != DT_F32 && p.inner % 8 == 0 && (uintptr_t)p.x % 16 == 0 && (uintptr_t)p.y % 8 == 0 && (uintptr_t)p.scale % 16 == 0) {
        const int64_t wgs8 = (p.outer * p.np * (p.inner / 8) + 255) / 256;
        if (wgs8 > 0x7fffffff) return -1;
        const dim3 grid((unsigned)wgs8);
        if (p.round_mode == 0 && p.y_dt == DT_E2M1) hipLaunchKernelGGL(mx_quant_inner8_kernel<DT_E2M1>, grid, dim3(256), 0, st, p);
        else if (p.round_mode == 0 && p.y_dt == DT_E4M3) hipLaunchKernelGGL(mx_quant_inner8_kernel<DT_E4M3>, grid, dim3(256), 0, st, p);
        else if (p.round_mode == 0 && p.y_dt == DT_E5M2) hipLaunchKernelGGL(mx_quant_inner8_kernel<DT_E5M2>, grid, dim3(256), 0, st, p);
        else hipLaunchKernelGGL(mx_quant_inner8_kernel<0>, grid, dim3(256), 0, st, p);
        return (int)hipGetLastError();
    }
    const int64_t iw = fp4 && p.inner > 1 ? p.inner / 2 : p.inner;
    const int64_t wgs = (p.outer * p.nblk * iw + 255) / 256;
    if (wgs > 0x7fffffff) return -1;
    hipLaunchKernelGGL(mx_quant_general_kernel, dim3((unsigned)wgs), dim3(256), 0, st, p);
    return (int)hipGetLastError();
}

template <int X_DT, int Y_DT>
static int launch_mx_quant(const MxQuantParams& p, int variant, hipStream_t st)
{
    const bool vec = p.block == 32 && p.cols % 8 == 0 && (uintptr_t)p.x % 16 == 0 && (uintptr_t)p.y % 8 == 0;
    const int64_t groups = p.rows * p.nblk;
    const bool wide = variant != 2 && p.block >= 64 && p.block <= 1024 && (p.block & (p.block - 1)) == 0 && p.cols % 8 == 0 &&
                      (uintptr_t)p.x % 16 == 0 && (uintptr_t)p.y % 8 == 0;
    if (wide) {
        const int ppl = p.block == 1024 ? 2 : 1;
        const int lg = __builtin_ctzll((unsigned long long)(p.block / 8 / ppl));
        const int64_t cpr = (p.cols + 512 * ppl - 1) / (512 * ppl);
        const int64_t wgs = (p.rows * cpr + 3) / 4;
        if (wgs > 0x7fffffff || cpr > 0x7fffffff) return -1;
        if (ppl == 2) hipLaunchKernelGGL((mx_quant_wideblock_kernel<X_DT, Y_DT, 2>), dim3((unsigned)wgs), dim3(256), 0, st, p, lg, (int)cpr);
        else hipLaunchKernelGGL((mx_quant_wideblock_kernel<X_DT, Y_DT, 1>), dim3((unsigned)wgs), dim3(256), 0, st, p, lg, (int)cpr);
        return (int)hipGetLastError();
    }
    if (variant != 2 && vec) {
        // four pairs per group once that still leaves every SIMD eight waves
        const int nb = groups * 4 / 64 >= (int64_t)4 * 8 * 1024 ? 4 : 1;
        const int64_t ngroups = (groups + nb - 1) / nb;
        const int64_t wgs = (ngroups * 4 + 255) / 256;
        if (wgs > 0x7fffffff) return -1;
        const bool flat = p.cols % 32 == 0 && (p.nblk & 1) == 0;
        auto go = [&](auto kernel) { hipLaunchKernelGGL(kernel, dim3((unsigned)wgs), dim3(256), 0, st, p, ngroups); };
        if (nb == 4) { if (flat) go(mx_quant_kernel<X_DT, Y_DT, 4, true>); else go(mx_quant_kernel<X_DT, Y_DT, 4, false>); }
        else { if (flat) go(mx_quant_kernel<X_DT, Y_DT, 1, true>); else go(mx_quant_kernel<X_DT, Y_DT, 1, false>); }
    } else {
        if (variant == 1) return -4;
        const int64_t wgs = (groups + 255) / 256;
        if (wgs > 0x7fffffff) return -1;
        hipLaunchKernelGGL((mx_quant_generic_kernel<X_DT, Y_DT>), dim3((unsigned)wgs), dim3(256), 0, st, p);
    }
    return (int)hipGetLastError();
}

template <int X_DT>
static int launch_mx_quant_x(const MxQuantParams& p, int y_dt, int variant, hipStream_t st)
{
    switch (y_dt) {
        case DT_E2M1: return launch_mx_quant<X_DT, DT_E2M1>(p, variant, st);
        case DT_E4M3: return launch_mx_quant<X_DT, DT_E4M3>(p, variant, st);
        case DT_E5M2: return launch_mx_quant<X_DT, DT_E5M2>(p, variant, st);
        default: return -2;
    }
}

}  // namespace opsnn

using namespace opsnn;

extern "C" int opsnnDynamicMxQuant(const OpsnnMxQuantArgs* a, void* stream)
{
    if (!a || !a->x || !a->y || !a->scale) return -1;
    if (a->axis_len > 0) return launch_mx_quant_general(*a, (hipStream_t)stream);
    if (a->rows <= 0 || a->cols <= 0) return -1;
    if (a->x_dtype != DT_F16 && a->x_dtype != DT_BF16) return -2;
    if (a->y_dtype == DT_E2M1 && (a->cols & 1)) return -2;
    MxQuantParams p{};
    p.x = (const uint16_t*)a->x; p.y = (uint8_t*)a->y; p.scale = (uint8_t*)a->scale;
    p.block = a->block ? (int)a->block : 32;
    p.scale_alg = a->scale_alg;
    if (p.block <= 0 || p.block % 32 != 0 || p.block > 1024 || (p.scale_alg != 0 && (p.scale_alg != 1 || a->y_dtype == DT_E2M1))) return -2;
    p.rows = a->rows; p.cols = a->cols; p.nblk = (a->cols + p.block - 1) / p.block; p.spitch = (p.nblk + 1) / 2 * 2;
    if (a->x_dtype == DT_BF16) return launch_mx_quant_x<DT_BF16>(p, a->y_dtype, a->force_variant, (hipStream_t)stream);
    return launch_mx_quant_x<DT_F16>(p, a->y_dtype, a->force_variant, (hipStream_t)stream);
}
