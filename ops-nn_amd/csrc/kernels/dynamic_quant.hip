// Dynamic per-token quantisation: the activation quantizer that feeds the quantized matmuls
// (aclnnDynamicQuant / aclnnDynamicQuantV2; formula quant/dynamic_quant/tests/assets/golden.py:17-122).
//
// Per row of x [rows, cols] (fp16 / bf16), every step a separately rounded fp32 operation:
//   v = x * smooth                                  (optional, one factor per column)
//   symmetric:   scale = max|v| * (1 / tmax);                           q = v / scale
//   asymmetric:  scale = (max v - min v) * (1 / tmax2);  offset = tmax - max v / scale;  q = v / scale + offset
//   y = int8 / int4: round half to even;  e4m3 / e5m2: the cast rounds
// HBM-bound: 2 bytes read and 1 (or 1/2) written per element, one pass.  A row lives in registers between the reduction and
// the quantisation: up to 8 pieces of 8 elements per thread, one wave per row up to 2048 columns, or 4096 with many rows (four rows
// per workgroup, reduction by lane exchange only), and one workgroup per row up to 16384 (partial results of the four waves
// through LDS).  Rows that are longer, or whose length is not a multiple of 8, take the two-pass kernel that reads x
// twice (the second time from cache).
#include "common.hip.h"
#include "launch.h"

namespace opsnn {

struct DynQuantParams {
    const uint16_t* x; const uint16_t* smooth; void* y; float* scale; float* offset;
    int64_t rows, cols;
    int y_dt; float tmax, rcp;   // rcp = 1 / tmax (symmetric) or 1 / tmax2
    const void* gi; int gi_i64; int64_t groups;   // per-expert smooth rows: expert e owns the rows below gi[e] that no earlier expert owns
};

// Smooth row of a row of x: p.smooth itself without experts; with experts the row of the first expert whose end lies
// above `row` (binary search; the ends ascend), nullptr-equivalent -1 past the last end.
__device__ __forceinline__ int64_t smooth_row_of(const DynQuantParams& p, int64_t row)
{
    if (!p.gi) return 0;
    int64_t lo = 0, hi = p.groups;   // first e in [lo, hi) with end(e) > row
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        const int64_t end = p.gi_i64 ? ((const int64_t*)p.gi)[mid] : (int64_t)((const int32_t*)p.gi)[mid];
        if (end > row) hi = mid;
        else lo = mid + 1;
    }
    return lo < p.groups ? lo : -1;
}

template <int X_DT>
__device__ __forceinline__ float x_to_f32(uint32_t h)
{
    if constexpr (X_DT == DT_BF16) return u2f(h << 16);
    else return f16_to_f32((uint16_t)h);
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

// How a row's elements are divided by its scale.  An IEEE division costs about a dozen instructions per element; with the
// correctly rounded reciprocal r of the scale (one division per row), q0 = RN(v * r), e = v - q0 * scale (exact in a
// fused multiply-add) and q = RN(q0 + e * r) give the correctly rounded quotient (Markstein's theorem) unless the scale's
// mantissa is all ones or an intermediate leaves the normal range -- rows where that could happen keep the division.
struct RowQuant {
    float scale, offset, rcp;
    bool ok;        // false: a row without range, its outputs are zeros
    bool fast;      // the reciprocal form is exact for this row
};

template <int Y_DT, bool ASYM>
__device__ __forceinline__ uint32_t quant_one(float v, const RowQuant& r)
{
    float q = 0.0f;
    if (r.ok) {
        if (r.fast) {
            const float q0 = __fmul_rn(v, r.rcp);
            q = __fmaf_rn(__fmaf_rn(-q0, r.scale, v), r.rcp, q0);
        } else {
            q = __fdiv_rn(v, r.scale);
        }
        if (ASYM) q = __fadd_rn(q, r.offset);
    }
    if constexpr (Y_DT == DT_E4M3 || Y_DT == DT_E5M2) {
        // |q| <= tmax up to the rounding of the division: clamped, the hardware conversion is the software rounding
        constexpr float tmax = Y_DT == DT_E4M3 ? 448.0f : 57344.0f;
        if (!(q == q)) return ((f2u(q) >> 24) & 0x80u) | 0x7fu;
        return cvt2_fp8_in_range<Y_DT>(fminf(fmaxf(q, -tmax), tmax), 0.0f) & 0xffu;
    } else {
        constexpr float lo = Y_DT == DT_I8 ? -128.0f : -8.0f, hi = Y_DT == DT_I8 ? 127.0f : 7.0f;
        float t = __builtin_rintf(q);
        t = __builtin_amdgcn_fmed3f((t == t) ? t : 0.0f, lo, hi);
        return (uint32_t)(int)t & (Y_DT == DT_I8 ? 0xffu : 0xfu);
    }
}

// scale / offset of a row from its reduced extremes
template <bool ASYM>
__device__ __forceinline__ RowQuant row_params(const DynQuantParams& p, float amax, float vmax, float vmin)
{
    RowQuant r;
    if (!ASYM) {
        r.scale = __fmul_rn(amax, p.rcp);
        r.offset = 0.0f;
    } else {
        r.scale = __fmul_rn(__fsub_rn(vmax, vmin), p.rcp);
        r.offset = __fsub_rn(p.tmax, __fdiv_rn(vmax, r.scale));
    }
    r.ok = r.scale > 0.0f && r.scale < __builtin_inff();
    if (!r.ok) r.offset = 0.0f;
    r.rcp = __fdiv_rn(1.0f, r.scale);
    // |v| <= max|v| = O(scale * tmax): with the scale in [2^-60, 2^60] and max|v| >= 2^-60 every product stays normal or
    // rounds to a quotient far below the first rounding boundary (1/2, or 2^-17 for e5m2)
    r.fast = r.ok && (f2u(r.scale) & 0x7fffffu) != 0x7fffffu && r.scale > 0x1p-60f && r.scale < 0x1p60f;
    return r;
}

// TPR threads per row (64: one wave, 256: the workgroup), pieces of 8 elements held in registers.
template <int X_DT, int Y_DT, bool ASYM, int TPR>
__global__ __launch_bounds__(256) void dynamic_quant_rows_kernel(DynQuantParams p)
{
    constexpr int RPW = 256 / TPR;   // rows per workgroup
    constexpr int MAXP = 8;
    __shared__ float red[3][4];
    const int t = threadIdx.x % TPR;
    const int64_t row = (int64_t)blockIdx.x * RPW + threadIdx.x / TPR;
    const int64_t srow = row < p.rows ? smooth_row_of(p, row) : -1;
    const bool live = row < p.rows && srow >= 0;   // whole waves: TPR is a multiple of 64
    const int64_t pieces = p.cols / 8;
    const uint4* smr = (const uint4*)(p.smooth + (srow > 0 ? srow : 0) * p.cols);
    const uint4* xr = (const uint4*)(p.x + (live ? row : 0) * p.cols);
    uint4 buf[MAXP];
    float amax = 0.0f, vmax = -__builtin_inff(), vmin = __builtin_inff();
    auto element = [&](const uint4& xv, const uint4& sv, int e) {
        const uint32_t w[4] = {xv.x, xv.y, xv.z, xv.w}, sw[4] = {sv.x, sv.y, sv.z, sv.w};
        float v = x_to_f32<X_DT>((w[e >> 1] >> (16 * (e & 1))) & 0xffffu);
        if (p.smooth) v = __fmul_rn(v, x_to_f32<X_DT>((sw[e >> 1] >> (16 * (e & 1))) & 0xffffu));
        return v;
    };
#pragma unroll
    for (int i = 0; i < MAXP; i++) {
        const int64_t c = (int64_t)i * TPR + t;
        if (live && c < pieces) {
            buf[i] = xr[c];
            uint4 sm = make_uint4(0, 0, 0, 0);
            if (p.smooth) sm = smr[c];
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float v = element(buf[i], sm, e);
                if (ASYM) { vmax = fmaxf(vmax, v); vmin = fminf(vmin, v); }
                else amax = fmaxf(amax, fabsf(v));
            }
        }
    }
    if (ASYM) { vmax = wave_max(vmax); vmin = -wave_max(-vmin); }
    else amax = wave_max(amax);
    if constexpr (TPR == 256) {
        const int w = threadIdx.x >> 6;
        if ((threadIdx.x & 63) == 0) { red[0][w] = amax; red[1][w] = vmax; red[2][w] = vmin; }
        __syncthreads();
        amax = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
        vmax = fmaxf(fmaxf(red[1][0], red[1][1]), fmaxf(red[1][2], red[1][3]));
        vmin = fminf(fminf(red[2][0], red[2][1]), fminf(red[2][2], red[2][3]));
    }
    if (!live) return;
    const RowQuant r = row_params<ASYM>(p, amax, vmax, vmin);
    if (t == 0) {
        p.scale[row] = r.scale;
        if (ASYM) p.offset[row] = r.offset;
    }
#pragma unroll
    for (int i = 0; i < MAXP; i++) {
        const int64_t c = (int64_t)i * TPR + t;
        if (c < pieces) {
            uint4 sm = make_uint4(0, 0, 0, 0);
            if (p.smooth) sm = smr[c];
            uint32_t lo = 0, hi = 0;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const uint32_t b = quant_one<Y_DT, ASYM>(element(buf[i], sm, e), r);
                if (Y_DT == DT_I4) lo |= b << (4 * e);
                else if (e < 4) lo |= b << (8 * e);
                else hi |= b << (8 * (e - 4));
            }
            if (Y_DT == DT_I4) ((uint32_t*)p.y)[row * pieces + c] = lo;
            else ((uint2*)p.y)[row * pieces + c] = make_uint2(lo, hi);
        }
    }
}

// Any row length: one workgroup per row, element-wise loads, x read twice.  int4 needs an even length (two per byte).
template <int X_DT, int Y_DT, bool ASYM>
__global__ __launch_bounds__(256) void dynamic_quant_two_pass_kernel(DynQuantParams p)
{
    __shared__ float red[3][4];
    const int64_t row = blockIdx.x;
    const uint16_t* xr = p.x + row * p.cols;
    const int64_t srow = smooth_row_of(p, row);
    if (srow < 0) return;   // the whole workgroup: past the last expert's rows
    const uint16_t* smr = p.smooth + srow * p.cols;
    float amax = 0.0f, vmax = -__builtin_inff(), vmin = __builtin_inff();
    auto element = [&](int64_t c) {
        float v = x_to_f32<X_DT>(xr[c]);
        if (p.smooth) v = __fmul_rn(v, x_to_f32<X_DT>(smr[c]));
        return v;
    };
    for (int64_t c = threadIdx.x; c < p.cols; c += 256) {
        const float v = element(c);
        amax = fmaxf(amax, fabsf(v));
        vmax = fmaxf(vmax, v);
        vmin = fminf(vmin, v);
    }
    amax = wave_max(amax); vmax = wave_max(vmax); vmin = -wave_max(-vmin);
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { red[0][w] = amax; red[1][w] = vmax; red[2][w] = vmin; }
    __syncthreads();
    amax = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
    vmax = fmaxf(fmaxf(red[1][0], red[1][1]), fmaxf(red[1][2], red[1][3]));
    vmin = fminf(fminf(red[2][0], red[2][1]), fminf(red[2][2], red[2][3]));
    const RowQuant r = row_params<ASYM>(p, amax, vmax, vmin);
    if (threadIdx.x == 0) {
        p.scale[row] = r.scale;
        if (ASYM) p.offset[row] = r.offset;
    }
    if (Y_DT == DT_I4) {
        uint8_t* yr = (uint8_t*)p.y + row * (p.cols / 2);
        for (int64_t c = threadIdx.x; c < p.cols / 2; c += 256)
            yr[c] = (uint8_t)(quant_one<Y_DT, ASYM>(element(2 * c), r) | (quant_one<Y_DT, ASYM>(element(2 * c + 1), r) << 4));
    } else {
        uint8_t* yr = (uint8_t*)p.y + row * p.cols;
        for (int64_t c = threadIdx.x; c < p.cols; c += 256) yr[c] = (uint8_t)quant_one<Y_DT, ASYM>(element(c), r);
    }
}

template <int X_DT, int Y_DT, bool ASYM>
static int launch_dynamic_quant(const DynQuantParams& p, int variant, hipStream_t st)
{
    const bool vec = p.cols % 8 == 0 && p.cols <= 8 * 8 * 256 && (uintptr_t)p.x % 16 == 0 && (uintptr_t)p.y % 8 == 0 &&
                     (!p.smooth || (uintptr_t)p.smooth % 16 == 0);
    if (variant == 2 || !vec) {
        if (variant == 1) return -4;
        hipLaunchKernelGGL((dynamic_quant_two_pass_kernel<X_DT, Y_DT, ASYM>), dim3((unsigned)p.rows), dim3(256), 0, st, p);
    } else if (p.cols <= 2048 || (p.cols <= 4096 && p.rows >= 16384)) {
        // one wave per row: no barrier, no LDS.  Up to 4096 columns (8 pieces per lane) when there are rows enough to
        // fill the SIMDs with such waves (65536 x 4096: 182 against 209 us; 2048 x 4096: 9.9 against 8.1 us)
        hipLaunchKernelGGL((dynamic_quant_rows_kernel<X_DT, Y_DT, ASYM, 64>), dim3((unsigned)((p.rows + 3) / 4)), dim3(256), 0, st, p);
    } else {
        hipLaunchKernelGGL((dynamic_quant_rows_kernel<X_DT, Y_DT, ASYM, 256>), dim3((unsigned)p.rows), dim3(256), 0, st, p);
    }
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------------------------
// "pertensor" and "perchannel": the extremes are reduced over many rows, so the work is split in kernels.  The scale
// buffer (and the offset buffer in the asymmetric form) first collects the extremes through integer atomics on an
// order-preserving key of the float (max|v| in scale; or max v in scale and min v in offset), the quantising kernel reads
// them from there and derives scale and offset per element group, and a last small kernel turns the collected extremes
// into the scale and offset values.  Maxima and minima do not depend on the order of the atomics: the result is exact.
__device__ __forceinline__ uint32_t float_key(float f)
{
    const uint32_t u = f2u(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_float(uint32_t k) { return u2f((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k); }

// slot of element (row, col): pertensor 0; perchannel (row / chan_rows) * cols + col
struct WideQuantParams {
    DynQuantParams p;
    int mode;            // 1 pertensor, 2 perchannel
    int64_t chan_rows, nslots;
    uint32_t* smax;      // = p.scale
    uint32_t* smin;      // = p.offset (asymmetric) or null
};

__global__ __launch_bounds__(256) void wide_quant_init_kernel(WideQuantParams w)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= w.nslots) return;
    w.smax[i] = w.smin ? float_key(-__builtin_inff()) : float_key(0.0f);
    if (w.smin) w.smin[i] = float_key(__builtin_inff());
}

// one thread per (row chunk of 64 rows, column): coalesced over columns; a workgroup covers 256 columns of one chunk
template <int X_DT>
__global__ __launch_bounds__(256) void wide_quant_reduce_kernel(WideQuantParams w)
{
    const DynQuantParams& p = w.p;
    const int64_t col = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t r0 = (int64_t)blockIdx.y * 64;
    const bool inside = col < p.cols;   // lanes past the last column stay for the wave reduction with neutral values
    float vmax = -__builtin_inff(), vmin = __builtin_inff();
    int64_t slot = -1;
    for (int64_t r = r0; inside && r < r0 + 64 && r < p.rows; r++) {
        const int64_t s = w.mode == 1 ? 0 : (r / w.chan_rows) * p.cols + col;
        if (s != slot && slot >= 0) {   // a new batch begins inside the chunk: hand in what was collected
            if (w.smin) { atomicMax(w.smax + slot, float_key(vmax)); atomicMin(w.smin + slot, float_key(vmin)); }
            else atomicMax(w.smax + slot, float_key(fmaxf(vmax, -vmin)));
            vmax = -__builtin_inff(); vmin = __builtin_inff();
        }
        slot = s;
        float v = x_to_f32<X_DT>(p.x[r * p.cols + col]);
        if (p.smooth) v = __fmul_rn(v, x_to_f32<X_DT>(p.smooth[w.mode == 1 ? col : r % w.chan_rows]));
        vmax = fmaxf(vmax, v);
        vmin = fminf(vmin, v);
    }
    if (w.mode == 1) {   // one slot for everybody: reduce the wave first
        vmax = wave_max(vmax);
        vmin = -wave_max(-vmin);
        if ((threadIdx.x & 63) != 0 || r0 >= p.rows) return;
        slot = 0;
    }
    if (slot < 0) return;
    if (w.smin) { atomicMax(w.smax + slot, float_key(vmax)); atomicMin(w.smin + slot, float_key(vmin)); }
    else atomicMax(w.smax + slot, float_key(fmaxf(vmax, -vmin)));
}

template <int X_DT, int Y_DT, bool ASYM>
__global__ __launch_bounds__(256) void wide_quant_apply_kernel(WideQuantParams w)
{
    const DynQuantParams& p = w.p;
    const int64_t pair = (int64_t)blockIdx.x * 256 + threadIdx.x;   // two neighbouring columns per thread (an int4 byte)
    const int64_t ppr = (p.cols + 1) / 2;
    if (pair >= p.rows * ppr) return;
    const int64_t row = pair / ppr, c0 = (pair % ppr) * 2;
    uint32_t out[2] = {0, 0};
    for (int e = 0; e < 2 && c0 + e < p.cols; e++) {
        const int64_t col = c0 + e;
        const int64_t slot = w.mode == 1 ? 0 : (row / w.chan_rows) * p.cols + col;
        const float a = key_float(w.smax[slot]);
        const RowQuant r = row_params<ASYM>(p, a, a, ASYM ? key_float(w.smin[slot]) : 0.0f);
        float v = x_to_f32<X_DT>(p.x[row * p.cols + col]);
        if (p.smooth) v = __fmul_rn(v, x_to_f32<X_DT>(p.smooth[w.mode == 1 ? col : row % w.chan_rows]));
        out[e] = quant_one<Y_DT, ASYM>(v, r);
    }
    if (Y_DT == DT_I4) ((uint8_t*)p.y)[(row * p.cols + c0) / 2] = (uint8_t)(out[0] | (out[1] << 4));
    else {
        ((uint8_t*)p.y)[row * p.cols + c0] = (uint8_t)out[0];
        if (c0 + 1 < p.cols) ((uint8_t*)p.y)[row * p.cols + c0 + 1] = (uint8_t)out[1];
    }
}

// ---- the same two passes for rows of whole 16-byte pieces (cols % 8 == 0, x 16-byte aligned) ----
// A workgroup is 64 pieces of 8 columns x 4 row lanes and walks `rpb` rows of one batch (rows that share their slots);
// a thread keeps its 8 columns' extremes (reduce) or their quantisation parameters (apply) in registers over its rows.
// blockIdx.x = block of 64 pieces, blockIdx.y = batch * chunks + chunk of rpb rows.
struct WideTile { int64_t col0, r_begin, r_end, batch; bool inside; };
__device__ __forceinline__ WideTile wide_tile(const WideQuantParams& w, int rpb, int chunks)
{
    WideTile t;
    const int64_t b = blockIdx.y / chunks, c = blockIdx.y - b * chunks;
    t.batch = b;
    t.col0 = ((int64_t)blockIdx.x * 64 + (threadIdx.x & 63)) * 8;
    t.inside = t.col0 < w.p.cols;
    t.r_begin = b * w.chan_rows + c * rpb;
    const int64_t batch_end = (b + 1) * w.chan_rows;
    t.r_end = t.r_begin + rpb < batch_end ? t.r_begin + rpb : batch_end;
    return t;
}
// the 8 values of a piece, smoothed: pertensor by the column's factor, perchannel by the row's
template <int X_DT>
__device__ __forceinline__ void wide_piece(const WideQuantParams& w, const WideTile& t, int64_t r, const float (&smc)[8], float (&v)[8])
{
    const uint4 xv = *(const uint4*)(w.p.x + r * w.p.cols + t.col0);
    const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
    float smr = 1.0f;
    if (w.p.smooth && w.mode == 2) smr = x_to_f32<X_DT>(w.p.smooth[r - t.batch * w.chan_rows]);
#pragma unroll
    for (int e = 0; e < 8; e++) {
        v[e] = x_to_f32<X_DT>((xw[e >> 1] >> (16 * (e & 1))) & 0xffffu);
        if (w.p.smooth) v[e] = __fmul_rn(v[e], w.mode == 1 ? smc[e] : smr);
    }
}
template <int X_DT>
__device__ __forceinline__ void wide_column_smooth(const WideQuantParams& w, const WideTile& t, float (&smc)[8])
{
#pragma unroll
    for (int e = 0; e < 8; e++) smc[e] = 1.0f;
    if (w.p.smooth && w.mode == 1 && t.inside) {
        const uint4 sv = *(const uint4*)(w.p.smooth + t.col0);
        const uint32_t sw[4] = {sv.x, sv.y, sv.z, sv.w};
#pragma unroll
        for (int e = 0; e < 8; e++) smc[e] = x_to_f32<X_DT>((sw[e >> 1] >> (16 * (e & 1))) & 0xffffu);
    }
}

template <int X_DT>
__global__ __launch_bounds__(256) void wide_quant_reduce8_kernel(WideQuantParams w, int rpb, int chunks)
{
    __shared__ float red[2][3][64][8];
    const WideTile t = wide_tile(w, rpb, chunks);
    const int rl = threadIdx.x >> 6, lv = threadIdx.x & 63;
    float smc[8], vmax[8], vmin[8];
    wide_column_smooth<X_DT>(w, t, smc);
#pragma unroll
    for (int e = 0; e < 8; e++) { vmax[e] = -__builtin_inff(); vmin[e] = __builtin_inff(); }
    if (t.inside) {
        for (int64_t r = t.r_begin + rl; r < t.r_end; r += 4) {
            float v[8];
            wide_piece<X_DT>(w, t, r, smc, v);
#pragma unroll
            for (int e = 0; e < 8; e++) { vmax[e] = fmaxf(vmax[e], v[e]); vmin[e] = fminf(vmin[e], v[e]); }
        }
    }
    if (rl > 0) {
#pragma unroll
        for (int e = 0; e < 8; e++) { red[0][rl - 1][lv][e] = vmax[e]; red[1][rl - 1][lv][e] = vmin[e]; }
    }
    __syncthreads();
    if (rl > 0) return;
#pragma unroll
    for (int j = 0; j < 3; j++)
#pragma unroll
        for (int e = 0; e < 8; e++) { vmax[e] = fmaxf(vmax[e], red[0][j][lv][e]); vmin[e] = fminf(vmin[e], red[1][j][lv][e]); }
    if (w.mode == 1) {   // one slot for everybody: the wave's extremes, one lane hands them in
        float a = vmax[0], b = vmin[0];
#pragma unroll
        for (int e = 1; e < 8; e++) { a = fmaxf(a, vmax[e]); b = fminf(b, vmin[e]); }
        a = wave_max(a);
        b = -wave_max(-b);
        if (lv != 0) return;
        if (w.smin) { atomicMax(w.smax, float_key(a)); atomicMin(w.smin, float_key(b)); }
        else atomicMax(w.smax, float_key(fmaxf(a, -b)));
        return;
    }
    if (!t.inside || t.r_begin >= t.r_end) return;
    const int64_t slot0 = t.batch * w.p.cols + t.col0;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        if (w.smin) { atomicMax(w.smax + slot0 + e, float_key(vmax[e])); atomicMin(w.smin + slot0 + e, float_key(vmin[e])); }
        else atomicMax(w.smax + slot0 + e, float_key(fmaxf(vmax[e], -vmin[e])));
    }
}

template <int X_DT, int Y_DT, bool ASYM>
__global__ __launch_bounds__(256) void wide_quant_apply8_kernel(WideQuantParams w, int rpb, int chunks)
{
    const WideTile t = wide_tile(w, rpb, chunks);
    if (!t.inside) return;
    const int rl = threadIdx.x >> 6;
    float smc[8];
    wide_column_smooth<X_DT>(w, t, smc);
    RowQuant rq[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
        if (w.mode == 1 && e > 0) { rq[e] = rq[0]; continue; }
        const int64_t slot = w.mode == 1 ? 0 : t.batch * w.p.cols + t.col0 + e;
        const float a = key_float(w.smax[slot]);
        rq[e] = row_params<ASYM>(w.p, a, a, ASYM ? key_float(w.smin[slot]) : 0.0f);
    }
    for (int64_t r = t.r_begin + rl; r < t.r_end; r += 4) {
        float v[8];
        wide_piece<X_DT>(w, t, r, smc, v);
        uint32_t q[8];
#pragma unroll
        for (int e = 0; e < 8; e++) q[e] = quant_one<Y_DT, ASYM>(v[e], rq[e]);
        if constexpr (Y_DT == DT_I4) {
            uint32_t o = 0;
#pragma unroll
            for (int e = 0; e < 8; e++) o |= q[e] << (4 * e);
            *(uint32_t*)((uint8_t*)w.p.y + (r * w.p.cols + t.col0) / 2) = o;
        } else {
            const uint32_t lo = q[0] | (q[1] << 8) | (q[2] << 16) | (q[3] << 24), hi = q[4] | (q[5] << 8) | (q[6] << 16) | (q[7] << 24);
            *(uint2*)((uint8_t*)w.p.y + r * w.p.cols + t.col0) = make_uint2(lo, hi);
        }
    }
}

template <bool ASYM>
__global__ __launch_bounds__(256) void wide_quant_finish_kernel(WideQuantParams w)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= w.nslots) return;
    const float a = key_float(w.smax[i]);
    const RowQuant r = row_params<ASYM>(w.p, a, a, ASYM ? key_float(w.smin[i]) : 0.0f);
    w.p.scale[i] = r.scale;
    if (ASYM) w.p.offset[i] = r.offset;
}

template <int X_DT, int Y_DT, bool ASYM>
static int launch_wide_quant(const DynQuantParams& p, int mode, int64_t chan_rows, hipStream_t st)
{
    WideQuantParams w{};
    w.p = p; w.mode = mode; w.chan_rows = mode == 2 ? chan_rows : p.rows;
    w.nslots = mode == 1 ? 1 : (p.rows / w.chan_rows) * p.cols;
    w.smax = (uint32_t*)p.scale; w.smin = ASYM ? (uint32_t*)p.offset : nullptr;
    const int64_t row_chunks = (p.rows + 63) / 64, pairs = p.rows * ((p.cols + 1) / 2);
    if (row_chunks > 65535 || (p.cols + 255) / 256 > 0x7fffffff || (pairs + 255) / 256 > 0x7fffffff || (w.nslots + 255) / 256 > 0x7fffffff) return -1;
    const dim3 slots((unsigned)((w.nslots + 255) / 256));
    hipLaunchKernelGGL(wide_quant_init_kernel, slots, dim3(256), 0, st, w);
    // rows of whole 16-byte pieces: the vector kernels, chunks of 64 rows (more when there would be too many workgroups)
    const int64_t batches = p.rows / w.chan_rows;
    int64_t rpb = 64;
    while (batches * ((w.chan_rows + rpb - 1) / rpb) > 65535) rpb *= 2;
    const int64_t chunks = (w.chan_rows + rpb - 1) / rpb;
    const bool vec = p.cols % 8 == 0 && (uintptr_t)p.x % 16 == 0 && (uintptr_t)p.y % 8 == 0 && (!p.smooth || (uintptr_t)p.smooth % 16 == 0) &&
                     rpb < (1 << 30) && chunks < (1 << 30);
    if (vec) {
        const dim3 grid((unsigned)((p.cols / 8 + 63) / 64), (unsigned)(batches * chunks));
        hipLaunchKernelGGL(wide_quant_reduce8_kernel<X_DT>, grid, dim3(256), 0, st, w, (int)rpb, (int)chunks);
        hipLaunchKernelGGL((wide_quant_apply8_kernel<X_DT, Y_DT, ASYM>), grid, dim3(256), 0, st, w, (int)rpb, (int)chunks);
    } else {
        hipLaunchKernelGGL(wide_quant_reduce_kernel<X_DT>, dim3((unsigned)((p.cols + 255) / 256), (unsigned)row_chunks), dim3(256), 0, st, w);
        hipLaunchKernelGGL((wide_quant_apply_kernel<X_DT, Y_DT, ASYM>), dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, st, w);
    }
    hipLaunchKernelGGL(wide_quant_finish_kernel<ASYM>, slots, dim3(256), 0, st, w);
    return (int)hipGetLastError();
}

template <int X_DT>
static int launch_wide_quant_x(const DynQuantParams& p, int mode, int64_t chan_rows, hipStream_t st)
{
    const bool asym = p.offset != nullptr;
    switch (p.y_dt) {
        case DT_I8: return asym ? launch_wide_quant<X_DT, DT_I8, true>(p, mode, chan_rows, st) : launch_wide_quant<X_DT, DT_I8, false>(p, mode, chan_rows, st);
        case DT_I4: return asym ? launch_wide_quant<X_DT, DT_I4, true>(p, mode, chan_rows, st) : launch_wide_quant<X_DT, DT_I4, false>(p, mode, chan_rows, st);
        case DT_E4M3: return asym ? launch_wide_quant<X_DT, DT_E4M3, true>(p, mode, chan_rows, st) : launch_wide_quant<X_DT, DT_E4M3, false>(p, mode, chan_rows, st);
        case DT_E5M2: return asym ? launch_wide_quant<X_DT, DT_E5M2, true>(p, mode, chan_rows, st) : launch_wide_quant<X_DT, DT_E5M2, false>(p, mode, chan_rows, st);
        default: return -2;
    }
}

template <int X_DT>
static int launch_dynamic_quant_x(const DynQuantParams& p, int variant, hipStream_t st)
{
    const bool asym = p.offset != nullptr;
    switch (p.y_dt) {
        case DT_I8: return asym ? launch_dynamic_quant<X_DT, DT_I8, true>(p, variant, st) : launch_dynamic_quant<X_DT, DT_I8, false>(p, variant, st);
        case DT_I4: return asym ? launch_dynamic_quant<X_DT, DT_I4, true>(p, variant, st) : launch_dynamic_quant<X_DT, DT_I4, false>(p, variant, st);
        case DT_E4M3: return asym ? launch_dynamic_quant<X_DT, DT_E4M3, true>(p, variant, st) : launch_dynamic_quant<X_DT, DT_E4M3, false>(p, variant, st);
        case DT_E5M2: return asym ? launch_dynamic_quant<X_DT, DT_E5M2, true>(p, variant, st) : launch_dynamic_quant<X_DT, DT_E5M2, false>(p, variant, st);
        default: return -2;
    }
}

}  // namespace opsnn

using namespace opsnn;

extern "C" int opsnnDynamicQuant(const OpsnnDynQuantArgs* a, void* stream)
{
    if (!a || !a->x || !a->y || !a->scale || a->rows <= 0 || a->cols <= 0 || a->rows > 0x7fffffff) return -1;
    if (a->x_dtype != DT_F16 && a->x_dtype != DT_BF16) return -2;
    DynQuantParams p{};
    switch (a->y_dtype) {
        case DT_I8: p.tmax = 127.0f; p.rcp = 1.0f / (a->offset ? 255.0f : 127.0f); break;
        case DT_I4: p.tmax = 7.0f; p.rcp = 1.0f / (a->offset ? 15.0f : 7.0f); break;
        case DT_E4M3: p.tmax = 448.0f; p.rcp = 1.0f / (a->offset ? 896.0f : 448.0f); break;
        case DT_E5M2: p.tmax = 57344.0f; p.rcp = 1.0f / (a->offset ? 114688.0f : 57344.0f); break;
        default: return -2;
    }
    if (a->y_dtype == DT_I4 && (a->cols & 1)) return -2;
    p.x = (const uint16_t*)a->x; p.smooth = (const uint16_t*)a->smooth; p.y = a->y; p.scale = a->scale; p.offset = a->offset;
    p.rows = a->rows; p.cols = a->cols; p.y_dt = a->y_dtype;
    if (a->group_index) {
        if (!a->smooth || a->groups <= 0 || (a->group_index_dtype != DT_I32 && a->group_index_dtype != 9 /* INT64 */)) return -2;
        p.gi = a->group_index; p.gi_i64 = a->group_index_dtype != DT_I32; p.groups = a->groups;
    }
    if (a->quant_mode == 1 || a->quant_mode == 2) {
        if (a->group_index || (a->quant_mode == 2 && (a->chan_rows <= 0 || a->rows % a->chan_rows != 0))) return -2;
        if (a->x_dtype == DT_BF16) return launch_wide_quant_x<DT_BF16>(p, a->quant_mode, a->chan_rows, (hipStream_t)stream);
        return launch_wide_quant_x<DT_F16>(p, a->quant_mode, a->chan_rows, (hipStream_t)stream);
    }
    if (a->quant_mode != 0) return -2;
    if (a->x_dtype == DT_BF16) return launch_dynamic_quant_x<DT_BF16>(p, a->force_variant, (hipStream_t)stream);
    return launch_dynamic_quant_x<DT_F16>(p, a->force_variant, (hipStream_t)stream);
}
