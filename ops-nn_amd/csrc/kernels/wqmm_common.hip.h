// Shared pieces of the weight-only decode kernels: launch parameters and the register-level dequantisation.
#pragma once
#include "launch.h"
#include "qgemm_core.hip.h"
#include <type_traits>

namespace opsnn {

struct WqParams {
    const uint16_t* x;       // [M, K] dense 16-bit
    const uint8_t* w;        // row n at w + n*ldw (bytes), K-contiguous
    int64_t ldw;
    const uint16_t* scale;   // element (g, n) at scale[g*s_rs + n*s_cs]
    const uint16_t* offset;  // same layout, or null
    int64_t s_rs, s_cs;
    const void* bias;
    int bias_dt;
    uint16_t* y;             // [M, N]
    int64_t M, N, K;
    int64_t group;           // elements per group (K if per-channel)
    int group_shift;         // log2(group) if it is a power of two, else -1
    int cpg_shift;           // streamlined kernel: log2(group / chunk), 31 for a per-channel scale
    int64_t m_base, m_rows;  // row slab handled by this launch
    // many-rows kernel: with m_slab > 0 the launch covers the rows m_base .. m_end - 1 in slabs of m_slab (= m_rows) rows,
    // one per blockIdx.y (the last one may be shorter)
    int64_t m_slab, m_end;
    // x-in-registers kernel with K split over workgroup columns (grid.y segments): fp32 partial sums [segments][M][N]
    float* part;
    // many-rows kernel with K split over blockIdx.z: ksplit segments of whole units of kunit k, as equal as that allows (K
    // stays the whole K), partial sums in part
    int ksplit;
    int64_t kunit;
    int cols64;              // launcher hint: up to 64 rows on the instance whose workgroups take 64 columns (K split over four waves)
    int w_float;             // weights are floating-point codes (4 bits: e2m1, 8 bits: e4m3), not two's-complement integers
    int scale_e8m0;          // scale is one e8m0 byte per element (MX), not a 16-bit value of x's dtype
    int mx8_rows;            // set by launch_wq_mx8_rows only: e4m3 codes with e8m0 scales per 32 on the many-rows kernel (MXFP8's x2)
    // fp8 block-scale form of the many-rows kernel (x is x1 widened to fp16, w is x2 in e4m3): fp32 scales per 128 x 128
    // block of w (bs2) and per row group and 128-block of x (bs1), output type of the call
    const float* bs1; const float* bs2;
    int64_t bs1_rs, bs1_cs, bs2_rs, bs2_cs;
    int bs_gsm, bs_out_dt;
};

typedef _Float16 h2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t u32(h2 v) { return __builtin_bit_cast(uint32_t, v); }

// ---- fp16 dequantisation: 8 int4 of one dword -> 4 packed pairs in element order [0,4], [1,5], [2,6], [3,7] ----
// q holds two's-complement nibbles; after xor 0x88888888 each nibble is w + 8 in 0..15.
__device__ __forceinline__ void dequant_i4_f16(uint32_t q, h2 off, h2 sc, bool has_off, h2 (&out)[4])
{
    const uint32_t u = q ^ 0x88888888u;
    const uint32_t u8 = u >> 8;
    const h2 c1032 = {(_Float16)-1032.0f, (_Float16)-1032.0f};
    const h2 c72 = {(_Float16)-72.0f, (_Float16)-72.0f};
    const h2 r16 = {(_Float16)0.0625f, (_Float16)0.0625f};
    h2 t0 = __builtin_bit_cast(h2, (u & 0x000F000Fu) | 0x64006400u);   // 1024 + (w+8)        elements 0, 4
    h2 t1 = __builtin_bit_cast(h2, (u & 0x00F000F0u) | 0x64006400u);   // 1024 + 16*(w+8)     elements 1, 5
    h2 t2 = __builtin_bit_cast(h2, (u8 & 0x000F000Fu) | 0x64006400u);  //                     elements 2, 6
    h2 t3 = __builtin_bit_cast(h2, (u8 & 0x00F000F0u) | 0x64006400u);  //                     elements 3, 7
    t0 = t0 + c1032;                                   // exact: w
    t2 = t2 + c1032;
    t1 = __builtin_elementwise_fma(t1, r16, c72);      // exact: (1024 + 16(w+8))/16 - 72 = w
    t3 = __builtin_elementwise_fma(t3, r16, c72);
    if (has_off) { t0 = t0 + off; t1 = t1 + off; t2 = t2 + off; t3 = t3 + off; }   // first rounding
    out[0] = t0 * sc; out[1] = t1 * sc; out[2] = t2 * sc; out[3] = t3 * sc;         // second rounding
}

// ---- fp16 dequantisation of 8 e2m1 codes of one dword -> 4 packed pairs in element order [0,4], [1,5], [2,6], [3,7] ----
// A code's three magnitude bits, placed at bits 11..9 of a half, read as the half 2^-14 times the code's value -- for the
// normal codes (exponent field 1..3 against a bias of 15 instead of 1) and for the two subnormal ones alike (0 and 2^-15 =
// 2^-14 * 0.5): one exact multiplication by 2^14 gives the weight, and the multiplication by the scale then rounds once,
// as the formula does (the weight is exact in fp16, T(w * s)).
__device__ __forceinline__ void dequant_fp4_f16(uint32_t q, h2 sc, h2 (&out)[4])
{
    const h2 k14 = {(_Float16)16384.0f, (_Float16)16384.0f};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t t = q >> (4 * i);
        const uint32_t bits = ((t & 0x00070007u) << 9) | ((t & 0x00080008u) << 12);
        out[i] = (__builtin_bit_cast(h2, bits) * k14) * sc;
    }
}

// ---- generic dequantisation of one weight to fp32 holding a value of x's dtype ----
template <int XDT>
__device__ __forceinline__ float round_x(float v)
{
    if constexpr (XDT == DT_F16) return (float)(_Float16)v;
    else return bf16_to_f32(bf16_bits(v));
}
template <int XDT>
__device__ __forceinline__ uint16_t bits_x(float v)
{
    if constexpr (XDT == DT_F16) return f16_bits(v);
    else return bf16_bits(v);
}
template <int XDT>
__device__ __forceinline__ float dequant_one(float w, float off, float sc, bool has_off)
{
    if (has_off) w = round_x<XDT>(w + off);
    return round_x<XDT>(w * sc);
}


}  // namespace opsnn
