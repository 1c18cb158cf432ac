// Weight pre-pack: one 4-bit value per 32-bit carrier element -> two values per byte, low nibble first.
//
// The device form of aclnnConvertWeightToINT4Pack, which the reference computes on the host between two copies
// (matmul/convert_weight_to_int4_pack/op_host/op_api/aclnn_convert_weight_to_int4_pack.cpp:79-126, 368-405):
//   int32 carrier:  nibble = value & 0xF
//   fp32 carrier:   the bit pattern, cut to sign + exponent + first mantissa bit, is looked up among the 16 fp4 e2m1
//                   values; a pattern that is none of them (0.75, 8.0, NaN, ...) gives code 0 with the sign dropped.
// HBM-bound: 4 bytes read and half a byte written per element.  A thread turns 16 elements (four 16-byte loads) into
// one 8-byte store; neighbouring threads read and write neighbouring pieces.
#include "common.hip.h"
#include "launch.h"

namespace opsnn {

// fp32 bits -> e2m1 code by the table of the reference (:43-63): after the cut the 9 bits sign-less exponent+mantissa
// are 0 (zero), 0xFC (0.5) or 0xFE..0x103 (1.0 .. 6.0); anything else is not in the table.
__device__ __forceinline__ uint32_t fp32_bits_to_e2m1(uint32_t u)
{
    const uint32_t mag = (u >> 22) & 0x1FFu, sign = (u >> 28) & 8u;
    if (mag == 0u) return sign;
    if (mag == 0xFCu) return sign | 1u;
    if (mag >= 0xFEu && mag <= 0x103u) return sign | (mag - 0xFCu);
    return 0u;
}

template <bool FP>
__device__ __forceinline__ uint32_t pack8(const uint4& a, const uint4& b)
{
    const uint32_t v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    uint32_t r = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) r |= (FP ? fp32_bits_to_e2m1(v[i]) : (v[i] & 15u)) << (4 * i);
    return r;
}

// n16 = count / 16 full pieces; the tail (count % 16 elements, even) is done by the last thread, byte by byte.
template <bool FP>
__global__ __launch_bounds__(256) void pack_b4_kernel(const uint32_t* __restrict__ src, uint8_t* __restrict__ dst, int64_t count)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t n16 = count / 16;
    if (t < n16) {
        const uint4* s = (const uint4*)(src + t * 16);
        const uint4 a = s[0], b = s[1], c = s[2], d = s[3];
        *(uint2*)(dst + t * 8) = make_uint2(pack8<FP>(a, b), pack8<FP>(c, d));
    } else if (t == n16) {
        for (int64_t i = n16 * 16; i + 1 < count; i += 2) {
            const uint32_t lo = FP ? fp32_bits_to_e2m1(src[i]) : (src[i] & 15u);
            const uint32_t hi = FP ? fp32_bits_to_e2m1(src[i + 1]) : (src[i + 1] & 15u);
            dst[i / 2] = (uint8_t)(lo | (hi << 4));
        }
    }
}

}  // namespace opsnn

using namespace opsnn;

extern "C" int opsnnPackB4(const void* src, int src_is_fp32, void* dst, int64_t count, void* stream)
{
    if (!src || !dst || count <= 0 || (count & 1) || (uintptr_t)src % 16 != 0 || (uintptr_t)dst % 8 != 0) return -1;
    const int64_t threads = count / 16 + 1;
    const dim3 grid((unsigned)((threads + 255) / 256)), block(256);
    if (grid.x == 0 || threads > (int64_t)0x7fffffff * 256) return -1;
    if (src_is_fp32) hipLaunchKernelGGL(pack_b4_kernel<true>, grid, block, 0, (hipStream_t)stream, (const uint32_t*)src, (uint8_t*)dst, count);
    else hipLaunchKernelGGL(pack_b4_kernel<false>, grid, block, 0, (hipStream_t)stream, (const uint32_t*)src, (uint8_t*)dst, count);
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------------------------
// aclnnTransQuantParamV2 / V3: fp32 scale (+ fp32 offset) -> the 64-bit packed quantisation parameter the per-tensor /
// per-channel matmul modes take (quant/trans_quant_param_v2/op_kernel/trans_quant_param_v2.h:224-300):
//   bits 0..31  the scale cut to sign, exponent and 10 mantissa bits -- truncated (round mode 0) or rounded to nearest
//               even with the carry running into the exponent, zero for a subnormal, infinity / NaN kept (round mode 1)
//   bits 37..45 rint(offset) clamped to [-256, 255] as a signed 9-bit field
//   bit 46      set
// A one-element scale or offset is broadcast; out has max(scale_len, offset_len) elements.
namespace opsnn {

__device__ __forceinline__ uint32_t scale_to_fp19(uint32_t u, int round_mode)
{
    if (round_mode == 0) return u & 0xFFFFE000u;
    const uint32_t sign = u >> 31;
    uint32_t exponent = (u >> 23) & 0xFFu, mant = (u & 0x7FFFFFu) >> 13;
    const uint32_t round_bit = (u >> 12) & 1u, sticky = u & 0xFFFu;
    uint32_t fp19;
    if (exponent == 0u) fp19 = sign << 18;
    else if (exponent == 255u) fp19 = (sign << 18) | (exponent << 10) | mant;
    else {
        if (round_bit && (sticky || (mant & 1u))) {
            mant += 1u;
            if (mant >= 1024u) { mant = 0u; exponent += 1u; }
        }
        fp19 = (sign << 18) | (exponent << 10) | mant;   // a carry out of exponent 254 gives 255 with mantissa 0: infinity
    }
    return fp19 << 13;
}

__global__ __launch_bounds__(256) void trans_quant_param_kernel(const float* __restrict__ scale, int64_t scale_len,
                                                                const float* __restrict__ offset, int64_t offset_len, int round_mode,
                                                                uint64_t* __restrict__ out, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    uint64_t v = (uint64_t)scale_to_fp19(f2u(scale[scale_len == 1 ? 0 : i]), round_mode) | (1ull << 46);
    if (offset) {
        float o = __builtin_rintf(offset[offset_len == 1 ? 0 : i]);
        o = (o == o) ? fminf(fmaxf(o, -256.0f), 255.0f) : 0.0f;
        v |= ((uint64_t)(int64_t)(int)o & 0x1FFull) << 37;
    }
    out[i] = v;
}

}  // namespace opsnn

extern "C" int opsnnTransQuantParam(const float* scale, int64_t scale_len, const float* offset, int64_t offset_len, int round_mode,
                                    uint64_t* out, void* stream)
{
    if (!scale || !out || scale_len <= 0 || (offset && offset_len <= 0) || (round_mode != 0 && round_mode != 1)) return -1;
    const int64_t n = offset && offset_len > scale_len ? offset_len : scale_len;
    if ((scale_len != 1 && scale_len != n) || (offset && offset_len != 1 && offset_len != n)) return -2;
    hipLaunchKernelGGL(trans_quant_param_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, scale, scale_len,
                       offset, offset ? offset_len : 0, round_mode, out, n);
    return (int)hipGetLastError();
}
