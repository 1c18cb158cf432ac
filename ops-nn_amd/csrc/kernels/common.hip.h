// Shared device helpers for the gfx950 quantized-matmul kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace opsnn {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef unsigned short v4us __attribute__((ext_vector_type(4)));

// Element type codes: the aclDataType values.
enum : int {
    DT_F32 = 0, DT_F16 = 1, DT_I8 = 2, DT_I32 = 3, DT_BF16 = 27, DT_I4 = 29,
    DT_E5M2 = 35, DT_E4M3 = 36, DT_E8M0 = 37, DT_E2M1 = 40, DT_E1M2 = 41, DT_U64 = 10
};

__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }

// fp32 -> bf16 bits, round to nearest even, NaN kept quiet.
__device__ __forceinline__ uint16_t bf16_bits(float f)
{
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
// Element i of the sum, in split order, of `splits` partial arrays of `total` elements each (the K split of the tile
// kernels); four loads in flight at a time.
template <typename T>
__device__ __forceinline__ T splitk_sum(const T* part, int splits, int64_t total, int64_t i)
{
    T v = part[i];
    int s = 1;
    for (; s + 3 < splits; s += 4) {
        const T a = part[(int64_t)s * total + i], b = part[(int64_t)(s + 1) * total + i];
        const T c = part[(int64_t)(s + 2) * total + i], d = part[(int64_t)(s + 3) * total + i];
        v = v + a; v = v + b; v = v + c; v = v + d;
    }
    for (; s < splits; s++) v = v + part[(int64_t)s * total + i];
    return v;
}
// Blocks of 256 threads for a grid-stride loop with one element per thread and pass.
inline unsigned splitk_reduce_grid(int64_t total)
{
    const int64_t want = (total + 255) / 256;
    return (unsigned)(want < 1 ? 1 : want > (1 << 20) ? (1 << 20) : want);
}
__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }
__device__ __forceinline__ uint16_t f16_bits(float f)
{
    _Float16 h = (_Float16)f;  // v_cvt_f16_f32: round to nearest even
    return __builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ float f16_to_f32(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }

// Round an fp32 value to the 16-bit output type and return its bits.
template <int DT>
__device__ __forceinline__ uint16_t to_b16(float f)
{
    if constexpr (DT == DT_BF16) return bf16_bits(f);
    else return f16_bits(f);
}

// Four fp32 values -> four 16-bit floats (round to nearest even) using the packed hardware conversions.
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));
// Two fp32 values -> packed bf16 pair (round to nearest even, v_cvt_pk_bf16_f32); element 0 in the low half.
__device__ __forceinline__ uint32_t pack2_bf16(v2f v)
{
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, v2bf));
}
template <int DT>
__device__ __forceinline__ v4us pack4_b16(v4f v)
{
    if constexpr (DT == DT_BF16) {
        v2f lo = {v[0], v[1]}, hi = {v[2], v[3]};
        v2bf a = __builtin_convertvector(lo, v2bf), b = __builtin_convertvector(hi, v2bf);   // v_cvt_pk_bf16_f32
        uint32_t ua = __builtin_bit_cast(uint32_t, a), ub = __builtin_bit_cast(uint32_t, b);
        v4us o = {(unsigned short)(ua & 0xffffu), (unsigned short)(ua >> 16), (unsigned short)(ub & 0xffffu), (unsigned short)(ub >> 16)};
        return o;
    } else {
        v2f lo = {v[0], v[1]}, hi = {v[2], v[3]};
        v2h a = __builtin_convertvector(lo, v2h), b = __builtin_convertvector(hi, v2h);
        uint32_t ua = __builtin_bit_cast(uint32_t, a), ub = __builtin_bit_cast(uint32_t, b);
        v4us o = {(unsigned short)(ua & 0xffffu), (unsigned short)(ua >> 16), (unsigned short)(ub & 0xffffu), (unsigned short)(ub >> 16)};
        return o;
    }
}

__device__ __forceinline__ float load_scalar_as_f32(const void* p, int dt, int64_t i)
{
    switch (dt) {
        case DT_F32: return ((const float*)p)[i];
        case DT_BF16: return bf16_to_f32(((const uint16_t*)p)[i]);
        case DT_F16: return f16_to_f32(((const uint16_t*)p)[i]);
        case DT_I32: return (float)((const int32_t*)p)[i];
        default: return 0.0f;
    }
}

__device__ __forceinline__ float e4m3_to_f32(uint32_t b)
{
    uint32_t e = (b >> 3) & 0xfu, m = b & 7u;
    float v;
    if (e == 15u && m == 7u) v = u2f(0x7fc00000u);
    else if (e == 0u) v = (float)m * 0.001953125f;
    else v = u2f(((e + 120u) << 23) | (m << 20));
    return (b & 0x80u) ? -v : v;
}
// fp32 -> e4m3fn bits, round to nearest even; NaN and magnitudes that round above 448 give NaN
__device__ __forceinline__ uint32_t f32_to_e4m3_bits(float f)
{
    const uint32_t u = f2u(f), sign = (u >> 24) & 0x80u, a = u & 0x7fffffffu;
    if (a > 0x43e80000u) return sign | 0x7fu;                          // NaN, and anything above 464 (the tie below the absent 480, which alone rounds to 448)
    if (a < 0x3a800000u) return sign;                                  // < 2^-10 rounds to zero
    int exp = (int)(a >> 23) - 127;
    if (exp < -6) exp = -6;                                            // subnormal quantum 2^-9
    const float q = u2f((uint32_t)(exp - 3 + 127) << 23);
    const float qinv = u2f((uint32_t)(127 + 3 - exp) << 23);           // 1 / q: both scalings are exact
    const float v = __fmul_rn(__builtin_rintf(__fmul_rn(u2f(a), qinv)), q);
    if (v < 0.015625f) return sign | (uint32_t)__fmul_rn(v, 512.0f);
    const uint32_t vb = f2u(v);
    return sign | ((((vb >> 23) - 127 + 7) << 3) | ((vb >> 20) & 7u));
}
// fp32 -> e5m2 bits, round to nearest even directly on the fp32 value; overflow gives infinity, NaN stays NaN
__device__ __forceinline__ uint32_t f32_to_e5m2_bits(float f)
{
    const uint32_t u = f2u(f), sign = (u >> 24) & 0x80u, a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return sign | 0x7fu;
    if (a >= 0x47700000u) return sign | 0x7cu;                         // >= 61440: the tie with the absent 65536 goes to infinity
    if (a <= 0x37000000u) return sign;                                 // <= 2^-17 rounds to zero
    int exp = (int)(a >> 23) - 127;
    if (exp < -14) exp = -14;                                          // subnormal quantum 2^-16
    const float q = u2f((uint32_t)(exp - 2 + 127) << 23), qinv = u2f((uint32_t)(127 + 2 - exp) << 23);
    const float v = __fmul_rn(__builtin_rintf(__fmul_rn(u2f(a), qinv)), q);
    if (v < 6.103515625e-05f) return sign | (uint32_t)__fmul_rn(v, 65536.0f);
    const uint32_t vb = f2u(v);
    return sign | ((((vb >> 23) - 127 + 15) << 2) | ((vb >> 21) & 3u));
}
// Two fp32 values -> two fp8 bytes (a in bits 0..7, b in bits 8..15) with the hardware conversion.  For every fp32 of
// either sign up to the format's largest finite value (448 / 57344), zeros and subnormal results included, it returns
// the byte of f32_to_e4m3_bits / f32_to_e5m2_bits (compared exhaustively on the device); callers clamp to that range and
// handle NaN themselves.
template <int Y_DT>
__device__ __forceinline__ uint32_t cvt2_fp8_in_range(float a, float b)
{
    if constexpr (Y_DT == DT_E4M3) return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu;
    else return (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(a, b, 0, false) & 0xffffu;
}
__device__ __forceinline__ float e5m2_to_f32(uint32_t b)
{
    // e5m2 is the upper byte of an IEEE binary16
    return f16_to_f32((uint16_t)(b << 8));
}
__device__ __forceinline__ float e2m1_to_f32(uint32_t c)
{
    uint32_t e = (c >> 1) & 3u, m = c & 1u;
    float v = (e == 0u) ? 0.5f * (float)m : u2f(((e + 126u) << 23) | (m << 22));
    return (c & 8u) ? -v : v;
}
__device__ __forceinline__ float e8m0_to_f32(uint32_t b)
{
    if (b == 0xffu) return u2f(0x7fc00000u);
    if (b == 0u) return u2f(0x00400000u);
    return u2f(b << 23);
}

// Decode element i of a dense buffer of 8-bit or 4-bit quantised values.
__device__ __forceinline__ float load_q_as_f32(const void* p, int dt, int64_t i)
{
    switch (dt) {
        case DT_I8: return (float)((const int8_t*)p)[i];
        case DT_E4M3: return e4m3_to_f32(((const uint8_t*)p)[i]);
        case DT_E5M2: return e5m2_to_f32(((const uint8_t*)p)[i]);
        case DT_I4: {
            uint32_t b = ((const uint8_t*)p)[i >> 1];
            int v = (int)((i & 1) ? (b >> 4) : (b & 15u));
            return (float)(v >= 8 ? v - 16 : v);
        }
        case DT_E2M1: {
            uint32_t b = ((const uint8_t*)p)[i >> 1];
            return e2m1_to_f32((i & 1) ? (b >> 4) : (b & 15u));
        }
        default: return 0.0f;
    }
}

__device__ __forceinline__ void store_f32_as(void* p, int dt, int64_t i, float v)
{
    switch (dt) {
        case DT_F32: ((float*)p)[i] = v; break;
        case DT_BF16: ((uint16_t*)p)[i] = bf16_bits(v); break;
        case DT_F16: ((uint16_t*)p)[i] = f16_bits(v); break;
        default: break;
    }
}

// 16-byte asynchronous copy global -> LDS.  `lds` must be wave-uniform; lane l lands at lds + 16*l.
__device__ __forceinline__ void async_copy16(const void* g, void* lds)
{
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                     (__attribute__((address_space(3))) void*)lds, 16, 0, 0);
}

// The same copy written out.  Through the builtin the compiler's wait-count pass sees an instruction that touches both
// memory paths, and while one is outstanding it answers every dependency on a global load or an LDS read with a wait
// for ALL outstanding operations of that kind (vmcnt(0) / lgkmcnt(0)) -- which empties a prefetch ring of ordinary
// global loads every time a copy is in flight.  Hidden from the pass, those loads are counted exactly; since the
// hardware counter also counts the hidden copies, the computed waits are at worst stricter than needed, never laxer.
// The caller waits for the copies themselves explicitly (wait_vmcnt + barrier before the LDS data is read).
__device__ __forceinline__ void async_copy16_uncounted(const void* g, void* lds)
{
    const uint32_t l = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)lds);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(l), "v"(g) : "memory", "m0");
}

// Asynchronous copies global -> LDS with the address as a wave-uniform 64-bit base in scalar registers plus a 32-bit byte
// offset per lane: the loop spends no vector instruction on addresses.  (Written out: hidden from the compiler's wait-count
// pass, like async_copy16_uncounted; the kernel waits for its copies by count.)  lds: wave-uniform LDS byte address.
// Five wait states stand between whatever precedes the statement and the load: the compiler inserts none for hazards it
// cannot see inside the statement, and a base that a vector instruction (v_readfirstlane) has just written into scalar
// registers needs that many before a memory instruction may read it.
__device__ __forceinline__ void copy16_sbase(const void* base, uint32_t voff, uint32_t lds)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds), "v"(voff), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void copy4_sbase(const void* base, uint32_t voff, uint32_t lds)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tglobal_load_lds_dword %1, %2" : : "s"(lds), "v"(voff), "s"(base) : "memory", "m0");
}

// Workgroup ids are dealt round-robin over the 8 XCDs; give each XCD (own L2) a contiguous
// range of logical tile ids so that neighbouring tiles share operand panels in one L2.
__device__ __forceinline__ uint32_t xcd_remap(uint32_t wg, uint32_t total)
{
    const uint32_t X = 8;
    uint32_t per = total / X, rem = total % X;
    uint32_t xcd = wg % X, idx = wg / X;
    // the first `rem` XCDs own per+1 tiles
    uint32_t base = xcd * per + (xcd < rem ? xcd : rem);
    return base + idx;
}

}  // namespace opsnn
