/*
 * CPU oracle for the quantized-matmul path -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference's numpy golden functions.  Only the
 * test-suite, the smoke check and the benchmark's CPU-baseline leg may link or
 * call this file; the product library never does.
 *
 * Each function cites the golden it follows (paths relative to the reference
 * tree, under matmul/):
 *   G3  = quant_batch_matmul_v3/tests/assets/qbmmv3_kernel_golden.py
 *   GW  = weight_quant_batch_matmul_v2/tests/assets/wqbmmv2_kernel_golden.py
 *   GU  = common/tests/st/arch35/matmul_golden_util.py
 *   GQ  = common/tests/st/arch35/matmul_quant_util.py
 *   G4  = quant_batch_matmul_v4/tests/assets/qbmmv4_kernel_golden.py
 *   GD  = ../quant/dynamic_quant/tests/assets/golden.py
 *
 * Arithmetic conventions shared with the golden: every float operation is a
 * separately rounded fp32 operation (this file is compiled with
 * -ffp-contract=off so the compiler cannot fuse a*b+c), casts to 16-bit types
 * round to nearest even, int8 x int8 accumulates exactly in int32.  The one
 * thing the golden leaves open is the summation order inside np.matmul (BLAS);
 * here it is ascending k.
 *
 * Pinning status (tests/test_oracle_*.py):
 *   codecs ............ pinned (exhaustive tables vs OCP definitions, torch CPU dtypes, reference constants)
 *   orc_qmm_int8_acc .. pinned (brute force, closed forms, identity operands)
 *   orc_qmm_pertoken .. pinned (float64 recomputation, operation-order cases, all-ones example)
 *   orc_qmm_tc ........ pinned (reduces to orc_qmm_pertoken with a constant row scale; hand-computed requant and
 *                       19-bit truncation cases; uint64 packing constants of the reference's utility)
 *   orc_qmm_pertoken_f8 pinned (integer-valued fp8 operands: sums exact in any order, numpy float64/float32
 *                       recomputation; reduces to orc_qmm_tc's double-scale branch when x1Scale is constant and no
 *                       truncation applies)
 *   orc_qmm_perblock .. pinned (reduces to pertoken formula with one K block; power-of-two scales exact; float64)
 *   orc_qmm_mx ........ pinned (power-of-two products are exact: equals integer arithmetic; float64); also serves
 *                       compute_mx of G4 (fp8 x fp4) and, with int8 operands, orc_qmm_perblock serves compute_per_tile
 *   orc_qmm_tcg ....... pinned for in-range values (numpy recomputation with independent codecs; unit scale reduces to
 *                       a plain fp32 matmul); fp32 -> fp8 overflow: parity unpinned (see the function)
 *   orc_qmm_i4_asym ... pinned (numpy int64 / float32 recomputation; zero offset and one group reduce to the
 *                       per-token formula)
 *   orc_wqbmm ......... pinned (hand-computed double-rounding cases; group==K equals per-channel; float64)
 *   orc_convert_weight_b4 pinned (int32 carriers: equals the golden utility's int4 packing orc_pack_int4_to_int32; fp32
 *                       carriers: the 16 fp4 values decode back through orc_e2m1_to_f32, off-table values hand-derived
 *                       from the mask and the table of the cited lines)
 *   orc_dynamic_quant . pinned for rows with a non-zero range (known answers chosen so that division by the type
 *                       maximum instead of multiplication by its reciprocal, round-half-away, or a 16-bit smooth
 *                       product each fail; numpy float32 recomputation; dequantisation error <= scale / 2); a row of
 *                       zeros (symmetric) or a constant row (asymmetric) divides by zero in the golden: parity unpinned,
 *                       this file writes zeros there; with per-expert smooth rows, the rows past the last expert's end (dropped
 *                       by the golden) are left untouched: parity unpinned
 *   orc_dynamic_quant_wide pinned (numpy float32 recomputation of the per-tensor and per-channel goldens; a tensor of one row / a
 *                       batch of one row reduces to orc_dynamic_quant)
 *   orc_dynamic_block_quant pinned (numpy float32 recomputation with torch's fp8 casts; a block with max 448 has scale 1
 *                       and returns x itself through the decimal rounding; min_scale cap and clipping by hand;
 *                       infinities and NaN by the golden's stated rules)
 *   orc_dynamic_mx_quant pinned (the OCP MX definition: shared exponent = floor(log2 max) - emax and round-to-nearest-even
 *                       onto the element grid with saturation, recomputed in numpy with torch's fp8 casts and a brute-force
 *                       nearest-grid-point search for e2m1; known answers for ties, saturation and the scale bytes; dequantised
 *                       values within half a grid step; scale algorithm 1 by its defining property, the smallest power of two
 *                       under which no element saturates; larger blocks by monotonicity against blocks of 32);
 *                       its general form (another axis, fp32 input, e1m2 elements, round / floor / ceil / trunc) by the modes'
 *                       definitions on the explicit e2m1 and e1m2 grids with every tie, by transposition against the
 *                       last-axis form, and by fp32 inputs that are 16-bit values; parity unpinned for fp32 inputs within an
 *                       ulp or two below a power of two, where the golden's float32 log2 rounds up
 *   orc_trans_quant_param pinned (the packing utility of the matmul golden and the reference's system-test formula in numpy;
 *                       its inverse orc_u64_to_deq_scale; hand-derived cases of the rounding mode: ties, carry into the
 *                       exponent, overflow to infinity, subnormal)
 *   hifloat8 .......... not implemented (decoder lives only in an absent third-party package): parity unpinned
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "oracle.h"

#define CLONES __attribute__((target_clones("avx512f", "avx2", "default")))

/* ------------------------------------------------------------------------- */
/* Codecs                                                                     */
/* ------------------------------------------------------------------------- */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* fp32 -> bf16, round to nearest even; NaN stays NaN (quiet). */
uint16_t orc_bf16_from_f32(float f)
{
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
float orc_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* fp32 -> fp16 (IEEE binary16), round to nearest even, gradual underflow, overflow to inf. */
uint16_t orc_f16_from_f32(float f)
{
    uint32_t u = f2u(f);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (a >= 0x47800000u) { /* >= 65536: inf; [65520, 65536) also rounds to inf below */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (a < 0x38800000u) { /* below the smallest normal 2^-14: subnormal result */
        if (a < 0x33000000u) return (uint16_t)sign; /* < 2^-25 rounds to zero (2^-25 itself ties to even = 0) */
        uint32_t e = a >> 23;                 /* biased fp32 exponent, 102..112 */
        uint32_t m = (a & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126u - e;            /* 14..24: value = m * 2^(e-150); half ulp16sub = 2^-24 */
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t r = a + 0xfffu + ((a >> 13) & 1u);
    r = (r - 0x38000000u) >> 13;
    if (r >= 0x7c00u) r = 0x7c00u;
    return (uint16_t)(sign | r);
}
float orc_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    if (e == 0) {
        if (m == 0) return u2f(sign);
        float v = (float)m * 5.9604644775390625e-08f; /* 2^-24 */
        return sign ? -v : v;
    }
    if (e == 31) return u2f(sign | 0x7f800000u | (m << 13));
    return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

/* OCP FP8 E4M3 (fn): bias 7, no inf, NaN = S.1111.111, max 448. */
float orc_e4m3_to_f32(uint8_t b)
{
    uint32_t e = (b >> 3) & 0xfu, m = b & 7u;
    float v;
    if (e == 15 && m == 7) return u2f(0x7fc00000u | ((uint32_t)(b & 0x80u) << 24));
    if (e == 0) v = (float)m * 0.001953125f; /* 2^-9 */
    else v = ldexpf((float)(8 + m), (int)e - 10);
    return (b & 0x80u) ? -v : v;
}
/* OCP FP8 E5M2: bias 15, IEEE-like inf/NaN. */
float orc_e5m2_to_f32(uint8_t b)
{
    uint32_t e = (b >> 2) & 0x1fu, m = b & 3u;
    float v;
    if (e == 31) return u2f(((uint32_t)(b & 0x80u) << 24) | 0x7f800000u | (m ? 0x400000u : 0u));
    if (e == 0) v = (float)m * 1.52587890625e-05f; /* 2^-16 */
    else v = ldexpf((float)(4 + m), (int)e - 17);
    return (b & 0x80u) ? -v : v;
}
/* fp32 -> e4m3fn, round to nearest even; NaN and magnitudes that round above 448 (anything above the tie 464) give NaN
 * (0x7f): the format has no infinity and the cast does not saturate -- the behaviour of torch.float8_e4m3fn, against which
 * tests/test_oracle_pins.py compares this function over the whole fp32 range. */
uint8_t orc_e4m3_from_f32(float f)
{
    uint32_t u = f2u(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    float a = fabsf(f);
    if (!(a == a)) return (uint8_t)(sign | 0x7f);
    if (a > 464.0f) return (uint8_t)(sign | 0x7f);  /* 464 is the tie between 448 and the absent 480: it alone stays 448 */
    if (a < 0.0009765625f) return sign;              /* < 2^-10 -> 0 (tie at 2^-10 goes to even = 0) */
    int e;
    (void)frexpf(a, &e);                             /* a = fr * 2^e, fr in [0.5,1) */
    int exp = e - 1;                                 /* a in [2^exp, 2^(exp+1)) */
    if (exp < -6) exp = -6;                          /* subnormal quantum 2^-9 */
    float q = ldexpf(1.0f, exp - 3);
    float n = a / q;                                 /* exact: power-of-two division */
    float r = nearbyintf(n);                         /* default rounding mode = nearest even */
    float v = r * q;
    /* encode v */
    if (v < 0.015625f) return (uint8_t)(sign | (uint8_t)(v * 512.0f));
    int e2;
    float fr = frexpf(v, &e2);
    uint32_t mant = (uint32_t)(fr * 16.0f) - 8u;
    return (uint8_t)(sign | (uint8_t)(((e2 - 1 + 7) << 3) | mant));
}

/* fp32 -> e5m2, round to nearest even; overflow to infinity, NaN stays NaN.  e5m2 is binary16 cut to two mantissa
 * bits, so the rounding is done directly on the fp32 value (not through binary16, which would round twice). */
uint8_t orc_e5m2_from_f32(float f)
{
    uint32_t u = f2u(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    float a = fabsf(f);
    if (!(a == a)) return (uint8_t)(sign | 0x7f);
    if (a >= 61440.0f) return (uint8_t)(sign | 0x7c);  /* the tie between 57344 and the absent 65536 goes to even = infinity */
    if (a <= 7.62939453125e-06f) return sign;          /* <= 2^-17: the tie with the smallest subnormal 2^-16 goes to 0 */
    int e;
    (void)frexpf(a, &e);
    int exp = e - 1;
    if (exp < -14) exp = -14;                          /* subnormal quantum 2^-16 */
    float q = ldexpf(1.0f, exp - 2);
    float v = nearbyintf(a / q) * q;
    if (v < 6.103515625e-05f) return (uint8_t)(sign | (uint8_t)(v * 65536.0f));
    int e2;
    float fr = frexpf(v, &e2);
    uint32_t mant = (uint32_t)(fr * 8.0f) - 4u;
    return (uint8_t)(sign | (uint8_t)(((e2 - 1 + 15) << 2) | mant));
}

/* FP4 E2M1 value table (GQ:329-346): codes 0..7 = {0,.5,1,1.5,2,3,4,6}, bit 3 = sign. */
static const float kE2M1[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};
float orc_e2m1_to_f32(uint8_t code) { return kE2M1[code & 15u]; }
/* E8M0: 2^(b-127); 0xFF = NaN. */
float orc_e8m0_to_f32(uint8_t b)
{
    if (b == 0xffu) return u2f(0x7fc00000u);
    if (b == 0) return u2f(0x00400000u); /* 2^-127, an fp32 subnormal */
    return u2f((uint32_t)b << 23);
}

void orc_vec_f32_to_bf16(const float* in, uint16_t* out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = orc_bf16_from_f32(in[i]); }
void orc_vec_bf16_to_f32(const uint16_t* in, float* out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = orc_bf16_to_f32(in[i]); }
void orc_vec_f32_to_f16(const float* in, uint16_t* out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = orc_f16_from_f32(in[i]); }
void orc_vec_f16_to_f32(const uint16_t* in, float* out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = orc_f16_to_f32(in[i]); }
void orc_vec_f32_to_e4m3(const float* in, uint8_t* out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = orc_e4m3_from_f32(in[i]); }
void orc_vec_e4m3_to_f32(const uint8_t* in, float* out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = orc_e4m3_to_f32(in[i]); }
void orc_vec_e5m2_to_f32(const uint8_t* in, float* out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = orc_e5m2_to_f32(in[i]); }
void orc_vec_e8m0_to_f32(const uint8_t* in, float* out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = orc_e8m0_to_f32(in[i]); }

/* groupSize = gsK | gsN << 16 | gsM << 32, zero fields read as 1 (GQ:179-191). */
void orc_unpack_groupsize(int64_t gs, int64_t* gsM, int64_t* gsN, int64_t* gsK)
{
    *gsM = (gs >> 32) & 0xffff; *gsN = (gs >> 16) & 0xffff; *gsK = gs & 0xffff;
    if (*gsM == 0) *gsM = 1;
    if (*gsN == 0) *gsN = 1;
    if (*gsK == 0) *gsK = 1;
}

/* Eight int4 values per int32, element i in bits 4i..4i+3 (GQ:228-273, 349-394). */
void orc_pack_int4_to_int32(const int8_t* in, int32_t* out, size_t n_packed)
{
    for (size_t i = 0; i < n_packed; i++) {
        uint32_t w = 0;
        for (int j = 0; j < 8; j++) w |= ((uint32_t)in[i * 8 + j] & 0xfu) << (4 * j);
        out[i] = (int32_t)w;
    }
}
/* aclnnConvertWeightToINT4Pack's host loop (convert_weight_to_int4_pack/op_host/op_api/
 * aclnn_convert_weight_to_int4_pack.cpp:79-126): one 4-bit value per 32-bit carrier element, packed two per byte with
 * the even element in the low nibble.  int32 carrier: the low four bits.  fp32 carrier: the bits are cut to sign,
 * exponent and first mantissa bit (mask 0xFFC00000) and looked up in the table of the 16 fp4 e2m1 values (:43-63); a
 * pattern that is not in the table gives code 0, sign included. */
static uint32_t convert_fp32_bits_to_e2m1(uint32_t bits)
{
    static const uint32_t mag_bits[8] = {0x00000000u, 0x3F000000u, 0x3F800000u, 0x3FC00000u,
                                         0x40000000u, 0x40400000u, 0x40800000u, 0x40C00000u};
    const uint32_t cut = bits & 0xFFC00000u;
    for (uint32_t c = 0; c < 8; c++) {
        if (cut == mag_bits[c]) return c;
        if (cut == (mag_bits[c] | 0x80000000u)) return c | 8u;
    }
    return 0u;
}
void orc_convert_weight_b4(const int32_t* w, int64_t count, int is_fp32, uint8_t* out)
{
    for (int64_t i = 0; i + 1 < count; i += 2) {
        uint32_t a = (uint32_t)w[i], b = (uint32_t)w[i + 1];
        if (is_fp32) { a = convert_fp32_bits_to_e2m1(a); b = convert_fp32_bits_to_e2m1(b); }
        out[i / 2] = (uint8_t)(((b & 0xFu) << 4) | (a & 0xFu));
    }
}
void orc_unpack_int32_to_int4(const int32_t* in, int8_t* out, size_t n_packed)
{
    for (size_t i = 0; i < n_packed; i++) {
        uint32_t w = (uint32_t)in[i];
        for (int j = 0; j < 8; j++) {
            int v = (int)((w >> (4 * j)) & 0xfu);
            out[i * 8 + j] = (int8_t)(v >= 8 ? v - 16 : v);
        }
    }
}

static size_t dtype_bits(int dt)
{
    switch (dt) {
        case ORC_F32: case ORC_I32: return 32;
        case ORC_F16: case ORC_BF16: return 16;
        case ORC_I8: case ORC_E4M3: case ORC_E5M2: case ORC_E8M0: return 8;
        case ORC_I4: case ORC_E2M1: return 4;
        default: return 0;
    }
}

/* Decode element i of a dense buffer to fp32 (every supported type converts exactly). */
static inline float load_as_f32(const void* p, int dt, size_t i)
{
    switch (dt) {
        case ORC_F32: return ((const float*)p)[i];
        case ORC_I32: return (float)((const int32_t*)p)[i];
        case ORC_F16: return orc_f16_to_f32(((const uint16_t*)p)[i]);
        case ORC_BF16: return orc_bf16_to_f32(((const uint16_t*)p)[i]);
        case ORC_I8: return (float)((const int8_t*)p)[i];
        case ORC_E4M3: return orc_e4m3_to_f32(((const uint8_t*)p)[i]);
        case ORC_E5M2: return orc_e5m2_to_f32(((const uint8_t*)p)[i]);
        case ORC_E8M0: return orc_e8m0_to_f32(((const uint8_t*)p)[i]);
        case ORC_I4: {
            uint8_t b = ((const uint8_t*)p)[i >> 1];
            int v = (i & 1) ? (b >> 4) : (b & 15);
            return (float)(v >= 8 ? v - 16 : v);
        }
        case ORC_E2M1: {
            uint8_t b = ((const uint8_t*)p)[i >> 1];
            return kE2M1[(i & 1) ? (b >> 4) : (b & 15)];
        }
        default: return NAN;
    }
}

/* cast_output_dtype (GU:68-73): fp32 -> y dtype, RNE. */
static inline void store_from_f32(void* p, int dt, size_t i, float v)
{
    switch (dt) {
        case ORC_F32: ((float*)p)[i] = v; break;
        case ORC_F16: ((uint16_t*)p)[i] = orc_f16_from_f32(v); break;
        case ORC_BF16: ((uint16_t*)p)[i] = orc_bf16_from_f32(v); break;
        default: break;
    }
}

/* Storage [rows, cols] (row-major, sub-byte types packed along cols) -> fp32 [R, C]
 * where (R, C) = (cols, rows) if transpose else (rows, cols). */
static float* decode_matrix(const void* src, int dt, int64_t rows, int64_t cols, int transpose)
{
    float* dst = (float*)malloc(sizeof(float) * (size_t)rows * (size_t)cols);
    if (!dst) return NULL;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < cols; c++) {
            float v = load_as_f32(src, dt, (size_t)(r * cols + c));
            if (transpose) dst[c * rows + r] = v; else dst[r * cols + c] = v;
        }
    return dst;
}

/* ------------------------------------------------------------------------- */
/* Contractions                                                               */
/* ------------------------------------------------------------------------- */

/* C[M,N] (+)= A[M,K(lda)] @ B[K,N(ldb)], fp32, ascending k, product and sum rounded separately. */
CLONES static void sgemm_tile(const float* A, int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                              int64_t m0, int64_t m1, int64_t n0, int64_t n1, int64_t K)
{
    for (int64_t m = m0; m < m1; m++) {
        float* c = C + m * ldc;
        for (int64_t k = 0; k < K; k++) {
            float a = A[m * lda + k];
            const float* b = B + k * ldb;
            for (int64_t n = n0; n < n1; n++) c[n] = c[n] + a * b[n];
        }
    }
}

static void sgemm_acc(const float* A, int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc, int64_t M,
                      int64_t N, int64_t K)
{
    const int64_t TM = 8, TN = 512;
    int64_t mt = (M + TM - 1) / TM, nt = (N + TN - 1) / TN;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t i = 0; i < mt; i++)
        for (int64_t j = 0; j < nt; j++) {
            int64_t m1 = (i + 1) * TM < M ? (i + 1) * TM : M;
            int64_t n1 = (j + 1) * TN < N ? (j + 1) * TN : N;
            sgemm_tile(A, lda, B, ldb, C, ldc, i * TM, m1, j * TN, n1, K);
        }
}

CLONES static void igemm_tile(const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb, int32_t* C, int64_t ldc,
                              int64_t m0, int64_t m1, int64_t n0, int64_t n1, int64_t K)
{
    for (int64_t m = m0; m < m1; m++) {
        int32_t* c = C + m * ldc;
        for (int64_t k = 0; k < K; k++) {
            int32_t a = A[m * lda + k];
            const int8_t* b = B + k * ldb;
            for (int64_t n = n0; n < n1; n++) c[n] += a * (int32_t)b[n];
        }
    }
}

/*
 * acc[M,N] = int32(x1) @ int32(x2)   (G3:614-634: both operands widened to int32, np.matmul).
 * x1 storage is [M,K] (or [K,M] if tA), x2 storage is [K,N] (or [N,K] if tB), int8.
 */
int orc_qmm_int8_acc(const int8_t* x1, const int8_t* x2, int64_t M, int64_t K, int64_t N, int tA, int tB,
                     int32_t* acc)
{
    int8_t* a = (int8_t*)x1;
    int8_t* b = (int8_t*)x2;
    if (tA) {
        a = (int8_t*)malloc((size_t)M * K);
        if (!a) return -1;
        for (int64_t k = 0; k < K; k++) for (int64_t m = 0; m < M; m++) a[m * K + k] = x1[k * M + m];
    }
    if (tB) {
        b = (int8_t*)malloc((size_t)N * K);
        if (!b) return -1;
#pragma omp parallel for schedule(static)
        for (int64_t n = 0; n < N; n++) for (int64_t k = 0; k < K; k++) b[k * N + n] = x2[n * K + k];
    }
    memset(acc, 0, sizeof(int32_t) * (size_t)M * N);
    const int64_t TM = 8, TN = 1024;
    int64_t mt = (M + TM - 1) / TM, nt = (N + TN - 1) / TN;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t i = 0; i < mt; i++)
        for (int64_t j = 0; j < nt; j++) {
            int64_t m1 = (i + 1) * TM < M ? (i + 1) * TM : M;
            int64_t n1 = (j + 1) * TN < N ? (j + 1) * TN : N;
            igemm_tile(a, K, b, N, acc, N, i * TM, m1, j * TN, n1, K);
        }
    if (tA) free(a);
    if (tB) free(b);
    return 0;
}

/*
 * compute_pertoken (G3:361-387), K-C / K-T modes.
 *   out = acc (+ int32 bias, integer domain)
 *   out = fp32(out) * x2Scale[n] * x1Scale[m]        -- evaluated left to right
 *   out = out + fp32(bias) for a float bias           -- after scaling (both golden branches agree)
 *   y   = cast(out)
 * x2s_len is 1 (K-T) or N (K-C).  x1s may be NULL (then treated as absent: T-C dynamic path of
 * compute_tc G3:390-475 without scale truncation, i.e. bf16/fp32 scale with float bias).
 */
int orc_qmm_pertoken_epilogue(const int32_t* acc, int64_t M, int64_t N, const float* x1s, const float* x2s,
                              int64_t x2s_len, const void* bias, int bias_dt, int y_dt, void* y)
{
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            int32_t a = acc[m * N + n];
            if (bias && bias_dt == ORC_I32) a += ((const int32_t*)bias)[n];
            float o = (float)a;
            o = o * x2s[x2s_len == 1 ? 0 : n];
            if (x1s) o = o * x1s[m];
            if (bias && bias_dt != ORC_I32) o = o + load_as_f32(bias, bias_dt, (size_t)n);
            store_from_f32(y, y_dt, (size_t)(m * N + n), o);
        }
    return 0;
}

int orc_qmm_pertoken(const int8_t* x1, const int8_t* x2, int64_t M, int64_t K, int64_t N, int tA, int tB,
                     const float* x1s, const float* x2s, int64_t x2s_len, const void* bias, int bias_dt, int y_dt,
                     void* y, int32_t* acc_out)
{
    int32_t* acc = acc_out ? acc_out : (int32_t*)malloc(sizeof(int32_t) * (size_t)M * N);
    if (!acc) return -1;
    int rc = orc_qmm_int8_acc(x1, x2, M, K, N, tA, tB, acc);
    if (rc == 0) rc = orc_qmm_pertoken_epilogue(acc, M, N, x1s, x2s, x2s_len, bias, bias_dt, y_dt, y);
    if (!acc_out) free(acc);
    return rc;
}

/*
 * compute_tc / compute_requant / compute_int32 (G3:390-506): the T-T / T-C family, one batch slice, with
 *   the mode rules of determine_quant_mode (G3:62-145): a one-element per-token scale with fp8 inputs is the
 *     "doublescale" form -- merged and truncated when x2Scale has one element too (T-T), multiplied separately
 *     when it has N (T-C);
 *   needs_scale_generate (GQ:62-72): int inputs, a one-element scale and a bias that is neither bf16 nor fp32 ->
 *     the scale keeps its upper 19 bits;
 *   is_bias_vec (G3:574-581): a float bias is added after the scaling for int inputs, and for fp8 inputs when a
 *     per-token scale is present; otherwise before it (an int32 bias is added to the int32 sums);
 *   the uint64 decoding of the aclnn-level golden (matmul/quant_batch_matmul_v4/tests/assets/
 *     qbmmv4_aclnn_golden.py:276-316): scale = fp32 from the low word with the upper 19 bits kept, offset =
 *     the x2Offset tensor if there is one, else the signed 9-bit field at bits 37..45.
 * scale_dt: ORC_F32, ORC_BF16 or ORC_U64.  y_dt ORC_I8 -> requant, ORC_I32 -> integer sums, else cast of the scaled sum.
 */
static float s9(float v)   /* f32_2_s9 (GQ:57-59): round half to even, clip to [-256, 255] */
{
    float r = rintf(v);
    return r < -256.0f ? -256.0f : (r > 255.0f ? 255.0f : r);
}

int orc_qmm_tc(const void* x1, const void* x2, int dt1, int dt2, int64_t M, int64_t K, int64_t N, int tA, int tB,
               const void* scale, int scale_dt, int64_t scale_len, const float* pertoken, const float* offset,
               int64_t offset_len, const void* bias, int bias_dt, int y_dt, void* y)
{
    const int is_int = dt1 == ORC_I8 || dt1 == ORC_I4;
    const int bias_float = bias && bias_dt != ORC_I32;
    float* sc = (float*)malloc(sizeof(float) * (size_t)scale_len);
    float* dec_off = NULL;
    if (!sc) return -1;
    for (int64_t i = 0; i < scale_len; i++) {
        if (scale_dt == ORC_U64) sc[i] = orc_u64_to_deq_scale(((const uint64_t*)scale)[i]);
        else sc[i] = load_as_f32(scale, scale_dt, (size_t)i);
    }
    if (y_dt == ORC_I8 && !offset && scale_dt == ORC_U64) {
        dec_off = (float*)malloc(sizeof(float) * (size_t)scale_len);
        if (!dec_off) return -1;
        for (int64_t i = 0; i < scale_len; i++) {
            int64_t raw = (int64_t)((((const uint64_t*)scale)[i] >> 37) & 0x1FF);
            if (raw & 0x100) raw -= 0x200;
            dec_off[i] = (float)raw;
        }
        offset = dec_off; offset_len = scale_len;
    }
    int32_t* iacc = NULL;
    float* facc = NULL;
    if (is_int) {
        iacc = (int32_t*)malloc(sizeof(int32_t) * (size_t)M * N);
        if (!iacc || orc_qmm_int8_acc((const int8_t*)x1, (const int8_t*)x2, M, K, N, tA, tB, iacc) != 0) return -1;
    } else {
        float* a = tA ? decode_matrix(x1, dt1, K, M, 1) : decode_matrix(x1, dt1, M, K, 0);
        float* b = tB ? decode_matrix(x2, dt2, N, K, 1) : decode_matrix(x2, dt2, K, N, 0);
        facc = (float*)calloc((size_t)M * N, sizeof(float));
        if (!a || !b || !facc) return -1;
        sgemm_acc(a, K, b, N, facc, N, M, N, K);
        free(a); free(b);
    }
    const int do_scale_gen = is_int && scale_len == 1 && !(bias && (bias_dt == ORC_BF16 || bias_dt == ORC_F32));
    const int is_bias_vec = bias_float && (is_int || pertoken != NULL);
    const int merge_trunc = pertoken != NULL && scale_len == 1;   /* T-T-doublescale */
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            const size_t i = (size_t)(m * N + n);
            const float s = sc[scale_len == 1 ? 0 : n];
            if (y_dt == ORC_I8) {            /* compute_requant (G3:478-496) */
                int32_t a = iacc[i];
                if (bias && bias_dt == ORC_I32) a += ((const int32_t*)bias)[n];
                float o = s9((float)a * s);
                if (offset) o = s9(o) + s9(offset[offset_len == 1 ? 0 : n]);
                o = o < -128.0f ? -128.0f : (o > 127.0f ? 127.0f : o);
                ((int8_t*)y)[i] = (int8_t)o;
                continue;
            }
            if (y_dt == ORC_I32) {           /* compute_int32 (G3:499-513) */
                int32_t a = iacc[i];
                if (bias && bias_dt == ORC_I32) ((int32_t*)y)[i] = a + ((const int32_t*)bias)[n];
                else if (bias) ((int32_t*)y)[i] = (int32_t)((float)a + load_as_f32(bias, bias_dt, (size_t)n));
                else ((int32_t*)y)[i] = a;
                continue;
            }
            float o;                         /* compute_tc (G3:390-475) */
            if (is_int) {
                int32_t a = iacc[i];
                if (!is_bias_vec && bias && bias_dt == ORC_I32) a += ((const int32_t*)bias)[n];
                o = (float)a;
            } else {
                o = facc[i];
            }
            if (!is_bias_vec && bias_float) o = o + load_as_f32(bias, bias_dt, (size_t)n);
            if (pertoken) {
                if (merge_trunc && !is_bias_vec) {
                    o = o * orc_scale_generate(s * pertoken[0]);
                } else {
                    const float s2 = do_scale_gen ? orc_scale_generate(s) : s;
                    o = o * s2;
                    o = o * pertoken[0];
                }
            } else {
                o = o * (do_scale_gen ? orc_scale_generate(s) : s);
            }
            if (is_bias_vec) o = o + load_as_f32(bias, bias_dt, (size_t)n);
            store_from_f32(y, y_dt, i, o);
        }
    free(sc); free(dec_off); free(iacc); free(facc);
    return 0;
}

/*
 * K-C / K-T with fp8 operands (G3:612-634 + compute_pertoken, G3:361-387): the matmul is done in fp32 on the decoded
 * operands, then  y = (acc * x2Scale[n]) * x1Scale[m];  + fp32 bias;  cast.  No truncation of either scale, no
 * integer bias (the checker admits FLOAT bias only for fp8 operands).
 */
int orc_qmm_pertoken_f8(const void* x1, const void* x2, int dt1, int dt2, int64_t M, int64_t K, int64_t N, int tA, int tB,
                        const float* x1s, const float* x2s, int64_t x2s_len, const float* bias, int y_dt, void* y)
{
    float* a = tA ? decode_matrix(x1, dt1, K, M, 1) : decode_matrix(x1, dt1, M, K, 0);
    float* b = tB ? decode_matrix(x2, dt2, N, K, 1) : decode_matrix(x2, dt2, K, N, 0);
    float* acc = (float*)calloc((size_t)M * N, sizeof(float));
    if (!a || !b || !acc) return -1;
    sgemm_acc(a, K, b, N, acc, N, M, N, K);
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            float o = acc[m * N + n];
            o = o * x2s[x2s_len == 1 ? 0 : n];
            o = o * x1s[m];
            if (bias) o = o + bias[n];
            store_from_f32(y, y_dt, (size_t)(m * N + n), o);
        }
    free(a); free(b); free(acc);
    return 0;
}

/*
 * compute_perblock (G3:237-358), G-B / B-B modes, one batch slice.
 *   for kb in range(ceil(K/gsK)):
 *       y += (fp32(x1[:, kb]) @ fp32(x2[kb, :])) * (x1Scale[m/gsM, kb] * x2Scale[kb, n/gsN])
 *   y (+ fp32 bias);  cast
 * Scale storage follows the operand's transposition (G3:276-286): x1s is [ceil(M/gsM), KB]
 * (or [KB, ceil(M/gsM)] if tA); x2s is [KB, ceil(N/gsN)] (or [ceil(N/gsN), KB] if tB).
 */
int orc_qmm_perblock(const void* x1, const void* x2, int dt1, int dt2, int64_t M, int64_t K, int64_t N, int tA,
                     int tB, const float* x1s, const float* x2s, int64_t gsM, int64_t gsN, int64_t gsK,
                     const float* bias, int y_dt, void* y)
{
    float* a = tA ? decode_matrix(x1, dt1, K, M, 1) : decode_matrix(x1, dt1, M, K, 0);
    float* b = tB ? decode_matrix(x2, dt2, N, K, 1) : decode_matrix(x2, dt2, K, N, 0);
    float* acc = (float*)calloc((size_t)M * N, sizeof(float));
    float* part = (float*)malloc(sizeof(float) * (size_t)M * N);
    if (!a || !b || !acc || !part) return -1;
    int64_t KB = (K + gsK - 1) / gsK, MB = (M + gsM - 1) / gsM, NB = (N + gsN - 1) / gsN;
    for (int64_t kb = 0; kb < KB; kb++) {
        int64_t k0 = kb * gsK, k1 = (kb + 1) * gsK < K ? (kb + 1) * gsK : K;
        memset(part, 0, sizeof(float) * (size_t)M * N);
        sgemm_acc(a + k0, K, b + k0 * N, N, part, N, M, N, k1 - k0);
#pragma omp parallel for schedule(static)
        for (int64_t m = 0; m < M; m++) {
            float s1 = tA ? x1s[kb * MB + m / gsM] : x1s[(m / gsM) * KB + kb];
            for (int64_t n = 0; n < N; n++) {
                float s2 = tB ? x2s[(n / gsN) * KB + kb] : x2s[kb * NB + n / gsN];
                float sc = s1 * s2;
                acc[m * N + n] = acc[m * N + n] + part[m * N + n] * sc;
            }
        }
    }
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            float o = acc[m * N + n];
            if (bias) o = o + bias[n];
            store_from_f32(y, y_dt, (size_t)(m * N + n), o);
        }
    free(a); free(b); free(acc); free(part);
    return 0;
}

/*
 * compute_mx (G3:153-234), MX (G-G) mode, one batch slice.
 *   x1f = fp32(x1) * repeat32(x1Scale),  x2f = fp32(x2) * repeat32(x2Scale)   (K zero-padded to the scale extent)
 *   y = x1f @ x2f (+ fp32 bias);  cast
 * Scale storage (e8m0 bytes): x1s [M, KS, 2] (or [KS, M, 2] if tA); x2s [KS, N, 2] (or [N, KS, 2] if tB),
 * KS = ceil(K/64); the scale for 32-wide K block kb is entry [.., kb/2, .., kb%2] (G3:171-197).
 * If ceil(K/32) is odd the last (pad) scale is dropped (G3:199-202).
 */
int orc_qmm_mx(const void* x1, const void* x2, int dt1, int dt2, int64_t M, int64_t K, int64_t N, int tA, int tB,
               const uint8_t* x1s, const uint8_t* x2s, const float* bias, int y_dt, void* y)
{
    float* a = tA ? decode_matrix(x1, dt1, K, M, 1) : decode_matrix(x1, dt1, M, K, 0);
    float* b = tB ? decode_matrix(x2, dt2, N, K, 1) : decode_matrix(x2, dt2, K, N, 0);
    float* acc = (float*)calloc((size_t)M * N, sizeof(float));
    if (!a || !b || !acc) return -1;
    int64_t KS = (K + 63) / 64;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; m++)
        for (int64_t k = 0; k < K; k++) {
            int64_t kb = k / 32;
            uint8_t s = tA ? x1s[((kb / 2) * M + m) * 2 + (kb & 1)] : x1s[(m * KS + kb / 2) * 2 + (kb & 1)];
            a[m * K + k] = a[m * K + k] * orc_e8m0_to_f32(s);
        }
#pragma omp parallel for schedule(static)
    for (int64_t k = 0; k < K; k++)
        for (int64_t n = 0; n < N; n++) {
            int64_t kb = k / 32;
            uint8_t s = tB ? x2s[(n * KS + kb / 2) * 2 + (kb & 1)] : x2s[((kb / 2) * N + n) * 2 + (kb & 1)];
            b[k * N + n] = b[k * N + n] * orc_e8m0_to_f32(s);
        }
    sgemm_acc(a, K, b, N, acc, N, M, N, K);
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            float o = acc[m * N + n];
            if (bias) o = o + bias[n];
            store_from_f32(y, y_dt, (size_t)(m * N + n), o);
        }
    free(a); free(b); free(acc);
    return 0;
}

/* truncate (GU:235-239): round an fp32 value through the intermediate 16-bit type. */
static inline float trunc_to(float v, int dt)
{
    if (dt == ORC_F16) return orc_f16_to_f32(orc_f16_from_f32(v));
    if (dt == ORC_BF16) return orc_bf16_to_f32(orc_bf16_from_f32(v));
    return v;
}

/*
 * compute_t_cg (G4:189-255): fp8 x1, fp4 x2 with a 16-bit scale per `gs` K elements, 64-bit packed output scale.
 *   w[k,n] = fp32( T8( fp32( T16( T16(x2[k,n]) * x2Scale[k/gs, n] ) ) ) )     T16 = the scale's dtype, T8 = x1's dtype
 *   y = (fp32(x1) @ w) * deq(yScale[n]) (+ fp32 bias);  cast            deq = u64_to_deq_scale (GQ:129-135)
 * x2 storage: [K, N] packed along N, or [N, K] packed along K if tB; x2Scale storage [K/gs, N], or [N, K/gs] if tB.
 * Only x1 = e4m3 is implemented.  fp32 -> e4m3 follows orc_e4m3_from_f32 (magnitudes that round above 448 give
 * NaN); the golden delegates that cast to a third-party package that is not available here, so its overflow
 * behaviour is parity unpinned -- in-range values are pinned by the exhaustive codec tables.
 */
int orc_qmm_tcg(const uint8_t* x1, const uint8_t* x2, int64_t M, int64_t K, int64_t N, int tB, const uint16_t* x2s,
                int s_dt, int64_t gs, const uint64_t* yscale, int64_t ylen, const float* bias, int y_dt, void* y)
{
    float* a = decode_matrix(x1, ORC_E4M3, M, K, 0);
    float* b = tB ? decode_matrix(x2, ORC_E2M1, N, K, 1) : decode_matrix(x2, ORC_E2M1, K, N, 0);
    float* acc = (float*)calloc((size_t)M * N, sizeof(float));
    if (!a || !b || !acc) return -1;
    const int64_t G = (K + gs - 1) / gs;
#pragma omp parallel for schedule(static)
    for (int64_t k = 0; k < K; k++)
        for (int64_t n = 0; n < N; n++) {
            const int64_t g = k / gs;
            const float sc = load_as_f32(x2s, s_dt, (size_t)(tB ? n * G + g : g * N + n));
            const float mid = trunc_to(trunc_to(b[k * N + n], s_dt) * sc, s_dt);
            b[k * N + n] = orc_e4m3_to_f32(orc_e4m3_from_f32(mid));
        }
    sgemm_acc(a, K, b, N, acc, N, M, N, K);
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            float o = acc[m * N + n];
            if (yscale) o = o * orc_u64_to_deq_scale(yscale[ylen == 1 ? 0 : n]);
            if (bias) o = o + bias[n];
            store_from_f32(y, y_dt, (size_t)(m * N + n), o);
        }
    free(a); free(b); free(acc);
    return 0;
}

/*
 * compute_int4_asymmetrical (G4:328-395): int4 x int4, one fp32 scale and one fp16 offset per 256 K elements and
 * column, one fp32 scale per row.
 *   acc[m,n] = sum_g ( fp32(sum_{k in g} x1*x2) - fp32(sum_{k in g} x1) * fp32(x2Offset[g,n]) ) * x2Scale[g,n]
 *   y = acc * x1Scale[m];  cast
 * x1 storage [M, K] packed along K; x2 storage [K, N] packed along N, or [N, K] packed along K if tB;
 * x2Scale / x2Offset storage [ceil(K/256), N] either way.  The integer sums are exact.
 */
int orc_qmm_i4_asym(const uint8_t* x1, const uint8_t* x2, int64_t M, int64_t K, int64_t N, int tB, const float* x1s,
                    const float* x2s, const uint16_t* x2o, int y_dt, void* y)
{
    const int64_t GK = 256, G = (K + GK - 1) / GK;
    float* a = decode_matrix(x1, ORC_I4, M, K, 0);
    float* b = tB ? decode_matrix(x2, ORC_I4, N, K, 1) : decode_matrix(x2, ORC_I4, K, N, 0);
    if (!a || !b) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            float out = 0.0f;
            for (int64_t g = 0; g < G; g++) {
                const int64_t k0 = g * GK, k1 = (g + 1) * GK < K ? (g + 1) * GK : K;
                int32_t mm = 0, rs = 0;
                for (int64_t k = k0; k < k1; k++) {
                    mm += (int32_t)a[m * K + k] * (int32_t)b[k * N + n];
                    rs += (int32_t)a[m * K + k];
                }
                const float off = (float)rs * orc_f16_to_f32(x2o[g * N + n]);
                out = out + ((float)mm - off) * x2s[g * N + n];
            }
            store_from_f32(y, y_dt, (size_t)(m * N + n), out * x1s[m]);
        }
    free(a); free(b);
    return 0;
}

/*
 * wqbmm_kernel_compute (GW:106-196) for the T / C / G / MX antiquant modes.
 *   per-tensor / per-channel (_compute_tc, GW:199-239) and per-group (_compute_pergroup, GW:242-297):
 *       w = T(T(w + offset) * scale)      with offset
 *       w = T(w * scale)                  without offset            T = round through x's dtype
 *   MX (_compute_mx, GW:300-352): w = T(fp4 * T16(2^e)) per 32 K (the scale is first rounded through
 *       fp16 when x is fp16)
 *   y = fp32(x) @ w  (+ fp32(bias));  if x is bf16 round through bf16;  cast to x's dtype
 *   (matmul_and_finalize / finalize, GW:85-103).
 *
 * weight storage: [K, N] (or [N, K] if tW), sub-byte packed along the storage's last axis.
 * scale/offset storage: [G, N] (or [N, G] if tW) with G = 1 or ceil(K/group); a scale with
 * scale_n == 1 is per-tensor.  scale_dt is x's dtype or ORC_E8M0.
 */
int orc_wqbmm(const void* x, int x_dt, const void* w, int w_dt, int64_t M, int64_t K, int64_t N, int tW,
              const void* scale, int scale_dt, int64_t scale_n, const void* offset, int64_t group,
              const void* bias, int bias_dt, void* y)
{
    int inter = x_dt;
    float* xf = decode_matrix(x, x_dt, M, K, 0);
    float* wf = tW ? decode_matrix(w, w_dt, N, K, 1) : decode_matrix(w, w_dt, K, N, 0);
    float* acc = (float*)calloc((size_t)M * N, sizeof(float));
    if (!xf || !wf || !acc) return -1;
    int mx = (scale_dt == ORC_E8M0);
    int64_t g = mx ? 32 : (group > 0 ? group : K);
    int64_t G = (K + g - 1) / g;
    if (scale_n == 1 || (!mx && group <= 0)) G = 1, g = K;
#pragma omp parallel for schedule(static)
    for (int64_t k = 0; k < K; k++) {
        int64_t gi = k / g;
        for (int64_t n = 0; n < N; n++) {
            int64_t sn = scale_n == 1 ? 0 : n;
            size_t si = (size_t)(tW ? sn * G + gi : gi * scale_n + sn);
            float s = load_as_f32(scale, scale_dt, si);
            float v = wf[k * N + n];
            if (inter == ORC_F16) v = trunc_to(v, ORC_F16); /* prepare_weight GW:53-62 (exact for every weight type) */
            if (mx) {
                if (inter == ORC_F16) s = trunc_to(s, ORC_F16);
                v = trunc_to(v * s, inter);
            } else if (offset) {
                float o = trunc_to(load_as_f32(offset, x_dt, si), inter);
                v = trunc_to(v + o, inter);
                v = trunc_to(v * s, inter);
            } else {
                v = trunc_to(v * s, inter);
            }
            wf[k * N + n] = v;
        }
    }
    sgemm_acc(xf, K, wf, N, acc, N, M, N, K);
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            float o = acc[m * N + n];
            if (bias) o = o + load_as_f32(bias, bias_dt, (size_t)n);
            if (x_dt == ORC_BF16) o = trunc_to(o, ORC_BF16);
            store_from_f32(y, x_dt, (size_t)(m * N + n), o);
        }
    free(xf); free(wf); free(acc);
    return 0;
}

/* scale_generate (GQ:50-54): keep the upper 19 bits of an fp32 scale. */
float orc_scale_generate(float s) { return u2f(f2u(s) & 0xFFFFE000u); }
/* u64_to_deq_scale (GQ:129-135): the low 32 bits hold an fp32 scale, truncated as above. */
float orc_u64_to_deq_scale(uint64_t v) { return u2f((uint32_t)v & 0xFFFFE000u); }

size_t orc_dtype_bits(int dt) { return dtype_bits(dt); }

/* ------------------------------------------------------------------------- */
/* Dynamic per-token quantisation (the activation quantizer before the matmul) */
/* ------------------------------------------------------------------------- */

/* GD:17-122 (_dynamic_quant_common, quant_mode "pertoken", no group index).  Per row of x [rows, cols]:
 *   v = fp32(x) * fp32(smooth)                      (smooth optional, one per column)
 *   symmetric:   scale = max|v| * (1 / tmax);                        q = v / scale
 *   asymmetric:  scale = (max v - min v) * (1 / tmax2);  offset = tmax - max v / scale;  q = v / scale + offset
 *   y = integer types: round half to even, then the cast; fp8 types: the cast itself rounds
 * with (tmax, tmax2) = (127, 255) int8, (7, 15) int4, (448, 896) e4m3, (57344, 114688) e5m2; 1 / tmax is an fp32 constant
 * and every operation is a separately rounded fp32 operation.  int4 results are packed two per byte, even column low.
 * A row whose scale is zero divides by zero in the golden (NaN through an integer cast): zeros are written instead. */
int orc_dynamic_quant_grouped(const void* x, int x_dt, int64_t rows, int64_t cols, const void* smooth, const int64_t* group_end,
                              int64_t groups, int y_dt, int symmetric, void* y, float* scale_out, float* offset_out);
int orc_dynamic_quant(const void* x, int x_dt, int64_t rows, int64_t cols, const void* smooth, int y_dt, int symmetric,
                      void* y, float* scale_out, float* offset_out)
{
    return orc_dynamic_quant_grouped(x, x_dt, rows, cols, smooth, NULL, 0, y_dt, symmetric, y, scale_out, offset_out);
}
/* With group_end (GD:52-64): smooth is [groups, cols], expert e owns the rows from group_end[e - 1] (0 for e = 0) up to
 * group_end[e]; an expert whose range is empty owns none.  The golden drops the rows from group_end[groups - 1] on; here they are
 * left untouched (parity unpinned for them). */
int orc_dynamic_quant_grouped(const void* x, int x_dt, int64_t rows, int64_t cols, const void* smooth, const int64_t* group_end,
                              int64_t groups, int y_dt, int symmetric, void* y, float* scale_out, float* offset_out)
{
    float tmax, tmax2;
    switch (y_dt) {
        case ORC_I8: tmax = 127.0f; tmax2 = 255.0f; break;
        case ORC_I4: tmax = 7.0f; tmax2 = 15.0f; break;
        case ORC_E4M3: tmax = 448.0f; tmax2 = 896.0f; break;
        case ORC_E5M2: tmax = 57344.0f; tmax2 = 114688.0f; break;
        default: return -1;
    }
    if ((x_dt != ORC_F16 && x_dt != ORC_BF16) || rows < 0 || cols <= 0 || (y_dt == ORC_I4 && (cols & 1))) return -1;
    if (!symmetric && !offset_out) return -1;
    const float rcp = 1.0f / (symmetric ? tmax : tmax2);
    float* v = (float*)malloc((size_t)cols * sizeof(float));
    if (!v) return -2;
    for (int64_t r = 0; r < rows; r++) {
        int64_t expert = 0;
        if (group_end) {
            while (expert < groups && group_end[expert] <= r) expert++;
            if (expert == groups) continue;
        }
        float vmax = -INFINITY, vmin = INFINITY, amax = 0.0f;
        for (int64_t c = 0; c < cols; c++) {
            float e = load_as_f32(x, x_dt, (size_t)(r * cols + c));
            if (smooth) e = e * load_as_f32(smooth, x_dt, (size_t)(expert * cols + c));
            v[c] = e;
            if (e > vmax) vmax = e;
            if (e < vmin) vmin = e;
            if (fabsf(e) > amax) amax = fabsf(e);
        }
        float scale, offset = 0.0f;
        if (symmetric) {
            scale = amax * rcp;
        } else {
            scale = (vmax - vmin) * rcp;
            offset = tmax - vmax / scale;
        }
        const int degenerate = !(scale > 0.0f) || !isfinite(scale);
        scale_out[r] = scale;
        if (!symmetric) offset_out[r] = degenerate ? 0.0f : offset;
        for (int64_t c = 0; c < cols; c++) {
            float q = 0.0f;
            if (!degenerate) {
                q = v[c] / scale;
                if (!symmetric) q = q + offset;
            }
            const size_t i = (size_t)(r * cols + c);
            if (y_dt == ORC_E4M3) ((uint8_t*)y)[i] = orc_e4m3_from_f32(q);
            else if (y_dt == ORC_E5M2) ((uint8_t*)y)[i] = orc_e5m2_from_f32(q);
            else {
                float rq = nearbyintf(q);
                const float lo = y_dt == ORC_I8 ? -128.0f : -8.0f, hi = y_dt == ORC_I8 ? 127.0f : 7.0f;
                if (!(rq == rq)) rq = 0.0f;
                if (rq < lo) rq = lo;
                if (rq > hi) rq = hi;
                const int iv = (int)rq;
                if (y_dt == ORC_I8) ((int8_t*)y)[i] = (int8_t)iv;
                else {
                    uint8_t* b = (uint8_t*)y + (i >> 1);
                    *b = (i & 1) ? (uint8_t)((*b & 0x0fu) | ((iv & 15) << 4)) : (uint8_t)((*b & 0xf0u) | (iv & 15));
                }
            }
        }
    }
    free(v);
    return 0;
}

/* Dynamic block quantisation to fp8 (the activation / weight quantizer of the block-scale matmul).
 * ../quant/dynamic_block_quant/tests/assets/golden.py:95-222, x [batch, rows, cols] in fp16 / bf16, blocks of rb x cb:
 *   amax  = max over the block of |x|, infinities and NaN counted as 0
 *   scale = fp32(amax / tmax), and min(scale, fp32(1 / min_scale)) when min_scale != 0   (tmax: 448 e4m3, 57344 e5m2)
 *   q     = fp32(x) / scale;  where x is infinite or NaN, q = x;  q clipped to +-tmax
 *   q     = rint(q * 1e8) / 1e8 in fp32  (numpy's round(q, 8) on a float32 array);  NaN -> +0
 *   y     = fp8(q), round to nearest even
 * scale_out is [batch, ceil(rows / rb), ceil(cols / cb)]. */
int orc_dynamic_block_quant(const void* x, int x_dt, int64_t batch, int64_t rows, int64_t cols, int64_t rb, int64_t cb,
                            double min_scale, int y_dt, uint8_t* y, float* scale_out)
{
    if ((x_dt != ORC_F16 && x_dt != ORC_BF16) || (y_dt != ORC_E4M3 && y_dt != ORC_E5M2)) return -1;
    if (batch <= 0 || rows <= 0 || cols <= 0 || rb <= 0 || cb <= 0 || min_scale < 0) return -1;
    const float tmax = y_dt == ORC_E4M3 ? 448.0f : 57344.0f;
    const int64_t nrb = (rows + rb - 1) / rb, ncb = (cols + cb - 1) / cb;
    for (int64_t b = 0; b < batch; b++)
        for (int64_t br = 0; br < nrb; br++)
            for (int64_t bc = 0; bc < ncb; bc++) {
                const int64_t r1 = (br + 1) * rb < rows ? (br + 1) * rb : rows, c1 = (bc + 1) * cb < cols ? (bc + 1) * cb : cols;
                float amax = 0.0f;
                for (int64_t r = br * rb; r < r1; r++)
                    for (int64_t c = bc * cb; c < c1; c++) {
                        const float v = fabsf(load_as_f32(x, x_dt, (size_t)((b * rows + r) * cols + c)));
                        if (isfinite(v) && v > amax) amax = v;
                    }
                float scale = amax / tmax;
                if (min_scale != 0) { const float cap = (float)(1.0 / min_scale); if (cap < scale) scale = cap; }
                scale_out[(b * nrb + br) * ncb + bc] = scale;
                for (int64_t r = br * rb; r < r1; r++)
                    for (int64_t c = bc * cb; c < c1; c++) {
                        const size_t i = (size_t)((b * rows + r) * cols + c);
                        const float v = load_as_f32(x, x_dt, i);
                        float q = isfinite(v) ? v / scale : v;
                        if (q > tmax) q = tmax;          /* np.clip leaves NaN alone, as these comparisons do */
                        if (q < -tmax) q = -tmax;
                        q = nearbyintf(q * 1e8f) / 1e8f;
                        if (!(q == q)) q = 0.0f;
                        y[i] = y_dt == ORC_E4M3 ? orc_e4m3_from_f32(q) : orc_e5m2_from_f32(q);
                    }
            }
    return 0;
}

/* Dynamic MX quantisation along the last axis (the quantizer of the MX matmuls).
 * ../quant/dynamic_mx_quant/tests/assets/golden.py:140-153 (shared exponent), 196-218 (element rounding), 263-330 (driver),
 * round mode "rint", scale algorithm 0, x [rows, cols] in fp16 / bf16, blocks of `block` elements (zero padded):
 *   amax      = max|x| over the block
 *   share_exp = floor(log2(amax)) - emax, -127 when amax == 0 or the result is lower; NaN when above 127 (amax infinite) or
 *               when the block holds a NaN          (emax: 2 for e2m1, 8 for e4m3, 15 for e5m2)
 *   q         = x / 2^share_exp                                                   (fp32; an exact scaling)
 *   e         = max(floor(log2|q|), emin), emin = 0 / -6 / -14;  q = rint(q / 2^e * 2^m) / 2^m * 2^e, m = 1 / 3 / 2 mantissa bits
 *   q clipped to +-tmax (6 / 448 / 57344); NaN -> 0;  y = the element code of q (exact: q is on the format's grid)
 *   scale byte = share_exp + 127 (e8m0), 0xFF for NaN;  scale rows are padded to an even count with byte 0
 * e2m1 codes are packed two per byte, even column in the low nibble.  scale_out is [rows, 2 * ceil(nblocks / 2)]. */
static uint8_t e2m1_code_of(float v)   /* v on the e2m1 grid */
{
    const float a = fabsf(v);
    uint8_t c = 0;
    for (uint8_t i = 0; i < 8; i++) if (kE2M1[i] == a) c = i;
    return (uint8_t)(c | (signbit(v) ? 8u : 0u));
}
int orc_dynamic_mx_quant_general(const void* x, int x_dt, int64_t outer, int64_t A, int64_t inner, int64_t block, int scale_alg,
                                 int round_mode, int y_dt, uint8_t* y, uint8_t* scale_out);
int orc_dynamic_mx_quant_alg(const void* x, int x_dt, int64_t rows, int64_t cols, int64_t block, int scale_alg, int y_dt, uint8_t* y,
                             uint8_t* scale_out)
{
    if (x_dt != ORC_F16 && x_dt != ORC_BF16) return -1;
    return orc_dynamic_mx_quant_general(x, x_dt, rows, cols, 1, block, scale_alg, 0, y_dt, y, scale_out);
}
int orc_dynamic_mx_quant(const void* x, int x_dt, int64_t rows, int64_t cols, int64_t block, int y_dt, uint8_t* y, uint8_t* scale_out)
{
    return orc_dynamic_mx_quant_alg(x, x_dt, rows, cols, block, 0, y_dt, y, scale_out);
}
/* The general form (GD:263-330 with its helpers): x is [outer, A, inner] and the blocks run along A; x in fp16, bf16 or fp32;
 * elements e2m1, e1m2 (emax 0, emin 0, two mantissa bits, maximum 1.75: the eight magnitudes k/4), e4m3, e5m2;
 * round_mode (_mx_round_mantissa, GD:181-197, applied to the element's mantissa scaled to an integer): 0 rint (ties to even),
 * 1 round (ties away from zero: floor(|v| + 0.5) with the sign), 2 floor, 3 ceil, 4 trunc.
 * scale_alg 1 (GD:156-176, fp8 elements only): share_exp is the exponent field of fp32(amax / tmax) minus 127, plus one when that
 * quotient is not a power of two (a normal number with mantissa bits, or a subnormal above 2^-127).
 * y has x's shape, 4-bit codes packed two per byte along the last axis (even flat index in the low nibble);
 * scale_out is [outer, ceil(nblocks / 2), inner, 2]: the two blocks of a pair side by side (_interleave, GD:235-262), a missing
 * second block padded with byte 0 (_pad_to_even pads with 2^-127). */
int orc_dynamic_mx_quant_general(const void* x, int x_dt, int64_t outer, int64_t A, int64_t inner, int64_t block, int scale_alg,
                                 int round_mode, int y_dt, uint8_t* y, uint8_t* scale_out)
{
    int emax, emin, mbits; float tmax;
    switch (y_dt) {
        case ORC_E2M1: emax = 2; emin = 0; mbits = 1; tmax = 6.0f; break;
        case ORC_E1M2: emax = 0; emin = 0; mbits = 2; tmax = 1.75f; break;
        case ORC_E4M3: emax = 8; emin = -6; mbits = 3; tmax = 448.0f; break;
        case ORC_E5M2: emax = 15; emin = -14; mbits = 2; tmax = 57344.0f; break;
        default: return -1;
    }
    const int fp4 = y_dt == ORC_E2M1 || y_dt == ORC_E1M2;
    if ((x_dt != ORC_F16 && x_dt != ORC_BF16 && x_dt != ORC_F32) || outer <= 0 || A <= 0 || inner <= 0 || block <= 0) return -1;
    if (fp4 && ((outer * A * inner) & 1)) return -1;
    if (scale_alg != 0 && (scale_alg != 1 || fp4)) return -1;
    if (round_mode < 0 || round_mode > 4) return -1;
    const int64_t nblk = (A + block - 1) / block, np = (nblk + 1) / 2;
    memset(scale_out, 0, (size_t)(outer * np * inner * 2));
    for (int64_t o = 0; o < outer; o++)
        for (int64_t in = 0; in < inner; in++)
            for (int64_t b = 0; b < nblk; b++) {
                const int64_t a1 = (b + 1) * block < A ? (b + 1) * block : A;
                float amax = 0.0f; int has_nan = 0;
                for (int64_t a = b * block; a < a1; a++) {
                    const float v = fabsf(load_as_f32(x, x_dt, (size_t)((o * A + a) * inner + in)));
                    if (v != v) has_nan = 1;
                    if (v > amax) amax = v;
                }
                float share;   /* an integer, or NaN */
                if (has_nan) share = NAN;
                else if (amax == 0.0f) share = -127.0f;
                else if (scale_alg == 1) {
                    if (isinf(amax)) share = NAN;
                    else {
                        const uint32_t u = f2u(amax / tmax);
                        int e = (int)(u >> 23);
                        const uint32_t mant = u & 0x7fffffu;
                        if ((e > 0 && e < 254 && mant > 0) || (e == 0 && mant > (1u << 22))) e += 1;
                        share = (float)(e - 127);
                    }
                }
                else {
                    share = floorf(log2f(amax)) - (float)emax;
                    if (share > 127.0f) share = NAN;
                    else if (share < -127.0f) share = -127.0f;
                }
                scale_out[((o * np + b / 2) * inner + in) * 2 + (b & 1)] = (share == share) ? (uint8_t)((int)share + 127) : 0xFFu;
                for (int64_t a = b * block; a < a1; a++) {
                    const size_t i = (size_t)((o * A + a) * inner + in);
                    float q = 0.0f;
                    if (share == share) {
                        q = load_as_f32(x, x_dt, i) / ldexpf(1.0f, (int)share);
                        float e = floorf(log2f(fabsf(q) + (q == 0.0f ? 1.0f : 0.0f)));
                        if (e < (float)emin) e = (float)emin;
                        const float pe = ldexpf(1.0f, (int)e), pm = ldexpf(1.0f, mbits);
                        float r = q / pe * pm;
                        switch (round_mode) {
                            case 0: r = nearbyintf(r); break;
                            case 1: { const float t = floorf(fabsf(r) + 0.5f); r = signbit(r) ? -t : t; break; }
                            case 2: r = floorf(r); break;
                            case 3: r = ceilf(r); break;
                            default: r = truncf(r); break;
                        }
                        q = r / pm * pe;
                        if (q > tmax) q = tmax;
                        if (q < -tmax) q = -tmax;
                        if (!(q == q)) q = 0.0f;
                    }
                    if (y_dt == ORC_E4M3) y[i] = orc_e4m3_from_f32(q);
                    else if (y_dt == ORC_E5M2) y[i] = orc_e5m2_from_f32(q);
                    else {
                        const uint8_t code = y_dt == ORC_E2M1 ? e2m1_code_of(q)
                                                              : (uint8_t)((uint8_t)(fabsf(q) * 4.0f) | (signbit(q) ? 8u : 0u));
                        uint8_t* pb = y + (i >> 1);
                        *pb = (i & 1) ? (uint8_t)((*pb & 0x0fu) | (code << 4)) : (uint8_t)((*pb & 0xf0u) | code);
                    }
                }
            }
    return 0;
}

/* aclnnTransQuantParamV2 / V3: the packed 64-bit quantisation parameter (../quant/trans_quant_param_v2/op_kernel/
 * trans_quant_param_v2.h:224-300; the same layout GQ:129-158 reads back).  round_mode 0 keeps the upper 19 bits of the scale;
 * round_mode 1 rounds the 23-bit mantissa to 10 bits, nearest even, the carry running into the exponent, a zero or subnormal
 * scale becoming a signed zero and infinity / NaN keeping their (truncated) bits.  The offset is rint'ed, clamped to
 * [-256, 255] and stored as 9 bits at bit 37; bit 46 is set.  One-element inputs are broadcast. */
void orc_trans_quant_param(const float* scale, int64_t scale_len, const float* offset, int64_t offset_len, int round_mode, uint64_t* out)
{
    const int64_t n = (offset && offset_len > scale_len) ? offset_len : scale_len;
    for (int64_t i = 0; i < n; i++) {
        const uint32_t u = f2u(scale[scale_len == 1 ? 0 : i]);
        uint32_t lo;
        if (round_mode == 0) lo = u & 0xFFFFE000u;
        else {
            const uint32_t sign = u >> 31;
            uint32_t e = (u >> 23) & 0xFFu, m = (u & 0x7FFFFFu) >> 13;
            if (e == 0) { m = 0; }
            else if (e != 255) {
                const uint32_t rest = u & 0x1FFFu;               /* the 13 dropped bits */
                if (rest > 0x1000u || (rest == 0x1000u && (m & 1u))) { m += 1; if (m == 1024u) { m = 0; e += 1; } }
            }
            lo = (sign << 31) | (e << 23) | (m << 13);
        }
        uint64_t v = (uint64_t)lo | (1ull << 46);
        if (offset) {
            float o = nearbyintf(offset[offset_len == 1 ? 0 : i]);
            if (!(o == o)) o = 0.0f;
            if (o < -256.0f) o = -256.0f;
            if (o > 255.0f) o = 255.0f;
            v |= ((uint64_t)(int64_t)(int)o & 0x1FFull) << 37;
        }
        out[i] = v;
    }
}

/* Dynamic quantisation with one scale for the whole tensor (mode 1, GD:66-94 with quant_mode "pertensor") or one per batch
 * and column, reduced over the second-to-last axis (mode 2, GD:125-176 _dynamic_quant_perchannel): x is
 * [rows / chan_rows, chan_rows, cols]; smooth has cols factors in mode 1 and chan_rows factors (one per row of a batch) in
 * mode 2.  The element formulas are those of orc_dynamic_quant.  scale_out / offset_out: 1 element, or (rows / chan_rows) * cols. */
int orc_dynamic_quant_wide(const void* x, int x_dt, int64_t rows, int64_t cols, int64_t chan_rows, int mode, const void* smooth, int y_dt,
                           int symmetric, void* y, float* scale_out, float* offset_out)
{
    float tmax, tmax2;
    switch (y_dt) {
        case ORC_I8: tmax = 127.0f; tmax2 = 255.0f; break;
        case ORC_I4: tmax = 7.0f; tmax2 = 15.0f; break;
        case ORC_E4M3: tmax = 448.0f; tmax2 = 896.0f; break;
        case ORC_E5M2: tmax = 57344.0f; tmax2 = 114688.0f; break;
        default: return -1;
    }
    if ((mode != 1 && mode != 2) || rows <= 0 || cols <= 0 || (y_dt == ORC_I4 && (cols & 1))) return -1;
    if (mode == 1) chan_rows = rows;
    if (chan_rows <= 0 || rows % chan_rows) return -1;
    const float rcp = 1.0f / (symmetric ? tmax : tmax2);
    const int64_t nb = rows / chan_rows, nslots = mode == 1 ? 1 : nb * cols;
    float* vmax = (float*)malloc((size_t)nslots * 3 * sizeof(float));
    if (!vmax) return -2;
    float *vmin = vmax + nslots, *amax = vmin + nslots;
    for (int64_t s = 0; s < nslots; s++) { vmax[s] = -INFINITY; vmin[s] = INFINITY; amax[s] = 0.0f; }
#define WIDE_VALUE(r, c) (load_as_f32(x, x_dt, (size_t)((r) * cols + (c))) * (smooth ? load_as_f32(smooth, x_dt, (size_t)(mode == 1 ? (c) : (r) % chan_rows)) : 1.0f))
#define WIDE_SLOT(r, c) (mode == 1 ? 0 : ((r) / chan_rows) * cols + (c))
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < cols; c++) {
            const float e = smooth ? WIDE_VALUE(r, c) : load_as_f32(x, x_dt, (size_t)(r * cols + c));
            const int64_t s = WIDE_SLOT(r, c);
            if (e > vmax[s]) vmax[s] = e;
            if (e < vmin[s]) vmin[s] = e;
            if (fabsf(e) > amax[s]) amax[s] = fabsf(e);
        }
    for (int64_t s = 0; s < nslots; s++) {
        float scale, offset = 0.0f;
        if (symmetric) scale = amax[s] * rcp;
        else { scale = (vmax[s] - vmin[s]) * rcp; offset = tmax - vmax[s] / scale; }
        const int degenerate = !(scale > 0.0f) || !isfinite(scale);
        scale_out[s] = scale;
        if (!symmetric) offset_out[s] = degenerate ? 0.0f : offset;
        amax[s] = degenerate ? 1.0f : 0.0f;   /* reused as the flag */
    }
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < cols; c++) {
            const int64_t s = WIDE_SLOT(r, c);
            const size_t i = (size_t)(r * cols + c);
            float q = 0.0f;
            if (amax[s] == 0.0f) {
                const float e = smooth ? WIDE_VALUE(r, c) : load_as_f32(x, x_dt, i);
                q = e / scale_out[s];
                if (!symmetric) q = q + offset_out[s];
            }
            if (y_dt == ORC_E4M3) ((uint8_t*)y)[i] = orc_e4m3_from_f32(q);
            else if (y_dt == ORC_E5M2) ((uint8_t*)y)[i] = orc_e5m2_from_f32(q);
            else {
                float rq = nearbyintf(q);
                const float lo = y_dt == ORC_I8 ? -128.0f : -8.0f, hi = y_dt == ORC_I8 ? 127.0f : 7.0f;
                if (!(rq == rq)) rq = 0.0f;
                if (rq < lo) rq = lo;
                if (rq > hi) rq = hi;
                const int iv = (int)rq;
                if (y_dt == ORC_I8) ((int8_t*)y)[i] = (int8_t)iv;
                else {
                    uint8_t* b = (uint8_t*)y + (i >> 1);
                    *b = (i & 1) ? (uint8_t)((*b & 0x0fu) | ((iv & 15) << 4)) : (uint8_t)((*b & 0xf0u) | (iv & 15));
                }
            }
        }
#undef WIDE_VALUE
#undef WIDE_SLOT
    free(vmax);
    return 0;
}
