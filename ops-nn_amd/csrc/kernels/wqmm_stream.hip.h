// Weight-only decode kernel, streamlined form: the shapes it takes are restricted so that the inner loop carries
// nothing but the essential work -- per 8 weights of a lane: the dequantisation (18 packed-fp16 / integer
// operations with an offset, 14 without), one 16-byte LDS read of x and one v_mfma_f32_16x16x32.
//
// Restrictions (the launcher checks them; anything else goes to the general kernel in wqmm.hip):
//   K is a multiple of the chunk KC (128 int4 / 64 int8 weights: what one wave load instruction covers per row);
//   the group size is a power-of-two multiple of KC, or the scale is per channel;
//   VSCALE: group == KC, a row's scales contiguous and 16-byte aligned, K/group a multiple of 8 -- then one
//           16-byte load per lane brings the scales of the next 8 chunks.
//
// Work split: a wave owns 16 weight rows (output columns).  WK = 1: the four waves of a workgroup take four row
// blocks and all of K.  WK = 4: they take one row block and every fourth chunk each (narrow N), and their partial
// sums meet in LDS in a fixed order.  Either way all four waves walk the same K slabs of x, staged once per
// workgroup in LDS (only the rows that exist, plus one zero row that the idle MFMA columns read).
//
// Weight pieces are fetched 8 chunks ahead: the register that a chunk has just been consumed from is reloaded
// with the chunk 8 further on, so 8 loads per lane are always in flight without a second register set.
#pragma once
#include "wqmm_common.hip.h"

namespace opsnn {

// ---- 8 consecutive-k weights of one lane -> MFMA row operand (8 values of x's dtype) ----
// piece: the lane's 16-byte weight piece; s: which 8 of its weights (int4: dword s, element order
// [0,4,1,5,2,6,3,7] matched by the staged x; int8: dwords 2s, 2s+1 in natural order).
struct DqConst {
    uint32_t mlo, mhi, clo, chi;   // int4 splice masks and exponent/sign constants, held in registers
};
__device__ __forceinline__ DqConst make_dq_const()
{
    DqConst c = {0x000F000Fu, 0x00F000F0u, 0x64086408u, 0x64806480u};
    asm volatile("" : "+v"(c.mlo), "+v"(c.mhi), "+v"(c.clo), "+v"(c.chi));   // not literals: see dequant8
    return c;
}

// NATURAL: the 8 values leave in k order (one more byte permute per register for int4 x fp16) for kernels whose x
// reaches LDS unpermuted.
template <int XDT, int WBITS, bool HAS_OFF, bool NATURAL = false>
__device__ __forceinline__ v4i dequant8(const v4i& piece, int s, uint16_t sb, uint16_t ob, const DqConst& dc)
{
    if constexpr (XDT == DT_F16) {
        const _Float16 sh = __builtin_bit_cast(_Float16, sb), oh = __builtin_bit_cast(_Float16, ob);
        const h2 sc = {sh, sh}, off = {oh, oh};
        h2 t0, t1, t2, t3;
        if constexpr (WBITS == 4) {
            // (q & mask) ^ c flips each nibble's sign bit (w + 8 in 0..15) and sets the exponent of 1024.0 in one
            // three-operand bit operation; the constants are kept in registers so that it stays one instruction
            const uint32_t q = (uint32_t)piece[s], q8 = q >> 8;
            const uint32_t mlo = dc.mlo, mhi = dc.mhi, clo = dc.clo, chi = dc.chi;
            const h2 c1032 = {(_Float16)-1032.0f, (_Float16)-1032.0f};
            const h2 c72 = {(_Float16)-72.0f, (_Float16)-72.0f};
            const h2 r16 = {(_Float16)0.0625f, (_Float16)0.0625f};
            t0 = __builtin_bit_cast(h2, (q & mlo) ^ clo);     // 1024 + (w+8): elements 0, 4
            t1 = __builtin_bit_cast(h2, (q & mhi) ^ chi);     // 1024 + 16(w+8): elements 1, 5
            t2 = __builtin_bit_cast(h2, (q8 & mlo) ^ clo);    // elements 2, 6
            t3 = __builtin_bit_cast(h2, (q8 & mhi) ^ chi);    // elements 3, 7
            t0 = t0 + c1032;                                // exact
            t2 = t2 + c1032;
            t1 = __builtin_elementwise_fma(t1, r16, c72);   // exact: (1024 + 16(w+8))/16 - 72
            t3 = __builtin_elementwise_fma(t3, r16, c72);
        } else {
            // bytes become w + 128 in 0..255 and are spliced under the exponent byte of 1024.0
            const uint32_t qa = (uint32_t)piece[2 * s] ^ 0x80808080u, qb = (uint32_t)piece[2 * s + 1] ^ 0x80808080u;
            const uint32_t magic = 0x64646464u;
            const h2 c1152 = {(_Float16)-1152.0f, (_Float16)-1152.0f};
            t0 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(magic, qa, 0x04010400u)) + c1152;   // elements 0, 1
            t1 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(magic, qa, 0x04030402u)) + c1152;   // elements 2, 3
            t2 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(magic, qb, 0x04010400u)) + c1152;   // elements 4, 5
            t3 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(magic, qb, 0x04030402u)) + c1152;   // elements 6, 7
        }
        if constexpr (HAS_OFF) { t0 = t0 + off; t1 = t1 + off; t2 = t2 + off; t3 = t3 + off; }   // first rounding
        t0 = t0 * sc; t1 = t1 * sc; t2 = t2 * sc; t3 = t3 * sc;                                  // second rounding
        if constexpr (NATURAL && WBITS == 4) {   // pairs (0,4) (1,5) (2,6) (3,7) -> (0,1) (2,3) (4,5) (6,7)
            return (v4i){(int)__builtin_amdgcn_perm(u32(t1), u32(t0), 0x05040100u), (int)__builtin_amdgcn_perm(u32(t3), u32(t2), 0x05040100u),
                         (int)__builtin_amdgcn_perm(u32(t1), u32(t0), 0x07060302u), (int)__builtin_amdgcn_perm(u32(t3), u32(t2), 0x07060302u)};
        }
        return (v4i){(int)u32(t0), (int)u32(t1), (int)u32(t2), (int)u32(t3)};
    } else {
        // bf16: no packed bf16 arithmetic on this chip, so the two steps run in fp32 with a hardware
        // round-to-nearest-even conversion to bf16 after each
        const float scf = bf16_to_f32(sb), off = bf16_to_f32(ob);
        float w[8];
        if constexpr (WBITS == 4) {
            const uint32_t q = (uint32_t)piece[s];
            const int ord[8] = {0, 4, 1, 5, 2, 6, 3, 7};
#pragma unroll
            for (int j = 0; j < 8; j++) w[j] = (float)(((int)(q << (28 - 4 * (NATURAL ? j : ord[j])))) >> 28);
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) w[j] = (float)(((int)((uint32_t)piece[2 * s + (j >> 2)] << (24 - 8 * (j & 3)))) >> 24);
        }
        v4i r;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float a = w[2 * j], b = w[2 * j + 1];
            if constexpr (HAS_OFF) {
                const v2f t = {a + off, b + off};
                const uint32_t pk = pack2_bf16(t);
                a = __builtin_bit_cast(float, pk << 16);
                b = __builtin_bit_cast(float, pk & 0xffff0000u);
            }
            const v2f t = {a * scf, b * scf};
            r[j] = (int)pack2_bf16(t);
        }
        return r;
    }
}

// ---- 8 floating-point weight codes of one lane -> MFMA row operand ----
// WBITS 4: the e2m1 codes of dword s, delivered in element order [0,4,1,5,2,6,3,7] like dequant8's int4 form (NATURAL:
// in element order, four byte permutes more); WBITS 8: the e4m3 codes of dwords 2s, 2s+1 in natural order.  Every code
// is exact in fp16 and in bf16, so T(w * scale) rounds once, in the multiplication: packed fp16 for fp16; for bf16 the
// exact fp16 value is widened to fp32, multiplied and rounded to bf16 by the hardware conversion.
template <int XDT, int WBITS, bool NATURAL = false>
__device__ __forceinline__ v4i dequant8_float(const v4i& piece, int s, uint16_t sb)
{
    if constexpr (NATURAL && WBITS == 4) {
        const v4i r = dequant8_float<XDT, WBITS, false>(piece, s, sb);   // halves (0,4) (1,5) (2,6) (3,7)
        const uint32_t a = (uint32_t)r[0], b = (uint32_t)r[1], c = (uint32_t)r[2], d = (uint32_t)r[3];
        return (v4i){(int)__builtin_amdgcn_perm(b, a, 0x05040100u), (int)__builtin_amdgcn_perm(d, c, 0x05040100u),
                     (int)__builtin_amdgcn_perm(b, a, 0x07060302u), (int)__builtin_amdgcn_perm(d, c, 0x07060302u)};
    }
    h2 w[4];   // the eight weights, exact, as fp16 pairs
    if constexpr (WBITS == 4) {
        const uint32_t q = (uint32_t)piece[s];
        const h2 k14 = {(_Float16)16384.0f, (_Float16)16384.0f};
#pragma unroll
        for (int i = 0; i < 4; i++) {   // see dequant_fp4_f16: magnitude bits at bits 11..9 of a half read as 2^-14 times the value
            const uint32_t t = q >> (4 * i);
            w[i] = __builtin_bit_cast(h2, ((t & 0x00070007u) << 9) | ((t & 0x00080008u) << 12)) * k14;
        }
    } else {
        const uint32_t d0 = (uint32_t)piece[2 * s], d1 = (uint32_t)piece[2 * s + 1];
        w[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d0, 1.0f, false);
        w[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d0, 1.0f, true);
        w[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d1, 1.0f, false);
        w[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d1, 1.0f, true);
    }
    if constexpr (XDT == DT_F16) {
        const _Float16 sh = __builtin_bit_cast(_Float16, sb);
        const h2 sc = {sh, sh};
        return (v4i){(int)u32(w[0] * sc), (int)u32(w[1] * sc), (int)u32(w[2] * sc), (int)u32(w[3] * sc)};
    } else {
        const float scf = bf16_to_f32(sb);
        v4i r;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const v2f t = {(float)w[i][0] * scf, (float)w[i][1] * scf};
            r[i] = (int)pack2_bf16(t);
        }
        return r;
    }
}

// NW waves per workgroup (4 or 8) = WN row blocks x WK waves that split K chunk by chunk.
template <int XDT, int WBITS, int MB, int NW, int WK, bool HAS_OFF, bool VSCALE>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(NW == 8 ? 4 : 2))) void wqmm_stream_kernel(WqParams p)
{
    static_assert(!(VSCALE && WK > 2), "vector scale loads: a wave's chunks are consecutive (WK 1) or every other one (WK 2)");
    constexpr int NT = NW * 64;
    constexpr int WN = NW / WK;
    constexpr int KPL = 128 / WBITS;     // k per 16-byte piece: 32 or 16
    constexpr int KC = 4 * KPL;          // k per chunk: 128 or 64 (64 bytes of a weight row either way)
    constexpr int STEPS = KC / 32;       // MFMA steps per chunk: 4 or 2
    constexpr int PF = (MB == 1 && WK == 1) ? 16 : 8;   // chunks per super-step = pieces in flight per lane
    constexpr int KX = 8 * KC / MB;      // k per LDS slab of x
    constexpr int CPS = KX / KC;         // chunks per slab: 8, 4, 2
    constexpr int CPSW = CPS / WK;       // of which this wave's
    static_assert(CPSW >= 1, "a slab must hold at least one chunk per K-split wave");
    constexpr int XROW = KX * 2 + 16;    // LDS row pitch (bytes); the pad makes the 16-byte reads conflict free
    constexpr int XPR = KX / 8;          // 16-byte pieces per x row per slab
    constexpr int XITEMS = 16 * MB * XPR / NT;
    extern __shared__ __attribute__((aligned(16))) char sx[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave / WK, wk = wave % WK;
    const int nrow = lane & 15, g = lane >> 4;
    const int64_t n0 = ((int64_t)blockIdx.x * WN + wn) * 16;
    const bool n_ok = n0 < p.N;
    const int64_t n = (n0 + nrow) < p.N ? (n0 + nrow) : p.N - 1;   // rows past the edge recompute the last one
    const int Ki = (int)p.K;
    const int NCW = Ki / (KC * WK);      // this wave's chunks: chunk index = cw * WK + wk
    const int NSLAB = (Ki + KX - 1) / KX;
    const int rows = (int)p.m_rows;      // 1 .. 16*MB rows of x in this launch
    const int xslab = (rows + 1) * XROW; // + the zero row

    const uint8_t* wptr = p.w + n * p.ldw + g * 16 + wk * 64;
    const uint16_t* srow = p.scale + n * p.s_cs;
    const uint16_t* orow = HAS_OFF ? p.offset + n * p.s_cs : nullptr;

    // ---- x staging ----
    v4i xreg[XITEMS];
    const int xtotal = rows * XPR;
    auto load_x = [&](int slab) {
#pragma unroll
        for (int it = 0; it < XITEMS; it++) {
            const int idx = it * NT + tid;
            if (it * NT >= xtotal) break;
            const int r = idx / XPR, c = idx % XPR;
            const int k = slab * KX + c * 8;
            v4i v = {0, 0, 0, 0};
            if (idx < xtotal && k < Ki) v = *(const v4i*)(p.x + (p.m_base + r) * p.K + k);
            xreg[it] = v;
        }
    };
    auto store_x = [&](int buf) {
        char* dst = sx + buf * xslab;
#pragma unroll
        for (int it = 0; it < XITEMS; it++) {
            const int idx = it * NT + tid;
            if (it * NT >= xtotal) break;
            const int r = idx / XPR, c = idx % XPR;
            v4i v = xreg[it];
            if constexpr (WBITS == 4 && XDT == DT_F16) {
                // halves [0..7] -> [0,4,1,5,2,6,3,7]: the order in which the nibble splicing yields pairs
                const uint32_t a0 = (uint32_t)v[0], a1 = (uint32_t)v[1], a2 = (uint32_t)v[2], a3 = (uint32_t)v[3];
                v = (v4i){(int)__builtin_amdgcn_perm(a2, a0, 0x05040100u), (int)__builtin_amdgcn_perm(a2, a0, 0x07060302u),
                          (int)__builtin_amdgcn_perm(a3, a1, 0x05040100u), (int)__builtin_amdgcn_perm(a3, a1, 0x07060302u)};
            } else if constexpr (WBITS == 4) {
                const uint32_t a0 = (uint32_t)v[0], a1 = (uint32_t)v[1], a2 = (uint32_t)v[2], a3 = (uint32_t)v[3];
                v = (v4i){(int)__builtin_amdgcn_perm(a2, a0, 0x05040100u), (int)__builtin_amdgcn_perm(a2, a0, 0x07060302u),
                          (int)__builtin_amdgcn_perm(a3, a1, 0x05040100u), (int)__builtin_amdgcn_perm(a3, a1, 0x07060302u)};
            }
            if (idx < xtotal) *(v4i*)(dst + r * XROW + c * 16) = v;
        }
    };
    // the zero row of both buffers
    for (int i = tid; i < 2 * (XROW / 16); i += NT) {
        const int buf = i / (XROW / 16), c = i % (XROW / 16);
        *(v4i*)(sx + buf * xslab + rows * XROW + c * 16) = (v4i){0, 0, 0, 0};
    }
    // LDS byte offset of this lane's column operand inside a slab buffer, per 16-row block
    int xoff[MB];
#pragma unroll
    for (int b = 0; b < MB; b++) {
        const int r = 16 * b + nrow;
        xoff[b] = (r < rows ? r : rows) * XROW + g * KPL * 2;
    }

    v4f acc[MB];
#pragma unroll
    for (int b = 0; b < MB; b++) acc[b] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
    const DqConst dqc = make_dq_const();

    // ---- weight / scale prefetch state ----
    v4i wq[PF];
    uint16_t sq[PF], oq[PF];   // !VSCALE: scale and offset of each chunk in flight
    constexpr int SV = PF * WK / 8;   // VSCALE: the scales (offsets) of the chunks a super-step spans, 8 per register quad
    v4i sv[SV], ov[SV], svn[SV], ovn[SV];
#pragma unroll
    for (int h = 0; h < SV; h++) sv[h] = ov[h] = svn[h] = ovn[h] = (v4i){0, 0, 0, 0};
    auto group_of = [&](int cw) { return ((cw * WK + wk) >> p.cpg_shift); };   // cpg_shift = 31 for per-channel
    auto fetch = [&](int j, int cw) {   // chunk cw of this wave into slot j
        wq[j] = *(const v4i*)(wptr + (int64_t)cw * (WK * 64));
        if constexpr (!VSCALE) {
            const int64_t so = (int64_t)group_of(cw) * p.s_rs;
            sq[j] = srow[so];
            if constexpr (HAS_OFF) oq[j] = orow[so];
        }
    };
#pragma unroll
    for (int j = 0; j < PF; j++) fetch(j, j < NCW ? j : NCW - 1);
    if constexpr (VSCALE) {
#pragma unroll
        for (int h = 0; h < SV; h++) {
            if (8 * h < NCW * WK) {
                svn[h] = *(const v4i*)(srow + 8 * h);
                if constexpr (HAS_OFF) ovn[h] = *(const v4i*)(orow + 8 * h);
            }
        }
    }
    load_x(0);
    store_x(0);
    if (NSLAB > 1) load_x(1);

    // one super-step: this wave's chunks c0 .. c0+7.  TAIL: some of them may not exist and the refills are clamped.
    auto superstep = [&](int c0, auto tail_tag) {
        constexpr bool TAIL = decltype(tail_tag)::value;
        if constexpr (VSCALE) {
#pragma unroll
            for (int h = 0; h < SV; h++) {
                sv[h] = svn[h]; ov[h] = ovn[h];
                if ((c0 + PF) * WK + 8 * h < NCW * WK) {
                    svn[h] = *(const v4i*)(srow + (c0 + PF) * WK + 8 * h);
                    if constexpr (HAS_OFF) ovn[h] = *(const v4i*)(orow + (c0 + PF) * WK + 8 * h);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < PF; j++) {
            const int cw = c0 + j;
            if (j % CPSW == 0) {
                // slab boundary: every wave has finished the previous slab and sees this one; the next slab moves
                // from registers into the buffer just vacated and the one after it starts loading
                const int slab = cw / CPSW;
                if (!TAIL || slab < NSLAB) {
                    __syncthreads();
                    if (slab + 1 < NSLAB) store_x((slab + 1) & 1);
                    if (slab + 2 < NSLAB) load_x(slab + 2);
                }
            }
            if (TAIL && cw >= NCW) continue;
            const int slab = cw / CPSW;
            const char* xs = sx + (slab & 1) * xslab + ((cw % CPSW) * WK + wk) * (KC * 2);
            uint16_t sb, ob = 0;
            if constexpr (VSCALE) {
                // this wave's chunk j of the super-step is chunk j*WK + wk of the span the scale quads cover
                if constexpr (WK == 1) {
                    sb = (uint16_t)((uint32_t)sv[j / 8][(j % 8) / 2] >> (16 * (j % 2)));
                    if constexpr (HAS_OFF) ob = (uint16_t)((uint32_t)ov[j / 8][(j % 8) / 2] >> (16 * (j % 2)));
                } else {
                    sb = (uint16_t)((uint32_t)sv[j / 4][j % 4] >> (16 * wk));
                    if constexpr (HAS_OFF) ob = (uint16_t)((uint32_t)ov[j / 4][j % 4] >> (16 * wk));
                }
            } else {
                sb = sq[j];
                if constexpr (HAS_OFF) ob = oq[j];
            }
#pragma unroll
            for (int s = 0; s < STEPS; s++) {
                const v4i aop = dequant8<XDT, WBITS, HAS_OFF>(wq[j], s, sb, ob, dqc);
#pragma unroll
                for (int b = 0; b < MB; b++) {
                    const v4i bop = *(const v4i*)(xs + xoff[b] + 16 * s);
                    if constexpr (XDT == DT_F16) {
                        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, aop), __builtin_bit_cast(v8h, bop), acc[b], 0, 0, 0);
                    } else {
                        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, aop), __builtin_bit_cast(v8bf, bop), acc[b], 0, 0, 0);
                    }
                }
            }
            // refill the slot with the chunk 8 further on
            if constexpr (TAIL) {
                const int nx = cw + PF;
                fetch(j, nx < NCW ? nx : NCW - 1);
            } else {
                fetch(j, cw + PF);
            }
        }
    };

    int c0 = 0;
    for (; c0 + 2 * PF <= NCW; c0 += PF) superstep(c0, std::false_type{});
    for (; c0 < NCW; c0 += PF) superstep(c0, std::true_type{});

    if constexpr (WK > 1) {
        __syncthreads();
        float* red = (float*)sx;
        if (wk > 0) {
#pragma unroll
            for (int b = 0; b < MB; b++)
#pragma unroll
                for (int i = 0; i < 4; i++) red[(((wn * (WK - 1) + (wk - 1)) * MB + b) * 4 + i) * 64 + lane] = acc[b][i];
        }
        __syncthreads();
        if (wk > 0) return;
#pragma unroll
        for (int j = 0; j < WK - 1; j++)
#pragma unroll
            for (int b = 0; b < MB; b++)
#pragma unroll
                for (int i = 0; i < 4; i++) acc[b][i] = acc[b][i] + red[(((wn * (WK - 1) + j) * MB + b) * 4 + i) * 64 + lane];
    }

    // D'[row = weight row n][col = x row m]: lane holds col m = lane%16, rows n = 4*(lane/16) + i
    if (!n_ok) return;
#pragma unroll
    for (int b = 0; b < MB; b++) {
        const int r = 16 * b + nrow;
        if (r >= rows) continue;
        const int64_t m = p.m_base + r;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int64_t nn = n0 + 4 * g + i;
            v[i] = acc[b][i];
            if (p.bias && nn < p.N) v[i] = v[i] + load_scalar_as_f32(p.bias, p.bias_dt, nn);
            if constexpr (XDT == DT_BF16) v[i] = bf16_to_f32(bf16_bits(v[i]));   // the golden rounds bf16 results twice (a no-op)
        }
        const int64_t nn0 = n0 + 4 * g;
        if (nn0 + 3 < p.N && (p.N % 4) == 0) {
            const v4us o = {bits_x<XDT>(v[0]), bits_x<XDT>(v[1]), bits_x<XDT>(v[2]), bits_x<XDT>(v[3])};
            *(v4us*)(p.y + m * p.N + nn0) = o;
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (nn0 + i < p.N) p.y[m * p.N + nn0 + i] = bits_x<XDT>(v[i]);
        }
    }
}

// ---- many rows of x (65 .. 128 per launch): a wave owns NB blocks of 16 weight rows ----
// With several 16-row blocks of x per weight block the loop stops being a stream: every MFMA needs an x fragment
// from LDS, and with one weight block per wave that is one 1 KB LDS read per MFMA (16 clocks), four times what the
// LDS delivers.  Here every x fragment read serves NB MFMAs (NB weight blocks of the same wave):
//   per 32-k step and wave: NB dequantisations, MB LDS reads, MB * NB MFMAs (16x16x32).
// Workgroup: 8 waves = WN column groups (16 * NB columns each) x WK waves that take every WK-th chunk of K; their
// partial sums meet in LDS in a fixed order at the end.  A slab of x is the WK chunks the waves work on at the same
// time, double-buffered, one barrier per slab.  x travels global -> LDS with 16-byte asynchronous copies (no
// registers, no vector ALU work), so it sits in LDS in k order and the dequantisation delivers k order too
// (dequant8<..., NATURAL>); rows are 16-byte-piece swizzled (piece ^ row % 16) instead of padded, because a copy
// instruction fills 1 KB of consecutive LDS.  Rows of the slab that x does not have repeat its last row: they only
// feed output rows that are never stored.
// A wave's loads complete in issue order, so waiting for its x copies of the next slab also waits for every weight
// load issued before them; with the weights PF = 2..4 chunks ahead and the x copies issued one slab ahead, first
// thing after the barrier, that costs the weight stream at most the lookahead beyond one slab.
// Scale and offset of a chunk travel with its weights (one 16-bit load each per row block).
// The launcher guarantees: N % (16 * NB) == 0, (K / KC) % (WK * PF) == 0, group a power-of-two multiple of KC or
// per channel, x rows 16-byte aligned.
// WF: 0 integer codes; 1 floating-point codes (e4m3) with one scale of x's type per channel; 2 e2m1 codes with e8m0
// scales per 32 k, a row's scale bytes contiguous: a lane's 32 weights of a chunk are exactly one group, so its scale
// is one byte per chunk, fetched with the weights like the 16-bit scales of the other forms.
// WF 3: the fp8 block-scale matmul (quant_batch_matmul_v3, G-B / B-B) with 17 .. 128 rows (MB = 4 up to 64 rows, else 8): x is x1 widened to fp16 by a
// pre-step, w is x2 in e4m3, widened in registers without a scale (exact products); a slab of x is exactly one
// 128-element scale block (WK = 2 chunks of 64), each wave chains its chunk's two instructions from a zero accumulator
// and folds the partial block sum in with one fused multiply-add by s1[m, kb] * s2[kb, n / 128] -- the products of the
// two scales for all blocks and the slab's rows are laid down in LDS once per workgroup (its 128 columns lie in one
// scale block of w).  The output type is the call's (bf16, fp16 or fp32).
// WF 4: the fp8 row / column scale form (K-C, K-T) of the same operands: one chain over all of K, and the epilogue
// computes (sum * x2Scale[n]) * x1Scale[m] + bias[n] (bs2 / bs1 with element strides bs2_cs / bs1_rs of 0 or 1).
// SLDS (integer codes, a row's scales contiguous, power-of-two group count): the workgroup lays all scales and offsets of
// its columns down in LDS once, one 32-bit word (scale | offset << 16) per column and group, instead of fetching two
// 16-bit values per row block and chunk from global memory.  Such a load is one instruction per 16-bit value and touches
// 16 cache lines (one per weight row): at 8192 x 28672 with groups of 128 they were half of all the cache-line requests
// of the loop (512 of 1024 per slab and CU, against about 0.45 requests per clock that a CU's texture path takes) --
// more than weights and x together; per-wave timestamps showed the waves stalled in the issue of their memory
// instructions (1180 of 4120 clocks per slab) and at the barrier behind them.
template <int XDT, int WBITS, int MB, int NB, int WN, int WK, bool HAS_OFF, int WF = 0, bool SLDS = false, bool KSP = false>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2))) void wqmm_rows_kernel(WqParams p)
{
    static_assert(!KSP || WF <= 4, "K in segments: the weight-only forms and the fp8 forms");
    static_assert(WN * WK == 8, "eight waves");
    static_assert(!SLDS || WF == 0 || WF == 2, "the scale table serves the integer forms and the e8m0 bytes of e2m1 codes");
    static_assert(WF == 0 || !HAS_OFF, "floating-point weight codes have no offset");
    static_assert(WF != 2 || WBITS == 4 || (WBITS == 8 && WK == 2), "e8m0 group scales: e2m1 codes, or e4m3 codes on the instances with two K waves");
    static_assert(WF != 3 || (WBITS == 8 && XDT == DT_F16 && WK == 2 && NB == 2), "the block-scale form: fp16 x, e4m3 w, a slab per 128-block");
    static_assert(WF != 4 || (WBITS == 8 && XDT == DT_F16 && !HAS_OFF), "the row / column scale form: fp16 x, e4m3 w");
    constexpr int NT = 512;
    if (p.m_slab > 0) {   // several row slabs in one launch: this workgroup's is number blockIdx.y
        p.m_base += (int64_t)blockIdx.y * p.m_slab;
        const int64_t left = p.m_end - p.m_base;
        p.m_rows = left < p.m_slab ? left : p.m_slab;
    }
    // More than 128 rows of x (MB = 12: up to 192, MB = 16: up to 256) with 4-bit weights: a lane's weight piece is 8 bytes instead of 16 (HP), so that a chunk is
    // 64 k per wave like an 8-bit one and two slab buffers of 256 rows fit the LDS (2 x 64 KB).  (Half-chunk slabs under
    // 16-byte pieces were built first: the wait for a chunk's second slab is a wait for everything older, the weight
    // fetch just issued included -- loads return in order --, and the 256-row instance ran at 224 us against the tile
    // kernel's 167.)
    constexpr bool HP = MB > 8 && WBITS == 4;
    constexpr int PB = HP ? 8 : 16;                // bytes of a lane's weight piece
    constexpr int KCH = 4 * (128 / WBITS);         // the chunk the launcher counts groups in (cpg_shift)
    constexpr int KPL = PB * 8 / WBITS, KC = 4 * KPL, STEPS = KC / 32;
    constexpr int PF = MB > 8 ? 4 : 8 / NB;   // of this wave's chunks in flight per row block (a chunk is 500 to 1000 clocks of MFMA work here)
    constexpr int XH = 1;
    constexpr int PPH = KPL / 8 / XH;    // 16-byte pieces of x per lane group and slab (= K steps per slab)
    constexpr int KX = WK * KC;          // k per chunk of the workgroup (all WK waves)
    constexpr int XROW = KX * 2 / XH;    // LDS row pitch (bytes)
    constexpr int XPR = KX / 8 / XH;     // 16-byte pieces per x row per slab
    constexpr int XBUF = 16 * MB * XROW; // one slab buffer
    constexpr int XITEMS = 16 * MB * XPR / NT;
    constexpr int NBL = (WF >= 3 || WF == 1 || SLDS) ? NB : NB * (HAS_OFF ? 3 : 2);   // loads of one weight fetch
    constexpr int LDS_MAIN = (2 * XBUF > WN * (WK - 1) * NB * MB * 4 * 64 * 4) ? 2 * XBUF : WN * (WK - 1) * NB * MB * 4 * 64 * 4;
    static_assert((16 * MB * XPR) % NT == 0 && XPR >= 16 && PF >= 2 && PPH >= 1 && STEPS == PPH * XH, "staging and prefetch shape");
    static_assert(MB <= 8 || (WF == 0 && SLDS) || WF == 1 || WF == 2, "the 192- / 256-row instances: integer codes with the scale table in LDS, or floating-point codes");
    static_assert(!(SLDS && WF == 2 && MB > 8) || WK == 2, "8-byte pieces: byte position of a lane's e8m0 scale inside the table word");
    // a lane's piece holds half a group of 32 codes (8-byte pieces of e2m1 codes, 16-byte pieces of e4m3 codes): two lane
    // groups share an e8m0 byte, a chunk of the wave holds two bytes and the table word of 128 k serves the chunks of both K waves
    constexpr bool E8H = (MB > 8 && WBITS == 4) || (WF == 2 && WBITS == 8);
    // K in segments: this workgroup's is number blockIdx.z.  Segments are whole units of p.kunit k (whole slabs of x and
    // whole groups), as equal as that allows, the longer ones first.  From here on p.K is the segment's length and x, w, the scales and
    // offsets start at the segment; a row of x keeps its pitch ldx.
    // (KSP instantiations; the others keep p as it came)
    const int64_t ldx = p.K;
    constexpr bool ksplit = KSP;
    if constexpr (KSP) {
        {
            const int z = (int)blockIdx.z, units = (int)(p.K / p.kunit), base = units / p.ksplit, rem = units % p.ksplit;
            const int64_t k0 = (int64_t)(z * base + (z < rem ? z : rem)) * p.kunit;
            p.x += k0;
            p.w += k0 * WBITS / 8;
            if constexpr (WF == 2) p.scale = (const uint16_t*)((const uint8_t*)p.scale + k0 / 32);   // one e8m0 byte per 32 k
            else if constexpr (WF == 3) {   // the block scales of the segment's first 128-block
                p.bs1 += (k0 / 128) * p.bs1_cs;
                p.bs2 += (k0 / 128) * p.bs2_rs;
            }
            else if (p.group < p.K) {
                const int64_t g0 = (k0 / p.group) * p.s_rs;
                p.scale += g0;
                if constexpr (HAS_OFF) p.offset += g0;
            }
            p.K = (int64_t)(base + (z < rem ? 1 : 0)) * p.kunit;
        }
    }
    extern __shared__ __attribute__((aligned(16))) char sx[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave / WK, wk = wave % WK;
    const int nrow = lane & 15, g = lane >> 4;
    int64_t n0 = ((int64_t)blockIdx.x * WN + wn) * (16 * NB);
    const bool n_ok = n0 < p.N;
    if (!n_ok) n0 = p.N - 16 * NB;       // a wave past the edge recomputes the last columns and stores nothing
    const int Ki = (int)p.K;
    const int NSLAB = Ki / KX;           // = chunks per wave
    const int rows = (int)p.m_rows;

    const uint8_t* wptr = p.w + (n0 + nrow) * p.ldw + g * PB + wk * (4 * PB);
    const int64_t wblk = 16 * p.ldw;     // bytes between the row blocks of a wave
    const uint16_t* srow = p.scale + (n0 + nrow) * p.s_cs;
    const uint16_t* orow = HAS_OFF ? p.offset + (n0 + nrow) * p.s_cs : nullptr;
    const int64_t sblk = 16 * p.s_cs;
    // WF 2: the byte of this lane's group in chunk 0 (8-byte pieces: a lane's 16 weights are half a group, two lanes share a byte)
    const uint8_t* srow8 = (const uint8_t*)p.scale + (n0 + nrow) * p.s_cs + (E8H ? g >> 1 : g);

    // x copies: instruction `it` of this thread fills LDS piece it*NT + tid of the buffer, i.e. position
    // (it*NT + tid) % XPR of row (it*NT + tid) / XPR, with the row's piece position ^ (row % 16)
    // Which 16-byte piece of a slab row sits where.  A 16-byte-per-lane LDS read is served 16 lanes at a time, two passes
    // per half-wave; measured with address patterns on this chip, the pass of lane l inside its half-wave is
    // bit 4 of l xor bit 2 of l (lanes 0-3, 8-11, 20-23, 28-31 go together), and a read runs at the full 256 bytes per
    // clock only if the 16 lanes of every pass hit 16 different 16-byte columns of the 256-byte bank row.  Here lane
    // l = 16 g + row reads piece (16 wk + 4 g + s) ^ row of a 512-byte row: lanes (g, row) and (g ^ 1, row ^ 4) share a pass
    // and, since bit 2 of the piece number is bit 0 of g, a column -- half the LDS rate.  So rows of 32 pieces store piece P
    // at position swap24(P) ^ (row % 16), bits 2 and 4 of the piece number exchanged: bit 2 of the position is then
    // wk ^ bit 2 of the row, the same for both lane groups of a half-wave, and the two passes split the columns evenly.
    constexpr bool SWAP24 = XPR == 32 && KPL == 32;
    auto piece_of_pos = [](int q) { return SWAP24 ? ((q & ~0x14) | ((q & 4) << 2) | ((q & 16) >> 2)) : q; };   // (its own inverse)
    // Byte offsets from the slab's first row at K position 0 (the launcher keeps rows * K * 2 below 4 GB).  Rows past the
    // last one repeat it.  With 16 pieces per slab row an instruction covers 32 whole rows and a thread keeps its piece
    // position, so offset(it) = min(offset(0) + it * 32 rows, offset of the same piece in the last row): two registers
    // instead of XITEMS (the 256-row instance has none to spare).
    constexpr bool XLIN = XPR == 16;
    uint32_t xsrc[XLIN ? 1 : XITEMS];
    uint32_t xsrc_max = 0;
    const uint16_t* xbase = p.x + p.m_base * ldx;
    const uint32_t xpitch = (uint32_t)ldx;
    (void)xsrc_max;
#pragma unroll
    for (int it = 0; it < (XLIN ? 1 : XITEMS); it++) {
        const int L = it * NT + tid;
        const int r = L / XPR, pos = L % XPR;
        const int rr = r < rows ? r : rows - 1;
        // piece q of a slab row: wave column q / (XPR / WK), lane group (q % (XPR / WK)) / PPH, K step q % PPH of the slab; in x
        // that is piece wk * (KC / 8) + g * (KPL / 8) + step of the chunk (the identity when a slab holds whole chunks)
        const int q = piece_of_pos(pos ^ (r & 15));
        const int src_piece = (q / (XPR / WK)) * (KC / 8) + ((q % (XPR / WK)) / PPH) * (KPL / 8) + q % PPH;
        xsrc[it] = ((uint32_t)rr * xpitch + (uint32_t)(src_piece * 8)) * 2u;
        if constexpr (XLIN) {
            xsrc[0] = ((uint32_t)r * xpitch + (uint32_t)(src_piece * 8)) * 2u;   // (r may lie past the last row: the minimum below puts it back)
            xsrc_max = ((uint32_t)(rows - 1) * xpitch + (uint32_t)(src_piece * 8)) * 2u;
        }
    }
    auto xsrc_at = [&](int it) -> uint32_t {
        if constexpr (XLIN) {
            const uint32_t o = xsrc[0] + (uint32_t)it * (uint32_t)(NT / XPR) * xpitch * 2u;
            return o < xsrc_max ? o : xsrc_max;
        } else {
            return xsrc[it];
        }
    };
    auto issue_x = [&](int slab) {   // slab = chunk * XH + half
        const uint32_t dst = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)sx + (slab & 1) * XBUF + wave * 1024;
        const uint16_t* src = xbase + (int64_t)(slab / XH) * KX + (slab % XH) * (PPH * 8);
        // (readfirstlane returns a signed int: each half goes through uint32_t before the halves are joined)
        const uint32_t sb_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)src);
        const uint32_t sb_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uintptr_t)src >> 32));
        const uint64_t sb = ((uint64_t)sb_hi << 32) | (uint64_t)sb_lo;
#pragma unroll
        for (int it = 0; it < XITEMS; it++) copy16_sbase((const void*)sb, xsrc_at(it), dst + it * NT * 16);
    };
    // the same in parts: copies it0 .. it0 + n - 1
    auto issue_x_part = [&](int slab, int it0, int n) {
        const uint32_t dst = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)sx + (slab & 1) * XBUF + wave * 1024;
        const uint16_t* src = xbase + (int64_t)(slab / XH) * KX + (slab % XH) * (PPH * 8);
        const uint32_t sb_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)src);
        const uint32_t sb_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uintptr_t)src >> 32));
        const uint64_t sb = ((uint64_t)sb_hi << 32) | (uint64_t)sb_lo;
#pragma unroll
        for (int it = it0; it < it0 + n; it++)
            if (it < XITEMS) copy16_sbase((const void*)sb, xsrc_at(it), dst + it * NT * 16);
    };
    // LDS byte offset of this lane's column operand inside a buffer, per 16-row block of x, at K step 0 (the lane's
    // weights cover k = g*KPL .. +KPL of the chunk, step s the 8 at 8s); step s is s pieces further on, which the
    // swizzle turns into an exclusive-or with 16s
    // (row block b of x lies b * 16 * XROW further on: an immediate offset of the read, since the swizzle only looks at the row's low four bits)
    const int xoff0 = nrow * XROW + (piece_of_pos(wk * (XPR / WK) + g * PPH) ^ nrow) * 16;
    auto xoff_at = [&](int b, int s) { return (xoff0 ^ (16 * s)) + b * (16 * XROW); };

    v4f acc[NB][MB];
#pragma unroll
    for (int q = 0; q < NB; q++)
#pragma unroll
        for (int b = 0; b < MB; b++) acc[q][b] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
    const DqConst dqc = make_dq_const();

    // WF 3: sct[kb][r] = s1[row r of the slab, kb] * s2[kb, this workgroup's column block], behind the x buffers (and the
    // partial sums that take their place at the end); complete behind the loop's first barrier
    float* sct = (float*)(sx + LDS_MAIN);
    if constexpr (WF == 3) {
        const int64_t nbw = ((int64_t)blockIdx.x * (16 * NB * WN)) / 128;
        for (int i = tid; i < NSLAB * 16 * MB; i += NT) {
            const int kb = i / (16 * MB), r = i - kb * (16 * MB);
            const int64_t m = p.m_base + (r < rows ? r : rows - 1);
            sct[i] = p.bs1[(m / p.bs_gsm) * p.bs1_rs + kb * p.bs1_cs] * p.bs2[kb * p.bs2_rs + nbw * p.bs2_cs];
        }
    }

    // SLDS: word (row rw of the workgroup's 16 NB WN columns, group gi) at stab[rw * P + (gi ^ swizzle(rw))], P = the power of
    // two at or above the groups per row; the swizzle (4 * (rw % 16), kept below P) spreads the 16 rows that one read touches
    // over the banks.  The table is complete behind the loop's first barrier.
    uint32_t* stab = (uint32_t*)(sx + LDS_MAIN);
    // groups of this workgroup's K (the last one may be short)
    const int sG = p.cpg_shift >= 31 ? 1 : (int)(((p.K / KCH) + (1ll << p.cpg_shift) - 1) >> p.cpg_shift);
    const int sP = sG <= 1 ? 1 : 1 << (32 - __builtin_clz((unsigned)(sG - 1)));    // a table row's pitch: the power of two at or above
    const int cpg_shift = p.cpg_shift >= 31 ? 31 : p.cpg_shift + (HP ? 1 : 0);   // chunks of this kernel per group
    int stab_row[NB], stab_sw[NB];
    (void)stab; (void)sG; (void)sP; (void)stab_row; (void)stab_sw;
    if constexpr (SLDS) {
        constexpr int RW = 16 * NB * WN;
        for (int i = tid; i < RW * sG; i += NT) {
            const int rw = i / sG, gi = i - rw * sG;
            int64_t nb0 = ((int64_t)blockIdx.x * WN + rw / (16 * NB)) * (16 * NB);
            if (nb0 >= p.N) nb0 = p.N - 16 * NB;
            const int64_t n = nb0 + rw % (16 * NB);
            uint32_t w;
            if constexpr (WF == 2) w = *(const uint32_t*)((const uint8_t*)p.scale + n * p.s_cs + 4 * gi);   // four e8m0 bytes: 128 k
            else w = p.scale[n * p.s_cs + gi];
            if constexpr (HAS_OFF) w |= (uint32_t)p.offset[n * p.s_cs + gi] << 16;
            stab[rw * sP + (gi ^ (((rw & 15) << 2) & (sP - 1)))] = w;
        }
#pragma unroll
        for (int q = 0; q < NB; q++) {
            const int rw = wn * (16 * NB) + 16 * q + nrow;
            stab_row[q] = rw * sP;
            stab_sw[q] = ((rw & 15) << 2) & (sP - 1);
        }
    }

    // WF 1: one scale per channel, read once.  WF 2 with the table: a table word holds the e8m0 bytes of 128 k; this lane's
    // 32 (8-byte pieces: 16) codes of a chunk belong to byte g of the chunk's word (g / 2 of the half that the chunk is)
    uint16_t sch[NB];
    const int e8sh = 8 * (E8H ? 2 * wk + (g >> 1) : g);
    (void)sch; (void)e8sh;
    if constexpr (WF == 1) {
#pragma unroll
        for (int q = 0; q < NB; q++) sch[q] = srow[q * sblk];
    }
    v4i wq[PF][NB];
    uint16_t sq[PF][NB], oq[PF][NB];
    auto fetch = [&](int j, int cw) {   // chunk cw of this wave (chunk cw * WK + wk of the row) into slot j
        const int64_t so = (int64_t)((cw * WK + wk) >> cpg_shift) * p.s_rs;
#pragma unroll
        for (int q = 0; q < NB; q++) {
            if constexpr (HP) {
                const v2i t = *(const v2i*)(wptr + q * wblk + (int64_t)cw * (WK * 4 * PB));
                wq[j][q] = (v4i){t[0], t[1], 0, 0};
            } else {
                wq[j][q] = *(const v4i*)(wptr + q * wblk + (int64_t)cw * (WK * 64));
            }
            if constexpr (SLDS) { sq[j][q] = 0; oq[j][q] = 0; continue; }
            if constexpr (WF >= 3 || WF == 1) sq[j][q] = 0;
            else if constexpr (WF == 2) sq[j][q] = srow8[q * sblk + (cw * WK + wk) * (KC / 32)];
            else sq[j][q] = srow[q * sblk + so];
            if constexpr (HAS_OFF) oq[j][q] = orow[q * sblk + so];
            else oq[j][q] = 0;
        }
    };
    // pieces of a chunk's work (all forms but the block-scale one, which has its own order below)
    v4i aop[NB];                   // the dequantised weights of the K step about to be multiplied
    auto load_sow = [&](int cw, uint32_t (&sow)[NB]) {
        if constexpr (SLDS) {
            const int gi = (cw * WK + wk) >> cpg_shift;
#pragma unroll
            for (int q = 0; q < NB; q++) {
                sow[q] = stab[stab_row[q] + (gi ^ stab_sw[q])];
                if constexpr (WF == 2) sow[q] = bits_x<XDT>(e8m0_to_f32((sow[q] >> e8sh) & 0xFFu));
            }
        } else if constexpr (WF == 1) {
#pragma unroll
            for (int q = 0; q < NB; q++) sow[q] = sch[q];
        } else {
#pragma unroll
            for (int q = 0; q < NB; q++) sow[q] = 0;
        }
    };
    auto dequant_step = [&](int j, int s, const uint32_t (&sow)[NB], v4i (&out)[NB]) {
#pragma unroll
        for (int q = 0; q < NB; q++) {
            if constexpr (WF == 0 && SLDS) out[q] = dequant8<XDT, WBITS, HAS_OFF, true>(wq[j][q], s, (uint16_t)sow[q], (uint16_t)(sow[q] >> 16), dqc);
            else if constexpr (WF == 0) out[q] = dequant8<XDT, WBITS, HAS_OFF, true>(wq[j][q], s, sq[j][q], oq[j][q], dqc);
            else if constexpr (WF == 1 || (WF == 2 && SLDS)) out[q] = dequant8_float<XDT, WBITS, true>(wq[j][q], s, (uint16_t)sow[q]);
            else if constexpr (WF == 4) {
                typedef _Float16 h2v __attribute__((ext_vector_type(2)));
                const uint32_t d0 = (uint32_t)wq[j][q][2 * s], d1 = (uint32_t)wq[j][q][2 * s + 1];
                const h2v w0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d0, 1.0f, false), w1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d0, 1.0f, true);
                const h2v w2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d1, 1.0f, false), w3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d1, 1.0f, true);
                out[q] = (v4i){(int)__builtin_bit_cast(uint32_t, w0), (int)__builtin_bit_cast(uint32_t, w1),
                               (int)__builtin_bit_cast(uint32_t, w2), (int)__builtin_bit_cast(uint32_t, w3)};
            }
            else out[q] = dequant8_float<XDT, WBITS, true>(wq[j][q], s, bits_x<XDT>(e8m0_to_f32(sq[j][q])));
        }
    };
    auto read_frags = [&](const char* xs, int s, v4i (&bops)[MB]) {
#pragma unroll
        for (int b = 0; b < MB; b++) bops[b] = *(const v4i*)(xs + xoff_at(b, s));
    };
    auto mma_step = [&](const v4i (&a)[NB], const v4i (&bops)[MB]) {
#pragma unroll
        for (int b = 0; b < MB; b++)
#pragma unroll
            for (int q = 0; q < NB; q++) {
                if constexpr (XDT == DT_F16) acc[q][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a[q]), __builtin_bit_cast(v8h, bops[b]), acc[q][b], 0, 0, 0);
                else acc[q][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a[q]), __builtin_bit_cast(v8bf, bops[b]), acc[q][b], 0, 0, 0);
            }
    };
    auto read_frags_part = [&](auto b0c, const char* xs, int s, v4i (&bops)[MB / 4]) {
        constexpr int B0 = decltype(b0c)::value;
#pragma unroll
        for (int b = 0; b < MB / 4; b++) bops[b] = *(const v4i*)(xs + xoff_at(B0 + b, s));
    };
    auto mma_part = [&](auto b0c, const v4i (&a)[NB], const v4i (&bops)[MB / 4]) {
        constexpr int B0 = decltype(b0c)::value;
#pragma unroll
        for (int b = 0; b < MB / 4; b++)
#pragma unroll
            for (int q = 0; q < NB; q++) {
                if constexpr (XDT == DT_F16) acc[q][B0 + b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a[q]), __builtin_bit_cast(v8h, bops[b]), acc[q][B0 + b], 0, 0, 0);
                else acc[q][B0 + b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a[q]), __builtin_bit_cast(v8bf, bops[b]), acc[q][B0 + b], 0, 0, 0);
            }
    };
#pragma unroll
    for (int j = 0; j < PF; j++) fetch(j, (MB > 8 || j < NSLAB) ? j : NSLAB - 1);   // (the 192- / 256-row instances: whole rounds)
    issue_x(0);
    wait_vmcnt<0>();

    // chunk cw of this wave, held in prefetch slot j
    auto chunk_step = [&](auto jc, auto lastc, const int cw) {
            constexpr int j = decltype(jc)::value;
            constexpr bool LAST_ROUND = decltype(lastc)::value;   // a step of the shorter round behind the loop
            uint32_t sow[NB];
#pragma unroll
            for (int h = 0; h < XH; h++) {
            // this thread's copies of the slab have landed (behind a chunk's first slab only the weight fetch issued after
            // them may be in flight; behind its second one nothing was issued)
            // (behind the loop everything: no refill follows a step there -- nothing would read it --, so the count of
            // loads behind the copies is not NBL)
            if (h > 0 || LAST_ROUND) wait_vmcnt<0>();
            else if (cw > 0) wait_vmcnt<NBL>();
            __syncthreads();   // the slab is complete and visible; every wave has finished the one before
            const int sl = cw * XH + h;
            // 256 rows: the slab's copies go out in pairs between the first groups of matrix instructions instead of in one
            // burst behind the barrier (eight waves x eight copies of 1 KB fill the memory pipeline's queue, and every wave
            // stood in front of its first matrix instruction until its last copy was accepted: a quarter of the slab's time)
            constexpr bool SPREAD = MB > 8 || (WF == 0 && PPH >= 2);
            const bool more_x = sl + 1 < NSLAB * XH;
            if (!SPREAD && more_x) issue_x(sl + 1);
            const char* xs = sx + (sl & 1) * XBUF;
            if constexpr (WF != 3) { if (h == 0) load_sow(cw, sow); }   // (behind the barrier: the first one also completes the scale table)
            if constexpr (WF == 3) {
                // this wave's half of block cw: two instructions per fragment pair from zero, then the fold
                v4i aw[NB][2];
#pragma unroll
                for (int q = 0; q < NB; q++) {
                    const v4i pc = wq[j][q];
#pragma unroll
                    for (int s = 0; s < 2; s++) {
                        typedef _Float16 h2v __attribute__((ext_vector_type(2)));
                        const uint32_t d0 = (uint32_t)pc[2 * s], d1 = (uint32_t)pc[2 * s + 1];
                        const h2v w0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d0, 1.0f, false), w1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d0, 1.0f, true);
                        const h2v w2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d1, 1.0f, false), w3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d1, 1.0f, true);
                        aw[q][s] = (v4i){(int)__builtin_bit_cast(uint32_t, w0), (int)__builtin_bit_cast(uint32_t, w1),
                                         (int)__builtin_bit_cast(uint32_t, w2), (int)__builtin_bit_cast(uint32_t, w3)};
                    }
                }
                const float* scr = sct + cw * (16 * MB) + nrow;
                if constexpr (MB > 4) {
                    // 128 rows: two row blocks at a time, and the fold of a pair rides behind the next pair's matrix
                    // instructions.  The empty asm statements pin each fold where it is written: left alone the compiler
                    // postpones the folds, keeps all eight blocks' partial sums alive and spills the weight prefetch.
                    v4f tp[2][NB];
                    float scp[2] = {0.0f, 0.0f};
#pragma unroll
                    for (int bp = 0; bp <= MB / 2; bp++) {
                        v4f tc[2][NB];
                        float scc[2] = {0.0f, 0.0f};
                        if (bp < MB / 2) {
#pragma unroll
                            for (int h = 0; h < 2; h++) {
                                const int b = 2 * bp + h;
                                const v4i b0 = *(const v4i*)(xs + xoff_at(b, 0)), b1 = *(const v4i*)(xs + xoff_at(b, 1));
                                scc[h] = scr[16 * b];
#pragma unroll
                                for (int q = 0; q < NB; q++)
                                    tc[h][q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, aw[q][0]), __builtin_bit_cast(v8h, b0), (v4f){0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
#pragma unroll
                                for (int q = 0; q < NB; q++)
                                    tc[h][q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, aw[q][1]), __builtin_bit_cast(v8h, b1), tc[h][q], 0, 0, 0);
                            }
                        }
                        if (bp > 0) {
#pragma unroll
                            for (int h = 0; h < 2; h++)
#pragma unroll
                                for (int q = 0; q < NB; q++) {
                                    v4f& a = acc[q][2 * (bp - 1) + h];
#pragma unroll
                                    for (int i = 0; i < 4; i++) a[i] = __builtin_fmaf(tp[h][q][i], scp[h], a[i]);
                                    asm volatile("" : "+v"(a));
                                }
                        }
#pragma unroll
                        for (int h = 0; h < 2; h++) {
                            scp[h] = scc[h];
#pragma unroll
                            for (int q = 0; q < NB; q++) tp[h][q] = tc[h][q];
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
#pragma unroll
                for (int b = 0; b < MB; b++) {
                    const v4i b0 = *(const v4i*)(xs + xoff_at(b, 0)), b1 = *(const v4i*)(xs + xoff_at(b, 1));
                    const float sc = scr[16 * b];
                    v4f t[NB];
#pragma unroll
                    for (int q = 0; q < NB; q++)
                        t[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, aw[q][0]), __builtin_bit_cast(v8h, b0), (v4f){0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
#pragma unroll
                    for (int q = 0; q < NB; q++)
                        t[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, aw[q][1]), __builtin_bit_cast(v8h, b1), t[q], 0, 0, 0);
#pragma unroll
                    for (int q = 0; q < NB; q++)
#pragma unroll
                        for (int i = 0; i < 4; i++) acc[q][b][i] = __builtin_fmaf(t[q][i], sc, acc[q][b][i]);
                }
                }
            }
            if constexpr (WF != 3) {
                // A slab's work: per K step the x fragments are requested first, so that they arrive in the shadow of the
                // step's dequantisation (vector ALU) instead of each pair of matrix instructions waiting for a read issued
                // just in front of it.
#pragma unroll
                for (int s = 0; s < PPH; s++) {
                    if constexpr (MB <= 8) {
                        v4i bops[MB];
                        read_frags(xs, s, bops);
                        __builtin_amdgcn_sched_barrier(0);
                        if constexpr (SPREAD) {   // the next slab's copies in two halves, behind the fragment requests of the first two steps
                            constexpr int CPH = (XITEMS + 1) / 2;
                            if (s < 2 && more_x) issue_x_part(sl + 1, s * CPH, CPH);
                        }
                        dequant_step(j, h * PPH + s, sow, aop);
                        mma_step(aop, bops);
                    } else {
                        // 256 rows: the fragments in four groups of four, two groups requested ahead of the matrix
                        // instructions that use them (all sixteen at once would need 64 registers beside 128 sums)
                        constexpr int Q = MB / 4;
                        v4i b0[Q], b1[Q], b2[Q], b3[Q];
                        read_frags_part(std::integral_constant<int, 0>{}, xs, s, b0);
                        read_frags_part(std::integral_constant<int, Q>{}, xs, s, b1);
                        __builtin_amdgcn_sched_barrier(0);
                        dequant_step(j, h * PPH + s, sow, aop);
                        __builtin_amdgcn_sched_barrier(0);
                        constexpr int CPG = (XITEMS + 3) / 4;   // copies behind each of the first step's four groups
                        if (s == 0 && more_x) issue_x_part(sl + 1, 0, CPG);
                        mma_part(std::integral_constant<int, 0>{}, aop, b0);
                        read_frags_part(std::integral_constant<int, 2 * Q>{}, xs, s, b2);
                        if (s == 0 && more_x) issue_x_part(sl + 1, CPG, CPG);
                        __builtin_amdgcn_sched_barrier(0);
                        mma_part(std::integral_constant<int, Q>{}, aop, b1);
                        read_frags_part(std::integral_constant<int, 3 * Q>{}, xs, s, b3);
                        if (s == 0 && more_x) issue_x_part(sl + 1, 2 * CPG, CPG);
                        __builtin_amdgcn_sched_barrier(0);
                        mma_part(std::integral_constant<int, 2 * Q>{}, aop, b2);
                        if (s == 0 && more_x) issue_x_part(sl + 1, 3 * CPG, CPG);
                        __builtin_amdgcn_sched_barrier(0);
                        mma_part(std::integral_constant<int, 3 * Q>{}, aop, b3);
                    }
                }
            }
            }
            if constexpr (!LAST_ROUND) {
                const int nx = cw + PF;
                fetch(j, nx < NSLAB ? nx : NSLAB - 1);   // past the end: a harmless reload of the last chunk
            }
    };
    // whole rounds of PF chunks, then the chunks of a last, shorter round (the same count for all waves).  The shorter round
    // stands behind the loop, not as an exit inside it: with the exit inside, the 256-row instance spilled 700 bytes per lane
    // and ran eight times as long.  The 192- / 256-row instances have whole rounds only (their launcher sees to it).
    int c0 = 0;
    for (; MB > 8 ? c0 < NSLAB : c0 + PF <= NSLAB; c0 += PF) {
        chunk_step(std::integral_constant<int, 0>{}, std::false_type{}, c0);
        chunk_step(std::integral_constant<int, 1>{}, std::false_type{}, c0 + 1);
        if constexpr (PF > 2) {
            chunk_step(std::integral_constant<int, 2>{}, std::false_type{}, c0 + 2);
            chunk_step(std::integral_constant<int, 3>{}, std::false_type{}, c0 + 3);
        }
        static_assert(PF == 2 || PF == 4, "prefetch slots");
    }
    if constexpr (MB <= 8) {
        if (c0 < NSLAB) chunk_step(std::integral_constant<int, 0>{}, std::true_type{}, c0);
        if constexpr (PF > 2) {
            if (c0 + 1 < NSLAB) chunk_step(std::integral_constant<int, 1>{}, std::true_type{}, c0 + 1);
            if (c0 + 2 < NSLAB) chunk_step(std::integral_constant<int, 2>{}, std::true_type{}, c0 + 2);
        }
    }

    if constexpr (WK > 1) {
        __syncthreads();   // x is no longer needed: its buffers take the partial sums
        float* red = (float*)sx;
        if (wk > 0) {
#pragma unroll
            for (int q = 0; q < NB; q++)
#pragma unroll
                for (int b = 0; b < MB; b++)
#pragma unroll
                    for (int i = 0; i < 4; i++) red[((((wn * (WK - 1) + (wk - 1)) * NB + q) * MB + b) * 4 + i) * 64 + lane] = acc[q][b][i];
        }
        __syncthreads();
        if (wk > 0) return;
#pragma unroll
        for (int j = 0; j < WK - 1; j++)
#pragma unroll
            for (int q = 0; q < NB; q++)
#pragma unroll
                for (int b = 0; b < MB; b++)
#pragma unroll
                    for (int i = 0; i < 4; i++) acc[q][b][i] = acc[q][b][i] + red[((((wn * (WK - 1) + j) * NB + q) * MB + b) * 4 + i) * 64 + lane];
    }

    // D'[row = weight row n][col = x row m]: lane holds col m = lane%16, rows n = 4*(lane/16) + i
    if (!n_ok) return;
#pragma unroll
    for (int q = 0; q < NB; q++) {
#pragma unroll
        for (int b = 0; b < MB; b++) {
            const int r = 16 * b + nrow;
            if (r >= rows) continue;
            const int64_t m = p.m_base + r;
            const int64_t nn0 = n0 + 16 * q + 4 * g;
            if constexpr (ksplit) {   // this segment's partial sums; bias and rounding follow in the kernel that adds the segments
                *(v4f*)(p.part + ((int64_t)blockIdx.z * p.M + m) * p.N + nn0) = acc[q][b];
                continue;
            }
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                v[i] = acc[q][b][i];
                if constexpr (WF == 4) v[i] = (v[i] * p.bs2[(nn0 + i) * p.bs2_cs]) * p.bs1[m * p.bs1_rs];
                if (p.bias) v[i] = v[i] + load_scalar_as_f32(p.bias, p.bias_dt, nn0 + i);
                if constexpr (XDT == DT_BF16) v[i] = bf16_to_f32(bf16_bits(v[i]));   // the golden rounds bf16 results twice (a no-op)
            }
            if constexpr (WF >= 3) {
                const v4f vv = {v[0], v[1], v[2], v[3]};
                if (p.bs_out_dt == DT_F32) *(v4f*)((float*)p.y + m * p.N + nn0) = vv;
                else *(v4us*)(p.y + m * p.N + nn0) = p.bs_out_dt == DT_BF16 ? pack4_b16<DT_BF16>(vv) : pack4_b16<DT_F16>(vv);
                continue;
            }
            const v4us o = {bits_x<XDT>(v[0]), bits_x<XDT>(v[1]), bits_x<XDT>(v[2]), bits_x<XDT>(v[3])};
            *(v4us*)(p.y + m * p.N + nn0) = o;   // N % 16 == 0 here: 8-byte aligned
        }
    }
}

// ---- few rows of x (rows * K * 2 bytes fit in LDS): x is staged whole, once per workgroup ----
// The four waves of a workgroup share one block of 16 weight rows at a time and take one contiguous quarter of K
// each; partial sums meet in LDS in a fixed order.  A workgroup walks several row blocks (blockIdx.x, + gridDim.x,
// ...) and its weight stream never stops: the refills issued while the last chunks of one row block are consumed
// already fetch the first chunks of the next, so the memory latency is paid once per workgroup, not per row block.
template <int XDT, int WBITS, bool HAS_OFF, bool VSCALE>
__global__ __launch_bounds__(256, 2) void wqmm_resx_kernel(WqParams p)
{
    constexpr int KPL = 128 / WBITS, KC = 4 * KPL, STEPS = KC / 32;
    constexpr int PF = 8;   // weight pieces in flight per lane
    extern __shared__ __attribute__((aligned(16))) char sx[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wk = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nrow = lane & 15, g = lane >> 4;
    const int Ki = (int)p.K;
    const int NCW = Ki / (KC * 4);       // chunks per wave and row block; wave wk owns chunks wk*NCW .. wk*NCW+NCW-1
    const int cbase = wk * NCW;
    const int rows = (int)p.m_rows;
    const int xrow = Ki * 2 + 16;        // LDS row pitch in bytes
    const int nblocks = (int)((p.N + 15) / 16);
    float* red = (float*)(sx + (rows + 1) * xrow);   // [2][3 waves][4][64] partial sums, double buffered by row-block parity

    // per-lane stream pointers of a row block (rows past the edge of N re-read the last row)
    auto row_of = [&](int rb) { const int64_t n = (int64_t)rb * 16 + nrow; return n < p.N ? n : p.N - 1; };
    auto wptr_of = [&](int rb) { return p.w + row_of(rb) * p.ldw + g * 16 + (int64_t)cbase * 64; };
    int rb = blockIdx.x;
    const uint8_t* wptr = wptr_of(rb);
    const uint16_t* srow = p.scale + row_of(rb) * p.s_cs;
    const uint16_t* orow = HAS_OFF ? p.offset + row_of(rb) * p.s_cs : nullptr;

    // x: rows * K/8 pieces of 16 bytes.  The first four pieces of every thread are requested before the weight stream
    // starts (loads return in issue order, and these are cache hits that must not queue behind it) and are written to
    // LDS after the weight requests have gone out; further pieces (more than one row of 8192) follow.
    const int xpr = Ki / 8, xtotal = rows * xpr;
    auto x_piece = [&](int idx) {
        const int r = idx / xpr, c = idx - r * xpr;
        return *(const v4i*)(p.x + (p.m_base + r) * p.K + c * 8);
    };
    auto x_store = [&](int idx, v4i v) {
        const int r = idx / xpr, c = idx - r * xpr;
        if constexpr (WBITS == 4) {
            // halves [0..7] -> [0,4,1,5,2,6,3,7]: the order in which the nibble splicing yields pairs
            const uint32_t a0 = (uint32_t)v[0], a1 = (uint32_t)v[1], a2 = (uint32_t)v[2], a3 = (uint32_t)v[3];
            v = (v4i){(int)__builtin_amdgcn_perm(a2, a0, 0x05040100u), (int)__builtin_amdgcn_perm(a2, a0, 0x07060302u),
                      (int)__builtin_amdgcn_perm(a3, a1, 0x05040100u), (int)__builtin_amdgcn_perm(a3, a1, 0x07060302u)};
        }
        *(v4i*)(sx + r * xrow + c * 16) = v;
    };
    v4i xfirst[4];
#pragma unroll
    for (int i = 0; i < 4; i++) xfirst[i] = x_piece((i * 256 + tid) < xtotal ? (i * 256 + tid) : 0);
    // VSCALE: the 8 scales (offsets) of a super-step are loaded one super-step ahead, before that super-step's weight
    // refills, so that waiting for them never drains the younger weight loads (loads complete in issue order)
    constexpr int SV = PF / 8;   // register quads of 8 scales per super-step
    static_assert(PF % 8 == 0, "a super-step holds whole quads of scales");
    v4i sv[SV], ov[SV], svn[SV], ovn[SV];
#pragma unroll
    for (int h = 0; h < SV; h++) {
        sv[h] = ov[h] = svn[h] = ovn[h] = (v4i){0, 0, 0, 0};
        if constexpr (VSCALE) {
            if (8 * h < NCW) {
                svn[h] = *(const v4i*)(srow + cbase + 8 * h);
                if constexpr (HAS_OFF) ovn[h] = *(const v4i*)(orow + cbase + 8 * h);
            }
        }
    }
    v4i wq[PF];
    uint16_t sq[PF], oq[PF];
    auto fetch = [&](int j, const uint8_t* wp, const uint16_t* sr, const uint16_t* orw, int cw) {
        wq[j] = *(const v4i*)(wp + (int64_t)cw * 64);
        if constexpr (!VSCALE) {
            const int64_t so = (int64_t)((cbase + cw) >> p.cpg_shift) * p.s_rs;
            sq[j] = sr[so];
            if constexpr (HAS_OFF) oq[j] = orw[so];
        }
    };
#pragma unroll
    for (int j = 0; j < PF; j++) fetch(j, wptr, srow, orow, j < NCW ? j : NCW - 1);

#pragma unroll
    for (int i = 0; i < 4; i++)
        if (i * 256 + tid < xtotal) x_store(i * 256 + tid, xfirst[i]);
    for (int idx = 1024 + tid; idx < xtotal; idx += 256) x_store(idx, x_piece(idx));
    for (int c = tid; c < xrow / 16; c += 256) *(v4i*)(sx + rows * xrow + c * 16) = (v4i){0, 0, 0, 0};
    const int xoff = (nrow < rows ? nrow : rows) * xrow + g * KPL * 2 + cbase * (KC * 2);
    const DqConst dqc = make_dq_const();
    __syncthreads();

    for (int it = 0; rb < nblocks; it++) {
        const int rb_next = rb + (int)gridDim.x;
        const bool has_next = rb_next < nblocks;
        const uint8_t* wptr_n = has_next ? wptr_of(rb_next) : wptr;
        const uint16_t* srow_n = has_next ? p.scale + row_of(rb_next) * p.s_cs : srow;
        const uint16_t* orow_n = HAS_OFF ? (has_next ? p.offset + row_of(rb_next) * p.s_cs : orow) : nullptr;
        v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};

        // LAST: the refills of this super-step run past the row block's chunks into the next row block
        auto superstep = [&](int c0, auto last_tag) {
            constexpr bool LAST = decltype(last_tag)::value;
            if constexpr (VSCALE) {
#pragma unroll
                for (int h = 0; h < SV; h++) {
                    sv[h] = svn[h]; ov[h] = ovn[h];
                    // the quad of chunks c0 + PF + 8h ..: in this row block, or wrapped into the next one
                    const int cn = c0 + PF + 8 * h;
                    if (!LAST || cn < NCW) {
                        svn[h] = *(const v4i*)(srow + cbase + cn);
                        if constexpr (HAS_OFF) ovn[h] = *(const v4i*)(orow + cbase + cn);
                    } else if (cn - NCW < NCW) {
                        svn[h] = *(const v4i*)(srow_n + cbase + cn - NCW);
                        if constexpr (HAS_OFF) ovn[h] = *(const v4i*)(orow_n + cbase + cn - NCW);
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < PF; j++) {
                const int cw = c0 + j;
                if (LAST && cw >= NCW) continue;
                const char* xs = sx + xoff + cw * (KC * 2);
                uint16_t sb, ob = 0;
                if constexpr (VSCALE) {
                    sb = (uint16_t)((uint32_t)sv[j / 8][(j % 8) / 2] >> (16 * (j % 2)));
                    if constexpr (HAS_OFF) ob = (uint16_t)((uint32_t)ov[j / 8][(j % 8) / 2] >> (16 * (j % 2)));
                } else {
                    sb = sq[j];
                    if constexpr (HAS_OFF) ob = oq[j];
                }
#pragma unroll
                for (int s = 0; s < STEPS; s++) {
                    const v4i aop = dequant8<XDT, WBITS, HAS_OFF>(wq[j], s, sb, ob, dqc);
                    const v4i bop = *(const v4i*)(xs + 16 * s);
                    if constexpr (XDT == DT_F16) {
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, aop), __builtin_bit_cast(v8h, bop), acc, 0, 0, 0);
                    } else {
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, aop), __builtin_bit_cast(v8bf, bop), acc, 0, 0, 0);
                    }
                }
                if constexpr (LAST) {
                    // slot j next holds chunk cw + PF of this row block, or, past its end, the chunk of the next row block
                    // that the slot serves first: chunk j of its first super-step (not cw + PF - NCW: that is the same only
                    // when a row block is a whole number of super-steps)
                    const int nx = cw + PF;
                    if (nx < NCW) fetch(j, wptr, srow, orow, nx);
                    else fetch(j, wptr_n, srow_n, orow_n, j < NCW ? j : NCW - 1);
                } else {
                    fetch(j, wptr, srow, orow, cw + PF);
                }
            }
        };
        int c0 = 0;
        for (; c0 + 2 * PF <= NCW; c0 += PF) superstep(c0, std::false_type{});
        for (; c0 < NCW; c0 += PF) superstep(c0, std::true_type{});

        // fixed-order reduction of the four K quarters (one barrier per row block; the buffer alternates)
        float* rd = red + (it & 1) * (3 * 4 * 64);
        if (wk > 0) {
#pragma unroll
            for (int i = 0; i < 4; i++) rd[((wk - 1) * 4 + i) * 64 + lane] = acc[i];
        }
        __syncthreads();
        if (wk == 0) {
#pragma unroll
            for (int j = 0; j < 3; j++)
#pragma unroll
                for (int i = 0; i < 4; i++) acc[i] = acc[i] + rd[(j * 4 + i) * 64 + lane];
            if (nrow < rows) {
                const int64_t n0 = (int64_t)rb * 16;
                const int64_t m = p.m_base + nrow;
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int64_t nn = n0 + 4 * g + i;
                    v[i] = acc[i];
                    if (p.bias && nn < p.N) v[i] = v[i] + load_scalar_as_f32(p.bias, p.bias_dt, nn);
                    if constexpr (XDT == DT_BF16) v[i] = bf16_to_f32(bf16_bits(v[i]));
                }
                const int64_t nn0 = n0 + 4 * g;
                if (nn0 + 3 < p.N && (p.N % 4) == 0) {
                    const v4us o = {bits_x<XDT>(v[0]), bits_x<XDT>(v[1]), bits_x<XDT>(v[2]), bits_x<XDT>(v[3])};
                    *(v4us*)(p.y + m * p.N + nn0) = o;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (nn0 + i < p.N) p.y[m * p.N + nn0 + i] = bits_x<XDT>(v[i]);
                }
            }
        }
        rb = rb_next; wptr = wptr_n; srow = srow_n; orow = orow_n;
    }
}

// ---- up to 16 rows of x, moderate K: x lives in REGISTERS ----
// A workgroup is NW = 8 or 16 waves; wave w owns the K range [w * K/NW, (w+1) * K/NW) of every block of 16 weight rows
// the workgroup walks (blockIdx.x, + gridDim.x, ...).  The x operands of that range -- NCH chunks x STEPS fragments of
// 16 bytes per lane -- are loaded once, before the weight stream starts, and stay in registers for the whole kernel:
// the loop has no LDS read, no x staging and no slab barrier, only the dequantisation and the MFMA.  The NW partial
// sums of a row block meet in LDS in a fixed order (one barrier per row block, buffer alternating); the wave whose turn
// it is (row block count % NW) adds them and stores.  As in the kernel above the weight stream runs across row blocks:
// the slot a chunk was consumed from is refilled with the chunk PF further on, in this row block or the next.
// Sixteen waves (four per SIMD, 128 registers each, 16 fragments of x) hide the dequantisation's vector work best.
// SCM, where a chunk's scale comes from: 0 one 16-bit load per chunk (any group that is a power-of-two multiple of the
// chunk, or per channel); 1 one scale per chunk, a row's scales contiguous: 8- or 16-byte loads one row block ahead;
// 2 (4-bit weights) one e8m0 byte per 32 weights, i.e. per lane piece, a row's bytes contiguous: 16-byte loads one row
// block ahead.  WFLT: the weights are floating-point codes (e2m1 / e4m3), no offset.
// TWO (eight waves x four chunks, the K split's smaller segment): x staged in two rounds through 64 KB of LDS, so that two
// such workgroups (at most 128 registers per lane) share a CU.
template <int XDT, int WBITS, int NW, int NCH, bool HAS_OFF, int SCM, bool WFLT = false, bool TWO = false>
__global__ __launch_bounds__(NW * 64) void wqmm_xreg_kernel(WqParams p)
{
    static_assert(!TWO || (NW == 8 && NCH == 4), "two workgroups per CU: the eight-wave, four-chunk shape");
    constexpr bool VSCALE = SCM == 1, MXS = SCM == 2;
    static_assert(!MXS || WBITS == 4, "one e8m0 byte per lane piece of 32 weights");
    static_assert(!WFLT || !HAS_OFF, "floating-point weight codes carry no offset");
    constexpr int KPL = 128 / WBITS, KC = 4 * KPL, STEPS = KC / 32;
    constexpr int PF = NW == 16 ? 4 : (NCH < 8 ? NCH : 8);   // weight pieces in flight per lane
    constexpr int NX = NCH * STEPS;                          // x fragments per lane
    static_assert(NW == 8 || NW == 16, "one or two workgroup halves per SIMD pair");
    static_assert(NX <= (NW == 16 ? 16 : 32), "x fragments must fit the register file beside the weight stream");
    static_assert(NCH % 4 == 0 && NCH >= PF, "whole groups of four chunks");
    // 256-byte units of x per wave; the staging takes them in one round when all waves' units fit 128 KB of LDS (TWO: 64 KB), else in two
    constexpr int NU = NX / 4, NR = NW * NU * 4096 <= (TWO ? 64 : 128) * 1024 ? 1 : 2, HU = NU / NR;
    static_assert(NU % NR == 0 && HU * 4096 >= 2048, "whole staging rounds that also hold the partial sums");
    extern __shared__ __attribute__((aligned(16))) char dyn[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nrow = lane & 15, g = lane >> 4;
    const int rows = (int)p.m_rows;
    // first chunk of this wave's K range; with K split over gridDim.y workgroup columns this workgroup's segment is the
    // blockIdx.y-th run of NW * NCH chunks
    const int cbase = ((int)blockIdx.y * NW + wave) * NCH;
    const int nblocks = (int)((p.N + 15) / 16);
    // chunks of this wave that lie inside K (the last segment of a K that is no whole number of segments has idle chunks:
    // their weights are fetched from the row's last chunk instead and nothing is multiplied)
    const int nlive = (int)(p.K / KC) - cbase;
    auto chunk_at = [&](int c) { return c < nlive ? c : (nlive > 0 ? nlive - 1 : -cbase); };   // (a wave with no live chunk reloads the row's first one)

    auto row_of = [&](int rb) { const int64_t n = (int64_t)rb * 16 + nrow; return n < p.N ? n : p.N - 1; };
    auto wptr_of = [&](int rb) { return p.w + row_of(rb) * p.ldw + g * 16 + (int64_t)cbase * 64; };
    // a row's scales: 16-bit elements, or (MXS) e8m0 bytes
    auto srow_of = [&](int rb) { return (const uint16_t*)((const char*)p.scale + row_of(rb) * p.s_cs * (MXS ? 1 : 2)); };
    int rb = blockIdx.x;
    const uint8_t* wptr = wptr_of(rb);
    const uint16_t* srow = srow_of(rb);
    const uint16_t* orow = HAS_OFF ? p.offset + row_of(rb) * p.s_cs : nullptr;

    // VSCALE: the NCH scales of this wave's K range as NCH/2 dwords; MXS: its 4 NCH scale bytes as NCH dwords (byte g of
    // dword c belongs to lane group g); fetched one row block ahead
    constexpr int SW = MXS ? NCH : NCH / 2;
    uint32_t sv[SW], ov[SW], svn[SW], ovn[SW];
    // (A wave with no live chunk fetches the row's first scales instead: nothing uses them.  A wave with some idle chunks
    // reads past the row's last scale, but not past its pitch: these loads are chosen only for rows whose pitch is a whole
    // number of 16-byte pieces.)
    const int cbs = nlive > 0 ? cbase : 0;
    auto load_scales = [&](const uint16_t* sr, const uint16_t* orw, uint32_t (&sd)[SW], uint32_t (&od)[SW]) {
        if constexpr (MXS) {
#pragma unroll
            for (int h = 0; h < NCH / 4; h++) {
                const v4i t = *(const v4i*)((const uint8_t*)sr + cbs * 4 + 16 * h);
#pragma unroll
                for (int e = 0; e < 4; e++) sd[4 * h + e] = (uint32_t)t[e];
            }
        } else if constexpr (NCH % 8 == 0) {
#pragma unroll
            for (int h = 0; h < NCH / 8; h++) {
                const v4i t = *(const v4i*)(sr + cbs + 8 * h);
#pragma unroll
                for (int e = 0; e < 4; e++) sd[4 * h + e] = (uint32_t)t[e];
                if constexpr (HAS_OFF) {
                    const v4i u = *(const v4i*)(orw + cbs + 8 * h);
#pragma unroll
                    for (int e = 0; e < 4; e++) od[4 * h + e] = (uint32_t)u[e];
                }
            }
        } else {
            const v2i t = *(const v2i*)(sr + cbs);
            sd[0] = (uint32_t)t[0]; sd[1] = (uint32_t)t[1];
            if constexpr (HAS_OFF) {
                const v2i u = *(const v2i*)(orw + cbs);
                od[0] = (uint32_t)u[0]; od[1] = (uint32_t)u[1];
            }
        }
    };
#pragma unroll
    for (int h = 0; h < SW; h++) sv[h] = ov[h] = svn[h] = ovn[h] = 0;
    if constexpr (VSCALE || MXS) load_scales(srow, orow, svn, ovn);
    v4i wq[PF];
    uint16_t sq[PF], oq[PF];
    auto fetch = [&](int j, const uint8_t* wp, const uint16_t* sr, const uint16_t* orw, int cw0) {
        const int cw = chunk_at(cw0);
        wq[j] = *(const v4i*)(wp + (int64_t)cw * 64);
        if constexpr (SCM == 0) {
            const int64_t so = (int64_t)((cbase + cw) >> p.cpg_shift) * p.s_rs;
            sq[j] = sr[so];
            if constexpr (HAS_OFF) oq[j] = orw[so];
        }
    };
#pragma unroll
    for (int j = 0; j < PF; j++) fetch(j, wptr, srow, orow, j);
    const DqConst dqc = make_dq_const();

    // x: the fragment (c, s) of lane (nrow, g) is row nrow, k = cbase*KC + c*KC + g*KPL + 8s .. +8.  Read straight from
    // global memory that is 64 lanes x 16 bytes out of 32 different cache lines per instruction; instead the wave's K
    // range travels through LDS once, in units of 16 rows x 256 bytes: four 16-byte asynchronous copies per unit, each
    // fetching four rows x 256 contiguous bytes, land the 16-byte segment `seg` of row m at position seg ^ m of the
    // row (conflict free for the 16-byte reads below), half of the range at a time where the whole of x would not fit.
    // Rows that x does not have repeat its last row: they only feed output rows that are never stored.
    v4i xr[NX];
    {
        char* stage = dyn + wave * (HU * 4096);
        const int cm = lane >> 4, cp = lane & 15;
        const uint16_t* xw = p.x + p.m_base * p.K + (int64_t)cbase * KC;   // (NU * 128 = NCH * KC elements per wave)
#pragma unroll
        for (int r = 0; r < NR; r++) {
#pragma unroll
            for (int ul = 0; ul < HU; ul++) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    if (4 * q < rows && (int64_t)cbase * KC + (r * HU + ul) * 128 < p.K) {   // (units past the end of K stay unread and unused)
                        const int m = 4 * q + cm;
                        const int mm = m < rows ? m : rows - 1;
                        async_copy16(xw + (int64_t)mm * p.K + (r * HU + ul) * 128 + ((cp ^ m) << 3), stage + ul * 4096 + q * 1024);
                    }
                }
            }
            wait_vmcnt<0>();
            asm volatile("" ::: "memory");
#pragma unroll
            for (int i = 0; i < NX; i++) {
                const int u = ((i / STEPS) * KC) / 128;   // the unit does not depend on the lane
                if (u / HU != r) continue;
                const int seg = (((i / STEPS) * KC) % 128 + g * KPL + 8 * (i % STEPS)) >> 3;
                v4i v = *(const v4i*)(stage + (u % HU) * 4096 + nrow * 256 + ((seg ^ nrow) << 4));
                if constexpr (WBITS == 4) {
                    // halves [0..7] -> [0,4,1,5,2,6,3,7]: the order in which the nibble splicing yields pairs
                    const uint32_t a0 = (uint32_t)v[0], a1 = (uint32_t)v[1], a2 = (uint32_t)v[2], a3 = (uint32_t)v[3];
                    v = (v4i){(int)__builtin_amdgcn_perm(a2, a0, 0x05040100u), (int)__builtin_amdgcn_perm(a2, a0, 0x07060302u),
                              (int)__builtin_amdgcn_perm(a3, a1, 0x05040100u), (int)__builtin_amdgcn_perm(a3, a1, 0x07060302u)};
                }
                xr[i] = v;
            }
            wait_lgkmcnt0();   // this wave's reads have retired before the next copies overwrite the units
            asm volatile("" ::: "memory");
        }
    }
    __syncthreads();   // the staging area now becomes the partial-sum buffers
    float* const red = (float*)dyn;   // [2][NW][256]

    for (int it = 0; rb < nblocks; it++) {
        const int rb_next = rb + (int)gridDim.x;
        const bool has_next = rb_next < nblocks;
        const uint8_t* wptr_n = has_next ? wptr_of(rb_next) : wptr;   // past the end: harmless reloads of this block
        const uint16_t* srow_n = has_next ? srow_of(rb_next) : srow;
        const uint16_t* orow_n = HAS_OFF ? (has_next ? p.offset + row_of(rb_next) * p.s_cs : orow) : nullptr;
        if constexpr (VSCALE || MXS) {
            // the next row block's scales are requested before the refills below fetch its weights (loads return in
            // issue order: waiting for a scale issued after them would drain the weight stream)
#pragma unroll
            for (int h = 0; h < SW; h++) { sv[h] = svn[h]; ov[h] = ovn[h]; }
            load_scales(srow_n, orow_n, svn, ovn);
        }
        v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int c = 0; c < NCH; c++) {
            const int j = c % PF;
            uint16_t sb, ob = 0;
            if constexpr (MXS) {
                // the scale goes through x's dtype (2^e: exact in bf16; fp16 flushes, denormalises or overflows it as the cast does)
                sb = bits_x<XDT>(e8m0_to_f32((sv[c] >> (8 * g)) & 0xffu));
            } else if constexpr (VSCALE) {
                sb = (uint16_t)(sv[c / 2] >> (16 * (c % 2)));
                if constexpr (HAS_OFF) ob = (uint16_t)(ov[c / 2] >> (16 * (c % 2)));
            } else {
                sb = sq[j];
                if constexpr (HAS_OFF) ob = oq[j];
            }
            if (c < nlive) {
#pragma unroll
            for (int s = 0; s < STEPS; s++) {
                v4i aop;
                if constexpr (WFLT) aop = dequant8_float<XDT, WBITS>(wq[j], s, sb);
                else aop = dequant8<XDT, WBITS, HAS_OFF>(wq[j], s, sb, ob, dqc);
                if constexpr (XDT == DT_F16) {
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, aop), __builtin_bit_cast(v8h, xr[c * STEPS + s]), acc, 0, 0, 0);
                } else {
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, aop), __builtin_bit_cast(v8bf, xr[c * STEPS + s]), acc, 0, 0, 0);
                }
            }
            }
            if (c + PF < NCH) fetch(j, wptr, srow, orow, c + PF);
            else fetch(j, wptr_n, srow_n, orow_n, c + PF - NCH);
        }

        // fixed-order reduction of the NW K ranges
        float* rd = red + (it & 1) * (NW * 256);
        *(v4f*)(rd + wave * 256 + lane * 4) = acc;
        __syncthreads();
        if (wave == (it & (NW - 1))) {
            v4f sum = *(const v4f*)(rd + lane * 4);
#pragma unroll 4
            for (int j = 1; j < NW; j++) sum = sum + *(const v4f*)(rd + j * 256 + lane * 4);
            if (nrow < rows && gridDim.y > 1) {   // K split: this segment's sums, as they are, for wq_splitk_reduce_kernel
                const int64_t m = p.m_base + nrow, nn0 = (int64_t)rb * 16 + 4 * g;
                float* dst = p.part + ((int64_t)blockIdx.y * p.M + m) * p.N + nn0;
                if (nn0 + 3 < p.N && (p.N % 4) == 0 && ((uintptr_t)p.part % 16) == 0) {
                    *(v4f*)dst = sum;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (nn0 + i < p.N) dst[i] = sum[i];
                }
            } else if (nrow < rows) {
                const int64_t n0 = (int64_t)rb * 16;
                const int64_t m = p.m_base + nrow;
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int64_t nn = n0 + 4 * g + i;
                    v[i] = sum[i];
                    if (p.bias && nn < p.N) v[i] = v[i] + load_scalar_as_f32(p.bias, p.bias_dt, nn);
                    if constexpr (XDT == DT_BF16) v[i] = bf16_to_f32(bf16_bits(v[i]));
                }
                const int64_t nn0 = n0 + 4 * g;
                if (nn0 + 3 < p.N && (p.N % 4) == 0) {
                    const v4us o = {bits_x<XDT>(v[0]), bits_x<XDT>(v[1]), bits_x<XDT>(v[2]), bits_x<XDT>(v[3])};
                    *(v4us*)(p.y + m * p.N + nn0) = o;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (nn0 + i < p.N) p.y[m * p.N + nn0 + i] = bits_x<XDT>(v[i]);
                }
            }
        }
        rb = rb_next; wptr = wptr_n; srow = srow_n; orow = orow_n;
    }
}

// Workgroups of the persistent kernel: two per CU (row blocks are dealt round-robin, so the workgroups i and
// i + CUs, which share a CU, together get an even share), or one per row block when there are fewer than that.
static inline unsigned resx_grid(int64_t nblocks)
{
    static const int cus = [] {
        int d = 0, n = 0;
        if (hipGetDevice(&d) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, d) != hipSuccess || n <= 0) n = 256;
        return n;
    }();
    const int64_t g = 2 * (int64_t)cus;
    return (unsigned)(nblocks < g ? nblocks : g);
}

template <int XDT, int WBITS, bool HAS_OFF, bool VSCALE>
static int launch_resx_one(const WqParams& p, hipStream_t st)
{
    const size_t lds = (size_t)(p.m_rows + 1) * (p.K * 2 + 16) + 2 * 3 * 4 * 64 * 4;
    auto k = wqmm_resx_kernel<XDT, WBITS, HAS_OFF, VSCALE>;
    static std::atomic<uint64_t> attr_set{0};   // one bit per device: the attribute belongs to the (kernel, device) pair
    if (!device_flag_test(attr_set)) {
        hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, 65536 + 8192);
        if (e != hipSuccess) return (int)e;
        device_flag_set(attr_set);
    }
    hipLaunchKernelGGL(k, dim3(resx_grid((p.N + 15) / 16)), dim3(256), lds, st, p);
    return (int)hipGetLastError();
}

// y[m, n] = rounded(sum over the K segments, in order, of part[s, m, n] + bias[n])
template <int XDT>
__global__ __launch_bounds__(256) void wq_splitk_reduce_kernel(const float* part, int splits, int64_t total, int64_t N, const void* bias, int bias_dt,
                                                               uint16_t* y)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        float v = splitk_sum(part, splits, total, i);
        if (bias) v = v + load_scalar_as_f32(bias, bias_dt, i % N);
        y[i] = bits_x<XDT>(v);
    }
}

// the fp8 forms of the many-rows kernel: out[m, n] = cast(epilogue(sum over the K segments, in order, of part[s, m, n])); the
// block-scale form has folded its scales in already, the row / column scale form (RC) computes
// (sum * x2Scale[n]) * x1Scale[m] + bias[n] here as the kernel's own epilogue does
template <bool RC>
__global__ __launch_bounds__(256) void rows_bs_splitk_reduce_kernel(const float* part, int splits, int64_t total, int64_t N, const float* rs, int64_t rs_stride,
                                                                    const float* cs, int64_t cs_stride, const float* bias, void* out, int out_dt)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        float v = splitk_sum(part, splits, total, i);
        if constexpr (RC) {
            const int64_t m = i / N, n = i - m * N;
            v = (v * cs[n * cs_stride]) * rs[m * rs_stride];
            if (bias) v = v + bias[n];
        }
        if (out_dt == DT_F32) ((float*)out)[i] = v;
        else ((uint16_t*)out)[i] = out_dt == DT_BF16 ? bf16_bits(v) : f16_bits(v);
    }
}

// One workgroup per CU (its waves fill the register file), or one per row block when there are fewer; with K split into
// `splits` segments one workgroup column per segment, the CUs shared between the columns.
template <int XDT, int WBITS, int NW, int NCH, bool HAS_OFF, int SCM, bool WFLT = false, bool TWO = false>
static int launch_xreg_one(const WqParams& p, hipStream_t st, int splits = 1)
{
    if constexpr (NW == 8 && NCH == 4 && !TWO) {
        if (splits > 1) return launch_xreg_one<XDT, WBITS, NW, NCH, HAS_OFF, SCM, WFLT, true>(p, st, splits);   // (measured at 16 x 28672 x 8192: 54 -> 42 us)
    }
    const int64_t nblocks = (p.N + 15) / 16;
    if (splits < 1 || splits > 16 || (splits > 1 && (!p.part || p.m_base != 0 || p.m_rows != p.M))) return -1;
    {   // the segments cover K, the last one with idle chunks worth at most a fifth of K; with idle chunks the vector scale
        // loads of a wave's last piece may reach past the row's last scale: the row's pitch must hold whole pieces
        const int64_t kc = 4 * (128 / WBITS), nch = p.K / kc, cover = (int64_t)splits * NW * NCH;
        if (p.K % 128 != 0 || cover < nch || (cover - nch) * 5 > nch || cover - nch >= (int64_t)NW * NCH) return -1;
        if (cover != nch && SCM == 1 && (p.s_cs % 8 != 0 || p.s_cs < nch)) return -1;
        if (cover != nch && SCM == 2 && (p.s_cs % 16 != 0 || p.s_cs < nch * 4)) return -1;
    }
    const int64_t g = ((int64_t)resx_grid(1ll << 40) / (TWO ? 1 : 2) + splits - 1) / splits;   // (resx_grid: two per CU)
    constexpr int STEPS = (4 * (128 / WBITS)) / 32;
    constexpr int NU = NCH * STEPS / 4;                  // units of 16 rows x 256 bytes per wave
    constexpr int lds = NW * NU * 4096 <= (TWO ? 64 : 128) * 1024 ? NW * NU * 4096 : NW * (NU / 2) * 4096;   // all of x, or half of it at a time
    auto k = wqmm_xreg_kernel<XDT, WBITS, NW, NCH, HAS_OFF, SCM, WFLT, TWO>;
    static std::atomic<uint64_t> attr_set{0};   // one bit per device: the attribute belongs to the (kernel, device) pair
    if (!device_flag_test(attr_set)) {
        hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return (int)e;
        device_flag_set(attr_set);
    }
    hipLaunchKernelGGL(k, dim3((unsigned)(nblocks < g ? nblocks : g), (unsigned)splits), dim3(NW * 64), lds, st, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || splits == 1) return (int)e;
    const int64_t total = p.M * p.N;
    hipLaunchKernelGGL(wq_splitk_reduce_kernel<XDT>, dim3(splitk_reduce_grid(total)), dim3(256), 0, st, (const float*)p.part, splits, total, p.N, p.bias,
                       p.bias_dt, p.y);
    return (int)hipGetLastError();
}

template <int XDT, int WBITS, int NW, int NCH>
static int launch_xreg_nch(const WqParams& p, bool has_off, bool vscale, hipStream_t st, int splits = 1)
{
    if (vscale) return has_off ? launch_xreg_one<XDT, WBITS, NW, NCH, true, 1>(p, st, splits) : launch_xreg_one<XDT, WBITS, NW, NCH, false, 1>(p, st, splits);
    return has_off ? launch_xreg_one<XDT, WBITS, NW, NCH, true, 0>(p, st, splits) : launch_xreg_one<XDT, WBITS, NW, NCH, false, 0>(p, st, splits);
}

// K = waves x chunks per wave x chunk.  Sixteen waves with 4 chunks each (8-bit weights: or 8), else eight waves with 4 or 8.
// The plan of wq_xreg_plan (launch.h; the workspace query uses the same function); force_nw == 8 keeps a K of 64 chunks
// on eight waves x eight chunks.  With more than one segment the call needs room for partial sums (`may_split`).
static inline bool xreg_shape(int wbits, int64_t K, int force_nw, int& nw, int& nch, int64_t M = 1, bool may_split = false, int* splits = nullptr,
                              bool* exact = nullptr)
{
    WqXregPlan pl;
    if (!wq_xreg_plan(wbits, M, K, pl)) return false;
    if (pl.splits > 1 && !(may_split && splits)) return false;
    if (!pl.exact && !exact) return false;
    if (force_nw == 8 && pl.splits == 1 && pl.exact && pl.nw == 16 && pl.nch == 4) pl = {8, 8, 1, true};
    nw = pl.nw; nch = pl.nch;
    if (splits) *splits = pl.splits;
    if (exact) *exact = pl.exact;
    return true;
}

template <int XDT, int WBITS>
static int launch_xreg(const WqParams& p, bool has_off, bool vscale, int force_nw, hipStream_t st)
{
    int nw = 0, nch = 0, splits = 1;
    bool exact = true;
    if (!xreg_shape(WBITS, p.K, force_nw, nw, nch, p.M, p.part != nullptr, &splits, &exact)) return OPSNN_NOT_TAKEN;
    if (nw == 16 && nch == 4) return launch_xreg_nch<XDT, WBITS, 16, 4>(p, has_off, vscale, st, splits);
    if constexpr (WBITS == 8) {
        if (nw == 16 && nch == 8) return launch_xreg_nch<XDT, WBITS, 16, 8>(p, has_off, vscale, st);
    }
    if (nw == 8 && nch == 4) return launch_xreg_nch<XDT, WBITS, 8, 4>(p, has_off, vscale, st, splits);
    if (nw == 8 && nch == 8) return launch_xreg_nch<XDT, WBITS, 8, 8>(p, has_off, vscale, st);
    return OPSNN_NOT_TAKEN;
}

// Floating-point weight codes without offset: e2m1 with e8m0 scales per 32 weights (mxfp4; a row's scale bytes contiguous and
// 16-byte aligned), e4m3 with one scale per channel.  p.cpg_shift must be set for the latter.
template <int XDT, int WBITS>
static int launch_xreg_float(const WqParams& p, hipStream_t st)
{
    int nw = 0, nch = 0, splits = 1;
    bool exact = true;
    if (!xreg_shape(WBITS, p.K, 0, nw, nch, p.M, p.part != nullptr, &splits, &exact)) return OPSNN_NOT_TAKEN;
    constexpr int SCM = WBITS == 4 ? 2 : 0;
    if (nw == 16 && nch == 4) return launch_xreg_one<XDT, WBITS, 16, 4, false, SCM, true>(p, st, splits);
    if constexpr (WBITS == 8) {
        if (nw == 16 && nch == 8) return launch_xreg_one<XDT, WBITS, 16, 8, false, SCM, true>(p, st);
    }
    if (nw == 8 && nch == 4) return launch_xreg_one<XDT, WBITS, 8, 4, false, SCM, true>(p, st, splits);
    if (nw == 8 && nch == 8) return launch_xreg_one<XDT, WBITS, 8, 8, false, SCM, true>(p, st);
    return OPSNN_NOT_TAKEN;
}

template <int XDT, int WBITS, int MB, int NW, int WK, bool HAS_OFF, bool VSCALE>
static int launch_stream_one(const WqParams& p, hipStream_t st)
{
    constexpr int KC = 4 * (128 / WBITS), KX = 8 * KC / MB, WN = NW / WK;
    const size_t lds_x = 2 * (size_t)(p.m_rows + 1) * (KX * 2 + 16);
    const size_t lds_red = WK > 1 ? (size_t)WN * (WK - 1) * MB * 4 * 64 * 4 : 0;
    const size_t lds = lds_x > lds_red ? lds_x : lds_red;
    const unsigned grid = (unsigned)((p.N + 16 * WN - 1) / (16 * WN));
    auto k = wqmm_stream_kernel<XDT, WBITS, MB, NW, WK, HAS_OFF, VSCALE>;
    static std::atomic<uint64_t> attr_set{0};   // one bit per device: the attribute belongs to the (kernel, device) pair
    if (!device_flag_test(attr_set)) {
        constexpr size_t lds_max = 2 * (size_t)(16 * MB + 1) * (KX * 2 + 16);
        hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_max);
        if (e != hipSuccess) return (int)e;
        device_flag_set(attr_set);
    }
    hipLaunchKernelGGL(k, dim3(grid), dim3(NW * 64), lds, st, p);
    return (int)hipGetLastError();
}

template <int XDT, int WBITS, int MB, int NB, int WN, int WK, bool HAS_OFF, int WF = 0, bool SLDS = false, bool KSP = false>
static int launch_rows_one(const WqParams& p, hipStream_t st)
{
    if constexpr (!KSP) {   // K in segments: the instantiations of the 64-row instance with 128-column workgroups that know them
        if (p.ksplit > 1) {
            if constexpr (MB == 4 && NB == 2 && WN == 4 && WK == 2 && WF <= 4 && !SLDS) return launch_rows_one<XDT, WBITS, MB, NB, WN, WK, HAS_OFF, WF, false, true>(p, st);
            else return -1;
        }
    }
    constexpr int KC = 4 * (128 / WBITS);
    constexpr int XH = (MB > 8 && WBITS == 4) ? 2 : 1;   // as in the kernel: 8-byte weight pieces, i.e. slabs of half the K, for more than 128 rows of x with 4-bit weights
    constexpr size_t lds_x = 2 * (size_t)(16 * MB) * (WK * KC * 2 / XH);
    size_t lds_stab = 0;
    const bool split = KSP;
    // (a split launch covers all rows: the kernel that adds the segments walks the whole output)
    if (split && (!p.part || p.ksplit < 2 || p.ksplit > 64 || p.m_base != 0 || (p.m_slab > 0 ? p.m_end : p.m_rows) != p.M)) return -1;
    // the longest K one workgroup walks: segments are whole units of p.kunit k (whole slabs of x, whole groups), as equal as
    // that allows
    constexpr int64_t KXS = (int64_t)WK * 4 * (((MB > 8 && WBITS == 4) ? 8 : 16) * 8 / WBITS);   // k per slab of x
    if (p.K % KXS != 0) return -1;
    if (MB > 8 && p.K % (4 * KXS) != 0) return OPSNN_NOT_TAKEN;   // the 192- / 256-row instances: whole rounds of four slabs
    int64_t kseg = p.K;
    if (split) {
        if (p.kunit <= 0 || p.kunit % KXS != 0 || p.K % p.kunit != 0 || p.K / p.kunit < p.ksplit || (p.group < p.K && p.kunit % p.group != 0)) return -1;
        kseg = (p.K / p.kunit + p.ksplit - 1) / p.ksplit * p.kunit;
    }
    // groups of that K, and the pitch of a scale table row: the power of two at or above
    const int64_t G = p.cpg_shift >= 31 ? 1 : (((kseg / KC) + (1ll << p.cpg_shift) - 1) >> p.cpg_shift);   // (the last group may be short)
    int64_t GP = 1;
    while (GP < G) GP *= 2;
    if constexpr ((WF == 0 || WF == 2) && !SLDS) {
        // the scales and offsets of the workgroup's columns in LDS when a row's scales are contiguous and the table fits
        // beside the x buffers (e2m1 codes: one word per 128 k, the four e8m0 bytes of a row read as a word; the caller
        // passes cpg_shift 0)
        const size_t red = (size_t)WN * (WK - 1) * NB * MB * 4 * 64 * 4;
        // (the caller counts a table word of 128 k in chunks: one of e2m1 codes, two of e4m3 codes)
        const bool rows_ok = WF == 2 ? (p.s_cs % 4 == 0 && (uintptr_t)p.scale % 4 == 0 && p.cpg_shift == (WBITS == 8 ? 1 : 0)) : (p.s_rs == 1 || G == 1);
        if (rows_ok && (lds_x > red ? lds_x : red) + (size_t)(16 * NB * WN) * GP * 4 <= 160 * 1024)
            return launch_rows_one<XDT, WBITS, MB, NB, WN, WK, HAS_OFF, WF, true, KSP>(p, st);
    }
    if constexpr (MB > 8 && WF == 0 && !SLDS) return OPSNN_NOT_TAKEN;   // integer codes: the 192- / 256-row instances exist with the scale table only
    else {
    if constexpr (SLDS) lds_stab = (size_t)(16 * NB * WN) * GP * 4;
    constexpr size_t lds_red = (size_t)WN * (WK - 1) * NB * MB * 4 * 64 * 4;
    constexpr size_t lds_main = lds_x > lds_red ? lds_x : lds_red;
    constexpr size_t lds_table = WF == 3 ? 65536 : 0;   // products of the block scales: (K / 128) * 16 MB floats, at most this
    const size_t lds = lds_main + (WF == 3 ? (size_t)(kseg / 128) * 16 * MB * 4 : 0) + lds_stab;
    if (lds > lds_main + lds_table + lds_stab) return OPSNN_NOT_TAKEN;
    const unsigned grid = (unsigned)((p.N + 16 * NB * WN - 1) / (16 * NB * WN));
    const int64_t slabs = p.m_slab > 0 ? (p.m_end - p.m_base + p.m_slab - 1) / p.m_slab : 1;
    if (slabs < 1 || slabs > 65535 || p.m_rows > 16 * MB || (p.m_slab > 0 && p.m_slab != p.m_rows)) return -1;
    auto k = wqmm_rows_kernel<XDT, WBITS, MB, NB, WN, WK, HAS_OFF, WF, SLDS, KSP>;
    static std::atomic<uint64_t> attr_set{0};   // one bit per device: the attribute belongs to the (kernel, device) pair
    if (!device_flag_test(attr_set)) {
        hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(SLDS ? 160 * 1024 : lds_main + lds_table));
        if (e != hipSuccess) return (int)e;
        device_flag_set(attr_set);
    }
    hipLaunchKernelGGL(k, dim3(grid, (unsigned)slabs, split ? (unsigned)p.ksplit : 1u), dim3(512), lds, st, p);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return (int)e;
    if (split) {
        const int64_t total = p.M * p.N;
        if constexpr (WF == 3) {
            hipLaunchKernelGGL(rows_bs_splitk_reduce_kernel<false>, dim3(splitk_reduce_grid(total)), dim3(256), 0, st, (const float*)p.part, p.ksplit, total,
                               p.N, (const float*)nullptr, (int64_t)0, (const float*)nullptr, (int64_t)0, (const float*)nullptr, (void*)p.y, p.bs_out_dt);
            return (int)hipGetLastError();
        }
        if constexpr (WF == 4) {
            hipLaunchKernelGGL(rows_bs_splitk_reduce_kernel<true>, dim3(splitk_reduce_grid(total)), dim3(256), 0, st, (const float*)p.part, p.ksplit, total,
                               p.N, p.bs1, p.bs1_rs, p.bs2, p.bs2_cs, (const float*)p.bias, (void*)p.y, p.bs_out_dt);
            return (int)hipGetLastError();
        }
        hipLaunchKernelGGL(wq_splitk_reduce_kernel<XDT>, dim3(splitk_reduce_grid(total)), dim3(256), 0, st, (const float*)p.part, p.ksplit, total, p.N,
                           p.bias, p.bias_dt, p.y);
        return (int)hipGetLastError();
    }
    return 0;
    }
}

struct WqStreamOpts {
    bool has_off, vscale, ksplit;
    bool rows;                // many-rows kernel eligible (row slabs of up to 128)
    bool rows_shape;          // ... as far as K, N and the scale layout go (rows also asks for 33 rows or more)
    bool resx, resx_vscale;   // whole-x-in-LDS kernel eligible, and with vector scale loads
    bool xreg, xreg_vscale;   // x-in-registers kernel eligible (up to 16 rows), and with vector scale loads
    int xreg_nw;              // 8: keep it to eight waves (tuning)
};

// One row slab (p.m_rows <= 128 with o.rows, else <= 64) of one dtype pair; defined once per pair in its own translation unit.
template <int XDT, int WBITS>
int launch_wq_stream(const WqParams& p, const WqStreamOpts& o, hipStream_t st);
// Up to 16 rows, floating-point weight codes (see launch_xreg_float); OPSNN_NOT_TAKEN if K does not split.
template <int XDT, int WBITS>
int launch_wq_xreg_float(const WqParams& p, hipStream_t st);
// One row slab of up to 256 rows, floating-point weight codes, on the many-rows kernel (WBITS 4: mxfp4 with a row's
// e8m0 bytes contiguous; 8: e4m3 with per-channel scales).  The caller has checked the kernel's shape conditions.
template <int XDT, int WBITS>
int launch_wq_rows_float(const WqParams& p, hipStream_t st);

#define OPSNN_WQ_STREAM_DEFINE(XDT, WBITS)                                                                          \
    template <>                                                                                                     \
    int launch_wq_xreg_float<XDT, WBITS>(const WqParams& p, hipStream_t st) { return launch_xreg_float<XDT, WBITS>(p, st); } \
    template <>                                                                                                     \
    int launch_wq_rows_float<XDT, WBITS>(const WqParams& p, hipStream_t st)                                         \
    {                                                                                                               \
        constexpr int WF = WBITS == 4 ? 2 : 1;                                                                      \
        if constexpr (WBITS == 8) {   /* e4m3 codes with e8m0 scales per 32 (no 64-column instance) */                 \
            if (p.scale_e8m0) {                                                                                     \
                if (p.m_rows > 192) return launch_rows_one<XDT, WBITS, 16, 2, 4, 2, false, 2>(p, st);               \
                if (p.m_rows > 128) return launch_rows_one<XDT, WBITS, 12, 2, 4, 2, false, 2>(p, st);               \
                return p.m_rows > 64 ? launch_rows_one<XDT, WBITS, 8, 2, 4, 2, false, 2>(p, st)                     \
                                     : launch_rows_one<XDT, WBITS, 4, 2, 4, 2, false, 2>(p, st);                    \
            }                                                                                                       \
        }                                                                                                           \
        if (p.m_rows > 192) return launch_rows_one<XDT, WBITS, 16, 2, 4, 2, false, WF>(p, st);                      \
        if (p.m_rows > 128) return launch_rows_one<XDT, WBITS, 12, 2, 4, 2, false, WF>(p, st);                      \
        if (p.cols64 && p.m_rows <= 64) return launch_rows_one<XDT, WBITS, 4, 2, 2, 4, false, WF>(p, st);           \
        return p.m_rows > 64 ? launch_rows_one<XDT, WBITS, 8, 2, 4, 2, false, WF>(p, st)                            \
                             : launch_rows_one<XDT, WBITS, 4, 2, 4, 2, false, WF>(p, st);                           \
    }                                                                                                               \
    template <int MB, int NW, int WK, bool VS>                                                                      \
    static int wq_stream_off(const WqParams& p, bool has_off, hipStream_t st)                                       \
    {                                                                                                               \
        return has_off ? launch_stream_one<XDT, WBITS, MB, NW, WK, true, VS>(p, st)                                 \
                       : launch_stream_one<XDT, WBITS, MB, NW, WK, false, VS>(p, st);                               \
    }                                                                                                               \
    template <int MB>                                                                                               \
    static int wq_stream_mb(const WqParams& p, const WqStreamOpts& o, hipStream_t st)                               \
    {                                                                                                               \
        return o.vscale ? wq_stream_off<MB, 4, 1, true>(p, o.has_off, st) : wq_stream_off<MB, 4, 1, false>(p, o.has_off, st); \
    }                                                                                                               \
    template <>                                                                                                     \
    int launch_wq_stream<XDT, WBITS>(const WqParams& p, const WqStreamOpts& o, hipStream_t st)                      \
    {                                                                                                               \
        if (o.xreg && p.m_rows <= 16) {                                                                             \
            const int rc = launch_xreg<XDT, WBITS>(p, o.has_off, o.xreg_vscale, o.xreg_nw, st);                     \
            if (rc != OPSNN_NOT_TAKEN) return rc;                                                                   \
        }                                                                                                           \
        if (o.resx) {                                                                                               \
            if (o.resx_vscale) return o.has_off ? launch_resx_one<XDT, WBITS, true, true>(p, st)                    \
                                                : launch_resx_one<XDT, WBITS, false, true>(p, st);                  \
            return o.has_off ? launch_resx_one<XDT, WBITS, true, false>(p, st)                                      \
                             : launch_resx_one<XDT, WBITS, false, false>(p, st);                                    \
        }                                                                                                           \
        if (o.rows && p.m_rows > 192) return o.has_off ? launch_rows_one<XDT, WBITS, 16, 2, 4, 2, true>(p, st)            \
                                                       : launch_rows_one<XDT, WBITS, 16, 2, 4, 2, false>(p, st);          \
        if (o.rows && p.m_rows > 128) return o.has_off ? launch_rows_one<XDT, WBITS, 12, 2, 4, 2, true>(p, st)            \
                                                       : launch_rows_one<XDT, WBITS, 12, 2, 4, 2, false>(p, st);          \
        if (o.rows && p.m_rows > 64) return o.has_off ? launch_rows_one<XDT, WBITS, 8, 2, 4, 2, true>(p, st)              \
                                                      : launch_rows_one<XDT, WBITS, 8, 2, 4, 2, false>(p, st);            \
        if (o.rows && p.cols64) return o.has_off ? launch_rows_one<XDT, WBITS, 4, 2, 2, 4, true>(p, st)                   \
                                                 : launch_rows_one<XDT, WBITS, 4, 2, 2, 4, false>(p, st);                 \
        if (o.rows) return o.has_off ? launch_rows_one<XDT, WBITS, 4, 2, 4, 2, true>(p, st)                               \
                                     : launch_rows_one<XDT, WBITS, 4, 2, 4, 2, false>(p, st);                             \
        if (o.ksplit && p.m_rows <= 16) return wq_stream_off<1, 4, 4, false>(p, o.has_off, st);                     \
        if (p.m_rows <= 16) return wq_stream_mb<1>(p, o, st);                                                       \
        if (p.m_rows <= 32) return wq_stream_mb<2>(p, o, st);                                                       \
        return wq_stream_mb<4>(p, o, st);                                                                           \
    }

}  // namespace opsnn
