// Weight-only quantized matmul for decode-shaped M (fp16 / bf16 activations, int4 / int8 weights).
//
//   y[m,n] = cast( sum_k x[m,k] * T(T(w[k,n] + offset[g,n]) * scale[g,n]) + bias[n] ),   g = k / group,
//   T = rounding through x's dtype (both dequantisation steps are rounded, as the reference's vector unit does:
//   matmul/weight_quant_batch_matmul_v2/op_kernel/arch35/n_first/basic_block_vf_nd.h:139-148; golden:
//   matmul/weight_quant_batch_matmul_v2/tests/assets/wqbmmv2_kernel_golden.py:199-297).
//
// The path is bound by the weight stream from HBM, so the kernel is built around it:
//   - the weight is consumed K-contiguous ("stored [N, K]"); every lane streams 16-byte pieces of one weight row
//     straight from global memory into registers -- each weight byte is used by exactly one wave, so it never
//     visits LDS -- with several pieces in flight per lane;
//   - a wave owns 16 output columns for all of K.  A 16-byte piece holds 32 int4 (16 int8) consecutive k of one
//     column; the four 16-lane groups of the wave take consecutive pieces, so one load instruction covers a
//     [16 n] x [128 k] (int8: [64 k]) weight block that lies inside one quantisation group whenever the group
//     size is a multiple of 128 (64);
//   - dequantisation happens in registers in x's own arithmetic: for fp16 the nibbles are spliced into the
//     mantissa of 1024.0 (exact), re-centred with one packed add or fma, then one packed fp16 add (offset) and
//     one packed fp16 multiply (scale) perform exactly the two roundings of the formula; for bf16 the same steps
//     run in fp32 with the hardware's round-to-nearest-even conversion to bf16 after each;
//   - the contraction is v_mfma_f32_16x16x32_{f16,bf16} with the weight block as the row operand and x as the
//     column operand (fp32 accumulation); for M = 1 fifteen of the sixteen columns are idle, which costs nothing
//     because the matrix pipe is far from being the limit;
//   - x is staged through LDS in K slabs shared by the workgroup's four waves, already permuted into the element
//     order the nibble splicing produces, so no weight register ever needs a shuffle.
// M > 64 is processed in row slabs of 64 (the weight is re-streamed per slab; such shapes are compute-bound).
#include "wqmm_stream.hip.h"

namespace opsnn {

int launch_wqmm_plain(const OpsnnWqmmArgs& a, hipStream_t st);

// MB: 16-row blocks of x handled per launch slab (1, 2 or 4).  WBITS: 4 or 8.
// WK: waves of the workgroup that split K between them (1, 2 or 4); the other 4/WK waves take different column
// blocks.  WK > 1 is for narrow N, where column blocks alone cannot fill the chip; partial sums meet in LDS and
// are added in a fixed order.
// WFLT: the weights are floating-point codes (e2m1 in 4 bits, e4m3 in 8), possibly with e8m0 scales per 32 k (MX:
// wqbmmv2_kernel_golden.py:300-352 -- the weight is exact in x's dtype, the scale goes through x's dtype, one rounding of
// the product); they take the element-wise dequantisation below.
template <int XDT, int WBITS, int MB, int WK, bool WFLT>
__global__ __launch_bounds__(256, 2) void wqmm_decode_kernel(WqParams p)
{
    constexpr int WN = 4 / WK;
    constexpr int KPL = 128 / WBITS;          // k elements per 16-byte piece per lane: 32 (int4) or 16 (int8)
    constexpr int KC = 4 * KPL;               // k per wave load instruction ("chunk"): 128 or 64
    constexpr int STEPS = KC / 32;            // MFMA steps per chunk: 4 or 2
    constexpr int PF = 8;                     // weight pieces in flight per lane = chunks per super-step
    constexpr int KX = (PF * KC) / MB;        // k per LDS slab of x
    constexpr int CPS = KX / KC;              // chunks per slab: 8, 4 or 2
    constexpr int ROWS = 16 * MB;
    constexpr int XROW = KX * 2 + 16;         // padded LDS row pitch in bytes (conflict-free 16-byte reads)
    constexpr int XSLAB = ROWS * XROW;
    constexpr int XITEMS = ROWS * (KX / 8) / 256;   // 16-byte x pieces staged per thread per slab
    static_assert(ROWS * (KX / 8) % 256 == 0, "x staging mapping");
    extern __shared__ __attribute__((aligned(16))) char sx[];   // 2 * XSLAB bytes (reused for the K-split reduction)

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave / WK, wk = wave % WK;
    const int nrow = lane & 15, g = lane >> 4;
    const int64_t n0 = ((int64_t)blockIdx.x * WN + wn) * 16;
    const bool n_ok = n0 < p.N;                       // whole wave idle past the edge (still joins barriers)
    const int64_t n = (n0 + nrow) < p.N ? (n0 + nrow) : p.N - 1;
    const bool has_off = p.offset != nullptr;
    const int Ki = (int)p.K, groupi = (int)p.group;
    const int NSLAB = (Ki + KX - 1) / KX;

    const uint8_t* wrow = p.w + n * p.ldw;
    const uint16_t* srow = p.scale + n * p.s_cs;
    const uint16_t* orow = has_off ? p.offset + n * p.s_cs : nullptr;

    // x staging: each thread moves XITEMS 16-byte pieces (8 consecutive halves) per slab; for int4 the halves are
    // permuted to [0,4,1,5,2,6,3,7] so that the pairs produced by the nibble splicing line up with pairs of x.
    v4i xreg[XITEMS];
    auto load_x = [&](int slab) {
#pragma unroll
        for (int it = 0; it < XITEMS; it++) {
            const int idx = it * 256 + tid;
            const int r = idx / (KX / 8), c = idx % (KX / 8);
            const int64_t m = p.m_base + r;
            const int k = slab * KX + c * 8;
            v4i v = {0, 0, 0, 0};
            if (r < p.m_rows && k + 8 <= Ki) v = *(const v4i*)(p.x + m * p.K + k);   // K % 8 == 0 on this path
            xreg[it] = v;
        }
    };
    auto store_x = [&](int buf) {
        char* dst = sx + buf * XSLAB;
#pragma unroll
        for (int it = 0; it < XITEMS; it++) {
            const int idx = it * 256 + tid;
            const int r = idx / (KX / 8), c = idx % (KX / 8);
            v4i v = xreg[it];
            if constexpr (WBITS == 4) {
                const uint32_t a0 = (uint32_t)v[0], a1 = (uint32_t)v[1], a2 = (uint32_t)v[2], a3 = (uint32_t)v[3];
                v4i o;
                o[0] = (int)((a0 & 0xffffu) | (a2 << 16));          // h0, h4
                o[1] = (int)((a0 >> 16) | (a2 & 0xffff0000u));      // h1, h5
                o[2] = (int)((a1 & 0xffffu) | (a3 << 16));          // h2, h6
                o[3] = (int)((a1 >> 16) | (a3 & 0xffff0000u));      // h3, h7
                v = o;
            }
            *(v4i*)(dst + r * XROW + c * 16) = v;
        }
    };

    v4f acc[MB];
#pragma unroll
    for (int b = 0; b < MB; b++) acc[b] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};

    // weight pieces with their group's scale and offset, fetched one super-step (PF chunks) ahead of their use;
    // with WK > 1 a wave only touches the chunks c with c % WK == wk
    v4i wq[PF];
    uint16_t sq[PF], oq[PF];
    auto load_w = [&](int c0) {
#pragma unroll
        for (int i = 0; i < PF; i++) {
            if (WK > 1 && (i % WK) != wk) continue;
            const int k = (c0 + i) * KC + g * KPL;
            // K is a multiple of KPL on this path; pieces past K read the row's last piece and are masked when used
            const int kk = k < Ki ? k : Ki - KPL;
            wq[i] = n_ok ? *(const v4i*)(wrow + (int64_t)kk * WBITS / 8) : (v4i){0, 0, 0, 0};
            const int gi = p.group_shift >= 0 ? (kk >> p.group_shift) : (kk / groupi);
            if (WFLT && p.scale_e8m0) sq[i] = bits_x<XDT>(e8m0_to_f32(((const uint8_t*)p.scale)[n * p.s_cs + (int64_t)gi * p.s_rs]));
            else sq[i] = srow[(int64_t)gi * p.s_rs];
            oq[i] = has_off ? orow[(int64_t)gi * p.s_rs] : (uint16_t)0;
        }
    };

    const int NCHUNK = (Ki + KC - 1) / KC;
    load_x(0);
    load_w(0);
    store_x(0);
    if (NSLAB > 1) load_x(1);

    for (int c0 = 0; c0 < NCHUNK; c0 += PF) {
        v4i cur[PF];
        uint16_t scur[PF], ocur[PF];
#pragma unroll
        for (int i = 0; i < PF; i++) { cur[i] = wq[i]; scur[i] = sq[i]; ocur[i] = oq[i]; }
        if (c0 + PF < NCHUNK) load_w(c0 + PF);
#pragma unroll
        for (int i = 0; i < PF; i++) {
            const int c = c0 + i;
            if (i % CPS == 0) {
                // slab boundary: every wave is done with the previous slab and sees the current one; the slab after
                // it moves from registers to the buffer just vacated, and the one after that starts loading
                const int slab = c / CPS;
                __syncthreads();
                if (slab + 1 < NSLAB) store_x((slab + 1) & 1);
                if (slab + 2 < NSLAB) load_x(slab + 2);
            }
            // chunks past the end of K: their weights count as zero, but the x slab they would read may never have been
            // written (one slab only), and 0 x NaN from stale LDS is NaN
            if (c >= NCHUNK) continue;
            if (WK > 1 && (i % WK) != wk) continue;
            const int slab = c / CPS;
            const char* xs = sx + (slab & 1) * XSLAB;
            const int k = c * KC + g * KPL;   // first k of this lane's piece
            const bool live = k < Ki;
            const uint16_t sb = scur[i], ob = ocur[i];
#pragma unroll
            for (int s = 0; s < STEPS; s++) {
                // operand A: this lane's 8 dequantised weights for MFMA step s
                v4i aop;
                if constexpr (XDT == DT_F16 && WBITS == 4 && !WFLT) {
                    const _Float16 sh = __builtin_bit_cast(_Float16, sb), oh = __builtin_bit_cast(_Float16, ob);
                    h2 o4[4];
                    dequant_i4_f16(live ? (uint32_t)cur[i][s] : 0x88888888u, (h2){oh, oh}, (h2){sh, sh}, has_off, o4);
                    if (!live) { o4[0] = o4[1] = o4[2] = o4[3] = (h2){(_Float16)0.0f, (_Float16)0.0f}; }
                    aop = (v4i){(int)u32(o4[0]), (int)u32(o4[1]), (int)u32(o4[2]), (int)u32(o4[3])};
                } else if constexpr (XDT == DT_F16 && WBITS == 4 && WFLT) {
                    // e2m1 codes (no offset in the formats that carry them): packed-fp16 form
                    const _Float16 sh = __builtin_bit_cast(_Float16, sb);
                    h2 o4[4];
                    dequant_fp4_f16(live ? (uint32_t)cur[i][s] : 0u, (h2){sh, sh}, o4);
                    if (!live) { o4[0] = o4[1] = o4[2] = o4[3] = (h2){(_Float16)0.0f, (_Float16)0.0f}; }
                    aop = (v4i){(int)u32(o4[0]), (int)u32(o4[1]), (int)u32(o4[2]), (int)u32(o4[3])};
                } else {
                    float scf, off;
                    if constexpr (XDT == DT_F16) { scf = f16_to_f32(sb); off = f16_to_f32(ob); }
                    else { scf = bf16_to_f32(sb); off = bf16_to_f32(ob); }
                    uint16_t e[8];
                    if constexpr (WBITS == 4) {
                        const uint32_t q = (uint32_t)cur[i][s];
                        const int ord[8] = {0, 4, 1, 5, 2, 6, 3, 7};   // element order of the staged x
#pragma unroll
                        for (int j = 0; j < 8; j++) {
                            float wv;
                            if constexpr (WFLT) {
                                wv = e2m1_to_f32((q >> (4 * ord[j])) & 15u);
                            } else {
                                int v = (int)((q >> (4 * ord[j])) & 15u);
                                wv = (float)(v >= 8 ? v - 16 : v);
                            }
                            e[j] = live ? bits_x<XDT>(dequant_one<XDT>(wv, off, scf, has_off)) : (uint16_t)0;
                        }
                    } else {
                        // int8: 16 bytes per piece, step s uses bytes 8s..8s+7 in natural order
#pragma unroll
                        for (int j = 0; j < 8; j++) {
                            const uint32_t q = (uint32_t)cur[i][2 * s + (j >> 2)];
                            const uint32_t byte = (q >> (8 * (j & 3))) & 0xffu;
                            const float wv = WFLT ? e4m3_to_f32(byte) : (float)(int)(int8_t)byte;
                            e[j] = live ? bits_x<XDT>(dequant_one<XDT>(wv, off, scf, has_off)) : (uint16_t)0;
                        }
                    }
                    aop = (v4i){(int)(e[0] | ((uint32_t)e[1] << 16)), (int)(e[2] | ((uint32_t)e[3] << 16)),
                                (int)(e[4] | ((uint32_t)e[5] << 16)), (int)(e[6] | ((uint32_t)e[7] << 16))};
                }
                // operand B: x[m = 16b + nrow][k = chunk + g*KPL + 8s + 0..7] (already permuted for int4)
                const int kofs = ((c % CPS) * KC + g * KPL + 8 * s) * 2;
#pragma unroll
                for (int b = 0; b < MB; b++) {
                    const v4i bop = *(const v4i*)(xs + (16 * b + nrow) * XROW + kofs);
                    if constexpr (XDT == DT_F16) {
                        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, aop), __builtin_bit_cast(v8h, bop), acc[b], 0, 0, 0);
                    } else {
                        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, aop), __builtin_bit_cast(v8bf, bop), acc[b], 0, 0, 0);
                    }
                }
            }
        }
    }

    if constexpr (WK > 1) {
        // fixed-order reduction of the K-split partial sums: wave (wn, wk) parks its sums, wave (wn, 0) adds them
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
        if (r >= p.m_rows) continue;
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

template <int XDT, int WBITS, int MB, int WK, bool WFLT = false>
static int launch_decode(const WqParams& p, hipStream_t st)
{
    constexpr int KC = 4 * (128 / WBITS), KX = 8 * KC / MB, WN = 4 / WK;
    const size_t lds = 2 * (size_t)(16 * MB) * (KX * 2 + 16);
    const unsigned grid = (unsigned)((p.N + 16 * WN - 1) / (16 * WN));
    auto k = wqmm_decode_kernel<XDT, WBITS, MB, WK, WFLT>;
    static std::atomic<uint64_t> attr_set{0};   // one bit per device: the attribute belongs to the (kernel, device) pair
    if (!device_flag_test(attr_set)) {
        hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        device_flag_set(attr_set);
    }
    hipLaunchKernelGGL(k, dim3(grid), dim3(256), lds, st, p);
    return (int)hipGetLastError();
}

template <int XDT, int WBITS, int MB, bool WFLT = false>
static int launch_wk(const WqParams& p, hipStream_t st)
{
    // split K between the waves of a workgroup when column blocks alone would leave most of the chip idle
    const int64_t nblocks = (p.N + 15) / 16;
    if (nblocks < 1024 && p.K >= 2048) return launch_decode<XDT, WBITS, MB, 4, WFLT>(p, st);
    return launch_decode<XDT, WBITS, MB, 1, WFLT>(p, st);
}

template <> int launch_wq_stream<DT_F16, 4>(const WqParams&, const WqStreamOpts&, hipStream_t);
template <> int launch_wq_stream<DT_F16, 8>(const WqParams&, const WqStreamOpts&, hipStream_t);
template <> int launch_wq_stream<DT_BF16, 4>(const WqParams&, const WqStreamOpts&, hipStream_t);
template <> int launch_wq_stream<DT_BF16, 8>(const WqParams&, const WqStreamOpts&, hipStream_t);
template <> int launch_wq_xreg_float<DT_F16, 4>(const WqParams&, hipStream_t);
template <> int launch_wq_xreg_float<DT_F16, 8>(const WqParams&, hipStream_t);
template <> int launch_wq_xreg_float<DT_BF16, 4>(const WqParams&, hipStream_t);
template <> int launch_wq_xreg_float<DT_BF16, 8>(const WqParams&, hipStream_t);

// Can the streamlined kernel take this problem, and in which form?
template <int WBITS>
static bool stream_eligible(WqParams& p, WqStreamOpts& o)
{
    constexpr int64_t KC = 4 * (128 / WBITS);
    if (p.K % KC != 0) return false;
    const int64_t nch = p.K / KC;
    if (p.group >= p.K) p.cpg_shift = 31;
    else {
        if (p.group % KC != 0) return false;
        const int64_t cpg = p.group / KC;
        if (cpg & (cpg - 1)) return false;
        p.cpg_shift = __builtin_ctzll((unsigned long long)cpg);
    }
    o.has_off = p.offset != nullptr;
    const int64_t nblocks = (p.N + 15) / 16;
    o.ksplit = p.M <= 16 && nblocks < 1024 && nch % 4 == 0 && nch >= 8;
    const int64_t ngroups = p.group >= p.K ? 1 : p.K / p.group;
    o.vscale = !o.ksplit && p.group == KC && p.s_rs == 1 && p.s_cs % 8 == 0 && ngroups % 8 == 0 &&
               (uintptr_t)p.scale % 16 == 0 && (!p.offset || (uintptr_t)p.offset % 16 == 0);
    // few rows: x whole in LDS (<= 64 KB), K in four contiguous quarters per workgroup
    o.resx = p.M <= 16 && nch % 4 == 0 && (p.M + 1) * (p.K * 2 + 16) <= 65536;
    o.resx_vscale = o.resx && p.group == KC && p.s_rs == 1 && p.s_cs % 8 == 0 && (nch / 4) % 8 == 0 &&
                    (uintptr_t)p.scale % 16 == 0 && (!p.offset || (uintptr_t)p.offset % 16 == 0);
    // 4 to 16 rows (fewer stay on the kernel above): x in registers, K in 8 or 16 contiguous ranges per workgroup
    constexpr int xreg_min = 4, xreg_nw = 0;   // (0: xreg_shape picks the wave count)
    int xnw = 0, xnch = 0;
    o.xreg_nw = xreg_nw;
    // (with room for partial sums also a K of several workgroup segments, and then fewer than 4 rows too where x does not fit the LDS)
    int xsplits = 1;
    bool xexact = true;
    o.xreg = p.M <= 16 && xreg_shape(WBITS, p.K, xreg_nw, xnw, xnch, p.M, p.part != nullptr, &xsplits, &xexact) && (p.M >= xreg_min || (xsplits > 1 && !o.resx));
    o.xreg_vscale = o.xreg && p.group == KC && p.s_rs == 1 && p.s_cs % 8 == 0 && p.s_cs >= nch &&
                    (uintptr_t)p.scale % 16 == 0 && (!p.offset || (uintptr_t)p.offset % 16 == 0);
    // more than 32 rows: two weight blocks per wave share every x fragment, up to 128 rows per pass over the weights
    // (needs whole groups of chunks in flight and whole wave tiles of columns)
    // (measured on 8192 x 28672 int4, streaming kernel / this one: 17 rows 45 / 53 us, 32 rows 51 / 53, 40 rows 64 / 53,
    // 48 rows 68 / 53, 64 rows 54; on 4096 x 4096: 32 rows 17.5 / 15.7, 40 rows 23.5 / 16.0; int8 8192 x 28672: 32 rows
    // 55 / 68, 40 rows 75 / 68: hence the switch at 33 rows)
    constexpr int rows_min = 33;
    // (the kernel addresses the x rows of a slab, up to 256, with 32-bit byte offsets)
    o.rows_shape = nch % 2 == 0 && p.N % 32 == 0 && p.N >= 256 && p.K < (1ll << 23);
    o.rows = p.M >= rows_min && o.rows_shape;
    return true;
}

const void* weight_cache_get(const void* src, int64_t K, int64_t N, int bits, int64_t nb, hipStream_t st);   // weight_cache.hip
template <int XDT, int WBITS>
int launch_wq_tile(const WqParams& p, hipStream_t st);   // wqmm_tile.hip
}  // namespace opsnn
extern "C" int opsnn_wq_tile_min();   // dispatch.hip
extern "C" int opsnn_wq_narrow_slabs();
namespace opsnn {

// Up to 64 rows per slab, `slabs` slabs, and still at most 128 workgroups of 128 columns: the instance whose workgroups
// take 64 columns (K split over four waves instead of two; needs K in whole x slabs of four chunks) doubles their number.
template <int WBITS>
static int use_cols64(int64_t rows, int64_t slabs, int64_t N, int64_t K)
{
    constexpr int64_t KC = 4 * (128 / WBITS);
    return (rows <= 64 && slabs * ((N + 127) / 128) <= 128 && K % (4 * KC) == 0 && N % 32 == 0 && opsnn_wq_narrow_slabs()) ? 1 : 0;
}

// rows per slab of a narrow weight's one-launch form (0: one pass at a time)
static int64_t narrow_n_slab(int64_t M, int64_t N) { return wq_narrow_slab_rows(M, N, opsnn_wq_narrow_slabs() != 0); }

// floating-point weight codes: the general kernel, in row slabs of 64
template <int XDT, int WBITS>
static int launch_slabs_float(WqParams p, hipStream_t st)
{
    // up to 16 rows: x in registers (mxfp4: e2m1 codes with a row's e8m0 bytes contiguous; e4m3 codes with per-channel scales)
    if (p.M <= 16 && !p.offset) {
        bool ok;
        if (WBITS == 4) ok = p.scale_e8m0 && p.group == 32 && p.s_rs == 1 && p.s_cs % 16 == 0 && p.s_cs >= p.K / 32 && (uintptr_t)p.scale % 16 == 0;
        else ok = !p.scale_e8m0 && p.group >= p.K;
        if (ok) {
            p.m_base = 0; p.m_rows = p.M; p.cpg_shift = 31;
            const int rc = launch_wq_xreg_float<XDT, WBITS>(p, st);
            if (rc != OPSNN_NOT_TAKEN) return rc;
        }
    }
    // more rows: the many-rows streaming kernel, up to 256 rows per pass over the weights
    {
        constexpr int64_t KC = 4 * (128 / WBITS);
        constexpr int rows_min = 17;
        bool ok = !p.offset && p.M >= rows_min && p.K % KC == 0 && (p.K / KC) % 2 == 0 && p.N % 32 == 0 && p.N >= 256 && p.K < (1ll << 23);
        const bool mx8 = WBITS == 8 && p.scale_e8m0 && p.mx8_rows;   // e4m3 codes with e8m0 scales per 32 (MXFP8's x2: launch_wq_mx8_rows)
        if (WBITS == 4 || mx8) ok = ok && p.scale_e8m0 && p.group == 32 && p.s_rs == 1;
        else ok = ok && !p.scale_e8m0 && p.group >= p.K;
        // (the kernel's scale table counts in words of four e8m0 bytes = 128 k: one chunk of e2m1 codes, two of e4m3 codes)
        const int cpg = WBITS == 4 ? 0 : mx8 ? 1 : 31;
        // (the 192- / 256-row instances want K in whole rounds of four x slabs)
        const int64_t nslab = narrow_n_slab(p.M, p.N);
        if (ok && (p.K / KC) % 8 != 0 && (nslab ? nslab : p.M) > 128) ok = false;
        if (ok) {
            // (a long K against few workgroups: K in segments as well, then on 128-column workgroups)
            int64_t kunit = 0;
            const int ks = p.part ? wq_rows_ksplit(WBITS, p.M, p.N, p.K, p.group, opsnn_wq_narrow_slabs() != 0, &kunit) : 1;
            p.ksplit = ks > 1 ? ks : 0;
            p.kunit = kunit;
            if (const int64_t slab = narrow_n_slab(p.M, p.N)) {   // narrow N: all row slabs in one launch
                p.cpg_shift = cpg;
                p.m_base = 0; p.m_rows = slab; p.m_slab = slab; p.m_end = p.M;
                p.cols64 = ks > 1 || mx8 ? 0 : use_cols64<WBITS>(slab, (p.M + slab - 1) / slab, p.N, p.K);
                return launch_wq_rows_float<XDT, WBITS>(p, st);
            }
            p.cols64 = ks > 1 || mx8 ? 0 : use_cols64<WBITS>(p.M, 1, p.N, p.K);
            // up to 128 rows one pass; more: whole passes of 256 rows and the rest in one (as for integer codes below)
            const int64_t slab = p.M <= 128 ? 128 : 256;
            p.cpg_shift = cpg;
            for (int64_t m0 = 0; m0 < p.M; m0 += slab) {
                p.m_base = m0;
                p.m_rows = (p.M - m0) < slab ? (p.M - m0) : slab;
                const int rc = launch_wq_rows_float<XDT, WBITS>(p, st);
                if (rc != 0) return rc;
            }
            return 0;
        }
    }
    for (int64_t m0 = 0; m0 < p.M; m0 += 64) {
        p.m_base = m0;
        p.m_rows = (p.M - m0) < 64 ? (p.M - m0) : 64;
        int rc;
        if (p.m_rows <= 16) rc = launch_wk<XDT, WBITS, 1, true>(p, st);
        else if (p.m_rows <= 32) rc = launch_wk<XDT, WBITS, 2, true>(p, st);
        else rc = launch_wk<XDT, WBITS, 4, true>(p, st);
        if (rc != 0) return rc;
    }
    return 0;
}

template <int XDT, int WBITS>
static int launch_slabs(WqParams p, hipStream_t st)
{
    // many rows: the dequantise-once tile kernel, one pass over the weight for up to 256 rows.  (Measured on 8192 x 28672
    // int4, group 128: 256 rows 165 us against 207 in two passes of the streaming kernel below; 128 rows 116 against 105,
    // 64 rows 94 against 69 -- hence the default switch at 129 rows; opsnnSetWqTileMin moves it.)
    // From 129 rows: first the 256-row instance of the many-rows kernel (one pass over the weights per 256 rows, every weight
    // dequantised once per wave and multiplied with all sixteen row blocks of x; needs the scale table in LDS), in equal
    // slabs of up to 256 rows; then the tile kernel.  (Measured on 8192 x 28672 int4, fp16: 256 rows 151-155 us against 170 on
    // the tile kernel, 192 rows 142-149 against 168.  Test hook: opsnnSetWqTileMin(m <= 128) sends such calls to the tile
    // kernel first.)
    // narrow N against a long K, from 17 rows: the row slabs in one launch and K in segments on top
    if (p.part && opsnn_wq_tile_min() > 128) {
        const int64_t slab = p.M <= 64 ? 0 : narrow_n_slab(p.M, p.N);
        int64_t kunit = 0;
        const int ks = wq_rows_ksplit(WBITS, p.M, p.N, p.K, p.group, opsnn_wq_narrow_slabs() != 0, &kunit);
        WqParams q = p;
        WqStreamOpts o{};
        if (ks > 1 && (p.M <= 64 || slab > 0) && stream_eligible<WBITS>(q, o) && o.rows_shape) {
            o.rows = true;   // (with K in segments the many-rows kernel is ahead from 17 rows: 48 x 28672 x 8192 int4 153 -> 53 us)
            q.m_base = 0; q.m_rows = q.M;
            if (slab > 0) { q.m_rows = slab; q.m_slab = slab; q.m_end = q.M; }
            q.ksplit = ks;
            q.kunit = kunit;
            const int rc = launch_wq_stream<XDT, WBITS>(q, o, st);
            if (rc != OPSNN_NOT_TAKEN) return rc;
        }
    }
    if (opsnn_wq_tile_min() > 128) {
        if (const int64_t slab = narrow_n_slab(p.M, p.N)) {   // narrow N: all row slabs in one launch
            WqParams q = p;
            WqStreamOpts o{};
            if (stream_eligible<WBITS>(q, o) && o.rows) {
                q.m_base = 0; q.m_rows = slab; q.m_slab = slab; q.m_end = q.M;
                q.cols64 = use_cols64<WBITS>(slab, (q.M + slab - 1) / slab, q.N, q.K);
                const int rc = launch_wq_stream<XDT, WBITS>(q, o, st);
                if (rc != OPSNN_NOT_TAKEN) return rc;
            }
        }
    }
    if (p.M > 128 && opsnn_wq_tile_min() > 128) {
        WqParams q = p;
        WqStreamOpts o{};
        if (stream_eligible<WBITS>(q, o) && o.rows) {
            // whole passes of 256 rows, then the rest in one pass (up to 128 rows: the smaller instances, whose time grows
            // with the rows they serve; measured at 300 rows: 256 + 44 rows 20 % ahead of two passes of 150)
            const int64_t slab = 256;
            bool taken = true;
            for (int64_t m0 = 0; m0 < q.M && taken; m0 += slab) {
                q.m_base = m0;
                q.m_rows = (q.M - m0) < slab ? (q.M - m0) : slab;
                const int rc = launch_wq_stream<XDT, WBITS>(q, o, st);
                // (the kernel's conditions look at K, N, the group size and the scale layout, not at the slab: a refusal
                // can only come before anything has been written)
                if (rc == OPSNN_NOT_TAKEN && m0 == 0) taken = false;
                else if (rc != 0) return rc;
            }
            if (taken) return 0;
        }
    }
    if (p.M >= opsnn_wq_tile_min() && p.M <= 256) {
        const int rc = launch_wq_tile<XDT, WBITS>(p, st);
        if (rc != OPSNN_NOT_TAKEN) return rc;
    }
    // more rows still: the same kernel in passes of up to 256 rows, in equal slabs (2048 rows: 8 passes over the weight
    // instead of 16 of the streaming kernel)
    if (p.M > 256 && opsnn_wq_tile_min() <= 256) {
        const int64_t passes = (p.M + 255) / 256;
        const int64_t slab = ((p.M + passes - 1) / passes + 15) / 16 * 16;
        bool taken = true;
        for (int64_t m0 = 0; m0 < p.M && taken; m0 += slab) {
            WqParams q = p;
            q.x = p.x + m0 * p.K;
            q.y = p.y + m0 * p.N;
            q.M = (p.M - m0) < slab ? (p.M - m0) : slab;
            const int rc = launch_wq_tile<XDT, WBITS>(q, st);
            // launch_wq_tile's conditions hold for every slab once they hold for the first (slabs are no larger, K % 64 == 0
            // keeps their x rows 16-byte aligned), so a refusal can only come before anything has been written
            if (rc == OPSNN_NOT_TAKEN && m0 == 0) taken = false;
            else if (rc != 0) return rc;
        }
        if (taken) return 0;
    }
    WqStreamOpts o{};
    const bool stream = stream_eligible<WBITS>(p, o);
    // rows per launch: as many as one pass over the weights can serve, in equal slabs
    int64_t slab = 64;
    if (stream && o.rows) {
        const int64_t passes = (p.M + 127) / 128;
        slab = ((p.M + passes - 1) / passes + 15) / 16 * 16;
        p.cols64 = use_cols64<WBITS>(p.M, 1, p.N, p.K);
    }
    for (int64_t m0 = 0; m0 < p.M; m0 += slab) {
        p.m_base = m0;
        p.m_rows = (p.M - m0) < slab ? (p.M - m0) : slab;
        int rc;
        if (stream) rc = launch_wq_stream<XDT, WBITS>(p, o, st);
        else if (p.m_rows <= 16) rc = launch_wk<XDT, WBITS, 1>(p, st);
        else if (p.m_rows <= 32) rc = launch_wk<XDT, WBITS, 2>(p, st);
        else rc = launch_wk<XDT, WBITS, 4>(p, st);
        if (rc != 0) return rc;
    }
    return 0;
}

// MXFP8 with 33 rows of x1 and more on the many-rows kernel: p.x is x1 widened to bf16 with its block scales folded in, p.w
// x2's e4m3 codes (K-contiguous), p.scale x2's e8m0 bytes (a row's bytes contiguous), p.y bf16.  The caller has checked the
// shape (the conditions of launch_slabs_float's many-rows branch); OPSNN_NOT_TAKEN if the kernel declines.
int launch_wq_mx8_rows(const WqParams& p0, hipStream_t st)
{
    WqParams p = p0;
    p.w_float = 1; p.scale_e8m0 = 1; p.mx8_rows = 1; p.group = 32; p.group_shift = 5; p.s_rs = 1; p.offset = nullptr;
    constexpr int64_t KC = 64;
    if (p.M < 17 || p.K % (2 * KC) != 0 || p.N % 32 != 0 || p.N < 256 || p.K >= (1ll << 23)) return OPSNN_NOT_TAKEN;
    const int64_t nslab = narrow_n_slab(p.M, p.N);
    if ((p.K / KC) % 8 != 0 && (nslab ? nslab : p.M) > 128) return OPSNN_NOT_TAKEN;
    return launch_slabs_float<DT_BF16, 8>(p, st);
}

int launch_wqmm_mfma(const OpsnnWqmmArgs& a0, hipStream_t st)
{
    OpsnnWqmmArgs a = a0;
    if (a.x_dtype != DT_F16 && a.x_dtype != DT_BF16) return OPSNN_NOT_TAKEN;
    const bool wflt = a.w_dtype == DT_E2M1 || a.w_dtype == DT_E4M3;
    if (a.w_dtype != DT_I4 && a.w_dtype != DT_I8 && !wflt) return OPSNN_NOT_TAKEN;
    const bool mx = wflt && a.scale_dtype == DT_E8M0;
    if (a.scale_dtype != a.x_dtype && !mx) return OPSNN_NOT_TAKEN;
    if (mx && (a.offset || a.group <= 0 || a.scale_n == 1)) return OPSNN_NOT_TAKEN;
    if (a.w_dtype == DT_E2M1 && a.offset) return OPSNN_NOT_TAKEN;   // the packed e2m1 dequantisation has no offset step
    const int wbits = (a.w_dtype == DT_I4 || a.w_dtype == DT_E2M1) ? 4 : 8;
    // up to 16 rows against a long K: the partial sums of the x-in-registers kernel's K split sit at the front of the workspace
    // (and those of the many-rows kernel's K split against a narrow N)
    float* part = nullptr;
    if (const int xs = wq_part_slices(wbits, a.M, a.N, a.K, a.group > 0 ? a.group : a.K, opsnn_wq_narrow_slabs() != 0); xs > 1 && a.workspace) {
        part = (float*)a.workspace;
        const uint64_t pb = ((uint64_t)xs * (uint64_t)a.M * (uint64_t)a.N * 4 + 255) / 256 * 256;
        const bool relayout = a.w.row_stride != 1 && a.K != 1;
        a.workspace = relayout ? (char*)a.workspace + pb : nullptr;
    }
    const int64_t kpl = 128 / wbits;
    if (a.K % kpl != 0 || a.K < kpl) return OPSNN_NOT_TAKEN;
    const int64_t group = a.group > 0 ? a.group : a.K;
    if (group % kpl != 0) return OPSNN_NOT_TAKEN;   // a lane's piece must lie inside one group
    if (a.w.row_stride != 1) {
        // weight is [K, N] with N contiguous: the K-contiguous copy comes from the weight cache when that is switched on,
        // else it is re-laid out into the workspace
        if (a.w.col_stride != 1 || a.w.row_stride != a.N || a.K == 1) return OPSNN_NOT_TAKEN;
        if (const void* cached = weight_cache_get(a.w.ptr, a.K, a.N, wbits, 1, st)) a.w.ptr = cached;
        else {
            if (!a.workspace) return OPSNN_NOT_TAKEN;
            int rc = wbits == 4 ? opsnnTranspose4(a.w.ptr, a.workspace, a.K, a.N, 1, st) : opsnnTranspose8(a.w.ptr, a.workspace, a.K, a.N, 1, st);
            if (rc != 0) return rc;
            a.w.ptr = a.workspace;
        }
        a.w.row_stride = 1; a.w.col_stride = a.K;
    }
    WqParams p{};
    p.x = (const uint16_t*)a.x;
    p.w = (const uint8_t*)a.w.ptr;
    p.ldw = a.w.col_stride * wbits / 8;
    p.scale = (const uint16_t*)a.scale.ptr; p.offset = (const uint16_t*)a.offset;
    p.s_rs = a.scale.row_stride; p.s_cs = a.scale_n == 1 ? 0 : a.scale.col_stride;
    p.bias = a.bias; p.bias_dt = a.bias_dtype;
    p.y = (uint16_t*)a.y; p.M = a.M; p.N = a.N; p.K = a.K; p.group = group;
    p.part = part;
    p.group_shift = (group & (group - 1)) == 0 ? __builtin_ctzll((unsigned long long)group) : -1;
    if (a.K >= (1ll << 31) || a.N >= (1ll << 31)) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)p.w | (uint64_t)p.ldw) % 16 || ((uintptr_t)p.x % 16) || (a.K % 8)) return OPSNN_NOT_TAKEN;
    if (wflt) {
        p.w_float = 1;
        p.scale_e8m0 = mx ? 1 : 0;
        if (a.x_dtype == DT_F16) return wbits == 4 ? launch_slabs_float<DT_F16, 4>(p, st) : launch_slabs_float<DT_F16, 8>(p, st);
        return wbits == 4 ? launch_slabs_float<DT_BF16, 4>(p, st) : launch_slabs_float<DT_BF16, 8>(p, st);
    }
    if (a.x_dtype == DT_F16) return wbits == 4 ? launch_slabs<DT_F16, 4>(p, st) : launch_slabs<DT_F16, 8>(p, st);
    return wbits == 4 ? launch_slabs<DT_BF16, 4>(p, st) : launch_slabs<DT_BF16, 8>(p, st);
}

}  // namespace opsnn
