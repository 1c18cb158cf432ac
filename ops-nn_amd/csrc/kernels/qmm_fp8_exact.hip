// fp8 e4m3 x fp8 e4m3 quantized matmul whose products and partial sums are exact: the operands are widened to fp16 in
// registers (every e4m3 value, subnormals included, is an fp16 value) and contracted by v_mfma_f32_16x16x32_f16.
//
//   block scales:      out[m,n] = cast( sum_kb ( sum_{k in block kb} x1[m,k] * x2[k,n] ) * ( s1[m/gsM, kb] * s2[kb, n/128] ) )
//   row/column scales: out[m,n] = cast( (sum_k x1[m,k] * x2[k,n]) * cs[n] * rs[m] + bias[n] )
//
// Formulas: matmul/quant_batch_matmul_v3/tests/assets/qbmmv3_kernel_golden.py:237-358 (the two block scales are
// multiplied together first, :337-343) and :361-387; device counterpart in the reference:
// matmul/common/cmct/epilogue/block_epilogue_pertile.h:502-642.
//
// Why not the 8-bit matrix instruction: on gfx950 it aligns its 128 products in a window narrower than fp32 (measured
// on N(0,1) data rounded to e4m3: mean error 1.2e-6, max 1.6e-5 of sum|terms| per instruction), which leaves about 1 %
// of the bf16 outputs one ulp from the fp32-accumulated result at K = 7168 and a few two ulps away where the terms
// cancel.  The fp16 instruction's products (22 significant bits) are summed like an fp32 accumulation or better
// (measured: bit-identical to the correctly rounded exact sum of 128 products in 99.5 % of cases, never further than
// fp32 ascending-k summation), at half the matrix rate.
//
// Tiling: 256 x 128 output tile per workgroup, 4 x 2 waves of 64 x 64 (4 x 4 fragments of 16 x 16).  The operands stay
// e4m3 bytes on the way global -> LDS (16-byte asynchronous copies, rows XOR-swizzled) and LDS -> registers, exactly as
// in qmm_fp8_block.hip; a lane's 32 bytes of a fragment become sixteen registers of fp16 pairs by sixteen
// v_cvt_scalef32_pk_f16_fp8 (unit scale).  The x1 fragments are widened once per K tile and stay (64 registers), the
// x2 fragments as they stream through.  One K tile is one 128-wide scale block: a chain of four instructions from a
// zero accumulator leaves the block's partial sums in four registers, and the vector ALU folds them into the fp32
// running sums (one fma each) one fragment pair later, in the shadow of the next chain.
#include "launch.h"
#include "qgemm_core.hip.h"

namespace opsnn {

struct Fp8xParams {
    const int8_t* a;
    const int8_t* b;
    int64_t lda, ldb, a_bs, b_bs;
    void* out;
    int64_t M, N, K;
    const float* s1;   // element (m/gsM, kb) at s1[(m/gsM)*s1_rs + kb*s1_cs]
    const float* s2;   // element (kb, nb) at s2[kb*s2_rs + nb*s2_cs]
    int64_t s1_rs, s1_cs, s1_bs, s2_rs, s2_cs, s2_bs;
    int gsM;           // 1 or 128
    // row / column scale mode: out = (sum * cs[n * cs_stride]) * rs[m * rs_stride] + bias[n]; strides 0 (one scale) or 1
    // ep_mode 1 (no row scale; a float bias is added BEFORE the scaling):   out = (sum + bias[n]) * cs[n]
    // ep_mode 2 (one row scale, one column scale, merged and truncated):    out = sum * trunc19(cs[0] * rs[0])
    // (compute_tc, qbmmv3_kernel_golden.py:390-475).  cs may be fp32, bf16 or 64-bit words (fp32 in the low word, upper
    // 19 bits kept); rs may be null (= 1).
    const float* rs;
    const void* cs;
    int rs_stride, cs_stride;
    int cs_dt, ep_mode;
    const void* bias;   // fp32, or 16-bit floats widened on the way in (bias_dt)
    int bias_dt;
    int64_t bias_bs;
    int64_t rs_bs, cs_bs;   // batch strides of rs / cs in elements (0: shared by all batches)
    // MX mode (template flag MXS): one e8m0 byte per 32 K and row, four per K tile (sa, sb: K-contiguous, 4-byte aligned
    // rows).  Every row has a base exponent; the widening conversion multiplies a block by 2^(byte - base), exactly (the
    // result is an fp16 value as long as byte - base is in [-15, 7]), and 2^(base - 127) comes back in through rs / cs.
    // a_c / b_c hold 127 - base per row; gate[0 .. gate_n) are flags of the pass that chose the bases: any flag set means
    // some row's bytes do not fit that window, and the kernel leaves the whole call to the launch that follows it.
    const uint8_t* sa;
    const uint8_t* sb;
    int64_t sa_rs, sb_rs, sa_bs, sb_bs;
    const int* a_c;
    const int* b_c;
    const int* gate;
    int gate_n;
    // K split over `splits` workgroups per tile (SPLIT instantiations, grid.z): fp32 partial sums [splits][batch][M][N] --
    // block scales already applied, row / column scales and bias not yet (fp8x_splitk_reduce_kernel applies them)
    int splits;
    float* part;
#if QG_DBG
    unsigned long long* dbg;   // timing harness only: per wave, loop clocks / barrier-wait clocks / K tiles
#endif
};

__device__ __forceinline__ const int8_t* uniform_ptr(const int8_t* p)
{
    const uint64_t u = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u), hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
    return (const int8_t*)(((uint64_t)hi << 32) | lo);
}

// Eight e4m3 bytes (two registers) -> eight fp16 values (four registers), exact.
// two of a dword's four fp8 codes -> fp16, exact: every e4m3 and every e5m2 value is an fp16 value (E5: the code is e5m2)
template <bool E5> __device__ __forceinline__ v2h cvt_lo(uint32_t d)
{
    if constexpr (E5) return __builtin_amdgcn_cvt_scalef32_pk_f16_bf8(d, 1.0f, false);
    else return __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d, 1.0f, false);
}
template <bool E5> __device__ __forceinline__ v2h cvt_hi(uint32_t d)
{
    if constexpr (E5) return __builtin_amdgcn_cvt_scalef32_pk_f16_bf8(d, 1.0f, true);
    else return __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d, 1.0f, true);
}
template <bool E5> __device__ __forceinline__ v8h widen8(int d0, int d1)
{
    const v2h a = cvt_lo<E5>((uint32_t)d0), b = cvt_hi<E5>((uint32_t)d0), c = cvt_lo<E5>((uint32_t)d1), d = cvt_hi<E5>((uint32_t)d1);
    return (v8h){a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}

// the same with the power of two `sc` multiplied in (e4m3 only): exact while the scaled value is an fp16 value
__device__ __forceinline__ v8h widen8_scaled(int d0, int d1, float sc)
{
    const v2h a = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((uint32_t)d0, sc, false), b = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((uint32_t)d0, sc, true);
    const v2h c = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((uint32_t)d1, sc, false), d = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((uint32_t)d1, sc, true);
    return (v8h){a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}

// FMT: bit 0 set = x1 holds e5m2 codes, bit 1 set = x2 does (else e4m3)
// MXS: MX block scales (e8m0 per 32 K) folded into the widening conversion; row / column epilogue (RC) with the bases
// The epilogue of the row / column scale forms for one output (Fp8xParams::ep_mode); rs = the row's scale (1 if none)
__device__ __forceinline__ float fp8x_rowcol_epilogue(const Fp8xParams& p, float v, float rs, int64_t bz, int64_t ni)
{
    const int64_t ci = bz * p.cs_bs + ni * p.cs_stride;
    float csv;
    if (p.cs_dt == DT_U64) csv = u2f((uint32_t)((const uint64_t*)p.cs)[ci] & 0xFFFFE000u);
    else if (p.cs_dt == DT_BF16) csv = bf16_to_f32(((const uint16_t*)p.cs)[ci]);
    else csv = ((const float*)p.cs)[ci];
    if (p.ep_mode == 1) {
        if (p.bias) v = v + load_scalar_as_f32(p.bias, p.bias_dt, bz * p.bias_bs + ni);
        v = v * csv;
    } else if (p.ep_mode == 2) {
        v = v * u2f(f2u(csv * rs) & 0xFFFFE000u);
    } else {
        v = (v * csv) * rs;
        if (p.bias) v = v + load_scalar_as_f32(p.bias, p.bias_dt, bz * p.bias_bs + ni);
    }
    return v;
}

template <int OUT_DT, bool RC, int FMT = 0, bool MXS = false, bool SPLIT = false>
__global__ __launch_bounds__(512, 1) void qmm_fp8_exact_kernel(Fp8xParams p, int tiles_m, int tiles_n)
{
    static_assert(!MXS || (RC && FMT == 0), "the MX mode is e4m3 x e4m3 with the row / column epilogue");
    constexpr bool AE5 = (FMT & 1) != 0, BE5 = (FMT & 2) != 0;
    constexpr int BM = 256, BN = 128, BK = 128, NT = 512;
    constexpr int CPR = BK / 16, RPW = 16 / CPR;
    constexpr int TM = 64, TN = 64, FM = TM / 16, FN = TN / 16;
    constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
    constexpr bool SCC = !RC || MXS;                 // a 4-byte copy per lane rides with every K tile
    constexpr int SC_BYTES = SCC ? NT * 4 : 0;       // block scales: BM s1 floats + the s2 float of the tile's n block; MX: four e8m0 bytes per tile row
    constexpr int STAGE = A_BYTES + B_BYTES + SC_BYTES;
    constexpr int RPI = NT / CPR;                    // 64 tile rows per copy instruction of the workgroup
    constexpr int NA = BM / RPI, NB = BN / RPI;
    constexpr int CPT = NA + NB + (SCC ? 1 : 0);
    // Three stages: the tile being consumed, the next one (complete at this tile's barrier) and one more in flight, so a
    // copy has two tile times to land.  With two stages a copy had one tile time, about 1.1 us of matrix work, and the
    // loaded latency of an L2 miss is longer: the loop ran at the pace of the memory latency (measured: copies and
    // barriers alone 0.70 ms of config 4's 1.0).
    constexpr int STAGES = 3;
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    if constexpr (MXS) {
        int f = 0;
        for (int i = 0; i < p.gate_n; i++) f |= p.gate[i];   // (every thread reads every flag: uniform loads)
        if (f) return;   // some row's scale bytes do not fit the exact window: the next launch computes the call
    }

    // Tile order: each XCD (own L2) gets a contiguous range of ids, and ids run down groups of GM row tiles and across
    // the columns inside a group, so the 32 tiles an XCD works on at a time form a GM x (32 / GM) block that shares
    // GM x1 panels and 32 / GM x2 panels (for GM = 4: 2 KB-steps of 256 KB instead of 557 KB with whole columns).
    constexpr int GM = 4;
    const uint32_t t = xcd_remap(blockIdx.x, (uint32_t)(tiles_m * tiles_n));
    const uint32_t gsz_full = (uint32_t)(GM * tiles_n), grp = t / gsz_full, in_grp = t % gsz_full;
    const int first_m = (int)grp * GM;
    const int gh = tiles_m - first_m < GM ? tiles_m - first_m : GM;
    const int tm = first_m + (int)(in_grp % (uint32_t)gh), tn = (int)(in_grp / (uint32_t)gh);
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    const int64_t bz = blockIdx.y;
    const int64_t lda = p.lda, ldb = p.ldb;
    const int8_t* A = p.a + bz * p.a_bs + m0 * lda;
    const int8_t* B = p.b + bz * p.b_bs + n0 * ldb;
    int KT = (int)(p.K / BK);
    int kt_first = 0;   // SPLIT: this workgroup's K tiles are kt_first .. kt_first + KT - 1 (at least one)
    if constexpr (SPLIT) {
        const int z = (int)blockIdx.z;
        kt_first = (int)((int64_t)z * KT / p.splits);
        KT = (int)((int64_t)(z + 1) * KT / p.splits) - kt_first;
        A += (int64_t)kt_first * BK;
        B += (int64_t)kt_first * BK;
    }

    // copies: instruction i of the workgroup fills tile rows i*64 .. i*64+63; this thread handles row i*64 + tid/8 and
    // the logical 16-byte chunk that belongs at position tid%8 of the swizzled row.  Rows past the matrix edge repeat
    // the last valid row: they only feed outputs that are never stored.
    const int crow = tid / CPR;
    const int cchunk = (tid % CPR) ^ ((crow / RPW) & (CPR - 1));
    const int a_rows = (int)((p.M - m0) < BM ? (p.M - m0) : BM);
    const int b_rows = (int)((p.N - n0) < BN ? (p.N - n0) : BN);
    uint32_t a_off[NA], b_off[NB];
#pragma unroll
    for (int i = 0; i < NA; i++) {
        int r = i * RPI + crow;
        r = r < a_rows ? r : a_rows - 1;
        a_off[i] = (uint32_t)(r * lda + cchunk * 16);
    }
#pragma unroll
    for (int i = 0; i < NB; i++) {
        int r = i * RPI + crow;
        r = r < b_rows ? r : b_rows - 1;
        b_off[i] = (uint32_t)(r * ldb + cchunk * 16);
    }
    // scale copy: lanes 0..255 (waves 0..3) fetch s1 of tile row `tid`, the others the s2 of this tile's n block: a
    // wave-uniform table base, a 32-bit byte offset per lane (the launcher checks that the tables stay below 4 GB)
    const char* sc_base = nullptr;
    uint32_t sc_off = 0;
    int64_t sc_step = 0;   // bytes per K tile
    if constexpr (MXS) {   // lanes 0..255: the four bytes of x1 row `tid`; the others: of x2 row tid - 256 (the last 128 lanes repeat the last row)
        if (wave < BM / 64) {
            const int r = tid < a_rows ? tid : a_rows - 1;
            sc_base = (const char*)(p.sa + bz * p.sa_bs + m0 * p.sa_rs);
            sc_off = (uint32_t)(r * p.sa_rs);
        } else {
            const int r = tid - BM < b_rows ? tid - BM : b_rows - 1;
            sc_base = (const char*)(p.sb + bz * p.sb_bs + n0 * p.sb_rs);
            sc_off = (uint32_t)(r * p.sb_rs);
        }
        sc_step = 4;
    } else if constexpr (!RC) {
        if (wave < BM / 64) {
            const int r = tid < a_rows ? tid : a_rows - 1;
            sc_base = (const char*)(p.s1 + bz * p.s1_bs);
            sc_off = (uint32_t)(((m0 + r) / p.gsM) * p.s1_rs * 4);
            sc_step = p.s1_cs * 4;
        } else {
            sc_base = (const char*)(p.s2 + bz * p.s2_bs + (n0 / 128) * p.s2_cs);
            sc_step = p.s2_rs * 4;
        }
    }
    if constexpr (SPLIT) sc_base += (int64_t)kt_first * sc_step;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)smem + (uint32_t)wave * 1024u;
    const uint32_t lds_sc0 = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)smem + A_BYTES + B_BYTES + (uint32_t)wave * 256u;
    auto issue_piece = [&](int kt, int stage, int idx) {
        const uint32_t sA = lds0 + stage * STAGE, sB = sA + A_BYTES;
        if (idx < NA) copy16_sbase(uniform_ptr(A + (int64_t)kt * BK), a_off[idx], sA + idx * NT * 16);
        else if (idx < NA + NB) copy16_sbase(uniform_ptr(B + (int64_t)kt * BK), b_off[idx - NA], sB + (idx - NA) * NT * 16);
        else copy4_sbase(uniform_ptr((const int8_t*)sc_base + (int64_t)kt * sc_step), sc_off, lds_sc0 + stage * STAGE);
    };
    auto issue_tile = [&](int kt) {
#pragma unroll
        for (int idx = 0; idx < CPT; idx++) issue_piece(kt, kt % STAGES, idx);
    };

    v4f acc[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; i++)
#pragma unroll
        for (int j = 0; j < FM; j++) acc[i][j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    // Fragment of a 16-row block, lane (row = lane%16, q = lane/16): the bytes [16q, 16q+16) and [64+16q, 64+16q+16) of
    // the row's 128 bytes of K; instruction s of the chain of four takes eight of them from both operands (K is the
    // contraction index: any assignment of K to lanes and steps is right as long as both operands use the same one).
    const int frow = lane & 15, fq = lane >> 4;
    const int key = (frow / RPW) & (CPR - 1);
    const int ch0 = (fq ^ key) << 4, ch1 = ((4 + fq) ^ key) << 4;
    const int a_rowbase = (wm * TM + frow) * BK;
    const int b_rowbase = A_BYTES + (wn * TN + frow) * BK;
    auto load_frag = [&](const char* st, int rowbase) -> v8i {
        const v4i lo = *(const v4i*)(st + rowbase + ch0);
        const v4i hi = *(const v4i*)(st + rowbase + ch1);
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };

    issue_tile(0);
    issue_tile(KT > 1 ? 1 : 0);   // (a K of one or two tiles repeats the last tile into stages nobody reads)
    issue_tile(KT > 2 ? 2 : KT - 1);
    wait_vmcnt<2 * CPT>();
    __builtin_amdgcn_s_barrier();

    // Registers: fa[j][s] the x1 fragments of the current tile as fp16 (eight values per K step s), fbc[2][s] the current
    // and the next x2 fragment as fp16, a_half[j] sixteen raw bytes per x1 fragment on their way to fp16 (first the low
    // halves of the next tile, then its high halves), b_raw the raw bytes of the next x2 fragment.
    v4i a_half[FM];
    v8i b_raw;
    v8h fa[FM][4], fbc[2][4];
    float sc[FM], scp[FM], s1raw[FM], s2raw = 0.0f;
    v4f part[2][FM];
    (void)sc; (void)scp; (void)s1raw; (void)s2raw; (void)part;
    // MX: raw scale dwords of the tile being converted (one per fragment row of this lane), 127 - base of those rows, and
    // the powers of two for the lane's two K blocks of a tile: bytes [16q, 16q+16) lie in block q/2, [64+16q, ..) in 2 + q/2
    uint32_t a_sraw[FM], b_sraw[FN];
    int a_c[FM], b_c[FN];
    float a_lo[FM], a_hi[FM], b_lo[FN], b_hi[FN];
    (void)a_sraw; (void)b_sraw; (void)a_c; (void)b_c; (void)a_lo; (void)a_hi; (void)b_lo; (void)b_hi;
    const int sblk = 8 * (fq >> 1);
    if constexpr (MXS) {
#pragma unroll
        for (int j = 0; j < FM; j++) {
            const int r = wm * TM + j * 16 + frow;
            a_c[j] = p.a_c[bz * p.rs_bs + m0 + (r < a_rows ? r : a_rows - 1)];
        }
#pragma unroll
        for (int i = 0; i < FN; i++) {
            const int r = wn * TN + i * 16 + frow;
            b_c[i] = p.b_c[bz * p.cs_bs + n0 + (r < b_rows ? r : b_rows - 1)];
        }
    }
    auto mx_pow = [&](uint32_t raw, int c, float& lo, float& hi) {
        lo = u2f((((raw >> sblk) & 0xFFu) + (uint32_t)c) << 23);
        hi = u2f((((raw >> (16 + sblk)) & 0xFFu) + (uint32_t)c) << 23);
    };
    auto read_scales = [&](const char* st) {
        if constexpr (MXS) {
            const uint32_t* sS = (const uint32_t*)(st + A_BYTES + B_BYTES);
#pragma unroll
            for (int j = 0; j < FM; j++) a_sraw[j] = sS[wm * TM + j * 16 + frow];
#pragma unroll
            for (int i = 0; i < FN; i++) b_sraw[i] = sS[BM + wn * TN + i * 16 + frow];
        } else if constexpr (!RC) {
            const float* sS = (const float*)(st + A_BYTES + B_BYTES);
            s2raw = sS[BM];
#pragma unroll
            for (int j = 0; j < FM; j++) s1raw[j] = sS[wm * TM + j * 16 + frow];
        }
    };
    auto widen4 = [&](int d, v8h& h, int half, float scl) {   // four bytes -> elements 4*half .. 4*half+3
        v2h lo, hi;
        if constexpr (MXS) {
            lo = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((uint32_t)d, scl, false);
            hi = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((uint32_t)d, scl, true);
        } else {
            lo = cvt_lo<BE5>((uint32_t)d); hi = cvt_hi<BE5>((uint32_t)d);
        }
        h[4 * half] = lo[0]; h[4 * half + 1] = lo[1]; h[4 * half + 2] = hi[0]; h[4 * half + 3] = hi[1];
    };
    auto widen_a = [&](int d0, int d1, int j, int s) -> v8h {   // K step s of x1 fragment j
        if constexpr (MXS) return widen8_scaled(d0, d1, s < 2 ? a_lo[j] : a_hi[j]);
        else return widen8<AE5>(d0, d1);
    };
    {   // first tile: everything converted up front
        read_scales(smem);
        if constexpr (MXS) {
#pragma unroll
            for (int j = 0; j < FM; j++) {
                mx_pow(a_sraw[j], a_c[j], a_lo[j], a_hi[j]);
                mx_pow(b_sraw[j], b_c[j], b_lo[j], b_hi[j]);
            }
        }
#pragma unroll
        for (int j = 0; j < FM; j++) {
            const v8i r = load_frag(smem, a_rowbase + j * 16 * BK);
#pragma unroll
            for (int s = 0; s < 4; s++) fa[j][s] = widen_a(r[2 * s], r[2 * s + 1], j, s);
            a_half[j] = __builtin_shufflevector(r, r, 4, 5, 6, 7);   // converted once more behind the first instructions (same values)
        }
        b_raw = load_frag(smem, b_rowbase);
#pragma unroll
        for (int s = 0; s < 4; s++) {
            if constexpr (MXS) fbc[0][s] = widen8_scaled(b_raw[2 * s], b_raw[2 * s + 1], s < 2 ? b_lo[0] : b_hi[0]);
            else fbc[0][s] = widen8<BE5>(b_raw[2 * s], b_raw[2 * s + 1]);
        }
#pragma unroll
        for (int j = 0; j < FM; j++) {
            sc[j] = 0.0f;   // multiplies the zero partial sums folded during the first tile's first fragment
            part[1][j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
    constexpr int CPS = (CPT + 3) / 4;   // copies issued behind each of the four instruction groups of the tile's last x2 fragment

    // Schedule.  A tile is FN x2 fragments; a fragment is four groups (K steps s) of FM matrix instructions, one per x1
    // fragment j, i.e. FM interleaved chains, so no instruction waits for the one issued just before it.  Everything the
    // vector ALU has to do rides behind those instructions, a few operations each:
    //   * the fold of the previous fragment's partial sums (one fused multiply-add per instruction);
    //   * the conversion of the next x2 fragment, requested at the start of this one, behind groups 2 and 3;
    //   * the conversion of the next tile's x1 fragments: K steps 0 and 1 behind groups 2 and 3 of the tile's LAST fragment
    //     (whose groups 0 and 1 were those steps' last readers; the bytes were requested behind the barrier, two groups
    //     earlier), steps 2 and 3 behind groups 1 and 2 of the next tile's first.
    // The barrier sits before the last fragment: the next tile is complete in LDS and every wave is done reading this one.
#if QG_DBG
    unsigned long long dbg_bar = 0, dbg_lgkm = 0;
    const unsigned long long dbg_c0 = clock64();
#endif
    // (the stage index is a compile-time constant of each of the three copies of the loop body: LDS offsets are immediates)
    auto k_step = [&](int kt, auto curc) {
        constexpr int cur = decltype(curc)::value;
        constexpr int nxt = cur == STAGES - 1 ? 0 : cur + 1;
        const char* st = smem + cur * STAGE;
        const char* stn = smem + nxt * STAGE;
        const int ktc = kt + 3 < KT ? kt + 3 : KT - 1;   // past the end the copies repeat the last tile into a stage nobody reads
#pragma unroll
        for (int i = 0; i < FN; i++) {
            if (i + 1 < FN) {
                b_raw = load_frag(st, b_rowbase + (i + 1) * 16 * BK);
            } else {
#if QG_DBG
                const unsigned long long c0 = clock64();
#endif
                wait_vmcnt<CPT>();   // tile kt+1 has landed (this thread's part); tile kt+2 may still be in flight
                wait_lgkmcnt0();
#if QG_DBG
                const unsigned long long c1 = clock64();
#endif
                __builtin_amdgcn_s_barrier();   // tile kt+1 is complete in LDS; every wave is done reading tile kt
#if QG_DBG
                dbg_lgkm += c1 - c0; dbg_bar += clock64() - c1;
#endif
                __builtin_amdgcn_sched_barrier(0);
                b_raw = load_frag(stn, b_rowbase);
#pragma unroll
                for (int j = 0; j < FM; j++)
                    a_half[j] = *(const v4i*)(stn + a_rowbase + j * 16 * BK + ch0);
                read_scales(stn);
            }
            if (!RC && i == 0) {
#pragma unroll
                for (int j = 0; j < FM; j++) {
                    scp[j] = sc[j];
                    sc[j] = s1raw[j] * s2raw;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < 4; s++) {
#pragma unroll
                for (int j = 0; j < FM; j++) {
                    if constexpr (RC) {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fbc[i & 1][s], fa[j][s], acc[i][j], 0, 0, 0);
                    } else {
                        part[i & 1][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fbc[i & 1][s], fa[j][s], s == 0 ? v4f{0.0f, 0.0f, 0.0f, 0.0f} : part[i & 1][j], 0, 0, 0);
                        // fold element j of x1 fragment s of the previous x2 fragment (for i == 0: the previous tile's last, with its scales)
                        if (i > 0) acc[i - 1][s][j] = __builtin_fmaf(part[(i - 1) & 1][s][j], sc[s], acc[i - 1][s][j]);
                        else acc[FN - 1][s][j] = __builtin_fmaf(part[1][s][j], scp[s], acc[FN - 1][s][j]);
                    }
                    if constexpr (MXS) {
                        // the next tile's scale bytes were requested behind the barrier; every conversion that used the
                        // current tile's has been issued (x2 fragments 1 .. FN-1 during the earlier fragments, the x1 high
                        // halves during the first)
                        if (i == FN - 1 && s == 1) {
                            mx_pow(a_sraw[j], a_c[j], a_lo[j], a_hi[j]);
                            mx_pow(b_sraw[j], b_c[j], b_lo[j], b_hi[j]);
                        }
                    }
                    if (s >= 2) {   // next x2 fragment: half a K step per instruction
                        const int idx = (s - 2) * 4 + j;
                        const int nf = (i + 1) % FN;
                        widen4(b_raw[idx], fbc[(i + 1) & 1][idx / 2], idx % 2, idx / 2 < 2 ? b_lo[nf] : b_hi[nf]);
                    }
                    if (i == FN - 1 && s >= 2)                // next tile's x1 fragments, K step s - 2 (low halves)
                        fa[j][s - 2] = widen_a(a_half[j][2 * (s - 2)], a_half[j][2 * (s - 2) + 1], j, s - 2);
                    if (i == 0 && (s == 1 || s == 2))         // this tile's x1 fragments, K steps 2 and 3 (high halves)
                        fa[j][1 + s] = widen_a(a_half[j][2 * (s - 1)], a_half[j][2 * (s - 1) + 1], j, 1 + s);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (i == FN - 1) {
                    if (s == 3) {   // the low halves are converted: fetch the high halves into the same registers
#pragma unroll
                        for (int j = 0; j < FM; j++)
                            a_half[j] = *(const v4i*)(stn + a_rowbase + j * 16 * BK + ch1);
                    }
#pragma unroll
                    for (int c = s * CPS; c < (s + 1) * CPS && c < CPT; c++) issue_piece(ktc, cur, c);   // tile kt+3 into the stage of tile kt
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };
    {
        int kt = 0;
        for (; kt + 3 <= KT; kt += 3) {
            k_step(kt, std::integral_constant<int, 0>{});
            k_step(kt + 1, std::integral_constant<int, 1>{});
            k_step(kt + 2, std::integral_constant<int, 2>{});
        }
        if (kt < KT) k_step(kt, std::integral_constant<int, 0>{});
        if (kt + 1 < KT) k_step(kt + 1, std::integral_constant<int, 1>{});
    }
#if QG_DBG
    if (lane == 0 && p.dbg) {
        unsigned long long* d = p.dbg + ((size_t)blockIdx.x * 8 + wave) * 4;
        d[0] = clock64() - dbg_c0; d[1] = dbg_bar; d[2] = dbg_lgkm; d[3] = (unsigned long long)KT;
    }
#endif
    if constexpr (!RC) {
#pragma unroll
        for (int j = 0; j < FM; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[FN - 1][j][r] = __builtin_fmaf(part[(FN - 1) & 1][j][r], sc[j], acc[FN - 1][j][r]);
    }
    wait_lgkmcnt0();   // the reads and copies past the last tile land before LDS is reused
    wait_vmcnt<0>();

    if constexpr (SPLIT) {
        // partial sums straight from the registers: a lane holds four consecutive columns of one row per fragment
        float* part = p.part + (((int64_t)blockIdx.z * gridDim.y + bz) * p.M) * p.N;
        const bool vec_ok4 = (p.N % 4) == 0 && ((uintptr_t)p.part % 16) == 0;
#pragma unroll
        for (int j = 0; j < FM; j++) {
            const int64_t m = m0 + wm * TM + j * 16 + frow;
#pragma unroll
            for (int i = 0; i < FN; i++) {
                const int64_t n = n0 + wn * TN + i * 16 + 4 * fq;
                if (m >= p.M) continue;
                if (vec_ok4 && n + 3 < p.N) {
                    *(v4f*)(part + m * p.N + n) = acc[i][j];
                } else {
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (n + r < p.N) part[m * p.N + n + r] = acc[i][j][r];
                }
            }
        }
        return;
    }
    // Epilogue: acc[i][j][r] is out[m = m_base + 16j + lane%16][n = n_base + 16i + 4*(lane/16) + r].  Each wave parks one
    // 16 x 64 block in a private LDS patch and reads it back row-wise, so that a store instruction writes whole
    // 128-byte lines (16 bytes per lane, 8 lanes per row).
    __syncthreads();
    typedef v4us __attribute__((may_alias)) v4us_a;
    typedef v4i __attribute__((may_alias)) v4i_a;
    constexpr int EP_PITCH = TN * 2 + 16;
    char* ep = smem + wave * (16 * EP_PITCH);
    static_assert(8 * 16 * EP_PITCH <= STAGES * STAGE, "epilogue staging fits in the operand stages");
    uint16_t* out = (uint16_t*)p.out + bz * p.M * p.N;
    const bool vec_ok = (p.N % 8) == 0 && ((uintptr_t)p.out % 16) == 0;
    const int er = lane >> 3, ec = lane & 7;
    float rs_j[FM];
    (void)rs_j;
    if constexpr (RC) {
#pragma unroll
        for (int j = 0; j < FM; j++) {
            const int64_t mrow = m0 + wm * TM + j * 16 + frow;
            rs_j[j] = p.rs ? p.rs[bz * p.rs_bs + (mrow < p.M ? mrow : p.M - 1) * p.rs_stride] : 1.0f;
        }
    }
#pragma unroll
    for (int j = 0; j < FM; j++) {
#pragma unroll
        for (int i = 0; i < FN; i++) {
            v4f v = acc[i][j];
            if constexpr (RC) {   // (sum * x2Scale[n]) * x1Scale[m] + bias[n], each operation rounded, as compute_pertoken orders them
                const int64_t nb = n0 + wn * TN + i * 16 + 4 * fq;
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = fp8x_rowcol_epilogue(p, v[r], rs_j[j], bz, nb + r < p.N ? nb + r : p.N - 1);
            }
            if constexpr (OUT_DT == DT_F32) {
                // fp32 output: the lane's four neighbouring columns are 16 bytes, four lanes a 64-byte piece of a row: stored as they are
                float* outf = (float*)p.out + bz * p.M * p.N;
                const int64_t m = m0 + wm * TM + j * 16 + frow, n = n0 + wn * TN + i * 16 + 4 * fq;
                if (m < p.M) {
                    if ((p.N % 4) == 0 && ((uintptr_t)p.out % 16) == 0 && n + 3 < p.N) *(v4f*)(outf + m * p.N + n) = v;
                    else {
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            if (n + r < p.N) outf[m * p.N + n + r] = v[r];
                    }
                }
            } else {
                *(v4us_a*)(ep + frow * EP_PITCH + (i * 16 + 4 * fq) * 2) = pack4_b16<OUT_DT>(v);
            }
        }
        if constexpr (OUT_DT == DT_F32) continue;
#pragma unroll
        for (int r = 0; r < 2; r++) {
            const int row = r * 8 + er;
            const v4i o = *(const v4i_a*)(ep + row * EP_PITCH + ec * 16);
            const int64_t m = m0 + wm * TM + j * 16 + row;
            const int64_t n = n0 + wn * TN + ec * 8;
            if (m < p.M) {
                if (vec_ok && n + 7 < p.N) {
                    *(v4i*)(out + m * p.N + n) = o;
                } else {
                    const uint16_t* oe = (const uint16_t*)&o;
#pragma unroll
                    for (int e = 0; e < 8; e++)
                        if (n + e < p.N) out[m * p.N + n + e] = oe[e];
                }
            }
        }
    }
}

// out[b, m, n] = the sum over the splits, in split order, of part[s, b, m, n], then the row / column epilogue (RC) and
// the rounding.  With gate flags (the MX mode) nothing is written when one is set: the launch that follows computes the call.
template <int OUT_DT, bool RC>
__global__ __launch_bounds__(256) void fp8x_splitk_reduce_kernel(Fp8xParams p, int64_t total)
{
    if (p.gate) {
        int f = 0;
        for (int i = 0; i < p.gate_n; i++) f |= p.gate[i];
        if (f) return;
    }
    const int64_t MN = p.M * p.N, stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        float v = splitk_sum(p.part, p.splits, total, i);
        if constexpr (RC) {
            const int64_t bz = i / MN, m = (i % MN) / p.N, n = i % p.N;
            v = fp8x_rowcol_epilogue(p, v, p.rs ? p.rs[bz * p.rs_bs + m * p.rs_stride] : 1.0f, bz, n);
        }
        if constexpr (OUT_DT == DT_F32) ((float*)p.out)[i] = v;
        else ((uint16_t*)p.out)[i] = OUT_DT == DT_BF16 ? bf16_bits(v) : f16_bits(v);
    }
}

template <int OUT_DT, bool RC, int FMT = 0, bool MXS = false>
static int launch_fp8_exact(const Fp8xParams& p, int64_t batch, hipStream_t st)
{
    const int tiles_m = (int)((p.M + 255) / 256), tiles_n = (int)((p.N + 127) / 128);
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)batch);
    const size_t lds = 3 * (size_t)(256 * 128 + 128 * 128 + ((RC && !MXS) ? 0 : 512 * 4));
    if (p.splits > 1) {   // K split over workgroups, then the sum of the partial sums, the epilogue and the rounding
        if (!p.part || p.splits > p.K / 128) return -1;
        auto ks = qmm_fp8_exact_kernel<DT_F32, RC, FMT, MXS, true>;
        static std::atomic<uint64_t> attr_set_s{0};
        if (!device_flag_test(attr_set_s)) {
            hipError_t e = hipFuncSetAttribute((const void*)ks, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return (int)e;
            device_flag_set(attr_set_s);
        }
        grid.z = (unsigned)p.splits;
        hipLaunchKernelGGL(ks, grid, dim3(512), lds, st, p, tiles_m, tiles_n);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return (int)e;
        const int64_t total = batch * p.M * p.N;
        const unsigned rgrid = splitk_reduce_grid(total);
        hipLaunchKernelGGL((fp8x_splitk_reduce_kernel<OUT_DT, RC>), dim3(rgrid), dim3(256), 0, st, p, total);
        return (int)hipGetLastError();
    }
    auto k = qmm_fp8_exact_kernel<OUT_DT, RC, FMT, MXS>;
    static std::atomic<uint64_t> attr_set{0};   // one bit per device: the attribute belongs to the (kernel, device) pair
    if (!device_flag_test(attr_set)) {
        hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        device_flag_set(attr_set);
    }
    hipLaunchKernelGGL(k, grid, dim3(512), lds, st, p, tiles_m, tiles_n);
    return (int)hipGetLastError();
}

// fp8 e4m3 block scales (G-B, B-B), K-contiguous operands, K % 128 == 0, 16-bit or fp32 output, no bias.
int launch_blockscale_exact(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk)
{
    if (a.x1_dtype != DT_E4M3 || a.x2_dtype != DT_E4M3) return OPSNN_NOT_TAKEN;
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16 && a.out_dtype != DT_F32) return OPSNN_NOT_TAKEN;
    if (a.bias) return OPSNN_NOT_TAKEN;
    if (a.gsK != 128 || a.gsN != 128 || (a.gsM != 1 && a.gsM != 128)) return OPSNN_NOT_TAKEN;
    if (a.K % 128 != 0 || a.M * a.N < 64 * 64 || a.x1.col_stride != 1 || a.x2.row_stride != 1) return OPSNN_NOT_TAKEN;
    Fp8xParams p{};
    p.a = (const int8_t*)a.x1.ptr; p.b = (const int8_t*)a.x2.ptr;
    p.lda = a.x1.row_stride; p.ldb = a.x2.col_stride; p.a_bs = a.x1.batch_stride; p.b_bs = a.x2.batch_stride;
    p.out = a.out; p.M = a.M; p.N = a.N; p.K = a.K;
    p.s1 = (const float*)a.x1_scale_mat.ptr; p.s1_rs = a.x1_scale_mat.row_stride; p.s1_cs = a.x1_scale_mat.col_stride;
    p.s1_bs = a.x1_scale_mat.batch_stride;
    p.s2 = (const float*)a.x2_scale_mat.ptr; p.s2_rs = a.x2_scale_mat.row_stride; p.s2_cs = a.x2_scale_mat.col_stride;
    p.s2_bs = a.x2_scale_mat.batch_stride;
    p.gsM = (int)a.gsM;
    if (((uintptr_t)p.a | (uintptr_t)p.b | (uint64_t)p.lda | (uint64_t)p.ldb | (uint64_t)p.a_bs | (uint64_t)p.b_bs) % 16) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)p.s1 | (uintptr_t)p.s2) % 4) return OPSNN_NOT_TAKEN;
    // the kernel addresses a row's s1 entries by a 32-bit byte offset from the batch's table, and operand rows of a tile
    // by 32-bit offsets from the tile's first row
    if (p.s1_rs < 0 || p.s1_cs < 0 || ((a.M + p.gsM - 1) / p.gsM) * p.s1_rs * 4 >= (1ll << 32)) return OPSNN_NOT_TAKEN;
    if (p.lda < 0 || p.ldb < 0 || 256 * p.lda >= (1ll << 32) || 128 * p.ldb >= (1ll << 32)) return OPSNN_NOT_TAKEN;
    p.splits = sk.splits; p.part = sk.part;
    if (a.out_dtype == DT_BF16) return launch_fp8_exact<DT_BF16, false>(p, a.batch, st);
    if (a.out_dtype == DT_F32) return launch_fp8_exact<DT_F32, false>(p, a.batch, st);
    return launch_fp8_exact<DT_F16, false>(p, a.batch, st);
}

// fp8 (e4m3 or e5m2, each operand by itself) with scales applied to the finished sums: one fp32 scale per row of x1 (or
// one, or none) and one per column of x2 (or one; fp32, bf16 or 64-bit words), optional fp32 bias.  ep_mode as in
// Fp8xParams: 0 = (sum * cs) * rs + bias (compute_pertoken; compute_tc with a per-token scale), 1 = (sum + bias) * cs,
// 2 = sum * trunc19(cs * rs).
int launch_rowcol_exact(const OpsnnQmmArgs& a, hipStream_t st, int ep_mode, SplitK sk)
{
    const bool e1 = a.x1_dtype == DT_E5M2, e2 = a.x2_dtype == DT_E5M2;
    if ((a.x1_dtype != DT_E4M3 && !e1) || (a.x2_dtype != DT_E4M3 && !e2)) return OPSNN_NOT_TAKEN;
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16 && a.out_dtype != DT_F32) return OPSNN_NOT_TAKEN;
    if (!a.x2_scale || (a.x2_scale_dtype != DT_F32 && a.x2_scale_dtype != DT_BF16 && a.x2_scale_dtype != DT_U64)) return OPSNN_NOT_TAKEN;
    if (ep_mode != 1 && !a.x1_scale) return OPSNN_NOT_TAKEN;
    if (a.bias && a.bias_dtype != DT_F32 && a.bias_dtype != DT_BF16 && a.bias_dtype != DT_F16) return OPSNN_NOT_TAKEN;
    if (a.K % 128 != 0 || a.M * a.N < 64 * 64 || a.x1.col_stride != 1 || a.x2.row_stride != 1) return OPSNN_NOT_TAKEN;
    Fp8xParams p{};
    p.a = (const int8_t*)a.x1.ptr; p.b = (const int8_t*)a.x2.ptr;
    p.lda = a.x1.row_stride; p.ldb = a.x2.col_stride; p.a_bs = a.x1.batch_stride; p.b_bs = a.x2.batch_stride;
    p.out = a.out; p.M = a.M; p.N = a.N; p.K = a.K; p.gsM = 1;
    p.rs = ep_mode == 1 ? nullptr : (const float*)a.x1_scale; p.rs_stride = a.x1_scale_len == 1 ? 0 : 1;
    p.cs = a.x2_scale; p.cs_stride = a.x2_scale_len == 1 ? 0 : 1; p.cs_dt = a.x2_scale_dtype;
    p.ep_mode = ep_mode;
    p.bias = a.bias; p.bias_dt = a.bias_dtype; p.bias_bs = a.bias_batch_stride;
    if (((uintptr_t)p.a | (uintptr_t)p.b | (uint64_t)p.lda | (uint64_t)p.ldb | (uint64_t)p.a_bs | (uint64_t)p.b_bs) % 16) return OPSNN_NOT_TAKEN;
    p.splits = sk.splits; p.part = sk.part;
    const bool bf = a.out_dtype == DT_BF16, f32 = a.out_dtype == DT_F32;
    switch ((e1 ? 1 : 0) | (e2 ? 2 : 0)) {
        case 0: return f32 ? launch_fp8_exact<DT_F32, true, 0>(p, a.batch, st) : bf ? launch_fp8_exact<DT_BF16, true, 0>(p, a.batch, st) : launch_fp8_exact<DT_F16, true, 0>(p, a.batch, st);
        case 1: return f32 ? launch_fp8_exact<DT_F32, true, 1>(p, a.batch, st) : bf ? launch_fp8_exact<DT_BF16, true, 1>(p, a.batch, st) : launch_fp8_exact<DT_F16, true, 1>(p, a.batch, st);
        case 2: return f32 ? launch_fp8_exact<DT_F32, true, 2>(p, a.batch, st) : bf ? launch_fp8_exact<DT_BF16, true, 2>(p, a.batch, st) : launch_fp8_exact<DT_F16, true, 2>(p, a.batch, st);
        default: return f32 ? launch_fp8_exact<DT_F32, true, 3>(p, a.batch, st) : bf ? launch_fp8_exact<DT_BF16, true, 3>(p, a.batch, st) : launch_fp8_exact<DT_F16, true, 3>(p, a.batch, st);
    }
}

// ---- MX (e8m0 scale per 32 K) on exact products ----
// Per row of a scale table [rows, K/32] (K-contiguous, nd = K/128 dwords per row): base = max byte - 7, c = 127 - base and
// 2^(base - 127).  With byte - base in [-15, 7] an e4m3 value times 2^(byte - base) is an fp16 value (largest 448 * 2^7,
// smallest 2^-9 * 2^-15 = 2^-24).  flags[block] = 1 when one of the block's rows holds a byte below max - 22 or the NaN
// code 255.  One wave per row at a time, 64 rows per workgroup.
__global__ __launch_bounds__(256) void mx_row_base_kernel(const uint8_t* __restrict__ s, int64_t rs, int64_t bs, int64_t rows, int64_t total, int nd,
                                                          int* __restrict__ c_out, float* __restrict__ pow_out, int* __restrict__ flags)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int bad = 0;
    for (int i = 0; i < 16; i++) {
        const int64_t r = (int64_t)blockIdx.x * 64 + wave * 16 + i;
        if (r >= total) break;
        const uint32_t* row = (const uint32_t*)(s + (r / rows) * bs + (r % rows) * rs);
        uint32_t mn = 255, mx = 0;
        for (int d = lane; d < nd; d += 64) {
            const uint32_t w = row[d];
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const uint32_t v = (w >> (8 * b)) & 0xFFu;
                mn = v < mn ? v : mn;
                mx = v > mx ? v : mx;
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const uint32_t a = (uint32_t)__shfl_xor((int)mn, o), b = (uint32_t)__shfl_xor((int)mx, o);
            mn = a < mn ? a : mn;
            mx = b > mx ? b : mx;
        }
        const int base = (int)mx - 7;
        if (lane == 0) {
            c_out[r] = 127 - base;
            pow_out[r] = ldexpf(1.0f, base - 127);
        }
        bad |= (mx == 255u || mx - mn > 22u) ? 1 : 0;
    }
    const int any = __syncthreads_or(bad);
    if (threadIdx.x == 0) flags[blockIdx.x] = any ? 1 : 0;
}

static inline uint64_t up256(uint64_t v) { return (v + 255) / 256 * 256; }

// Bytes of workspace the exact MXFP8 route wants in front of everything else: 127 - base and 2^(base - 127) per row of
// both operands, and the flags.
uint64_t mx_exact_bytes(const OpsnnQmmArgs& a)
{
    if (a.x1_dtype != DT_E4M3 || a.x2_dtype != DT_E4M3) return 0;
    if (a.M <= 0 || a.N <= 0 || a.K < 64 || a.batch <= 0) return 0;
    const uint64_t rows = (uint64_t)a.batch * (uint64_t)(a.M + a.N);
    return up256(rows * 8) + up256(((rows + 63) / 64 + 2) * 4);
}

// MXFP8 with exact products: the bases pass, this kernel, and -- computing
// only when a flag is set -- the tile kernel on the scaled 8-bit instruction.  `a`: both operands e4m3, K-contiguous,
// K % 128 == 0, scale rows K-contiguous; `region`: mx_exact_bytes(a) bytes.  OPSNN_NOT_TAKEN before anything is launched.
int launch_mx_exact(const OpsnnQmmArgs& a, void* region, hipStream_t st, SplitK sk)
{
    if (!region || (uintptr_t)region % 16) return OPSNN_NOT_TAKEN;
    if (a.x1_dtype != DT_E4M3 || a.x2_dtype != DT_E4M3) return OPSNN_NOT_TAKEN;
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16 && a.out_dtype != DT_F32) return OPSNN_NOT_TAKEN;
    if (a.bias && a.bias_dtype != DT_F32 && a.bias_dtype != DT_BF16 && a.bias_dtype != DT_F16) return OPSNN_NOT_TAKEN;
    if (a.K % 128 != 0 || a.M * a.N < 64 * 64 || a.x1.col_stride != 1 || a.x2.row_stride != 1) return OPSNN_NOT_TAKEN;
    if (a.x1_scale_mat.col_stride != 2 || a.x2_scale_mat.col_stride != 2) return OPSNN_NOT_TAKEN;
    const int64_t nb1 = a.x1_scale_mat.batch_stride == 0 ? 1 : a.batch, nb2 = a.x2_scale_mat.batch_stride == 0 ? 1 : a.batch;
    Fp8xParams p{};
    p.a = (const int8_t*)a.x1.ptr; p.b = (const int8_t*)a.x2.ptr;
    p.lda = a.x1.row_stride; p.ldb = a.x2.col_stride; p.a_bs = a.x1.batch_stride; p.b_bs = a.x2.batch_stride;
    p.out = a.out; p.M = a.M; p.N = a.N; p.K = a.K; p.gsM = 1;
    p.sa = (const uint8_t*)a.x1_scale_mat.ptr; p.sb = (const uint8_t*)a.x2_scale_mat.ptr;
    p.sa_rs = a.x1_scale_mat.row_stride; p.sb_rs = a.x2_scale_mat.row_stride;
    p.sa_bs = a.x1_scale_mat.batch_stride; p.sb_bs = a.x2_scale_mat.batch_stride;
    if (((uintptr_t)p.a | (uintptr_t)p.b | (uint64_t)p.lda | (uint64_t)p.ldb | (uint64_t)p.a_bs | (uint64_t)p.b_bs) % 16) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)p.sa | (uintptr_t)p.sb | (uint64_t)p.sa_rs | (uint64_t)p.sb_rs | (uint64_t)p.sa_bs | (uint64_t)p.sb_bs) % 4) return OPSNN_NOT_TAKEN;
    const int64_t rows1 = nb1 * a.M, rows2 = nb2 * a.N;
    const uint64_t all_rows = (uint64_t)a.batch * (uint64_t)(a.M + a.N);
    int* c1 = (int*)region;
    int* c2 = c1 + rows1;
    float* pw1 = (float*)((char*)region + all_rows * 4);
    float* pw2 = pw1 + rows1;
    int* flags = (int*)((char*)region + up256(all_rows * 8));
    const int g1 = (int)((rows1 + 63) / 64), g2 = (int)((rows2 + 63) / 64), nd = (int)(a.K / 128);
    hipLaunchKernelGGL(mx_row_base_kernel, dim3((unsigned)g1), dim3(256), 0, st, p.sa, p.sa_rs, p.sa_bs, a.M, rows1, nd, c1, pw1, flags);
    hipLaunchKernelGGL(mx_row_base_kernel, dim3((unsigned)g2), dim3(256), 0, st, p.sb, p.sb_rs, p.sb_bs, a.N, rows2, nd, c2, pw2, flags + g1);
    p.a_c = c1; p.b_c = c2;
    p.rs = pw1; p.rs_stride = 1; p.rs_bs = nb1 == 1 ? 0 : a.M;
    p.cs = pw2; p.cs_stride = 1; p.cs_bs = nb2 == 1 ? 0 : a.N; p.cs_dt = DT_F32;
    p.ep_mode = 0;
    p.bias = a.bias; p.bias_dt = a.bias_dtype; p.bias_bs = a.bias_batch_stride;
    p.gate = flags; p.gate_n = g1 + g2;
    p.splits = sk.splits; p.part = sk.part;
    const int rc = a.out_dtype == DT_F32    ? launch_fp8_exact<DT_F32, true, 0, true>(p, a.batch, st)
                   : a.out_dtype == DT_BF16 ? launch_fp8_exact<DT_BF16, true, 0, true>(p, a.batch, st)
                                            : launch_fp8_exact<DT_F16, true, 0, true>(p, a.batch, st);
    if (rc != 0) return rc;
    QgemmParams g{};
    g.a = p.a; g.b = p.b; g.lda = p.lda; g.ldb = p.ldb; g.a_bs = p.a_bs; g.b_bs = p.b_bs;
    g.out = a.out; g.M = a.M; g.N = a.N; g.ldc = a.N; g.KB = a.K;
    g.bias = a.bias; g.bias_dt = a.bias_dtype; g.bias_bs = a.bias_batch_stride;
    g.sa = p.sa; g.sb = p.sb; g.sa_rs = p.sa_rs; g.sb_rs = p.sb_rs; g.sa_bs = p.sa_bs; g.sb_bs = p.sb_bs;
    g.gate = flags; g.gate_n = g1 + g2;
    if (a.M <= 128 || a.N <= 128) return qgemm_launch<MODE_MXFP8, 128, 128, 128, 2, 2, 2, 1>(g, a.batch, a.out_dtype, st);
    return qgemm_launch<MODE_MXFP8, 256, 256, 128, 2, 2, 2, 1>(g, a.batch, a.out_dtype, st);
}

}  // namespace opsnn
