// fp8 e4m3 x fp8 e4m3 quantized matmul with fp32 block scales (G-B: 1x128 / 128x128, B-B: 128x128 / 128x128).
//
//   out[m,n] = cast( sum_kb ( sum_{k in block kb} x1[m,k] * x2[k,n] ) * ( s1[m/gsM, kb] * s2[kb, n/128] ) )
//
// Formula: matmul/quant_batch_matmul_v3/tests/assets/qbmmv3_kernel_golden.py:237-358 (the two scales are
// multiplied together first, :337-343); device counterpart in the reference:
// matmul/common/cmct/epilogue/block_epilogue_pertile.h:502-642 (matrix unit per 128-K tile, vector unit
// scale-accumulate in fp32).
//
// The same split is used here and for the same reason.  One K tile of the pipeline is exactly one 128-wide scale
// block, and one v_mfma_f32_16x16x128_f8f6f4 contracts all of it: issued from a zero accumulator it leaves the
// block's partial products in four registers, which the vector ALU folds into the fp32 running sum with one fused
// multiply-add per element while the matrix pipe is busy with the next fragment.  (With 32x32x64 instructions a
// block takes a chain of two, sixteen result registers and a wait for the chain before the fold can start: the
// compiler serialised matrix and vector work, 4000 clocks per K tile against 3650 now.)  Starting every block from
// zero also keeps the matrix pipe's reduced-width product aligner working on operands of one block's magnitude
// only, never against the large running sum.
//
// Tiling: (64*WGM) x 256 output tile per workgroup, WGM x 2 waves, each wave owns 64 x 128 (4 x 8 fragments of
// 16 x 16): the running sums must be vector registers (the vector ALU updates them), which bounds the per-wave
// tile.  In the x2-fragment x x1-fragment orientation every lane owns one output row m per fragment, so s1[m, kb]
// is a per-lane scalar, and a wave's 128 columns lie inside one 128-wide n block, so s2[kb, nb] is wave-uniform.
// Operands stream global -> LDS with 16-byte async copies (XOR-swizzled rows), the scales of a block with
// 4-byte async copies into the same stage.
#include "launch.h"
#include "qgemm_core.hip.h"

namespace opsnn {
const void* weight_cache_get(const void* src, int64_t K, int64_t N, int bits, int64_t nb, hipStream_t st);   // weight_cache.hip

struct Fp8BlkParams {
    const int8_t* a;
    const int8_t* b;
    int64_t lda, ldb, a_bs, b_bs;
    void* out;
    int64_t M, N, K;
    const float* s1;   // element (m/gsM, kb) at s1[(m/gsM)*s1_rs + kb*s1_cs]
    const float* s2;   // element (kb, nb) at s2[kb*s2_rs + nb*s2_cs]
    int64_t s1_rs, s1_cs, s1_bs, s2_rs, s2_cs, s2_bs;
    int gsM;           // 1 or 128
    // MX mode: one e8m0 byte per 32 K elements, K-contiguous per row; fp32 bias or null
    const uint8_t* sa;
    const uint8_t* sb;
    int64_t sa_rs, sb_rs, sa_bs, sb_bs;
    const float* bias;   // FP8_MX_W4: elements of bias_dt (fp32 or 16-bit)
    int bias_dt;
    int64_t bias_bs;
    // row / column scale mode (fp8 K-C, K-T and the double-scale modes that multiply separately):
    // out = (sum * cs[n * cs_stride]) * rs[m * rs_stride] + bias[n]; strides 0 (one scale) or 1
    const float* rs;
    const float* cs;
    int rs_stride, cs_stride;
    // K split over `splits` workgroups per tile (SPLIT instantiations, grid.z): fp32 partial sums [splits][batch][M][N]
    int splits;
    float* part;
#if QG_DBG
    unsigned long long* dbg;   // timing harness only (see qgemm_core.hip.h)
#endif
};

// Three modes of one kernel.  FP8_BLOCK: fp32 block scales folded in by the vector ALU (above).  FP8_MX (MXFP8): the
// e8m0 scales of the tile's four 32-element blocks go into the instruction, which then accumulates straight into the
// running sums (no fold, no partial-sum registers).  Measured against summing every 128 elements from zero and adding
// in fp32: the same error (1.0 % of bf16 outputs one ulp off the exactly rounded result at K = 7168..16384, either way
// -- the error is made inside the instruction, between blocks whose scales differ), 1.4x the speed.  FP8_ROWCOL: plain
// fp8 products accumulated in the instruction, one fp32 scale per output row and one per column applied in the epilogue
// (fp8 K-C / K-T and the double-scale modes that multiply separately; no scale copies at all).
// a wave-uniform pointer, held in scalar registers
__device__ __forceinline__ const int8_t* scalar_ptr(const int8_t* p)
{
    const uint64_t u = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u), hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
    return (const int8_t*)(((uint64_t)hi << 32) | lo);
}

enum : int { FP8_BLOCK = 0, FP8_MX = 1, FP8_ROWCOL = 2, FP8_MX_W4 = 3, I8_BLOCK = 4 };

template <int WGM, int STAGES, int OUT_DT, int MODE = FP8_BLOCK, bool SPLIT = false>
__global__ __launch_bounds__(WGM * 128, 1) void qmm_fp8_block_kernel(Fp8BlkParams p, int tiles_m, int tiles_n)
{
    static_assert(!SPLIT || MODE != FP8_ROWCOL, "partial sums leave before the epilogue's scales: the modes whose sums carry their scales");
    constexpr bool W4 = MODE == FP8_MX_W4;     // MX with fp4 e2m1 x2 (fp8 x fp4): x2 rows are 64 bytes per K tile
    constexpr bool MX = MODE == FP8_MX || W4;  // e8m0 scales inside the instruction
    constexpr bool RC = MODE == FP8_ROWCOL;    // plain fp8 products, one scale per row and per column in the epilogue
    constexpr bool I8 = MODE == I8_BLOCK;      // int8 operands with the block scales of FP8_BLOCK ("per-tile" of quant_batch_matmul_v4)
    constexpr bool BLK = MODE == FP8_BLOCK || I8;   // fp32 block scales folded in by the vector ALU
    static_assert(!MX || WGM == 4, "MX mode: one scale copy per thread covers the 256 + 256 rows of the tile");
    constexpr int BM = 64 * WGM, BN = 256, BK = 128, NT = WGM * 128;   // WGM x 2 waves of 64 x 128 each
    constexpr int CPR = BK / 16, RPW = 16 / CPR;
    constexpr int TM = 64, TN = 128, FM = TM / 16, FN = TN / 16;      // 4 x 8 fragments of 16 x 16 per wave
    constexpr int BKB = W4 ? BK / 2 : BK;        // bytes of an x2 row per K tile
    constexpr int CPRB = BKB / 16, RPWB = 16 / CPRB;
    constexpr int A_BYTES = BM * BK, B_BYTES = BN * BKB;
    constexpr int SC_BYTES = NT * 4;             // BM s1 floats + 2 s2 floats, one 4-byte copy per lane
    constexpr int STAGE = A_BYTES + B_BYTES + SC_BYTES;
    constexpr int RPI = NT / CPR, RPIB = NT / CPRB;   // rows per copy instruction of the workgroup
    constexpr int NA = BM / RPI, NB = BN / RPIB;
    constexpr int CPT = NA + NB + (RC ? 0 : 1);   // operand copies and, unless the scales wait for the epilogue, one scale copy
    static_assert(STAGES * CPT < 64, "stage count");
    extern __shared__ __attribute__((aligned(16))) char smem[];

#if QG_DBG
    const unsigned long long dbg_t0 = wall_clock64();
    unsigned long long dbg_vm = 0, dbg_bar = 0, dbg_n = 0;
#endif
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    const uint32_t t = xcd_remap(blockIdx.x, (uint32_t)(tiles_m * tiles_n));
    const int tm = (int)(t % (uint32_t)tiles_m), tn = (int)(t / (uint32_t)tiles_m);
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    const int64_t bz = blockIdx.y;
    const int64_t lda = p.lda, ldb = p.ldb;
    const int8_t* A = p.a + bz * p.a_bs + m0 * lda;
    const int8_t* B = p.b + bz * p.b_bs + n0 * ldb;
    int KT = (int)(p.K / BK);
    int kt_first = 0;   // SPLIT: this workgroup's K tiles are kt_first .. kt_first + KT - 1 (at least one: the launcher splits at most KT / 4 ways)
    if constexpr (SPLIT) {
        const int z = (int)blockIdx.z;
        kt_first = (int)((int64_t)z * KT / p.splits);
        KT = (int)((int64_t)(z + 1) * KT / p.splits) - kt_first;
        A += (int64_t)kt_first * BK;
        B += (int64_t)kt_first * BKB;
    }

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
    const int crowb = tid / CPRB;
    const int cchunkb = (tid % CPRB) ^ ((crowb / RPWB) & (CPRB - 1));
#pragma unroll
    for (int i = 0; i < NB; i++) {
        int r = i * RPIB + crowb;
        r = r < b_rows ? r : b_rows - 1;
        b_off[i] = (uint32_t)(r * ldb + cchunkb * 16);
    }
    // Scale copy: lanes 0..BM-1 fetch s1 of tile row `tid`, lanes BM, BM+1 fetch s2 of the tile's two n blocks,
    // the rest re-fetch a valid word (their LDS slots are never read).
    const float* sc_src = nullptr;
    int64_t sc_step = 0;
    if constexpr (RC) {
    } else if constexpr (MX) {   // the four scale bytes of tile row `tid` (x1 rows, then x2 rows) for one K tile
        if (tid < BM) {
            const int r = tid < a_rows ? tid : a_rows - 1;
            sc_src = (const float*)(p.sa + bz * p.sa_bs + (m0 + r) * p.sa_rs);
        } else {
            int r = tid - BM;
            r = r < b_rows ? r : b_rows - 1;
            sc_src = (const float*)(p.sb + bz * p.sb_bs + (n0 + r) * p.sb_rs);
        }
        sc_step = 1;
    } else {
        const float* s1 = p.s1 + bz * p.s1_bs;
        const float* s2 = p.s2 + bz * p.s2_bs;
        if (tid < BM) {
            int r = tid < a_rows ? tid : a_rows - 1;
            sc_src = s1 + ((m0 + r) / p.gsM) * p.s1_rs;
            sc_step = p.s1_cs;
        } else {
            int64_t nb = n0 / 128 + ((tid - BM) & 1);
            const int64_t nbmax = (p.N + 127) / 128 - 1;
            nb = nb < nbmax ? nb : nbmax;
            sc_src = s2 + nb * p.s2_cs;
            sc_step = p.s2_rs;
        }
    }

    if constexpr (SPLIT && !RC) sc_src += (int64_t)kt_first * sc_step;

    // copy instruction `idx` (0 .. CPT-1) of K tile kt: x1 rows, then x2 rows, then the scales
    // The tile's base addresses are pinned in scalar registers (which also hides them from loop-invariant code
    // motion), so that every copy addresses memory as scalar base + 32-bit lane offset instead of keeping a 64-bit
    // pointer per copy in vector registers.
    auto issue_piece = [&](int kt, int stage, int idx) {
        char* sA = smem + stage * STAGE + wave * 1024;
        char* sB = sA + A_BYTES;
        const int8_t* Ak = scalar_ptr(A + (int64_t)kt * BK);
        const int8_t* Bk = scalar_ptr(B + (int64_t)kt * BKB);
        if (idx < NA) async_copy16(Ak + a_off[idx], sA + idx * NT * 16);
        else if (idx < NA + NB) async_copy16(Bk + b_off[idx - NA], sB + (idx - NA) * NT * 16);
        else async_copy4(sc_src + (int64_t)kt * sc_step, smem + stage * STAGE + A_BYTES + B_BYTES + wave * 256);
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

    // Operand fragment of the 16x16x128 instruction, lane (row = lane%16, q = lane/16): the 32 bytes [32q, 32q+32) of
    // the row's 128 bytes of K.  (K is the contraction index: any assignment of K to lanes is right as long as both
    // operands use the same one.)
    const int frow = lane & 15, fq = lane >> 4;
    const int key = (frow / RPW) & (CPR - 1);
    const int a_rowbase = (wm * TM + frow) * BK;
    const int b_rowbase = A_BYTES + (wn * TN + frow) * BKB;
    // MX mode, where the position of K matters: the instruction takes registers 0..3 of lane group q as the 16 elements
    // [16q, 16q+16) of K and registers 4..7 as [64+16q, 64+16q+16), so the 32-element block b lies in lane groups
    // 2(b%2), 2(b%2)+1, register half b/2 -- and it is scaled by the scale byte that the lanes of GROUP b supply
    // (measured on the device with one-hot scale patterns; the 32x32x64 form is built the same way from two lane halves).
    const int mx0 = (fq ^ key) << 4, mx1 = ((4 + fq) ^ key) << 4;
    auto load_frag = [&](const char* st, int rowbase) -> v8i {
        // every mode reads the chunk pair (q, 4 + q): for the modes without scales inside the instruction any assignment
        // of K to lanes is right, and this one is free of LDS bank conflicts (the pair (2q, 2q + 1) cost four conflict
        // cycles per read: SQ_LDS_BANK_CONFLICT 68M -> 1.8M cycles on config 4 in the kernel of qmm_fp8_exact.hip)
        const v4i lo = *(const v4i*)(st + rowbase + mx0);
        const v4i hi = *(const v4i*)(st + rowbase + mx1);
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };
    // fp4 x2 fragment (W4): a 4-bit operand is four registers, and lane group q holds the 32 CONSECUTIVE elements
    // [32q, 32q+32) of K in them (block q, scaled by its own lanes' byte) -- unlike the 8-bit operand above, whose
    // groups hold two runs of 16.  Measured with one-hot operands: the instruction pairs K indices, not lane groups.
    // Rows are stored in four 16-byte pieces, piece c at position c ^ (row / 4) % 4.
    const int keyb = (frow / RPWB) & (CPRB - 1);
    const int w4off = (fq ^ keyb) << 4;
    auto load_frag_b = [&](const char* st, int rowbase) -> v8i {
        if constexpr (W4) {
            const v4i lo = *(const v4i*)(st + rowbase + w4off);
            return (v8i){lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
        } else {
            return load_frag(st, rowbase);
        }
    };

    // Pipeline (two stages).  The loop is rotated: on entry to tile kt its x1 fragments, its first x2 fragment and its
    // scales are already on their way to registers.  The x2 fragments stream through two register sets, each requested
    // one fragment ahead.  Before the LAST fragment of the tile: wait for this thread's copies of tile kt+1, barrier
    // (tile kt+1 is complete in LDS, every wave has read all it needs of tile kt); then, in the shadow of the last
    // fragment's MFMAs, start the copy of tile kt+2 into the freed stage and request tile kt+1's first operands, each x1
    // fragment as soon as the MFMA that reads its predecessor has been issued.
    // One MFMA contracts a whole scale block from a zero accumulator; the vector ALU folds the four partial sums of the
    // previous x2 fragment into the running sums while the matrix pipe works on the current one (the last fragment of
    // a tile is folded during the first of the next).  The fences keep this issue order.
    static_assert(STAGES == 2, "the rotated loop below is written for two stages");
    issue_tile(0);
    if (KT > 1) {
        issue_tile(1);
        wait_vmcnt<CPT>();
    } else {
        wait_vmcnt<0>();
    }
    __builtin_amdgcn_s_barrier();
#if QG_DBG
    const unsigned long long dbg_t1 = wall_clock64();
    const unsigned long long dbg_c1 = clock64();
#endif
    v8i fa[FM], fb[2];
    float sc[FM], s1raw[FM], s2raw;          // block-scale mode
    uint32_t sca[FM], saraw[FM], sbraw[2];   // MX mode: this lane's scale byte sits in bits 0..7 once shifted by 8 * fq
    (void)sc; (void)s1raw; (void)s2raw; (void)sca; (void)saraw; (void)sbraw;
    using part_t = std::conditional_t<I8, v4i, v4f>;   // a block's partial sums: exact int32 for int8 operands
    part_t part[2][FM];
    auto read_scales = [&](const char* st) {
        if constexpr (RC) {
        } else if constexpr (MX) {
            const uint32_t* sS = (const uint32_t*)(st + A_BYTES + B_BYTES);
#pragma unroll
            for (int j = 0; j < FM; j++) saraw[j] = sS[wm * TM + j * 16 + frow];
        } else {
            const float* sS = (const float*)(st + A_BYTES + B_BYTES);
            s2raw = sS[BM + wn];
#pragma unroll
            for (int j = 0; j < FM; j++) s1raw[j] = sS[wm * TM + j * 16 + frow];
        }
    };
    auto read_bscale = [&](const char* st, int i) -> uint32_t {   // MX: the scale dword of this lane's row of x2 fragment i
        return ((const uint32_t*)(st + A_BYTES + B_BYTES))[BM + wn * TN + i * 16 + frow];
    };
    {
        const char* st = smem;
        read_scales(st);
#pragma unroll
        for (int j = 0; j < FM; j++) fa[j] = load_frag(st, a_rowbase + j * 16 * BK);
        fb[0] = load_frag_b(st, b_rowbase);
        if constexpr (MX) sbraw[0] = read_bscale(st, 0);
#pragma unroll
        for (int j = 0; j < FM; j++) {
            sc[j] = 0.0f;   // multiplies the zero partial sums in the first tile's first fragment
            part[1][j] = part_t{0, 0, 0, 0};
        }
    }
    constexpr int CPS = (CPT + FM - 1) / FM;   // copies issued behind each of the last fragment's MFMAs

    for (int kt = 0; kt < KT; kt++) {
        const char* st = smem + (kt & 1) * STAGE;
        const char* stn = smem + ((kt + 1) & 1) * STAGE;
        // past the end the copies repeat the last tile (into a stage nobody reads any more): no branches in the loop
        const int ktc = kt + 2 < KT ? kt + 2 : KT - 1;
#pragma unroll
        for (int i = 0; i < FN; i++) {
            if (i + 1 < FN) {
                fb[(i + 1) & 1] = load_frag_b(st, b_rowbase + (i + 1) * 16 * BKB);
                if constexpr (MX) sbraw[(i + 1) & 1] = read_bscale(st, i + 1);
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_waitcnt(0xc07f | ((MX && !W4 ? 3 : 2) << 8));   // lgkmcnt: all but the reads just issued
            } else {
#if QG_DBG
                wait_lgkmcnt0();
                const unsigned long long c0 = clock64();
#endif
                wait_vmcnt<0>();
                wait_lgkmcnt0();
#if QG_DBG
                const unsigned long long c1 = clock64();
#endif
                __builtin_amdgcn_s_barrier();
#if QG_DBG
                const unsigned long long c2 = clock64();
                dbg_vm += c1 - c0; dbg_bar += c2 - c1; dbg_n++;
#endif
                __builtin_amdgcn_sched_barrier(0);
                read_scales(stn);
                fb[0] = load_frag_b(stn, b_rowbase);
                if constexpr (MX) sbraw[0] = read_bscale(stn, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            uint32_t scb = 0x7f7f7f7fu;
            if constexpr (MX) {
                if (i == 0) {   // this tile's x1 scales (requested behind the previous tile's barrier)
#pragma unroll
                    for (int j = 0; j < FM; j++) sca[j] = saraw[j] >> (8 * fq);
                }
                scb = sbraw[i & 1] >> (8 * fq);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int j = 0; j < FM; j++) {
                if constexpr (MX)   // the instruction applies both scales: accumulate in place, nothing to fold
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[i & 1], fa[j], acc[i][j], W4 ? 4 : 0, 0, 0, (int)scb, 0, (int)sca[j]);
                else if constexpr (RC)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[i & 1], fa[j], acc[i][j], 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
                else if constexpr (I8) {   // two 64-byte steps; the block's integer sum is exact
                    const v4i t = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_shufflevector(fb[i & 1], fb[i & 1], 0, 1, 2, 3),
                                                                        __builtin_shufflevector(fa[j], fa[j], 0, 1, 2, 3), v4i{0, 0, 0, 0}, 0, 0, 0);
                    part[i & 1][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_shufflevector(fb[i & 1], fb[i & 1], 4, 5, 6, 7),
                                                                           __builtin_shufflevector(fa[j], fa[j], 4, 5, 6, 7), t, 0, 0, 0);
                } else
                    part[i & 1][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[i & 1], fa[j], v4f{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0,
                                                                                      0x7f7f7f7f, 0, 0x7f7f7f7f);
                __builtin_amdgcn_sched_barrier(0);
                if (i == FN - 1) {
                    fa[j] = load_frag(stn, a_rowbase + j * 16 * BK);
#pragma unroll
                    for (int c = j * CPS; c < (j + 1) * CPS && c < CPT; c++) issue_piece(ktc, kt & 1, c);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if constexpr (!BLK) {
                } else if (i > 0) {
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[i - 1][j][r] = __builtin_fmaf((float)part[(i - 1) & 1][j][r], sc[j], acc[i - 1][j][r]);
                } else {   // the previous tile's last fragment, still with that tile's scales
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[FN - 1][j][r] = __builtin_fmaf((float)part[1][j][r], sc[j], acc[FN - 1][j][r]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (BLK && i == 0) {   // from here on this tile's scales
#pragma unroll
                for (int j = 0; j < FM; j++) sc[j] = s1raw[j] * s2raw;
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < FM; j++) {
        if constexpr (BLK) {
#pragma unroll
            for (int r = 0; r < 4; r++) acc[FN - 1][j][r] = __builtin_fmaf((float)part[1][j][r], sc[j], acc[FN - 1][j][r]);
        }
    }
    wait_lgkmcnt0();   // the reads and copies past the last tile land before LDS is reused
    wait_vmcnt<0>();

    // Epilogue: acc[i][j][r] is out[m = m_base + 16j + lane%16][n = n_base + 16i + 4*(lane/16) + r].  Each wave parks
    // one 16 x 128 block in a private LDS patch and reads it back row-wise, so that every store instruction writes
    // whole 128-byte lines (16 bytes per lane, 16 lanes per row) instead of 8 bytes in each of 16 rows.
    __syncthreads();   // every wave is done with the operand stages
#if QG_DBG
    const unsigned long long dbg_t2 = wall_clock64();
    const unsigned long long dbg_c2 = clock64();
#endif
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
    typedef v4us __attribute__((may_alias)) v4us_a;
    typedef v4i __attribute__((may_alias)) v4i_a;
    constexpr int EP_PITCH = TN * 2 + 16;
    char* ep = smem + wave * (16 * EP_PITCH);
    static_assert(WGM * 2 * 16 * EP_PITCH <= STAGES * STAGE, "epilogue staging fits in the operand stages");
    uint16_t* out = (uint16_t*)p.out + bz * p.M * p.N;
    const bool vec_ok = (p.N % 8) == 0 && ((uintptr_t)p.out % 16) == 0;
    const int er = lane >> 4, ec = lane & 15;
    float rs_j[FM];   // row / column scale mode: the scale of this lane's output row in each x1 fragment
    (void)rs_j;
    if constexpr (RC) {
#pragma unroll
        for (int j = 0; j < FM; j++) {
            const int64_t mrow = m0 + wm * TM + j * 16 + frow;
            rs_j[j] = p.rs[(mrow < p.M ? mrow : p.M - 1) * p.rs_stride];
        }
    }
#pragma unroll
    for (int j = 0; j < FM; j++) {
#pragma unroll
        for (int i = 0; i < FN; i++) {
            v4f v = acc[i][j];
            if constexpr (RC) {   // (sum * x2Scale[n]) * x1Scale[m], each product rounded, as compute_pertoken orders them
                const int64_t nb = n0 + wn * TN + i * 16 + 4 * fq;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float c = p.cs[(nb + r < p.N ? nb + r : p.N - 1) * p.cs_stride];
                    v[r] = (v[r] * c) * rs_j[j];
                }
            }
            if constexpr (MX || RC || I8) {
                if (p.bias) {
                    const int64_t nb = n0 + wn * TN + i * 16 + 4 * fq;
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int64_t bi = bz * p.bias_bs + (nb + r < p.N ? nb + r : p.N - 1);
                        v[r] = v[r] + (W4 ? load_scalar_as_f32(p.bias, p.bias_dt, bi) : p.bias[bi]);
                    }
                }
            }
            *(v4us_a*)(ep + frow * EP_PITCH + (i * 16 + 4 * fq) * 2) = pack4_b16<OUT_DT>(v);
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int row = r * 4 + er;
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
#if QG_DBG
    {
        const unsigned long long dbg_t3 = wall_clock64();
        wait_vmcnt<0>();
        const unsigned long long dbg_t4 = wall_clock64();
        if (lane == 0 && p.dbg) {
            unsigned long long* d = p.dbg + ((size_t)blockIdx.x * (WGM * 2) + wave) * 16;
            d[0] = dbg_t0; d[1] = dbg_t1; d[2] = dbg_t2; d[3] = dbg_t3; d[4] = dbg_t4; d[5] = dbg_vm; d[6] = dbg_bar; d[7] = dbg_n; d[8] = dbg_c2 - dbg_c1;
        }
    }
#endif
}

// out[b, m, n] = rounded(sum over the splits, in split order, of part[s, b, m, n] + bias[b, n])
template <int OUT_DT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* part, int splits, int64_t total, int64_t MN, int64_t N,
                                                            const void* bias, int bias_dt, int64_t bias_bs, uint16_t* out)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        float v = splitk_sum(part, splits, total, i);
        if (bias) v = v + load_scalar_as_f32(bias, bias_dt, (i / MN) * bias_bs + i % N);
        out[i] = OUT_DT == DT_BF16 ? bf16_bits(v) : f16_bits(v);
    }
}

template <int WGM, int STAGES, int OUT_DT, int MODE = FP8_BLOCK>
static int launch_fp8_block(const Fp8BlkParams& p, int64_t batch, hipStream_t st)
{
    constexpr int BM = 64 * WGM;
    int tiles_m = (int)((p.M + BM - 1) / BM), tiles_n = (int)((p.N + 255) / 256);
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)batch);
    size_t lds = (size_t)STAGES * (BM * 128 + 256 * (MODE == FP8_MX_W4 ? 64 : 128) + WGM * 128 * 4);
    if constexpr (MODE == FP8_MX_W4 || MODE == I8_BLOCK) {
        if (p.splits > 1) {   // K split over workgroups, then the sum of the partial sums, the bias and the rounding
            if (!p.part || p.splits > p.K / 128) return -1;
            auto ks = qmm_fp8_block_kernel<WGM, STAGES, DT_F32, MODE, true>;
            static std::atomic<uint64_t> attr_set_s{0};
            if (!device_flag_test(attr_set_s)) {
                hipError_t e = hipFuncSetAttribute((const void*)ks, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
                if (e != hipSuccess) return (int)e;
                device_flag_set(attr_set_s);
            }
            grid.z = (unsigned)p.splits;
            hipLaunchKernelGGL(ks, grid, dim3(WGM * 128), lds, st, p, tiles_m, tiles_n);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return (int)e;
            const int64_t total = batch * p.M * p.N;
            const unsigned rgrid = splitk_reduce_grid(total);
            hipLaunchKernelGGL(splitk_reduce_kernel<OUT_DT>, dim3(rgrid), dim3(256), 0, st, (const float*)p.part, p.splits, total,
                               p.M * p.N, p.N, (const void*)p.bias, MODE == FP8_MX_W4 ? p.bias_dt : DT_F32, p.bias_bs, (uint16_t*)p.out);
            return (int)hipGetLastError();
        }
    }
    auto k = qmm_fp8_block_kernel<WGM, STAGES, OUT_DT, MODE>;
    static std::atomic<uint64_t> attr_set{0};   // one bit per device: the attribute belongs to the (kernel, device) pair
    if (!device_flag_test(attr_set)) {
        hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        device_flag_set(attr_set);
    }
    hipLaunchKernelGGL(k, grid, dim3(WGM * 128), lds, st, p, tiles_m, tiles_n);
    return (int)hipGetLastError();
}

int launch_mxfp8_wide(const QgemmParams& p, int fn, int64_t batch, int out_dt, hipStream_t st);   // qmm_int8_wide.hip
extern "C" int opsnn_mx8_wide();   // dispatch.hip

// MXFP8 (e4m3 x e4m3, e8m0 scale per 32 K) on the same kernel in MX mode.  Operands and scales must be K-contiguous with
// K % 128 == 0 (four scale bytes per row per K tile); out[m,n] = sum_k (x1 s1)(x2 s2) + fp32 bias.
int launch_mxfp8_mfma(const OpsnnQmmArgs& a, hipStream_t st)
{
    Fp8BlkParams p{};
    p.a = (const int8_t*)a.x1.ptr; p.b = (const int8_t*)a.x2.ptr;
    p.lda = a.x1.row_stride; p.ldb = a.x2.col_stride; p.a_bs = a.x1.batch_stride; p.b_bs = a.x2.batch_stride;
    p.out = a.out; p.M = a.M; p.N = a.N; p.K = a.K; p.gsM = 1;
    p.sa = (const uint8_t*)a.x1_scale_mat.ptr; p.sb = (const uint8_t*)a.x2_scale_mat.ptr;
    p.sa_rs = a.x1_scale_mat.row_stride; p.sb_rs = a.x2_scale_mat.row_stride;
    p.sa_bs = a.x1_scale_mat.batch_stride; p.sb_bs = a.x2_scale_mat.batch_stride;
    p.bias = (const float*)a.bias; p.bias_bs = a.bias_batch_stride;
    if (a.K % 128 != 0 || a.x1.col_stride != 1 || a.x2.row_stride != 1) return OPSNN_NOT_TAKEN;
    if (a.x1_scale_mat.col_stride != 2 || a.x2_scale_mat.col_stride != 2) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)p.a | (uintptr_t)p.b | (uint64_t)p.lda | (uint64_t)p.ldb | (uint64_t)p.a_bs | (uint64_t)p.b_bs) % 16) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)p.sa | (uintptr_t)p.sb | (uint64_t)p.sa_rs | (uint64_t)p.sb_rs | (uint64_t)p.sa_bs | (uint64_t)p.sb_bs) % 4) return OPSNN_NOT_TAKEN;
    if (a.bias && a.bias_dtype != DT_F32) return OPSNN_NOT_TAKEN;
    // Large problems: the four-wave kernel with the tile width that fills its rounds of CUs best, as for the row/column
    // scale modes below (K % 512 == 0 and 16-byte aligned scale rows, else it declines).  opsnnSetMx8Wide(8 or 9) forces that
    // kernel with that width (tests, tuning), 0 forbids it.
    {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        const int forced = opsnn_mx8_wide();
        const int64_t tm = (a.M + 255) / 256, tn = (a.N + 255) / 256;
        int wide_fn = 0;
        if (forced >= 8 && forced <= 9) {
            wide_fn = forced;
        } else if (forced != 0 && a.K >= 1024 && tm * tn * a.batch * 4 >= (int64_t)cus * 3) {
            const int64_t block_cost = (tm * tn * a.batch + cus - 1) / cus * 10;
            int64_t wide_cost = INT64_MAX;
            for (int fn = 8; fn <= 9; fn++) {   // wider tiles leave no room in LDS for the scale slots
                const int64_t tiles = tm * ((a.N + 32 * fn - 1) / (32 * fn)) * a.batch;
                const int64_t cost = (tiles + cus - 1) / cus * (fn + 2);
                if (cost < wide_cost) { wide_cost = cost; wide_fn = fn; }
            }
            if (wide_cost > block_cost) wide_fn = 0;
        }
        if (wide_fn) {
            QgemmParams g{};
            g.a = p.a; g.b = p.b; g.lda = p.lda; g.ldb = p.ldb; g.a_bs = p.a_bs; g.b_bs = p.b_bs;
            g.out = a.out; g.M = a.M; g.N = a.N; g.ldc = a.N; g.KB = a.K;
            g.bias = a.bias; g.bias_dt = DT_F32; g.bias_bs = a.bias_batch_stride;
            g.sa = p.sa; g.sb = p.sb; g.sa_rs = p.sa_rs; g.sb_rs = p.sb_rs; g.sa_bs = p.sa_bs; g.sb_bs = p.sb_bs;
            const int rc = launch_mxfp8_wide(g, wide_fn, a.batch, a.out_dtype, st);
            if (rc != OPSNN_NOT_TAKEN) return rc;
        }
    }
    if (a.out_dtype == DT_BF16) return launch_fp8_block<4, 2, DT_BF16, FP8_MX>(p, a.batch, st);
    if (a.out_dtype == DT_F16) return launch_fp8_block<4, 2, DT_F16, FP8_MX>(p, a.batch, st);
    return OPSNN_NOT_TAKEN;
}

int launch_f8_wide(const QgemmParams& p, int fn, int64_t batch, int out_dt, hipStream_t st);   // qmm_int8_wide.hip
int launch_blockscale_exact(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk = {});   // qmm_fp8_exact.hip
int launch_rowcol_exact(const OpsnnQmmArgs& a, hipStream_t st, int ep_mode, SplitK sk = {});

// fp8 e4m3 x fp4 e2m1 with e8m0 scales per 32 K on both operands (compute_mx of quant_batch_matmul_v4,
// qbmmv4_kernel_golden.py:119-186): the MX mode with a 4-bit x2.  x2 [N, K] K-contiguous (two elements per byte),
// K % 128 == 0, bias fp32 or 16-bit.
int launch_mx_a8w4_decode(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk);   // qmm_fp8_decode.hip

int launch_mx_a8w4_mfma(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk)
{
    if (a.x1_dtype != DT_E4M3 || a.x2_dtype != DT_E2M1) return OPSNN_NOT_TAKEN;
    {   // up to 32 rows: the stream over x2 with x1 in registers
        const int rc = launch_mx_a8w4_decode(a, st, sk);
        if (rc != OPSNN_NOT_TAKEN) return rc;
        if (a.M <= 16) sk = SplitK{};   // (the partial sums were laid out for the kernel above; the tile kernel runs unsplit)
    }
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16) return OPSNN_NOT_TAKEN;
    if (a.K % 128 != 0 || a.M * a.N < 64 * 64 || a.x1.col_stride != 1 || a.x2.row_stride != 1) return OPSNN_NOT_TAKEN;
    if (a.x1_scale_mat.col_stride != 2 || a.x2_scale_mat.col_stride != 2) return OPSNN_NOT_TAKEN;
    if (a.bias && a.bias_dtype != DT_F32 && a.bias_dtype != DT_BF16 && a.bias_dtype != DT_F16) return OPSNN_NOT_TAKEN;
    Fp8BlkParams p{};
    p.a = (const int8_t*)a.x1.ptr; p.b = (const int8_t*)a.x2.ptr;
    p.lda = a.x1.row_stride; p.ldb = a.x2.col_stride / 2;   // bytes per x2 row
    p.a_bs = a.x1.batch_stride; p.b_bs = a.x2.batch_stride / 2;
    p.out = a.out; p.M = a.M; p.N = a.N; p.K = a.K; p.gsM = 1;
    p.sa = (const uint8_t*)a.x1_scale_mat.ptr; p.sb = (const uint8_t*)a.x2_scale_mat.ptr;
    p.sa_rs = a.x1_scale_mat.row_stride; p.sb_rs = a.x2_scale_mat.row_stride;
    p.sa_bs = a.x1_scale_mat.batch_stride; p.sb_bs = a.x2_scale_mat.batch_stride;
    p.bias = (const float*)a.bias; p.bias_dt = a.bias_dtype; p.bias_bs = a.bias_batch_stride;
    if (a.x2.col_stride % 2) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)p.a | (uintptr_t)p.b | (uint64_t)p.lda | (uint64_t)p.ldb | (uint64_t)p.a_bs | (uint64_t)p.b_bs) % 16) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)p.sa | (uintptr_t)p.sb | (uint64_t)p.sa_rs | (uint64_t)p.sb_rs | (uint64_t)p.sa_bs | (uint64_t)p.sb_bs) % 4) return OPSNN_NOT_TAKEN;
    p.splits = sk.splits; p.part = sk.part;
    if (a.out_dtype == DT_BF16) return launch_fp8_block<4, 2, DT_BF16, FP8_MX_W4>(p, a.batch, st);
    return launch_fp8_block<4, 2, DT_F16, FP8_MX_W4>(p, a.batch, st);
}

// fp8 e4m3 x e4m3 with one fp32 scale per row of x1 (or one for all of it) and one per column of x2 (or one):
// K-C, K-T and the double-scale modes whose two scales are multiplied in separately
// (qbmmv3_kernel_golden.py:361-387 and :432-441).  out = (sum * x2Scale[n]) * x1Scale[m] + fp32 bias.
// Needs K-contiguous operands with K % 128 == 0 and a 16-bit output; anything else stays on the plain kernel.
int launch_fp8_rowcol_mfma(const OpsnnQmmArgs& a, hipStream_t st, bool merged_scales_ok, SplitK sk)
{
    if (a.x1_dtype != DT_E4M3 || a.x2_dtype != DT_E4M3) return OPSNN_NOT_TAKEN;
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16) return OPSNN_NOT_TAKEN;
    if (!a.x1_scale || !a.x2_scale || a.x2_scale_dtype != DT_F32) return OPSNN_NOT_TAKEN;
    if (a.x1_scale_len != 1 && a.x1_scale_len != a.M) return OPSNN_NOT_TAKEN;
    if (a.x2_scale_len != 1 && a.x2_scale_len != a.N) return OPSNN_NOT_TAKEN;
    // both scales one element and no bias is the double-scale mode whose scales are merged and truncated: plain kernel
    // (callers whose scales are not that mode's say so)
    if (!merged_scales_ok && a.x1_scale_len == 1 && a.x2_scale_len == 1 && !a.bias) return OPSNN_NOT_TAKEN;
    if (a.K % 128 != 0 || a.M * a.N < 64 * 64 || a.x1.col_stride != 1 || a.x2.row_stride != 1) return OPSNN_NOT_TAKEN;
    if (!opsnnGetFp8Fast() || (a.bias && a.bias_dtype != DT_F32)) {   // exact products and sums unless the caller asked for the 8-bit matrix instruction (whose epilogue takes an fp32 bias only)
        const int rc = launch_rowcol_exact(a, st, 0, sk);
        if (rc != OPSNN_NOT_TAKEN) return rc;
    }
    if (a.bias && a.bias_dtype != DT_F32) return OPSNN_NOT_TAKEN;
    Fp8BlkParams p{};
    p.a = (const int8_t*)a.x1.ptr; p.b = (const int8_t*)a.x2.ptr;
    p.lda = a.x1.row_stride; p.ldb = a.x2.col_stride; p.a_bs = a.x1.batch_stride; p.b_bs = a.x2.batch_stride;
    p.out = a.out; p.M = a.M; p.N = a.N; p.K = a.K; p.gsM = 1;
    p.rs = (const float*)a.x1_scale; p.rs_stride = a.x1_scale_len == 1 ? 0 : 1;
    p.cs = (const float*)a.x2_scale; p.cs_stride = a.x2_scale_len == 1 ? 0 : 1;
    p.bias = (const float*)a.bias; p.bias_bs = a.bias_batch_stride;
    if (((uintptr_t)p.a | (uintptr_t)p.b | (uint64_t)p.lda | (uint64_t)p.ldb | (uint64_t)p.a_bs | (uint64_t)p.b_bs) % 16) return OPSNN_NOT_TAKEN;
    // Large problems go to the four-wave kernel (one wave per SIMD, 128 x 16n register tiles: fewer LDS reads and half the
    // matrix instructions per flop of the int8 form) with the tile width 256 x 32n, n = 8..11, that fills its rounds of
    // CUs best (cost in rounds x 32-column units); the 8-wave kernel below keeps the small and the short-K problems.
    {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        const int64_t tm = (a.M + 255) / 256, tn = (a.N + 255) / 256;
        if (a.K >= 1024 && tm * tn * a.batch * 4 >= cus * 3) {
            const int64_t block_cost = (tm * tn * a.batch + cus - 1) / cus * 10;   // tile cost = width / 32 + 2, as for int8
            int64_t wide_cost = INT64_MAX;
            int wide_fn = 0;
            for (int fn = 8; fn <= 11; fn++) {
                const int64_t tiles = tm * ((a.N + 32 * fn - 1) / (32 * fn)) * a.batch;
                const int64_t cost = (tiles + cus - 1) / cus * (fn + 2);
                if (cost < wide_cost) { wide_cost = cost; wide_fn = fn; }
            }
            if (wide_cost <= block_cost) {   // at equal cost too: measured 211 against 260 us on 4096 x 8192 x 8192
                QgemmParams g{};
                g.a = p.a; g.b = p.b; g.lda = p.lda; g.ldb = p.ldb; g.a_bs = p.a_bs; g.b_bs = p.b_bs;
                g.out = a.out; g.M = a.M; g.N = a.N; g.ldc = a.N; g.KB = a.K;
                g.x1s = (const float*)a.x1_scale; g.x1s_one = a.x1_scale_len == 1 ? 1 : 0;
                g.x2s = a.x2_scale; g.x2s_dt = DT_F32; g.x2s_len = a.x2_scale_len;
                g.bias = a.bias; g.bias_dt = DT_F32; g.bias_bs = a.bias_batch_stride;
                const int rc = launch_f8_wide(g, wide_fn, a.batch, a.out_dtype, st);
                if (rc != OPSNN_NOT_TAKEN) return rc;
            }
        }
    }
    if (a.M >= 512) {
        if (a.out_dtype == DT_BF16) return launch_fp8_block<4, 2, DT_BF16, FP8_ROWCOL>(p, a.batch, st);
        return launch_fp8_block<4, 2, DT_F16, FP8_ROWCOL>(p, a.batch, st);
    }
    if (a.out_dtype == DT_BF16) return launch_fp8_block<2, 2, DT_BF16, FP8_ROWCOL>(p, a.batch, st);
    return launch_fp8_block<2, 2, DT_F16, FP8_ROWCOL>(p, a.batch, st);
}

int launch_blockscale_decode(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk);   // qmm_fp8_decode.hip
int launch_blockscale_rows(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk);     // qmm_fp8_rows.hip

int launch_blockscale_mfma(const OpsnnQmmArgs& a0, hipStream_t st, SplitK sk)
{
    OpsnnQmmArgs a = a0;
    const bool i8 = a.x1_dtype == DT_I8 && a.x2_dtype == DT_I8;   // the per-tile mode of quant_batch_matmul_v4 (qbmmv4_kernel_golden.py:258-325)
    if (!i8 && (a.x1_dtype != DT_E4M3 || a.x2_dtype != DT_E4M3)) return OPSNN_NOT_TAKEN;
    const bool out32 = a.out_dtype == DT_F32 && !i8;   // fp32 output: the exact kernel only
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16 && !out32) return OPSNN_NOT_TAKEN;
    if (a.bias && !(i8 && a.bias_dtype == DT_F32)) return OPSNN_NOT_TAKEN;
    if (a.gsK != 128 || a.gsN != 128 || (a.gsM != 1 && a.gsM != 128)) return OPSNN_NOT_TAKEN;
    // (fewer than 64 x 64 outputs: only the few-rows stream over x2 below, which wants 256 columns -- one row against a long K
    // is no work for one thread per output)
    const bool tiny = a.M * a.N < 64 * 64;
    if (a.K % 128 != 0 || a.x1.col_stride != 1 || (tiny && !(a.M <= 32 && a.N >= 256))) return OPSNN_NOT_TAKEN;
    if (a.x2.row_stride != 1) {
        // x2 is [K, N] with N contiguous: re-lay it out K-contiguous in the workspace (scales keep their layout)
        if (a.x2.col_stride != 1 || a.x2.row_stride != a.N) return OPSNN_NOT_TAKEN;
        if (a.x2.batch_stride != 0 && a.x2.batch_stride != a.K * a.N) return OPSNN_NOT_TAKEN;
        const int64_t nb = a.x2.batch_stride == 0 ? 1 : a.batch;
        if (const void* cached = weight_cache_get(a.x2.ptr, a.K, a.N, 8, nb, st)) a.x2.ptr = cached;   // the weight cache, when on
        else {
            if (!a.workspace) return OPSNN_NOT_TAKEN;
            int rc = opsnnTranspose8(a.x2.ptr, a.workspace, a.K, a.N, nb, st);
            if (rc != 0) return rc;
            a.x2.ptr = a.workspace;
        }
        a.x2.row_stride = 1; a.x2.col_stride = a.K;
    }
    if (!i8 && a0.x2.row_stride == 1) {   // 17 .. 128 rows: x1 widened into the workspace, then the many-rows streaming kernel
        const int rc = launch_blockscale_rows(a, st, sk);
        if (rc != OPSNN_NOT_TAKEN) return rc;
    }
    {   // up to 16 rows (32 in two passes where the kernel above does not apply): the stream over x2 with x1 in registers
        const int rc = launch_blockscale_decode(a, st, sk);
        if (rc != OPSNN_NOT_TAKEN) return rc;
    }
    if (tiny) return OPSNN_NOT_TAKEN;
    if (a.M <= (i8 ? 16 : 32)) sk = SplitK{};   // (with so few rows the partial sums were laid out for the kernel above; the tile kernels run unsplit)
    if (!i8 && (!opsnnGetFp8Fast() || out32)) {   // exact products and sums unless the caller asked for the 8-bit matrix instruction
        const int rc = launch_blockscale_exact(a, st, sk);
        if (rc != OPSNN_NOT_TAKEN || out32) return rc;
    }
    Fp8BlkParams p{};
    p.a = (const int8_t*)a.x1.ptr; p.b = (const int8_t*)a.x2.ptr;
    p.lda = a.x1.row_stride; p.ldb = a.x2.col_stride; p.a_bs = a.x1.batch_stride; p.b_bs = a.x2.batch_stride;
    p.out = a.out; p.M = a.M; p.N = a.N; p.K = a.K;
    p.s1 = (const float*)a.x1_scale_mat.ptr; p.s1_rs = a.x1_scale_mat.row_stride; p.s1_cs = a.x1_scale_mat.col_stride;
    p.s1_bs = a.x1_scale_mat.batch_stride;
    p.s2 = (const float*)a.x2_scale_mat.ptr; p.s2_rs = a.x2_scale_mat.row_stride; p.s2_cs = a.x2_scale_mat.col_stride;
    p.s2_bs = a.x2_scale_mat.batch_stride;
    p.gsM = (int)a.gsM;
    p.bias = (const float*)a.bias; p.bias_dt = DT_F32; p.bias_bs = a.bias_batch_stride;
    if (((uintptr_t)p.a | (uintptr_t)p.b | (uint64_t)p.lda | (uint64_t)p.ldb | (uint64_t)p.a_bs | (uint64_t)p.b_bs) % 16) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)p.s1 | (uintptr_t)p.s2) % 4) return OPSNN_NOT_TAKEN;
    // 256 x 256 tiles (8 waves) halve the operand traffic per flop; 128 x 256 (4 waves) keeps small M efficient
    const bool big = a.M >= 512;
    if (i8) {
        p.splits = sk.splits; p.part = sk.part;
        if (big) return a.out_dtype == DT_BF16 ? launch_fp8_block<4, 2, DT_BF16, I8_BLOCK>(p, a.batch, st) : launch_fp8_block<4, 2, DT_F16, I8_BLOCK>(p, a.batch, st);
        return a.out_dtype == DT_BF16 ? launch_fp8_block<2, 2, DT_BF16, I8_BLOCK>(p, a.batch, st) : launch_fp8_block<2, 2, DT_F16, I8_BLOCK>(p, a.batch, st);
    }
    if (big) {
        if (a.out_dtype == DT_BF16) return launch_fp8_block<4, 2, DT_BF16>(p, a.batch, st);
        return launch_fp8_block<4, 2, DT_F16>(p, a.batch, st);
    }
    if (a.out_dtype == DT_BF16) return launch_fp8_block<2, 2, DT_BF16>(p, a.batch, st);
    return launch_fp8_block<2, 2, DT_F16>(p, a.batch, st);
}

}  // namespace opsnn
