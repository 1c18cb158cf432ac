// Shared tile-GEMM core for the 8-bit / 4-bit quantized matmuls on gfx950.
//
// One kernel template, specialised by MODE:
//   MODE_I8     int8 x int8 -> int32 (v_mfma_i32_32x32x32_i8), per-token / per-channel dequant epilogue
//   MODE_MXFP4  fp4 e2m1 x fp4 e2m1 with e8m0 scales per 32 K (v_mfma_scale_f32_32x32x64_f8f6f4), bias epilogue
//   MODE_MXFP8  fp8 e4m3 x fp8 e4m3 with e8m0 scales per 32 K (same instruction, 8-bit formats)
// Both operands are K-contiguous ("x2 stored [N, K]") with 16-byte aligned rows.  Everything is addressed in
// BYTES of the packed operand rows, so int8 and fp4 share all data movement (32 bytes of K per row per MFMA)
// and fp8 uses 64.
//
//   - BM x BN output tile per workgroup, WGM x WGN waves, each wave owns a (BM/WGM) x (BN/WGN) sub-tile of
//     32x32 MFMA fragments with accumulators held in registers for the whole K loop;
//   - K tiles of BK bytes are copied global -> LDS asynchronously (16 B per lane, no register round trip),
//     STAGES deep; MX scale bytes ride along as 4-byte async copies;
//   - LDS rows are XOR-swizzled in 16-byte chunks so the MFMA operand reads are bank-conflict free;
//   - the MFMA is issued as x2-fragment x x1-fragment so every lane ends up with four consecutive n of one
//     output row: epilogue vectors load as float4 and the 16-bit results leave as 8-byte stores.
#pragma once
#include <type_traits>
// -DQG_DBG=1 adds per-wave timestamps (start, loop start/end, end) and the clocks spent waiting for copies and at the
// barrier, written to QgemmParams::dbg (16 x 8 bytes per wave); for timing harnesses, never set in the library build.
#ifndef QG_DBG
#define QG_DBG 0
#endif

#include "common.hip.h"

namespace opsnn {

enum : int { MODE_I8 = 0, MODE_MXFP4 = 1, MODE_MXFP8 = 2 };

struct QgemmParams {
    const int8_t* a;   // x1 rows, K-contiguous
    const int8_t* b;   // x2 rows (one per n), K-contiguous
    int64_t lda, ldb;  // row strides in bytes
    int64_t a_bs, b_bs;  // batch strides in bytes (0 = broadcast)
    void* out;         // 16-bit floats; element (m, n) of batch b at out[(b*M + m)*ldc + n]
    int64_t M, N, KB;  // KB = bytes of K per operand row
    int64_t ldc;       // output row pitch in elements (N, or wider when this launch covers a column range)
    // MODE_I8 epilogue: out = cast(fp32(acc + ib[n]) * x2s[n] * x1s[m] + fb[n])
    const float* x1s;
    int x1s_one;       // x1s is one scale for every row (honoured by the four-wave kernel only)
    const void* x2s;   // FLOAT / BF16, or UINT64 words whose low 32 bits are the fp32 scale
    int x2s_dt;
    int64_t x2s_len;
    int x2s_trunc;     // keep only the upper 19 bits of the scale (always done for UINT64 words)
    // integer outputs of MODE_I8 (OUT_DT INT32: acc + ib[n];  INT8: clip(s9(s9(fp32(acc + ib[n]) * x2s[n]) + s9(off[n])), the offset
    // from x2off or, for UINT64 scale words, from their bits 37..45; s9 = round half to even, clamp to [-256, 255])
    const float* x2off;
    int64_t x2off_len;
    // bias: int32 / 16-bit / fp32 for MODE_I8, fp32 for the MX modes
    const void* bias;
    int bias_dt;
    int64_t bias_bs;
    // MX: one e8m0 byte per 32 K elements, K-contiguous per row
    const uint8_t* sa;
    const uint8_t* sb;
    int64_t sa_rs, sb_rs, sa_bs, sb_bs;
    // When set: the launch computes only if one of gate[0 .. gate_n) is non-zero (the flags of the pass that prepares the
    // exact MX route, whose kernel then left the call to this one); otherwise every workgroup returns at once.
    const int* gate;
    int gate_n;
    // K split over `splits` workgroups per tile (SPLIT instantiations, grid.z): partial sums [splits][batch][M][N] -- int32
    // for MODE_I8 (qg_i8_splitk_reduce_kernel adds them exactly and applies the epilogue), fp32 with the MX scales applied
    // for the MX modes (qg_mx_splitk_reduce_kernel adds them in split order, then the bias)
    int splits;
    int32_t* part;
#if QG_DBG
    unsigned long long* dbg;
#endif
};

__device__ __attribute__((aligned(16))) static const int8_t g_zero16[16] = {0};

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding: vmcnt = imm[3:0] | imm[15:14] << 4).
template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt range");
    __builtin_amdgcn_s_waitcnt((N & 15) | (((N >> 4) & 3) << 14) | (7 << 4) | (15 << 8));
}
__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(15 | (3 << 14) | (7 << 4) | (0 << 8)); }

// 4-byte asynchronous copy global -> LDS; lane l lands at lds + 4*l.
__device__ __forceinline__ void async_copy4(const void* g, void* lds)
{
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                     (__attribute__((address_space(3))) void*)lds, 4, 0, 0);
}

template <int MODE, int BM, int BN, int BK, int WGM, int WGN, int STAGES, int MINWG, bool KTAIL, int OUT_DT, bool SPLIT = false>
__global__ __launch_bounds__(WGM* WGN * 64, MINWG) void qgemm_kernel(QgemmParams p, int tiles_m, int tiles_n)
{
    static_assert(!SPLIT || !KTAIL, "the K split: whole K tiles");
    constexpr bool MX = MODE != MODE_I8;
    constexpr int NT = WGM * WGN * 64;
    constexpr int CPR = BK / 16;                 // 16-byte chunks per LDS row
    constexpr int RPW = 16 / CPR;                // rows per 256-byte LDS bank wrap
    constexpr int TM = BM / WGM, TN = BN / WGN;  // per-wave tile
    constexpr int FM = TM / 32, FN = TN / 32;
    constexpr int KSTEP = MODE == MODE_MXFP8 ? 64 : 32;  // bytes of K per row per MFMA
    constexpr int FREG = KSTEP / 8;                      // operand dwords per lane per fragment
    constexpr int KS = BK / KSTEP;                       // MFMA K steps per tile
    constexpr int SCB = MX ? BK / (MODE == MODE_MXFP8 ? 32 : 16) : 0;  // scale bytes per row per tile
    constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
    constexpr int SCW = MX ? SCB / 4 : 1;                // scale dwords per row per tile
    // Eight scale bytes per row per tile (fp4, BK = 128): one 16-byte copy per row brings the scales of TWO K tiles
    // (a 4-byte copy per row costs a whole cache-line request for 4 useful bytes, as many requests as the operands
    // themselves); they live in a ring of two slots behind the operand stages.
    constexpr bool SC16 = MX && SCB == 8;
    constexpr int SC_BYTES = (MX && !SC16) ? (BM + BN) * SCB : 0;
    constexpr int STAGE = A_BYTES + B_BYTES + SC_BYTES;
    constexpr int SC_RING = STAGES * STAGE;              // SC16: two slots of (BM + BN) * 16 bytes from here
    constexpr int RPI = NT / CPR;                // tile rows covered by one copy instruction of the workgroup
    constexpr int NA = BM / RPI, NB = BN / RPI;  // copy instructions per thread per tile
    constexpr int NSC = MX ? (SC16 ? (BM + BN) / NT : (BM + BN) * SCW / NT) : 0; // scale-copy instructions per thread (SC16: per tile pair)
    constexpr int CPT = NA + NB + (SC16 ? 0 : NSC);     // copies per tile that the wait counts step by
    static_assert(CPR == 8 || CPR == 4, "BK must be 64 or 128");
    static_assert(BM % RPI == 0 && BN % RPI == 0, "tile rows must be a multiple of the rows one copy pass covers");
    static_assert(STAGES >= 2 && STAGES * CPT < 64, "stage count");
    static_assert(KS % 2 == 0, "operand double buffer parity");
    static_assert(!MX || SCB == 4 || SCB == 8, "MX tiles carry four or eight scale bytes per row");
    static_assert(!MX || (SC16 ? (BM + BN) % NT == 0 : ((BM + BN) * SCW) % NT == 0), "scale copy mapping");
    static_assert(!SC16 || STAGES == 2, "paired scale copies are waited for with the two-stage counts");
    static_assert(!MX || !KTAIL, "MX fast path takes whole K tiles only");
    extern __shared__ __attribute__((aligned(16))) char smem[];

#if QG_DBG
    const unsigned long long dbg_t0 = wall_clock64();
    unsigned long long dbg_vm = 0, dbg_bar = 0, dbg_n = 0;
#endif
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    if constexpr (MX) {
        if (p.gate) {
            int f = 0;
            for (int i = 0; i < p.gate_n; i++) f |= p.gate[i];   // every thread reads every flag: uniform loads, no LDS for a vote
            if (!f) return;
        }
    }

    // Tile order: each XCD (own L2) gets a contiguous range of ids, and ids run down groups of GM row tiles and across the
    // columns inside a group, so that the 32 tiles an XCD works on at a time form a GM x (32 / GM) block sharing GM x1
    // panels and 32 / GM x2 panels (with whole columns of 16 row tiles it was 16 + 2 panels per K step, and every x1 panel
    // was fetched once per pair of columns).
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
    const int64_t K = p.KB;
    int KT = (int)((K + BK - 1) / BK);
    int kt_first = 0;
    if constexpr (SPLIT) {   // this workgroup's K tiles: kt_first .. kt_first + KT - 1 (at least STAGES: the launcher splits at most KT / 4 ways)
        // (tiles whose scales travel in pairs are dealt in pairs)
        constexpr int U = (MX && BK / (MODE == MODE_MXFP8 ? 32 : 16) == 8) ? 2 : 1;
        const int z = (int)blockIdx.z, units = KT / U;
        kt_first = (int)((int64_t)z * units / p.splits) * U;
        KT = (int)((int64_t)(z + 1) * units / p.splits) * U - kt_first;
        A += (int64_t)kt_first * BK;
        B += (int64_t)kt_first * BK;
    }

    // LDS layout of one operand tile: row r holds CPR chunks of 16 bytes; logical chunk c is stored at position
    // c ^ key(r), key(r) = (r / RPW) % CPR, so that 16 consecutive rows at one logical chunk hit 16 different
    // 16-byte bank groups.
    // Async copies: copy instruction i of the workgroup fills LDS chunks [i*NT, (i+1)*NT), i.e. tile rows
    // i*RPI .. i*RPI+RPI-1; this thread always handles row i*RPI + tid/CPR and the chunk computed below.
    // Rows past the matrix edge are clamped to the last valid row: they only feed outputs that are never stored.
    const int crow = tid / CPR;
    const int cchunk = (tid % CPR) ^ ((crow / RPW) & (CPR - 1));  // RPI is a multiple of RPW*CPR: same key for every i
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
    const int8_t* const zero_page = g_zero16;
    // MX scales: the stacked [x1 rows; x2 rows] of the tile need SCW dwords of scale bytes each per K tile; copy
    // number c = i*NT + tid moves dword c % SCW of stacked row c / SCW, so a row's scale bytes are contiguous in LDS.
    const uint8_t* sc_src[NSC > 0 ? NSC : 1];
    if constexpr (MX) {
#pragma unroll
        for (int i = 0; i < NSC; i++) {
            const int c = i * NT + tid;
            const int r = SC16 ? c : c / SCW, part = SC16 ? 0 : c % SCW;
            if (r < BM) {
                int rr = r < a_rows ? r : a_rows - 1;
                sc_src[i] = p.sa + bz * p.sa_bs + (m0 + rr) * p.sa_rs + part * 4;
            } else {
                int rr = r - BM;
                rr = rr < b_rows ? rr : b_rows - 1;
                sc_src[i] = p.sb + bz * p.sb_bs + (n0 + rr) * p.sb_rs + part * 4;
            }
            if constexpr (SPLIT) sc_src[i] += SC16 ? (int64_t)(kt_first >> 1) * 16 : (int64_t)kt_first * SCB;
        }
    }

    auto issue_tile = [&](int kt, auto with_scales) {   // with_scales: SC16 only, true for even tiles
        (void)with_scales;
        char* sA = smem + (kt % STAGES) * STAGE + wave * 1024;
        char* sB = sA + A_BYTES;
        const int64_t k0 = (int64_t)kt * BK;
        const int8_t* Ak = A + k0;
        const int8_t* Bk = B + k0;
        const bool kok = !KTAIL || (k0 + cchunk * 16) < K;
#pragma unroll
        for (int i = 0; i < NA; i++) {
            const int8_t* g = Ak + a_off[i];
            if constexpr (KTAIL) g = kok ? g : zero_page;
            async_copy16(g, sA + i * NT * 16);
        }
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const int8_t* g = Bk + b_off[i];
            if constexpr (KTAIL) g = kok ? g : zero_page;
            async_copy16(g, sB + i * NT * 16);
        }
        if constexpr (SC16) {
            if constexpr (decltype(with_scales)::value) {   // scales of tiles kt and kt+1; the slot's last reader was tile kt-1
                char* sS = smem + SC_RING + ((kt >> 1) & 1) * ((BM + BN) * 16) + wave * 1024;
#pragma unroll
                for (int i = 0; i < NSC; i++) async_copy16(sc_src[i] + (int64_t)(kt >> 1) * 16, sS + i * NT * 16);
            }
        } else if constexpr (MX) {
            char* sS = smem + (kt % STAGES) * STAGE + A_BYTES + B_BYTES + wave * 256;
#pragma unroll
            for (int i = 0; i < NSC; i++) async_copy4(sc_src[i] + (int64_t)kt * SCB, sS + i * NT * 4);
        }
    };

    using Acc = std::conditional_t<MODE == MODE_I8, v16i, v16f>;
    Acc acc[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; i++)
#pragma unroll
        for (int j = 0; j < FM; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    // Operand fragments, lane (row = lane%32, half = lane/32):
    //   32-byte K steps (int8, fp4): the lane's four operand dwords are bytes [16*half, 16*half+16) of the step;
    //   64-byte K steps (fp8): dwords 0-3 are bytes [16*half, +16) and dwords 4-7 bytes [32+16*half, +16) -- the
    //   8-bit form of the instruction consumes K in two 32-element blocks, dwords 0-3 of all lanes first.  The
    //   lane's scale byte belongs to block `half`, whichever registers hold that block's data.
    const int frow = lane & 31;
    const int fkc = lane >> 5;
    const int key = (frow / RPW) & (CPR - 1);  // 32-row fragments start at multiples of RPW*CPR rows
    const int swz = fkc ^ key;                 // KSTEP 32: chunk 2s + half
    const int swz0 = fkc ^ key;                // KSTEP 64: chunks 4s + half and 4s + 2 + half (see load_frags)
    const int swz1 = (2 + fkc) ^ key;
    const int a_rowbase = (wm * TM + frow) * BK;
    const int b_rowbase = A_BYTES + (wn * TN + frow) * BK;

    typedef int frag_t __attribute__((ext_vector_type(FREG)));
    frag_t fa[2][FM], fb[2][FN];
    uint32_t sca[FM], scb[FN];  // MX: this lane's scale bytes of the current tile, moved into place (see place_scales)
    (void)swz; (void)swz0; (void)swz1; (void)sca; (void)scb;

    auto load_frags = [&](int kt, int s, int buf) {
        const char* st = smem + (kt % STAGES) * STAGE;
        if constexpr (KSTEP == 32) {
            const char* base = st + (((2 * s) ^ swz) << 4);
#pragma unroll
            for (int j = 0; j < FM; j++) fa[buf][j] = *(const frag_t*)(base + a_rowbase + j * 32 * BK);
#pragma unroll
            for (int i = 0; i < FN; i++) fb[buf][i] = *(const frag_t*)(base + b_rowbase + i * 32 * BK);
        } else {
            const char* b0 = st + (((4 * s) ^ swz0) << 4);
            const char* b1 = st + (((4 * s) ^ swz1) << 4);
#pragma unroll
            for (int j = 0; j < FM; j++) {
                const v4i lo = *(const v4i*)(b0 + a_rowbase + j * 32 * BK), hi = *(const v4i*)(b1 + a_rowbase + j * 32 * BK);
                fa[buf][j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int i = 0; i < FN; i++) {
                const v4i lo = *(const v4i*)(b0 + b_rowbase + i * 32 * BK), hi = *(const v4i*)(b1 + b_rowbase + i * 32 * BK);
                fb[buf][i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
        }
    };
    // MX: byte b of a row's scale bytes of a tile covers the tile's K block b (32 elements).  MFMA step s of a lane
    // in K half h multiplies block 2s + h.
    // Four bytes per row and tile (SCW == 1): the dword is shifted right by 8h and the instruction's byte select
    // picks byte 2s.
    // Eight bytes per row and tile (SC16): one 8-byte LDS read brings both dwords (d0, d1) of the tile -- 4-byte reads
    // at the ring's 16-byte row pitch take three times as long as conflict-free ones (measured: 3.75 against 1.31
    // clocks per wave read), so fewer and wider reads -- and one byte permute packs this lane's four scales into one
    // register, [d0.b(h), d1.b(h), d0.b(h+2), d1.b(h+2)]: step s selects byte 2 (s % 2) + s / 2.
    typedef uint32_t raw_t __attribute__((ext_vector_type(SC16 ? 2 : 1)));
    const uint32_t sc_sel = fkc ? 0x07030501u : 0x06020400u;
    (void)sc_sel;
    auto read_scales_raw = [&](int kt, raw_t (&ra)[FM], raw_t (&rb)[FN]) {
        if constexpr (MX) {
            const char* sS;
            int pitch, off;
            if constexpr (SC16) {
                sS = smem + SC_RING + ((kt >> 1) & 1) * ((BM + BN) * 16);
                pitch = 16; off = (kt & 1) * 8;
            } else {
                sS = smem + (kt % STAGES) * STAGE + A_BYTES + B_BYTES;
                pitch = SCB; off = 0;
            }
#pragma unroll
            for (int j = 0; j < FM; j++) ra[j] = *(const raw_t*)(sS + (wm * TM + j * 32 + frow) * pitch + off);
#pragma unroll
            for (int i = 0; i < FN; i++) rb[i] = *(const raw_t*)(sS + (BM + wn * TN + i * 32 + frow) * pitch + off);
        }
    };
    auto place_scales = [&](const raw_t (&ra)[FM], const raw_t (&rb)[FN]) {
        if constexpr (SC16) {
#pragma unroll
            for (int j = 0; j < FM; j++) sca[j] = __builtin_amdgcn_perm(ra[j][1], ra[j][0], sc_sel);
#pragma unroll
            for (int i = 0; i < FN; i++) scb[i] = __builtin_amdgcn_perm(rb[i][1], rb[i][0], sc_sel);
        } else {
#pragma unroll
            for (int j = 0; j < FM; j++) sca[j] = ra[j][0] >> (8 * fkc);
#pragma unroll
            for (int i = 0; i < FN; i++) scb[i] = rb[i][0] >> (8 * fkc);
        }
    };
    auto load_scales = [&](int kt) {   // the scales of tile kt, ready to use
        if constexpr (MX) {
            raw_t ra[FM], rb[FN];
            read_scales_raw(kt, ra, rb);
            place_scales(ra, rb);
        }
    };
    auto mma = [&](int buf, auto sidx) {
        constexpr int S = decltype(sidx)::value;
        (void)S;
#pragma unroll
        for (int i = 0; i < FN; i++)
#pragma unroll
            for (int j = 0; j < FM; j++) {
                if constexpr (MODE == MODE_I8) {
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[buf][i], fa[buf][j], acc[i][j], 0, 0, 0);
                } else if constexpr (MODE == MODE_MXFP4) {
                    const v4i z = {0, 0, 0, 0};  // fp4 operands occupy the first four of the eight operand dwords
                    const v8i bb = __builtin_shufflevector(fb[buf][i], z, 0, 1, 2, 3, 4, 5, 6, 7);
                    const v8i aa = __builtin_shufflevector(fa[buf][j], z, 0, 1, 2, 3, 4, 5, 6, 7);
                    constexpr int SEL = SC16 ? 2 * (S % 2) + S / 2 : 2 * S;
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bb, aa, acc[i][j], 4, 4, SEL, (int)scb[i], SEL, (int)sca[j]);
                } else {
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[buf][i], fa[buf][j], acc[i][j], 0, 0, 2 * S, (int)scb[i], 2 * S, (int)sca[j]);
                }
            }
    };
    auto interleave = [&](bool with_copies) {
        // (FM+FN) groups of {MFMAs, one LDS read (+ async copies)}: memory instructions issue in the MFMA shadow
        constexpr int NCOPY = NA + NB + NSC;
        constexpr int CPG = (NCOPY + FM + FN - 1) / (FM + FN);
#pragma unroll
        for (int g = 0; g < FM + FN; g++) {
            __builtin_amdgcn_sched_group_barrier(0x008, (FM * FN) / (FM + FN), 0);
            __builtin_amdgcn_sched_group_barrier(0x100, KSTEP / 32, 0);
            if (with_copies) __builtin_amdgcn_sched_group_barrier(0x020, CPG, 0);
        }
    };

    // Pipeline.  All STAGES stages are kept in flight.  The loop is rotated so that its single barrier sits in
    // front of the LAST K step of a tile: on entry to iteration kt the operands of K step 0 are already in
    // registers; K steps 0..KS-2 multiply while the operands of the following step are read; then
    //   wait for this thread's copies of tile kt+1, barrier (tile kt+1 is complete in LDS and every wave has
    //   finished reading tile kt, whose last operands now sit in registers),
    //   start the copy of tile kt+STAGES into the freed stage, read K step 0 of tile kt+1, multiply the last step.
#pragma unroll
    for (int i = 0; i < STAGES; i++)
        if (i < KT) {
            if (i % 2 == 0) issue_tile(i, std::true_type{});
            else issue_tile(i, std::false_type{});
        }
    if (KT >= STAGES) wait_vmcnt<(STAGES - 1) * CPT>();
    else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
#if QG_DBG
    const unsigned long long dbg_t1 = wall_clock64();
    const unsigned long long dbg_c1 = clock64();
#endif
    load_frags(0, 0, 0);
    load_scales(0);

    auto k_tile = [&](int kt, auto issue, auto next, auto even) {
        constexpr bool ISSUE = decltype(issue)::value, NEXT = decltype(next)::value;
        raw_t ra[FM], rb[FN];   // raw scale bytes of the next tile on their way in
        (void)ra; (void)rb;
        if constexpr (KS >= 4) {
            load_frags(kt, 1, 1);
            mma(0, std::integral_constant<int, 0>{});
            interleave(false);
            load_frags(kt, 2, 0);
            mma(1, std::integral_constant<int, 1>{});
            interleave(false);
            load_frags(kt, 3, 1);
            mma(0, std::integral_constant<int, 2>{});
            interleave(false);
        } else {
            load_frags(kt, 1, 1);
            mma(0, std::integral_constant<int, 0>{});
            interleave(false);
        }
#if QG_DBG
        wait_lgkmcnt0();
        const unsigned long long c0 = clock64();
#endif
        if constexpr (NEXT) {
            if constexpr (ISSUE) wait_vmcnt<(STAGES - 2) * CPT>();
            else wait_vmcnt<0>();
        }
        wait_lgkmcnt0();  // this wave's reads of the stage about to be recycled have retired
#if QG_DBG
        const unsigned long long c1 = clock64();
#endif
        __builtin_amdgcn_s_barrier();
#if QG_DBG
        const unsigned long long c2 = clock64();
        dbg_vm += c1 - c0; dbg_bar += c2 - c1; dbg_n++;
#endif
        if constexpr (NEXT && MX) {
            // the next tile's scale bytes are requested ahead of its operands (LDS returns in order) and moved
            // into place only after this tile's last MFMAs, which still use the current ones, have been issued
            read_scales_raw(kt + 1, ra, rb);
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (ISSUE) issue_tile(kt + STAGES, even);
        if constexpr (NEXT) load_frags(kt + 1, 0, 0);
        mma(1, std::integral_constant<int, KS - 1>{});
        if constexpr (NEXT) interleave(ISSUE);
        if constexpr (NEXT && MX) {
            __builtin_amdgcn_sched_barrier(0);
            place_scales(ra, rb);
        }
    };
    using T = std::true_type;
    using F = std::false_type;
    int kt = 0;
    if constexpr (SC16) {   // KT is even: tiles go in pairs, the even one also starts the pair's scale copy
        for (; kt + STAGES < KT; kt += 2) {
            k_tile(kt, T{}, T{}, T{});
            k_tile(kt + 1, T{}, T{}, F{});
        }
    } else {
        for (; kt + STAGES < KT; kt++) k_tile(kt, T{}, T{}, F{});
    }
    for (; kt + 1 < KT; kt++) k_tile(kt, F{}, T{}, F{});
    k_tile(kt, F{}, F{}, F{});
    if constexpr (SPLIT) {
        // partial sums straight from the registers (acc[i][j][r]: n = n_base + 8*(r/4) + 4*(lane/32) + r%4, m = m_base + lane%32)
        typedef std::conditional_t<MODE == MODE_I8, v4i, v4f> quad_t;
        typedef std::conditional_t<MODE == MODE_I8, int32_t, float> elem_t;
        elem_t* part = (elem_t*)p.part + (((int64_t)blockIdx.z * gridDim.y + bz) * p.M) * p.N;
        const bool vec_ok4 = (p.N % 4) == 0 && ((uintptr_t)p.part % 16) == 0;
#pragma unroll
        for (int j = 0; j < FM; j++) {
            const int64_t m = m0 + wm * TM + j * 32 + (lane & 31);
#pragma unroll
            for (int i = 0; i < FN; i++) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int64_t n = n0 + wn * TN + i * 32 + 8 * q + 4 * (lane >> 5);
                    if (m >= p.M) continue;
                    const quad_t o = {acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]};
                    if (vec_ok4 && n + 3 < p.N) {
                        *(quad_t*)(part + m * p.N + n) = o;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (n + e < p.N) part[m * p.N + n + e] = o[e];
                    }
                }
            }
        }
        return;
    }
    __syncthreads();  // all operand reads done before LDS is reused below
#if QG_DBG
    const unsigned long long dbg_t2 = wall_clock64();
    const unsigned long long dbg_c2 = clock64();
#endif

    // Epilogue.  acc[i][j][r]: n = n_base + 8*(r/4) + 4*(lane/32) + r%4,  m = m_base + lane%32.
    // Per-row and per-column terms are first widened to fp32 in LDS, so the unrolled part is branch-free:
    // absent terms are the neutral elements 1.0f, 0 and -0.0f.
    float* sS2 = (float*)smem;
    float* sFb = sS2 + BN;
    int32_t* sIb = (int32_t*)(sFb + BN);
    float* sS1 = (float*)(sIb + BN);
    {
        const bool has_ib = MODE == MODE_I8 && p.bias && p.bias_dt == DT_I32;
        const bool has_fb = p.bias && p.bias_dt != DT_I32;
        for (int i = tid; i < BN; i += NT) {
            int64_t n = n0 + i;
            if (n >= p.N) n = p.N - 1;
            if constexpr (MODE == MODE_I8) {
                const int64_t si = p.x2s_len == 1 ? 0 : n;
                float sv = p.x2s_dt == DT_U64 ? u2f((uint32_t)((const uint64_t*)p.x2s)[si]) : load_scalar_as_f32(p.x2s, p.x2s_dt, si);
                if (p.x2s_trunc || p.x2s_dt == DT_U64) sv = u2f(f2u(sv) & 0xFFFFE000u);
                sS2[i] = sv;
                sIb[i] = has_ib ? ((const int32_t*)p.bias)[bz * p.bias_bs + n] : 0;
            }
            sFb[i] = has_fb ? load_scalar_as_f32(p.bias, p.bias_dt, bz * p.bias_bs + n) : -0.0f;
        }
        if constexpr (MODE == MODE_I8) {
            for (int i = tid; i < BM; i += NT) {
                int64_t m = m0 + i;
                if (m >= p.M) m = p.M - 1;
                sS1[i] = p.x1s ? p.x1s[m] : 1.0f;
            }
        }
    }
    if constexpr (OUT_DT == DT_I32 || OUT_DT == DT_I8) {
        // Integer outputs leave straight from the registers: a lane holds four consecutive columns of one row per register
        // quad, 16 bytes (INT32) or 4 bytes (INT8) per store.
        static_assert(MODE == MODE_I8, "integer outputs belong to the int8 mode");
        float* sOff = (float*)smem + 3 * BN + BM;
        const bool has_off = p.x2off != nullptr || p.x2s_dt == DT_U64;
        if (OUT_DT == DT_I8 && has_off) {
            for (int i = tid; i < BN; i += NT) {
                int64_t n = n0 + i;
                if (n >= p.N) n = p.N - 1;
                float off;
                if (p.x2off) off = p.x2off[p.x2off_len == 1 ? 0 : n];
                else {
                    int raw = (int)((((const uint64_t*)p.x2s)[p.x2s_len == 1 ? 0 : n] >> 37) & 0x1FF);
                    off = (float)(raw & 0x100 ? raw - 0x200 : raw);
                }
                const float r = __builtin_rintf(off);
                sOff[i] = r < -256.0f ? -256.0f : (r > 255.0f ? 255.0f : r);
            }
        }
        __syncthreads();
        const bool vec_ok = (p.ldc % 4) == 0 && ((uintptr_t)p.out % 16) == 0;
#pragma unroll
        for (int j = 0; j < FM; j++) {
            const int64_t m = m0 + wm * TM + j * 32 + frow;
#pragma unroll
            for (int i = 0; i < FN; i++) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int nl = wn * TN + i * 32 + 8 * q + 4 * fkc;
                    const int64_t n = n0 + nl;
                    const v4i ib = *(const v4i*)(sIb + nl);
                    v4i o;
                    if constexpr (OUT_DT == DT_I32) {
#pragma unroll
                        for (int e = 0; e < 4; e++) o[e] = acc[i][j][q * 4 + e] + ib[e];
                        if (m < p.M) {
                            int32_t* dst = (int32_t*)p.out + (bz * p.M + m) * p.ldc + n;
                            if (vec_ok && n + 3 < p.N) *(v4i*)dst = o;
                            else {
#pragma unroll
                                for (int e = 0; e < 4; e++)
                                    if (n + e < p.N) dst[e] = o[e];
                            }
                        }
                    } else {
                        const v4f s2 = *(const v4f*)(sS2 + nl);
                        uint32_t packed = 0;
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            float t = __builtin_rintf((float)(acc[i][j][q * 4 + e] + ib[e]) * s2[e]);
                            t = t < -256.0f ? -256.0f : (t > 255.0f ? 255.0f : t);
                            if (has_off) t = t + sOff[nl + e];
                            t = t < -128.0f ? -128.0f : (t > 127.0f ? 127.0f : t);
                            o[e] = (int)t;
                            packed |= ((uint32_t)o[e] & 0xffu) << (8 * e);
                        }
                        if (m < p.M) {
                            int8_t* dst = (int8_t*)p.out + (bz * p.M + m) * p.ldc + n;
                            if (vec_ok && n + 3 < p.N) *(uint32_t*)dst = packed;
                            else {
#pragma unroll
                                for (int e = 0; e < 4; e++)
                                    if (n + e < p.N) dst[e] = (int8_t)o[e];
                            }
                        }
                    }
                }
            }
        }
        return;
    }
    if constexpr (OUT_DT == DT_F32) {
        // FLOAT output (the MX modes): like the integer outputs, straight from the registers, 16 bytes per lane
        static_assert(MODE != MODE_I8, "the int8 mode has no FLOAT output here");
        __syncthreads();
        const bool vec_ok = (p.ldc % 4) == 0 && ((uintptr_t)p.out % 16) == 0;
#pragma unroll
        for (int j = 0; j < FM; j++) {
            const int64_t m = m0 + wm * TM + j * 32 + frow;
#pragma unroll
            for (int i = 0; i < FN; i++) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int nl = wn * TN + i * 32 + 8 * q + 4 * fkc;
                    const int64_t n = n0 + nl;
                    const v4f fbv = *(const v4f*)(sFb + nl);
                    v4f v;
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = acc[i][j][q * 4 + e] + fbv[e];
                    if (m < p.M) {
                        float* dst = (float*)p.out + (bz * p.M + m) * p.ldc + n;
                        if (vec_ok && n + 3 < p.N) *(v4f*)dst = v;
                        else {
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                if (n + e < p.N) dst[e] = v[e];
                        }
                    }
                }
            }
        }
        return;
    }
    __syncthreads();
    uint16_t* out = (uint16_t*)p.out + bz * p.M * p.ldc;
    // Results leave through LDS: a lane holds 4 consecutive columns of one row per register quad, which would make
    // every store instruction touch 32 rows with 16 bytes each.  Instead each wave parks one 32-row block of its
    // sub-tile in a private LDS patch (row pitch TN*2+16 bytes) and reads it back row-wise, so that a store
    // instruction writes whole 128-byte lines (16 bytes per lane, TN/8 lanes per row).
    typedef v4us __attribute__((may_alias)) v4us_a;   // the patch is written as 16-bit quads and read as dword quads
    typedef v4i __attribute__((may_alias)) v4i_a;
    constexpr int EP_PITCH = TN * 2 + 16;
    constexpr int EP_BYTES = 32 * EP_PITCH;
    constexpr int EP_BASE = (3 * BN + BM) * 4;
    static_assert(EP_BASE + WGM * WGN * EP_BYTES <= STAGES * STAGE, "epilogue staging fits in the operand stages");
    char* ep = smem + EP_BASE + wave * EP_BYTES;
    constexpr int LPR = TN / 8;          // lanes per row when every lane moves 16 bytes
    constexpr int RPI2 = 64 / LPR;       // rows per store instruction
    const int er = lane / LPR, ec = lane % LPR;
    const bool vec_ok = (p.ldc % 8) == 0 && ((uintptr_t)p.out % 16) == 0;
#pragma unroll
    for (int j = 0; j < FM; j++) {
        const int ml = wm * TM + j * 32 + frow;
        float s1 = 1.0f;
        if constexpr (MODE == MODE_I8) s1 = sS1[ml];
#pragma unroll
        for (int i = 0; i < FN; i++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int nw = i * 32 + 8 * q + 4 * fkc;   // column inside the wave's sub-tile
                const int nl = wn * TN + nw;
                const v4f fbv = *(const v4f*)(sFb + nl);
                v4f v;
                if constexpr (MODE == MODE_I8) {
                    const v4f s2 = *(const v4f*)(sS2 + nl);
                    const v4i ib = *(const v4i*)(sIb + nl);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        float tv = (float)(acc[i][j][q * 4 + e] + ib[e]);
                        tv = tv * s2[e];
                        tv = tv * s1;
                        v[e] = tv + fbv[e];
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = acc[i][j][q * 4 + e] + fbv[e];
                }
                *(v4us_a*)(ep + frow * EP_PITCH + nw * 2) = pack4_b16<OUT_DT>(v);
            }
        }
        // this wave's 32 x TN block is complete in its patch (LDS operations of one wave complete in order)
#pragma unroll
        for (int r = 0; r < 32 / RPI2; r++) {
            const int row = r * RPI2 + er;
            const v4i o = *(const v4i_a*)(ep + row * EP_PITCH + ec * 16);
            const int64_t m = m0 + wm * TM + j * 32 + row;
            const int64_t n = n0 + wn * TN + ec * 8;
            if (m < p.M) {
                if (vec_ok && n + 7 < p.N) {
                    *(v4i*)(out + m * p.ldc + n) = o;
                } else {
                    const uint16_t* oe = (const uint16_t*)&o;
#pragma unroll
                    for (int e = 0; e < 8; e++)
                        if (n + e < p.N) out[m * p.ldc + n + e] = oe[e];
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
            unsigned long long* d = p.dbg + ((size_t)blockIdx.x * (WGM * WGN) + wave) * 16;
            d[0] = dbg_t0; d[1] = dbg_t1; d[2] = dbg_t2; d[3] = dbg_t3; d[4] = dbg_t4; d[5] = dbg_vm; d[6] = dbg_bar; d[7] = dbg_n; d[8] = dbg_c2 - dbg_c1;
        }
    }
#endif
}

// MODE_I8 after a K split: out[b, m, n] = rounded(fp32(sum of the partial sums + ib[n]) * x2s[n] * x1s[m] + fb[n]), the
// terms as the tile kernel's epilogue stages them
template <int OUT_DT>
__global__ __launch_bounds__(256) void qg_i8_splitk_reduce_kernel(QgemmParams p, int64_t total)
{
    const int64_t MN = p.M * p.N, stride = (int64_t)gridDim.x * blockDim.x;
    const bool has_ib = p.bias && p.bias_dt == DT_I32, has_fb = p.bias && p.bias_dt != DT_I32;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int32_t a = splitk_sum(p.part, p.splits, total, i);
        const int64_t bz = i / MN, m = (i % MN) / p.N, n = i % p.N;
        const int64_t si = p.x2s_len == 1 ? 0 : n;
        float sv = p.x2s_dt == DT_U64 ? u2f((uint32_t)((const uint64_t*)p.x2s)[si]) : load_scalar_as_f32(p.x2s, p.x2s_dt, si);
        if (p.x2s_trunc || p.x2s_dt == DT_U64) sv = u2f(f2u(sv) & 0xFFFFE000u);
        const int32_t ib = has_ib ? ((const int32_t*)p.bias)[bz * p.bias_bs + n] : 0;
        const float fb = has_fb ? load_scalar_as_f32(p.bias, p.bias_dt, bz * p.bias_bs + n) : -0.0f;
        const float s1 = p.x1s ? p.x1s[m] : 1.0f;
        float tv = (float)(a + ib);
        tv = tv * sv;
        tv = tv * s1;
        const float v = tv + fb;
        ((uint16_t*)p.out)[(bz * p.M + m) * p.ldc + n] = OUT_DT == DT_BF16 ? bf16_bits(v) : f16_bits(v);
    }
}

// The MX modes after a K split: out[b, m, n] = rounded(sum of the fp32 partial sums, in split order, + bias[n])
template <int OUT_DT>
__global__ __launch_bounds__(256) void qg_mx_splitk_reduce_kernel(QgemmParams p, int64_t total)
{
    const int64_t MN = p.M * p.N, stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        float v = splitk_sum((const float*)p.part, p.splits, total, i);
        const int64_t bz = i / MN, m = (i % MN) / p.N, n = i % p.N;
        if (p.bias) v = v + load_scalar_as_f32(p.bias, p.bias_dt, bz * p.bias_bs + n);
        const int64_t o = (bz * p.M + m) * p.ldc + n;
        if constexpr (OUT_DT == DT_F32) ((float*)p.out)[o] = v;
        else ((uint16_t*)p.out)[o] = OUT_DT == DT_BF16 ? bf16_bits(v) : f16_bits(v);
    }
}

// The K split of an MX mode (p.splits > 1, whole K tiles, no gate): the tile kernel per split, then the reduction.
template <int MODE, int BM, int BN, int BK, int WGM, int WGN, int STAGES, int MINWG>
static int qgemm_launch_split_mx(const QgemmParams& p, int64_t batch, int out_dt, hipStream_t st)
{
    static_assert(MODE != MODE_I8, "the MX modes");
    constexpr int SCB = BK / (MODE == MODE_MXFP8 ? 32 : 16);
    constexpr int U = SCB == 8 ? 2 : 1;
    if (!p.part || p.splits < 2 || p.gate || (p.KB % (BK * U)) != 0 || p.splits > p.KB / BK / U / 2) return -1;
    int tiles_m = (int)((p.M + BM - 1) / BM), tiles_n = (int)((p.N + BN - 1) / BN);
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)batch, (unsigned)p.splits);
    const size_t lds = SCB == 8 ? (size_t)STAGES * (BM + BN) * BK + 2 * (BM + BN) * 16 : (size_t)STAGES * ((BM + BN) * BK + (BM + BN) * SCB);
    auto k = qgemm_kernel<MODE, BM, BN, BK, WGM, WGN, STAGES, MINWG, false, DT_F32, true>;
    static std::atomic<uint64_t> attr_set{0};
    if (!device_flag_test(attr_set)) {
        hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        device_flag_set(attr_set);
    }
    hipLaunchKernelGGL(k, grid, dim3(WGM * WGN * 64), lds, st, p, tiles_m, tiles_n);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    const int64_t total = batch * p.M * p.N;
    const unsigned rgrid = splitk_reduce_grid(total);
    if (out_dt == DT_BF16) hipLaunchKernelGGL(qg_mx_splitk_reduce_kernel<DT_BF16>, dim3(rgrid), dim3(256), 0, st, p, total);
    else if (out_dt == DT_F16) hipLaunchKernelGGL(qg_mx_splitk_reduce_kernel<DT_F16>, dim3(rgrid), dim3(256), 0, st, p, total);
    else if (out_dt == DT_F32) hipLaunchKernelGGL(qg_mx_splitk_reduce_kernel<DT_F32>, dim3(rgrid), dim3(256), 0, st, p, total);
    else return -2;
    return (int)hipGetLastError();
}

// The K split of MODE_I8 (p.splits > 1, K a multiple of BK): the tile kernel per split, then the reduction.
template <int BM, int BN, int BK, int WGM, int WGN, int STAGES, int MINWG>
static int qgemm_launch_split_i8(const QgemmParams& p, int64_t batch, int out_dt, hipStream_t st)
{
    if (!p.part || p.splits < 2 || (p.KB % BK) != 0 || p.splits > p.KB / BK / 2) return -1;
    if (out_dt != DT_BF16 && out_dt != DT_F16) return -2;
    int tiles_m = (int)((p.M + BM - 1) / BM), tiles_n = (int)((p.N + BN - 1) / BN);
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)batch, (unsigned)p.splits);
    const size_t lds = (size_t)STAGES * (BM + BN) * BK;
    auto k = qgemm_kernel<MODE_I8, BM, BN, BK, WGM, WGN, STAGES, MINWG, false, DT_I32, true>;
    static std::atomic<uint64_t> attr_set{0};
    if (!device_flag_test(attr_set)) {
        hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        device_flag_set(attr_set);
    }
    hipLaunchKernelGGL(k, grid, dim3(WGM * WGN * 64), lds, st, p, tiles_m, tiles_n);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    const int64_t total = batch * p.M * p.N;
    const unsigned rgrid = splitk_reduce_grid(total);
    if (out_dt == DT_BF16) hipLaunchKernelGGL(qg_i8_splitk_reduce_kernel<DT_BF16>, dim3(rgrid), dim3(256), 0, st, p, total);
    else hipLaunchKernelGGL(qg_i8_splitk_reduce_kernel<DT_F16>, dim3(rgrid), dim3(256), 0, st, p, total);
    return (int)hipGetLastError();
}

template <int MODE, int BM, int BN, int BK, int WGM, int WGN, int STAGES, int MINWG, bool KTAIL, int OUT_DT>
static int qgemm_launch_one(const QgemmParams& p, int64_t batch, hipStream_t st)
{
    constexpr bool MX = MODE != MODE_I8;
    int tiles_m = (int)((p.M + BM - 1) / BM), tiles_n = (int)((p.N + BN - 1) / BN);
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)batch);
    constexpr int SCB = MX ? BK / (MODE == MODE_MXFP8 ? 32 : 16) : 0;   // scale bytes per row per tile
    size_t lds = SCB == 8 ? (size_t)STAGES * (BM + BN) * BK + 2 * (BM + BN) * 16   // scales in their own ring of two slots
                          : (size_t)STAGES * ((BM + BN) * BK + (BM + BN) * SCB);
    auto k = qgemm_kernel<MODE, BM, BN, BK, WGM, WGN, STAGES, MINWG, KTAIL, OUT_DT>;
    static std::atomic<uint64_t> attr_set{0};   // one bit per device: the attribute belongs to the (kernel, device) pair
    if (!device_flag_test(attr_set)) {
        hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        device_flag_set(attr_set);
    }
    hipLaunchKernelGGL(k, grid, dim3(WGM * WGN * 64), lds, st, p, tiles_m, tiles_n);
    return (int)hipGetLastError();
}

// Picks the K-tail and output-type instantiation.
template <int MODE, int BM, int BN, int BK, int WGM, int WGN, int STAGES, int MINWG>
static int qgemm_launch(const QgemmParams& p, int64_t batch, int out_dt, hipStream_t st)
{
    const bool bf = out_dt == DT_BF16;
    if constexpr (MODE == MODE_I8) {
        if (out_dt == DT_I32 || out_dt == DT_I8) return -2;   // qgemm_launch_int
        if ((p.KB % BK) != 0) {
            return bf ? qgemm_launch_one<MODE, BM, BN, BK, WGM, WGN, STAGES, MINWG, true, DT_BF16>(p, batch, st)
                      : qgemm_launch_one<MODE, BM, BN, BK, WGM, WGN, STAGES, MINWG, true, DT_F16>(p, batch, st);
        }
    }
    if constexpr (MODE != MODE_I8) {
        if (out_dt == DT_F32) return qgemm_launch_one<MODE, BM, BN, BK, WGM, WGN, STAGES, MINWG, false, DT_F32>(p, batch, st);
    }
    return bf ? qgemm_launch_one<MODE, BM, BN, BK, WGM, WGN, STAGES, MINWG, false, DT_BF16>(p, batch, st)
              : qgemm_launch_one<MODE, BM, BN, BK, WGM, WGN, STAGES, MINWG, false, DT_F16>(p, batch, st);
}

// MODE_I8 with an INT32 or INT8 output (instantiated only for the tile shapes the int8 launcher uses for them).
template <int BM, int BN, int BK, int WGM, int WGN, int STAGES, int MINWG>
static int qgemm_launch_int(const QgemmParams& p, int64_t batch, int out_dt, hipStream_t st)
{
    const bool tail = (p.KB % BK) != 0;
    if (out_dt == DT_I32)
        return tail ? qgemm_launch_one<MODE_I8, BM, BN, BK, WGM, WGN, STAGES, MINWG, true, DT_I32>(p, batch, st)
                    : qgemm_launch_one<MODE_I8, BM, BN, BK, WGM, WGN, STAGES, MINWG, false, DT_I32>(p, batch, st);
    if (out_dt == DT_I8)
        return tail ? qgemm_launch_one<MODE_I8, BM, BN, BK, WGM, WGN, STAGES, MINWG, true, DT_I8>(p, batch, st)
                    : qgemm_launch_one<MODE_I8, BM, BN, BK, WGM, WGN, STAGES, MINWG, false, DT_I8>(p, batch, st);
    return -2;
}

}  // namespace opsnn
