// int8 x int8 (and fp8 e4m3 x e4m3) tile kernel with one wave per SIMD and a 256 x (32*FN) output tile, FN = 8..11.
//
// Why a second int8 tile kernel: a GEMM runs in rounds of one tile per CU, and with a fixed 256 x 256 tile a shape
// such as 2048 x 11008 needs 1.34 rounds -- the last third of a round costs a whole one (or a second launch of small
// tiles with its own prologue, epilogue and launch gap).  Here the tile WIDTH is a template parameter in steps of 32
// columns, and the launcher picks the width whose tile count fills whole rounds: 11008 columns = 32 tiles of 352, times
// 8 row tiles = 256 tiles = one round of 256 CUs.
//
// What makes a 256 x 352 tile possible is the register file: 256 x 352 int32 sums are 352 KB of the CU's 512 KB.  So the
// workgroup is FOUR waves, one per SIMD, each with the SIMD's whole register file (512 registers per lane): a wave owns
// 128 x (16*FN) outputs as 8 x FN fragments of 16 x 16 (v_mfma_i32_16x16x64_i8, two per 128-byte K tile and fragment
// pair), i.e. up to 352 accumulator registers, 64 registers of x1 fragments held for the whole K tile, and the x2
// fragments streaming through two sets of 8, each requested one fragment (16 MFMAs = 256 clocks) ahead.  A wave reads
// (8 + FN) fragments from LDS for 16 * FN MFMAs -- less than half the LDS traffic per MFMA of the 8-wave kernels.
//
// With one wave per SIMD there is no partner wave to fill in while this one waits, so nothing may wait:
//   - the loop is software-pipelined: the barrier sits in front of the last x2 fragment of a tile, and in the shadow of
//     that fragment's 16 MFMAs the wave requests the next tile's first x2 fragment and its x1 fragments, each half of
//     a fragment as soon as the last MFMA that reads the old half has been issued; the next tile then starts on the
//     halves that came first (lgkmcnt counts, never "wait for everything"; the fp8 forms read whole fragments per
//     instruction and do wait for all of them at the start of a tile);
//   - the global -> LDS copies are written as inline assembly, because of what the compiler does with the builtin (see
//     dma_copy16), and are spread over the first fragments of the tile instead of being issued in one burst;
//   - two stages of (256 + 32*FN) x 128 bytes fill the LDS (155,648 of 163,840 bytes at FN = 11): the copies of tile
//     kt+1 are issued during tile kt into the stage that the barrier at the end of tile kt-1 freed, and are waited
//     for in front of the barrier at the end of tile kt.
// Measured on 2048 x 4096 x 11008 (bf16 out): 90-92 us against 103 us for 256 x 256 tiles on 8192 columns plus a second
// launch of 128 x 128 tiles on the remaining 2816; at 256 x 256 (FN = 8) it is level with the 8-wave kernel
// (62-64 against 65 us on 2048 x 4096 x 8192, 540 against 560 us on 8192^3).
//
// F8 = true: the same kernel on fp8 e4m3 operands for the modes with one scale per row and per column (K-C, K-T,
// separately multiplied double scale): one v_mfma_f32_16x16x128_f8f6f4 per fragment pair and K tile instead of two
// int8 instructions, float sums, and the same epilogue without the integer bias.
//
// MXS = true (with F8): MXFP8.  A K tile needs four e8m0 bytes per row; one 16-byte copy per row brings the scales of
// FOUR tiles into one of two slots behind the operand stages (a 4-byte copy per row and tile costs a cache-line request
// for four useful bytes -- as many requests as the operands themselves, and the kernel ran no faster than the 8-wave
// one).  Each lane reads the dword of its row with its fragment and shifts its own block's byte down (lane group q
// supplies the scale of block q, see qmm_fp8_block.hip), and the scaled form of the instruction applies them.  Needs
// K % 512 == 0, 16-byte aligned scale rows and FN <= 9 (the slots must fit into LDS).
//
// Epilogue formula and its order of operations: the K-C / K-T golden, as in qgemm_core.hip.h
// (matmul/quant_batch_matmul_v3/tests/assets/qbmmv3_kernel_golden.py): out = cast(fp32(acc + ib[n]) * x2s[n] * x1s[m] + fb[n]).
#include "launch.h"
#include "qgemm_core.hip.h"

namespace opsnn {

// acc += a (16 x 64 int8, rows = output columns) x b (64 x 16 int8), with the accumulator pinned to one register class.
// The wave's sums outnumber the 256 accumulation registers; left to itself the compiler puts all of them in that class
// and copies the overflow in and out around every instruction (244 copies per K tile at FN = 11).  Written out, the
// first 64 fragments live in accumulation registers and the rest in ordinary vector registers, and nothing moves.
// (The compiler does not see an MFMA here: dependent instructions are kept eight apart by the loop order, and the
// epilogue waits out the write-to-read hazard itself.)
template <bool AG>
__device__ __forceinline__ void mfma_i8_16x16x64(v4i& c, const v4i a, const v4i b)
{
    if constexpr (AG) asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    else asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}

// acc += a (16 x 128 fp8 e4m3) x b (128 x 16 fp8 e4m3), fp32 sums; see mfma_i8_16x16x64 for the register classes
template <bool AG>
__device__ __forceinline__ void mfma_f8_16x16x128(v4f& c, const v8i a, const v8i b)
{
    if constexpr (AG) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    else asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}

// the scaled form: sa / sb hold, in their low byte, the e8m0 scale of this lane's 32-element block of a / b
template <bool AG>
__device__ __forceinline__ void mfma_f8_16x16x128_scaled(v4f& c, const v8i a, const v8i b, uint32_t sa, uint32_t sb)
{
    if constexpr (AG) asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0]" : "+a"(c) : "v"(a), "v"(b), "v"(sa), "v"(sb));
    else asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0]" : "+v"(c) : "v"(a), "v"(b), "v"(sa), "v"(sb));
}

// 16-byte asynchronous copy global -> LDS, written out: lane l reads sbase + voff(l) and lands at lds_base + LDS_IMM + 16*l.
// Through the builtin the compiler's wait-count pass sees an instruction that touches both memory paths and from then
// on answers every dependency on an LDS read with a wait for ALL outstanding reads, including the ones issued a moment
// ago for the next fragment; hidden from it, the pass counts exactly.  The copies' own completion is waited for
// explicitly (vmcnt + barrier) wherever LDS is read.
template <int LDS_IMM>
__device__ __forceinline__ void dma_copy16(const int8_t* sbase, uint32_t voff, uint32_t lds_base)
{
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 : : "s"(lds_base), "v"(voff), "s"(sbase), "n"(LDS_IMM) : "memory", "m0", "scc");
}

// the same copy with a 64-bit address per lane
template <int LDS_IMM>
__device__ __forceinline__ void dma_copy16v(const void* g, uint32_t lds_base)
{
    asm volatile("s_add_u32 m0, %0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_base), "v"(g), "n"(LDS_IMM) : "memory", "m0", "scc");
}

template <int FN, int OUT_DT, bool F8 = false, bool MXS = false>
__global__ __launch_bounds__(256, 1) void qgemm_i8_wide_kernel(QgemmParams p, int tiles_m, int tiles_n)
{
    static_assert(!MXS || F8, "block scales ride on the fp8 form");
    constexpr int SLOTS = F8 ? 8 : 16;   // MFMAs per x2 fragment
    constexpr int NT = 256, BM = 256, TM = 128, FM = TM / 16, TN = 16 * FN, BN = 2 * TN, BK = 128, STAGES = 2;
    constexpr int CPR = BK / 16, RPW = 16 / CPR;
    constexpr int NSC = MXS ? (BM + BN + NT - 1) / NT : 0;   // scale copies per thread and four K tiles: 16 bytes per tile row
    constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK, STAGE = A_BYTES + B_BYTES;
    constexpr int SC_RING = 2 * STAGE, SC_SLOT = NSC * NT * 16;   // two scale slots behind the operand stages
    static_assert(SC_RING + 2 * SC_SLOT <= 163840, "operand stages and scale slots must fit into LDS");
    constexpr int RPI = NT / CPR;                 // 32 tile rows per copy instruction of the workgroup
    constexpr int NA = BM / RPI, NB = BN / RPI;   // 8 and FN
    constexpr int CPT = NA + NB;
    static_assert(FN >= 2 && STAGES * CPT < 64, "copy counts must fit the wait counter");
    extern __shared__ __attribute__((aligned(16))) char smem[];

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
    const int KT = (int)(p.KB / BK);

    // Copies: instruction i of the workgroup fills LDS chunks [i*NT, (i+1)*NT) of an operand, i.e. tile rows
    // 32i .. 32i+31; this thread moves chunk (tid % 8) ^ key of row 32i + tid/8.  Rows past the matrix edge repeat the
    // last valid row: they only feed outputs that are never stored.
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
    auto scalar_ptr = [](const int8_t* q) -> const int8_t* {   // a wave-uniform pointer, held in scalar registers
        const uint64_t u = (uint64_t)q;
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u), hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
        return (const int8_t*)(((uint64_t)hi << 32) | lo);
    };
    const uint32_t lds_raw = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem);
    const uint32_t lds0 = lds_raw + wave * 1024;
    // MXFP8: scale copy `c` of this thread moves 16 scale bytes (four K tiles) of tile row c*NT + tid (x1 rows, then x2
    // rows; rows past the tile repeat its last one into padding that nobody reads)
    const uint8_t* sc_src[NSC > 0 ? NSC : 1];
    if constexpr (MXS) {
#pragma unroll
        for (int c = 0; c < NSC; c++) {
            const int r = c * NT + tid;
            if (r < BM) {
                const int rr = r < a_rows ? r : a_rows - 1;
                sc_src[c] = p.sa + bz * p.sa_bs + (m0 + rr) * p.sa_rs;
            } else {
                int rr = r - BM;
                rr = rr < b_rows ? rr : b_rows - 1;
                sc_src[c] = p.sb + bz * p.sb_bs + (n0 + rr) * p.sb_rs;
            }
        }
    }
    auto issue_piece = [&](int kt, int stage, auto idx_c) {
        constexpr int idx = decltype(idx_c)::value;
        const uint32_t sS = lds0 + stage * STAGE;
        if constexpr (idx < NA) dma_copy16<idx * NT * 16>(scalar_ptr(A + (int64_t)kt * BK), a_off[idx], sS);
        else dma_copy16<A_BYTES + (idx - NA) * NT * 16>(scalar_ptr(B + (int64_t)kt * BK), b_off[idx - NA], sS);
    };
    auto issue_scales = [&](int group) {   // the scales of K tiles 4*group .. 4*group+3 into slot group % 2
        if constexpr (MXS) {
            const uint32_t slot = lds0 + SC_RING + (group & 1) * SC_SLOT;
            [&]<int... C>(std::integer_sequence<int, C...>) {
                (dma_copy16v<C * NT * 16>(sc_src[C] + (int64_t)group * 16, slot), ...);
            }(std::make_integer_sequence<int, NSC>{});
        }
    };
    auto for_copies = [&](auto&& f) {   // f(integral_constant<int, c>) for c = 0 .. CPT-1
        [&]<int... C>(std::integer_sequence<int, C...>) { (f(std::integral_constant<int, C>{}), ...); }(std::make_integer_sequence<int, CPT>{});
    };
    auto issue_tile = [&](int kt) {
        for_copies([&](auto c) { issue_piece(kt, kt % STAGES, c); });
    };

    using acc_t = std::conditional_t<F8, v4f, v4i>;
    acc_t acc[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; i++)
#pragma unroll
        for (int j = 0; j < FM; j++) acc[i][j] = acc_t{0, 0, 0, 0};

    // Operand fragment of the 16x16x64 instruction pair, lane (row = lane%16, q = lane/16): bytes [16q, 16q+16) of the
    // row's 128 bytes of K for the first instruction, [64+16q, +16) for the second.  (K is the contraction index: any
    // assignment of K to lanes is right as long as both operands use the same one.)
    const int frow = lane & 15, fq = lane >> 4;
    const int key = (frow / RPW) & (CPR - 1);
    const int ch0 = (fq ^ key) << 4, ch1 = ((4 + fq) ^ key) << 4;
    const int a_rowbase = (wm * TM + frow) * BK;
    const int b_rowbase = A_BYTES + (wn * TN + frow) * BK;
    auto load_lo = [&](const char* st, int rowbase) -> v4i { return *(const v4i*)(st + rowbase + ch0); };
    auto load_hi = [&](const char* st, int rowbase) -> v4i { return *(const v4i*)(st + rowbase + ch1); };

    // The copies of tile kt+1 are issued evenly over the first SPREAD fragments of tile kt (into the stage that the
    // barrier at the end of tile kt-1 freed) and are waited for at the end of tile kt.  Issued in one burst they fill
    // the memory pipeline's queue and the wave -- the only one on its SIMD -- stalls in front of its MFMAs:
    // measured 102.6 us (burst behind the last fragment) against 90.4 us (spread) for 2048 x 4096 x 11008.
    constexpr int SPREAD = 4;
    static_assert(SPREAD <= FN, "the copies are issued within one tile");
    issue_tile(0);
    issue_scales(0);
    wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    // Fragments are kept as halves (lo: the first instruction's 64 bytes of K, hi: the second's), so that a half can be
    // replaced as soon as its last reader has been issued.
    // The x2 fragments alternate between fb[0] and fb[1]; fragment 0 of the NEXT tile is requested into fb[FN % 2].  For
    // odd FN that is fb[1], and the tile starts by moving it to fb[0] (eight register moves per K tile).
    v4i fal[FM], fah[FM], fbl[2], fbh[2];
    fbl[FN & 1] = load_lo(smem, b_rowbase);
    fbh[FN & 1] = load_hi(smem, b_rowbase);
#pragma unroll
    for (int j = 0; j < FM; j++) fal[j] = load_lo(smem, a_rowbase + j * 16 * BK);
#pragma unroll
    for (int j = 0; j < FM; j++) fah[j] = load_hi(smem, a_rowbase + j * 16 * BK);
    // MXFP8: the scale dword of this lane's row in each x1 fragment (raw, then shifted to this lane's block) and in the
    // x2 fragments (alternating like fb)
    uint32_t sar[FM], sca[FM], sbr[2];
    (void)sar; (void)sca; (void)sbr;
    // the scale dword of K tile kt for tile row r: slot (kt / 4) % 2, 16 bytes per row, dword kt % 4
    auto scale_base = [&](int kt) -> const char* { return smem + SC_RING + ((kt >> 2) & 1) * SC_SLOT + (kt & 3) * 4; };
    auto a_scale = [&](const char* sb, int j) -> uint32_t { return *(const uint32_t*)(sb + (wm * TM + j * 16 + frow) * 16); };
    auto b_scale = [&](const char* sb, int i) -> uint32_t { return *(const uint32_t*)(sb + (BM + wn * TN + i * 16 + frow) * 16); };
    if constexpr (MXS) {
        sbr[FN & 1] = b_scale(scale_base(0), 0);
#pragma unroll
        for (int j = 0; j < FM; j++) sar[j] = a_scale(scale_base(0), j);
    }

    for (int kt = 0; kt < KT; kt++) {
        const char* st = smem + (kt & 1) * STAGE;
        const char* stn = smem + ((kt + 1) & 1) * STAGE;
        // past the end the copies repeat the last tile (into a stage nobody reads any more): no branches in the loop
        const int ktc = kt + 1 < KT ? kt + 1 : KT - 1;
        const int cstage = (kt + 1) & 1;
        auto spread_copies = [&](int slot) {   // slot = index within the tile of the MFMA just issued
            for_copies([&](auto c) {
                if ((decltype(c)::value * SPREAD * SLOTS) / CPT == slot) issue_piece(ktc, cstage, c);
            });
        };
        if constexpr (F8) {
#pragma unroll
            for (int i = 0; i < FN; i++) {
                if (i + 1 < FN) {
                    if (i == 0) {   // one instruction reads both halves of a fragment: everything requested so far is needed now
                        wait_lgkmcnt0();
                        if (FN & 1) {
                            fbl[0] = fbl[1]; fbh[0] = fbh[1];
                            if constexpr (MXS) sbr[0] = sbr[1];
                        }
                        if constexpr (MXS) {
#pragma unroll
                            for (int j = 0; j < FM; j++) sca[j] = sar[j] >> (8 * fq);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    fbl[(i + 1) & 1] = load_lo(st, b_rowbase + (i + 1) * 16 * BK);
                    fbh[(i + 1) & 1] = load_hi(st, b_rowbase + (i + 1) * 16 * BK);
                    if constexpr (MXS) sbr[(i + 1) & 1] = b_scale(scale_base(kt), i + 1);
                    __builtin_amdgcn_sched_barrier(0);
                    if (i > 0) __builtin_amdgcn_s_waitcnt(0xc07f | ((MXS ? 3 : 2) << 8));   // all but the reads just issued
                } else {
                    wait_vmcnt<0>();
                    wait_lgkmcnt0();
                    __builtin_amdgcn_s_barrier();
                    __builtin_amdgcn_sched_barrier(0);
                    fbl[(i + 1) & 1] = load_lo(stn, b_rowbase);
                    fbh[(i + 1) & 1] = load_hi(stn, b_rowbase);
                    if constexpr (MXS) sbr[(i + 1) & 1] = b_scale(scale_base(kt + 1), 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                const v8i b8 = __builtin_shufflevector(fbl[i & 1], fbh[i & 1], 0, 1, 2, 3, 4, 5, 6, 7);
                uint32_t scb = 0;
                if constexpr (MXS) {
                    scb = sbr[i & 1] >> (8 * fq);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int j = 0; j < FM; j++) {
                    const v8i a8 = __builtin_shufflevector(fal[j], fah[j], 0, 1, 2, 3, 4, 5, 6, 7);
                    if constexpr (MXS) {
                        if (i * FM + j < 64) mfma_f8_16x16x128_scaled<true>(acc[i][j], b8, a8, scb, sca[j]);
                        else mfma_f8_16x16x128_scaled<false>(acc[i][j], b8, a8, scb, sca[j]);
                    } else if constexpr (F8) {   // (the int8 instantiation never compiles this call)
                        if (i * FM + j < 64) mfma_f8_16x16x128<true>(acc[i][j], b8, a8);
                        else mfma_f8_16x16x128<false>(acc[i][j], b8, a8);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    spread_copies(i * SLOTS + j);
                    if constexpr (MXS) {
                        // first tile of a group of four: fetch the next group's scales, if there is one (its slot's last
                        // reader was the tile before this one)
                        if (i == SPREAD && j == 0 && (kt & 3) == 0 && kt + 4 < KT) issue_scales((kt >> 2) + 1);
                    }
                    if (i == FN - 1) {
                        fal[j] = load_lo(stn, a_rowbase + j * 16 * BK);
                        fah[j] = load_hi(stn, a_rowbase + j * 16 * BK);
                        if constexpr (MXS) sar[j] = a_scale(scale_base(kt + 1), j);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        } else {
#pragma unroll
        for (int i = 0; i < FN; i++) {
            if (i + 1 < FN) {
                if (i == 0) {
                    // Outstanding, oldest first: this tile's first x2 fragment, the lo halves of its x1 fragments, their hi
                    // halves.  The first eight instructions need all but the hi halves.
                    __builtin_amdgcn_s_waitcnt(0xc07f | (FM << 8));
                    if (FN & 1) { fbl[0] = fbl[1]; fbh[0] = fbh[1]; }
                    __builtin_amdgcn_sched_barrier(0);
                }
                fbl[(i + 1) & 1] = load_lo(st, b_rowbase + (i + 1) * 16 * BK);
                fbh[(i + 1) & 1] = load_hi(st, b_rowbase + (i + 1) * 16 * BK);
                __builtin_amdgcn_sched_barrier(0);
                if (i > 0) __builtin_amdgcn_s_waitcnt(0xc07f | (2 << 8));   // lgkmcnt: all but the two reads just issued
            } else {
                // every read of tile kt by this wave has been issued; its own copies of tile kt+1 must have landed
                wait_vmcnt<0>();
                wait_lgkmcnt0();
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
                fbl[(i + 1) & 1] = load_lo(stn, b_rowbase);
                fbh[(i + 1) & 1] = load_hi(stn, b_rowbase);
            }
            __builtin_amdgcn_sched_barrier(0);
            const v4i blo = fbl[i & 1], bhi = fbh[i & 1];
            // the two instructions of a fragment pair are eight instructions apart: no back-to-back dependent MFMAs
#pragma unroll
            for (int j = 0; j < FM; j++) {
                if (i * FM + j < 64) mfma_i8_16x16x64<true>(acc[i][j], blo, fal[j]);
                else mfma_i8_16x16x64<false>(acc[i][j], blo, fal[j]);
                __builtin_amdgcn_sched_barrier(0);
                spread_copies(i * 16 + j);
                if (i == FN - 1) fal[j] = load_lo(stn, a_rowbase + j * 16 * BK);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (i == 0) {   // now the hi halves: all but the two reads issued at the top of the tile
                __builtin_amdgcn_s_waitcnt(0xc07f | (2 << 8));
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int j = 0; j < FM; j++) {
                if (i * FM + j < 64) mfma_i8_16x16x64<true>(acc[i][j], bhi, fah[j]);
                else mfma_i8_16x16x64<false>(acc[i][j], bhi, fah[j]);
                __builtin_amdgcn_sched_barrier(0);
                spread_copies(i * 16 + 8 + j);
                if (i == FN - 1) {
                    fah[j] = load_hi(stn, a_rowbase + j * 16 * BK);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        }
    }
    wait_lgkmcnt0();   // the reads and copies past the last tile land before LDS is reused
    wait_vmcnt<0>();
    asm volatile("s_nop 15\n\ts_nop 15");   // the last MFMAs' results must be written before ordinary instructions read them
    __syncthreads();   // every wave is done with the operand stages

    // Epilogue.  acc[i][j][r] is out[m = m_base + 16j + lane%16][n = n_base + 16i + 4*(lane/16) + r].  Per-row and
    // per-column terms are first widened to fp32 in LDS (absent terms are the neutral elements 1.0f, 0 and -0.0f).
    float* sS2 = (float*)smem;
    float* sFb = sS2 + BN;
    int32_t* sIb = (int32_t*)(sFb + BN);
    float* sS1 = (float*)(sIb + BN);
    {
        const bool has_ib = p.bias && p.bias_dt == DT_I32;
        const bool has_fb = p.bias && p.bias_dt != DT_I32;
        for (int i = tid; i < BN; i += NT) {
            int64_t n = n0 + i;
            if (n >= p.N) n = p.N - 1;
            const int64_t si = p.x2s_len == 1 ? 0 : n;
            float sv = 1.0f;
            if constexpr (!MXS) {
                sv = p.x2s_dt == DT_U64 ? u2f((uint32_t)((const uint64_t*)p.x2s)[si]) : load_scalar_as_f32(p.x2s, p.x2s_dt, si);
                if (p.x2s_trunc || p.x2s_dt == DT_U64) sv = u2f(f2u(sv) & 0xFFFFE000u);
            }
            sS2[i] = sv;
            sIb[i] = has_ib ? ((const int32_t*)p.bias)[bz * p.bias_bs + n] : 0;
            sFb[i] = has_fb ? load_scalar_as_f32(p.bias, p.bias_dt, bz * p.bias_bs + n) : -0.0f;
        }
        for (int i = tid; i < BM; i += NT) {
            int64_t m = m0 + i;
            if (m >= p.M) m = p.M - 1;
            sS1[i] = p.x1s ? p.x1s[p.x1s_one ? 0 : m] : 1.0f;
        }
    }
    if constexpr (OUT_DT == DT_I32 || OUT_DT == DT_I8) {
        // Integer outputs (no per-row scale): INT32 = acc + ib[n]; INT8 = clip(s9(s9(fp32(acc + ib[n]) * s2[n]) + s9(off[n])), the
        // offset from p.x2off or from bits 37..45 of a UINT64 scale word, s9 = round half to even and clamp to [-256, 255].
        // They leave straight from the registers: four consecutive columns of one row per lane and fragment.
        static_assert(!F8 && !MXS, "integer outputs belong to the int8 mode");
        float* sOff = (float*)smem + 3 * BN + BM;
        const bool has_off = p.x2off != nullptr || p.x2s_dt == DT_U64;
        if (OUT_DT == DT_I8 && has_off) {
            for (int i = tid; i < BN; i += NT) {
                int64_t n = n0 + i;
                if (n >= p.N) n = p.N - 1;
                float off;
                if (p.x2off) off = p.x2off[p.x2off_len == 1 ? 0 : n];
                else {
                    const int raw = (int)((((const uint64_t*)p.x2s)[p.x2s_len == 1 ? 0 : n] >> 37) & 0x1FF);
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
            const int64_t m = m0 + wm * TM + j * 16 + frow;
#pragma unroll
            for (int i = 0; i < FN; i++) {
                const int nl = wn * TN + i * 16 + 4 * fq;
                const int64_t n = n0 + nl;
                const v4i ib = *(const v4i*)(sIb + nl);
                v4i o;
                if constexpr (OUT_DT == DT_I32) {
#pragma unroll
                    for (int e = 0; e < 4; e++) o[e] = acc[i][j][e] + ib[e];
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
                        float t = __builtin_rintf((float)(acc[i][j][e] + ib[e]) * s2[e]);
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
        return;
    }
    __syncthreads();
    // Results leave straight from the registers: a lane holds four consecutive columns of one row per fragment (8 bytes of
    // 16-bit output); the four lanes that share a row cover 32 contiguous bytes.  Parking each 16 x TN block in an LDS patch
    // to form 16-byte stores over whole rows was measured 5 us slower per launch on 2048 x 11008 (with one wave per SIMD
    // nothing hides the patch's write-to-read round trips; the int32 output of the same kernel, stored directly, beat the
    // 16-bit one although it writes twice the bytes).
    uint16_t* out = (uint16_t*)p.out + bz * p.M * p.ldc;
    const bool vec_ok = (p.ldc % 4) == 0 && ((uintptr_t)p.out % 8) == 0;
#pragma unroll
    for (int j = 0; j < FM; j++) {
        const float s1 = sS1[wm * TM + j * 16 + frow];
        const int64_t m = m0 + wm * TM + j * 16 + frow;
#pragma unroll
        for (int i = 0; i < FN; i++) {
            const int nl = wn * TN + i * 16 + 4 * fq;   // column inside the workgroup's tile
            const v4f fbv = *(const v4f*)(sFb + nl);
            const v4f s2 = *(const v4f*)(sS2 + nl);
            const v4i ib = *(const v4i*)(sIb + nl);
            v4f v;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float tv;
                if constexpr (F8) tv = acc[i][j][e];
                else tv = (float)(acc[i][j][e] + ib[e]);
                tv = tv * s2[e];
                tv = tv * s1;
                v[e] = tv + fbv[e];
            }
            const v4us o4 = pack4_b16<OUT_DT>(v);
            const int64_t n = n0 + nl;
            if (m < p.M) {
                if (vec_ok && n + 3 < p.N) *(v4us*)(out + m * p.ldc + n) = o4;
                else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (n + e < p.N) out[m * p.ldc + n + e] = o4[e];
                }
            }
        }
    }
}

template <int FN, int OUT_DT, bool F8 = false, bool MXS = false>
static int launch_wide_one(const QgemmParams& p, int64_t batch, hipStream_t st)
{
    constexpr int BM = 256, BN = 32 * FN, BK = 128;
    const int tiles_m = (int)((p.M + BM - 1) / BM), tiles_n = (int)((p.N + BN - 1) / BN);
    const size_t lds = (size_t)2 * (BM + BN) * BK + (MXS ? (size_t)2 * ((BM + BN + 255) / 256) * 4096 : 0);
    auto k = qgemm_i8_wide_kernel<FN, OUT_DT, F8, MXS>;
    static std::atomic<uint64_t> attr_set{0};   // one bit per device: the attribute belongs to the (kernel, device) pair
    if (!device_flag_test(attr_set)) {
        hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        device_flag_set(attr_set);
    }
    hipLaunchKernelGGL(k, dim3((unsigned)(tiles_m * tiles_n), (unsigned)batch), dim3(256), lds, st, p, tiles_m, tiles_n);
    return (int)hipGetLastError();
}

// Tile width 32 * fn columns, fn = 8..11.  Needs what the int8 fast path needs (K-contiguous 16-byte aligned operands,
// 16-bit output) and K % 128 == 0.
int launch_int8_wide(const QgemmParams& p, int fn, int64_t batch, int out_dt, hipStream_t st)
{
    if (p.KB % 128 != 0 || p.KB < 128) return OPSNN_NOT_TAKEN;
    if (out_dt == DT_I32 || out_dt == DT_I8) {   // integer epilogue: no per-row scale, no floating bias
        if (p.x1s || (p.bias && p.bias_dt != DT_I32)) return OPSNN_NOT_TAKEN;
        const bool i32 = out_dt == DT_I32;
        switch (fn) {
            case 8: return i32 ? launch_wide_one<8, DT_I32>(p, batch, st) : launch_wide_one<8, DT_I8>(p, batch, st);
            case 9: return i32 ? launch_wide_one<9, DT_I32>(p, batch, st) : launch_wide_one<9, DT_I8>(p, batch, st);
            case 10: return i32 ? launch_wide_one<10, DT_I32>(p, batch, st) : launch_wide_one<10, DT_I8>(p, batch, st);
            case 11: return i32 ? launch_wide_one<11, DT_I32>(p, batch, st) : launch_wide_one<11, DT_I8>(p, batch, st);
            default: return OPSNN_NOT_TAKEN;
        }
    }
    if (out_dt != DT_BF16 && out_dt != DT_F16) return OPSNN_NOT_TAKEN;
    const bool bf = out_dt == DT_BF16;
    switch (fn) {
        case 8: return bf ? launch_wide_one<8, DT_BF16>(p, batch, st) : launch_wide_one<8, DT_F16>(p, batch, st);
        case 9: return bf ? launch_wide_one<9, DT_BF16>(p, batch, st) : launch_wide_one<9, DT_F16>(p, batch, st);
        case 10: return bf ? launch_wide_one<10, DT_BF16>(p, batch, st) : launch_wide_one<10, DT_F16>(p, batch, st);
        case 11: return bf ? launch_wide_one<11, DT_BF16>(p, batch, st) : launch_wide_one<11, DT_F16>(p, batch, st);
        default: return OPSNN_NOT_TAKEN;
    }
}

}  // namespace opsnn

namespace opsnn {

// The fp8 e4m3 instantiation: p.x1s / p.x2s / fp32 bias as for int8 (x1s_one: one scale for all rows), no integer bias.
int launch_f8_wide(const QgemmParams& p, int fn, int64_t batch, int out_dt, hipStream_t st)
{
    if (p.KB % 128 != 0 || p.KB < 128) return OPSNN_NOT_TAKEN;
    if (out_dt != DT_BF16 && out_dt != DT_F16) return OPSNN_NOT_TAKEN;
    const bool bf = out_dt == DT_BF16;
    switch (fn) {
        case 8: return bf ? launch_wide_one<8, DT_BF16, true>(p, batch, st) : launch_wide_one<8, DT_F16, true>(p, batch, st);
        case 9: return bf ? launch_wide_one<9, DT_BF16, true>(p, batch, st) : launch_wide_one<9, DT_F16, true>(p, batch, st);
        case 10: return bf ? launch_wide_one<10, DT_BF16, true>(p, batch, st) : launch_wide_one<10, DT_F16, true>(p, batch, st);
        case 11: return bf ? launch_wide_one<11, DT_BF16, true>(p, batch, st) : launch_wide_one<11, DT_F16, true>(p, batch, st);
        default: return OPSNN_NOT_TAKEN;
    }
}

}  // namespace opsnn

namespace opsnn {

// MXFP8: p.sa / p.sb (one e8m0 byte per 32 K elements, K-contiguous per row, 16-byte aligned rows), fp32 bias,
// K % 512 == 0, fn 8 or 9.
int launch_mxfp8_wide(const QgemmParams& p, int fn, int64_t batch, int out_dt, hipStream_t st)
{
    if (p.KB % 512 != 0 || p.KB < 512 || !p.sa || !p.sb) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)p.sa | (uintptr_t)p.sb | (uint64_t)p.sa_rs | (uint64_t)p.sb_rs | (uint64_t)p.sa_bs | (uint64_t)p.sb_bs) % 16) return OPSNN_NOT_TAKEN;
    if (out_dt != DT_BF16 && out_dt != DT_F16) return OPSNN_NOT_TAKEN;
    const bool bf = out_dt == DT_BF16;
    switch (fn) {
        case 8: return bf ? launch_wide_one<8, DT_BF16, true, true>(p, batch, st) : launch_wide_one<8, DT_F16, true, true>(p, batch, st);
        case 9: return bf ? launch_wide_one<9, DT_BF16, true, true>(p, batch, st) : launch_wide_one<9, DT_F16, true, true>(p, batch, st);
        default: return OPSNN_NOT_TAKEN;
    }
}

}  // namespace opsnn
