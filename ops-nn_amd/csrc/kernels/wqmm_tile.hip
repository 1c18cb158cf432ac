// Weight-only matmul with many rows of x: one pass over the weight, every weight dequantised exactly once.
//
//   y = x @ T(T(w + offset) * scale) + bias,  T = rounding through x's dtype
// (wqbmmv2_kernel_golden.py:199-297; device counterpart in the reference: the vector-unit antiquant in front of the cube,
// matmul/weight_quant_batch_matmul_v2/op_kernel/arch35/n_first/basic_block_vf_nd.h:139-148).
//
// With more than a few rows of x the work is a GEMM, not a stream: 2 * M * N * K flops against N * K weights.  The decode
// kernels of wqmm_stream.hip.h dequantise a weight block per 16..128 rows of x, so 256 rows read and dequantise the weight
// twice.  Here a workgroup owns BM rows of x (all of them, up to 256) and 128 weight rows (output columns); per K step of
// 64 it
//   * dequantises its 128 x 64 weights ONCE (two 8-weight groups per thread, the two roundings of the golden in x's own
//     arithmetic) and writes them as 16-bit values into LDS -- one step ahead, in the shadow of the matrix instructions,
//   * receives the BM x 64 tile of x by 16-byte asynchronous global -> LDS copies, two steps ahead,
//   * and contracts both with v_mfma_f32_16x16x32 (x's dtype), every wave a 64 x (128 / WGN) sub-tile.
// Raw weights, scales and offsets also travel by asynchronous global -> LDS copies, into a small staging area that
// belongs to the issuing wave: every lane later reads back bytes its own wave fetched, so an s_waitcnt of the wave is
// all the synchronisation they need.  No memory instruction of the loop has a register destination: the copies are
// written as inline assembly and waited for by explicit counts (batches are issued in a fixed order and complete in
// order, so "all but the newest batch" is one s_waitcnt), and the compiler, which cannot know when such an instruction
// completes, has no register to move or reuse too early.
// One barrier per K step: behind it every wave has finished the previous step's LDS reads, so the x stage that step read
// and the weight stage before it may be overwritten.
//
// Built with -DOPSNN_WQ_AUDIT the kernel issues no copy: it records the addresses the copies would touch, and the
// launcher checks them against the tensors on the host (a development aid for changes to the addressing).
#include "wqmm_stream.hip.h"
#ifdef OPSNN_WQ_AUDIT
#include <cstdio>
#include <vector>
#endif

namespace opsnn {

typedef int v2i_t __attribute__((ext_vector_type(2)));

// Asynchronous global -> LDS copies the compiler does not count.  The address is a 64-bit scalar base plus a 32-bit
// unsigned offset per lane; m0 holds the (wave-uniform) LDS destination: lane l lands at m0 + 16 l (16-byte form) or
// m0 + 4 l (4-byte form).  The caller waits with wait_vmcnt.
#ifdef OPSNN_WQ_AUDIT
// Address audit (a debugging build): instead of copying, every thread records the lowest and highest global byte
// address and the highest LDS byte offset each class of copy would touch; the launcher checks them on the host and
// refuses to run the real kernel if one lies outside its tensor.
struct WqAudit { unsigned long long lo[4], hi[4]; unsigned int lds_hi, pad; };
#define WQ_AUDIT_ARG , int cls, WqAudit& au
#define WQ_AUDIT_PASS(c) , c, au
__device__ __forceinline__ void dma16(uint64_t base, uint32_t off, uint32_t lds WQ_AUDIT_ARG)
{
    const unsigned long long a = base + off;
    au.lo[cls] = a < au.lo[cls] ? a : au.lo[cls];
    au.hi[cls] = a + 16 > au.hi[cls] ? a + 16 : au.hi[cls];
    const unsigned int l = lds + 16 * (threadIdx.x & 63) + 16;
    au.lds_hi = l > au.lds_hi ? l : au.lds_hi;
}
__device__ __forceinline__ void dma4(uint64_t base, uint32_t off, uint32_t lds WQ_AUDIT_ARG)
{
    const unsigned long long a = base + off;
    au.lo[cls] = a < au.lo[cls] ? a : au.lo[cls];
    au.hi[cls] = a + 4 > au.hi[cls] ? a + 4 : au.hi[cls];
    const unsigned int l = lds + 4 * (threadIdx.x & 63) + 4;
    au.lds_hi = l > au.lds_hi ? l : au.lds_hi;
}
#else
#define WQ_AUDIT_PASS(c)
__device__ __forceinline__ void dma16(uint64_t base, uint32_t off, uint32_t lds)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds), "v"(off), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void dma4(uint64_t base, uint32_t off, uint32_t lds)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" : : "s"(lds), "v"(off), "s"(base) : "memory", "m0");
}
#endif
__device__ __forceinline__ uint64_t uniform64(uint64_t v)
{
    // (the builtin returns a signed int: each half goes through uint32_t, or the low half would sign-extend into the high one)
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return (uint64_t)lo | ((uint64_t)hi << 32);
}

// A raw unit is what one weight copy instruction per thread brings: 64 bytes of each of the 128 weight rows, i.e. SPS
// steps of K (two for int4, one for int8), with the scales and offsets of the groups those steps touch.
template <int WBITS, bool HAS_OFF> constexpr int wq_tile_unit_bytes() { return 1024 + (HAS_OFF ? 512 : 256); }   // per wave
constexpr int WQ_TILE_UNITS = 2;   // raw units in LDS per wave
template <int BM> constexpr size_t wq_tile_lds_bytes() { return 3 * (size_t)BM * 128 + 2 * (size_t)128 * 128 + WQ_TILE_UNITS * 8 * (size_t)(1024 + 512); }

template <int XDT, int WBITS, int BM, bool HAS_OFF>
__global__ __launch_bounds__(512, 1) void wqmm_tile_kernel(WqParams p)
{
    constexpr int BN = 128, BK = 64, NT = 512;
    constexpr int WGM = BM / 64, WGN = 8 / WGM;            // 8 waves: BM 256 -> 4 x 2, 128 -> 2 x 4, 64 -> 1 x 8
    constexpr int TN = BN / WGN, FM = 4, FN = TN / 16;     // wave tile 64 x TN
    constexpr int XS = 3, WS = 2;                          // stages of x and of the dequantised weights
    constexpr int RP = WQ_TILE_UNITS;
    constexpr int SPS = WBITS == 4 ? 2 : 1;                // steps per raw unit
    constexpr int X_BYTES = BM * BK * 2, W_BYTES = BN * BK * 2;
    constexpr int NX = BM / 64;                            // x copies per thread and step (64 rows of 128 bytes per instruction)
    constexpr int NRAW = 2 + (HAS_OFF ? 1 : 0);            // copies per thread and unit: weights, scales (, offsets)
    constexpr int UNIT = 1024 + 512;                       // staging bytes per wave and unit: 1024 weights, 256 scales, 256 offsets
    extern __shared__ __attribute__((aligned(16))) char smem[];
    char* const sx = smem;
    char* const sw = smem + XS * X_BYTES;
    char* const sraw = sw + WS * W_BYTES;                  // [RP units][8 waves][UNIT]
    const uint32_t lds0 = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)smem;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const int64_t n0 = (int64_t)blockIdx.x * BN;
    const int KT = (int)(p.K / BK);
    const int NU = (KT + SPS - 1) / SPS;                   // raw units
    const int M = (int)p.M;

    // x copies: instruction i fills tile rows 64 i .. 64 i + 63; this thread moves the 16-byte chunk that belongs at
    // position tid % 8 of row 64 i + tid / 8 (rows are chunk-swizzled: logical chunk c sits at c ^ (row / 2) % 8)
    const int crow = tid >> 3;
    const int cchunk = (tid & 7) ^ ((crow >> 1) & 7);
    uint32_t xoff[NX];
#pragma unroll
    for (int i = 0; i < NX; i++) {
        int r = i * 64 + crow;
        r = r < M ? r : M - 1;                             // rows past the end repeat the last one; their outputs are not stored
        xoff[i] = (uint32_t)r * (uint32_t)(p.K * 2) + cchunk * 16;
    }
    const uint64_t xbase = uniform64((uint64_t)(uintptr_t)p.x);
    // weights: thread (row = tid / 4, part = tid % 4) copies bytes 16 part .. 16 part + 15 of its row's 64 bytes of a unit,
    // and dequantises the 16 weights k = 16 part .. 16 part + 15 of every step of that row
    const int wrow = tid >> 2, wpart = tid & 3;
    const int64_t wn_g = (n0 + wrow) < p.N ? (n0 + wrow) : p.N - 1;
    // what this lane copies.  int8: its own 16 bytes (row tid / 4, bytes 16 part ..).  int4: a unit holds two steps, and
    // the staging area is laid out [step][row][32 bytes] so that the 8-byte reads of a step are conflict free: lane l
    // of the wave copies bytes 32 (l / 32) + 16 (l % 2) .. of row (l % 32) / 2
    const int frow_l = WBITS == 4 ? (wave * 16 + ((lane & 31) >> 1)) : wrow;
    const int fbyte = WBITS == 4 ? ((lane >> 5) * 32 + (lane & 1) * 16) : wpart * 16;
    const int64_t fn_g = (n0 + frow_l) < p.N ? (n0 + frow_l) : p.N - 1;
    const uint32_t woff = (uint32_t)(fn_g - n0) * (uint32_t)p.ldw + fbyte;
    const uint64_t wbase = uniform64((uint64_t)(uintptr_t)p.w + (uint64_t)n0 * (uint64_t)p.ldw);
    // scales and offsets: lane (row, j = tid % 4) copies the 4-byte word around the row's scale of group g0 + j, g0 the
    // group of the unit's first step (a 16-bit element travels inside the aligned word that holds it: same page, never
    // past a mapping); the thread that dequantises (row, any part) reads word row * 4 + (g - g0) back
    const uint32_t spg = p.group >= p.K ? (uint32_t)KT : (uint32_t)(p.group / BK);   // steps per group
    const int spg_shift = (spg & (spg - 1)) == 0 ? __builtin_ctz(spg) : -1;
    auto group_of_step = [&](uint32_t t) { return spg_shift >= 0 ? t >> spg_shift : t / spg; };
    const uint32_t glast = (uint32_t)((p.K + p.group - 1) / p.group) - 1;
    const uint64_t sbase = uniform64((uint64_t)(uintptr_t)p.scale & ~(uint64_t)3);
    const uint64_t obase = HAS_OFF ? uniform64((uint64_t)(uintptr_t)p.offset & ~(uint64_t)3) : 0;
    const uint32_t s_el0 = (uint32_t)(((uintptr_t)p.scale >> 1) & 1) + (uint32_t)wn_g * (uint32_t)p.s_cs;   // element index from sbase, group 0
    const uint32_t o_el0 = HAS_OFF ? (uint32_t)(((uintptr_t)p.offset >> 1) & 1) + (uint32_t)wn_g * (uint32_t)p.s_cs : 0;
    const uint32_t srs = (uint32_t)p.s_rs;
    const int wkey = (wrow >> 1) & 7;
    char* const wdst = sw + wrow * (BK * 2);
    const int wc0 = ((2 * wpart) ^ wkey) << 4, wc1 = ((2 * wpart + 1) ^ wkey) << 4;
    const uint32_t raw_wave = (uint32_t)(XS * X_BYTES + WS * W_BYTES) + wave * UNIT;   // byte offset in smem, unit 0

#ifdef OPSNN_WQ_AUDIT
    WqAudit au;
    for (int c = 0; c < 4; c++) { au.lo[c] = ~0ull; au.hi[c] = 0; }
    au.lds_hi = 0; au.pad = 0;
#endif
    // Copies never have a register destination, so one issued for a step or unit past the end is harmless: it repeats
    // the last one's bytes into a stage nobody reads again, and every batch has the same number of instructions.
    auto issue_x = [&](int it) {          // x tile of step it into its stage
        const uint32_t kt = (uint32_t)(it < KT ? it : KT - 1);
        const uint64_t b = xbase + (uint64_t)kt * (BK * 2);
        const uint32_t dx = lds0 + (uint32_t)(it % XS) * X_BYTES + wave * 1024;
#pragma unroll
        for (int i = 0; i < NX; i++) dma16(b, xoff[i], dx + i * (NT * 16) WQ_AUDIT_PASS(0));
    };
    auto issue_unit = [&](int u) {        // raw unit u into its slot
        const uint32_t uc = (uint32_t)(u < NU ? u : NU - 1);
        const uint32_t dst = lds0 + raw_wave + (uint32_t)(u % RP) * (8 * UNIT);
        dma16(wbase + (uint64_t)uc * 64, woff, dst WQ_AUDIT_PASS(1));
        uint32_t g = group_of_step(uc * SPS) + wpart;
        g = g < glast ? g : glast;
        dma4(sbase, ((s_el0 + g * srs) * 2) & ~3u, dst + 1024 WQ_AUDIT_PASS(2));
        if constexpr (HAS_OFF) dma4(obase, ((o_el0 + g * srs) * 2) & ~3u, dst + 1280 WQ_AUDIT_PASS(3));
    };

    v4f acc[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; i++)
#pragma unroll
        for (int j = 0; j < FM; j++) acc[i][j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    const DqConst dqc = make_dq_const();
    const int frow = lane & 15, fq = lane >> 4;
    const int fkey = (frow >> 1) & 7;
    const int a_rowbase = (wm * 64 + frow) * (BK * 2);
    const int b_rowbase = (wn * TN + frow) * (BK * 2);

    // raw material of step t (t may be KT: then the last unit's bytes, dequantised for nobody)
    struct Raw { v4i piece; uint32_t sword, oword, g; };
    auto read_raw = [&](int t) {
        Raw r;
        const int u = t / SPS;
        const char* raw = smem + raw_wave + (u % RP) * (8 * UNIT);
        const uint32_t tc = (uint32_t)(t < KT ? t : KT - 1);
        r.g = group_of_step(tc);
        const uint32_t g0 = group_of_step((uint32_t)(u < NU ? u : NU - 1) * SPS);
        if constexpr (WBITS == 4) {
            const v2i_t q = *(const v2i_t*)(raw + (t % SPS) * 512 + (lane >> 2) * 32 + wpart * 8);
            r.piece = v4i{q[0], q[1], 0, 0};
        } else {
            r.piece = *(const v4i*)(raw + lane * 16);
        }
        const uint32_t slot = (lane & ~3) + (r.g - g0);
        r.sword = *(const uint32_t*)(raw + 1024 + slot * 4);
        r.oword = HAS_OFF ? *(const uint32_t*)(raw + 1280 + slot * 4) : 0u;
        return r;
    };
    auto dequant_to = [&](const Raw& r, int t) {   // -> dequantised weights of step t in their LDS stage
        const uint16_t sb = (uint16_t)(r.sword >> (((s_el0 + r.g * srs) & 1) * 16));
        const uint16_t ob = HAS_OFF ? (uint16_t)(r.oword >> (((o_el0 + r.g * srs) & 1) * 16)) : (uint16_t)0;
        const v4i lo = dequant8<XDT, WBITS, HAS_OFF, true>(r.piece, 0, sb, ob, dqc);
        const v4i hi = dequant8<XDT, WBITS, HAS_OFF, true>(r.piece, 1, sb, ob, dqc);
        char* d = wdst + (t % WS) * W_BYTES;
        *(v4i*)(d + wc0) = lo;
        *(v4i*)(d + wc1) = hi;
    };

    // ---- prologue: every unit slot filled, x tiles 0 and 1 on their way, the weights of step 0 dequantised ----
    for (int u = 0; u < RP; u++) issue_unit(u);
    issue_x(0);
    issue_x(1);
    wait_vmcnt<0>();
    asm volatile("" ::: "memory");
    {
        const Raw r0 = read_raw(0);
        dequant_to(r0, 0);
    }
    // two-step units arrive early enough for the raw material of step it + 2 to be read during step it (a full step
    // before its dequantisation): rn carries it over; one-step units are read at the top of the step that dequantises
    constexpr bool EARLY = SPS == 2;
    Raw rn = read_raw(1);
    // (one step per unit: unit 0 is spent, and the loop's first batch refills unit 1's slot, so unit RP goes out here)
    if constexpr (SPS == 1) issue_unit(RP);

    // ---- step it: the matrix instructions of step it, and the dequantisation of step it + 1 in their shadow ----
    // Batch of step it (issued behind its barrier): x tile it + 2; and, if a unit's slot has just been read for the
    // last time (every step for one-step units: unit it + 1; even steps for two-step units: unit it / 2), the unit
    // RP further on.  Copies complete in order, so "all but the newest batch" is one counter value.
    auto load_frags = [&](const char* ax, const char* bw, int half, v4i (&fa)[FM], v4i (&fb)[FN]) {
        const int coff = ((4 * half + fq) ^ fkey) << 4;
#pragma unroll
        for (int j = 0; j < FM; j++) fa[j] = *(const v4i*)(ax + a_rowbase + j * 16 * (BK * 2) + coff);
#pragma unroll
        for (int i = 0; i < FN; i++) fb[i] = *(const v4i*)(bw + b_rowbase + i * 16 * (BK * 2) + coff);
    };
    auto mma = [&](const v4i (&fa)[FM], const v4i (&fb)[FN]) {
#pragma unroll
        for (int i = 0; i < FN; i++)
#pragma unroll
            for (int j = 0; j < FM; j++) {
                if constexpr (XDT == DT_F16)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, fb[i]), __builtin_bit_cast(v8h, fa[j]), acc[i][j], 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, fb[i]), __builtin_bit_cast(v8bf, fa[j]), acc[i][j], 0, 0, 0);
            }
    };
    v4i fa1[FM], fb1[FN];                    // second-half fragments of the previous step
#pragma unroll
    for (int j = 0; j < FM; j++) fa1[j] = v4i{0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < FN; i++) fb1[i] = v4i{0, 0, 0, 0};
    auto step = [&](int it, auto parity_c) {
        constexpr int PAR = decltype(parity_c)::value;       // it % 2 for two-step units, 0 otherwise
        constexpr int NEWEST = NX + ((SPS == 1 || PAR == 1) ? NRAW : 0);   // size of the batch of step it - 1
        wait_vmcnt<NEWEST>();
        asm volatile("" ::: "memory");
        if constexpr (!EARLY) rn = read_raw(it + 1);
        __syncthreads();   // step it's weights (written during step it - 1) and x tile are complete; every wave is done with step it - 1's LDS reads
        issue_x(it + 2);
        if constexpr (SPS == 1) issue_unit(it + 1 + RP);
        else if constexpr (PAR == 0) issue_unit(it / 2 + RP);
        const char* ax = sx + (it % XS) * X_BYTES;
        const char* bw = sw + (it % WS) * W_BYTES;
        // The fragments of the step's second K half stay in registers across the barrier: their matrix instructions run
        // at the start of the next step, while that step's first fragments are on their way from LDS (and the first
        // half's run while the second half's fragments arrive).
        v4i fa0[FM], fb0[FN];
        load_frags(ax, bw, 0, fa0, fb0);
        mma(fa1, fb1);                       // step it - 1, second half (zeros before step 0)
        dequant_to(rn, it + 1);
        if constexpr (EARLY) rn = read_raw(it + 2);
        load_frags(ax, bw, 1, fa1, fb1);
        mma(fa0, fb0);                       // step it, first half
    };
    constexpr std::integral_constant<int, 0> even{};
    constexpr std::integral_constant<int, 1> odd{};
    int it = 0;
    for (; it + 1 < KT; it += 2) {
        step(it, even);
        step(it + 1, odd);
    }
    if (it < KT) step(it, even);
    mma(fa1, fb1);     // the last step's second half
    wait_vmcnt<0>();   // the copies issued for steps past the end
#ifdef OPSNN_WQ_AUDIT
    ((WqAudit*)(uintptr_t)p.m_base)[(size_t)blockIdx.x * NT + tid] = au;
    return;
#endif

    // acc[i][j][r] is y[m = wm * 64 + 16 j + lane % 16][n = n0 + wn * TN + 16 i + 4 (lane / 16) + r]
#pragma unroll
    for (int j = 0; j < FM; j++) {
        const int m = wm * 64 + j * 16 + frow;
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < FN; i++) {
            const int64_t n = n0 + wn * TN + i * 16 + 4 * fq;
            v4f v = acc[i][j];
            if (p.bias) {
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = v[r] + load_scalar_as_f32(p.bias, p.bias_dt, (n + r) < p.N ? (n + r) : p.N - 1);
            }
            const v4us o = pack4_b16<XDT>(v);
            uint16_t* dst = p.y + (int64_t)m * p.N + n;
            if (n + 3 < p.N && (p.N % 4) == 0) {
                *(v4us*)dst = o;
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (n + r < p.N) dst[r] = o[r];
            }
        }
    }
}

template <int XDT, int WBITS, int BM>
static int launch_tile_bm(const WqParams& p, hipStream_t st)
{
    const size_t lds = wq_tile_lds_bytes<BM>();
    const dim3 grid((unsigned)((p.N + 127) / 128));
    auto launch = [&](auto kern) -> int {
        static std::atomic<uint64_t> attr_set{0};   // one bit per device: the attribute belongs to the (kernel, device) pair
        if (!device_flag_test(attr_set)) {
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return (int)e;
            device_flag_set(attr_set);
        }
#ifdef OPSNN_WQ_AUDIT
        {
            const size_t n = (size_t)grid.x * 512;
            WqAudit* d = nullptr;
            if (hipMalloc((void**)&d, n * sizeof(WqAudit)) != hipSuccess) return -100;
            WqParams q = p;
            q.m_base = (int64_t)(uintptr_t)d;
            hipLaunchKernelGGL(kern, grid, dim3(512), lds, st, q);
            std::vector<WqAudit> h(n);
            if (hipStreamSynchronize(st) != hipSuccess || hipMemcpy(h.data(), d, n * sizeof(WqAudit), hipMemcpyDeviceToHost) != hipSuccess) return -101;
            (void)hipFree(d);
            const int64_t ngr = (p.K + p.group - 1) / p.group;
            const unsigned long long lo[4] = {(unsigned long long)(uintptr_t)p.x, (unsigned long long)(uintptr_t)p.w,
                                              (unsigned long long)(uintptr_t)p.scale & ~3ull, (unsigned long long)(uintptr_t)p.offset & ~3ull};
            const unsigned long long sext = (unsigned long long)(((p.N - 1) * p.s_cs + (ngr - 1) * p.s_rs + 1) * 2);
            const unsigned long long hi[4] = {lo[0] + (unsigned long long)(p.M * p.K * 2), lo[1] + (unsigned long long)(p.N * p.ldw),
                                              (((unsigned long long)(uintptr_t)p.scale + sext) + 3) & ~3ull, (((unsigned long long)(uintptr_t)p.offset + sext) + 3) & ~3ull};
            size_t bad = 0;
            for (size_t i = 0; i < n; i++) {
                for (int c = 0; c < 4; c++) {
                    if (h[i].hi[c] == 0) continue;   // class never used
                    if (h[i].lo[c] < lo[c] || h[i].hi[c] > hi[c]) {
                        if (bad < 8) fprintf(stderr, "wq audit: thread %zu class %d touches [%llx, %llx) outside [%llx, %llx)\n", i, c, h[i].lo[c], h[i].hi[c], lo[c], hi[c]);
                        bad++;
                    }
                }
                if (h[i].lds_hi > lds) { if (bad < 8) fprintf(stderr, "wq audit: thread %zu LDS end %u > %zu\n", i, h[i].lds_hi, lds); bad++; }
            }
            fprintf(stderr, "wq audit: M %lld N %lld K %lld group %lld: %zu threads, %zu out of bounds\n", (long long)p.M, (long long)p.N, (long long)p.K, (long long)p.group, n, bad);
            return bad ? -102 : -103;   // either way the real kernel does not run in this build
        }
#endif
        hipLaunchKernelGGL(kern, grid, dim3(512), lds, st, p);
        return (int)hipGetLastError();
    };
    if (p.offset) return launch(wqmm_tile_kernel<XDT, WBITS, BM, true>);
    return launch(wqmm_tile_kernel<XDT, WBITS, BM, false>);
}

// Takes M in 49..256 with K-contiguous weights, K a multiple of 64 and groups that are multiples of 64 (or one per column).
template <int XDT, int WBITS>
int launch_wq_tile(const WqParams& p, hipStream_t st)
{
    if (p.M < 1 || p.M > 256 || p.K % (WBITS == 4 ? 128 : 64) != 0) return OPSNN_NOT_TAKEN;   // whole 64-byte units per weight row
    if (p.group < p.K && p.group % 64 != 0) return OPSNN_NOT_TAKEN;
    // 32-bit lane offsets: x, 128 weight rows, and the scale table
    if (p.M * p.K * 2 >= (1ll << 32) || p.ldw < 0 || 128 * p.ldw >= (1ll << 32)) return OPSNN_NOT_TAKEN;
    if (p.s_cs < 0 || p.s_rs < 0) return OPSNN_NOT_TAKEN;
    const int64_t ngroups = (p.K + p.group - 1) / p.group;
    if ((p.N * p.s_cs + ngroups * p.s_rs + 2) * 2 >= (1ll << 32)) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)p.w | (uint64_t)p.ldw) % 16 || ((uintptr_t)p.x % 16)) return OPSNN_NOT_TAKEN;
    if (p.M <= 64) return launch_tile_bm<XDT, WBITS, 64>(p, st);
    if (p.M <= 128) return launch_tile_bm<XDT, WBITS, 128>(p, st);
    return launch_tile_bm<XDT, WBITS, 256>(p, st);
}
template int launch_wq_tile<DT_F16, 4>(const WqParams&, hipStream_t);
template int launch_wq_tile<DT_F16, 8>(const WqParams&, hipStream_t);
template int launch_wq_tile<DT_BF16, 4>(const WqParams&, hipStream_t);
template int launch_wq_tile<DT_BF16, 8>(const WqParams&, hipStream_t);

}  // namespace opsnn
