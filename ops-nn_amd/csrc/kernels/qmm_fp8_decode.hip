// fp8 e4m3 x fp8 e4m3 with block scales (G-B, B-B) for up to 16 rows of x1 per pass: the decode shape of an fp8 model.
//
//   out[m,n] = cast( sum_kb ( sum_{k in block kb} x1[m,k] * x2[k,n] ) * ( s1[m/gsM, kb] * s2[kb, n/128] ) )
//
// Formula: matmul/quant_batch_matmul_v3/tests/assets/qbmmv3_kernel_golden.py:237-358 (the two block scales are multiplied
// together first, :337-343).  Arithmetic as in qmm_fp8_exact.hip: the operands are widened to fp16 (exact), the products
// are exact, a block's sum is an fp32 accumulation inside v_mfma_f32_16x16x32_f16 chained over the block's four steps from
// a zero accumulator, and one fused multiply-add per output folds it into the running sum.
//
// With so few rows the work is a stream over x2 (N * K bytes), not a GEMM: a 256-row tile kernel spends 16 times the
// matrix work and conversions on rows that do not exist.  Here, as in the x-in-registers kernel of wqmm_stream.hip.h:
//   * the workgroup's NW waves split K into NW equal ranges of NBLK scale blocks; a wave keeps the fp16 fragments of
//     x1 for its range in registers for the whole launch (16 registers per block),
//   * all waves work on the same 16 columns of the output (16 rows of the K-contiguous x2) at a time and the workgroup
//     walks column blocks blockIdx.x, + gridDim.x, ...; the stream of x2 pieces (16 bytes per lane) never stops: the
//     refills issued while one column block is multiplied already fetch the next one's pieces,
//   * a lane's 16-byte piece of an x2 row feeds two matrix instructions (bytes 0..7 and 8..15); which k a lane holds
//     inside an instruction does not matter as long as both operands agree, and x1's fragments are cut the same way,
//   * the NW partial sums of a column block meet in LDS (double-buffered, one barrier per column block) and one wave,
//     taking turns, adds them in wave order and stores 16 x 16 outputs.
// The order of the fp32 additions differs from the golden's ascending blocks (NW ranges are added at the end): the bar
// of the exact tile kernel.
#include <cstdlib>

#include "launch.h"
#include "common.hip.h"

namespace opsnn {
namespace {

struct Fp8DecParams {
    const uint8_t* a;   // x1 [M, K], K contiguous
    const uint8_t* b;   // x2 as [N, K], K contiguous
    int64_t lda, ldb;
    void* out; int out_dt;
    int64_t M, N, K;
    const float* s1; int64_t s1_rs, s1_cs;
    const float* s2; int64_t s2_rs, s2_cs;
    int gsM;
    // row / column scale form (RC): out = (sum * cs[n * cs_stride]) * rs[m * rs_stride] + bias[n]; strides 0 (one scale) or 1
    const float* rs; const float* cs; const float* bias;
    int rs_stride, cs_stride;
    // K in segments (SEG instantiations, gridDim.y of them): fp32 sums of this pass's rows, slice s at part + s * part_slice
    float* part; int64_t part_slice;
};

// 8 e4m3 bytes (two dwords) -> 8 fp16 in byte order
__device__ __forceinline__ v4i widen8_e4m3(uint32_t d0, uint32_t d1)
{
    typedef _Float16 h2v __attribute__((ext_vector_type(2)));
    const h2v w0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d0, 1.0f, false), w1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d0, 1.0f, true);
    const h2v w2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d1, 1.0f, false), w3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d1, 1.0f, true);
    return (v4i){(int)__builtin_bit_cast(uint32_t, w0), (int)__builtin_bit_cast(uint32_t, w1), (int)__builtin_bit_cast(uint32_t, w2),
                 (int)__builtin_bit_cast(uint32_t, w3)};
}

// I8: int8 operands with the same block scales and an fp32 bias (the per-tile mode of quant_batch_matmul_v4,
// qbmmv4_kernel_golden.py:258-325): a lane's 16-byte piece is one operand of v_mfma_i32_16x16x64_i8 as it is, a block's
// sum is two of them from a zero accumulator (an exact integer below 2^21), converted to fp32 for the fold.
// SEG: K is cut into gridDim.y segments of NW * NBLK blocks, one workgroup column each; wave w of segment s takes the
// NBLK blocks from (s NW + w) NBLK on, and a wave whose blocks lie past the end of K (in the last segment; K is a whole
// number of NBLK blocks) runs along on the last blocks and contributes zeros.  With more than one segment the
// workgroup stores its fp32 sums for fp8dec_reduce_kernel, which adds the segments in order and applies the epilogue.
template <int NW, int NBLK, bool RC, bool I8 = false, bool SEG = false>
__global__ __launch_bounds__(NW * 64) void fp8_block_decode_kernel(Fp8DecParams p)
{
    static_assert(!(RC && I8), "int8: the block-scale form only");
    constexpr int NCH = 2 * NBLK;                    // 64-byte chunks of an x2 row in a wave's K range
    constexpr int PF = NW == 16 ? (NCH < 4 ? NCH : 4) : NCH;   // pieces in flight per lane; divides NCH
    static_assert(NCH % PF == 0, "a piece's slot must not depend on the column block");
    extern __shared__ __attribute__((aligned(16))) float red[];   // [2][NW][256]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nrow = lane & 15, q = lane >> 4;
    int kb0 = wave * NBLK;
    bool live = true;
    if constexpr (SEG) {
        const int nbk = (int)(p.K / 128);
        kb0 = ((int)blockIdx.y * NW + wave) * NBLK;
        live = kb0 < nbk;
        if (!live) kb0 = nbk - NBLK;
    }
    const int64_t kbase = (int64_t)kb0 * 128;
    const int nblocks = (int)((p.N + 15) / 16);
    const int M = (int)p.M;

    // x1: lane (m = lane % 16, q) holds, for chunk c and half h, the 8 elements k = kbase + 64 c + 16 q + 8 h .. + 7
    v4i xf[NCH][2];
#pragma unroll
    for (int c = 0; c < NCH; c++) {
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (nrow < M) raw = *(const uint4*)(p.a + (int64_t)nrow * p.lda + kbase + 64 * c + 16 * q);
        if constexpr (I8) {
            xf[c][0] = (v4i){(int)raw.x, (int)raw.y, (int)raw.z, (int)raw.w};
        } else {
            xf[c][0] = widen8_e4m3(raw.x, raw.y);
            xf[c][1] = widen8_e4m3(raw.z, raw.w);
        }
    }
    // the scales of this lane's row of x1 for the wave's blocks (rows past M: the last row's, their outputs are not stored)
    float s1v[NBLK];
    if constexpr (!RC) {
        const int64_t mr = (nrow < M ? nrow : M - 1) / p.gsM;
#pragma unroll
        for (int j = 0; j < NBLK; j++) s1v[j] = p.s1[mr * p.s1_rs + (kb0 + j) * p.s1_cs];
    }

    auto wload = [&](int rb, int c) {
        const int64_t n = (int64_t)rb * 16 + nrow;
        return *(const uint4*)(p.b + (n < p.N ? n : p.N - 1) * p.ldb + kbase + 64 * c + 16 * q);   // columns past the edge repeat the last one
    };
    int rb = blockIdx.x;
    uint4 wq[PF];
#pragma unroll
    for (int i = 0; i < PF; i++) wq[i] = wload(rb < nblocks ? rb : nblocks - 1, i);

    for (int it = 0; rb < nblocks; it++, rb += (int)gridDim.x) {
        const int rbn = rb + (int)gridDim.x < nblocks ? rb + (int)gridDim.x : rb;   // past the end: a harmless reload
        const int64_t n0 = (int64_t)rb * 16;
        float s2v[NBLK];
        if constexpr (!RC) {
#pragma unroll
            for (int j = 0; j < NBLK; j++) s2v[j] = p.s2[(kb0 + j) * p.s2_rs + (n0 / 128) * p.s2_cs];
        }
        v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < NBLK; j++) {
            v4f t = RC ? acc : (v4f){0.0f, 0.0f, 0.0f, 0.0f};   // RC: one chain over the whole range
            v4i ti = {0, 0, 0, 0};
#pragma unroll
            for (int cc = 0; cc < 2; cc++) {
                const int c = 2 * j + cc;
                const uint4 cur = wq[c % PF];
                wq[c % PF] = c + PF < NCH ? wload(rb, c + PF) : wload(rbn, c + PF - NCH);
                if constexpr (I8) {
                    ti = __builtin_amdgcn_mfma_i32_16x16x64_i8((v4i){(int)cur.x, (int)cur.y, (int)cur.z, (int)cur.w}, xf[c][0], ti, 0, 0, 0);
                } else {
                    const v4i w0 = widen8_e4m3(cur.x, cur.y), w1 = widen8_e4m3(cur.z, cur.w);
                    t = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, w0), __builtin_bit_cast(v8h, xf[c][0]), t, 0, 0, 0);
                    t = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, w1), __builtin_bit_cast(v8h, xf[c][1]), t, 0, 0, 0);
                }
            }
            if constexpr (I8) t = (v4f){(float)ti[0], (float)ti[1], (float)ti[2], (float)ti[3]};
            if constexpr (RC) acc = t;
            else {
                const float sc = s1v[j] * s2v[j];
#pragma unroll
                for (int r = 0; r < 4; r++) acc[r] = __builtin_fmaf(t[r], sc, acc[r]);
            }
        }
        // acc[r]: m = lane % 16, n = n0 + 4 (lane / 16) + r, over this wave's K range
        if constexpr (SEG) {
            if (!live) acc = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
        }
        float* mine = red + ((it & 1) * NW + wave) * 256;
        *(v4f*)(mine + lane * 4) = acc;
        __syncthreads();
        if (wave != (it & (NW - 1))) continue;
        const float* all = red + (it & 1) * NW * 256 + lane * 4;
        v4f sum = *(const v4f*)all;
#pragma unroll 4
        for (int w = 1; w < NW; w++) {
            const v4f o = *(const v4f*)(all + w * 256);
#pragma unroll
            for (int r = 0; r < 4; r++) sum[r] = sum[r] + o[r];
        }
        if (nrow >= M) continue;
        const int64_t n = n0 + 4 * q;
        if constexpr (SEG) {
            if (gridDim.y > 1) {
                float* dst = p.part + (int64_t)blockIdx.y * p.part_slice + (int64_t)nrow * p.N + n;
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (n + r < p.N) dst[r] = sum[r];
                continue;
            }
        }
        if constexpr (RC) {   // (sum * x2Scale[n]) * x1Scale[m] + bias[n], each operation rounded
            const float rsv = p.rs[(int64_t)nrow * p.rs_stride];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int64_t ni = n + r < p.N ? n + r : p.N - 1;
                sum[r] = (sum[r] * p.cs[ni * p.cs_stride]) * rsv;
                if (p.bias) sum[r] = sum[r] + p.bias[ni];
            }
        } else if (p.bias) {
#pragma unroll
            for (int r = 0; r < 4; r++) sum[r] = sum[r] + p.bias[n + r < p.N ? n + r : p.N - 1];
        }
        if (p.out_dt == DT_F32) {
            float* dst = (float*)p.out + (int64_t)nrow * p.N + n;
#pragma unroll
            for (int r = 0; r < 4; r++)
                if (n + r < p.N) dst[r] = sum[r];
        } else {
            const v4us o = p.out_dt == DT_BF16 ? pack4_b16<DT_BF16>(sum) : pack4_b16<DT_F16>(sum);
            uint16_t* dst = (uint16_t*)p.out + (int64_t)nrow * p.N + n;
            if ((p.N % 4) == 0 && ((uintptr_t)p.out % 8) == 0 && n + 3 < p.N) *(v4us*)dst = o;
            else {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (n + r < p.N) dst[r] = o[r];
            }
        }
    }
}

// out = epilogue(sum over the K segments, in order, of part[s]) for one pass of up to 16 rows: the block-scale form adds the
// bias, the row / column scale form (RC) computes (sum * x2Scale[n]) * x1Scale[m] + bias[n]
template <bool RC>
__global__ __launch_bounds__(256) void fp8dec_reduce_kernel(Fp8DecParams p, int splits)
{
    const int64_t total = p.M * p.N, stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        float v = p.part[i];
        for (int s = 1; s < splits; s++) v = v + p.part[(int64_t)s * p.part_slice + i];
        const int64_t m = i / p.N, n = i - m * p.N;
        if constexpr (RC) v = (v * p.cs[n * p.cs_stride]) * p.rs[m * p.rs_stride];
        if (p.bias) v = v + p.bias[n];
        if (p.out_dt == DT_F32) ((float*)p.out)[i] = v;
        else ((uint16_t*)p.out)[i] = p.out_dt == DT_BF16 ? bf16_bits(v) : f16_bits(v);
    }
}

template <int NW, int NBLK, bool RC, bool I8 = false, bool SEG = false>
int launch_decode_one(const Fp8DecParams& p, hipStream_t st, int splits = 1)
{
    if constexpr (!SEG) {
        if (splits > 1 || p.K != (int64_t)NW * NBLK * 128) return launch_decode_one<NW, NBLK, RC, I8, true>(p, st, splits);
    }
    const int64_t nbk = p.K / 128;
    if (splits < 1 || splits > 16 || nbk % NBLK != 0 || nbk < NBLK || (int64_t)splits * NW * NBLK < nbk || (splits > 1 && !p.part)) return -1;
    const int nblocks = (int)((p.N + 15) / 16);
    const int cus = 256 / splits;   // the CUs shared between the segments' workgroup columns
    const int grid = nblocks < cus ? nblocks : cus;
    const size_t lds = (size_t)2 * NW * 256 * sizeof(float);
    hipLaunchKernelGGL((fp8_block_decode_kernel<NW, NBLK, RC, I8, SEG>), dim3((unsigned)grid, (unsigned)splits), dim3(NW * 64), lds, st, p);
    if (hipError_t e = hipGetLastError(); e != hipSuccess || splits == 1) return (int)e;
    hipLaunchKernelGGL(fp8dec_reduce_kernel<RC>, dim3(splitk_reduce_grid(p.M * p.N)), dim3(256), 0, st, p, splits);
    return (int)hipGetLastError();
}

template <bool RC, bool I8 = false>
int launch_decode_split(const Fp8DecParams& p, int nw, int nblk, hipStream_t st, int splits = 1)
{
    if (nw == 16) {
        if (nblk == 1) return launch_decode_one<16, 1, RC, I8>(p, st, splits);
        if (nblk == 2) return launch_decode_one<16, 2, RC, I8>(p, st, splits);
        if (nblk == 4) return launch_decode_one<16, 4, RC, I8>(p, st, splits);
        return -1;
    }
    switch (nblk) {
        case 1: return launch_decode_one<8, 1, RC, I8>(p, st, splits);
        case 2: return launch_decode_one<8, 2, RC, I8>(p, st, splits);
        case 3: return launch_decode_one<8, 3, RC, I8>(p, st, splits);
        case 4: return launch_decode_one<8, 4, RC, I8>(p, st, splits);
        case 5: return launch_decode_one<8, 5, RC, I8>(p, st, splits);
        case 6: return launch_decode_one<8, 6, RC, I8>(p, st, splits);
        case 7: return launch_decode_one<8, 7, RC, I8>(p, st, splits);
        default: return -1;
    }
}


// ---- fp8 e4m3 x fp4 e2m1 with e8m0 scales per 32 elements of K (the MX mode of quant_batch_matmul_v4,
// qbmmv4_kernel_golden.py:119-186), up to 16 rows of x1 per pass ----
// The same stream over x2, here N * K / 2 bytes: a lane's 16-byte piece is the 32 consecutive elements of one scale
// block, four lanes cover the 128 elements of one v_mfma_scale_f32_16x16x128_f8f6f4, and the instruction applies both
// operands' scales (one byte per lane: lane group q supplies block q) and accumulates in place -- the arithmetic of the
// tile kernel's FP8_MX_W4 form.  The 8-bit operand's lane group q holds elements [16q, 16q + 16) and [64 + 16q, + 16) of
// the 128, the 4-bit operand's [32q, 32q + 32): the instruction pairs K indices, not lane groups.
struct MxW4DecParams {
    const uint8_t* a;    // x1 [M, K] e4m3, K contiguous
    const uint8_t* b;    // x2 as [N, K / 2] bytes, K contiguous, two e2m1 per byte
    int64_t lda, ldb;    // bytes per row
    const uint8_t* sa;   // e8m0 [M, K / 32], K contiguous
    const uint8_t* sb;   // e8m0 [N, K / 32]
    int64_t sa_rs, sb_rs;
    void* out; int out_dt;
    int64_t M, N, K;
    const void* bias; int bias_dt;
    // K in segments (SEG instantiations, gridDim.y of them): fp32 sums of this pass's rows, slice s at part + s * part_slice
    float* part; int64_t part_slice;
};

// SEG: as in fp8_block_decode_kernel -- gridDim.y segments of NW * NCH chunks, idle waves past the end of K, fp32 sums
// for mxw4dec_reduce_kernel when there is more than one segment.
template <int NW, int NCH, bool SEG = false>
__global__ __launch_bounds__(NW * 64) void mx_a8w4_decode_kernel(MxW4DecParams p)
{
    extern __shared__ __attribute__((aligned(16))) float red[];   // [2][NW][256]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nrow = lane & 15, q = lane >> 4;
    int64_t kbase = (int64_t)wave * (NCH * 128);   // this wave's K range, in elements
    bool live = true;
    if constexpr (SEG) {
        kbase = ((int64_t)blockIdx.y * NW + wave) * (NCH * 128);
        live = kbase < p.K;
        if (!live) kbase = p.K - NCH * 128;
    }
    const int nblocks = (int)((p.N + 15) / 16);
    const int M = (int)p.M;

    // x1: chunk c of this lane's row, bytes [16q, +16) and [64 + 16q, +16) of the chunk's 128; the scale of block q
    v8i xf[NCH];
    int xs[NCH];
#pragma unroll
    for (int c = 0; c < NCH; c++) {
        uint4 lo = make_uint4(0, 0, 0, 0), hi = make_uint4(0, 0, 0, 0);
        uint32_t sw = 0x7f7f7f7fu;
        if (nrow < M) {
            const uint8_t* src = p.a + (int64_t)nrow * p.lda + kbase + 128 * c + 16 * q;
            lo = *(const uint4*)src;
            hi = *(const uint4*)(src + 64);
            sw = *(const uint32_t*)(p.sa + (int64_t)nrow * p.sa_rs + kbase / 32 + 4 * c);
        }
        xf[c] = (v8i){(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
        xs[c] = (int)(sw >> (8 * q));
    }

    auto wload = [&](int rb, int c) {
        const int64_t n = (int64_t)rb * 16 + nrow;
        return *(const uint4*)(p.b + (n < p.N ? n : p.N - 1) * p.ldb + (kbase + 128 * c) / 2 + 16 * q);   // columns past the edge repeat the last one
    };
    // x2's scale bytes: the wave's range is NCH words of four per row; lane (row, q) fetches word 4 i + q (one load
    // instruction per four chunks, 16 rows x one 16-byte run each) and chunk c's word comes over from lane (row, c % 4)
    constexpr int NSW = (NCH + 3) / 4;
    auto sload = [&](int rb, int i) {
        const int64_t n = (int64_t)rb * 16 + nrow;
        const int w = 4 * i + q < NCH ? 4 * i + q : NCH - 1;
        return *(const uint32_t*)(p.sb + (n < p.N ? n : p.N - 1) * p.sb_rs + kbase / 32 + 4 * w);
    };
    int rb = blockIdx.x;
    uint4 wq[NCH];
    uint32_t sq[NSW];
#pragma unroll
    for (int c = 0; c < NCH; c++) wq[c] = wload(rb, c);
#pragma unroll
    for (int i = 0; i < NSW; i++) sq[i] = sload(rb, i);

    for (int it = 0; rb < nblocks; it++, rb += (int)gridDim.x) {
        const int rbn = rb + (int)gridDim.x < nblocks ? rb + (int)gridDim.x : rb;   // past the end: a harmless reload
        const int64_t n0 = (int64_t)rb * 16;
        v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
        uint32_t sws[NCH];
#pragma unroll
        for (int c = 0; c < NCH; c++) sws[c] = (uint32_t)__shfl((int)sq[c / 4], nrow + 16 * (c % 4));
#pragma unroll
        for (int i = 0; i < NSW; i++) sq[i] = sload(rbn, i);
#pragma unroll
        for (int c = 0; c < NCH; c++) {
            const uint4 cur = wq[c];
            const uint32_t sw = sws[c];
            wq[c] = wload(rbn, c);   // the next column block's piece takes the register this one leaves
            const v8i wf = {(int)cur.x, (int)cur.y, (int)cur.z, (int)cur.w, 0, 0, 0, 0};
            acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf[c], acc, 4, 0, 0, (int)(sw >> (8 * q)), 0, xs[c]);
        }
        // acc[r]: m = lane % 16, n = n0 + 4 (lane / 16) + r, over this wave's K range
        if constexpr (SEG) {
            if (!live) acc = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
        }
        float* mine = red + ((it & 1) * NW + wave) * 256;
        *(v4f*)(mine + lane * 4) = acc;
        __syncthreads();
        if (wave != (it & (NW - 1))) continue;
        const float* all = red + (it & 1) * NW * 256 + lane * 4;
        v4f sum = *(const v4f*)all;
#pragma unroll 4
        for (int w = 1; w < NW; w++) {
            const v4f o = *(const v4f*)(all + w * 256);
#pragma unroll
            for (int r = 0; r < 4; r++) sum[r] = sum[r] + o[r];
        }
        if (nrow >= M) continue;
        const int64_t n = n0 + 4 * q;
        if constexpr (SEG) {
            if (gridDim.y > 1) {
                float* dst = p.part + (int64_t)blockIdx.y * p.part_slice + (int64_t)nrow * p.N + n;
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (n + r < p.N) dst[r] = sum[r];
                continue;
            }
        }
        if (p.bias) {
#pragma unroll
            for (int r = 0; r < 4; r++) sum[r] = sum[r] + load_scalar_as_f32(p.bias, p.bias_dt, n + r < p.N ? n + r : p.N - 1);
        }
        const v4us o = p.out_dt == DT_BF16 ? pack4_b16<DT_BF16>(sum) : pack4_b16<DT_F16>(sum);
        uint16_t* dst = (uint16_t*)p.out + (int64_t)nrow * p.N + n;
        if ((p.N % 4) == 0 && ((uintptr_t)p.out % 8) == 0 && n + 3 < p.N) *(v4us*)dst = o;
        else {
#pragma unroll
            for (int r = 0; r < 4; r++)
                if (n + r < p.N) dst[r] = o[r];
        }
    }
}

// out = cast(sum over the K segments, in order, of part[s] + bias) for one pass of up to 16 rows
__global__ __launch_bounds__(256) void mxw4dec_reduce_kernel(MxW4DecParams p, int splits)
{
    const int64_t total = p.M * p.N, stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        float v = p.part[i];
        for (int s = 1; s < splits; s++) v = v + p.part[(int64_t)s * p.part_slice + i];
        if (p.bias) v = v + load_scalar_as_f32(p.bias, p.bias_dt, i % p.N);
        ((uint16_t*)p.out)[i] = p.out_dt == DT_BF16 ? bf16_bits(v) : f16_bits(v);
    }
}

template <int NW, int NCH, bool SEG = false>
int launch_mxw4_one(const MxW4DecParams& p, hipStream_t st, int splits = 1)
{
    if constexpr (!SEG) {
        if (splits > 1 || p.K != (int64_t)NW * NCH * 128) return launch_mxw4_one<NW, NCH, true>(p, st, splits);
    }
    const int64_t nbk = p.K / 128;
    if (splits < 1 || splits > 16 || nbk % NCH != 0 || nbk < NCH || (int64_t)splits * NW * NCH < nbk || (splits > 1 && !p.part)) return -1;
    const int nblocks = (int)((p.N + 15) / 16);
    const int cus = 256 / splits;   // the CUs shared between the segments' workgroup columns
    const int grid = nblocks < cus ? nblocks : cus;
    const size_t lds = (size_t)2 * NW * 256 * sizeof(float);
    hipLaunchKernelGGL((mx_a8w4_decode_kernel<NW, NCH, SEG>), dim3((unsigned)grid, (unsigned)splits), dim3(NW * 64), lds, st, p);
    if (hipError_t e = hipGetLastError(); e != hipSuccess || splits == 1) return (int)e;
    hipLaunchKernelGGL(mxw4dec_reduce_kernel, dim3(splitk_reduce_grid(p.M * p.N)), dim3(256), 0, st, p, splits);
    return (int)hipGetLastError();
}


// ---- MXFP8: fp8 e4m3 x fp8 e4m3 with e8m0 scales per 32 elements of K on both operands (the MX mode of
// quant_batch_matmul_v4, qbmmv4_kernel_golden.py:119-186), up to 16 rows of x1 per pass ----
// The stream of fp8_block_decode_kernel with the scales folded into the widening conversion: an e4m3 value times a power of
// two is a bf16 value (v_cvt_scalef32_pk_bf16_fp8 with the scale 2^(byte - 127): exact wherever fp32 itself would hold the
// scaled value), the product of two bf16 values is an fp32 value, and v_mfma_f32_16x16x32_bf16 sums such products in fp32
// -- one chain over the wave's whole K range, no fold per block.  A lane's 16-byte piece lies inside one 32-element block,
// so one scale byte serves it; x2's scale bytes arrive as words of four (128 elements) per row: lane (row, q) fetches word
// 4 i + q of the wave's range and the word of chunk c comes over from lane (row, (c / 2) % 4).  K segments and idle
// waves as in fp8_block_decode_kernel<..., SEG>.
struct Mx8DecParams {
    const uint8_t* a;    // x1 [M, K] e4m3, K contiguous
    const uint8_t* b;    // x2 as [N, K], K contiguous
    int64_t lda, ldb;
    const uint8_t* sa;   // e8m0 [M, K / 32], K contiguous
    const uint8_t* sb;   // e8m0 [N, K / 32]
    int64_t sa_rs, sb_rs;
    void* out; int out_dt;
    int64_t M, N, K;
    const float* bias;
    float* part; int64_t part_slice;
};

// 8 e4m3 bytes (two dwords) times the scale -> 8 bf16 in byte order
__device__ __forceinline__ v4i widen8_e4m3_bf16(uint32_t d0, uint32_t d1, float sc)
{
    typedef __bf16 b2v __attribute__((ext_vector_type(2)));
    const b2v w0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d0, sc, false), w1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d0, sc, true);
    const b2v w2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d1, sc, false), w3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d1, sc, true);
    return (v4i){(int)__builtin_bit_cast(uint32_t, w0), (int)__builtin_bit_cast(uint32_t, w1), (int)__builtin_bit_cast(uint32_t, w2),
                 (int)__builtin_bit_cast(uint32_t, w3)};
}

template <int NW, int NBLK>
__global__ __launch_bounds__(NW * 64) void mx8_decode_kernel(Mx8DecParams p)
{
    constexpr int NCH = 2 * NBLK;                    // 64-byte chunks of an x2 row in a wave's K range
    constexpr int PF = NW == 16 ? (NCH < 4 ? NCH : 4) : NCH;   // pieces in flight per lane; divides NCH
    constexpr int NSW = (NBLK + 3) / 4;              // scale-word fetches per column block
    static_assert(NCH % PF == 0, "a piece's slot must not depend on the column block");
    extern __shared__ __attribute__((aligned(16))) float red[];   // [2][NW][256]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nrow = lane & 15, q = lane >> 4;
    const int nbk = (int)(p.K / 128);
    int kb0 = ((int)blockIdx.y * NW + wave) * NBLK;
    const bool live = kb0 < nbk;
    if (!live) kb0 = nbk - NBLK;
    const int64_t kbase = (int64_t)kb0 * 128;
    const int nblocks = (int)((p.N + 15) / 16);
    const int M = (int)p.M;

    // x1: lane (m = lane % 16, q) holds, for chunk c and half h, the 8 elements k = kbase + 64 c + 16 q + 8 h .. + 7, scaled
    v4i xf[NCH][2];
#pragma unroll
    for (int c = 0; c < NCH; c++) {
        uint4 raw = make_uint4(0, 0, 0, 0);
        float sc = 1.0f;
        if (nrow < M) {
            raw = *(const uint4*)(p.a + (int64_t)nrow * p.lda + kbase + 64 * c + 16 * q);
            sc = e8m0_to_f32(p.sa[(int64_t)nrow * p.sa_rs + (kbase + 64 * c + 16 * q) / 32]);
        }
        xf[c][0] = widen8_e4m3_bf16(raw.x, raw.y, sc);
        xf[c][1] = widen8_e4m3_bf16(raw.z, raw.w, sc);
    }

    auto wload = [&](int rb, int c) {
        const int64_t n = (int64_t)rb * 16 + nrow;
        return *(const uint4*)(p.b + (n < p.N ? n : p.N - 1) * p.ldb + kbase + 64 * c + 16 * q);   // columns past the edge repeat the last one
    };
    auto sload = [&](int rb, int i) {
        const int64_t n = (int64_t)rb * 16 + nrow;
        const int w = 4 * i + q < NBLK ? 4 * i + q : NBLK - 1;
        return *(const uint32_t*)(p.sb + (n < p.N ? n : p.N - 1) * p.sb_rs + kbase / 32 + 4 * w);
    };
    int rb = blockIdx.x;
    uint4 wq[PF];
    uint32_t sq[NSW];
#pragma unroll
    for (int i = 0; i < PF; i++) wq[i] = wload(rb < nblocks ? rb : nblocks - 1, i);
#pragma unroll
    for (int i = 0; i < NSW; i++) sq[i] = sload(rb < nblocks ? rb : nblocks - 1, i);

    for (int it = 0; rb < nblocks; it++, rb += (int)gridDim.x) {
        const int rbn = rb + (int)gridDim.x < nblocks ? rb + (int)gridDim.x : rb;   // past the end: a harmless reload
        const int64_t n0 = (int64_t)rb * 16;
        uint32_t sws[NBLK];
#pragma unroll
        for (int j = 0; j < NBLK; j++) sws[j] = (uint32_t)__shfl((int)sq[j / 4], nrow + 16 * (j % 4));
#pragma unroll
        for (int i = 0; i < NSW; i++) sq[i] = sload(rbn, i);
        v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int c = 0; c < NCH; c++) {
            const uint4 cur = wq[c % PF];
            wq[c % PF] = c + PF < NCH ? wload(rb, c + PF) : wload(rbn, c + PF - NCH);
            const float sc = e8m0_to_f32((sws[c / 2] >> (8 * (2 * (c % 2) + (q >> 1)))) & 0xffu);
            const v4i w0 = widen8_e4m3_bf16(cur.x, cur.y, sc), w1 = widen8_e4m3_bf16(cur.z, cur.w, sc);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, w0), __builtin_bit_cast(v8bf, xf[c][0]), acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, w1), __builtin_bit_cast(v8bf, xf[c][1]), acc, 0, 0, 0);
        }
        // acc[r]: m = lane % 16, n = n0 + 4 (lane / 16) + r, over this wave's K range
        if (!live) acc = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
        float* mine = red + ((it & 1) * NW + wave) * 256;
        *(v4f*)(mine + lane * 4) = acc;
        __syncthreads();
        if (wave != (it & (NW - 1))) continue;
        const float* all = red + (it & 1) * NW * 256 + lane * 4;
        v4f sum = *(const v4f*)all;
#pragma unroll 4
        for (int w = 1; w < NW; w++) {
            const v4f o = *(const v4f*)(all + w * 256);
#pragma unroll
            for (int r = 0; r < 4; r++) sum[r] = sum[r] + o[r];
        }
        if (nrow >= M) continue;
        const int64_t n = n0 + 4 * q;
        if (gridDim.y > 1) {
            float* dst = p.part + (int64_t)blockIdx.y * p.part_slice + (int64_t)nrow * p.N + n;
#pragma unroll
            for (int r = 0; r < 4; r++)
                if (n + r < p.N) dst[r] = sum[r];
            continue;
        }
        if (p.bias) {
#pragma unroll
            for (int r = 0; r < 4; r++) sum[r] = sum[r] + p.bias[n + r < p.N ? n + r : p.N - 1];
        }
        if (p.out_dt == DT_F32) {
            float* dst = (float*)p.out + (int64_t)nrow * p.N + n;
#pragma unroll
            for (int r = 0; r < 4; r++)
                if (n + r < p.N) dst[r] = sum[r];
        } else {
            const v4us o = p.out_dt == DT_BF16 ? pack4_b16<DT_BF16>(sum) : pack4_b16<DT_F16>(sum);
            uint16_t* dst = (uint16_t*)p.out + (int64_t)nrow * p.N + n;
            if ((p.N % 4) == 0 && ((uintptr_t)p.out % 8) == 0 && n + 3 < p.N) *(v4us*)dst = o;
            else {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (n + r < p.N) dst[r] = o[r];
            }
        }
    }
}

// out = cast(sum over the K segments, in order, of part[s] + bias) for one pass of up to 16 rows
__global__ __launch_bounds__(256) void mx8dec_reduce_kernel(Mx8DecParams p, int splits)
{
    const int64_t total = p.M * p.N, stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        float v = p.part[i];
        for (int s = 1; s < splits; s++) v = v + p.part[(int64_t)s * p.part_slice + i];
        if (p.bias) v = v + p.bias[i % p.N];
        if (p.out_dt == DT_F32) ((float*)p.out)[i] = v;
        else ((uint16_t*)p.out)[i] = p.out_dt == DT_BF16 ? bf16_bits(v) : f16_bits(v);
    }
}

template <int NW, int NBLK>
int launch_mx8_one(const Mx8DecParams& p, hipStream_t st, int splits)
{
    const int64_t nbk = p.K / 128;
    if (splits < 1 || splits > 16 || nbk % NBLK != 0 || nbk < NBLK || (int64_t)splits * NW * NBLK < nbk || (splits > 1 && !p.part)) return -1;
    const int nblocks = (int)((p.N + 15) / 16);
    const int cus = 256 / splits;   // the CUs shared between the segments' workgroup columns
    const int grid = nblocks < cus ? nblocks : cus;
    const size_t lds = (size_t)2 * NW * 256 * sizeof(float);
    hipLaunchKernelGGL((mx8_decode_kernel<NW, NBLK>), dim3((unsigned)grid, (unsigned)splits), dim3(NW * 64), lds, st, p);
    if (hipError_t e = hipGetLastError(); e != hipSuccess || splits == 1) return (int)e;
    hipLaunchKernelGGL(mx8dec_reduce_kernel, dim3(splitk_reduce_grid(p.M * p.N)), dim3(256), 0, st, p, splits);
    return (int)hipGetLastError();
}

}  // namespace

// fp8 e4m3 block scales (or int8 per-tile: the same scales, an fp32 bias, 16-bit output) with up to 32 rows of x1 (two
// passes beyond 16), K-contiguous operands, K a whole number of 128-element blocks as qmm_decode_plan lays them out (more
// than one segment only with room for the partial sums in sk); OPSNN_NOT_TAKEN otherwise.
int launch_blockscale_decode(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk)
{
    const bool i8 = a.x1_dtype == DT_I8 && a.x2_dtype == DT_I8;
    if ((!i8 && (a.x1_dtype != DT_E4M3 || a.x2_dtype != DT_E4M3)) || a.batch != 1) return OPSNN_NOT_TAKEN;
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16 && !(a.out_dtype == DT_F32 && !i8)) return OPSNN_NOT_TAKEN;
    if (a.bias && !(i8 && a.bias_dtype == DT_F32)) return OPSNN_NOT_TAKEN;
    // (int8: 17 .. 32 rows are one pass of the tile kernel with K split, ahead of two passes here: 32 x 18432 x 7168 66 us here, 42 there)
    if (a.M > (i8 ? 16 : 32) || a.N < 256) return OPSNN_NOT_TAKEN;
    if (a.gsK != 128 || a.gsN != 128 || (a.gsM != 1 && a.gsM != 128)) return OPSNN_NOT_TAKEN;
    if (a.K % 128 != 0 || a.x1.col_stride != 1 || a.x2.row_stride != 1) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)a.x1.ptr | (uintptr_t)a.x2.ptr | (uint64_t)a.x1.row_stride | (uint64_t)a.x2.col_stride) % 16) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)a.x1_scale_mat.ptr | (uintptr_t)a.x2_scale_mat.ptr) % 4) return OPSNN_NOT_TAKEN;
    if (a.x1.row_stride < a.K || a.x2.col_stride < a.K) return OPSNN_NOT_TAKEN;
    QmmDecodePlan pl;
    if (!qmm_decode_plan(a.K, sk.part != nullptr, pl) || pl.splits > (sk.part ? sk.splits : 1)) return OPSNN_NOT_TAKEN;
    for (int64_t m0 = 0; m0 < a.M; m0 += 16) {
        Fp8DecParams p{};
        p.M = a.M - m0 < 16 ? a.M - m0 : 16; p.N = a.N; p.K = a.K;
        p.a = (const uint8_t*)a.x1.ptr + m0 * a.x1.row_stride; p.b = (const uint8_t*)a.x2.ptr;
        p.lda = a.x1.row_stride; p.ldb = a.x2.col_stride;
        p.out_dt = a.out_dtype;
        p.out = (char*)a.out + m0 * a.N * (a.out_dtype == DT_F32 ? 4 : 2);
        p.part = sk.part ? sk.part + m0 * a.N : nullptr; p.part_slice = a.M * a.N;
        p.gsM = (int)a.gsM;
        // gsM 1: the pass's own rows of the scale table; gsM 128: up to 32 rows share row 0
        p.s1 = (const float*)a.x1_scale_mat.ptr + (a.gsM == 1 ? m0 * a.x1_scale_mat.row_stride : 0);
        p.s1_rs = a.x1_scale_mat.row_stride; p.s1_cs = a.x1_scale_mat.col_stride;
        p.s2 = (const float*)a.x2_scale_mat.ptr; p.s2_rs = a.x2_scale_mat.row_stride; p.s2_cs = a.x2_scale_mat.col_stride;
        p.bias = (const float*)a.bias;
        const int rc = i8 ? launch_decode_split<false, true>(p, pl.nw, pl.nblk, st, pl.splits) : launch_decode_split<false>(p, pl.nw, pl.nblk, st, pl.splits);
        if (rc != 0) return rc;
    }
    return 0;
}

// fp8 e4m3 with one fp32 scale per row of x1 (or one) and one per column of x2 (or one), optional fp32 bias -- the form
// (sum * x2Scale) * x1Scale + bias of compute_pertoken (qbmmv3_kernel_golden.py:361-387) -- for up to 32 rows.
int launch_rowcol_decode(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk)
{
    if (a.x1_dtype != DT_E4M3 || a.x2_dtype != DT_E4M3 || a.batch != 1) return OPSNN_NOT_TAKEN;
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16 && a.out_dtype != DT_F32) return OPSNN_NOT_TAKEN;
    if (!a.x1_scale || !a.x2_scale || a.x2_scale_dtype != DT_F32 || (a.bias && a.bias_dtype != DT_F32)) return OPSNN_NOT_TAKEN;
    if (a.M > 32 || a.N < 256 || a.x1.col_stride != 1 || a.x2.row_stride != 1) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)a.x1.ptr | (uintptr_t)a.x2.ptr | (uint64_t)a.x1.row_stride | (uint64_t)a.x2.col_stride) % 16) return OPSNN_NOT_TAKEN;
    if (a.x1.row_stride < a.K || a.x2.col_stride < a.K) return OPSNN_NOT_TAKEN;
    QmmDecodePlan pl;
    if (!qmm_decode_plan(a.K, sk.part != nullptr, pl) || pl.splits > (sk.part ? sk.splits : 1)) return OPSNN_NOT_TAKEN;
    for (int64_t m0 = 0; m0 < a.M; m0 += 16) {
        Fp8DecParams p{};
        p.M = a.M - m0 < 16 ? a.M - m0 : 16; p.N = a.N; p.K = a.K;
        p.a = (const uint8_t*)a.x1.ptr + m0 * a.x1.row_stride; p.b = (const uint8_t*)a.x2.ptr;
        p.lda = a.x1.row_stride; p.ldb = a.x2.col_stride;
        p.out_dt = a.out_dtype;
        p.out = (char*)a.out + m0 * a.N * (a.out_dtype == DT_F32 ? 4 : 2);
        p.rs_stride = a.x1_scale_len == 1 ? 0 : 1; p.cs_stride = a.x2_scale_len == 1 ? 0 : 1;
        p.rs = (const float*)a.x1_scale + (p.rs_stride ? m0 : 0);
        p.cs = (const float*)a.x2_scale; p.bias = (const float*)a.bias;
        p.part = sk.part ? sk.part + m0 * a.N : nullptr; p.part_slice = a.M * a.N;
        const int rc = launch_decode_split<true>(p, pl.nw, pl.nblk, st, pl.splits);
        if (rc != 0) return rc;
    }
    return 0;
}

// fp8 x fp4 MX with up to 32 rows of x1 (two passes beyond 16): K a whole number of 128-element chunks that 16 waves
// share 2 or 4 each, or 8 waves 1 .. 7 each; K-contiguous operands and scales; OPSNN_NOT_TAKEN otherwise.
int launch_mx_a8w4_decode(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk)
{
    if (a.x1_dtype != DT_E4M3 || a.x2_dtype != DT_E2M1 || a.batch != 1) return OPSNN_NOT_TAKEN;
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16) return OPSNN_NOT_TAKEN;
    // (17 rows and more: one pass of the tile kernel with K split, ahead of two passes here)
    if (a.M > 16 || a.N < 256 || a.K % 128 != 0 || a.x1.col_stride != 1 || a.x2.row_stride != 1 || a.x2.col_stride % 2) return OPSNN_NOT_TAKEN;
    if (a.x1_scale_mat.col_stride != 2 || a.x2_scale_mat.col_stride != 2) return OPSNN_NOT_TAKEN;   // [rows, K / 64, 2]: a row's bytes contiguous
    if (a.bias && a.bias_dtype != DT_F32 && a.bias_dtype != DT_BF16 && a.bias_dtype != DT_F16) return OPSNN_NOT_TAKEN;
    const int64_t ldb = a.x2.col_stride / 2;
    if (a.x1.row_stride < a.K || ldb < a.K / 2) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)a.x1.ptr | (uintptr_t)a.x2.ptr | (uint64_t)a.x1.row_stride | (uint64_t)ldb) % 16) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)a.x1_scale_mat.ptr | (uintptr_t)a.x2_scale_mat.ptr | (uint64_t)a.x1_scale_mat.row_stride | (uint64_t)a.x2_scale_mat.row_stride) % 4)
        return OPSNN_NOT_TAKEN;
    if (a.x1_scale_mat.row_stride < a.K / 32 || a.x2_scale_mat.row_stride < a.K / 32) return OPSNN_NOT_TAKEN;
    QmmDecodePlan pl;
    if (!qmm_decode_plan(a.K, sk.part != nullptr, pl, true) || pl.splits > (sk.part ? sk.splits : 1)) return OPSNN_NOT_TAKEN;
    const int nw = pl.nw, nch = pl.nblk, splits = pl.splits;
    for (int64_t m0 = 0; m0 < a.M; m0 += 16) {
        MxW4DecParams p{};
        p.M = a.M - m0 < 16 ? a.M - m0 : 16; p.N = a.N; p.K = a.K;
        p.a = (const uint8_t*)a.x1.ptr + m0 * a.x1.row_stride; p.b = (const uint8_t*)a.x2.ptr;
        p.lda = a.x1.row_stride; p.ldb = ldb;
        p.sa = (const uint8_t*)a.x1_scale_mat.ptr + m0 * a.x1_scale_mat.row_stride; p.sb = (const uint8_t*)a.x2_scale_mat.ptr;
        p.sa_rs = a.x1_scale_mat.row_stride; p.sb_rs = a.x2_scale_mat.row_stride;
        p.out_dt = a.out_dtype; p.out = (char*)a.out + m0 * a.N * 2;
        p.bias = a.bias; p.bias_dt = a.bias_dtype;
        p.part = sk.part ? sk.part + m0 * a.N : nullptr; p.part_slice = a.M * a.N;
        int rc = -1;
        if (nw == 16) rc = nch == 2 ? launch_mxw4_one<16, 2>(p, st, splits) : nch == 4 ? launch_mxw4_one<16, 4>(p, st, splits) : -1;
        else switch (nch) {
            case 1: rc = launch_mxw4_one<8, 1>(p, st, splits); break;
            case 2: rc = launch_mxw4_one<8, 2>(p, st, splits); break;
            case 3: rc = launch_mxw4_one<8, 3>(p, st, splits); break;
            case 4: rc = launch_mxw4_one<8, 4>(p, st, splits); break;
            case 5: rc = launch_mxw4_one<8, 5>(p, st, splits); break;
            case 6: rc = launch_mxw4_one<8, 6>(p, st, splits); break;
            case 7: rc = launch_mxw4_one<8, 7>(p, st, splits); break;
            default: break;
        }
        if (rc != 0) return rc;
    }
    return 0;
}

// MXFP8 with up to 32 rows of x1 (two passes beyond 16): K-contiguous operands and scale rows ([rows, K / 64, 2] bytes), K a
// whole number of 128-element blocks as qmm_decode_plan lays them out; OPSNN_NOT_TAKEN otherwise.
int launch_mxfp8_decode(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk)
{
    if (a.x1_dtype != DT_E4M3 || a.x2_dtype != DT_E4M3 || a.batch != 1) return OPSNN_NOT_TAKEN;
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16 && a.out_dtype != DT_F32) return OPSNN_NOT_TAKEN;
    if (a.M > 32 || a.N < 256 || a.K % 128 != 0 || a.x1.col_stride != 1 || a.x2.row_stride != 1) return OPSNN_NOT_TAKEN;
    if (a.x1_scale_mat.col_stride != 2 || a.x2_scale_mat.col_stride != 2) return OPSNN_NOT_TAKEN;   // [rows, K / 64, 2]: a row's bytes contiguous
    if (a.bias && a.bias_dtype != DT_F32) return OPSNN_NOT_TAKEN;
    if (a.x1.row_stride < a.K || a.x2.col_stride < a.K) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)a.x1.ptr | (uintptr_t)a.x2.ptr | (uint64_t)a.x1.row_stride | (uint64_t)a.x2.col_stride) % 16) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)a.x2_scale_mat.ptr | (uint64_t)a.x2_scale_mat.row_stride) % 4) return OPSNN_NOT_TAKEN;
    if (a.x1_scale_mat.row_stride < a.K / 32 || a.x2_scale_mat.row_stride < a.K / 32) return OPSNN_NOT_TAKEN;
    QmmDecodePlan pl;
    if (!qmm_decode_plan(a.K, sk.part != nullptr, pl) || pl.splits > (sk.part ? sk.splits : 1)) return OPSNN_NOT_TAKEN;
    for (int64_t m0 = 0; m0 < a.M; m0 += 16) {
        Mx8DecParams p{};
        p.M = a.M - m0 < 16 ? a.M - m0 : 16; p.N = a.N; p.K = a.K;
        p.a = (const uint8_t*)a.x1.ptr + m0 * a.x1.row_stride; p.b = (const uint8_t*)a.x2.ptr;
        p.lda = a.x1.row_stride; p.ldb = a.x2.col_stride;
        p.sa = (const uint8_t*)a.x1_scale_mat.ptr + m0 * a.x1_scale_mat.row_stride; p.sb = (const uint8_t*)a.x2_scale_mat.ptr;
        p.sa_rs = a.x1_scale_mat.row_stride; p.sb_rs = a.x2_scale_mat.row_stride;
        p.out_dt = a.out_dtype; p.out = (char*)a.out + m0 * a.N * (a.out_dtype == DT_F32 ? 4 : 2);
        p.bias = (const float*)a.bias;
        p.part = sk.part ? sk.part + m0 * a.N : nullptr; p.part_slice = a.M * a.N;
        int rc = -1;
        if (pl.nw == 16) rc = pl.nblk == 1 ? launch_mx8_one<16, 1>(p, st, pl.splits) : pl.nblk == 2 ? launch_mx8_one<16, 2>(p, st, pl.splits)
                              : pl.nblk == 4 ? launch_mx8_one<16, 4>(p, st, pl.splits) : -1;
        else switch (pl.nblk) {
            case 1: rc = launch_mx8_one<8, 1>(p, st, pl.splits); break;
            case 2: rc = launch_mx8_one<8, 2>(p, st, pl.splits); break;
            case 3: rc = launch_mx8_one<8, 3>(p, st, pl.splits); break;
            case 4: rc = launch_mx8_one<8, 4>(p, st, pl.splits); break;
            case 5: rc = launch_mx8_one<8, 5>(p, st, pl.splits); break;
            case 6: rc = launch_mx8_one<8, 6>(p, st, pl.splits); break;
            case 7: rc = launch_mx8_one<8, 7>(p, st, pl.splits); break;
            default: break;
        }
        if (rc != 0) return rc;
    }
    return 0;
}

}  // namespace opsnn
