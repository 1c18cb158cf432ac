// int4 x int4 with one fp32 scale and one fp16 offset of x2 per group of 256 K elements and column, one fp32 scale of
// x1 per row ("K-G" of quant_batch_matmul_v4), on the matrix cores.
//
//   out[m,n] = cast( x1s[m] * sum_g ( fp32(sum_{k in g} x1*x2) - fp32(sum_{k in g} x1) * fp32(off[g,n]) ) * s2[g,n] )
//
// Formula and operation order: matmul/quant_batch_matmul_v4/tests/assets/qbmmv4_kernel_golden.py:328-395.  The integer
// sums of a group are exact (at most 256 products of magnitude 64), so the result is the golden's bit for bit whatever
// the order inside a group; the groups are folded in ascending order with separately rounded fp32 operations.
//
// This chip has no 4-bit integer matrix instruction.  Every int4 value is an fp8 e4m3 value, the products (magnitude at
// most 64) and a group's sum (at most 16384) are small integers, and v_mfma_f32_16x16x128_f8f6f4 adds them without
// loss, so the group sum leaves the matrix pipe as the fp32 the fold needs and no conversion is spent on it.
//
// A pre-step writes both operands as e4m3 bytes into the workspace, zero-padded to whole tiles (rows to 128, K to 256)
// and stored block by block: the 128 rows x 256 bytes of one tile and group, followed by 1 KiB of that group's fp32
// side values (x1: the negated row sums; x2: scales, then offsets), are one contiguous block that already is the LDS
// image (16-byte chunks of a row xor-swizzled by the row, so that fragment reads are free of bank conflicts).  The
// matrix kernel fetches a block with linear 16-byte asynchronous copies: consecutive addresses spread over all memory
// channels (rows 4096 bytes apart would all fall into one), and the side values arrive in LDS with the tile instead of
// costing every wave eight vector loads per group.
//
// The matrix kernel: 128 x 128 output tile per workgroup, eight waves of 64 x 32 (4 x 2 fragments of 16 x 16), one K
// tile = one group, two matrix instructions per fragment pair from a zero accumulator, then the fold on the vector
// ALU, three operations per output and group:  sum += fma(-rowsum, off, t) * s2.  The product rowsum * off is exact in
// fp32 (an integer of magnitude at most 2048 times an fp16 value has at most 22 significant bits), so the fused form
// rounds exactly where the golden's separate subtraction does.  A wave issues in order, so the three kinds of work
// are interleaved in the source: the copies of group g + 1 (into the other of two LDS buffers) go out between the
// matrix instructions of group g, and the fold of group g - 1 fills the vector ALU meanwhile; one barrier per group.
#include "launch.h"
#include "qgemm_core.hip.h"

namespace opsnn {
namespace {

constexpr int64_t KG_GROUP = 256, KG_TILE = 128;
constexpr int64_t KG_ROWS = KG_TILE * KG_GROUP, KG_BLOCK = KG_ROWS + 1024;   // operand bytes of one tile and group; with its side values
inline int64_t kg_rup(int64_t v, int64_t m) { return (v + m - 1) / m * m; }
inline uint64_t kg_a256(uint64_t v) { return (v + 255) / 256 * 256; }

struct KgLayout {
    int64_t Mp, Np, Kp, G;
    uint64_t o_b, total;   // byte offset of the x2 blocks in the workspace (the x1 blocks sit at 0)
};

bool kg_layout(const OpsnnQmmArgs& a, KgLayout& L)
{
    if (a.x1_dtype != DT_I4 || a.x2_dtype != DT_I4 || a.batch != 1 || a.gsK != KG_GROUP) return false;
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16) return false;
    if (!a.x1_scale || !a.x2_scale_mat.ptr || !a.x2_offset_mat.ptr || a.bias) return false;
    // both operands K-contiguous with rows that start on a byte
    if (a.x1.col_stride != 1 || a.x1.row_stride % 2 != 0 || a.x1.row_stride < a.K) return false;
    if (a.x2.row_stride != 1 || a.x2.col_stride % 2 != 0 || a.x2.col_stride < a.K) return false;
    if (a.K % 2 != 0 || a.M * a.N < 32 * 32) return false;
    L.Mp = kg_rup(a.M, KG_TILE); L.Np = kg_rup(a.N, KG_TILE); L.Kp = kg_rup(a.K, KG_GROUP); L.G = L.Kp / KG_GROUP;
    L.o_b = (uint64_t)(L.Mp / KG_TILE * L.G * KG_BLOCK);
    L.total = L.o_b + (uint64_t)(L.Np / KG_TILE * L.G * KG_BLOCK);
    return true;
}

// 16 int4 (8 bytes) of row r -> 16 e4m3 bytes in the block layout; rows past `rows` and columns past K become zero.
// ld: elements between rows.  WITH_RS: the block's first side value array gets -fp32(sum of the row over the group)
// (exact: at most 256 values of magnitude 8); the 16 threads of one row and group are neighbours in one wave.
template <bool WITH_RS>
__global__ __launch_bounds__(256) void kg_widen_kernel(const uint8_t* __restrict__ src, int64_t rows, int64_t K, int64_t ld,
                                                       int8_t* __restrict__ dst, int64_t rows_p, int64_t Kp, int64_t G)
{
    const int64_t per_row = Kp / 16;   // a multiple of 16; rows_p * per_row is a multiple of the block size
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= rows_p * per_row) return;
    const int64_t r = idx / per_row, kc = idx - r * per_row, k0 = kc * 16;
    uint64_t nib = 0;   // 16 nibbles, element k0 + e in bits [4 e, 4 e + 4)
    if (r < rows && k0 < K) {
        const uint8_t* p = src + ((r * ld + k0) >> 1);   // ld and k0 are even: the row piece starts on a byte
        if (k0 + 16 <= K && ((uintptr_t)p & 7) == 0) nib = *(const uint64_t*)p;
        else {
#pragma unroll
            for (int b = 0; b < 8; b++)
                if (k0 + 2 * b < K) nib |= (uint64_t)p[b] << (8 * b);   // K is even: both nibbles of the byte are inside the row
        }
    }
    // e4m3 of the two's-complement nibble n: 0..7 -> 0, 1, 2, ... 7; 8..15 -> -8, -7, ... -1
    constexpr uint64_t POS = 0x4E4C4A4844403800ull, NEG = 0xB8C0C4C8CACCCED0ull;
    uint32_t o[4] = {0, 0, 0, 0};
    int32_t s = 0;
#pragma unroll
    for (int e = 0; e < 16; e++) {
        const uint32_t n = (uint32_t)(nib >> (4 * e)) & 15u;
        const uint32_t f = (uint32_t)(((n & 8u) ? NEG : POS) >> (8 * (n & 7u))) & 0xffu;
        o[e / 4] |= f << (8 * (e % 4));
        s += (int32_t)(n ^ 8u) - 8;
    }
    const int64_t g = kc >> 4, c = kc & 15;
    int8_t* block = dst + ((r >> 7) * G + g) * KG_BLOCK;
    *(uint4*)(block + ((r & 127) << 8) + ((c ^ (r & 15)) << 4)) = make_uint4(o[0], o[1], o[2], o[3]);
    if (WITH_RS) {
#pragma unroll
        for (int d = 8; d >= 1; d >>= 1) s += __shfl_xor(s, d, 16);
        if (c == 0) ((float*)(block + KG_ROWS))[r & 127] = -(float)s;
    }
}

// fp32 scale[g, n] and offset[g, n] into the side values of the x2 blocks (zeros for padded columns and groups)
__global__ __launch_bounds__(256) void kg_scales_kernel(OpsnnMat sc, OpsnnMat of, int64_t N, int64_t Np, int64_t G, int64_t Greal, int8_t* __restrict__ dst)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= G * Np) return;
    const int64_t g = idx / Np, n = idx - g * Np;
    float s = 0.0f, o = 0.0f;
    if (n < N && g < Greal) {
        s = ((const float*)sc.ptr)[g * sc.row_stride + n * sc.col_stride];
        o = load_scalar_as_f32(of.ptr, DT_F16, g * of.row_stride + n * of.col_stride);
    }
    float* side = (float*)(dst + ((n >> 7) * G + g) * KG_BLOCK + KG_ROWS);
    side[n & 127] = s;
    side[128 + (n & 127)] = o;
}

template <int OUT_DT>
__global__ __launch_bounds__(512) void kg_gemm_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ B, const float* __restrict__ x1s,
                                                      uint16_t* __restrict__ out, int64_t M, int64_t N, int G)
{
    constexpr int FM = 4, FN = 2;
    constexpr int ROWS = (int)KG_ROWS, BLOCK = (int)KG_BLOCK, BUF = 2 * BLOCK;   // LDS: two buffers of an x1 block and an x2 block
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2, wn = wave & 3;
    const int frow = lane & 15, fq = lane >> 4;
    const int m0 = blockIdx.y * 128, n0 = blockIdx.x * 128;

    // Copies of one group: eight per wave for the operand rows (copy c of the workgroup's 2 x 4 moves 8 KiB, this
    // wave's share is 1 KiB of it), and waves 0 and 1 move the side values of the x1 and the x2 block.
    const int8_t* ga = A + (int64_t)blockIdx.y * G * BLOCK;
    const int8_t* gb = B + (int64_t)blockIdx.x * G * BLOCK;
    auto copy_rows = [&](int g, int buf, int c) {   // c = 0..7, compile-time after unrolling
        const int8_t* src = (c < 4 ? ga : gb) + (int64_t)g * BLOCK + (c & 3) * 8192 + tid * 16;
        async_copy16_uncounted(src, lds + buf * BUF + (c < 4 ? 0 : BLOCK) + (c & 3) * 8192 + wave * 1024);
    };
    auto copy_side = [&](int g, int buf) {
        if (wave < 2) {
            const int8_t* src = (wave == 0 ? ga : gb) + (int64_t)g * BLOCK + ROWS + lane * 16;
            async_copy16_uncounted(src, lds + buf * BUF + wave * BLOCK + ROWS);
        }
    };

    v4f sum[FN][FM], tp[FN][FM];   // running sums; the previous group's integer sums, folded while this group is multiplied
    float rsp[FM];
    v4f s2q[FN], ofq[FN];
#pragma unroll
    for (int i = 0; i < FN; i++) {
        s2q[i] = ofq[i] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < FM; j++) sum[i][j] = tp[i][j] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for (int j = 0; j < FM; j++) rsp[j] = 0.0f;
    auto fold = [&](int i, int j) {
#pragma unroll
        for (int r = 0; r < 4; r++) sum[i][j][r] = sum[i][j][r] + __builtin_fmaf(rsp[j], ofq[i][r], tp[i][j][r]) * s2q[i][r];
    };

#pragma unroll
    for (int c = 0; c < 8; c++) copy_rows(0, 0, c);
    copy_side(0, 0);
    for (int g = 0; g < G; g++) {
        // this wave's copies of group g have landed; behind the barrier everybody's have, and every wave has finished
        // its reads of the other buffer (group g - 1)
        wait_vmcnt<0>();
        __syncthreads();
        const int buf = g & 1;
        const bool more = g + 1 < G;
        const char* la = lds + buf * BUF + (wm * 64 + frow) * 256;
        const char* lb = lds + buf * BUF + BLOCK + (wn * 32 + frow) * 256;
        // this group's side values, for its fold during the next group (by then the buffer is being refilled)
        float rsv[FM];
        v4f s2v[FN], ofv[FN];
#pragma unroll
        for (int j = 0; j < FM; j++) rsv[j] = *(const float*)(lds + buf * BUF + ROWS + (wm * 64 + 16 * j + frow) * 4);
#pragma unroll
        for (int i = 0; i < FN; i++) {
            const char* sv = lds + buf * BUF + BLOCK + ROWS + (wn * 32 + 16 * i + 4 * fq) * 4;
            s2v[i] = *(const v4f*)sv;
            ofv[i] = *(const v4f*)(sv + 512);
        }
        if (more) copy_side(g + 1, buf ^ 1);
        v4f t[FN][FM];
#pragma unroll
        for (int s = 0; s < 2; s++) {
            // lane (row, q) holds bytes [128 s + 32 q, + 32) of its row: the same K for both operands
            const int p0 = ((8 * s + 2 * fq) ^ frow) << 4, p1 = ((8 * s + 2 * fq + 1) ^ frow) << 4;
            v8i fa[FM], fb[FN];
#pragma unroll
            for (int j = 0; j < FM; j++) {
                const v4i lo = *(const v4i*)(la + j * 16 * 256 + p0), hi = *(const v4i*)(la + j * 16 * 256 + p1);
                fa[j] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
#pragma unroll
            for (int i = 0; i < FN; i++) {
                const v4i lo = *(const v4i*)(lb + i * 16 * 256 + p0), hi = *(const v4i*)(lb + i * 16 * 256 + p1);
                fb[i] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
            if (more) {
#pragma unroll
                for (int c = 0; c < 4; c++) copy_rows(g + 1, buf ^ 1, 4 * s + c);
            }
#pragma unroll
            for (int i = 0; i < FN; i++)
#pragma unroll
                for (int j = 0; j < FM; j++) {
                    t[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[i], fa[j], s == 0 ? (v4f){0.0f, 0.0f, 0.0f, 0.0f} : t[i][j], 0, 0, 0,
                                                                               0x7f7f7f7f, 0, 0x7f7f7f7f);
                    if (i == s) fold(i, j);   // half of the previous group's fold in the shadow of each step
                }
        }
        // t[i][j][r] is the group's integer sum for m = 16 j + lane % 16, n = 16 i + 4 (lane / 16) + r of the wave tile
#pragma unroll
        for (int i = 0; i < FN; i++) {
            s2q[i] = s2v[i];
            ofq[i] = ofv[i];
#pragma unroll
            for (int j = 0; j < FM; j++) tp[i][j] = t[i][j];
        }
#pragma unroll
        for (int j = 0; j < FM; j++) rsp[j] = rsv[j];
    }
#pragma unroll
    for (int i = 0; i < FN; i++)
#pragma unroll
        for (int j = 0; j < FM; j++) fold(i, j);

    const bool vec_ok = (N % 4) == 0 && ((uintptr_t)out % 8) == 0;
#pragma unroll
    for (int j = 0; j < FM; j++) {
        const int64_t m = m0 + wm * 64 + 16 * j + frow;
        if (m >= M) continue;
        const float s1 = x1s[m];
#pragma unroll
        for (int i = 0; i < FN; i++) {
            const int64_t n = n0 + wn * 32 + 16 * i + 4 * fq;
            v4f v = sum[i][j];
#pragma unroll
            for (int r = 0; r < 4; r++) v[r] = v[r] * s1;
            const v4us o = pack4_b16<OUT_DT>(v);
            if (vec_ok && n + 3 < N) *(v4us*)(out + m * N + n) = o;
            else {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (n + r < N) out[m * N + n + r] = o[r];
            }
        }
    }
}

}  // namespace

uint64_t kg_workspace_bytes(const OpsnnQmmArgs& a)
{
    KgLayout L;
    return kg_layout(a, L) ? L.total : 0;
}

int launch_kg_mfma(const OpsnnQmmArgs& a, hipStream_t st)
{
    KgLayout L;
    if (!kg_layout(a, L) || !a.workspace || (uintptr_t)a.workspace % 16 != 0) return OPSNN_NOT_TAKEN;
    int8_t* a8 = (int8_t*)a.workspace;
    int8_t* b8 = a8 + L.o_b;
    const int64_t Greal = (a.K + KG_GROUP - 1) / KG_GROUP;
    auto blocks = [](int64_t n) { return dim3((unsigned)((n + 255) / 256)); };
    hipLaunchKernelGGL(kg_widen_kernel<true>, blocks(L.Mp * (L.Kp / 16)), dim3(256), 0, st, (const uint8_t*)a.x1.ptr, a.M, a.K, a.x1.row_stride, a8, L.Mp,
                       L.Kp, L.G);
    hipLaunchKernelGGL(kg_widen_kernel<false>, blocks(L.Np * (L.Kp / 16)), dim3(256), 0, st, (const uint8_t*)a.x2.ptr, a.N, a.K, a.x2.col_stride, b8, L.Np,
                       L.Kp, L.G);
    hipLaunchKernelGGL(kg_scales_kernel, blocks(L.G * L.Np), dim3(256), 0, st, a.x2_scale_mat, a.x2_offset_mat, a.N, L.Np, L.G, Greal, b8);
    const dim3 grid((unsigned)(L.Np / KG_TILE), (unsigned)(L.Mp / KG_TILE));
    constexpr int KG_LDS = 2 * 2 * (int)KG_BLOCK;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kg_gemm_kernel<DT_BF16>, hipFuncAttributeMaxDynamicSharedMemorySize, KG_LDS);
        if (e == hipSuccess) e = hipFuncSetAttribute((const void*)kg_gemm_kernel<DT_F16>, hipFuncAttributeMaxDynamicSharedMemorySize, KG_LDS);
        if (e != hipSuccess) return (int)e;
        attr_set = true;
    }
    if (a.out_dtype == DT_BF16)
        hipLaunchKernelGGL(kg_gemm_kernel<DT_BF16>, grid, dim3(512), KG_LDS, st, a8, b8, (const float*)a.x1_scale, (uint16_t*)a.out, a.M, a.N, (int)L.G);
    else
        hipLaunchKernelGGL(kg_gemm_kernel<DT_F16>, grid, dim3(512), KG_LDS, st, a8, b8, (const float*)a.x1_scale, (uint16_t*)a.out, a.M, a.N, (int)L.G);
    return (int)hipGetLastError();
}

}  // namespace opsnn
