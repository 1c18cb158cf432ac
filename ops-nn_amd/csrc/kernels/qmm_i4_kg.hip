// int4 x int4 with one fp32 scale and one fp16 offset of x2 per group of 256 K elements and column, one fp32 scale of
// x1 per row ("K-G" of quant_batch_matmul_v4), on the matrix cores.
//
//   out[m,n] = cast( x1s[m] * sum_g ( fp32(sum_{k in g} x1*x2) - fp32(sum_{k in g} x1) * fp32(off[g,n]) ) * s2[g,n] )
//
// Formula and operation order: matmul/quant_batch_matmul_v4/tests/assets/qbmmv4_kernel_golden.py:328-395.  The integer
// sums of a group are exact (at most 256 products of magnitude 64), so the result is the golden's bit for bit whatever
// the order inside a group; the groups are folded in ascending order with separately rounded fp32 operations.
//
// This chip has no 4-bit integer matrix instruction, so a pre-step widens both operands to int8 in the workspace --
// zero-padded to whole tiles (rows to 128, K to 256), so that the matrix kernel reads only memory laid out by this
// file -- together with the row sums of x1 per group and zero-padded fp32 copies of the scales and offsets.
// The matrix kernel: 128 x 128 output tile per workgroup, eight waves of 64 x 32 (4 x 2 fragments of 16 x 16), one K
// tile = one group (256 bytes per row), v_mfma_i32_16x16x64_i8 chained over the group's four 64-byte steps from a
// zero accumulator, then the fold on the vector ALU (five operations per output and group).  The next group's
// operands are fetched into registers while the current one is multiplied, and written to the one LDS buffer between
// two barriers; rows are stored with their 16-byte chunks xor-swizzled by row so that the fragment reads are free of
// bank conflicts.
#include "launch.h"
#include "common.hip.h"

namespace opsnn {
namespace {

constexpr int64_t KG_GROUP = 256, KG_TILE = 128;
inline int64_t kg_rup(int64_t v, int64_t m) { return (v + m - 1) / m * m; }
inline uint64_t kg_a256(uint64_t v) { return (v + 255) / 256 * 256; }

struct KgLayout {
    int64_t Mp, Np, Kp, G;
    uint64_t o_b, o_rs, o_s2, o_of, total;   // byte offsets in the workspace (the widened x1 sits at 0)
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
    if (L.Mp * L.Kp >= (1ll << 31) || L.Np * L.Kp >= (1ll << 31)) return false;   // 32-bit offsets inside the kernels
    L.o_b = kg_a256((uint64_t)L.Mp * L.Kp);
    L.o_rs = L.o_b + kg_a256((uint64_t)L.Np * L.Kp);
    L.o_s2 = L.o_rs + kg_a256((uint64_t)L.Mp * L.G * 4);
    L.o_of = L.o_s2 + kg_a256((uint64_t)L.G * L.Np * 4);
    L.total = L.o_of + kg_a256((uint64_t)L.G * L.Np * 4);
    return true;
}

// 16 int4 (8 bytes) of row r -> 16 int8; rows past `rows` and columns past K become zero.  ld: elements between rows.
__global__ __launch_bounds__(256) void kg_widen_kernel(const uint8_t* __restrict__ src, int64_t rows, int64_t K, int64_t ld,
                                                       int8_t* __restrict__ dst, int64_t rows_p, int64_t Kp)
{
    const int64_t per_row = Kp / 16;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= rows_p * per_row) return;
    const int64_t r = idx / per_row, k0 = (idx - r * per_row) * 16;
    uint32_t o[4] = {0, 0, 0, 0};
    if (r < rows) {
#pragma unroll
        for (int b = 0; b < 8; b++) {
            const int64_t k = k0 + 2 * b;
            if (k < K) {   // K is even: both nibbles of the byte are inside the row
                const uint32_t byte = src[(r * ld + k) >> 1];
                const uint32_t lo = (uint32_t)(((int32_t)(int8_t)(byte << 4)) >> 4) & 0xffu;   // sign-extended low nibble
                const uint32_t hi = (uint32_t)(((int32_t)(int8_t)byte) >> 4) & 0xffu;
                o[b / 2] |= (lo | (hi << 8)) << (16 * (b % 2));
            }
        }
    }
    *(uint4*)(dst + r * Kp + k0) = make_uint4(o[0], o[1], o[2], o[3]);
}

// rs[m * G + g] = fp32 of the sum of the widened x1 over group g (exact: at most 256 values of magnitude 8)
__global__ __launch_bounds__(256) void kg_rowsum_kernel(const int8_t* __restrict__ a8, int64_t Mp, int64_t Kp, int64_t G, float* __restrict__ rs)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= Mp * G) return;
    const int64_t m = idx / G, g = idx - m * G;
    const uint4* p = (const uint4*)(a8 + m * Kp + g * KG_GROUP);
    int32_t s = 0;
#pragma unroll 4
    for (int i = 0; i < 16; i++) {
        const uint4 v = p[i];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 4; e++)
            s += (int32_t)(int8_t)w[e] + (int32_t)(int8_t)(w[e] >> 8) + (int32_t)(int8_t)(w[e] >> 16) + (int32_t)(int8_t)(w[e] >> 24);
    }
    rs[idx] = (float)s;
}

// fp32 copies of scale[g, n] and offset[g, n] with the columns padded to Np (zeros)
__global__ __launch_bounds__(256) void kg_scales_kernel(OpsnnMat sc, OpsnnMat of, int64_t N, int64_t Np, int64_t G, int64_t Greal,
                                                        float* __restrict__ s2p, float* __restrict__ ofp)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= G * Np) return;
    const int64_t g = idx / Np, n = idx - g * Np;
    float s = 0.0f, o = 0.0f;
    if (n < N && g < Greal) {
        s = ((const float*)sc.ptr)[g * sc.row_stride + n * sc.col_stride];
        o = load_scalar_as_f32(of.ptr, DT_F16, g * of.row_stride + n * of.col_stride);
    }
    s2p[idx] = s;
    ofp[idx] = o;
}

template <int OUT_DT>
__global__ __launch_bounds__(512) void kg_gemm_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ B, const float* __restrict__ rs,
                                                      const float* __restrict__ s2p, const float* __restrict__ ofp,
                                                      const float* __restrict__ x1s, uint16_t* __restrict__ out,
                                                      int64_t M, int64_t N, int Kp, int Np, int G)
{
    constexpr int FM = 4, FN = 2;
    __shared__ __attribute__((aligned(16))) char lds[2 * 128 * 256];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2, wn = wave & 3;
    const int frow = lane & 15, fq = lane >> 4;
    const int m0 = blockIdx.y * 128, n0 = blockIdx.x * 128;   // inside the padded operands by construction of the grid

    // staging: chunk idx = tid + 512 i of an operand tile is row idx / 16, 16-byte chunk idx % 16
    v4i ra[4], rb[4];
    auto gload = [&](int g) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int idx = tid + 512 * i, r = idx >> 4, c = idx & 15;
            ra[i] = *(const v4i*)(A + (int64_t)(m0 + r) * Kp + g * 256 + c * 16);
            rb[i] = *(const v4i*)(B + (int64_t)(n0 + r) * Kp + g * 256 + c * 16);
        }
    };
    auto lstore = [&]() {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int idx = tid + 512 * i, r = idx >> 4, c = idx & 15;
            *(v4i*)(lds + r * 256 + ((c ^ (r & 15)) << 4)) = ra[i];
            *(v4i*)(lds + 32768 + r * 256 + ((c ^ (r & 15)) << 4)) = rb[i];
        }
    };

    v4f sum[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; i++)
#pragma unroll
        for (int j = 0; j < FM; j++) sum[i][j] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};

    const char* la = lds + (wm * 64 + frow) * 256;
    const char* lb = lds + 32768 + (wn * 32 + frow) * 256;
    gload(0);
    for (int g = 0; g < G; g++) {
        __syncthreads();   // every wave has read the previous group
        lstore();
        __syncthreads();
        if (g + 1 < G) gload(g + 1);
        float rsv[FM];
        v4f s2v[FN], ofv[FN];
#pragma unroll
        for (int j = 0; j < FM; j++) rsv[j] = rs[(int64_t)(m0 + wm * 64 + 16 * j + frow) * G + g];
#pragma unroll
        for (int i = 0; i < FN; i++) {
            const int64_t o = (int64_t)g * Np + n0 + wn * 32 + 16 * i + 4 * fq;
            s2v[i] = *(const v4f*)(s2p + o);
            ofv[i] = *(const v4f*)(ofp + o);
        }
        v4i t[FN][FM];
#pragma unroll
        for (int i = 0; i < FN; i++)
#pragma unroll
            for (int j = 0; j < FM; j++) t[i][j] = (v4i){0, 0, 0, 0};
#pragma unroll
        for (int s = 0; s < 4; s++) {
            // lane (row, q) holds bytes [64 s + 16 q, + 16) of its row: the same K for both operands
            const int pos = ((4 * s + fq) ^ frow) << 4;
            v4i fa[FM], fb[FN];
#pragma unroll
            for (int j = 0; j < FM; j++) fa[j] = *(const v4i*)(la + j * 16 * 256 + pos);
#pragma unroll
            for (int i = 0; i < FN; i++) fb[i] = *(const v4i*)(lb + i * 16 * 256 + pos);
#pragma unroll
            for (int i = 0; i < FN; i++)
#pragma unroll
                for (int j = 0; j < FM; j++) t[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[i], fa[j], t[i][j], 0, 0, 0);
        }
        // t[i][j][r] is the group's integer sum for m = 16 j + lane % 16, n = 16 i + 4 (lane / 16) + r of the wave tile
#pragma unroll
        for (int i = 0; i < FN; i++)
#pragma unroll
            for (int j = 0; j < FM; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float off = rsv[j] * ofv[i][r];
                    sum[i][j][r] = sum[i][j][r] + ((float)t[i][j][r] - off) * s2v[i][r];
                }
    }

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
    char* ws = (char*)a.workspace;
    int8_t* a8 = (int8_t*)ws;
    int8_t* b8 = (int8_t*)(ws + L.o_b);
    float* rs = (float*)(ws + L.o_rs);
    float* s2p = (float*)(ws + L.o_s2);
    float* ofp = (float*)(ws + L.o_of);
    const int64_t Greal = (a.K + KG_GROUP - 1) / KG_GROUP;
    auto blocks = [](int64_t n) { return dim3((unsigned)((n + 255) / 256)); };
    hipLaunchKernelGGL(kg_widen_kernel, blocks(L.Mp * (L.Kp / 16)), dim3(256), 0, st, (const uint8_t*)a.x1.ptr, a.M, a.K, a.x1.row_stride, a8, L.Mp, L.Kp);
    hipLaunchKernelGGL(kg_widen_kernel, blocks(L.Np * (L.Kp / 16)), dim3(256), 0, st, (const uint8_t*)a.x2.ptr, a.N, a.K, a.x2.col_stride, b8, L.Np, L.Kp);
    hipLaunchKernelGGL(kg_rowsum_kernel, blocks(L.Mp * L.G), dim3(256), 0, st, a8, L.Mp, L.Kp, L.G, rs);
    hipLaunchKernelGGL(kg_scales_kernel, blocks(L.G * L.Np), dim3(256), 0, st, a.x2_scale_mat, a.x2_offset_mat, a.N, L.Np, L.G, Greal, s2p, ofp);
    const dim3 grid((unsigned)(L.Np / KG_TILE), (unsigned)(L.Mp / KG_TILE));
    if (a.out_dtype == DT_BF16)
        hipLaunchKernelGGL(kg_gemm_kernel<DT_BF16>, grid, dim3(512), 0, st, a8, b8, rs, s2p, ofp, (const float*)a.x1_scale, (uint16_t*)a.out, a.M, a.N,
                           (int)L.Kp, (int)L.Np, (int)L.G);
    else
        hipLaunchKernelGGL(kg_gemm_kernel<DT_F16>, grid, dim3(512), 0, st, a8, b8, rs, s2p, ofp, (const float*)a.x1_scale, (uint16_t*)a.out, a.M, a.N,
                           (int)L.Kp, (int)L.Np, (int)L.G);
    return (int)hipGetLastError();
}

}  // namespace opsnn
