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
// matrix kernel fetches a block with linear 16-byte asynchronous copies (one base address per group, no swizzle or row
// arithmetic per lane), and the side values arrive in LDS with the tile instead of costing every wave eight vector
// loads per group.
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

void* weight_cache_blob3(const void* src, const void* src2, const void* src3, int64_t K, int64_t N, int bits, int64_t nb, uint64_t bytes, hipStream_t st,
                         bool* fresh);   // weight_cache.hip
void weight_cache_commit(void* buffer, hipStream_t st);
void weight_cache_abandon(void* buffer);

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
    if (L.G * ((L.Mp + L.Np) / 16 + (L.Np + 255) / 256) >= (1ll << 31)) return false;   // workgroups of the pre-step
    L.o_b = (uint64_t)(L.Mp / KG_TILE * L.G * KG_BLOCK);
    L.total = L.o_b + (uint64_t)(L.Np / KG_TILE * L.G * KG_BLOCK);
    return true;
}

struct KgPrepare {
    const uint8_t* x[2];   // x1 [M, K] and x2 [N, K], K contiguous, two elements per byte
    int64_t rows[2], ld[2], K;
    int8_t* blocks[2];
    int rows_p[2], G, Greal;
    OpsnnMat sc, of;
    int64_t N;
    uint32_t first[3];   // first workgroup of the x2 blocks, of their side values, and the grid size
};

// The pre-step, one launch: the first workgroups write the x1 blocks, the next the x2 blocks, the last the side values
// of the x2 blocks; within a role the group is the fastest index.  Operand roles: a workgroup takes 16 rows of one group, a thread 16 int4 (8 bytes) -> 16 e4m3
// bytes in the block layout; rows past the operand's and columns past K become zero.  For x1 the 16 threads of a row
// (neighbours in one wave) also add up its elements, and the block's first side value array gets -fp32(sum) (exact: at
// most 256 values of magnitude 8).  Side value role: a thread takes one column: fp32 scale[g, n] and offset[g, n],
// zeros for padded columns and groups.
__global__ __launch_bounds__(256) void kg_prepare_kernel(KgPrepare p)
{
    const uint32_t bid = blockIdx.x;
    const int role = bid >= p.first[1] ? 2 : bid >= p.first[0] ? 1 : 0, tid = threadIdx.x;
    const uint32_t local = bid - (role == 2 ? p.first[1] : role == 1 ? p.first[0] : 0u);
    const uint32_t bx = local / (uint32_t)p.G;
    const int g = (int)(local - bx * (uint32_t)p.G);
    if (role == 2) {
        const int64_t n = (int64_t)bx * 256 + tid;
        if (n >= p.rows_p[1]) return;
        float s = 0.0f, o = 0.0f;
        if (n < p.N && g < p.Greal) {
            s = ((const float*)p.sc.ptr)[g * p.sc.row_stride + n * p.sc.col_stride];
            o = load_scalar_as_f32(p.of.ptr, DT_F16, g * p.of.row_stride + n * p.of.col_stride);
        }
        float* side = (float*)(p.blocks[1] + ((n >> 7) * p.G + g) * KG_BLOCK + KG_ROWS);
        side[n & 127] = s;
        side[128 + (n & 127)] = o;
        return;
    }
    const int64_t r = (int64_t)bx * 16 + (tid >> 4), K = p.K;
    const int c = tid & 15;
    const int64_t k0 = (int64_t)g * KG_GROUP + c * 16;
    uint64_t nib = 0;   // 16 nibbles, element k0 + e in bits [4 e, 4 e + 4)
    if (r < p.rows[role] && k0 < K) {
        const uint8_t* src = p.x[role] + ((r * p.ld[role] + k0) >> 1);   // ld and k0 are even: the row piece starts on a byte
        if (k0 + 16 <= K && ((uintptr_t)src & 7) == 0) nib = *(const uint64_t*)src;
        else {
#pragma unroll
            for (int b = 0; b < 8; b++)
                if (k0 + 2 * b < K) nib |= (uint64_t)src[b] << (8 * b);   // K is even: both nibbles of the byte are inside the row
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
    int8_t* block = p.blocks[role] + ((r >> 7) * p.G + g) * KG_BLOCK;
    *(uint4*)(block + ((r & 127) << 8) + ((c ^ (r & 15)) << 4)) = make_uint4(o[0], o[1], o[2], o[3]);
    if (role == 0) {
#pragma unroll
        for (int d = 8; d >= 1; d >>= 1) s += __shfl_xor(s, d, 16);
        if (c == 0) ((float*)(block + KG_ROWS))[r & 127] = -(float)s;
    }
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

    v4f sum[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; i++)
#pragma unroll
        for (int j = 0; j < FM; j++) sum[i][j] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};

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
            // t[i][j][r] becomes the group's integer sum for m = 16 j + lane % 16, n = 16 i + 4 (lane / 16) + r of the wave tile;
            // a fragment pair is folded as soon as its second instruction is out, in the shadow of the following ones
#pragma unroll
            for (int i = 0; i < FN; i++)
#pragma unroll
                for (int j = 0; j < FM; j++) {
                    t[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[i], fa[j], s == 0 ? (v4f){0.0f, 0.0f, 0.0f, 0.0f} : t[i][j], 0, 0, 0,
                                                                               0x7f7f7f7f, 0, 0x7f7f7f7f);
                    if (s == 1) {
#pragma unroll
                        for (int r = 0; r < 4; r++) sum[i][j][r] = sum[i][j][r] + __builtin_fmaf(rsv[j], ofv[i][r], t[i][j][r]) * s2v[i][r];
                    }
                }
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
    // The x2 blocks depend on the weights, their scales and their offsets only: with the weight cache on they are
    // written by the first call and found by the later ones.
    int8_t* a8 = (int8_t*)a.workspace;
    int8_t* b8 = a8 + L.o_b;
    bool fresh = false;
    const bool dense = a.x2.col_stride == a.K && a.x2_scale_mat.row_stride == a.N && a.x2_scale_mat.col_stride == 1 &&
                       a.x2_offset_mat.row_stride == a.N && a.x2_offset_mat.col_stride == 1;   // what the cache key does not tell apart
    void* cached = dense ? weight_cache_blob3(a.x2.ptr, a.x2_scale_mat.ptr, a.x2_offset_mat.ptr, a.K, a.N, 4, 1, L.total - L.o_b, st, &fresh) : nullptr;
    if (cached) b8 = (int8_t*)cached;
    KgPrepare p;
    p.x[0] = (const uint8_t*)a.x1.ptr; p.x[1] = (const uint8_t*)a.x2.ptr;
    p.rows[0] = a.M; p.rows[1] = a.N;
    p.ld[0] = a.x1.row_stride; p.ld[1] = a.x2.col_stride;
    p.K = a.K;
    p.blocks[0] = a8; p.blocks[1] = b8;
    p.rows_p[0] = (int)L.Mp; p.rows_p[1] = (int)L.Np;
    p.G = (int)L.G; p.Greal = (int)((a.K + KG_GROUP - 1) / KG_GROUP);
    p.sc = a.x2_scale_mat; p.of = a.x2_offset_mat;
    p.N = a.N;
    const bool x1_only = cached && !fresh;
    const int64_t wg0 = L.G * (L.Mp / 16), wg1 = x1_only ? 0 : L.G * (L.Np / 16), wg2 = x1_only ? 0 : L.G * ((L.Np + 255) / 256);
    p.first[0] = (uint32_t)wg0; p.first[1] = (uint32_t)(wg0 + wg1); p.first[2] = (uint32_t)(wg0 + wg1 + wg2);
    hipLaunchKernelGGL(kg_prepare_kernel, dim3(p.first[2]), dim3(256), 0, st, p);
    if (cached && fresh) {
        if (hipGetLastError() != hipSuccess) { weight_cache_abandon(cached); return (int)hipErrorLaunchFailure; }
        weight_cache_commit(cached, st);
    }
    const dim3 grid((unsigned)(L.Np / KG_TILE), (unsigned)(L.Mp / KG_TILE));
    constexpr int KG_LDS = 2 * 2 * (int)KG_BLOCK;
    static std::atomic<uint64_t> attr_set{0};   // one bit per device: the attribute belongs to the (kernel, device) pair
    if (!device_flag_test(attr_set)) {
        hipError_t e = hipFuncSetAttribute((const void*)kg_gemm_kernel<DT_BF16>, hipFuncAttributeMaxDynamicSharedMemorySize, KG_LDS);
        if (e == hipSuccess) e = hipFuncSetAttribute((const void*)kg_gemm_kernel<DT_F16>, hipFuncAttributeMaxDynamicSharedMemorySize, KG_LDS);
        if (e != hipSuccess) return (int)e;
        device_flag_set(attr_set);
    }
    if (a.out_dtype == DT_BF16)
        hipLaunchKernelGGL(kg_gemm_kernel<DT_BF16>, grid, dim3(512), KG_LDS, st, a8, b8, (const float*)a.x1_scale, (uint16_t*)a.out, a.M, a.N, (int)L.G);
    else
        hipLaunchKernelGGL(kg_gemm_kernel<DT_F16>, grid, dim3(512), KG_LDS, st, a8, b8, (const float*)a.x1_scale, (uint16_t*)a.out, a.M, a.N, (int)L.G);
    return (int)hipGetLastError();
}

}  // namespace opsnn
