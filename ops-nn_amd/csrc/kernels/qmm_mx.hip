// MX quantized matmul: fp4 e2m1 (or fp8 e4m3) operands with one e8m0 scale per 32 K elements.
//
//   out[m,n] = cast( sum_k (x1[m,k] * 2^(s1[m,k/32]-127)) * (x2[k,n] * 2^(s2[k/32,n]-127)) + bias[n] )
//
// Formula and scale layouts: matmul/quant_batch_matmul_v3/tests/assets/qbmmv3_kernel_golden.py:153-234; the
// device counterpart in the reference is the MX block-mmad (matmul/common/cmct/block/block_mmad_mx.h).
// Here the contraction and the scaling are one instruction, v_mfma_scale_f32_32x32x64_f8f6f4: each lane hands
// the matrix core its 32 K elements together with the e8m0 byte that scales exactly those 32 elements, so the
// MX block size (32) and the hardware operand block coincide and no dequantised copy is ever formed.
//
// Fast paths: operands and scales K-contiguous, K % 128 == 0, 16-bit output.  fp4: qgemm_core.hip.h, MODE_MXFP4
// (K % 512 == 0 takes 256-element K tiles, otherwise 128-element ones); fp8: the MX mode of the kernel in
// qmm_fp8_block.hip.  An N-contiguous x2 (data [K, N], scales [K/64, N, 2]) is first re-laid out into the
// workspace.  K % 128 != 0 (K a whole number of 32-element blocks): both operands and both scale tables (x2's after that re-layout, if it was needed) are first
// copied into the workspace with K rounded up to 128, the new elements zero and their scales a repeat of the row's last one (zero products
// change no sum).  All of this is planned before the first pre-step is launched.  Everything else runs the plain kernel.
#include "launch.h"
#include "qgemm_core.hip.h"

namespace opsnn {

// dst[c, r] = src[r, c] for 16-bit elements: the paired e8m0 scales [K/64, N, 2] -> [N, K/64, 2].
__global__ __launch_bounds__(256) void transpose16_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                          int64_t rows, int64_t cols)
{
    __shared__ uint16_t tile[32][33];
    const int64_t bz = blockIdx.z;
    src += bz * rows * cols;
    dst += bz * rows * cols;
    const int64_t r0 = (int64_t)blockIdx.y * 32, c0 = (int64_t)blockIdx.x * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for (int i = ty; i < 32; i += 8) {
        int64_t r = r0 + i, c = c0 + tx;
        tile[i][tx] = (r < rows && c < cols) ? src[r * cols + c] : 0;
    }
    __syncthreads();
    for (int i = ty; i < 32; i += 8) {
        int64_t c = c0 + i, r = r0 + tx;
        if (c < cols && r < rows) dst[c * rows + r] = tile[tx][i];
    }
}

}  // namespace opsnn
extern "C" int opsnnTranspose16(const void* src, void* dst, int64_t rows, int64_t cols, int64_t batch, void* stream)
{
    if (!src || !dst || rows <= 0 || cols <= 0 || batch <= 0 || batch > 65535) return -1;
    dim3 grid((unsigned)((cols + 31) / 32), (unsigned)((rows + 31) / 32), (unsigned)batch);
    if (grid.y > 65535u) return -2;
    hipLaunchKernelGGL(opsnn::transpose16_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t*)src, (uint16_t*)dst, rows, cols);
    return (int)hipGetLastError();
}
namespace opsnn {

static inline uint64_t align_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }
extern "C" bool opsnn_force_plain();   // dispatch.hip

// ---- K % 128 != 0 (whole MX blocks: K % 32 == 0) ----
// rows of kb bytes (pitch ld) -> rows of kbp bytes, the tail filled with the byte `fill`; E = bytes per thread.  E == 16:
// kb is a multiple of 16.  E == 2 (scale rows): kb counts the bytes that scale existing elements; the second byte of a
// source pair may lie past it (K % 64 == 32) and is replaced like the rest of the tail, whatever the caller left there.
// Scale tails repeat the row's last valid byte; data tails are zero.
template <int E>
__global__ __launch_bounds__(256) void mx_pad_rows_kernel(const uint8_t* __restrict__ src, int64_t ld, int64_t bs, uint8_t* __restrict__ dst,
                                                          int64_t rows, int64_t kb, int64_t kbp, uint32_t fill)
{
    const int64_t c = (int64_t)blockIdx.x * 64 + (threadIdx.x & 63), r = (int64_t)blockIdx.y * 4 + (threadIdx.x >> 6);
    if (c * E >= kbp || r >= rows) return;
    const uint8_t* s = src + (int64_t)blockIdx.z * bs + r * ld + c * E;
    uint8_t* d = dst + ((int64_t)blockIdx.z * rows + r) * kbp + c * E;
    if constexpr (E == 16) {
        *(uint4*)d = c * E < kb ? *(const uint4*)s : make_uint4(fill, fill, fill, fill);
    } else {
        // the tail repeats the row's last valid scale byte (its elements are zero, so any finite scale will do, and this
        // one leaves the spread of the row's scales as it was: the exact MXFP8 route looks at that spread)
        (void)fill;
        const uint32_t last = (src + (int64_t)blockIdx.z * bs + r * ld)[kb - 1];
        uint16_t v = (uint16_t)(last | (last << 8));
        if (c * 2 + 1 < kb) v = *(const uint16_t*)s;
        else if (c * 2 < kb) v = (uint16_t)((v & 0xFF00u) | s[0]);
        *(uint16_t*)d = v;
    }
}

struct MxPad {
    int64_t Kp, nb1, nb2, snb1, snb2;
    uint64_t o_x2, o_s1, o_s2, total;
};

// Whether the padding pre-step serves this call, and its workspace layout.
static bool mx_pad_layout(const OpsnnQmmArgs& a, MxPad& L)
{
    const bool fp4 = a.x1_dtype == DT_E2M1 && a.x2_dtype == DT_E2M1, fp8 = a.x1_dtype == DT_E4M3 && a.x2_dtype == DT_E4M3;
    const bool a8w4 = a.x1_dtype == DT_E4M3 && a.x2_dtype == DT_E2M1;   // the matrix-core kernel of that mode: 16-bit output, fp32 or 16-bit bias
    if ((!fp4 && !fp8 && !a8w4) || a.K % 128 == 0 || a.K % 32 != 0 || a.M * a.N < 64 * 64) return false;
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16 && !(a.out_dtype == DT_F32 && !a8w4)) return false;
    if (a.bias && a.bias_dtype != DT_F32 && !(a8w4 && (a.bias_dtype == DT_BF16 || a.bias_dtype == DT_F16))) return false;
    const int64_t epb1 = a.x1_dtype == DT_E2M1 ? 2 : 1, epb2 = a.x2_dtype == DT_E2M1 ? 2 : 1, ks = (a.K + 63) / 64;   // elements per byte; scale pairs per row
    if (a.x1.col_stride != 1 || a.x2.row_stride != 1) return false;
    if (a.x1_scale_mat.col_stride != 2 || a.x1_scale_mat.row_stride != ks * 2) return false;
    if (a.x2_scale_mat.col_stride != 2 || a.x2_scale_mat.row_stride != ks * 2) return false;
    if (a.x1.batch_stride < 0 || a.x2.batch_stride < 0 || a.x1_scale_mat.batch_stride < 0 || a.x2_scale_mat.batch_stride < 0) return false;
    // 16-byte pieces of the data rows, 2-byte pieces of the scale rows
    if (((uintptr_t)a.x1.ptr | (uintptr_t)a.x2.ptr | (uint64_t)(a.x1.row_stride / epb1) | (uint64_t)(a.x2.col_stride / epb2) |
         (uint64_t)(a.x1.batch_stride / epb1) | (uint64_t)(a.x2.batch_stride / epb2)) % 16) return false;
    if (((uintptr_t)a.x1_scale_mat.ptr | (uintptr_t)a.x2_scale_mat.ptr | (uint64_t)a.x1_scale_mat.batch_stride | (uint64_t)a.x2_scale_mat.batch_stride) % 2) return false;
    if ((a.M + 3) / 4 > 65535 || (a.N + 3) / 4 > 65535) return false;
    L.Kp = (a.K + 127) / 128 * 128;
    L.nb1 = a.x1.batch_stride == 0 && a.batch > 1 ? 1 : a.batch;
    L.nb2 = a.x2.batch_stride == 0 ? 1 : a.batch;
    L.snb1 = a.x1_scale_mat.batch_stride == 0 && a.batch > 1 ? 1 : a.batch;
    L.snb2 = a.x2_scale_mat.batch_stride == 0 ? 1 : a.batch;
    const uint64_t ksp = (uint64_t)L.Kp / 64;
    L.o_x2 = align_up((uint64_t)L.nb1 * a.M * (L.Kp / epb1), 256);
    L.o_s1 = L.o_x2 + align_up((uint64_t)L.nb2 * a.N * (L.Kp / epb2), 256);
    L.o_s2 = L.o_s1 + align_up((uint64_t)L.snb1 * a.M * ksp * 2, 256);
    L.total = L.o_s2 + align_up((uint64_t)L.snb2 * a.N * ksp * 2, 256);
    return true;
}

// Launches the four copies and rewrites `a` as the same call on the padded operands.
static int mx_pad_prestep(OpsnnQmmArgs& a, const MxPad& L, hipStream_t st)
{
    if (!a.workspace || (uintptr_t)a.workspace % 16) return OPSNN_NOT_TAKEN;
    const int64_t epb1 = a.x1_dtype == DT_E2M1 ? 2 : 1, epb2 = a.x2_dtype == DT_E2M1 ? 2 : 1;
    const int64_t kb1 = a.K / epb1, kbp1 = L.Kp / epb1, kb2 = a.K / epb2, kbp2 = L.Kp / epb2, ks2 = (a.K + 63) / 64 * 2, ksp2 = L.Kp / 64 * 2;
    const int64_t sv = a.K / 32;   // scale bytes per row that scale existing elements
    uint8_t* w = (uint8_t*)a.workspace;
    auto grid = [](int64_t pieces, int64_t rows, int64_t nb) { return dim3((unsigned)((pieces + 63) / 64), (unsigned)((rows + 3) / 4), (unsigned)nb); };
    hipLaunchKernelGGL(mx_pad_rows_kernel<16>, grid(kbp1 / 16, a.M, L.nb1), dim3(256), 0, st, (const uint8_t*)a.x1.ptr, a.x1.row_stride / epb1,
                       a.x1.batch_stride / epb1, w, a.M, kb1, kbp1, 0u);
    hipLaunchKernelGGL(mx_pad_rows_kernel<16>, grid(kbp2 / 16, a.N, L.nb2), dim3(256), 0, st, (const uint8_t*)a.x2.ptr, a.x2.col_stride / epb2,
                       a.x2.batch_stride / epb2, w + L.o_x2, a.N, kb2, kbp2, 0u);
    hipLaunchKernelGGL(mx_pad_rows_kernel<2>, grid(ksp2 / 2, a.M, L.snb1), dim3(256), 0, st, (const uint8_t*)a.x1_scale_mat.ptr, ks2,
                       a.x1_scale_mat.batch_stride, w + L.o_s1, a.M, sv, ksp2, 0x7f7fu);
    hipLaunchKernelGGL(mx_pad_rows_kernel<2>, grid(ksp2 / 2, a.N, L.snb2), dim3(256), 0, st, (const uint8_t*)a.x2_scale_mat.ptr, ks2,
                       a.x2_scale_mat.batch_stride, w + L.o_s2, a.N, sv, ksp2, 0x7f7fu);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    a.x1 = OpsnnMat{w, L.Kp, 1, L.nb1 == 1 && a.batch > 1 ? 0 : a.M * L.Kp};
    a.x2 = OpsnnMat{w + L.o_x2, 1, L.Kp, L.nb2 == 1 && a.batch > 1 ? 0 : a.N * L.Kp};
    a.x1_scale_mat = OpsnnMat{w + L.o_s1, ksp2, 2, L.snb1 == 1 && a.batch > 1 ? 0 : a.M * ksp2};
    a.x2_scale_mat = OpsnnMat{w + L.o_s2, ksp2, 2, L.snb2 == 1 && a.batch > 1 ? 0 : a.N * ksp2};
    a.K = L.Kp;
    a.workspace = nullptr;
    return 0;
}

uint64_t mx_exact_bytes(const OpsnnQmmArgs& a);           // qmm_fp8_exact.hip
int launch_mx_exact(const OpsnnQmmArgs& a, void* region, hipStream_t st, SplitK sk);

// ---- x2 stored [K, N] with N contiguous (data dense, scales [K/64, N, 2]) ----
// The kernels stream K-contiguous operands: data and scales are first re-laid out, per batch, at 256-byte aligned pitches.
struct MxRelayout {
    int64_t nb, snb;                 // batches of the data / of the scales (1 when every batch shares them)
    uint64_t data_one, scale_one, bytes;
};

static bool mx_relayout_layout(const OpsnnQmmArgs& a, MxRelayout& R)
{
    if (a.x2.row_stride == 1 || a.K == 1 || a.K % 32 != 0) return false;
    const int64_t ks = (a.K + 63) / 64, epb = a.x2_dtype == DT_E2M1 ? 2 : 1;
    if (a.x2.col_stride != 1 || a.x2.row_stride != a.N) return false;
    if (epb == 2 && (a.N & 1)) return false;   // the 4-bit transposition works on byte pairs
    if (a.x2_scale_mat.row_stride != 2 || a.x2_scale_mat.col_stride != a.N * 2) return false;
    if (a.x2.batch_stride != 0 && a.x2.batch_stride != a.K * a.N) return false;
    R.nb = a.x2.batch_stride == 0 ? 1 : a.batch;
    R.snb = a.x2_scale_mat.batch_stride == 0 ? 1 : a.batch;
    if (R.snb != 1 && a.x2_scale_mat.batch_stride != ks * a.N * 2) return false;
    if (R.nb > 65535 || R.snb > 65535) return false;
    R.data_one = align_up((uint64_t)a.N * a.K / epb, 256);
    R.scale_one = align_up((uint64_t)a.N * ks * 2, 256);
    R.bytes = R.data_one * (uint64_t)R.nb + R.scale_one * (uint64_t)R.snb;
    return true;
}

// `a` as the same call on the copies at `w` (which the passes of mx_relayout_run fill)
static void mx_relayout_view(OpsnnQmmArgs& a, const MxRelayout& R, char* w)
{
    const int64_t ks = (a.K + 63) / 64, epb = a.x2_dtype == DT_E2M1 ? 2 : 1;
    char* wscale = w + R.data_one * R.nb;
    a.x2.ptr = w; a.x2.row_stride = 1; a.x2.col_stride = a.K; a.x2.batch_stride = R.nb == 1 ? 0 : (int64_t)(R.data_one * epb);
    a.x2_scale_mat.ptr = wscale; a.x2_scale_mat.row_stride = ks * 2; a.x2_scale_mat.col_stride = 2;
    a.x2_scale_mat.batch_stride = R.snb == 1 ? 0 : (int64_t)R.scale_one;
}

static int mx_relayout_run(const OpsnnQmmArgs& a, const MxRelayout& R, char* w, hipStream_t st)
{
    const int64_t ks = (a.K + 63) / 64, epb = a.x2_dtype == DT_E2M1 ? 2 : 1;
    char* wscale = w + R.data_one * R.nb;
    for (int64_t b = 0; b < R.nb; b++) {  // per batch because of the aligned pitch
        const char* src = (const char*)a.x2.ptr + b * (a.K * a.N / epb);
        const int rc = epb == 2 ? opsnnTranspose4(src, w + b * R.data_one, a.K, a.N, 1, st) : opsnnTranspose8(src, w + b * R.data_one, a.K, a.N, 1, st);
        if (rc != 0) return rc;
    }
    for (int64_t b = 0; b < R.snb; b++) {
        dim3 grid((unsigned)((a.N + 31) / 32), (unsigned)((ks + 31) / 32), 1);
        hipLaunchKernelGGL(transpose16_kernel, grid, dim3(256), 0, st, (const uint16_t*)((const char*)a.x2_scale_mat.ptr + b * (ks * a.N * 2)),
                           (uint16_t*)(wscale + b * R.scale_one), ks, a.N);
    }
    return (int)hipGetLastError();
}

// What every matrix-core route of this file needs of the call, whatever x2's layout and K's tail: checked before any
// pre-step is launched or a cache entry made.
static bool mx_call_ok(const OpsnnQmmArgs& a)
{
    const bool fp4 = a.x1_dtype == DT_E2M1 && a.x2_dtype == DT_E2M1, fp8 = a.x1_dtype == DT_E4M3 && a.x2_dtype == DT_E4M3;
    const bool a8w4 = a.x1_dtype == DT_E4M3 && a.x2_dtype == DT_E2M1;
    if (!fp4 && !fp8 && !a8w4) return false;
    if (a8w4) {   // launch_mx_a8w4_mfma (qmm_fp8_block.hip): a tile kernel, and a streaming kernel for up to 32 rows
        if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16) return false;
        if (a.bias && a.bias_dtype != DT_F32 && a.bias_dtype != DT_BF16 && a.bias_dtype != DT_F16) return false;
        if (a.K % 32 != 0 || a.x1.col_stride != 1 || a.x1_scale_mat.col_stride != 2) return false;
        const bool few_rows = a.M <= 32 && a.N >= 256 && a.batch == 1;
        if (!few_rows && a.M * a.N < 64 * 64) return false;
        return (((uintptr_t)a.x1.ptr | (uint64_t)a.x1.row_stride | (uint64_t)a.x1.batch_stride) % 16) == 0;
    }
    if (a.out_dtype != DT_BF16 && a.out_dtype != DT_F16 && a.out_dtype != DT_F32) return false;
    if (a.bias && a.bias_dtype != DT_F32) return false;
    // (fewer than 64 x 64 outputs: only MXFP8's few-rows stream over x2, which wants 256 columns)
    if (a.K % 32 != 0 || (a.M * a.N < 64 * 64 && !(fp8 && a.M <= 32 && a.N >= 256 && a.batch == 1 && a.K % 128 == 0))) return false;
    const int64_t ks = (a.K + 63) / 64, epb = fp4 ? 2 : 1;
    if (a.x1.col_stride != 1 || a.x1_scale_mat.col_stride != 2 || a.x1_scale_mat.row_stride != ks * 2) return false;
    if (((uintptr_t)a.x1.ptr | (uint64_t)(a.x1.row_stride / epb) | (uint64_t)(a.x1.batch_stride / epb)) % 16) return false;
    if (a.K % 128 == 0 && ((uintptr_t)a.x1_scale_mat.ptr | (uint64_t)a.x1_scale_mat.row_stride | (uint64_t)a.x1_scale_mat.batch_stride) % 4) return false;
    return true;
}

// Bytes behind the exact route's tables: the K-contiguous copies of an N-contiguous x2, then the padded copies of a K tail.
static uint64_t mx_rest_bytes(const OpsnnQmmArgs& a0)
{
    if (a0.force_variant == OPSNN_VARIANT_PLAIN || opsnn_force_plain() || !mx_call_ok(a0)) return 0;
    OpsnnQmmArgs a = a0;
    uint64_t total = 0;
    MxRelayout R;
    if (mx_relayout_layout(a, R)) {
        total = align_up(R.bytes, 256);
        mx_relayout_view(a, R, (char*)(uintptr_t)256);   // any aligned address: only the layout matters below
    }
    MxPad L;
    if (mx_pad_layout(a, L)) total += L.total;
    return total;
}

// Workspace of an MX call: in front, what the exact route of MXFP8 needs (nothing for the other operand pairs), then the
// re-laid-out and padded operand copies.
uint64_t mxfp8_rows_workspace(const OpsnnQmmArgs& a);   // qmm_fp8_rows.hip
int launch_mxfp8_rows(const OpsnnQmmArgs& a, void* region, hipStream_t st, SplitK sk);
// (in front of that: the bf16 copy of x1 for MXFP8 with 33 .. 256 rows on the many-rows kernel)
static uint64_t mx_rows_bytes(const OpsnnQmmArgs& a)
{
    // (whether or not opsnnSetFp8Fast is on: a workspace must not depend on a switch that may change between the two phases)
    if (a.force_variant == OPSNN_VARIANT_PLAIN || opsnn_force_plain() || !mx_call_ok(a)) return 0;
    return align_up(mxfp8_rows_workspace(a), 256);
}
uint64_t mx_workspace_bytes(const OpsnnQmmArgs& a)
{
    const bool matrix_cores = a.force_variant != OPSNN_VARIANT_PLAIN && !opsnn_force_plain();
    return mx_rows_bytes(a) + (matrix_cores ? mx_exact_bytes(a) : 0) + mx_rest_bytes(a);
}

void* weight_cache_blob(const void* src, const void* src2, int64_t K, int64_t N, int bits, int64_t nb, uint64_t bytes, hipStream_t st, bool* fresh);
void weight_cache_commit(void* buffer, hipStream_t st);   // weight_cache.hip
void weight_cache_abandon(void* buffer);
int launch_mxfp8_mfma(const OpsnnQmmArgs& a, hipStream_t st);   // qmm_fp8_block.hip
int launch_mx_a8w4_mfma(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk);   // qmm_fp8_block.hip
int launch_mxfp8_decode(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk);   // qmm_fp8_decode.hip

int launch_mx_mfma(const OpsnnQmmArgs& a0, hipStream_t st, SplitK sk)
{
    if (!mx_call_ok(a0)) return OPSNN_NOT_TAKEN;
    OpsnnQmmArgs a = a0;
    const bool fp4 = a.x1_dtype == DT_E2M1 && a.x2_dtype == DT_E2M1;
    const bool fp8 = a.x1_dtype == DT_E4M3 && a.x2_dtype == DT_E4M3;
    // MXFP8 runs on exact products by default (with two 8-bit operands the scaled matrix instruction aligns its products in
    // a window narrower than fp32: measured on 4096 x 8192 x 8192 with scale exponents in [-4, 4], 1 % of the bf16 outputs
    // one ulp off and the largest relative error above 2^-7); opsnnSetFp8Fast(1) asks for the 8-bit instruction.  The exact
    // route's tables sit in front of the workspace.  With a 4-bit x2 the same instruction is as close to the fp32 sums as
    // exact products are (measured on the same shapes), so that mode keeps it.
    char* rows_region = nullptr;
    if (const uint64_t rb = mx_rows_bytes(a0); rb && a.workspace) {
        rows_region = (char*)a.workspace;
        a.workspace = rows_region + rb;
    }
    char* mxx = nullptr;
    if (const uint64_t front = mx_exact_bytes(a0); front && a.workspace) {
        mxx = (char*)a.workspace;
        a.workspace = mxx + front;
    }
    const bool exact = mxx && !opsnnGetFp8Fast();

    // Pre-steps, planned in full before the first of them is launched: an N-contiguous x2 is re-laid out K-contiguous (into
    // the weight cache's buffer for this operand when the cache is on -- a hit skips the passes -- else into the workspace);
    // a K tail (K % 128 == 64) then continues on zero-padded copies of all four operands.
    MxRelayout R;
    const bool relayout = mx_relayout_layout(a, R);
    if (!relayout && a.x2.row_stride != 1) return OPSNN_NOT_TAKEN;
    OpsnnQmmArgs planned = a;
    if (relayout) mx_relayout_view(planned, R, (char*)(uintptr_t)256);
    MxPad L;
    const bool pad = mx_pad_layout(planned, L);
    if (!pad && planned.K % 128 != 0) return OPSNN_NOT_TAKEN;
    if (planned.x2_scale_mat.col_stride != 2 || (fp4 || fp8 ? planned.x2_scale_mat.row_stride != (planned.K + 63) / 64 * 2 : planned.x2_scale_mat.row_stride % 4 != 0)) return OPSNN_NOT_TAKEN;
    if (pad && (!a.workspace || (uintptr_t)a.workspace % 16)) return OPSNN_NOT_TAKEN;
    if (relayout) {
        bool fresh = false;
        char* w = (char*)weight_cache_blob(a.x2.ptr, a.x2_scale_mat.ptr, a.K, a.N, a.x2_dtype == DT_E2M1 ? 4 : 8, R.nb * 16 + R.snb, R.bytes, st, &fresh);
        const bool cached = w != nullptr;
        if (!cached) {
            if (!a.workspace || (uintptr_t)a.workspace % 16) return OPSNN_NOT_TAKEN;
            w = (char*)a.workspace;
            a.workspace = w + align_up(R.bytes, 256);
        }
        if (!cached || fresh) {
            const int rc = mx_relayout_run(a, R, w, st);
            if (rc != 0) {
                if (cached) weight_cache_abandon(w);
                return rc;
            }
        }
        if (cached && fresh) weight_cache_commit(w, st);
        mx_relayout_view(a, R, w);
    }
    if (pad) {
        if (!mx_pad_layout(a, L)) return OPSNN_NOT_TAKEN;   // (the same answer as for the planned view: its conditions do not look at x2's address beyond its alignment)
        const int rc = mx_pad_prestep(a, L, st);
        if (rc != 0) return rc;
    }
    if (a.x1_dtype == DT_E4M3 && a.x2_dtype == DT_E2M1) return launch_mx_a8w4_mfma(a, st, sk);   // fp8 x fp4: qmm_fp8_block.hip
    if (fp8 && rows_region) {   // MXFP8 with 33 .. 256 rows: the many-rows streaming kernel on bf16 operands (exact products)
        if (!opsnnGetFp8Fast()) {
            const int rc = launch_mxfp8_rows(a, rows_region, st, sk);
            if (rc != OPSNN_NOT_TAKEN) return rc;
        }
        sk = SplitK{};   // (any partial sums were laid out for the kernel above; the tile kernels run unsplit)
    }
    if (fp8 && a.M <= 32) {   // MXFP8 with up to 32 rows: the stream over x2 with x1 in registers (exact products)
        const int rc = launch_mxfp8_decode(a, st, sk);
        if (rc != OPSNN_NOT_TAKEN) return rc;
        if (a.M * a.N < 64 * 64) return OPSNN_NOT_TAKEN;
        sk = SplitK{};   // (the partial sums were laid out for the kernel above; the tile kernels run unsplit)
    }
    // MXFP8 runs on the block kernel of qmm_fp8_block.hip in MX mode (16x16x128 instructions, 64 x 128 per wave, the
    // pipeline tuned for the fp8 block-scale path); the 32x32x64 tile kernel stays available on request
    // (OPSNN_VARIANT_MX_FP8_MFMA) for comparison.  The 8-bit forms of the matrix instruction sum their products with a
    // reduced-width aligner (measured: mean error 1e-5 of sum|terms| per instruction); fp4 products are exact in that
    // datapath.
    const int64_t ks = a.K / 64;  // scale pairs per row
    const int64_t epb = fp4 ? 2 : 1;  // elements per byte

    QgemmParams g{};
    g.a = (const int8_t*)a.x1.ptr; g.b = (const int8_t*)a.x2.ptr;
    g.lda = a.x1.row_stride / epb; g.ldb = a.x2.col_stride / epb;
    g.a_bs = a.x1.batch_stride / epb; g.b_bs = a.x2.batch_stride / epb;
    g.out = a.out; g.M = a.M; g.N = a.N; g.ldc = a.N; g.KB = a.K / epb;
    g.bias = a.bias; g.bias_dt = a.bias_dtype; g.bias_bs = a.bias_batch_stride;
    g.sa = (const uint8_t*)a.x1_scale_mat.ptr; g.sb = (const uint8_t*)a.x2_scale_mat.ptr;
    g.sa_rs = a.x1_scale_mat.row_stride; g.sb_rs = a.x2_scale_mat.row_stride;
    g.sa_bs = a.x1_scale_mat.batch_stride; g.sb_bs = a.x2_scale_mat.batch_stride;
    if (((uintptr_t)g.a | (uintptr_t)g.b | (uint64_t)g.lda | (uint64_t)g.ldb | (uint64_t)g.a_bs | (uint64_t)g.b_bs) % 16) return OPSNN_NOT_TAKEN;
    if (((uintptr_t)g.sa | (uintptr_t)g.sb | (uint64_t)g.sa_rs | (uint64_t)g.sb_rs | (uint64_t)g.sa_bs | (uint64_t)g.sb_bs) % 4) return OPSNN_NOT_TAKEN;
    if (fp8 && exact) {
        const int rc = launch_mx_exact(a, mxx, st, sk);
        if (rc != OPSNN_NOT_TAKEN) return rc;
    }
    const bool small = a.M <= 128 || a.N <= 128;
    if (fp4) {
        // few tiles against a long K: K split over workgroups (fp32 partial sums in front of the workspace), on the tiles
        // chosen below
        const bool split = sk.splits > 1 && sk.part && a.force_variant == 0 && a.K % 256 == 0;
        if (split) { g.splits = sk.splits; g.part = (int32_t*)sk.part; }
        // 128 x 128 tiles also when 256 x 256 ones would be at most 64, a quarter of the CUs (1024 x 4096 x 4096: 22.9 against 28.0 us; at 128 tiles of 256 x 256 it is 42 against 32)
        const int64_t t256 = ((a.M + 255) / 256) * ((a.N + 255) / 256) * a.batch;
        if (small || t256 <= 64 || a.force_variant == OPSNN_VARIANT_MX_128) {
            if (split) return qgemm_launch_split_mx<MODE_MXFP4, 128, 128, 64, 2, 2, 4, 1>(g, a.batch, a.out_dtype, st);
            return qgemm_launch<MODE_MXFP4, 128, 128, 64, 2, 2, 4, 1>(g, a.batch, a.out_dtype, st);
        }
        // K tiles of 128 bytes (256 elements) with the scales of two tiles per 16-byte copy: needs an even number of
        // such tiles and 16-byte aligned scale rows
        const bool sc16 = a.K % 512 == 0 &&
                          (((uintptr_t)g.sa | (uintptr_t)g.sb | (uint64_t)g.sa_rs | (uint64_t)g.sb_rs | (uint64_t)g.sa_bs | (uint64_t)g.sb_bs) % 16) == 0;
        if (sc16) {
            if (split) return qgemm_launch_split_mx<MODE_MXFP4, 256, 256, 128, 2, 4, 2, 1>(g, a.batch, a.out_dtype, st);
            return qgemm_launch<MODE_MXFP4, 256, 256, 128, 2, 4, 2, 1>(g, a.batch, a.out_dtype, st);
        }
        if (split) return qgemm_launch_split_mx<MODE_MXFP4, 256, 256, 64, 2, 2, 4, 1>(g, a.batch, a.out_dtype, st);
        return qgemm_launch<MODE_MXFP4, 256, 256, 64, 2, 2, 4, 1>(g, a.batch, a.out_dtype, st);
    }
    // FLOAT output: the tile kernel, whose epilogue stores fp32 straight from the registers
    if (a.out_dtype == DT_F32 || a.force_variant == OPSNN_VARIANT_MX_FP8_MFMA || a.force_variant == OPSNN_VARIANT_MX_128) {   // (also the chained-K variants of the tests)
        if (small || a.force_variant == OPSNN_VARIANT_MX_128) return qgemm_launch<MODE_MXFP8, 128, 128, 128, 2, 2, 2, 1>(g, a.batch, a.out_dtype, st);
        return qgemm_launch<MODE_MXFP8, 256, 256, 128, 2, 2, 2, 1>(g, a.batch, a.out_dtype, st);
    }
    // few rows: the 128 x 128 tiles of the tile kernel (the block kernel's 128 x 256 tiles leave most CUs' matrix work on
    // rows that do not exist and half as many workgroups to stream x2)
    if (a.M <= 256) return qgemm_launch<MODE_MXFP8, 128, 128, 128, 2, 2, 2, 1>(g, a.batch, a.out_dtype, st);
    return launch_mxfp8_mfma(a, st);
}

}  // namespace opsnn
