// FRACTAL_NZ <-> ND re-layout of a byte matrix: the reference's cube layout of a right operand, accepted by the
// ...WeightNz / ...Nz entry points and produced by aclnnConvertWeightToINT4Pack when asked for.
//
// A [rows, row_bytes] matrix in NZ form is the 4-D array [ceil(row_bytes / c0), ceil(rows / 16), 16, c0]:
//     nz[b / c0][r / 16][r % 16][b % c0] = nd[r][b]
// (matmul/common/tests/st/arch35/matmul_golden_util.py:76-114 and :284-313;
//  matmul/convert_weight_to_int4_pack/op_host/op_api/aclnn_convert_weight_to_int4_pack.cpp:318-366), padding zero.
// c0 is 32 bytes for 8-bit elements and 8 or 16 bytes (16 or 32 elements) for 4-bit elements.
#include "common.hip.h"
#include "launch.h"

namespace opsnn {

// One thread per 8-byte piece; 16 consecutive threads take the 16 rows of one fractal, so the NZ side is accessed in
// contiguous runs of 16 * c0 bytes and the ND side in pieces of c0 bytes per row.
template <bool TO_ND>
__global__ __launch_bounds__(256) void nz_relayout_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int64_t rows,
                                                          int64_t row_bytes, int c0, int64_t pieces_per_row, int64_t y1)
{
    const int64_t bz = blockIdx.y;
    const int64_t x1 = (row_bytes + c0 - 1) / c0;
    const uint8_t* s = src + bz * (TO_ND ? x1 * y1 * 16 * c0 : rows * row_bytes);
    uint8_t* d = dst + bz * (TO_ND ? rows * row_bytes : x1 * y1 * 16 * c0);
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    // t = ((rblk * pieces_per_row) + p) * 16 + r0
    const int r0 = (int)(t & 15);
    const int64_t q = t >> 4;
    const int64_t p = q % pieces_per_row, rblk = q / pieces_per_row;
    const int64_t r = rblk * 16 + r0;
    if (rblk >= y1) return;
    const int64_t b0 = p * 8;
    const int64_t nz_off = (b0 / c0) * (y1 * 16 * c0) + rblk * (16 * c0) + (int64_t)r0 * c0 + (b0 % c0);
    const int64_t nd_off = r * row_bytes + b0;
    const int n = (int)((row_bytes - b0) < 8 ? (row_bytes - b0) : 8);
    if (TO_ND) {
        if (r >= rows) return;
        if (n == 8 && ((uintptr_t)(s + nz_off) % 8) == 0 && ((uintptr_t)(d + nd_off) % 8) == 0) {
            *(uint64_t*)(d + nd_off) = *(const uint64_t*)(s + nz_off);
        } else {
            for (int i = 0; i < n; i++) d[nd_off + i] = s[nz_off + i];
        }
    } else {
        // padding rows and padding bytes of the fractals are written as zero
        uint8_t v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        if (r < rows)
            for (int i = 0; i < n; i++) v[i] = s[nd_off + i];
        for (int i = 0; i < 8 && (b0 % c0) + i < c0; i++) d[nz_off + i] = v[i];
    }
}

}  // namespace opsnn

using namespace opsnn;

static int nz_launch(bool to_nd, const void* src, void* dst, int64_t rows, int64_t row_bytes, int c0, int64_t batch, void* stream)
{
    if (!src || !dst || rows <= 0 || row_bytes <= 0 || batch <= 0 || batch > 65535) return -1;
    if (c0 != 8 && c0 != 16 && c0 != 32) return -2;
    const int64_t y1 = (rows + 15) / 16;
    // NZ -> ND needs the pieces that hold data; ND -> NZ also writes the padding pieces up to a whole c0
    const int64_t pieces = to_nd ? (row_bytes + 7) / 8 : ((row_bytes + c0 - 1) / c0) * (c0 / 8);
    const int64_t threads = y1 * pieces * 16;
    const int64_t blocks = (threads + 255) / 256;
    if (blocks > 0x7fffffffll) return -3;
    dim3 grid((unsigned)blocks, (unsigned)batch);
    if (to_nd)
        hipLaunchKernelGGL(nz_relayout_kernel<true>, grid, dim3(256), 0, (hipStream_t)stream, (const uint8_t*)src, (uint8_t*)dst, rows,
                           row_bytes, c0, pieces, y1);
    else
        hipLaunchKernelGGL(nz_relayout_kernel<false>, grid, dim3(256), 0, (hipStream_t)stream, (const uint8_t*)src, (uint8_t*)dst, rows,
                           row_bytes, c0, pieces, y1);
    return (int)hipGetLastError();
}

extern "C" int opsnnNzToNd(const void* nz, void* nd, int64_t rows, int64_t row_bytes, int c0_bytes, int64_t batch, void* stream)
{
    return nz_launch(true, nz, nd, rows, row_bytes, c0_bytes, batch, stream);
}
extern "C" int opsnnNdToNz(const void* nd, void* nz, int64_t rows, int64_t row_bytes, int c0_bytes, int64_t batch, void* stream)
{
    return nz_launch(false, nd, nz, rows, row_bytes, c0_bytes, batch, stream);
}
