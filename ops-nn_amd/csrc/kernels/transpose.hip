// Dense 2-D transposes of 8-bit and packed 4-bit matrices: the offline relayout that turns an
// N-contiguous right operand ([K, N] rows) into the K-contiguous form the MFMA kernels stream.
// Stands where the reference converts ND weights to its fractal NZ layout
// (matmul/convert_weight_to_int4_pack/op_host/op_api/aclnn_convert_weight_to_int4_pack.cpp:318-366).
#include "common.hip.h"
#include "launch.h"

namespace opsnn {

// 64x64 byte tile through LDS (+4 pad keeps the column reads off one bank).
__global__ __launch_bounds__(256) void transpose8_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                         int64_t rows, int64_t cols)
{
    __shared__ uint8_t tile[64][68];
    const int64_t bz = blockIdx.z;
    src += bz * rows * cols;
    dst += bz * rows * cols;
    const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int i = ty; i < 64; i += 4) {
        int64_t r = r0 + i, c = c0 + tx;
        tile[i][tx] = (r < rows && c < cols) ? src[r * cols + c] : 0;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        int64_t c = c0 + i, r = r0 + tx;
        if (c < cols && r < rows) dst[c * rows + r] = tile[tx][i];
    }
}

// 4-bit: src byte (r, c/2) holds columns c (low nibble) and c+1; dst byte (c, r/2) holds rows r (low) and r+1.
__global__ __launch_bounds__(256) void transpose4_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                         int64_t rows, int64_t cols)
{
    __shared__ uint8_t tile[64][68];  // one nibble per byte
    const int64_t bz = blockIdx.z;
    src += bz * rows * (cols / 2);
    dst += bz * cols * (rows / 2);
    const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 bytes = 64 nibbles per row
    for (int i = ty; i < 64; i += 8) {
        int64_t r = r0 + i, c = c0 + 2 * tx;
        uint8_t b = (r < rows && c < cols) ? src[r * (cols / 2) + c / 2] : 0;
        tile[i][2 * tx] = b & 15u;
        tile[i][2 * tx + 1] = b >> 4;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 8) {
        int64_t c = c0 + i, r = r0 + 2 * tx;
        if (c < cols && r < rows) dst[c * (rows / 2) + r / 2] = (uint8_t)(tile[2 * tx][i] | (tile[2 * tx + 1][i] << 4));
    }
}

// dst (dense [batch, rows, cols], two elements per byte, low nibble = even column) = the 4-bit elements at
// off + b * bs + r * rs + c * cs (in elements) of the packed storage at base: any view whose batch dims collapse into one stride
__global__ __launch_bounds__(256) void gather4_kernel(const uint8_t* __restrict__ base, int64_t off, int64_t rows, int64_t cols,
                                                      int64_t bs, int64_t rs, int64_t cs, uint8_t* __restrict__ dst)
{
    const int64_t cb = (int64_t)blockIdx.x * 256 + threadIdx.x, b = blockIdx.z;
    if (2 * cb >= cols) return;
    for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) {
        const int64_t e0 = off + b * bs + r * rs + 2 * cb * cs, e1 = e0 + cs;
        const uint32_t n0 = (base[e0 >> 1] >> ((e0 & 1) * 4)) & 15u, n1 = (base[e1 >> 1] >> ((e1 & 1) * 4)) & 15u;
        dst[(b * rows + r) * (cols / 2) + cb] = (uint8_t)(n0 | (n1 << 4));
    }
}

// the same for 8-bit elements
__global__ __launch_bounds__(256) void gather8_kernel(const uint8_t* __restrict__ base, int64_t off, int64_t rows, int64_t cols,
                                                      int64_t bs, int64_t rs, int64_t cs, uint8_t* __restrict__ dst)
{
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x, b = blockIdx.z;
    if (c >= cols) return;
    for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) dst[(b * rows + r) * cols + c] = base[off + b * bs + r * rs + c * cs];
}

}  // namespace opsnn

using namespace opsnn;

extern "C" int opsnnGather8(const void* base, int64_t offset, int64_t batch, int64_t rows, int64_t cols, int64_t batch_stride, int64_t row_stride,
                            int64_t col_stride, void* dst, void* stream)
{
    if (!base || !dst || rows <= 0 || cols <= 0 || batch <= 0 || batch > 65535) return -1;
    if (offset < 0 || batch_stride < 0 || row_stride < 0 || col_stride < 0) return -1;
    dim3 grid((unsigned)((cols + 255) / 256), (unsigned)(rows < 65535 ? rows : 65535), (unsigned)batch);
    hipLaunchKernelGGL(gather8_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const uint8_t*)base, offset, rows, cols, batch_stride, row_stride,
                       col_stride, (uint8_t*)dst);
    return (int)hipGetLastError();
}

extern "C" int opsnnGather4(const void* base, int64_t offset, int64_t batch, int64_t rows, int64_t cols, int64_t batch_stride, int64_t row_stride,
                            int64_t col_stride, void* dst, void* stream)
{
    if (!base || !dst || rows <= 0 || cols <= 0 || batch <= 0 || batch > 65535 || (cols & 1)) return -1;
    if (offset < 0 || batch_stride < 0 || row_stride < 0 || col_stride < 0) return -1;
    dim3 grid((unsigned)((cols / 2 + 255) / 256), (unsigned)(rows < 65535 ? rows : 65535), (unsigned)batch);
    hipLaunchKernelGGL(gather4_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const uint8_t*)base, offset, rows, cols, batch_stride, row_stride,
                       col_stride, (uint8_t*)dst);
    return (int)hipGetLastError();
}

extern "C" int opsnnTranspose8(const void* src, void* dst, int64_t rows, int64_t cols, int64_t batch, void* stream)
{
    if (!src || !dst || rows <= 0 || cols <= 0 || batch <= 0 || batch > 65535) return -1;
    dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64), (unsigned)batch);
    if (grid.y > 65535u) return -2;
    hipLaunchKernelGGL(transpose8_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const uint8_t*)src, (uint8_t*)dst,
                       rows, cols);
    return (int)hipGetLastError();
}

extern "C" int opsnnTranspose4(const void* src, void* dst, int64_t rows, int64_t cols, int64_t batch, void* stream)
{
    if (!src || !dst || rows <= 0 || cols <= 0 || batch <= 0 || batch > 65535) return -1;
    if ((rows & 1) || (cols & 1)) return -3;
    dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64), (unsigned)batch);
    if (grid.y > 65535u) return -2;
    hipLaunchKernelGGL(transpose4_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const uint8_t*)src, (uint8_t*)dst,
                       rows, cols);
    return (int)hipGetLastError();
}

extern "C" int opsnnDeviceInfo(int* cu_count, int* clock_khz, int64_t* hbm_bytes, char* arch, int arch_len)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return (int)e;
    if (cu_count) *cu_count = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    if (hbm_bytes) *hbm_bytes = (int64_t)prop.totalGlobalMem;
    if (arch && arch_len > 0) {
        int i = 0;
        for (; i < arch_len - 1 && prop.gcnArchName[i]; i++) arch[i] = prop.gcnArchName[i];
        arch[i] = 0;
    }
    return 0;
}
