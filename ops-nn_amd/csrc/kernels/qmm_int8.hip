// int8 x int8 -> int32 quantized matmul with the fused per-token / per-channel dequant epilogue
// (K-C, K-T and dynamic T-C modes).  gfx950 only.
//
//   acc[m,n] = sum_k int32(x1[m,k]) * int32(x2[k,n])                 exact
//   out[m,n] = cast( fp32(acc + int32 bias[n]) * x2Scale[n] * x1Scale[m] + float bias[n] )
//
// The multiplication order and the place of the bias follow the reference's golden
// (matmul/quant_batch_matmul_v3/tests/assets/qbmmv3_kernel_golden.py:361-387) and its device epilogue
// (matmul/quant_batch_matmul_v3/op_kernel/arch35/qbmm_mix_online_dynamic.h:648-736).
//
// Fast path: both operands K-contiguous ("x2 stored [N, K]"), 16-byte aligned rows: the shared MFMA tile
// kernel of qgemm_core.hip.h in MODE_I8.  Anything else (odd K, unaligned or strided operands, int32 or fp32
// output) runs the plain strided kernel below.
#include <cstdlib>

#include "launch.h"
#include "qgemm_core.hip.h"

namespace opsnn {
const void* weight_cache_get(const void* src, int64_t K, int64_t N, int bits, int64_t nb, hipStream_t st);   // weight_cache.hip

struct QmmI8Params {
    const int8_t* a;  // x1
    const int8_t* b;  // x2
    int64_t a_rs, a_cs, a_bs;  // strides of logical [M,K]
    int64_t b_rs, b_cs, b_bs;  // strides of logical [K,N]
    void* out;
    int64_t M, N, K;
    const float* x1s;
    const void* x2s;
    int x2s_dt;
    int64_t x2s_len;
    int x2s_trunc;
    const void* bias;
    int bias_dt;
    int64_t bias_bs;
    int out_dt;
};

// ---------------------------------------------------------------------------------------------
// Plain strided kernel: one thread per output element.  Any strides, any K.
// ---------------------------------------------------------------------------------------------
__global__ void qmm_i8_plain(QmmI8Params p)
{
    const int64_t nchunks = (p.N + blockDim.x - 1) / blockDim.x;
    int64_t m = blockIdx.x / nchunks;
    int64_t n = (blockIdx.x % nchunks) * (int64_t)blockDim.x + threadIdx.x;
    int64_t bz = blockIdx.y;
    if (n >= p.N) return;
    const int8_t* a = p.a + bz * p.a_bs + m * p.a_rs;
    const int8_t* b = p.b + bz * p.b_bs + n * p.b_cs;
    int32_t acc = 0;
    for (int64_t k = 0; k < p.K; k++) acc += (int32_t)a[k * p.a_cs] * (int32_t)b[k * p.b_rs];
    int64_t o = (bz * p.M + m) * p.N + n;
    if (p.out_dt == DT_I32) {
        if (p.bias && p.bias_dt == DT_I32) acc += ((const int32_t*)p.bias)[bz * p.bias_bs + n];
        ((int32_t*)p.out)[o] = acc;
        return;
    }
    if (p.bias && p.bias_dt == DT_I32) acc += ((const int32_t*)p.bias)[bz * p.bias_bs + n];
    float v = (float)acc;
    {
        const int64_t si = p.x2s_len == 1 ? 0 : n;
        float sv = p.x2s_dt == DT_U64 ? u2f((uint32_t)((const uint64_t*)p.x2s)[si]) : load_scalar_as_f32(p.x2s, p.x2s_dt, si);
        if (p.x2s_trunc || p.x2s_dt == DT_U64) sv = u2f(f2u(sv) & 0xFFFFE000u);
        v = v * sv;
    }
    if (p.x1s) v = v * p.x1s[m];
    if (p.bias && p.bias_dt != DT_I32) v = v + load_scalar_as_f32(p.bias, p.bias_dt, bz * p.bias_bs + n);
    store_f32_as(p.out, p.out_dt, o, v);
}

}  // namespace opsnn

using namespace opsnn;

extern "C" bool opsnn_force_plain();
extern "C" void opsnn_note_plain(const char* mode, int forced, int64_t batch, int64_t M, int64_t N, int64_t K);   // dispatch.hip
namespace opsnn {
int launch_int8_wide(const QgemmParams& p, int fn, int64_t batch, int out_dt, hipStream_t st);   // qmm_int8_wide.hip
}

static int64_t cu_count()
{
    static const int n = [] {
        int d = 0, c = 0;
        if (hipGetDevice(&d) != hipSuccess || hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, d) != hipSuccess || c <= 0) c = 256;
        return c;
    }();
    return n;
}

// OPSNN_NOT_TAKEN: an INT8 output was asked for and the shape does not fit the MFMA kernels (the caller falls back).
extern "C" __attribute__((visibility("hidden"))) int opsnn_qmm_int8_impl(const OpsnnQmmArgs* a, void* stream);
extern "C" __attribute__((visibility("hidden"))) int opsnn_qmm_k_pad(const OpsnnQmmArgs* a, int mode, void* stream, OpsnnQmmArgs* b);   // dispatch.hip
extern "C" __attribute__((visibility("hidden"))) void opsnn_qmm_splitk_carve(const OpsnnQmmArgs* a, int mode, OpsnnQmmArgs* c, SplitK* sk);   // dispatch.hip
static int qmm_int8_impl(const OpsnnQmmArgs* a, void* stream, SplitK sk);
extern "C" int opsnnQmmInt8(const OpsnnQmmArgs* a, void* stream)
{
    WeightCacheScope cache_scope;
    OpsnnQmmArgs padded, carved;
    SplitK sk;
    if (a && a->x1.ptr && a->x2.ptr && a->M > 0 && a->N > 0 && a->K > 0 && a->batch > 0) {
        opsnn_qmm_splitk_carve(a, 0, &carved, &sk);   // few tiles against a long K: the partial sums of a K split come first in the workspace
        a = &carved;
        const int prc = opsnn_qmm_k_pad(a, 0, stream, &padded);   // K % 16 != 0: zero-padded K-contiguous copies
        if (prc == 0) a = &padded;
        else if (prc != OPSNN_NOT_TAKEN) return prc;
    }
    const int rc = qmm_int8_impl(a, stream, sk);
    return rc == OPSNN_NOT_TAKEN ? -2 : rc;
}
extern "C" int opsnn_qmm_int8_impl(const OpsnnQmmArgs* a, void* stream) { return qmm_int8_impl(a, stream, SplitK{}); }
// opsnnQmmInt8 without the K split: the workspace is opsnn_qmm_workspace_base(a, 0) bytes (for the entry point whose
// workspace is a fixed array)
extern "C" __attribute__((visibility("hidden"))) int opsnn_qmm_int8_nosplit(const OpsnnQmmArgs* a, void* stream)
{
    WeightCacheScope cache_scope;
    OpsnnQmmArgs padded;
    if (a && a->x1.ptr && a->x2.ptr && a->M > 0 && a->N > 0 && a->K > 0 && a->batch > 0) {
        const int prc = opsnn_qmm_k_pad(a, 0, stream, &padded);
        if (prc == 0) a = &padded;
        else if (prc != OPSNN_NOT_TAKEN) return prc;
    }
    const int rc = qmm_int8_impl(a, stream, SplitK{});
    return rc == OPSNN_NOT_TAKEN ? -2 : rc;
}
static int qmm_int8_impl(const OpsnnQmmArgs* a, void* stream, SplitK sk)
{
    if (!a || !a->x1.ptr || !a->x2.ptr || !a->out || !a->x2_scale) return -1;
    if (a->x1_dtype != DT_I8 || a->x2_dtype != DT_I8) return -2;
    if (a->M <= 0 || a->N <= 0 || a->K <= 0 || a->batch <= 0) return -3;
    hipStream_t st = (hipStream_t)stream;
    QmmI8Params p;
    p.a = (const int8_t*)a->x1.ptr; p.a_rs = a->x1.row_stride; p.a_cs = a->x1.col_stride; p.a_bs = a->x1.batch_stride;
    p.b = (const int8_t*)a->x2.ptr; p.b_rs = a->x2.row_stride; p.b_cs = a->x2.col_stride; p.b_bs = a->x2.batch_stride;
    p.out = a->out; p.M = a->M; p.N = a->N; p.K = a->K;
    p.x1s = (const float*)a->x1_scale; p.x2s = a->x2_scale; p.x2s_dt = a->x2_scale_dtype; p.x2s_len = a->x2_scale_len; p.x2s_trunc = a->x2_scale_trunc;
    p.bias = a->bias; p.bias_dt = a->bias_dtype; p.bias_bs = a->bias_batch_stride; p.out_dt = a->out_dtype;

    // x2 stored N-major ([K, N] rows): relayout into the workspace as [N, K] first.
    bool b_kmajor = (p.b_rs == 1);
    bool a_kmajor = (p.a_cs == 1);
    // INT32 / INT8 outputs (the static-quantisation modes: no per-token scale; bias absent or INT32) run on the 8-wave tile
    // kernels with an integer epilogue
    const bool int_out = (p.out_dt == DT_I32 || p.out_dt == DT_I8) && !a->x1_scale && (!a->bias || a->bias_dtype == DT_I32);
    bool b16 = (p.out_dt == DT_BF16 || p.out_dt == DT_F16) || int_out;
    int variant = a->force_variant;
    if (opsnn_force_plain()) variant = OPSNN_VARIANT_PLAIN;
    // (fewer than 64 x 64 outputs stay on the plain kernel unless K is long: one row against 3584 x 18944 is no work for one
    // thread per output -- 2.4 ms there, 20 us on a 128 x 128 tile with K split)
    const bool enough = p.M * p.N >= 64 * 64 || (p.N >= 256 && p.M * p.N * p.K >= (1ll << 22));
    bool want_fast = b16 && a_kmajor && variant != OPSNN_VARIANT_PLAIN && enough && (p.K % 16) == 0 &&
                     (p.a_rs % 16) == 0 && ((uintptr_t)p.a % 16) == 0 && (p.a_bs % 16) == 0;
    if (want_fast && !b_kmajor && p.b_cs == 1 && p.b_rs == p.N && (p.b_bs == 0 || p.b_bs == p.K * p.N)) {
        int64_t nb = p.b_bs == 0 ? 1 : a->batch;
        const void* copy = weight_cache_get(p.b, p.K, p.N, 8, nb, st);   // the weight cache, when it is switched on
        if (!copy && a->workspace) {
            int rc = opsnnTranspose8(p.b, a->workspace, p.K, p.N, nb, stream);
            if (rc != 0) return rc;
            copy = a->workspace;
        }
        if (copy) {
            p.b = (const int8_t*)copy; p.b_rs = 1; p.b_cs = p.K; p.b_bs = p.b_bs == 0 ? 0 : p.K * p.N;
            b_kmajor = true;
        }
    }
    bool fast = want_fast && b_kmajor && (p.b_cs % 16) == 0 && ((uintptr_t)p.b % 16) == 0 && (p.b_bs % 16) == 0;
    if (fast) {
        QgemmParams g{};
        g.a = p.a; g.b = p.b; g.lda = p.a_rs; g.ldb = p.b_cs; g.a_bs = p.a_bs; g.b_bs = p.b_bs;
        g.out = p.out; g.M = p.M; g.N = p.N; g.ldc = p.N; g.KB = p.K;
        g.x1s = p.x1s; g.x2s = p.x2s; g.x2s_dt = p.x2s_dt; g.x2s_len = p.x2s_len; g.x2s_trunc = a->x2_scale_trunc;
        g.bias = p.bias; g.bias_dt = p.bias_dt; g.bias_bs = p.bias_bs;
        if (int_out) {
            g.x2off = a->x2_offset; g.x2off_len = a->x2_offset_len;
            if (p.M <= 128 || p.N <= 128 || p.M * p.N <= 256 * 256 * 64) return qgemm_launch_int<128, 128, 128, 2, 2, 2, 1>(g, a->batch, p.out_dt, st);
            // the four-wave kernel under the conditions and with the tile width of the 16-bit outputs below
            const int64_t cus = cu_count();
            const int64_t tm = (p.M + 255) / 256, tn = (p.N + 255) / 256;
            // (OPSNN_VARIANT_I8_256_W8_K128 keeps the call on the 8-wave kernel: the tests compare the two)
            if (variant != OPSNN_VARIANT_I8_256_W8_K128 && p.K % 128 == 0 && p.K >= 3072 && tm * tn * a->batch * 4 >= cus * 3) {
                int64_t best = INT64_MAX;
                int best_fn = 0;
                for (int fn = 8; fn <= 11; fn++) {
                    const int64_t tiles = tm * ((p.N + 32 * fn - 1) / (32 * fn)) * a->batch;
                    const int64_t cost = (tiles + cus - 1) / cus * (fn + 2);
                    if (cost < best) { best = cost; best_fn = fn; }
                }
                if (best <= (tm * tn * a->batch + cus - 1) / cus * 10) {
                    const int rc = launch_int8_wide(g, best_fn, a->batch, p.out_dt, st);
                    if (rc != OPSNN_NOT_TAKEN) return rc;
                }
            }
            return qgemm_launch_int<256, 256, 128, 2, 4, 2, 1>(g, a->batch, p.out_dt, st);
        }
        if (variant >= OPSNN_VARIANT_I8_WIDE8 && variant <= OPSNN_VARIANT_I8_WIDE11) {
            const int rc = launch_int8_wide(g, variant, a->batch, p.out_dt, st);
            if (rc != OPSNN_NOT_TAKEN) return rc;
        }
        switch (variant) {
            case OPSNN_VARIANT_I8_256: return qgemm_launch<MODE_I8, 256, 256, 128, 2, 2, 2, 1>(g, a->batch, p.out_dt, st);
            case OPSNN_VARIANT_I8_128: return qgemm_launch<MODE_I8, 128, 128, 128, 2, 2, 2, 1>(g, a->batch, p.out_dt, st);
            case OPSNN_VARIANT_I8_256x128_S3: return qgemm_launch<MODE_I8, 256, 128, 64, 2, 2, 3, 2>(g, a->batch, p.out_dt, st);
            case OPSNN_VARIANT_I8_256_W8: return qgemm_launch<MODE_I8, 256, 256, 64, 2, 4, 4, 1>(g, a->batch, p.out_dt, st);
            case OPSNN_VARIANT_I8_256_S4: return qgemm_launch<MODE_I8, 256, 256, 64, 2, 2, 4, 1>(g, a->batch, p.out_dt, st);
            case OPSNN_VARIANT_I8_256_W8_K128: return qgemm_launch<MODE_I8, 256, 256, 128, 2, 4, 2, 1>(g, a->batch, p.out_dt, st);
            default: break;
        }
        if (p.M <= 128 || p.N <= 128 || p.M * p.N <= 256 * 256 * 64) {
            if (sk.splits > 1 && p.K % 128 == 0) {   // few tiles against a long K: K split over workgroups, integer partial sums
                g.splits = sk.splits; g.part = (int32_t*)sk.part;
                return qgemm_launch_split_i8<128, 128, 128, 2, 2, 2, 1>(g, a->batch, p.out_dt, st);
            }
            return qgemm_launch<MODE_I8, 128, 128, 128, 2, 2, 2, 1>(g, a->batch, p.out_dt, st);
        }
        // Large shapes: 256x256 tiles, one per CU at a time, are the most economical in operand traffic, but only
        // whole rounds of them keep every CU busy.  Columns that fill whole rounds go to that kernel; the remaining
        // columns (less than one round) go to 128x128 tiles, two workgroups per CU, in a second launch.
        const int64_t cus = cu_count();
        const int64_t tm = (p.M + 255) / 256, tn = (p.N + 255) / 256;
        // Cost of a strategy in units of "one round of tiles, per 32 columns of tile width".  The four-wave kernel
        // takes tiles of 256 x 32n columns, n = 8..11: the width whose tile count wastes the least of its last round
        // wins (2048 x 11008: 256 tiles of 352 columns, one round, 13 units against 10 + 6 for the split below).
        int64_t wide_cost = INT64_MAX;
        int wide_fn = 0;
        // (from 24 K tiles up: with fewer the 8-wave kernels, whose second wave per SIMD covers prologue and epilogue,
        // are ahead -- 8192 x 1024 x 8192: 96 against 114 us, 4096 x 2048 x 14336: 147 against 154; and from 3/4 of a round of 256 x 256 tiles up)
        if (p.K % 128 == 0 && p.K >= 3072 && tm * tn * a->batch * 4 >= cus * 3) {
            for (int fn = 8; fn <= 11; fn++) {
                const int64_t tiles = tm * ((p.N + 32 * fn - 1) / (32 * fn)) * a->batch;
                const int64_t cost = (tiles + cus - 1) / cus * (fn + 2);   // + 2: what a tile costs beyond its width (8192^3: 3 rounds of 352 columns 495 us, 4 of 256 529 us)
                if (cost < wide_cost) { wide_cost = cost; wide_fn = fn; }
            }
        }
        if (p.K >= 1024 && tm * tn * a->batch >= cus && a->batch == 1) {
            const int64_t rounds = tm * tn / cus;
            const int64_t cols_a = rounds * cus / tm;            // column tiles in whole rounds
            const bool split_ok = cols_a >= 1 && cols_a * tm * 8 >= rounds * cus * 7;   // at least 7/8 of those rounds is filled
            const int64_t split_cost = split_ok ? rounds * 10 + (cols_a * 256 < p.N ? 6 : 0) : INT64_MAX;   // measured: the remainder launch costs 5/8 of a round
            if (wide_fn && wide_cost <= split_cost) {
                const int rc = launch_int8_wide(g, wide_fn, a->batch, p.out_dt, st);
                if (rc != OPSNN_NOT_TAKEN) return rc;
            }
            if (split_ok) {
                const int64_t na = cols_a * 256 < p.N ? cols_a * 256 : p.N;
                QgemmParams ga = g;
                ga.N = na;
                int rc = qgemm_launch<MODE_I8, 256, 256, 128, 2, 4, 2, 1>(ga, 1, p.out_dt, st);
                if (rc != 0 || na == p.N) return rc;
                QgemmParams gb = g;
                gb.N = p.N - na;
                gb.b = g.b + na * g.ldb;
                gb.out = (uint16_t*)g.out + na;
                if (g.x2s_len != 1) gb.x2s = (const char*)g.x2s + na * (g.x2s_dt == DT_U64 ? 8 : g.x2s_dt == DT_F32 ? 4 : 2);
                if (g.bias) gb.bias = (const char*)g.bias + na * (g.bias_dt == DT_I32 || g.bias_dt == DT_F32 ? 4 : 2);
                return qgemm_launch<MODE_I8, 128, 128, 128, 2, 2, 2, 1>(gb, 1, p.out_dt, st);
            }
        }
        if (wide_fn) {
            const int rc = launch_int8_wide(g, wide_fn, a->batch, p.out_dt, st);
            if (rc != OPSNN_NOT_TAKEN) return rc;
        }
        return qgemm_launch<MODE_I8, 256, 128, 64, 2, 2, 3, 2>(g, a->batch, p.out_dt, st);
    }
    if (p.out_dt == DT_I8) return OPSNN_NOT_TAKEN;   // the strided kernel below has no requantising epilogue
    opsnn_note_plain("int8 per-token x per-channel quant matmul", variant == OPSNN_VARIANT_PLAIN, a->batch, p.M, p.N, p.K);
    dim3 block(256), grid((unsigned)(((p.N + 255) / 256) * p.M), (unsigned)a->batch);
    hipLaunchKernelGGL(qmm_i8_plain, grid, block, 0, st, p);
    return (int)hipGetLastError();
}

