// Launcher entry points for the block-scale, MX and weight-only paths, and workspace sizing.
// Each launcher first offers the call to the MFMA kernel family for that mode; whatever that family
// does not take (odd shapes, strided layouts, rarely used dtype pairs) runs on the plain kernels.
#include <cstdlib>

#include "common.hip.h"
#include "launch.h"

namespace opsnn {
int launch_blockscale_plain(const OpsnnQmmArgs& a, hipStream_t st);
int launch_mx_plain(const OpsnnQmmArgs& a, hipStream_t st);
int launch_tc_plain(const OpsnnQmmArgs& a, hipStream_t st);
int launch_group_plain(const OpsnnQmmArgs& a, bool tcg, hipStream_t st);
int launch_wqmm_plain(const OpsnnWqmmArgs& a, hipStream_t st);
// Return OPSNN_NOT_TAKEN when the arguments are outside what the fast kernels handle.
int launch_blockscale_mfma(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk = {});
int launch_fp8_rowcol_mfma(const OpsnnQmmArgs& a, hipStream_t st, bool merged_scales_ok, SplitK sk = {});
int launch_rowcol_exact(const OpsnnQmmArgs& a, hipStream_t st, int ep_mode, SplitK sk = {});   // qmm_fp8_exact.hip
int launch_rowcol_decode(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk);   // qmm_fp8_decode.hip
uint64_t blockscale_rows_workspace(const OpsnnQmmArgs& a);         // qmm_fp8_rows.hip
int blockscale_rows_ksplit(const OpsnnQmmArgs& a);
uint64_t rowcol_rows_workspace(const OpsnnQmmArgs& a);
int launch_rowcol_rows(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk);
int rowcol_rows_ksplit(const OpsnnQmmArgs& a);
int mxfp8_rows_ksplit(const OpsnnQmmArgs& a);
int launch_tcg_mfma(const OpsnnQmmArgs& a, hipStream_t st);
uint64_t tcg_workspace_bytes(const OpsnnQmmArgs& a);
int launch_kg_mfma(const OpsnnQmmArgs& a, hipStream_t st);   // qmm_i4_kg.hip
uint64_t kg_workspace_bytes(const OpsnnQmmArgs& a);
int launch_mx_mfma(const OpsnnQmmArgs& a, hipStream_t st, SplitK sk = {});
int launch_wqmm_mfma(const OpsnnWqmmArgs& a, hipStream_t st);
uint64_t mx_workspace_bytes(const OpsnnQmmArgs& a);
}  // namespace opsnn

using namespace opsnn;

// Routing switches, process-wide.  OPSNN_FORCE_PLAIN is read ONCE when the library is loaded (no getenv on the call
// path); every switch can be changed at run time through its setter.
//   OPSNN_FORCE_PLAIN=1 / opsnnSetForcePlain(1): every call runs on the plain one-thread-per-output kernels (the parity
//   tests compare them bit for bit with the oracle);
//   opsnnSetMx8Wide(n) (test hook): MXFP8 on the four-wave kernel with 256 x 32n tiles, n = 8 or 9; 0 never; -1 the selector
//   decides (default);
//   opsnnSetWqTileMin(m) (test hook): weight-only int4/int8 calls with m .. 256 rows of x run on the dequantise-once tile
//   kernel (default 129: below that the streaming kernels are faster);
//   opsnnSetWqNarrowSlabs(on) (test hook): 0 keeps weight-only calls against a narrow weight (at most 128 workgroups of 128
//   columns) on one pass per launch, as wide ones run, so that small test shapes reach every instance of the many-rows kernel
//   (default 1: their rows go out as equal slabs in one launch).
static int g_wq_tile_min = 129;
static int g_wq_narrow_slabs = 1;
extern "C" void opsnnSetWqNarrowSlabs(int on) { __atomic_store_n(&g_wq_narrow_slabs, on ? 1 : 0, __ATOMIC_RELAXED); }
extern "C" __attribute__((visibility("hidden"))) int opsnn_wq_narrow_slabs() { return __atomic_load_n(&g_wq_narrow_slabs, __ATOMIC_RELAXED); }
extern "C" void opsnnSetWqTileMin(int m) { __atomic_store_n(&g_wq_tile_min, m, __ATOMIC_RELAXED); }
extern "C" __attribute__((visibility("hidden"))) int opsnn_wq_tile_min() { return __atomic_load_n(&g_wq_tile_min, __ATOMIC_RELAXED); }
static int g_force_plain = [] { const char* e = getenv("OPSNN_FORCE_PLAIN"); return (e && *e && *e != '0') ? 1 : 0; }();
static int g_mx8_wide = -1;
extern "C" void opsnnSetForcePlain(int on) { __atomic_store_n(&g_force_plain, on ? 1 : 0, __ATOMIC_RELAXED); }
extern "C" void opsnnSetMx8Wide(int n) { __atomic_store_n(&g_mx8_wide, n, __ATOMIC_RELAXED); }
extern "C" __attribute__((visibility("hidden"))) bool opsnn_force_plain() { return __atomic_load_n(&g_force_plain, __ATOMIC_RELAXED) != 0; }
extern "C" __attribute__((visibility("hidden"))) int opsnn_mx8_wide() { return __atomic_load_n(&g_mx8_wide, __ATOMIC_RELAXED); }

// A hook of the parity tests: fills the LDS of every compute unit with all-ones bytes (NaN as fp32, fp16, bf16 and e4m3), so
// that a kernel launched next which reads LDS it has not written gives results the tests can tell from correct ones.  One
// workgroup fits a compute unit at a time (the whole 160 KiB); each stays a few tens of microseconds, so a launch of four
// per unit reaches them all.
__global__ __launch_bounds__(1024) void lds_fill_kernel(int spins)
{
    extern __shared__ uint32_t lds_all[];
    volatile uint32_t* v = lds_all;
    for (int i = threadIdx.x; i < 163840 / 4; i += 1024) v[i] = 0xffffffffu;
    for (int i = 0; i < spins; i++) __builtin_amdgcn_s_sleep(16);
}
extern "C" int opsnnDebugFillLds(void* stream)
{
    static std::atomic<uint64_t> attr_set{0};
    if (!opsnn::device_flag_test(attr_set)) {
        hipError_t e = hipFuncSetAttribute((const void*)lds_fill_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 163840);
        if (e != hipSuccess) return (int)e;
        opsnn::device_flag_set(attr_set);
    }
    hipLaunchKernelGGL(lds_fill_kernel, dim3(1024), dim3(1024), 163840, (hipStream_t)stream, 64);
    return (int)hipGetLastError();
}

// fp8 x fp8 arithmetic of the block-scale and row/column-scale modes: 0 (default) exact products and sums on the fp16
// matrix instruction, 1 the 8-bit matrix instruction (about 1.5x faster, sums aligned in a narrower window).  The
// initial value comes from OPSNN_FP8_FAST, read once.
static int g_fp8_fast = [] { const char* e = getenv("OPSNN_FP8_FAST"); return (e && *e && *e != '0') ? 1 : 0; }();
extern "C" void opsnnSetFp8Fast(int fast) { __atomic_store_n(&g_fp8_fast, fast ? 1 : 0, __ATOMIC_RELAXED); }
extern "C" int opsnnGetFp8Fast(void) { return __atomic_load_n(&g_fp8_fast, __ATOMIC_RELAXED); }

// OPSNN_LOG=1 (read once, like the switches above): one line on stderr whenever a call of more than 10^7 multiply-adds
// lands on a plain one-thread-per-output kernel without having been sent there -- those kernels are the parity
// reference and the route of last resort, three to four orders of magnitude slower than the matrix-core kernels.
static const bool g_log = [] { const char* e = getenv("OPSNN_LOG"); return e && *e && *e != '0'; }();
extern "C" __attribute__((visibility("hidden"))) void opsnn_note_plain(const char* mode, int forced, int64_t batch, int64_t M, int64_t N, int64_t K)
{
    if (!g_log || forced || opsnn_force_plain()) return;
    const double macs = (double)batch * (double)M * (double)N * (double)K;
    if (macs <= 1e7) return;
    fprintf(stderr, "[opsnn] %s: batch %lld, %lld x %lld x %lld (%.3g multiply-adds) runs on the plain kernel: no matrix-core route takes "
                    "this combination of layout, strides, dtypes and shape\n", mode, (long long)batch, (long long)M, (long long)K, (long long)N, macs);
}
#define NOTE_PLAIN(mode, a) opsnn_note_plain(mode, (a)->force_variant == OPSNN_VARIANT_PLAIN, (a)->batch, (a)->M, (a)->N, (a)->K)

static bool qmm_args_ok(const OpsnnQmmArgs* a)
{
    return a && a->x1.ptr && a->x2.ptr && a->out && a->M > 0 && a->N > 0 && a->K > 0 && a->batch > 0 && a->batch <= 65535;
}

// ---- K tail ----
// The matrix-core kernels walk K in tiles of 128 bytes fetched by 16-byte copies: they take K % 128 == 0 (int8: K % 16 == 0)
// and 16-byte aligned rows.  Any other K of an 8-bit operand pair is first copied, both operands, into K-contiguous rows
// padded with zeros to the next multiple of 128 (zero products change no sum, integer or floating point; the scale
// tables of the block-scale modes already have ceil(K / 128) entries).  The copies live in the workspace: two passes
// over the operands instead of the one-thread-per-output kernel.
namespace {
__global__ __launch_bounds__(256) void pad_k8_kernel(const uint8_t* __restrict__ src, int64_t o_stride, int64_t k_stride, int64_t b_stride,
                                                     uint8_t* __restrict__ dst, int64_t rows, int64_t K, int64_t Kp, int k_fast)
{
    // one thread per 16-byte piece of the output; threadIdx.x runs along the dimension that is contiguous in the source
    const int64_t chunks = Kp / 16;
    const int64_t ix = (int64_t)blockIdx.x * 64 + (threadIdx.x & 63), iy = (int64_t)blockIdx.y * 4 + (threadIdx.x >> 6);
    const int64_t c = k_fast ? ix : iy, o = k_fast ? iy : ix;
    if (c >= chunks || o >= rows) return;
    const uint8_t* s = src + (int64_t)blockIdx.z * b_stride + o * o_stride;
    uint32_t v[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const int64_t k = c * 16 + j;
        const uint32_t b = k < K ? s[k * k_stride] : 0u;
        v[j >> 2] |= b << (8 * (j & 3));
    }
    *(uint4*)(dst + ((int64_t)blockIdx.z * rows + o) * Kp + c * 16) = make_uint4(v[0], v[1], v[2], v[3]);
}

int launch_pad_k8(const OpsnnMat& m, bool k_is_col, int64_t rows, int64_t K, int64_t Kp, int64_t nb, void* dst, hipStream_t st)
{
    const int64_t o_stride = k_is_col ? m.row_stride : m.col_stride, k_stride = k_is_col ? m.col_stride : m.row_stride;
    const int k_fast = k_stride == 1 || o_stride != 1;
    const int64_t chunks = Kp / 16;
    const int64_t nx = k_fast ? chunks : rows, ny = k_fast ? rows : chunks;
    if ((ny + 3) / 4 > 65535 || nb > 65535) return OPSNN_NOT_TAKEN;
    const dim3 grid((unsigned)((nx + 63) / 64), (unsigned)((ny + 3) / 4), (unsigned)nb);
    hipLaunchKernelGGL(pad_k8_kernel, grid, dim3(256), 0, st, (const uint8_t*)m.ptr, o_stride, k_stride, m.batch_stride, (uint8_t*)dst, rows, K, Kp, k_fast);
    return (int)hipGetLastError();
}

inline int64_t round_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

// Padded K (a multiple of 128) if the call is one that the padding pre-step serves, else 0.
// mode as in opsnnQmmWorkspace.
int64_t k_pad_for(const OpsnnQmmArgs& a, int mode)
{
    if (a.force_variant == OPSNN_VARIANT_PLAIN || opsnn_force_plain()) return 0;
    if (a.M * a.N < 64 * 64) return 0;   // below the matrix-core kernels' own minimum
    const bool i8 = a.x1_dtype == DT_I8 && a.x2_dtype == DT_I8, f8 = a.x1_dtype == DT_E4M3 && a.x2_dtype == DT_E4M3;
    const bool f8any = (a.x1_dtype == DT_E4M3 || a.x1_dtype == DT_E5M2) && (a.x2_dtype == DT_E4M3 || a.x2_dtype == DT_E5M2);
    // an operand the matrix-core kernels cannot fetch as it lies (not K-contiguous, or rows not 16-byte aligned) is gathered
    // by the same copy; a dense N-contiguous x2 is not: the int8 and block-scale launchers transpose it themselves, faster
    const bool x1_ok = a.x1.col_stride == 1 && (((uint64_t)a.x1.row_stride | (uint64_t)a.x1.batch_stride | (uintptr_t)a.x1.ptr) % 16) == 0;
    const bool x2_k = a.x2.row_stride == 1 && (((uint64_t)a.x2.col_stride | (uint64_t)a.x2.batch_stride | (uintptr_t)a.x2.ptr) % 16) == 0;
    const bool x2_n = a.x2.col_stride == 1 && a.x2.row_stride == a.N && (a.x2.batch_stride == 0 || a.x2.batch_stride == a.K * a.N);
    bool tail = false;
    if (mode == 0) tail = i8 && (a.K % 16 != 0 || !x1_ok || !(x2_k || x2_n));
    else if (mode == 1) tail = (f8 || i8) && a.gsK == 128 && (a.K % 128 != 0 || !x1_ok || !(x2_k || x2_n));
    else if (mode == 3) {
        // (the fp8 members of this family have no transposition step of their own)
        const bool f8_16 = f8any && (a.out_dtype == DT_BF16 || a.out_dtype == DT_F16 || a.out_dtype == DT_F32) && (!a.bias || a.bias_dtype == DT_F32);
        tail = (i8 && !a.x1_scale && (a.K % 16 != 0 || !x1_ok || !(x2_k || x2_n))) || (f8_16 && (a.K % 128 != 0 || !x1_ok || !x2_k));
    }
    if (!tail || a.K < 16) return 0;
    if (a.x1.batch_stride < 0 || a.x2.batch_stride < 0) return 0;
    return round_up(a.K, 128);
}
uint64_t k_pad_bytes(const OpsnnQmmArgs& a, int64_t Kp)
{
    const uint64_t nb2 = a.x2.batch_stride == 0 ? 1 : (uint64_t)a.batch, nb1 = a.x1.batch_stride == 0 && a.batch > 1 ? 1 : (uint64_t)a.batch;
    return round_up((int64_t)(nb1 * (uint64_t)a.M * (uint64_t)Kp), 256) + nb2 * (uint64_t)a.N * (uint64_t)Kp;
}
// Launches the two copies and returns, in b, the same call on the padded operands (K = Kp, no workspace needed any more).
int k_pad_prestep(const OpsnnQmmArgs& a, int64_t Kp, hipStream_t st, OpsnnQmmArgs& b)
{
    if (!a.workspace) return OPSNN_NOT_TAKEN;
    const int64_t nb2 = a.x2.batch_stride == 0 ? 1 : a.batch, nb1 = a.x1.batch_stride == 0 && a.batch > 1 ? 1 : a.batch;
    uint8_t* w1 = (uint8_t*)a.workspace;
    uint8_t* w2 = w1 + round_up(nb1 * a.M * Kp, 256);
    int rc = launch_pad_k8(a.x1, true, a.M, a.K, Kp, nb1, w1, st);
    if (rc != 0) return rc;
    rc = launch_pad_k8(a.x2, false, a.N, a.K, Kp, nb2, w2, st);
    if (rc != 0) return rc;
    b = a;
    b.K = Kp;
    b.x1 = OpsnnMat{w1, Kp, 1, nb1 == 1 && a.batch > 1 ? 0 : a.M * Kp};
    b.x2 = OpsnnMat{w2, 1, Kp, nb2 == 1 && a.batch > 1 ? 0 : a.N * Kp};
    b.workspace = nullptr;
    return 0;
}
}  // namespace

// OPSNN_NOT_TAKEN if the call needs no padding (or has no workspace); 0 with *b filled after launching the copies
extern "C" __attribute__((visibility("hidden"))) int opsnn_qmm_k_pad(const OpsnnQmmArgs* a, int mode, void* stream, OpsnnQmmArgs* b)
{
    const int64_t Kp = k_pad_for(*a, mode);
    if (!Kp) return OPSNN_NOT_TAKEN;
    return k_pad_prestep(*a, Kp, (hipStream_t)stream, *b);
}

// The K split of a call that will run with few tiles on the tile kernel of qmm_fp8_block.hip (fp8 x fp4 MX and int8
// per-tile from 33 rows) or on the exact fp8 kernel of qmm_fp8_exact.hip (fp8 block scales from 129 rows, MXFP8 from 33):
// 1 = none.  Looks only at what the caller passed (shapes, types), so that the workspace query and the launch agree; a
// route that ends on another kernel leaves the partial sums' share of the workspace unused.
static int splitk_for(const OpsnnQmmArgs& a, int mode)
{
    if (a.force_variant != 0 || opsnn_force_plain()) return 1;   // (a pinned kernel variant runs as it is)
    const bool out16 = a.out_dtype == DT_BF16 || a.out_dtype == DT_F16;
    const bool f8 = a.x1_dtype == DT_E4M3 && a.x2_dtype == DT_E4M3;
    // up to 32 rows of fp8 with block scales or row / column scales, or of int8 per-tile: the decode kernel's K segments
    const bool a8w4 = mode == 2 && a.x1_dtype == DT_E4M3 && a.x2_dtype == DT_E2M1;
    const bool i8pt = mode == 1 && a.x1_dtype == DT_I8 && a.x2_dtype == DT_I8;
    if (a.M <= ((i8pt || a8w4) ? 16 : 32) && a.batch == 1 && a.N >= 256 &&
        ((mode == 1 && (f8 || i8pt) && a.gsK == 128 && a.gsN == 128) ||
         (mode == 3 && f8 && a.x1_scale && a.x2_scale) || (a8w4 && out16) || (mode == 2 && f8))) {
        QmmDecodePlan pl;
        const int sd = qmm_decode_plan(a.K, true, pl, a8w4) ? pl.splits : 1;
        // (17 .. 32 rows of fp8 with block scales may also run on the many-rows kernel, with its own segments: room for either)
        const int sr = mode == 1 && f8 ? blockscale_rows_ksplit(a) : mode == 3 && f8 ? rowcol_rows_ksplit(a) : mode == 2 && f8 ? mxfp8_rows_ksplit(a) : 1;
        return sd > sr ? sd : sr;
    }
    // 33 .. 128 rows of fp8 with block scales or row / column scales on the many-rows kernel
    if ((mode == 1 || mode == 3) && f8 && a.M <= 128) {
        if (const int sr = mode == 1 ? blockscale_rows_ksplit(a) : rowcol_rows_ksplit(a); sr > 1) return sr;
    }
    // 33 .. 256 rows of MXFP8 on the many-rows kernel
    if (mode == 2 && f8 && a.M <= 256) {
        if (const int sr = mxfp8_rows_ksplit(a); sr > 1) return sr;
    }
    // (fewer than 64 x 64 outputs are the plain kernels' -- except int8 with few outputs against a long K, qmm_int8.hip)
    const bool tiny = a.M * a.N < 64 * 64;
    if ((tiny && !(a.N >= 256 && a.M * a.N * a.K >= (1ll << 22))) || a.K < 1024) return 1;
    int64_t bm, bn = 256, kunit = 128;
    double tile_us;   // one K tile (kunit elements) of the kernel in question, measured on calls with few tiles
    double bytes_per_us = 5.0e6;   // what its partial sums' traffic was measured to cost (splitk_factor)
    // int8 with per-token / per-channel scales on 128 x 128 tiles (the selector's choice up to 256 x 256 x 64 outputs; whole K
    // tiles): integer partial sums, so the result stays bit-identical
    if ((mode == 0 || (mode == 3 && !a.x1_scale)) && a.x1_dtype == DT_I8 && a.x2_dtype == DT_I8 && out16 && a.K % 128 == 0 &&
        (a.M <= 128 || a.N <= 128 || a.M * a.N <= 256 * 256 * 64)) {
        // (a 128 x 128 int8 tile is quick, and the partial sums cost their own traffic: measured at 4096 x 4096 in eight
        // splits, 64 rows 20 -> 15 us, 128 rows 19.5 -> 22, 256 rows in four 21 -> 24)
        bm = 128; bn = 128; tile_us = 0.55; bytes_per_us = 2.4e6;
    }
    else if (tiny) return 1;
    // MXFP4: 128 x 128 tiles when 256 x 256 ones would be few (the launcher's rule), K tiles counted in 256 elements
    else if (mode == 2 && a.x1_dtype == DT_E2M1 && a.x2_dtype == DT_E2M1 && (out16 || a.out_dtype == DT_F32)) {
        const int64_t t256 = ((a.M + 255) / 256) * ((a.N + 255) / 256) * a.batch;
        bm = bn = (a.M <= 128 || a.N <= 128 || t256 <= 64) ? 128 : 256;
        kunit = 256;
        tile_us = bm == 128 ? 0.6 : 1.3; bytes_per_us = 2.4e6;
    }
    else if (a.M <= 16) return 1;   // (up to 16 rows the streaming kernels take the modes below)
    else if (mode == 2 && a.x1_dtype == DT_E4M3 && a.x2_dtype == DT_E2M1 && out16) { bm = 256; tile_us = 1.8; }
    else if (mode == 1 && a.x1_dtype == DT_I8 && a.x2_dtype == DT_I8 && a.gsK == 128 && a.gsN == 128 && out16) { bm = a.M >= 512 ? 256 : 128; tile_us = 1.8; }
    else if (mode == 1 && f8 && a.gsK == 128 && a.gsN == 128 && !a.bias && a.M > 128 && (out16 || a.out_dtype == DT_F32)) { bm = 256; bn = 128; tile_us = 1.4; }
    else if (mode == 2 && f8 && (out16 || a.out_dtype == DT_F32)) { bm = 256; bn = 128; tile_us = 1.4; }
    else if (mode == 3 && (a.x1_dtype == DT_E4M3 || a.x1_dtype == DT_E5M2) && (a.x2_dtype == DT_E4M3 || a.x2_dtype == DT_E5M2) && a.M > 128 &&
             (out16 || a.out_dtype == DT_F32)) { bm = 256; bn = 128; tile_us = 1.4; }
    else return 1;
    const int64_t tiles = ((a.M + bm - 1) / bm) * ((a.N + bn - 1) / bn) * a.batch;
    return splitk_factor(tiles, (a.K + kunit - 1) / kunit, tile_us, a.M * a.N * a.batch, bytes_per_us);
}
static uint64_t splitk_bytes(const OpsnnQmmArgs& a, int splits)
{
    return splits > 1 ? (uint64_t)round_up((int64_t)splits * a.batch * a.M * a.N * 4, 256) : 0;
}
static uint64_t qmm_workspace_base(const OpsnnQmmArgs* a, int mode);
// Takes the partial sums' share off the front of the workspace: `c` is the call as the launchers below see it.
static SplitK splitk_carve(const OpsnnQmmArgs& a, int mode, OpsnnQmmArgs& c)
{
    SplitK sk;
    c = a;
    const int s = splitk_for(a, mode);
    if (s > 1 && a.workspace) {
        sk.splits = s;
        sk.part = (float*)a.workspace;
        c.workspace = qmm_workspace_base(&a, mode) ? (char*)a.workspace + splitk_bytes(a, s) : nullptr;
    }
    return sk;
}

// For the launchers of other files: the call with the partial sums' share taken off the front of its workspace.
extern "C" __attribute__((visibility("hidden"))) void opsnn_qmm_splitk_carve(const OpsnnQmmArgs* a, int mode, OpsnnQmmArgs* c, SplitK* sk)
{
    *sk = splitk_carve(*a, mode, *c);
}

extern "C" int opsnnQmmBlockScale(const OpsnnQmmArgs* a0, void* stream)
{
    WeightCacheScope cache_scope;
    if (!qmm_args_ok(a0) || !a0->x1_scale_mat.ptr || !a0->x2_scale_mat.ptr) return -1;
    const OpsnnQmmArgs* a = a0;
    if (a->force_variant != OPSNN_VARIANT_PLAIN && !opsnn_force_plain()) {
        OpsnnQmmArgs b, c;
        const SplitK sk = splitk_carve(*a0, 1, c);
        a = &c;
        const int64_t Kp = k_pad_for(*a, 1);
        if (Kp) {
            int rc = k_pad_prestep(*a, Kp, (hipStream_t)stream, b);
            if (rc == 0) rc = launch_blockscale_mfma(b, (hipStream_t)stream, sk);
            if (rc != OPSNN_NOT_TAKEN) return rc;
        }
        int rc = launch_blockscale_mfma(*a, (hipStream_t)stream, sk);
        if (rc != OPSNN_NOT_TAKEN) return rc;
        if (a->force_variant != 0) return -4;
    }
    NOTE_PLAIN("block-scale quant matmul", a0);
    return launch_blockscale_plain(*a0, (hipStream_t)stream);
}

extern "C" int opsnnQmmMx(const OpsnnQmmArgs* a, void* stream)
{
    WeightCacheScope cache_scope;
    if (!qmm_args_ok(a) || !a->x1_scale_mat.ptr || !a->x2_scale_mat.ptr) return -1;
    if (a->force_variant != OPSNN_VARIANT_PLAIN && !opsnn_force_plain()) {
        OpsnnQmmArgs c;
        const SplitK sk = splitk_carve(*a, 2, c);
        int rc = launch_mx_mfma(c, (hipStream_t)stream, sk);
        if (rc != OPSNN_NOT_TAKEN) return rc;
        if (a->force_variant != 0) return -4;
    }
    NOTE_PLAIN("MX quant matmul", a);
    return launch_mx_plain(*a, (hipStream_t)stream);
}

// Per-tensor / per-channel family.  The int8 MFMA kernels cover int8 operands with a 16-bit, INT32 or INT8 output (the
// latter two through their integer epilogue), the fp8 row/column-scale kernel covers e4m3 operands with separately
// multiplied scales; the rest (e5m2 operands, merged and truncated double scales, fp32 output, odd layouts) runs on the
// plain kernel.
extern "C" __attribute__((visibility("hidden"))) int opsnn_qmm_int8_impl(const OpsnnQmmArgs* a, void* stream);   // qmm_int8.hip
extern "C" int opsnnQmmTc(const OpsnnQmmArgs* a, void* stream)
{
    WeightCacheScope cache_scope;
    if (!qmm_args_ok(a) || !a->x2_scale) return -1;
    const bool i8 = a->x1_dtype == DT_I8 && a->x2_dtype == DT_I8;
    const bool f8 = (a->x1_dtype == DT_E4M3 || a->x1_dtype == DT_E5M2) && (a->x2_dtype == DT_E4M3 || a->x2_dtype == DT_E5M2);
    if (!i8 && !f8) return -2;
    if (a->x2_scale_len != 1 && a->x2_scale_len != a->N) return -2;
    if (a->x1_scale && ((a->x1_scale_len != 1 && a->x1_scale_len != a->M) || !f8)) return -2;
    if (a->out_dtype == DT_I8 || a->out_dtype == DT_I32) { if (!i8) return -2; }
    // fp8 with few output tiles against a long K: the partial sums of a K split sit at the front of the workspace
    OpsnnQmmArgs carved;
    SplitK sk;
    if (f8 && a->force_variant != OPSNN_VARIANT_PLAIN && !opsnn_force_plain()) {
        sk = splitk_carve(*a, 3, carved);
        a = &carved;
    }
    OpsnnQmmArgs padded;
    if (const int64_t Kp = k_pad_for(*a, 3)) {   // K tail: continue on zero-padded K-contiguous copies
        const int rc = k_pad_prestep(*a, Kp, (hipStream_t)stream, padded);
        if (rc == 0) a = &padded;
        else if (rc != OPSNN_NOT_TAKEN) return rc;
    }
    // int8 operands, 16-bit output, no per-token scale: out = fp32(acc + int32 bias) * scale' + float bias, where scale'
    // is the scale with only its upper 19 bits kept for 64-bit words and for a one-element scale without a bf16 / fp32
    // bias (qbmmv3_kernel_golden.py:403-475).  That is the per-token x per-channel formula with x1_scale = 1: the MFMA
    // kernel computes it bit-identically.
    if (i8 && !a->x1_scale && (a->out_dtype == DT_BF16 || a->out_dtype == DT_F16) && a->force_variant != OPSNN_VARIANT_PLAIN &&
        !opsnn_force_plain()) {
        OpsnnQmmArgs b = *a;
        b.x2_scale_trunc = a->x2_scale_dtype == DT_U64 ||
                           (a->x2_scale_len == 1 && !(a->bias && (a->bias_dtype == DT_BF16 || a->bias_dtype == DT_F32)));
        return opsnnQmmInt8(&b, stream);
    }
    // int8 operands with an INT32 output (sums + int32 bias) or an INT8 output (requantised): integer epilogue of the MFMA
    // kernel, bit-identical; a float bias with INT32 output stays on the plain kernel
    if (i8 && !a->x1_scale && (a->out_dtype == DT_I32 || a->out_dtype == DT_I8) && (!a->bias || a->bias_dtype == DT_I32) &&
        a->force_variant != OPSNN_VARIANT_PLAIN && !opsnn_force_plain()) {
        OpsnnQmmArgs b = *a;
        b.x2_scale_trunc = 0;   // UINT64 words are always truncated; a float scale is used as it is
        const int rc = opsnn_qmm_int8_impl(&b, stream);
        if (rc != OPSNN_NOT_TAKEN) return rc;
    }
    // fp8 operands, 16-bit output: the forms of compute_tc (qbmmv3_kernel_golden.py:390-475) on the exact matrix-core kernel --
    // no per-token scale: (sum + float bias) * scale; both scales one element and no bias: sum * trunc19(scale * pertoken);
    // otherwise (sum * scale) * pertoken + bias.  The last form with e4m3 operands and an fp32 scale goes on to the
    // launcher below, which also knows the 8-bit-instruction variant; e5m2 operands, bf16 and 64-bit scale words, and
    // the other two forms run here.
    if (f8 && a->force_variant != OPSNN_VARIANT_PLAIN && !opsnn_force_plain()) {
        const int ep = !a->x1_scale ? 1 : (a->x1_scale_len == 1 && a->x2_scale_len == 1 && !a->bias) ? 2 : 0;
        if (ep == 0) {   // 17 .. 128 rows: the many-rows streaming kernel; up to 16 (32 in two passes where that does not apply): x1 in registers
            int rc = launch_rowcol_rows(*a, (hipStream_t)stream, sk);
            if (rc != OPSNN_NOT_TAKEN) return rc;
            rc = launch_rowcol_decode(*a, (hipStream_t)stream, sk);
            if (rc != OPSNN_NOT_TAKEN) return rc;
        }
        // (up to 32 rows the partial sums were laid out for the kernel above; the tile kernels run unsplit)
        const SplitK sk_tiles = a->M <= 32 ? SplitK{} : sk;
        const bool e4 = a->x1_dtype == DT_E4M3 && a->x2_dtype == DT_E4M3;
        if (ep != 0 || !e4 || a->x2_scale_dtype != DT_F32 || a->out_dtype == DT_F32) {
            const int rc = launch_rowcol_exact(*a, (hipStream_t)stream, ep, sk_tiles);
            if (rc != OPSNN_NOT_TAKEN) return rc;
        }
    }
    // fp8 e4m3 operands with a row scale and a column scale that are multiplied in separately (K-C, K-T, T-C with the
    // one-element x1Scale): matrix-core kernel when the layout allows, else the plain kernel
    if (f8 && a->x1_scale && a->force_variant != OPSNN_VARIANT_PLAIN && !opsnn_force_plain()) {
        const int rc = launch_fp8_rowcol_mfma(*a, (hipStream_t)stream, false, a->M <= 32 ? SplitK{} : sk);
        if (rc != OPSNN_NOT_TAKEN) return rc;
    }
    NOTE_PLAIN("per-tensor / per-channel quant matmul", a);
    return launch_tc_plain(*a, (hipStream_t)stream);
}

extern "C" int opsnnQmmGroup(const OpsnnQmmArgs* a, void* stream)
{
    WeightCacheScope cache_scope;
    if (!qmm_args_ok(a) || a->batch != 1 || a->gsK <= 0 || !a->x2_scale_mat.ptr) return -1;
    const bool tcg = a->x1_dtype == DT_E4M3 && a->x2_dtype == DT_E2M1;
    const bool i4 = a->x1_dtype == DT_I4 && a->x2_dtype == DT_I4;
    if (tcg) {
        if (a->x2_scale_dtype != DT_BF16 && a->x2_scale_dtype != DT_F16) return -2;
        if (a->y_scale && a->y_scale_len != 1 && a->y_scale_len != a->N) return -2;
        if (a->bias && a->bias_dtype != DT_F32) return -2;
    } else if (i4) {
        if (!a->x1_scale || !a->x2_offset_mat.ptr || a->bias) return -2;
    } else {
        return -2;
    }
    if (a->out_dtype != DT_BF16 && a->out_dtype != DT_F16 && a->out_dtype != DT_F32) return -2;
    if (tcg && a->force_variant != OPSNN_VARIANT_PLAIN && !opsnn_force_plain()) {
        const int rc = launch_tcg_mfma(*a, (hipStream_t)stream);
        if (rc != OPSNN_NOT_TAKEN) return rc;
    }
    if (i4 && a->force_variant != OPSNN_VARIANT_PLAIN && !opsnn_force_plain()) {
        const int rc = launch_kg_mfma(*a, (hipStream_t)stream);
        if (rc != OPSNN_NOT_TAKEN) return rc;
    }
    NOTE_PLAIN(tcg ? "fp8 x fp4 group quant matmul" : "int4 K-G quant matmul", a);
    return launch_group_plain(*a, tcg, (hipStream_t)stream);
}

extern "C" int opsnnWqmm(const OpsnnWqmmArgs* a, void* stream)
{
    WeightCacheScope cache_scope;
    if (!a || !a->x || !a->w.ptr || !a->scale.ptr || !a->y || a->M <= 0 || a->N <= 0 || a->K <= 0) return -1;
    if (a->force_variant != OPSNN_VARIANT_PLAIN && !opsnn_force_plain()) {
        int rc = launch_wqmm_mfma(*a, (hipStream_t)stream);
        if (rc != OPSNN_NOT_TAKEN) return rc;
        if (a->force_variant != 0) return -4;
    }
    opsnn_note_plain("weight-only matmul", a->force_variant == OPSNN_VARIANT_PLAIN, 1, a->M, a->N, a->K);
    return launch_wqmm_plain(*a, (hipStream_t)stream);
}

// mode: 0 = int8 per-token/per-channel, 1 = block scale, 2 = MX, 3 = per-tensor / per-channel family, 4 = K-group modes.
// The MFMA kernels stream a K-contiguous right operand ("x2 stored [N, K]").  An N-contiguous x2 is
// first re-laid out into the workspace; callers who keep x2 in [N, K] form (transposeX2 = true or a
// transposed view) need no workspace and skip that pass.
extern "C" uint64_t opsnnQmmWorkspace(const OpsnnQmmArgs* a, int mode)
{
    if (!a) return 0;
    return splitk_bytes(*a, splitk_for(*a, mode)) + qmm_workspace_base(a, mode);   // partial sums of a K split in front
}

extern "C" __attribute__((visibility("hidden"))) uint64_t opsnn_qmm_workspace_base(const OpsnnQmmArgs* a, int mode)
{
    return a ? qmm_workspace_base(a, mode) : 0;
}

static uint64_t qmm_workspace_base(const OpsnnQmmArgs* a, int mode)
{
    if (const int64_t Kp = k_pad_for(*a, mode)) return k_pad_bytes(*a, Kp);
    if (mode == 2) return mx_workspace_bytes(*a);
    if (mode == 1 && a->x2.row_stride == 1 && a->force_variant != OPSNN_VARIANT_PLAIN && !opsnn_force_plain()) {
        if (const uint64_t b = blockscale_rows_workspace(*a)) return b;   // fp8 block scales with 17 .. 128 rows: x1 widened to fp16
    }
    // per-tensor / per-channel family: int8 operands share the int8 kernels and their re-layout; fp8 needs none
    if (mode == 3 && a->x2.row_stride == 1 && a->force_variant != OPSNN_VARIANT_PLAIN && !opsnn_force_plain()) {
        if (const uint64_t b = rowcol_rows_workspace(*a)) return b;   // fp8 row / column scales with 17 .. 128 rows: x1 widened to fp16
    }
    if (mode == 3 && !(a->x1_dtype == DT_I8 && a->x2_dtype == DT_I8 && !a->x1_scale)) return 0;
    // K-group modes: the re-quantised weight of the fp8 x fp4 group-scale mode; the widened operands, row sums and fp32
    // scale / offset copies of the int4 mode with offsets
    if (mode == 4) return a->x1_dtype == DT_I4 ? kg_workspace_bytes(*a) : tcg_workspace_bytes(*a);
    if (a->x2.row_stride == 1 || a->K == 1) return 0;           // already K-contiguous
    if (a->x2.col_stride != 1 || a->x2.row_stride != a->N) return 0;  // not a dense [K, N]: plain kernel
    uint64_t bits = (a->x2_dtype == DT_I4 || a->x2_dtype == DT_E2M1) ? 4 : 8;
    uint64_t nb = a->x2.batch_stride == 0 ? 1 : (uint64_t)a->batch;
    return ((uint64_t)a->N * (uint64_t)a->K * bits / 8) * nb;
}

extern "C" uint64_t opsnnWqmmWorkspace(const OpsnnWqmmArgs* a)
{
    if (!a || a->M <= 0 || a->N <= 0 || a->K <= 0) return 0;
    const uint64_t bits = (a->w_dtype == DT_I4 || a->w_dtype == DT_E2M1) ? 4 : 8;
    // up to 16 rows against a long K: fp32 partial sums of the x-in-registers kernel's K split, in front of everything else
    // (from 17 rows against a narrow N and a long K: those of the many-rows kernel's K split)
    uint64_t part = 0;
    if (const int xs = wq_part_slices((int)bits, a->M, a->N, a->K, a->group > 0 ? a->group : a->K, opsnn_wq_narrow_slabs() != 0); xs > 1 && a->force_variant != OPSNN_VARIANT_PLAIN && !opsnn_force_plain())
        part = ((uint64_t)xs * (uint64_t)a->M * (uint64_t)a->N * 4 + 255) / 256 * 256;
    if (a->w.row_stride == 1 || a->K == 1) return part;
    if (a->w.col_stride != 1 || a->w.row_stride != a->N) return part;
    return part + (uint64_t)a->N * (uint64_t)a->K * bits / 8;
}
