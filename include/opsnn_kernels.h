/*
 * Thin C ABI over the gfx950 HIP kernels of the quantized-matmul path: plain
 * pointers, sizes and type codes, no tensor objects.  The aclnn entry points
 * (include/aclnnop/*.h) are built on exactly these calls; a host that already
 * owns device buffers and a HIP stream can call them directly.
 *
 * These launchers have no single counterpart in the reference: together they
 * stand where the reference has host tiling plus device kernels --
 *   opsnnQmmInt8        <- quant_batch_matmul_v3 K-C/K-T/T-C kernel
 *                          (matmul/quant_batch_matmul_v3/op_kernel/arch35/qbmm_mix_online_dynamic.h:387-388, 648-736)
 *   opsnnQmmTc          <- the same kernel family's per-tensor / per-channel epilogues (fixpipe dequant and requant,
 *                          matmul/quant_batch_matmul_v3/op_kernel/arch35/qbmm_cube_on_the_fly.h:159-162)
 *   opsnnQmmBlockScale  <- per-tile kernel (matmul/common/cmct/epilogue/block_epilogue_pertile.h:502-642)
 *   opsnnQmmMx          <- MX kernel (matmul/common/cmct/block/block_mmad_mx.h)
 *   opsnnWqmm           <- weight_quant_batch_matmul_v2 arch35 kernels
 *                          (matmul/weight_quant_batch_matmul_v2/op_kernel/arch35/n_first/basic_block_vf_nd.h:139-148)
 *   opsnnTranspose*     <- the reference's ND->NZ weight relayout (offline weight pre-pack)
 *
 * All functions return 0 on success, a negative value for an argument the
 * kernels cannot take (nothing launched), or a positive hipError_t.
 * Type codes are the aclDataType values.  `stream` is a hipStream_t.
 * Every launcher is asynchronous on `stream`.
 */
#ifndef OPSNN_KERNELS_H_
#define OPSNN_KERNELS_H_
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define OPSNN_API __attribute__((visibility("default")))

/* A matrix operand: element (r, c) of batch b lives at element index
 * b*batch_stride + r*row_stride + c*col_stride (strides in elements, also for 4-bit types). */
typedef struct {
    const void* ptr;
    int64_t row_stride;
    int64_t col_stride;
    int64_t batch_stride;
} OpsnnMat;

typedef struct {
    int64_t M, N, K, batch;
    OpsnnMat x1;          /* logical [M, K] */
    OpsnnMat x2;          /* logical [K, N] */
    int x1_dtype, x2_dtype;
    void* out;            /* [batch, M, N] dense */
    int out_dtype;        /* BF16 / FLOAT16 / FLOAT / INT32 */
    const void* x1_scale; /* see each launcher */
    const void* x2_scale;
    int x2_scale_dtype;   /* FLOAT or BF16 (opsnnQmmInt8, opsnnQmmTc: also UINT64) */
    int64_t x2_scale_len; /* 1 or N */
    const void* bias;     /* [N] or NULL */
    int bias_dtype;       /* INT32 / BF16 / FLOAT16 / FLOAT */
    int64_t bias_batch_stride;
    /* block-scale and MX modes */
    int64_t gsM, gsN, gsK;
    /* block mode: x1_scale_mat is logical [ceil(M/gsM), ceil(K/gsK)], x2_scale_mat logical [ceil(K/gsK), ceil(N/gsN)].
     * MX mode: the e8m0 byte for row r (m or n) and 32-wide K block kb is
     *          ptr[r*row_stride + (kb/2)*col_stride + kb%2]  (the reference stores K scales in pairs). */
    OpsnnMat x1_scale_mat;
    OpsnnMat x2_scale_mat;
    void* workspace;       /* opsnnQmmWorkspace() bytes, or NULL if that is 0 */
    int force_variant;     /* 0 = selector decides; >0 pins a kernel variant (tuning and tests) */
    /* per-tensor / per-channel family (opsnnQmmTc) */
    int64_t x1_scale_len;  /* opsnnQmmTc: 1 = one fp32 scale for all of x1 ("double scale" with fp8 inputs), M = one per row (fp8 K-C / K-T); 0 if x1_scale is NULL */
    const float* x2_offset;/* fp32 [1] or [N], int8 output only; NULL = take it from the packed 64-bit scale */
    int64_t x2_offset_len;
    /* K-group family (opsnnQmmGroup) */
    const void* y_scale;   /* UINT64 [1] or [N]: fp32 scale in the low word, upper 19 bits kept */
    int64_t y_scale_len;
    OpsnnMat x2_offset_mat;/* FLOAT16, logical [ceil(K/gsK), N] */
    /* opsnnQmmInt8: keep only the upper 19 bits of x2_scale (the reference's scale truncation; always applied to
     * UINT64 scale words, whose low 32 bits are the fp32 scale) */
    int x2_scale_trunc;
} OpsnnQmmArgs;

/* int8 x int8 -> int32, then  out = fp32(acc + int32 bias) * x2_scale[n] * x1_scale[m] + float bias.
 * x1_scale: fp32 [M] or NULL. */
OPSNN_API int opsnnQmmInt8(const OpsnnQmmArgs* a, void* stream);
/* opsnnQmmInt8 for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments and results as
 * opsnnQmmInt8, except that `workspace` is ignored: when x2 is stored [K, N] with N contiguous, the K-contiguous copy
 * the matrix-core kernel reads goes into an array of OPSNN_STATIC_SCRATCH_BYTES inside the library's device image
 * instead.  The call makes no hipMalloc / hipFree.  A call whose opsnnQmmWorkspace(a, 0) exceeds that size launches nothing and
 * returns OPSNN_ERR_SCRATCH_TOO_SMALL (text in aclGetRecentErrMsg).  All calls on one device share the one array:
 * calls that overlap in time on one device (different streams, different threads) race on it; calls on one stream
 * are ordered and safe.  Each device the library is loaded on holds the array until the process ends. */
#define OPSNN_STATIC_SCRATCH_BYTES (64ll << 20)
#define OPSNN_ERR_SCRATCH_TOO_SMALL (-6)
OPSNN_API int opsnnQmmInt8Static(const OpsnnQmmArgs* a, void* stream);
/* fp8 x fp8 with fp32 block scales: out = sum_kb (x1_kb @ x2_kb) * (s1[m/gsM,kb] * s2[kb,n/gsN]). */
OPSNN_API int opsnnQmmBlockScale(const OpsnnQmmArgs* a, void* stream);
/* Arithmetic of the fp8 e4m3 x e4m3 block-scale and row/column-scale modes (opsnnQmmBlockScale, opsnnQmmTc, the fp8 x fp4
 * group-scale mode of opsnnQmmGroup), process-wide:
 *   0 (default)  the operands are widened to fp16 in registers (exact) and contracted by the fp16 matrix instruction:
 *                products exact, sums as good as an fp32 accumulation -- the results meet the reference's acceptance
 *                (max relative error 2^-7, mean 2^-10, 99.9 % within rtol 1e-3) like an fp32-accumulating device;
 *   1            the 8-bit matrix instruction, about 1.5x faster; it aligns the 128 products of one instruction in a
 *                window narrower than fp32, which leaves about 1 % of bf16 outputs one ulp off at K = 7168.
 * The initial value is taken from the environment variable OPSNN_FP8_FAST (unset or 0: exact). */
OPSNN_API void opsnnSetFp8Fast(int fast);
OPSNN_API int opsnnGetFp8Fast(void);
/* Routing switches, process-wide.  The first also starts from the environment variable OPSNN_FORCE_PLAIN, read once when
 * the library is loaded; the others are hooks of the parity tests, which compare two kernels on the same call:
 *   opsnnSetForcePlain(1)  every call runs on the plain one-thread-per-output kernels (bit-identical to the CPU oracle);
 *   opsnnSetMx8Wide(n)     MXFP8 on the four-wave kernel with 256 x 32n tiles (n = 8, 9), 0 never, -1 automatic;
 *   opsnnSetWqTileMin(m)   weight-only int4/int8 calls with m .. 256 rows of x run on the dequantise-once tile kernel
 *                          (default 129; 1 sends every eligible call there, 257 none);
 *   opsnnSetWqNarrowSlabs(0) weight-only calls against a narrow weight (N <= 16384) run one pass of up to 256 rows per
 *                          launch, as wide ones do (default 1: equal row slabs of 64 .. 256 rows, all in one launch). */
OPSNN_API void opsnnSetForcePlain(int on);
OPSNN_API void opsnnSetMx8Wide(int n);
OPSNN_API void opsnnSetWqTileMin(int m);
OPSNN_API void opsnnSetWqNarrowSlabs(int on);
/* Another hook of the parity tests: fills the LDS of every compute unit with all-ones bytes (NaN in every floating-point
 * format used here) on `stream`, so that the next kernel shows if it reads LDS that it has not written.  0 or a HIP status. */
OPSNN_API int opsnnDebugFillLds(void* stream);
/* Opt-in cache of re-laid-out right operands.  The matrix-core kernels stream a K-contiguous right operand; x2 / weight
 * stored [K, N] with N contiguous is re-laid out inside every call (into the caller's workspace) unless this cache is on:
 * then opsnnQmmInt8, opsnnQmmBlockScale, opsnnQmmMx (data and scales) and opsnnWqmm keep the K-contiguous copy in device memory of the library's own, keyed
 * by the operand's address, shape, element width and batch count, and later calls with the same operand skip the pass
 * (the workspace is then not touched).  It has no counterpart among the reference's entry points: the reference folds the
 * re-layout into its graphs offline (weight_quant_batch_matmul_v2_transpose_fusion_pass.cpp,
 * quant_batch_matmul_v4_transpose_fusion_pass.cpp).
 *   opsnnSetWeightCache(max_bytes)  0 switches the cache off and frees it (the default; OPSNN_WEIGHT_CACHE_MB sets the
 *                                   initial limit); entries are evicted least recently used first;
 *   opsnnWeightCacheClear()         frees every entry.  The cache cannot see a weight change: call this before
 *                                   overwriting, freeing or re-using the memory of an operand that may be cached;
 *   opsnnWeightCacheInvalidate(ptr, bytes)  frees the entries made from operands (data, scales or offsets) whose address
 *                                   lies in [ptr, ptr + bytes) (bytes = 0: equals ptr) and returns their number: the
 *                                   per-weight form of the call above, for a caller that updates one weight in place;
 *   opsnnWeightCacheStats(...)      entries, bytes held, hits and misses so far (any pointer may be NULL).
 * Calls made while their stream is being captured into a graph bypass the cache. */
OPSNN_API void opsnnSetWeightCache(int64_t max_bytes);
OPSNN_API void opsnnWeightCacheClear(void);
OPSNN_API int opsnnWeightCacheInvalidate(const void* ptr, uint64_t bytes);
OPSNN_API void opsnnWeightCacheStats(int64_t* entries, int64_t* bytes, int64_t* hits, int64_t* misses);
/* MX: fp4/fp8 operands, e8m0 scale per 32 K. out = (x1*s1) @ (x2*s2) + fp32 bias. */
OPSNN_API int opsnnQmmMx(const OpsnnQmmArgs* a, void* stream);
/* Per-tensor / per-channel scales (T-T, T-C): int8 or fp8 (e4m3, e5m2) operands;
 *   x2_scale FLOAT / BF16 [1] or [N], or UINT64 [1] or [N] (fp32 scale in the low word, upper 19 bits kept; signed 9-bit
 *   offset at bits 37..45); optional one-element x1_scale with fp8 inputs; out BF16 / FLOAT16 / FLOAT, INT32 (integer
 *   sums + bias) or INT8 (requantised: clip(s9(s9(acc * scale)) + s9(offset))).
 * Reference formulas: matmul/quant_batch_matmul_v3/tests/assets/qbmmv3_kernel_golden.py:390-513. */
OPSNN_API int opsnnQmmTc(const OpsnnQmmArgs* a, void* stream);
/* K-group modes of quant_batch_matmul_v4 (gsK = K elements per group):
 *   fp8 e4m3 x fp4 e2m1 ("T-CG"): x2_scale_mat BF16 / FLOAT16 logical [ceil(K/gsK), N] (dtype in x2_scale_dtype);
 *     w = e4m3(T16(T16(x2) * scale)); out = (x1 @ w) * deq(y_scale[n]) + fp32 bias;
 *   int4 x int4 with offsets (gsK = 256): x1_scale fp32 [M], x2_scale_mat fp32 and x2_offset_mat fp16 logical
 *     [ceil(K/256), N]; out = x1_scale[m] * sum_g (x1_g @ x2_g - rowsum(x1_g) * offset[g,n]) * scale[g,n].
 * Reference formulas: matmul/quant_batch_matmul_v4/tests/assets/qbmmv4_kernel_golden.py:189-255, 328-395.
 * (The MX fp8 x fp4 mode of that file runs through opsnnQmmMx and its int8 per-tile mode through opsnnQmmBlockScale.) */
OPSNN_API int opsnnQmmGroup(const OpsnnQmmArgs* a, void* stream);
/* Device workspace bytes a launcher needs for these arguments (0 if none).  mode names the entry point the arguments
 * are for: 0 opsnnQmmInt8, 1 opsnnQmmBlockScale, 2 opsnnQmmMx, 3 opsnnQmmTc, 4 opsnnQmmGroup (the fp8 x fp4 mode's
 * re-quantised weight, N * K bytes plus the decoded output scale, or the int4 mode's operands rewritten as e4m3 bytes in
 * tile blocks padded to whole tiles, each with its row sums or fp32 scales and offsets, when the mode's matrix-core path
 * applies). */
OPSNN_API uint64_t opsnnQmmWorkspace(const OpsnnQmmArgs* a, int mode);

typedef struct {
    int64_t M, N, K;
    const void* x;        /* [M, K] dense, FLOAT16 or BF16 */
    int x_dtype;
    OpsnnMat w;           /* logical [K, N]; INT8 / INT4 / FLOAT8_E4M3FN / FLOAT4_E2M1 */
    int w_dtype;
    OpsnnMat scale;       /* logical [G, N] with G = 1 or ceil(K/group); x's dtype, or FLOAT8_E8M0 */
    int scale_dtype;
    int64_t scale_n;      /* N, or 1 for per-tensor */
    const void* offset;   /* same layout as scale, or NULL */
    int64_t group;        /* 0 = per-channel / per-tensor */
    const void* bias;     /* [N] or NULL */
    int bias_dtype;
    void* y;              /* [M, N] dense, x's dtype */
    void* workspace;      /* opsnnWqmmWorkspace() bytes, or NULL if that is 0 */
    int force_variant;
} OpsnnWqmmArgs;

/* y = x @ T(T(w + offset) * scale) + bias, T = rounding through x's dtype. */
OPSNN_API int opsnnWqmm(const OpsnnWqmmArgs* a, void* stream);
OPSNN_API uint64_t opsnnWqmmWorkspace(const OpsnnWqmmArgs* a);

/* dst[c, r] = src[r, c] for a dense [rows, cols] matrix of 8-bit elements (batched). */
OPSNN_API int opsnnTranspose8(const void* src, void* dst, int64_t rows, int64_t cols, int64_t batch, void* stream);
/* Same for 4-bit elements packed two per byte along the last axis (low nibble = even index);
 * rows and cols must be even. */
OPSNN_API int opsnnTranspose4(const void* src, void* dst, int64_t rows, int64_t cols, int64_t batch, void* stream);
/* The dense copy of a strided view of packed 4-bit elements: dst[b, r, c] (two per byte, cols even) = element
 * offset + b * batch_stride + r * row_stride + c * col_stride of the storage at base (offset and strides in elements, none
 * negative).  What aclnnQuantMatmulV5 does to a non-contiguous 4-bit operand before anything else, in place of the
 * reference's l0op::Contiguous (matmul/quant_batch_matmul_v4/op_host/op_api/quant_matmul_common_check.cpp:106-123). */
OPSNN_API int opsnnGather4(const void* base, int64_t offset, int64_t batch, int64_t rows, int64_t cols, int64_t batch_stride,
                           int64_t row_stride, int64_t col_stride, void* dst, void* stream);
/* The same for 8-bit elements: the MX modes of aclnnQuantMatmulV5 gather a strided fp8 operand this way (the other 8-bit
 * modes gather inside their launchers, together with the padding of a K tail). */
OPSNN_API int opsnnGather8(const void* base, int64_t offset, int64_t batch, int64_t rows, int64_t cols, int64_t batch_stride,
                           int64_t row_stride, int64_t col_stride, void* dst, void* stream);

/* The same for 16-bit elements (pairs of e8m0 MX scales, 16-bit group scales). */
OPSNN_API int opsnnTranspose16(const void* src, void* dst, int64_t rows, int64_t cols, int64_t batch, void* stream);

/* FRACTAL_NZ <-> ND re-layout of a dense [rows, row_bytes] byte matrix (batched): nz[b / c0][r / 16][r % 16][b % c0] =
 * nd[r][b], the NZ array being [ceil(row_bytes / c0), ceil(rows / 16), 16, c0] with zero padding; c0_bytes is 32 for 8-bit
 * elements, 8 or 16 for 4-bit elements (16 or 32 elements per fractal row).  Layout definition:
 * matmul/common/tests/st/arch35/matmul_golden_util.py:76-114, 284-313. */
OPSNN_API int opsnnNzToNd(const void* nz, void* nd, int64_t rows, int64_t row_bytes, int c0_bytes, int64_t batch, void* stream);
OPSNN_API int opsnnNdToNz(const void* nd, void* nz, int64_t rows, int64_t row_bytes, int c0_bytes, int64_t batch, void* stream);

/* Weight pre-pack: `count` 4-bit values, one per 32-bit carrier element (int32: value & 0xF; fp32: the fp4 e2m1 code of
 * the value, 0 for a value that is not one of the 16), into count / 2 bytes, low nibble = even index.  count even, src
 * 16-byte and dst 8-byte aligned.  Device form of the host loop in
 * matmul/convert_weight_to_int4_pack/op_host/op_api/aclnn_convert_weight_to_int4_pack.cpp:79-126. */
OPSNN_API int opsnnPackB4(const void* src, int src_is_fp32, void* dst, int64_t count, void* stream);

/* fp32 scale (and optional fp32 offset) -> the 64-bit packed quantisation parameter of the per-tensor / per-channel
 * matmul modes: the scale cut to 19 bits in the low word (round_mode 0: truncated, 1: rounded to nearest even), the offset
 * as a signed 9-bit integer at bits 37..45, bit 46 set.  A one-element scale or offset is broadcast; out has
 * max(scale_len, offset_len) elements.  Device kernel of the reference: quant/trans_quant_param_v2/op_kernel/
 * trans_quant_param_v2.h:224-300. */
OPSNN_API int opsnnTransQuantParam(const float* scale, int64_t scale_len, const float* offset, int64_t offset_len, int round_mode,
                                   uint64_t* out, void* stream);

/* Dynamic per-token quantisation of x [rows, cols] (FLOAT16 / BF16, dense): per row a scale (and, when `offset` is not
 * NULL, an offset: the asymmetric form) and the quantised row y in INT8, INT4 (two per byte, even column in the low nibble;
 * cols even), FLOAT8_E4M3FN or FLOAT8_E5M2.  smooth: NULL or [cols] factors of x's dtype.  Formula:
 * quant/dynamic_quant/tests/assets/golden.py:17-122 (pertoken, with or without group_index).  A row without range (all zeros; asymmetric: constant)
 * gets scale 0 and zeros.  force_variant: 0 automatic, 1 the register-resident kernel, 2 the two-pass kernel. */
typedef struct {
    const void* x; int x_dtype;
    const void* smooth;
    void* y; int y_dtype;
    float* scale;
    float* offset;
    int64_t rows, cols;
    int force_variant;
    /* per-expert smooth factors: group_index[e] (INT32 or INT64, ascending) is the row where expert e's rows end, and smooth
     * is then [groups, cols]; rows from group_index[groups - 1] on are left untouched.  NULL: one smooth row for all. */
    const void* group_index; int group_index_dtype;
    int64_t groups;
    /* quant_mode 0: one scale per row (above).  1 "pertensor": one scale (and offset) for the whole tensor, scale[1].
     * 2 "perchannel": x is [rows / chan_rows, chan_rows, cols], one scale per batch and column (the reduction runs over the
     * chan_rows axis), scale [rows / chan_rows, cols], and smooth holds chan_rows factors, one per row of a batch.  In modes
     * 1 and 2 the scale / offset buffers hold intermediate values until the call's last kernel has run. */
    int quant_mode;
    int64_t chan_rows;
} OpsnnDynQuantArgs;
OPSNN_API int opsnnDynamicQuant(const OpsnnDynQuantArgs* a, void* stream);

/* Dynamic block quantisation of x [batch, rows, cols] (FLOAT16 / BF16, dense) to FLOAT8_E4M3FN / FLOAT8_E5M2 with one
 * fp32 scale per block of row_block x col_block elements, scale [batch, ceil(rows / row_block), ceil(cols / col_block)];
 * min_scale >= 0 caps the scale at 1 / min_scale (0: no cap).  Formula:
 * quant/dynamic_block_quant/tests/assets/golden.py:95-222.  force_variant: 0 automatic, 1 the lane-group kernel
 * (row_block == 1, cols % 8 == 0), 2 the workgroup-per-block kernel. */
typedef struct {
    const void* x; int x_dtype;
    void* y; int y_dtype;
    float* scale;
    int64_t batch, rows, cols;
    int64_t row_block, col_block;
    double min_scale;
    int force_variant;
} OpsnnBlockQuantArgs;
OPSNN_API int opsnnDynamicBlockQuant(const OpsnnBlockQuantArgs* a, void* stream);

/* Dynamic MX quantisation of x [rows, cols] (FLOAT16 / BF16, dense) along the columns in blocks of `block` (32 by default): y in FLOAT4_E2M1
 * (two per byte, even column in the low nibble; cols even), FLOAT8_E4M3FN or FLOAT8_E5M2, and one FLOAT8_E8M0 scale per
 * block, scale [rows, 2 * ceil(ceil(cols / 32) / 2)] (rows padded to an even number of bytes with 0).  Formula:
 * quant/dynamic_mx_quant/tests/assets/golden.py:140-153, 196-218, 263-330 (round mode "rint", scale algorithm 0).
 * force_variant: 0 automatic, 1 the lane-group kernel (block 32, cols % 8 == 0), 2 the one-thread-per-block kernel. */
typedef struct {
    const void* x; int x_dtype;
    void* y; int y_dtype;
    void* scale;
    int64_t rows, cols;
    int force_variant;
    int64_t block;    /* elements per scale block: a multiple of 32 up to 1024; 0 means 32 */
    int scale_alg;    /* 0: scale 2^(floor(log2 max) - emax); 1 (fp8 outputs only): max / typeMax rounded up to a power of two */
    /* General form, used when axis_len > 0 (rows and cols are then ignored): x is [outer, axis_len, inner] and the blocks run
     * along axis_len; x may also be FLOAT, y also FLOAT4_E1M2; round_mode 0 rint, 1 round (ties away from zero), 2 floor,
     * 3 ceil, 4 trunc.  scale is [outer, ceil(nblocks / 2), inner, 2].  4-bit outputs need an even inner (or, with
     * inner == 1, an even axis_len). */
    int64_t outer, axis_len, inner;
    int round_mode;
} OpsnnMxQuantArgs;
OPSNN_API int opsnnDynamicMxQuant(const OpsnnMxQuantArgs* a, void* stream);

/* Device properties the selector uses. */
OPSNN_API int opsnnDeviceInfo(int* cu_count, int* clock_khz, int64_t* hbm_bytes, char* arch, int arch_len);

#ifdef __cplusplus
}
#endif
#endif
