"""Per-tensor / per-channel quantized matmul (T-T, T-C): 64-bit packed scales, int8 requantisation, int32 output,
19-bit scale truncation, fp8 operands with the one-element per-token scale ("double scale") or one scale per row (K-C).

CPU part: the oracle's orc_qmm_tc is pinned by recomputing the reference formulas
(matmul/quant_batch_matmul_v3/tests/assets/qbmmv3_kernel_golden.py:390-513) independently in numpy on small
cases, by hand-computed requantisation values, and by the case that reduces to the per-token function.
GPU part: the library through the aclnn C ABI must be bit-identical to the oracle for integer operands (exact
int32 sums, the same fp32 operation order) and for fp8 operands too (the kernel sums in ascending k like the oracle).
"""
import numpy as np
import pytest

import cases
import oracle_api as orc


def trunc19(a):
    return (np.asarray(a, np.float32).view(np.uint32) & np.uint32(0xFFFFE000)).view(np.float32)


def s9(a):
    return np.clip(np.round(np.asarray(a, np.float32)), -256, 255).astype(np.float32)


def test_requant_hand_values():
    # acc = 1*3 + 2*4 = 11; 11 * 0.5 = 5.5 -> 6 (half to even); offset 2.5 -> 2; 6 + 2 = 8
    x1 = np.array([[1, 2]], np.int8); x2 = np.array([[3], [4]], np.int8)
    sc = orc.pack_u64_scale(np.array([0.5], np.float32))
    y = orc.qmm_tc(x1, x2, orc.I8, orc.I8, 1, 2, 1, False, False, sc, orc.U64, None, np.array([2.5], np.float32), None, 0, orc.I8)
    assert y[0, 0] == 8
    # 4.5 -> 4 (half to even); no offset tensor: the offset packed in the scale word is used (-3)
    sc = orc.pack_u64_scale(np.array([4.5 / 11], np.float32), np.array([-3.0], np.float32))
    y = orc.qmm_tc(x1, x2, orc.I8, orc.I8, 1, 2, 1, False, False, sc, orc.U64, None, None, None, 0, orc.I8)
    want = np.float32(11) * trunc19(np.float32(4.5 / 11))
    assert y[0, 0] == int(np.clip(s9(want) - 3, -128, 127))
    # saturation: 11 * 100 -> s9 clips to 255, + 10 -> 265 -> int8 clips to 127; negative side to -128
    sc = orc.pack_u64_scale(np.array([100.0, -100.0], np.float32))
    x2b = np.array([[3, 3], [4, 4]], np.int8)
    y = orc.qmm_tc(x1, x2b, orc.I8, orc.I8, 1, 2, 2, False, False, sc, orc.U64, None, np.array([10.0], np.float32), None, 0, orc.I8)
    assert list(y[0]) == [127, -128]


def test_packed_scale_layout():
    # bit 46 set, fp32 bits low, offset field at 37..45 (two's complement 9 bits)
    w = orc.pack_u64_scale(np.array([1.0], np.float32), np.array([-1.0], np.float32))[0]
    assert int(w) & 0xFFFFFFFF == 0x3F800000 and (int(w) >> 46) & 1 == 1 and (int(w) >> 37) & 0x1FF == 0x1FF
    assert orc.lib().orc_u64_to_deq_scale(int(w)) == 1.0
    # a scale with low mantissa bits loses them: 0.1 = 0x3DCCCCCD -> 0x3DCCC000
    w = orc.pack_u64_scale(np.array([0.1], np.float32))[0]
    assert np.float32(orc.lib().orc_u64_to_deq_scale(int(w))).view(np.uint32) == 0x3DCCC000


@pytest.mark.parametrize("scale_len,bias_dt,y_dt", [(1, "i32", "f16"), ("N", "i32", "f16"), (1, "f16", "f16"), (1, "bf16", "bf16"),
                                                    ("N", None, "bf16"), (1, None, "i32"), ("N", "i32", "i32"), ("N", "i32", "i8")])
def test_int8_formulas_against_numpy(scale_len, bias_dt, y_dt):
    M, K, N = 7, 40, 12
    rng = np.random.default_rng(5)
    x1 = rng.integers(-127, 128, (M, K), dtype=np.int8); x2 = rng.integers(-127, 128, (K, N), dtype=np.int8)
    sf = rng.uniform(1e-3, 1e-2, 1 if scale_len == 1 else N).astype(np.float32)
    codes = {"i32": orc.I32, "f16": orc.F16, "bf16": orc.BF16, "i8": orc.I8, None: 0}
    if bias_dt == "i32":
        bias = rng.integers(-500, 500, N).astype(np.int32); bias_f = None
    elif bias_dt is None:
        bias = None
    else:
        bias_f = rng.normal(0, 1, N).astype(np.float32)
        bias = orc.f32_to_b16(bias_f, codes[bias_dt]); bias_f = orc.b16_to_f32(bias, codes[bias_dt])
    u64 = y_dt == "i8"
    scale = orc.pack_u64_scale(sf) if u64 else sf
    got = orc.qmm_tc(x1, x2, orc.I8, orc.I8, M, K, N, False, False, scale, orc.U64 if u64 else orc.F32, None, None, bias,
                     codes[bias_dt], codes[y_dt])
    acc = x1.astype(np.int32) @ x2.astype(np.int32)
    if y_dt == "i32":
        want = acc + bias if bias is not None else acc
        assert np.array_equal(got, want)
        return
    if y_dt == "i8":
        o = s9((acc + bias).astype(np.float32) * trunc19(sf))
        want = np.clip(s9(o) + np.float32(0), -128, 127).astype(np.int8)   # offset field of the packed word is 0
        assert np.array_equal(got, want)
        return
    # compute_tc: int32 bias before scaling; float bias after (int operands); a one-element scale is truncated to
    # 19 bits unless the bias is bf16 / fp32
    s = sf
    if scale_len == 1 and bias_dt not in ("bf16",):
        s = trunc19(sf)
    o = (acc + bias if bias_dt == "i32" else acc).astype(np.float32) * s
    if bias_dt in ("f16", "bf16"):
        o = o + bias_f
    want = orc.f32_to_b16(o.astype(np.float32), codes[y_dt])
    assert np.array_equal(got, want)


def test_tc_without_truncation_equals_pertoken_function():
    # T-C with N scales and a float bias is the per-token formula with no row scale: the already pinned function
    M, K, N = 9, 64, 20
    rng = np.random.default_rng(6)
    x1 = rng.integers(-127, 128, (M, K), dtype=np.int8); x2 = rng.integers(-127, 128, (N, K), dtype=np.int8)
    sf = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    bias = orc.f32_to_bf16(rng.normal(0, 1, N).astype(np.float32))
    a = orc.qmm_tc(x1, x2, orc.I8, orc.I8, M, K, N, False, True, sf, orc.F32, None, None, bias, orc.BF16, orc.BF16)
    b = orc.qmm_pertoken(x1, x2, M, K, N, False, True, None, sf, bias, orc.BF16, orc.BF16)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("scale_len", [1, "N"])
def test_fp8_double_scale_against_numpy(scale_len):
    # fp8 operands, one-element per-token scale, fp32 bias (added after the scaling).  With a one-element x2 scale
    # the bias-after form still multiplies separately (the merged, truncated product is the no-bias cube path).
    M, K, N = 5, 32, 8
    rng = np.random.default_rng(7)
    x1 = orc.f32_to_e4m3(rng.normal(0, 1, (M, K)).astype(np.float32)); x2 = orc.f32_to_e4m3(rng.normal(0, 1, (K, N)).astype(np.float32))
    sf = rng.uniform(0.05, 0.5, 1 if scale_len == 1 else N).astype(np.float32)
    pt = np.array([1.37], np.float32)
    bias = rng.normal(0, 1, N).astype(np.float32)
    mm = np.zeros((M, N), np.float32)
    a, b = orc.e4m3_to_f32(x1), orc.e4m3_to_f32(x2)
    for k in range(K):   # ascending k, fp32
        mm = (mm + a[:, k:k + 1] * b[k:k + 1, :]).astype(np.float32)
    got = orc.qmm_tc(x1, x2, orc.E4M3, orc.E4M3, M, K, N, False, False, sf, orc.F32, pt, None, bias, orc.F32, orc.F16)
    want = orc.f32_to_f16(((mm * sf).astype(np.float32) * pt[0]).astype(np.float32) + bias)
    assert np.array_equal(got, want)
    # without a bias and with a one-element x2 scale the two scales are merged and truncated to 19 bits
    got = orc.qmm_tc(x1, x2, orc.E4M3, orc.E4M3, M, K, N, False, False, sf, orc.F32, pt, None, None, 0, orc.F32)
    if scale_len == 1:
        want = mm * trunc19(sf * pt[0])
    else:
        want = (mm * sf).astype(np.float32) * pt[0]
    assert np.array_equal(got, want.astype(np.float32))


def test_fp8_pertoken_against_numpy():
    """fp8 operands with one scale per row of x1 (K-C) or additionally one for all of x2 (K-T): compute_pertoken on the
    fp32 matmul, (acc * x2Scale) * x1Scale[m] + bias, nothing truncated (qbmmv3_kernel_golden.py:361-387, 612-634)."""
    M, K, N = 6, 48, 10
    rng = np.random.default_rng(11)
    # integer-valued operands: every product and partial sum is an exact fp32 integer, so the summation order cannot matter
    xi1 = rng.integers(-6, 7, (M, K)).astype(np.float32); xi2 = rng.integers(-6, 7, (K, N)).astype(np.float32)
    x1, x2 = orc.f32_to_e4m3(xi1), orc.f32_to_e4m3(xi2)
    assert np.array_equal(orc.e4m3_to_f32(x1), xi1)
    mm = (xi1.astype(np.float64) @ xi2.astype(np.float64)).astype(np.float32)
    s1 = rng.uniform(0.5, 2.0, M).astype(np.float32); bias = rng.normal(0, 1, N).astype(np.float32)
    for s2 in (rng.uniform(0.05, 0.5, N).astype(np.float32), np.array([0.1], np.float32)):   # 0.1 has low mantissa bits: no truncation
        want = ((mm * s2).astype(np.float32) * s1[:, None]).astype(np.float32)
        got = orc.qmm_pertoken_f8(x1, x2, orc.E4M3, orc.E4M3, M, K, N, False, False, s1, s2, None, orc.F32)
        assert np.array_equal(got, want)
        got = orc.qmm_pertoken_f8(x1, x2, orc.E4M3, orc.E4M3, M, K, N, False, False, s1, s2, bias, orc.BF16)
        assert np.array_equal(got, orc.f32_to_bf16((want + bias).astype(np.float32)))
    # a transposed x2 is the same matrix; the multiplication order is (acc * s2) * s1, not acc * (s2 * s1)
    s2 = rng.uniform(0.05, 0.5, N).astype(np.float32)
    a = orc.qmm_pertoken_f8(x1, x2, orc.E4M3, orc.E4M3, M, K, N, False, False, s1, s2, None, orc.F32)
    b = orc.qmm_pertoken_f8(x1, np.ascontiguousarray(x2.T), orc.E4M3, orc.E4M3, M, K, N, False, True, s1, s2, None, orc.F32)
    assert np.array_equal(a, b)
    other = mm * (s2[None, :] * s1[:, None]).astype(np.float32)
    assert not np.array_equal(a, other.astype(np.float32))
    # general fp8 values: ascending-k fp32 sums like every other float path of the oracle, and with a constant row scale
    # the function equals the double-scale branch of orc_qmm_tc that multiplies separately (per-channel x2 scale)
    y1 = orc.f32_to_e4m3(rng.normal(0, 1, (M, K)).astype(np.float32)); y2 = orc.f32_to_e4m3(rng.normal(0, 1, (K, N)).astype(np.float32))
    acc = np.zeros((M, N), np.float32)
    fa, fb = orc.e4m3_to_f32(y1), orc.e4m3_to_f32(y2)
    for k in range(K):
        acc = (acc + fa[:, k:k + 1] * fb[k:k + 1, :]).astype(np.float32)
    got = orc.qmm_pertoken_f8(y1, y2, orc.E4M3, orc.E4M3, M, K, N, False, False, s1, s2, bias, orc.F32)
    assert np.array_equal(got, (((acc * s2).astype(np.float32) * s1[:, None]).astype(np.float32) + bias).astype(np.float32))
    const = np.full(M, 1.37, np.float32)
    a = orc.qmm_pertoken_f8(y1, y2, orc.E4M3, orc.E4M3, M, K, N, False, False, const, s2, bias, orc.F16)
    b = orc.qmm_tc(y1, y2, orc.E4M3, orc.E4M3, M, K, N, False, False, s2, orc.F32, const[:1], None, bias, orc.F32, orc.F16)
    assert np.array_equal(a, b)


GPU_CASES = [
    # M, K, N, in, scale dtype, scale len, bias, out, tB, pertoken, offset len
    (16, 32, 16, "i8", "u64", 1, "i32", "f16", False, False, 0),      # the reference's A8W8FP16_pertensor row
    (16, 32, 16, "i8", "u64", "N", "i32", "f16", False, False, 0),    # A8W8FP16_perchannel
    (16, 32, 16, "i8", "u64", 1, "i32", "i8", False, False, 1),       # A8W8C8_pertensor_offset
    (16, 32, 16, "i8", "u64", "N", "i32", "i8", False, False, 1),     # A8W8C8_perchannel_offset
    (33, 200, 70, "i8", "u64", "N", "i32", "i8", True, False, "N"),
    (33, 200, 70, "i8", "u64", "N", None, "i8", False, False, 0),     # offset taken from the packed word (zero)
    (40, 96, 50, "i8", "f32", 1, "i32", "bf16", True, False, 0),      # per-tensor float scale: 19-bit truncation
    (40, 96, 50, "i8", "f32", 1, "f32", "bf16", True, False, 0),      # fp32 bias: no truncation of the scale
    (40, 96, 50, "i8", "bf16", 1, None, "bf16", False, False, 0),
    (40, 96, 50, "i8", "f32", "N", "i32", "i32", False, False, 0),
    # large enough for the MFMA tile kernel (int8 operands, 16-bit output), K-contiguous and N-contiguous x2
    (128, 256, 192, "i8", "u64", "N", "i32", "f16", True, False, 0),
    (100, 192, 136, "i8", "f32", 1, "i32", "bf16", True, False, 0),   # truncated per-tensor float scale
    (128, 256, 192, "i8", "u64", 1, "i32", "bf16", False, False, 0),
    (96, 320, 160, "i8", "f32", 1, "f32", "bf16", True, False, 0),    # fp32 bias: scale not truncated
    (96, 320, 160, "i8", "bf16", "N", "bf16", "bf16", True, False, 0),
    # few tiles against a long K: the int8 kernel's K split (integer partial sums: bit-identical), packed scale words with
    # the 19-bit truncation, K-contiguous and N-contiguous x2
    (64, 4096, 256, "i8", "u64", "N", "i32", "f16", True, False, 0),
    (200, 8192, 520, "i8", "f32", 1, "i32", "bf16", False, False, 0),
    # INT8 (requantised) and INT32 outputs on the MFMA kernel's integer epilogue: 128 x 128 and 256 x 256 tiles, K tails,
    # ragged and odd N, N-contiguous x2 (re-laid out into the workspace), offsets from the tensor and from the packed word
    (128, 256, 192, "i8", "u64", "N", "i32", "i8", True, False, "N"),
    (300, 384, 260, "i8", "u64", 1, "i32", "i8", True, False, 1),
    (300, 400, 260, "i8", "f32", "N", "i32", "i32", True, False, 0),
    (300, 400, 261, "i8", "u64", "N", None, "i8", True, False, 0),
    (640, 1024, 520, "i8", "f32", "N", None, "i32", False, False, 0),
    (2048, 512, 2304, "i8", "u64", "N", "i32", "i8", True, False, "N"),
    (2048, 528, 2301, "i8", "f32", "N", "i32", "i32", True, False, 0),
    (16, 32, 16, "e4m3", "f32", "N", "f32", "f16", False, True, 0),   # FP8E4M3..dynamic_tc_bias_float
    (16, 32, 16, "e5m2", "f32", "N", "f32", "bf16", False, True, 0),  # FP8E5M2..dynamic_tc_bias_float
    (37, 160, 48, "e4m3", "f32", 1, None, "bf16", True, True, 0),     # both scales one element: merged and truncated
    (37, 160, 48, "e4m3", "u64", "N", None, "f32", True, False, 0),   # T-C without a per-token scale: packed scale
    (37, 160, 48, "e4m3", "u64", 1, "f32", "f16", False, False, 0),   # float bias before the scaling (no per-token scale)
    # fp8 with one scale per row of x1: K-C and K-T (compute_pertoken on the fp32 matmul)
    (37, 160, 48, "e4m3", "f32", "N", "f32", "bf16", True, "M", 0),
    (37, 160, 48, "e4m3", "f32", 1, None, "f32", False, "M", 0),
    (16, 64, 24, "e5m2", "f32", "N", "f32", "f16", False, "M", 0),
]


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N,in_dt,s_dt,s_len,bias_dt,out_dt,tB,pt,off_len", GPU_CASES)
def test_gpu_matches_oracle(gpu, M, K, N, in_dt, s_dt, s_len, bias_dt, out_dt, tB, pt, off_len):
    m = gpu
    dt = {"i8": m.ACL_INT8, "e4m3": m.ACL_FLOAT8_E4M3FN, "e5m2": m.ACL_FLOAT8_E5M2, "u64": m.ACL_UINT64, "f32": m.ACL_FLOAT,
          "bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "i32": m.ACL_INT32, None: None}
    print(f"case tc {M}x{K}x{N} in={in_dt} scale={s_dt}/{s_len} bias={bias_dt} out={out_dt} tB={tB} pt={pt} off={off_len}", flush=True)
    inp = cases.make_tc_inputs(m, M, K, N, M + N, dt[in_dt], dt[s_dt], 1 if s_len == 1 else N, dt[bias_dt], tB, pertoken=pt,
                               offset_len=N if off_len == "N" else off_len, e5m2=in_dt == "e5m2")
    want = cases.oracle_tc(m, inp, M, K, N, dt[out_dt])
    got = cases.run_tc_aclnn(m, inp, M, K, N, dt[out_dt])
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ"


@pytest.mark.gpu
@pytest.mark.parametrize("fast", [False, True])
@pytest.mark.parametrize("M,K,N,s_len,bias,out_dt,pt", [
    (300, 384, 260, "N", True, "bf16", "M"),      # K-C, ragged tiles, 128-row tile instance
    (640, 1024, 520, "N", False, "f16", "M"),     # 256-row tile instance
    (128, 256, 192, 1, True, "bf16", "M"),        # K-T
    (128, 512, 256, "N", True, "f16", True),      # one-element x1Scale with a per-channel x2Scale: multiplied separately
    # enough tiles for the four-wave kernel with 256 x 32n tiles: 4 x 65 tiles of 256 x 256 would take 2 rounds of 256 CUs,
    # 4 x 60 tiles of 256 x 288 one (ragged last column tile; one-element x1Scale in the second case)
    (1000, 1024, 16600, "N", True, "bf16", "M"),
    (1024, 1024, 16640, "N", False, "f16", True),
    # up to 32 rows (x1 in registers, x2 streamed once per 16 rows): K shared by 16 waves and by 8, ragged columns, one pass
    # and two, one-element scales
    (1, 4096, 512, "N", True, "bf16", "M"),
    (16, 7168, 1000, "N", False, "f16", "M"),
    (20, 2048, 264, "N", True, "bf16", "M"),
    (32, 1024, 256, 1, True, "f16", True),
    # ... a K that one workgroup's waves do not share exactly: one segment with idle waves, K segments with partial sums
    (16, 3584, 264, "N", True, "bf16", "M"),
    (16, 11008, 256, "N", True, "f16", "M"),
    (9, 18432, 520, "N", False, "bf16", "M"),
    (16, 13824, 256, 1, True, "f16", True),
    # 33 .. 64 rows (N % 32 == 0, K % 512 == 0): x1 widened into the workspace, the many-rows streaming kernel
    (40, 2048, 512, "N", True, "bf16", "M"),
    (64, 7168, 288, "N", False, "f16", "M"),
    (33, 512, 256, 1, True, "f16", True),
    # 65 .. 128 rows: the same kernel's 128-row instance
    (65, 1024, 288, "N", True, "bf16", "M"),
    (128, 3584, 512, "N", False, "f16", "M"),
    (100, 512, 256, 1, True, "bf16", True),
    # ... K in whole 128-element blocks but no whole rounds of the chunk pipeline; K segments against a narrow x2 (86 blocks in
    # five, 148 in eight, 144 in four with two row slabs, 108 at 17 .. 32 rows)
    (40, 1664, 256, "N", True, "bf16", "M"),
    (64, 11008, 512, "N", True, "f16", "M"),
    (50, 18944, 256, "N", False, "bf16", "M"),
    (128, 18432, 1024, 1, True, "f16", True),
    (24, 13824, 384, "N", True, "bf16", "M"),
])
def test_gpu_fp8_row_and_column_scales_on_the_matrix_cores(gpu, M, K, N, s_len, bias, out_dt, pt, fast):
    """fp8 e4m3 K-C / K-T / T-C-double-scale on the matrix cores (K-contiguous x2, K % 128 == 0, 16-bit output).  Default:
    exact fp16 products, the bar of any fp32-accumulating device (max rel 2^-7, mean rel 2^-10, 99.9 % within 1e-3).
    fast (opsnnSetFp8Fast(1)): the 8-bit matrix instruction sums with a reduced-width aligner, bar mean rel <= 2^-10,
    max rel <= 10 * 2^-7 on a floored denominator, >= 97 % within 1e-3.  The same call forced onto the plain kernel is
    bit-identical to the oracle."""
    import os
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16}
    print(f"case fp8 row/col scales {M}x{K}x{N} scale_len={s_len} bias={bias} out={out_dt} pt={pt}", flush=True)
    inp = cases.make_tc_inputs(m, M, K, N, M + N, m.ACL_FLOAT8_E4M3FN, m.ACL_FLOAT, 1 if s_len == 1 else N, m.ACL_FLOAT if bias else None,
                               True, pertoken=pt)
    want = cases.oracle_tc(m, inp, M, K, N, dt[out_dt])
    m.lib().opsnnSetFp8Fast(1 if fast else 0)
    try:
        got = cases.run_tc_aclnn(m, inp, M, K, N, dt[out_dt])
    finally:
        m.lib().opsnnSetFp8Fast(0)
    code = orc.BF16 if out_dt == "bf16" else orc.F16
    g, w = orc.b16_to_f32(got, code), orc.b16_to_f32(want, code)
    assert np.isfinite(g).all()
    mx, mean = orc.rel_err_stats(g, w)
    assert mean <= 2.0 ** -10 and mx <= (10 if fast else 1) * 2.0 ** -7, f"max rel {mx:.3e} mean rel {mean:.3e}"
    assert orc.isclose_fraction(g, w) <= (3e-2 if fast else 1e-3)
    assert not np.array_equal(got, np.full_like(got, 0x7F7F))
    m.lib().opsnnSetForcePlain(1)
    try:
        exact = cases.run_tc_aclnn(m, inp, M, K, N, dt[out_dt])
    finally:
        m.lib().opsnnSetForcePlain(0)
    assert np.array_equal(exact, want)


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N,in_dt,s_dt,s_len,bias,out_dt,tB,pt", [
    # no per-token scale (the scale is then a packed 64-bit word, 19 bits kept): (sum + float bias) * scale
    (256, 2048, 384, "e4m3", "u64", "N", True, "bf16", True, False),
    (300, 384, 260, "e4m3", "u64", 1, False, "f16", True, False),
    # both scales one element, no bias: merged and truncated
    (256, 1024, 256, "e4m3", "f32", 1, False, "bf16", True, True),
    # one-element per-token scale with a bias: multiplied separately, bias after
    (200, 384, 136, "e4m3", "f32", 1, True, "f16", True, True),
    # e5m2 operands: per-token x per-channel with bias, packed scale without a per-token scale, one scale per row
    (256, 2048, 256, "e5m2", "f32", "N", True, "bf16", True, True),
    (130, 384, 200, "e5m2", "u64", "N", False, "f16", True, False),
    (128, 256, 192, "e5m2", "f32", "N", True, "bf16", True, "M"),
    # K tails and an N-contiguous x2: gathered into zero-padded K-contiguous copies first
    (256, 1000, 264, "e4m3", "u64", "N", True, "bf16", True, False),
    (128, 512, 256, "e4m3", "f32", 1, False, "f16", False, True),
    (160, 200, 136, "e5m2", "f32", "N", True, "bf16", False, True),
    # fp32 output (stored straight from the sums' registers): the three forms, ragged columns, a K tail
    (256, 1024, 384, "e4m3", "f32", "N", True, "f32", True, "M"),
    (200, 512, 130, "e4m3", "u64", "N", True, "f32", True, False),
    (128, 256, 256, "e5m2", "f32", 1, False, "f32", True, True),
    (130, 1000, 264, "e4m3", "f32", "N", False, "f32", True, "M"),
])
def test_gpu_fp8_tc_forms_on_the_matrix_cores(gpu, M, K, N, in_dt, s_dt, s_len, bias, out_dt, tB, pt):
    """The fp8 members of the per-tensor / per-channel family with a 16-bit output on the exact matrix-core kernel (fp16
    products of the widened operands, fp32 sums): bar of any fp32-accumulating device; the same call on the plain kernel is
    bit-identical to the oracle (test_gpu_matches_oracle covers the small shapes that stay there)."""
    m = gpu
    dt = {"e4m3": m.ACL_FLOAT8_E4M3FN, "e5m2": m.ACL_FLOAT8_E5M2, "u64": m.ACL_UINT64, "f32": m.ACL_FLOAT, "bf16": m.ACL_BF16,
          "f16": m.ACL_FLOAT16}
    print(f"case fp8 tc form {M}x{K}x{N} in={in_dt} scale={s_dt}/{s_len} bias={bias} out={out_dt} tB={tB} pt={pt}", flush=True)
    if out_dt == "f32":
        # the matrix-core route is the one taken: the plain kernel would be bit-identical to the oracle, this one differs in
        # the order of the sums only
        inp = cases.make_tc_inputs(m, M, K, N, M + K, dt[in_dt], dt[s_dt], 1 if s_len == 1 else N, m.ACL_FLOAT if bias else None, tB,
                                   pertoken=pt, e5m2=in_dt == "e5m2")
        want = cases.oracle_tc(m, inp, M, K, N, m.ACL_FLOAT)
        got = cases.run_tc_aclnn(m, inp, M, K, N, m.ACL_FLOAT)
        assert got.dtype == np.float32 and np.isfinite(got).all()
        mx, mean = orc.rel_err_stats(got, want)
        assert mean <= 2.0 ** -16 and orc.isclose_fraction(got, want) == 0.0, f"max rel {mx:.3e} mean rel {mean:.3e}"
        return
    inp = cases.make_tc_inputs(m, M, K, N, M + K, dt[in_dt], dt[s_dt], 1 if s_len == 1 else N, m.ACL_FLOAT if bias else None, tB,
                               pertoken=pt, e5m2=in_dt == "e5m2")
    want = cases.oracle_tc(m, inp, M, K, N, dt[out_dt])
    got = cases.run_tc_aclnn(m, inp, M, K, N, dt[out_dt])
    code = orc.BF16 if out_dt == "bf16" else orc.F16
    g, w = orc.b16_to_f32(got, code), orc.b16_to_f32(want, code)
    assert np.isfinite(g).all()
    mx, mean = orc.rel_err_stats(g, w)
    assert mean <= 2.0 ** -10 and mx <= 2.0 ** -7, f"max rel {mx:.3e} mean rel {mean:.3e}"
    assert orc.isclose_fraction(g, w) <= 1e-3
    differ = float(np.mean(got != want))
    print(f"   {differ:.2e} of outputs differ from the ascending-k oracle", flush=True)
    assert differ < 2e-2   # summation order only: a wrong scale decoding or epilogue order would change most outputs
