"""K-group modes of quant_batch_matmul_v4 behind aclnnQuantMatmulV5: fp8 x fp4 MX, fp8 x fp4 with 16-bit group
scales and a packed output scale (T-CG), int8 per-tile, int4 x int4 with per-group scales and offsets.

CPU part: the two new oracle functions are pinned by independent numpy recomputations of the reference formulas
(matmul/quant_batch_matmul_v4/tests/assets/qbmmv4_kernel_golden.py:189-255, 328-395) and by special cases that
reduce to plain matrix products; the MX and per-tile modes reuse oracle functions that are pinned elsewhere (int8
per-tile partial sums are integers below 2^24, so the fp32 sums of the block-scale function are exact).
GPU part: the library through the aclnn C ABI must be bit-identical to the oracle (plain kernels, same operation order).
"""
import numpy as np
import pytest

import cases
import oracle_api as orc


def fp4_decode(packed):
    return cases.FP4_VALUES[orc.unpack_nibbles(packed)]


def i4_decode(packed):
    v = orc.unpack_nibbles(packed).astype(np.int32)
    return np.where(v >= 8, v - 16, v)


def matmul_ascending(a, b):
    out = np.zeros((a.shape[0], b.shape[1]), np.float32)
    for k in range(a.shape[1]):
        out = (out + a[:, k:k + 1] * b[k:k + 1, :]).astype(np.float32)
    return out


@pytest.mark.parametrize("s_dt", ["bf16", "f16"])
def test_tcg_against_numpy(s_dt):
    M, K, N = 5, 64, 12
    rng = np.random.default_rng(3)
    x1 = orc.f32_to_e4m3(rng.normal(0, 1, (M, K)).astype(np.float32))
    x2 = orc.pack_nibbles(rng.integers(0, 16, size=(N, K), dtype=np.uint8))
    sf = rng.uniform(0.05, 60, (N, K // 32)).astype(np.float32)
    to16, from16, code = (orc.f32_to_bf16, orc.bf16_to_f32, orc.BF16) if s_dt == "bf16" else (orc.f32_to_f16, orc.f16_to_f32, orc.F16)
    s2 = to16(sf)
    ysf = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    ys = orc.pack_u64_scale(ysf)
    bias = rng.normal(0, 1, N).astype(np.float32)
    # w = e4m3(T16(fp4 * scale)); the fp4 values are exact in both 16-bit types
    w = fp4_decode(x2).T                                         # [K, N]
    sc = np.repeat(from16(s2).T, 32, axis=0)                     # [K, N]
    mid = from16(to16((w * sc).astype(np.float32)))
    wq = orc.e4m3_to_f32(orc.f32_to_e4m3(mid))
    deq = (ysf.view(np.uint32) & np.uint32(0xFFFFE000)).view(np.float32)
    want = orc.f32_to_f16(((matmul_ascending(orc.e4m3_to_f32(x1), wq) * deq).astype(np.float32) + bias).astype(np.float32))
    got = orc.qmm_tcg(x1, x2, M, K, N, True, s2, code, 32, ys, bias, orc.F16)
    assert np.array_equal(got, want)
    # the untransposed storage gives the same result
    x2_kn = orc.pack_nibbles(np.ascontiguousarray(orc.unpack_nibbles(x2).T))
    s2_kn = np.ascontiguousarray(s2.T)
    assert np.array_equal(orc.qmm_tcg(x1, x2_kn, M, K, N, False, s2_kn, code, 32, ys, bias, orc.F16), want)


def test_tcg_unit_scales_is_a_plain_product():
    # scale 1.0 and an output scale of 1.0: fp4 values survive both roundings, the result is x1 @ x2 in fp32
    M, K, N = 4, 32, 8
    rng = np.random.default_rng(4)
    x1 = orc.f32_to_e4m3(rng.integers(-4, 5, (M, K)).astype(np.float32))
    x2 = orc.pack_nibbles(rng.integers(0, 16, size=(N, K), dtype=np.uint8))
    s2 = orc.f32_to_bf16(np.ones((N, 1), np.float32))
    ys = orc.pack_u64_scale(np.ones(N, np.float32))
    got = orc.qmm_tcg(x1, x2, M, K, N, True, s2, orc.BF16, 32, ys, None, orc.F32)
    want = orc.e4m3_to_f32(x1).astype(np.float64) @ fp4_decode(x2).T.astype(np.float64)   # small half-integers: exact
    assert np.array_equal(got.astype(np.float64), want)


def test_i4_asym_against_numpy():
    M, K, N = 6, 600, 10      # 600 = 2 full groups of 256 and a ragged third
    rng = np.random.default_rng(5)
    x1 = orc.pack_nibbles(rng.integers(0, 16, size=(M, K), dtype=np.uint8))
    x2 = orc.pack_nibbles(rng.integers(0, 16, size=(N, K), dtype=np.uint8))
    G = 3
    s1 = rng.uniform(0.01, 0.1, (M, 1)).astype(np.float32)
    s2 = rng.uniform(0.01, 0.1, (G, N)).astype(np.float32)
    off = orc.f32_to_f16(rng.uniform(-8, 8, (G, N)).astype(np.float32))
    a, b = i4_decode(x1).astype(np.int64), i4_decode(x2).T.astype(np.int64)
    out = np.zeros((M, N), np.float32)
    for g in range(G):
        ks = slice(256 * g, min(256 * (g + 1), K))
        mm = (a[:, ks] @ b[ks, :]).astype(np.float32)
        rs = a[:, ks].sum(axis=1, keepdims=True).astype(np.float32)
        o = (rs * orc.f16_to_f32(off[g:g + 1, :])).astype(np.float32)
        out = (out + ((mm - o).astype(np.float32) * s2[g:g + 1, :]).astype(np.float32)).astype(np.float32)
    want = orc.f32_to_bf16((out * s1).astype(np.float32))
    assert np.array_equal(orc.qmm_i4_asym(x1, x2, M, K, N, True, s1, s2, off, orc.BF16), want)


def test_i4_asym_without_offsets_is_the_per_token_formula():
    # zero offsets, one group, power-of-two scales: out = (x1 @ x2) * s2[n] * s1[m] exactly, as in compute_pertoken
    M, K, N = 5, 256, 7
    rng = np.random.default_rng(6)
    x1 = orc.pack_nibbles(rng.integers(0, 16, size=(M, K), dtype=np.uint8))
    x2 = orc.pack_nibbles(rng.integers(0, 16, size=(N, K), dtype=np.uint8))
    s1 = (2.0 ** rng.integers(-6, -1, (M, 1))).astype(np.float32)
    s2 = (2.0 ** rng.integers(-6, -1, (1, N))).astype(np.float32)
    off = np.zeros((1, N), np.uint16)
    acc = i4_decode(x1).astype(np.int64) @ i4_decode(x2).T.astype(np.int64)
    want = (acc.astype(np.float64) * s2.astype(np.float64) * s1.astype(np.float64)).astype(np.float32)
    assert np.array_equal(orc.qmm_i4_asym(x1, x2, M, K, N, True, s1, s2, off, orc.F32), want)


def test_pertile_i8_partial_sums_are_exact():
    # the block-scale oracle sums int8 products in fp32; per 128-K tile they are integers below 2^24, so the result
    # equals the int32-matmul formulation of compute_per_tile (qbmmv4_kernel_golden.py:258-325)
    M, K, N = 4, 300, 140
    rng = np.random.default_rng(7)
    x1 = np.full((M, K), 127, np.int8); x2 = np.full((K, N), -127, np.int8)     # worst case magnitude
    x1[1:] = rng.integers(-127, 128, (M - 1, K)); x2[:, 1:] = rng.integers(-127, 128, (K, N - 1))
    s1 = rng.uniform(1e-3, 1e-2, (M, 3)).astype(np.float32); s2 = rng.uniform(1e-3, 1e-2, (3, 2)).astype(np.float32)
    bias = rng.normal(0, 1, N).astype(np.float32)
    out = np.zeros((M, N), np.float32)
    for kb in range(3):
        ks = slice(128 * kb, min(128 * (kb + 1), K))
        mm = (x1[:, ks].astype(np.int32) @ x2[ks, :].astype(np.int32)).astype(np.float32)
        sc = (s1[:, kb:kb + 1] * np.repeat(s2[kb:kb + 1, :], 128, axis=1)[:, :N]).astype(np.float32)
        out = (out + (mm * sc).astype(np.float32)).astype(np.float32)
    want = orc.f32_to_bf16((out + bias).astype(np.float32))
    got = orc.qmm_perblock(x1, x2, orc.I8, orc.I8, M, K, N, False, False, s1, s2, 1, 128, 128, bias, orc.BF16)
    assert np.array_equal(got, want)


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N,tB", [(16, 128, 128, True), (33, 192, 72, True), (20, 256, 64, True)])
def test_gpu_a8w4_mx(gpu, M, K, N, tB):
    m = gpu
    print(f"case a8w4 mx {M}x{K}x{N} tB={tB}", flush=True)
    inp = cases.make_a8w4_mx_inputs(m, M, K, N, M + N, tB)
    want = cases.oracle_a8w4_mx(m, inp, M, K, N, tB, m.ACL_FLOAT16)
    got = cases.run_a8w4_mx_aclnn(m, inp, M, K, N, tB, m.ACL_FLOAT16)
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ"


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N", [(64, 128, 64), (300, 384, 260), (512, 2048, 520), (100, 1024, 1000), (1024, 4096, 1024),
                                   # up to 32 rows: x1 in registers, x2 streamed once per 16 rows; K shared by 16 waves (2 or 4
                                   # chunks of 128 each) or by 8 (1 .. 7), ragged columns, two passes
                                   (16, 4096, 512), (9, 8192, 264), (24, 1024, 520), (1, 7168, 384), (32, 3072, 256),
                                   (16, 2048, 256),
                                   # ... a K that one workgroup's waves do not share exactly: one segment with idle waves (28
                                   # chunks), K segments with fp32 partial sums (86, 144, 19 chunks; two passes; one row)
                                   (16, 3584, 256), (16, 11008, 264), (7, 2432, 512), (1, 18944, 384), (3, 128, 256), (16, 640, 264),
                                   # 17 .. 32 rows: the tile kernel, with K split where the tiles are few
                                   (32, 18432, 256), (24, 4096, 512), (17, 11008, 264),
                                   # few tiles against a long K: K split over 2 .. 16 workgroups per tile, fp32 partial sums in the
                                   # workspace, summed in split order (also (512, 2048, 520), (100, 1024, 1000) and
                                   # (1024, 4096, 1024) above); a column count that is no multiple of 4
                                   (128, 4096, 4096), (40, 8192, 256), (77, 1024, 258), (200, 2048, 1000)])
def test_gpu_a8w4_mx_on_the_matrix_cores(gpu, M, K, N):
    """fp8 x fp4 MX with K % 128 == 0 and enough outputs runs on the scaled matrix instruction with a 4-bit x2 operand.
    With a 4-bit operand the instruction's sums are as close to the fp32-accumulated ones as exact fp16 products are
    (measured at these shapes and at 4096 x 8192 x 8192 / 16 x 8192 x 28672: the same share of bit-identical outputs), so
    the bar is the stated one: max rel 2^-7, mean rel 2^-10, 99.9 % within rtol = atol = 1e-3.  The same call on the plain
    kernel is bit-identical to the oracle."""
    m = gpu
    print(f"case a8w4 mx mfma {M}x{K}x{N}", flush=True)
    inp = cases.make_a8w4_mx_inputs(m, M, K, N, M + N, True)
    want = cases.oracle_a8w4_mx(m, inp, M, K, N, True, m.ACL_FLOAT16)
    got = cases.run_a8w4_mx_aclnn(m, inp, M, K, N, True, m.ACL_FLOAT16)
    g, w = orc.b16_to_f32(got, orc.F16), orc.b16_to_f32(want, orc.F16)
    assert np.isfinite(g).all()
    mx, mean = orc.rel_err_stats(g, w)
    assert mx <= 2.0 ** -7 and mean <= 2.0 ** -10, f"max rel {mx:.3e} mean rel {mean:.3e}"
    assert orc.isclose_fraction(g, w) <= 1e-3
    m.lib().opsnnSetForcePlain(1)
    try:
        exact = cases.run_a8w4_mx_aclnn(m, inp, M, K, N, True, m.ACL_FLOAT16)
    finally:
        m.lib().opsnnSetForcePlain(0)
    assert np.array_equal(exact, want)


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N,s_dt,out_dt,ys_i64", [(16, 64, 16, "bf16", "f16", False), (16, 64, 16, "bf16", "f16", True),
                                                      (37, 256, 50, "f16", "bf16", False), (9, 128, 130, "bf16", "bf16", False)])
def test_gpu_tcg(gpu, M, K, N, s_dt, out_dt, ys_i64):
    m = gpu
    print(f"case tcg {M}x{K}x{N} scale={s_dt} out={out_dt} yscale int64={ys_i64}", flush=True)
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16}
    inp = cases.make_tcg_inputs(m, M, K, N, M + N, dt[s_dt])
    want = cases.oracle_tcg(m, inp, M, K, N, dt[out_dt])
    got = cases.run_tcg_aclnn(m, inp, M, K, N, dt[out_dt], m.ACL_INT64 if ys_i64 else None)
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ"


@pytest.mark.gpu
@pytest.mark.parametrize("fast", [False, True])
@pytest.mark.parametrize("M,K,N,s_dt,out_dt", [(64, 128, 64, "bf16", "bf16"), (300, 384, 260, "f16", "f16"),
                                               (512, 2048, 520, "bf16", "bf16"), (1024, 1024, 2048, "bf16", "f16"),
                                               # few rows: the streaming kernels behind the same prologue (x1 in registers up
                                               # to 16 rows, two passes up to 32, the many-rows kernel from 17 to 128)
                                               (16, 4096, 512, "bf16", "bf16"), (9, 2048, 264, "f16", "f16"),
                                               (24, 1024, 520, "bf16", "f16"), (40, 2048, 512, "bf16", "bf16"),
                                               (100, 1024, 256, "f16", "bf16"),
                                               # K tails (K % 128 = 32, 64, 96): the re-quantised weight and a copy of x1 in
                                               # rows padded with zeros to the next multiple of 128
                                               (300, 416, 260, "bf16", "bf16"), (16, 1984, 512, "f16", "f16"),
                                               (64, 1120, 256, "bf16", "f16")])
def test_gpu_tcg_on_the_matrix_cores(gpu, M, K, N, s_dt, out_dt, fast):
    """fp8 x fp4 with 16-bit group scales, K % 128 == 0 and enough outputs: a prologue writes the re-quantised e4m3 weight
    (the oracle's bytes) into the workspace and the fp8 matrix-core kernel does the product with the decoded output scale
    per column (every third group scale is negative here).  Default (exact fp16 products): max rel 2^-7, mean rel 2^-10,
    99.9 % within rtol = atol = 1e-3.  fast (the 8-bit matrix instruction): the dot product's backward-error bound with
    the instruction's alignment error against sum|terms|, mean rel <= 2^-10.  The same call on the plain kernel is
    bit-identical to the oracle."""
    import os
    m = gpu
    print(f"case tcg mfma {M}x{K}x{N} scale={s_dt} out={out_dt}", flush=True)
    dt = {"bf16": (m.ACL_BF16, orc.BF16), "f16": (m.ACL_FLOAT16, orc.F16)}
    inp = cases.make_tcg_inputs(m, M, K, N, M + N, dt[s_dt][0])
    inp["s2"] = inp["s2"] ^ ((np.arange(inp["s2"].size, dtype=np.uint32).reshape(inp["s2"].shape) % 3 == 0).astype(np.uint16) << 15)
    want = cases.oracle_tcg(m, inp, M, K, N, dt[out_dt][0])
    m.lib().opsnnSetFp8Fast(1 if fast else 0)
    try:
        got = cases.run_tcg_aclnn(m, inp, M, K, N, dt[out_dt][0])
    finally:
        m.lib().opsnnSetFp8Fast(0)
    odt = dt[out_dt][1]
    g, w = orc.b16_to_f32(got, odt), orc.b16_to_f32(want, odt)
    assert np.isfinite(g).all()
    mx, mean = orc.rel_err_stats(g, w)
    if fast:
        pos = dict(inp, x1=inp["x1"] & 0x7F, x2=inp["x2"] & 0x77, s2=inp["s2"] & 0x7FFF)
        abs_sum = orc.b16_to_f32(cases.oracle_tcg(m, pos, M, K, N, dt[out_dt][0]), odt).astype(np.float64)
        err = np.abs(g.astype(np.float64) - w)
        bound = 2.0 ** -7 * np.abs(w) + 2.0 ** -14 * abs_sum
        assert float((err / np.maximum(bound, 1e-30)).max()) <= 1.0 and mean <= 2.0 ** -10, f"max rel {mx:.3e} mean rel {mean:.3e}"
    else:
        assert mx <= 2.0 ** -7 and mean <= 2.0 ** -10, f"max rel {mx:.3e} mean rel {mean:.3e}"
        assert orc.isclose_fraction(g, w) <= 1e-3
    m.lib().opsnnSetForcePlain(1)
    try:
        exact = cases.run_tcg_aclnn(m, inp, M, K, N, dt[out_dt][0])
    finally:
        m.lib().opsnnSetForcePlain(0)
    assert np.array_equal(exact, want)


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N,tB", [(16, 256, 128, True), (40, 300, 200, False), (7, 128, 130, True)])
def test_gpu_pertile_i8(gpu, M, K, N, tB):
    m = gpu
    print(f"case int8 per-tile {M}x{K}x{N} tB={tB}", flush=True)
    inp = cases.make_pertile_i8_inputs(m, M, K, N, M + N, tB)
    want = cases.oracle_pertile_i8(m, inp, M, K, N, tB, m.ACL_BF16)
    got = cases.run_pertile_i8_aclnn(m, inp, M, K, N, tB, m.ACL_BF16)
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ"


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N,tB", [(128, 256, 256, True), (300, 384, 260, True), (640, 1024, 520, False),
                                      # up to 32 rows: x1 in registers, x2 streamed once per 16 rows (int8 instructions)
                                      (16, 4096, 512, True), (9, 2048, 264, True), (24, 1024, 520, True), (16, 1024, 256, False),
                                      (1, 7168, 384, True),
                                      # ... a K that one workgroup's waves do not share exactly: idle waves, K segments
                                      (16, 3584, 256, True), (16, 11008, 264, True), (20, 18432, 256, True), (5, 128, 256, True),
                                      # few tiles against a long K: the K split ((640, 1024, 520) above: with the re-layout of
                                      # an N-contiguous x2 behind the partial sums in the workspace)
                                      (128, 4096, 4096, True), (40, 8192, 256, True), (96, 1024, 258, True), (200, 2048, 1000, False)])
def test_gpu_pertile_i8_on_the_matrix_cores(gpu, M, K, N, tB):
    """int8 per-tile with K % 128 == 0 and enough outputs runs on the block-scale kernel with int8 instructions: the
    block sums are exact integers, the fold into the running sum is a fused multiply-add (one rounding where the oracle
    has two), so the bar is max rel <= 2^-7 and mean rel <= 2^-10; forced onto the plain kernel the call is bit-identical."""
    import os
    m = gpu
    print(f"case int8 per-tile mfma {M}x{K}x{N} tB={tB}", flush=True)
    inp = cases.make_pertile_i8_inputs(m, M, K, N, M + N, tB)
    want = cases.oracle_pertile_i8(m, inp, M, K, N, tB, m.ACL_BF16)
    got = cases.run_pertile_i8_aclnn(m, inp, M, K, N, tB, m.ACL_BF16)
    g, w = orc.b16_to_f32(got, orc.BF16), orc.b16_to_f32(want, orc.BF16)
    assert np.isfinite(g).all()
    mx, mean = orc.rel_err_stats(g, w)
    assert mx <= 2.0 ** -7 and mean <= 2.0 ** -10, f"max rel {mx:.3e} mean rel {mean:.3e}"
    assert orc.isclose_fraction(g, w) <= 1e-3
    m.lib().opsnnSetForcePlain(1)
    try:
        exact = cases.run_pertile_i8_aclnn(m, inp, M, K, N, tB, m.ACL_BF16)
    finally:
        m.lib().opsnnSetForcePlain(0)
    assert np.array_equal(exact, want)


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N,out_dt", [(9, 1024, 256, "bf16"), (9, 1024, 256, "f16"), (33, 2048, 512, "bf16"),
                                          # several row and column tiles, ragged in both; one group; a last group of 128; the
                                          # one-thread-per-output kernel (fewer than 32 x 32 outputs)
                                          (130, 1024, 512, "bf16"), (257, 4096, 768, "f16"), (1, 1024, 1280, "bf16"),
                                          (3, 1024, 256, "f16")])
def test_gpu_i4_asym(gpu, M, K, N, out_dt):
    """int4 x int4 with group scales and offsets: the matrix-core kernel (operands widened to int8 in the workspace) is
    bit-identical to the oracle, as the integer group sums are exact and the fp32 fold follows the golden's order."""
    m = gpu
    print(f"case int4 K-G {M}x{K}x{N} out={out_dt}", flush=True)
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16}
    inp = cases.make_i4_asym_inputs(m, M, K, N, M + N)
    want = cases.oracle_i4_asym(m, inp, M, K, N, dt[out_dt])
    got = cases.run_i4_asym_aclnn(m, inp, M, K, N, dt[out_dt])
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ"


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N,variant", [(130, 768, 200, 0), (70, 400, 1030, 0), (33, 250, 36, 0), (130, 768, 200, "plain")])
def test_gpu_i4_asym_kernel_level_ragged_shapes(gpu, M, K, N, variant):
    """opsnnQmmGroup called directly with shapes the aclnn layer does not let through (it wants K % 1024 == 0 and
    N % 256 == 0): ragged row and column tiles and a partial last group, against the oracle bit for bit."""
    m = gpu
    print(f"case int4 K-G kernel level {M}x{K}x{N} variant={variant}", flush=True)
    inp = cases.make_i4_asym_inputs(m, M, K, N, M + N + K)
    want = cases.oracle_i4_asym(m, inp, M, K, N, m.ACL_BF16)
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items()}
    d_out = m.DeviceBuffer(M * N * 2); d_out.fill(0xFF)
    G = -(-K // 256)
    a = m.OpsnnQmmArgs()
    a.M, a.N, a.K, a.batch = M, N, K, 1
    a.x1 = m.OpsnnMat(d["x1"].ptr, K, 1, 0)
    a.x2 = m.OpsnnMat(d["x2"].ptr, 1, K, 0)
    a.x1_dtype = a.x2_dtype = m.ACL_INT4
    a.out, a.out_dtype = d_out.ptr, m.ACL_BF16
    a.x1_scale = d["s1"].ptr
    a.gsM, a.gsN, a.gsK = 1, 1, 256
    a.x2_scale_mat = m.OpsnnMat(d["s2"].ptr, N, 1, 0)
    a.x2_offset_mat = m.OpsnnMat(d["off"].ptr, N, 1, 0)
    a.x2_scale_dtype = m.ACL_FLOAT
    a.force_variant = m.VARIANT_PLAIN if variant == "plain" else m.VARIANT_AUTO
    need = m.lib().opsnnQmmWorkspace(a, 4)
    assert (need > 0) == (M * N >= 1024)
    ws = m.DeviceBuffer(need) if need else None
    a.workspace = ws.ptr if ws else None
    assert m.lib().opsnnQmmGroup(a, None) == 0
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    got = d_out.to_host(np.uint16, (M, N))
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ"


@pytest.mark.gpu
@pytest.mark.parametrize("pattern", ["all_min", "min_with_units", "alternating", "sparse_units"])
def test_gpu_i4_asym_extreme_group_sums(gpu, pattern):
    """The matrix-core kernel multiplies the int4 operands as e4m3 bytes and takes the group sum from the matrix
    pipe as fp32.  That is exact only if the pipe adds 256 products of magnitude up to 64 onto a running sum of up
    to 16384 without dropping low bits: checked here on operands built to need every bit (largest products
    throughout with a few products of magnitude 1 among them, sums that cancel, lone units), bit for bit against
    the oracle's integer sums."""
    m = gpu
    M, K, N = 64, 1024, 256
    print(f"case int4 K-G extreme sums pattern={pattern}", flush=True)
    rng = np.random.default_rng(7)
    inp = cases.make_i4_asym_inputs(m, M, K, N, 11)
    a = np.full((M, K), 8, dtype=np.uint8)   # nibble 8 = -8
    b = np.full((N, K), 8, dtype=np.uint8)
    if pattern == "min_with_units":
        # most products 64, a handful of +-1 and +-7 at random places of each row
        for mat in (a, b):
            idx = rng.integers(0, K, size=(mat.shape[0], 24))
            vals = rng.choice(np.array([1, 15, 7, 9], dtype=np.uint8), size=idx.shape)
            np.put_along_axis(mat, idx, vals, axis=1)
    elif pattern == "alternating":
        a[:, 1::2] = 7          # -8, 7, -8, 7 ... against -8 everywhere: +64 and -56 alternate
        b[1::2, :] = 7          # and against 7 everywhere in every other column
    elif pattern == "sparse_units":
        a[:] = 0
        b[:] = 0
        for mat in (a, b):
            idx = rng.integers(0, K, size=(mat.shape[0], 40))
            np.put_along_axis(mat, idx, rng.choice(np.array([1, 15], dtype=np.uint8), size=idx.shape), axis=1)
        a[:, ::256] = 8
        b[:, ::256] = 8         # one product of 64 per group next to the units
    inp["x1"], inp["x2"] = orc.pack_nibbles(a), orc.pack_nibbles(b)
    if pattern in ("all_min", "min_with_units"):
        # offset -8 takes the bulk (x2 = -8) out of every group: what is left of a group is the small integer
        # sum x1 * (x2 + 8), so one lost unit of the group sum changes the output beyond any rounding
        inp["off"] = orc.f32_to_f16(np.full(inp["off"].shape, -8.0, dtype=np.float32))
    want = cases.oracle_i4_asym(m, inp, M, K, N, m.ACL_BF16)
    got = cases.run_i4_asym_aclnn(m, inp, M, K, N, m.ACL_BF16)
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ"
    # the output rounds to bf16: compare the fp16 output too (three more bits of the fold's result)
    want = cases.oracle_i4_asym(m, inp, M, K, N, m.ACL_FLOAT16)
    got = cases.run_i4_asym_aclnn(m, inp, M, K, N, m.ACL_FLOAT16)
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} fp16 outputs differ"
