"""GPU parity for the fp8 block-scale, MX and weight-only paths.

Two bars.  (1) The plain kernels evaluate the golden formulas operation by operation in ascending-k order, as
the oracle does, so they must match it bit for bit.  (2) The MFMA kernels accumulate in another order (as the
reference hardware and BLAS do); for them the bar is: max relative error <= 2^-7 and mean relative error <= 2^-10
against the fp32-accumulated oracle (denominator floored at 1 % of the mean magnitude), plus the reference's own
acceptance rule (>= 99.9 % of elements within rtol = atol = 1e-3).  The fp8 block-scale and row/column-scale modes
and the MX modes with fp8 operands run by default on exact fp16 products (that bar); their opt-in 8-bit
matrix-instruction form (opsnnSetFp8Fast) is held to the looser bars written out in check_close.
"""
import os

import numpy as np
import pytest

import cases
import oracle_api as orc

pytestmark = pytest.mark.gpu

MAX_REL, MEAN_REL = 2.0 ** -7, 2.0 ** -10


def check_close(got_bits, want_bits, dt, what, exact=False, fp8_mfma=False, abs_sum=None):
    if exact:
        if not np.array_equal(got_bits, want_bits):
            bad = np.argwhere(got_bits != want_bits)
            raise AssertionError(f"{what}: {len(bad)} of {got_bits.size} differ, first at {bad[0]}")
        return
    got, want = orc.b16_to_f32(got_bits, dt), orc.b16_to_f32(want_bits, dt)
    if not np.isfinite(got).all():
        bad = np.argwhere(~np.isfinite(got))
        raise AssertionError(f"{what}: {len(bad)} non-finite outputs of {got.size}, first at {bad[0]}, last at {bad[-1]}")
    mx, mean = orc.rel_err_stats(got, want)
    frac = orc.isclose_fraction(got, want)
    if abs_sum is not None:
        # MX scales of neighbouring blocks differ by up to 2^16 in these inputs, and one 8-bit matrix instruction adds
        # four such blocks with its reduced-width aligner (error about 1e-5 of sum|terms|, measured): where the terms
        # cancel, that error is large against the RESULT however it is computed in fp32-with-alignment hardware.  The
        # bar that fits is the dot product's backward-error bound: two 16-bit roundings of the result plus 2^-14 of
        # sum|terms| per element, with the mean relative error held to 2^-10 as everywhere.
        err = np.abs(got.astype(np.float64) - want)
        bound = MAX_REL * np.abs(want) + 2.0 ** -14 * abs_sum
        worst = float((err / np.maximum(bound, 1e-30)).max())
        assert worst <= 1.0 and mean <= MEAN_REL, f"{what}: error / bound {worst:.3f}, mean rel {mean:.3e}"
        assert frac <= 3e-2, f"{what}: {frac:.2e} of elements outside rtol=atol=1e-3"
        return
    if fp8_mfma:
        # The 8-bit matrix instruction sums its 64 products with a reduced-width aligner (about 1e-5 of
        # sum|terms| per instruction, measured), so 16-bit outputs flip by one ulp far more often than with exact
        # products.  Bar: mean rel <= 2^-10 as everywhere, max rel within the community standard's MARE bound
        # 10 * 2^-7 (experimental/optim/apply_ftrl/README.md:113), and no more than 3 % one-ulp flips.
        assert mean <= MEAN_REL and mx <= 10 * MAX_REL, f"{what}: max rel {mx:.3e} mean rel {mean:.3e}"
        assert frac <= 3e-2, f"{what}: {frac:.2e} of elements outside rtol=atol=1e-3"
        return
    assert mx <= MAX_REL and mean <= MEAN_REL, f"{what}: max rel {mx:.3e} mean rel {mean:.3e}"
    assert frac <= 1e-3, f"{what}: {frac:.2e} of elements outside rtol=atol=1e-3"


def plain(flag):
    """Route through the plain kernels (set) or let the selector choose (unset)."""
    import opsnn
    opsnn.lib().opsnnSetForcePlain(1 if flag else 0)


@pytest.fixture(autouse=True)
def _reset_env(opsnn):
    yield
    opsnn.lib().opsnnSetForcePlain(0)
    opsnn.lib().opsnnSetMx8Wide(-1)
    opsnn.lib().opsnnSetFp8Fast(0)


@pytest.mark.parametrize("path", ["plain", "exact", "fast"])
@pytest.mark.parametrize("M,K,N,tB,gsM", [
    (128, 512, 256, True, 1), (128, 512, 256, False, 1), (100, 300, 200, True, 1), (256, 384, 384, True, 128),
    (130, 256, 130, False, 128), (1, 1024, 256, True, 1),
    (512, 1024, 768, True, 1), (300, 512, 520, True, 1), (384, 2048, 512, False, 1), (256, 1024, 256, True, 128),
    (700, 384, 520, True, 1), (640, 256, 264, False, 128),     # ragged edges in both directions, several row tiles
    # few tiles against a long K (also (512, 1024, 768), (384, 2048, 512) and (256, 1024, 256) above): K split over 2 .. 16
    # workgroups per tile on the exact path, partial sums in the workspace
    (300, 4096, 1000, True, 1), (256, 7168, 2048, True, 128), (200, 8192, 130, False, 1),
])
def test_fp8_blockscale(gpu, M, K, N, tB, gsM, path):
    """plain: one thread per output, bit-identical.  exact (the default): e4m3 widened to fp16, exact products, the bar
    of any fp32-accumulating device.  fast: the 8-bit matrix instruction (opsnnSetFp8Fast(1)), looser bar."""
    m = gpu
    print(f"case fp8 block M={M} K={K} N={N} tB={tB} gsM={gsM} path={path}", flush=True)
    inp = cases.make_blockscale_inputs(m, M, K, N, M + N, tB, gsM)
    want = cases.oracle_blockscale(m, inp, M, K, N, tB, m.ACL_BF16)
    plain(path == "plain")
    m.lib().opsnnSetFp8Fast(1 if path == "fast" else 0)
    got = cases.run_blockscale_aclnn(m, inp, M, K, N, tB, m.ACL_BF16)
    check_close(got, want, orc.BF16, "fp8 block scale", exact=path == "plain", fp8_mfma=path == "fast")


@pytest.mark.parametrize("M,K,N,tB,gsM,fast", [(256, 1024, 384, True, 1, False), (300, 512, 262, False, 128, False), (128, 200, 256, True, 1, False),
                                               (256, 1024, 384, True, 1, True)])
def test_fp8_blockscale_fp32_output(gpu, M, K, N, tB, gsM, fast):
    """FLOAT output of the block-scale modes: the exact matrix-core kernel stores its fp32 sums as they are (ragged
    columns, an N-contiguous x2, a K tail; with the 8-bit instruction requested the exact kernel still serves it)."""
    m = gpu
    print(f"case fp8 block fp32 out M={M} K={K} N={N} tB={tB} gsM={gsM} fast={fast}", flush=True)
    inp = cases.make_blockscale_inputs(m, M, K, N, M + N, tB, gsM)
    want = cases.oracle_blockscale(m, inp, M, K, N, tB, m.ACL_FLOAT)
    m.lib().opsnnSetFp8Fast(1 if fast else 0)
    got = cases.run_blockscale_aclnn(m, inp, M, K, N, tB, m.ACL_FLOAT)
    assert got.dtype == np.float32 and np.isfinite(got).all()
    mx, mean = orc.rel_err_stats(got, want)
    print(f"   max rel {mx:.3e} mean rel {mean:.3e}, {float(np.mean(got != want)):.3f} of fp32 outputs differ in some bit", flush=True)
    assert mean <= 2.0 ** -16 and orc.isclose_fraction(got, want) == 0.0
    assert not np.array_equal(got, want) or K <= 256   # the matrix-core route: its sums run in another order than the oracle's
    plain(True)
    assert np.array_equal(cases.run_blockscale_aclnn(m, inp, M, K, N, tB, m.ACL_FLOAT), want)


def _rows_ksplit(wbits, M, N, K, group):
    """The many-rows kernel's K segments (the library's rule, restated): 1 = K in one piece."""
    if M < 17 or N % 32 or N < 256 or K < 4096:
        return 1
    wg = -(-N // 128)
    slabs = 1
    if M > 64:
        if wg > 128:
            return 1
        n = max(min(256 // wg, -(-M // 64)), -(-M // 256))
        if n < 2:
            return 1
        slab = -(-(-(-M // n)) // 16) * 16
        slabs = -(-M // slab)
    wgs, kx = slabs * wg, 2 * 4 * (128 // wbits)
    unit = kx
    if group < K:
        unit = max(kx, group)
        if unit % group or unit % kx:
            return 1
    if wgs > 128 or K % unit:
        return 1
    if K < 8192 and (K % (2 * kx) == 0 or wgs > 64 or M < 33):
        return 1
    s = min(256 // wgs, 8, K // 2048, K // unit)
    if s == 2 and wgs > 64 and K < 12288:
        return 1
    return s if s >= 2 else 1


@pytest.mark.parametrize("M,K,N,gsM,out", [
    # up to 16 rows (one pass): K shared by 16 waves (2048, 4096, 8192) or by 8 (1024, 3072, 5120, 6144, 7168); ragged columns;
    # more column blocks than workgroups (N = 8192: 512 blocks on 256 workgroups) and fewer
    (1, 2048, 256, 1, "bf16"), (16, 4096, 512, 1, "f16"), (7, 8192, 8192, 1, "bf16"), (16, 1024, 264, 1, "bf16"),
    (5, 3072, 1000, 1, "f16"), (16, 5120, 384, 1, "f32"), (9, 6144, 256, 128, "bf16"), (16, 7168, 2304, 1, "bf16"),
    # K that the waves of one workgroup do not share exactly: one segment with idle waves (28 blocks on 16 waves of two), or K
    # segments over workgroup columns with fp32 partial sums and a second kernel (86 blocks: three segments of 16 x 2; 144:
    # three of 8 x 6; 108: seven of 16 x 1; 19: three of 8 x 1; 148 in two passes: five of 16 x 2)
    (5, 3584, 264, 1, "f16"), (16, 11008, 512, 1, "bf16"), (16, 18432, 256, 1, "bf16"), (12, 13824, 384, 128, "f32"),
    (16, 2432, 256, 1, "f16"), (32, 18944, 264, 1, "bf16"), (4, 128, 256, 1, "bf16"), (16, 640, 272, 1, "f32"),
    # 17 .. 32 rows where the many-rows kernel does not apply (N % 128, K % 512): two passes; one scale row for all of x1 (B-B)
    (17, 2048, 520, 1, "bf16"), (32, 7168, 520, 128, "f16"), (24, 1024, 256, 1, "f32"), (20, 4096, 256, 1, "f32"),
    # 17 .. 64 rows (N % 128 == 0, K % 512 == 0): x1 widened into the workspace, the many-rows streaming kernel
    (33, 2048, 512, 1, "bf16"), (64, 8192, 1024, 1, "f16"), (50, 7168, 256, 128, "bf16"), (64, 512, 384, 1, "f32"),
    (40, 1536, 2304, 1, "bf16"),
    # 65 .. 128 rows: the same kernel's 128-row instance
    (65, 2048, 512, 1, "bf16"), (128, 7168, 1024, 1, "f16"), (100, 1024, 256, 128, "f32"), (96, 16384, 256, 1, "bf16"),
    # ... K in whole scale blocks but no whole rounds of the chunk pipeline; K segments against a narrow x2 (86 blocks in five,
    # 148 in eight, 144 in four with two row slabs; 17 .. 32 rows as well)
    (40, 1664, 256, 1, "bf16"), (64, 11008, 512, 1, "f16"), (50, 18944, 256, 128, "bf16"), (128, 18432, 1024, 1, "f32"),
    (24, 13824, 384, 1, "bf16"),
])
def test_fp8_blockscale_decode_rows(gpu, M, K, N, gsM, out):
    """The block-scale modes with up to 32 rows of x1 (x2 K-contiguous): x1 stays in registers as exact fp16 and x2 is
    streamed once per 16 rows; exact products, fp32 sums per block, one fused multiply-add per block (the exact tile
    kernel's arithmetic, its bar)."""
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "f32": m.ACL_FLOAT}[out]
    print(f"case fp8 block decode M={M} K={K} N={N} gsM={gsM} out={out}", flush=True)
    inp = cases.make_blockscale_inputs(m, M, K, N, M + N + K, True, gsM)
    want = cases.oracle_blockscale(m, inp, M, K, N, True, dt)
    got = cases.run_blockscale_aclnn(m, inp, M, K, N, True, dt)
    if out == "f32":
        assert np.isfinite(got).all()
        mx, mean = orc.rel_err_stats(got, want)
        assert mean <= 2.0 ** -16 and orc.isclose_fraction(got, want) == 0.0, f"max rel {mx:.3e} mean rel {mean:.3e}"
    else:
        check_close(got, want, orc.BF16 if out == "bf16" else orc.F16, "fp8 block scale, decode rows")
        differ = float(np.mean(got != want))
        print(f"   {differ:.2e} of outputs differ from the ascending-block oracle", flush=True)
        assert differ < 2e-2
    if M > 32 and N % 128 == 0:   # phase 1 plans the fp16 copy of x1 (and the partial sums of a K split): the many-rows route is the one taken
        d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
        x1 = m.Tensor((M, K), m.ACL_FLOAT8_E4M3FN, d["x1"]); x2 = m.Tensor((N, K), m.ACL_FLOAT8_E4M3FN, d["x2"])
        s1 = m.Tensor(inp["s1"].shape[1:], m.ACL_FLOAT, d["s1"]); s2 = m.Tensor(inp["s2"].shape[1:], m.ACL_FLOAT, d["s2"])
        o = m.Tensor((M, N), dt, m.DeviceBuffer(M * N * 4))
        rc, ws, ex = m.quant_matmul_v5_get_workspace(x1, x2, s1, s2, o, transpose_x2=True, group_size=(gsM << 32) | (128 << 16) | 128)
        ks = _rows_ksplit(8, M, N, K, K)
        part = -(-ks * M * N * 4 // 256) * 256 if ks > 1 else 0
        assert rc == 0 and ws == part + M * K * 2, (rc, ws, ks)
        m.lib().aclDestroyAclOpExecutor(ex)
    plain(True)
    assert np.array_equal(cases.run_blockscale_aclnn(m, inp, M, K, N, True, dt), want)


def test_fp8_blockscale_exact_path_is_nearly_bit_identical(gpu):
    """The exact path differs from the ascending-k fp32 oracle only by summation order: at K = 2048 far fewer than
    0.5 % of bf16 outputs may differ at all (the 8-bit instruction leaves about 1 % one ulp off)."""
    m = gpu
    M, K, N = 512, 2048, 512
    inp = cases.make_blockscale_inputs(m, M, K, N, 11, True, 1)
    want = cases.oracle_blockscale(m, inp, M, K, N, True, m.ACL_BF16)
    got = cases.run_blockscale_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    differ = float(np.mean(got != want))
    print(f"exact path: {differ:.2e} of bf16 outputs differ from the oracle", flush=True)
    assert differ < 5e-3


def test_fp8_blockscale_group_size_inferred(gpu):
    """groupSize 0 is inferred from the scale shapes (quant_matmul_checker.cpp:700-722)."""
    m = gpu
    inp = cases.make_blockscale_inputs(m, 128, 256, 256, 1, True, 1)
    a = cases.run_blockscale_aclnn(m, inp, 128, 256, 256, True, m.ACL_BF16)
    b = cases.run_blockscale_aclnn(m, inp, 128, 256, 256, True, m.ACL_BF16, group_size=0)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("use_plain", [True, False, "fast"])
@pytest.mark.parametrize("M,K,N,tB,fp4", [
    (128, 256, 256, True, True), (128, 256, 256, False, True), (197, 960, 854, True, True), (64, 128, 64, True, False),
    (64, 320, 96, False, False), (33, 192, 50, True, True),
    (512, 1024, 768, True, True), (300, 512, 260, True, True), (300, 512, 260, False, True), (256, 2048, 512, True, False),
    (260, 384, 300, False, False),
    # fp4 with K % 512 == 0 takes 256-element K tiles (scales of two tiles per copy): odd and even pair counts, ragged edges
    (260, 1536, 300, True, True), (512, 2048, 264, False, True), (384, 768, 256, True, True),
    # MXFP8 on the block kernel: ragged tiles, one K tile, many K tiles, N-contiguous x2
    (300, 128, 260, True, False), (512, 4096, 256, True, False), (100, 1024, 520, False, False),
    # MXFP4 with few tiles against a long K: the K split on 128 x 128 tiles (which also replace 256 x 256 ones when those
    # would be at most 32), on 256 x 256 tiles with paired scale copies (K % 512 == 0) and without
    (64, 8192, 512, True, True), (256, 8192, 1024, True, True), (257, 8192, 4200, True, True), (257, 7936, 4200, True, True),
    (40, 8192, 300, False, True),
])
def test_mx(gpu, M, K, N, tB, fp4, use_plain):
    """plain: bit-identical.  Default: MXFP4 on the scaled 4-bit instruction (its products and sums are exact), MXFP8 on
    exact fp16 products with the block scales folded into the widening -- both at the stated bar.  fast: MXFP8 on the scaled
    8-bit matrix instruction (four 32-element blocks per instruction), held to the backward-error bound of check_close."""
    m = gpu
    fast = use_plain == "fast"
    if fast and fp4:
        pytest.skip("MXFP4 has one matrix-core form")
    print(f"case mx M={M} K={K} N={N} tB={tB} fp4={fp4} plain={use_plain}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, K + N, tB, fp4)
    bias = np.random.default_rng(1).normal(0, 1, N).astype(np.float32)
    want = cases.oracle_mx(m, inp, M, K, N, tB, m.ACL_BF16, bias)
    plain(use_plain is True)
    m.lib().opsnnSetFp8Fast(1 if fast else 0)
    got = cases.run_mx_aclnn(m, inp, M, K, N, tB, m.ACL_BF16, bias)
    abs_sum = None
    if fast:   # sum |x1 s1 x2 s2| per element: the oracle on the inputs with their sign bits cleared
        pos = dict(inp, x1=inp["x1"] & 0x7F, x2=inp["x2"] & 0x7F)
        abs_sum = orc.b16_to_f32(cases.oracle_mx(m, pos, M, K, N, tB, m.ACL_BF16), orc.BF16).astype(np.float64)
    check_close(got, want, orc.BF16, "mx", exact=use_plain is True, fp8_mfma=fast, abs_sum=abs_sum)


@pytest.mark.parametrize("exp_range,batch", [(10, 1), (11, 2), (14, 1), (4, 3)])
def test_mxfp8_exact_window(gpu, exp_range, batch):
    """The exact MXFP8 route folds a block's scale into the widening conversion as 2^(byte - base) with one base per row,
    exact while byte - base stays in [-15, 7].  Exponent ranges +-10 and +-11 (a spread of up to 22 binades inside a row)
    reach the fp16 subnormals and must still meet the stated bar; +-14 exceeds the window in some row, the bases pass flags
    it and the call runs on the scaled 8-bit instruction instead (its looser bar)."""
    m = gpu
    M, K, N = 300, 1024, 260
    print(f"case mxfp8 window exp_range={exp_range} batch={batch}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, 3 + exp_range, True, False, batch=batch, exp_range=exp_range)
    want = cases.oracle_mx(m, inp, M, K, N, True, m.ACL_BF16)
    got = cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    if exp_range <= 11:
        check_close(got, want, orc.BF16, "mxfp8 exact window")
    else:
        pos = dict(inp, x1=inp["x1"] & 0x7F, x2=inp["x2"] & 0x7F)
        abs_sum = orc.b16_to_f32(cases.oracle_mx(m, pos, M, K, N, True, m.ACL_BF16), orc.BF16).astype(np.float64)
        check_close(got, want, orc.BF16, "mxfp8 beyond the window", fp8_mfma=True, abs_sum=abs_sum)


@pytest.mark.parametrize("M,K,N,exp_range,out", [
    # up to 32 rows of x1 against a K-contiguous x2: K shared by 16 waves (4096, 8192) or by 8 (3072, 7168), ragged columns, two
    # passes; a K that one workgroup's waves do not share exactly (28 blocks: idle waves; 86, 144, 148: K segments with fp32
    # partial sums); one row and fewer than 64 x 64 outputs; scale exponents over +-30 binades (no window as on the tiles)
    (1, 4096, 512, 4, "bf16"), (16, 7168, 1000, 4, "bf16"), (9, 8192, 264, 4, "f16"), (32, 3072, 256, 4, "bf16"),
    # (the long sums with fp16 output: fp32 sums in another order than the oracle's flip one bf16 result in a thousand by an
    # ulp, which is four times the 1e-3 the bar allows)
    (16, 3584, 256, 4, "f32"), (16, 11008, 264, 4, "f16"), (20, 18432, 256, 4, "f16"), (1, 18944, 384, 4, "f16"),
    (16, 2048, 320, 30, "f32"), (12, 4096, 256, 14, "bf16"), (2, 128, 256, 4, "bf16"), (16, 384, 264, 4, "f16"),
])
def test_mxfp8_few_rows(gpu, M, K, N, exp_range, out):
    """MXFP8 with up to 32 rows: x1 in registers and x2 streamed once per 16 rows, both widened to bf16 with their block's
    scale folded in (exact), fp32 sums in the matrix instruction -- the stated bar, with the plain kernel bit-identical."""
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "f32": m.ACL_FLOAT}[out]
    print(f"case mxfp8 few rows M={M} K={K} N={N} exp_range={exp_range} out={out}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, K + N + M, True, False, exp_range=exp_range)
    bias = np.random.default_rng(1).normal(0, 1, N).astype(np.float32) if M % 2 == 0 else None
    want = cases.oracle_mx(m, inp, M, K, N, True, dt, bias)
    plain(False)
    got = cases.run_mx_aclnn(m, inp, M, K, N, True, dt, bias)
    if out == "f32":
        assert np.isfinite(got).all()
        pos = dict(inp, x1=inp["x1"] & 0x7F, x2=inp["x2"] & 0x7F)
        abs_sum = cases.oracle_mx(m, pos, M, K, N, True, dt).astype(np.float64) + (np.abs(bias) if bias is not None else 0.0)
        err = np.abs(got.astype(np.float64) - want.astype(np.float64))
        assert (err <= 2.0 ** -18 * abs_sum + 1e-30).all(), f"worst error / sum of magnitudes: {float((err / (abs_sum + 1e-30)).max()):.3e}"
    else:
        check_close(got, want, orc.BF16 if out == "bf16" else orc.F16, "mxfp8 few rows")
    plain(True)
    assert np.array_equal(cases.run_mx_aclnn(m, inp, M, K, N, True, dt, bias), want)


@pytest.mark.parametrize("M,K,N,exp_range", [
    # 17 .. 256 rows, bf16 output, K-contiguous x2: the 64- and 128-row instances, row slabs against a narrow x2 (N = 320: three
    # workgroups), a last workgroup of 32 columns, a K of whole 128-element slabs that is no whole round (1664, 11008), K
    # segments with partial sums (18432 against 256 columns), the 192- and 256-row instances against more than 128 workgroups,
    # scale exponents over +-30 binades
    (17, 2048, 256, 4), (24, 8192, 512, 4),
    (33, 1024, 256, 4), (64, 7168, 1024, 4), (100, 4096, 288, 4), (128, 1664, 512, 4), (200, 2048, 320, 4),
    (96, 11008, 512, 4), (64, 18432, 256, 4), (192, 1536, 16640, 4), (256, 1024, 16640, 4), (48, 2048, 512, 30),
    (130, 640, 16640, 4),       # (more than 128 rows per workgroup with a K that is no whole round of the 256-row instance: the tiles)
])
def test_mxfp8_many_rows(gpu, M, K, N, exp_range):
    """MXFP8 with 17 .. 256 rows: x1 widened to bf16 with its block scales into the workspace, then the many-rows streaming
    kernel on e4m3 codes with e8m0 group scales (exact products, fp32 sums) -- the stated bar; the plain kernel bit-identical."""
    m = gpu
    print(f"case mxfp8 many rows M={M} K={K} N={N} exp_range={exp_range}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, K + N + M, True, False, exp_range=exp_range)
    bias = np.random.default_rng(1).normal(0, 1, N).astype(np.float32) if M % 2 == 0 else None
    want = cases.oracle_mx(m, inp, M, K, N, True, m.ACL_BF16, bias)
    plain(False)
    got = cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16, bias)
    check_close(got, want, orc.BF16, "mxfp8 many rows")
    plain(True)
    assert np.array_equal(cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16, bias), want)


@pytest.mark.parametrize("M,K,N,tB,fp4,bias", [(256, 1024, 384, True, True, True), (300, 512, 262, True, True, False), (128, 512, 256, False, True, True),
                                               (200, 960, 264, True, True, False), (256, 1024, 384, True, False, True), (130, 256, 200, True, False, False)])
def test_mx_fp32_output(gpu, M, K, N, tB, fp4, bias):
    """FLOAT output of the MX modes on the tile kernels (fp32 sums plus bias stored straight from the registers): small
    and large tiles, ragged columns, an N-contiguous x2, a K tail of half a tile; the plain kernel is bit-identical."""
    m = gpu
    print(f"case mx fp32 out M={M} K={K} N={N} tB={tB} fp4={fp4} bias={bias}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, K + N, tB, fp4)
    b = np.random.default_rng(1).normal(0, 1, N).astype(np.float32) if bias else None
    want = cases.oracle_mx(m, inp, M, K, N, tB, m.ACL_FLOAT, b)
    got = cases.run_mx_aclnn(m, inp, M, K, N, tB, m.ACL_FLOAT, b)
    assert got.dtype == np.float32 and np.isfinite(got).all()
    pos = dict(inp, x1=inp["x1"] & (0x77 if fp4 else 0x7F), x2=inp["x2"] & (0x77 if fp4 else 0x7F))
    abs_sum = cases.oracle_mx(m, pos, M, K, N, tB, m.ACL_FLOAT).astype(np.float64)
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    # fp4 products are exact and the sums run in fp32: a few ulps of the sum of magnitudes; the 8-bit instruction aligns
    # its 128 products in a narrower window (see check_close)
    bound = (2.0 ** -20 if fp4 else 2.0 ** -14) * abs_sum + 1e-30
    assert (err <= bound).all(), f"worst error / sum of magnitudes: {float((err / (abs_sum + 1e-30)).max()):.3e}"
    plain(True)
    assert np.array_equal(cases.run_mx_aclnn(m, inp, M, K, N, tB, m.ACL_FLOAT, b), want)


@pytest.mark.parametrize("fn", [8, 9])
@pytest.mark.parametrize("M,K,N,tB,batch,bias", [
    (300, 512, 700, True, 1, True),      # one group of four K tiles, ragged rows and columns
    (512, 2048, 288, True, 1, False),    # four groups (both scale slots reused), exactly one tile at n = 9
    (260, 1536, 1000, False, 2, True),   # three groups, N-contiguous x2 (re-laid out first), batched
])
def test_mxfp8_on_the_four_wave_kernel(gpu, fn, M, K, N, tB, batch, bias):
    """MXFP8 forced onto the one-wave-per-SIMD kernel with 256 x 32n tiles, n = 8 or 9 (it is chosen by itself only for
    problems of at least 3/4 of a round of CUs with K % 512 == 0): the bar of the default MXFP8 kernel (backward-error
    bound, see check_close)."""
    m = gpu
    print(f"case mxfp8 four-wave kernel n={fn} M={M} K={K} N={N} tB={tB} batch={batch} bias={bias}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, fn + M, tB, False, batch=batch)
    b = np.random.default_rng(2).normal(0, 1, N).astype(np.float32) if bias else None
    want = cases.oracle_mx(m, inp, M, K, N, tB, m.ACL_BF16, b)
    pos = dict(inp, x1=inp["x1"] & 0x7F, x2=inp["x2"] & 0x7F)
    abs_sum = orc.b16_to_f32(cases.oracle_mx(m, pos, M, K, N, tB, m.ACL_BF16), orc.BF16).astype(np.float64)
    m.lib().opsnnSetMx8Wide(fn)
    m.lib().opsnnSetFp8Fast(1)   # the scaled 8-bit instruction is the opt-in form of MXFP8
    try:
        got = cases.run_mx_aclnn(m, inp, M, K, N, tB, m.ACL_BF16, b)
    finally:
        m.lib().opsnnSetMx8Wide(-1)
        m.lib().opsnnSetFp8Fast(0)
    check_close(got, want, orc.BF16, "mxfp8 four-wave", fp8_mfma=True, abs_sum=abs_sum)


@pytest.mark.parametrize("M,K,N,batch,bias", [
    (512, 2048, 1024, 2, True),     # 16 whole tiles in two batches
    (768, 1024, 768, 3, False),     # 27 tiles: the grouped tile order with a ragged last group of row tiles
    (256, 4096, 2048, 1, True),     # one row of tiles, a long K loop
    (1024, 1024, 512, 5, True),     # five batches of 8 tiles
])
def test_mxfp4_batched_whole_tiles(gpu, M, K, N, batch, bias):
    """Batched MXFP4 on whole 256 x 256 tiles (config 5's form at small sizes): the stated bar against the oracle, and the
    same columns bit for bit when one more column tile makes the launch ragged (another tile count and tile order)."""
    m = gpu
    print(f"case mxfp4 whole tiles M={M} K={K} N={N} batch={batch} bias={bias}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, M + batch, True, True, batch=batch)
    b = np.random.default_rng(4).normal(0, 1, N).astype(np.float32) if bias else None
    want = cases.oracle_mx(m, inp, M, K, N, True, m.ACL_BF16, b)
    got = cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16, b)
    check_close(got, want, orc.BF16, "mxfp4 whole tiles")
    # eight more columns: a ragged last column tile; the shared columns must agree bit for bit
    inp2 = cases.make_mx_inputs(m, M, K, N + 8, M + batch, True, True, batch=batch)
    inp2["x1"], inp2["s1"] = inp["x1"], inp["s1"]
    inp2["x2"][:, :N], inp2["s2"][:, :N] = inp["x2"], inp["s2"]
    b2 = np.concatenate([b, np.zeros(8, np.float32)]) if bias else None
    got2 = cases.run_mx_aclnn(m, inp2, M, K, N + 8, True, m.ACL_BF16, b2)
    assert np.array_equal(got2[:, :, :N], got), "whole-tile and ragged launches differ on shared columns"


@pytest.mark.parametrize("M,K,N,batch", [(96, 256, 128, 3), (256, 1024, 264, 2)])
def test_mx_batched(gpu, M, K, N, batch):
    m = gpu
    inp = cases.make_mx_inputs(m, M, K, N, 4, True, True, batch=batch)
    want = cases.oracle_mx(m, inp, M, K, N, True, m.ACL_BF16)
    got = cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    check_close(got, want, orc.BF16, "mx batched")


@pytest.mark.parametrize("use_plain", [True, False])
@pytest.mark.parametrize("M,K,N,x_dt,w_dt,group,tW,off,bias", [
    (16, 512, 256, "bf16", "i8", 0, False, False, None),      # config 1 shape class
    (16, 512, 256, "bf16", "i8", 0, True, True, "f32"),
    (1, 1024, 512, "f16", "i4", 128, False, True, None),       # config 3 shape class
    (16, 1024, 512, "f16", "i4", 128, True, True, "f16"),
    (64, 512, 384, "f16", "i4", 128, True, True, None),
    (256, 512, 256, "f16", "i4", 128, False, True, None),
    (7, 320, 130, "bf16", "i4", 64, False, True, "bf16"),
    (5, 256, 64, "f16", "i8", 32, True, False, None),
    (33, 864, 212, "f16", "i4", 96, False, True, None),         # ragged groups (864 = 9 * 96)
    (4, 256, 128, "bf16", "e4m3", 0, True, False, "bf16"),
    (33, 384, 130, "f16", "e4m3", 0, False, False, "f16"),     # fp8 weights, N-contiguous, fp16 (weight, scale and product rounded through fp16)
    # mxfp4 weights with e8m0 scales per 32 K (_compute_mx): the reference's own case a16mxf4_nd_weight_fp4 (2 x 64 x 128,
    # fp16, [K, N] storage), a decode shape in both layouts and both activation types, an odd number of 32-blocks, a bias
    (2, 64, 128, "f16", "fp4", 32, False, False, None),
    (1, 4096, 512, "f16", "fp4", 32, True, False, None),
    (1, 4096, 512, "bf16", "fp4", 32, False, False, None),
    (16, 1024, 384, "bf16", "fp4", 32, True, False, "bf16"),
    (5, 96, 66, "f16", "fp4", 32, False, False, "f16"),
    (40, 2048, 256, "f16", "fp4", 32, True, False, None),
    # ... on the matrix cores these take the general decode kernel: a K split between waves (narrow N, K >= 2048), several
    # row slabs, e4m3 weights (per channel: the only form the API admits)
    (16, 4096, 1024, "bf16", "fp4", 32, True, False, None),
    (130, 2048, 512, "f16", "fp4", 32, True, False, "f16"),
    (100, 2048, 512, "bf16", "e4m3", 0, True, False, None),
    (16, 4096, 320, "f16", "e4m3", 0, True, False, None),
    # shapes the streamlined decode kernel takes: vector scale loads (group 128 int4, K/128 a multiple of 8) ...
    (1, 2048, 528, "f16", "i4", 128, True, True, None),
    (16, 3072, 272, "f16", "i4", 128, True, False, "f16"),
    (32, 1024, 260, "f16", "i4", 128, True, True, None),
    (64, 2048, 256, "f16", "i4", 128, True, True, "f16"),
    (48, 1024, 256, "bf16", "i4", 128, True, True, None),
    (16, 1024, 256, "f16", "i8", 64, True, True, None),
    # ... scalar scale loads: wider groups, ragged chunk counts, N-contiguous weight, per-channel
    (3, 1280, 144, "f16", "i4", 256, True, True, None),
    (20, 1280, 144, "f16", "i4", 256, False, False, None),
    (16, 1152, 8208, "f16", "i4", 128, True, True, None),       # 9 groups: not a multiple of 8; 513 row blocks
    (9, 640, 96, "bf16", "i8", 128, True, True, "bf16"),
    (64, 1024, 320, "bf16", "i8", 0, True, False, None),
    # ... x whole in LDS with more row blocks than workgroups (513 on 512) and a row block that is no whole number of
    # eight-chunk super-steps (4, 3 and 4 chunks per wave): the refills that run into the next row block
    (3, 2048, 8208, "f16", "i4", 128, True, True, None),
    (16, 1536, 8240, "bf16", "i4", 0, True, False, "bf16"),
    (9, 1024, 8208, "f16", "i8", 64, True, True, None),
    # ... K split between the waves of a workgroup (narrow N, M <= 16)
    (16, 4096, 256, "bf16", "i8", 0, True, False, None),
    (1, 4096, 200, "f16", "i4", 128, True, True, "f16"),
    (11, 2048, 64, "f16", "i8", 0, False, True, None),
    # ... many rows (several weight blocks per wave share each x fragment): 49..64 rows, 65..128, and two passes
    (50, 2048, 288, "bf16", "i4", 128, True, False, "bf16"),   # 49..64 rows: the 64-row instance, ragged row count
    (64, 1024, 256, "f16", "i8", 64, True, True, None),
    (100, 2048, 512, "f16", "i4", 128, True, True, None),
    (128, 1024, 256, "f16", "i8", 64, True, True, "f16"),
    (200, 2048, 320, "bf16", "i4", 256, True, True, None),
    (256, 1024, 256, "f16", "i4", 128, True, False, "f16"),
    (130, 1024, 256, "bf16", "i8", 0, False, False, "bf16"),
    # ... more than 256 rows: the dequantise-once tile kernel in passes of equal slabs (three of 208 rows, the last ragged;
    # two of 144), and the streaming kernel's slabs where the tile kernel does not apply (a group of 32)
    (600, 1024, 384, "f16", "i4", 128, True, True, "f16"),
    (280, 512, 256, "bf16", "i8", 0, True, False, None),
    (300, 1024, 256, "f16", "i4", 32, True, True, None),
])
def test_weight_only(gpu, M, K, N, x_dt, w_dt, group, tW, off, bias, use_plain):
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "f32": m.ACL_FLOAT, "i8": m.ACL_INT8, "i4": m.ACL_INT4,
          "e4m3": m.ACL_FLOAT8_E4M3FN, "fp4": m.ACL_FLOAT4_E2M1, None: None}
    print(f"case wq M={M} K={K} N={N} x={x_dt} w={w_dt} g={group} tW={tW} off={off} bias={bias} plain={use_plain}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M * 7 + N, dt[x_dt], dt[w_dt], group, tW, off, dt[bias])
    want = cases.oracle_wq(m, inp, M, K, N)
    plain(use_plain)
    got = cases.run_wq_aclnn(m, inp, M, K, N)
    check_close(got, want, dt[x_dt], "weight-only", exact=use_plain)


@pytest.mark.parametrize("M,K,N,x_dt,w_dt,group,tW,off,bias", [
    # 64-, 128- and 256-row instances; int4 (two K steps per weight copy) and int8 (one); groups of 64, 128, 256 and
    # per channel; ragged rows and columns; a single K step; N-contiguous weight (re-laid out first); bias
    (64, 512, 384, "f16", "i4", 128, True, True, None),
    (50, 2048, 288, "bf16", "i4", 128, True, False, "bf16"),
    (64, 1024, 256, "f16", "i8", 64, True, True, None),
    (60, 256, 100, "bf16", "i4", 64, True, True, None),
    (64, 128, 128, "f16", "i4", 0, True, False, None),
    (64, 64, 128, "f16", "i8", 0, True, True, None),
    (1, 1024, 256, "f16", "i4", 128, True, True, None),
    (100, 2048, 512, "f16", "i4", 128, True, True, None),
    (128, 1024, 256, "f16", "i8", 64, True, True, "f16"),
    (77, 192, 130, "f16", "i8", 64, True, True, None),
    (130, 1024, 256, "bf16", "i8", 0, False, False, "bf16"),
    (200, 2048, 320, "bf16", "i4", 256, True, True, None),
    (256, 1024, 256, "f16", "i4", 128, True, False, "f16"),
    (256, 512, 256, "f16", "i4", 128, False, True, None),
    (129, 1152, 200, "bf16", "i4", 384, True, True, None),      # three groups of 384 = 6 steps each
    (256, 320, 136, "f16", "i8", 0, True, False, None),         # five steps (odd count)
])
def test_weight_only_tile_kernel(gpu, M, K, N, x_dt, w_dt, group, tW, off, bias):
    """The dequantise-once tile kernel, which by itself takes 129 .. 256 rows of x, forced onto every row count it has an
    instance for (opsnnSetWqTileMin(1)); the bar of the other matrix-instruction kernels."""
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "i8": m.ACL_INT8, "i4": m.ACL_INT4, None: None}
    print(f"case wq tile kernel M={M} K={K} N={N} x={x_dt} w={w_dt} g={group} tW={tW} off={off} bias={bias}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M * 5 + N, dt[x_dt], dt[w_dt], group, tW, off, dt[bias])
    want = cases.oracle_wq(m, inp, M, K, N)
    plain(False)
    m.lib().opsnnSetWqTileMin(1)
    try:
        got = cases.run_wq_aclnn(m, inp, M, K, N)
    finally:
        m.lib().opsnnSetWqTileMin(129)
    check_close(got, want, dt[x_dt], "weight-only tile kernel")



@pytest.mark.parametrize("M,K,N,x_dt,w_dt,group,tW,off,bias", [
    # 129 .. 256 rows on the 256-row instance of the many-rows kernel (a weight row's scales contiguous, a power-of-two
    # group count, K a multiple of two chunk pairs, N % 32 == 0): int4 with half-chunk x slabs, int8 with whole ones;
    # ragged row counts (the slab's missing rows repeat the last one), ragged last column block, per-channel scales, bias
    (256, 2048, 512, "f16", "i4", 128, True, True, None),
    (200, 4096, 288, "f16", "i4", 128, True, False, "f16"),
    (129, 1024, 256, "bf16", "i4", 256, True, True, None),
    (256, 1024, 320, "bf16", "i4", 0, True, False, "bf16"),
    (256, 1024, 512, "f16", "i8", 128, True, True, None),
    (177, 2048, 256, "bf16", "i8", 0, True, False, None),
    (193, 2048, 256, "f16", "i4", 128, True, True, "f16"),     # one row more than the 192-row instance takes
    (192, 1024, 288, "f16", "i8", 128, True, True, None),
    # more than 256 rows: whole passes of 256, then the rest on the instance that fits it (44, 8 and 200 rows here)
    (300, 1024, 256, "f16", "i4", 128, True, True, None),
    (520, 1024, 288, "bf16", "i4", 128, True, False, "bf16"),
    (712, 1024, 256, "f16", "i8", 128, True, True, None),
])
def test_weight_only_256_row_instance(gpu, M, K, N, x_dt, w_dt, group, tW, off, bias):
    """From 129 rows of x: passes of up to 256 rows on the many-rows kernel's 256-row instance (the default route for these
    row counts; the tile kernel takes what it declines): the bar of the other matrix-instruction kernels, and the same call
    on the tile kernel (opsnnSetWqTileMin(1)) within the same bar of the oracle."""
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "i8": m.ACL_INT8, "i4": m.ACL_INT4, None: None}
    print(f"case wq 256-row instance M={M} K={K} N={N} x={x_dt} w={w_dt} g={group} tW={tW} off={off} bias={bias}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M * 7 + N, dt[x_dt], dt[w_dt], group, tW, off, dt[bias])
    want = cases.oracle_wq(m, inp, M, K, N)
    plain(False)
    # these weights are narrow: by default the rows go out as equal slabs of 64 .. 256 rows in one launch; with the hook the
    # call runs one pass of up to 256 rows per launch, as against a wide weight -- the instance this test is about
    narrow = cases.run_wq_aclnn(m, inp, M, K, N)
    check_close(narrow, want, dt[x_dt], "weight-only, row slabs in one launch")
    m.lib().opsnnSetWqNarrowSlabs(0)
    try:
        got = cases.run_wq_aclnn(m, inp, M, K, N)
    finally:
        m.lib().opsnnSetWqNarrowSlabs(1)
    check_close(got, want, dt[x_dt], "weight-only 256-row instance")
    m.lib().opsnnSetWqTileMin(1)
    try:
        tile = cases.run_wq_aclnn(m, inp, M, K, N)
    finally:
        m.lib().opsnnSetWqTileMin(129)
    check_close(tile, want, dt[x_dt], "weight-only tile kernel")


@pytest.mark.parametrize("M,K,N,x_dt,w_dt,group,off,bias", [
    # up to 64 rows per slab against a narrow weight, K in whole groups of 16 chunks (int4 / mxfp4: K % 2048 == 0, int8 / e4m3:
    # K % 1024 == 0): workgroups of 64 columns with K split over four waves; ragged last workgroup, scale table in LDS and
    # per-lane scales, per-channel scales, four slabs of 64 rows in one launch
    (64, 2048, 288, "f16", "i4", 128, True, None),
    (49, 4096, 256, "bf16", "i4", 0, False, "bf16"),
    (50, 1024, 320, "f16", "i8", 128, True, None),
    (64, 3072, 256, "bf16", "i8", 64, True, None),          # 48 groups per row: table rows of 64 words
    (64, 2048, 256, "bf16", "fp4", 32, False, None),
    (33, 6144, 288, "f16", "fp4", 32, False, "f16"),        # K / 128 = 48: table rows of 64 words
    (33, 1024, 288, "f16", "e4m3", 0, False, None),
    (200, 2048, 512, "f16", "i4", 128, True, "f16"),
    (130, 1024, 256, "bf16", "e4m3", 0, False, None),
    # K in whole x slabs (two chunks on 128-column workgroups, four on 64-column ones) but no whole rounds of the chunk
    # pipeline: a shorter last round behind the loop, on the 64- and 128-row instances; the 192- / 256-row ones decline
    (64, 1280, 256, "f16", "i4", 128, True, None),            # five slabs on 128-column workgroups
    (64, 2816, 256, "f16", "i4", 512, True, None),            # ... and a short last group (5.5 groups): six table entries per row
    (100, 3072, 288, "bf16", "i4", 2048, True, "bf16"),       # one and a half groups
    (64, 1408, 256, "bf16", "i8", 256, True, None),
    (64, 1536, 288, "bf16", "i4", 128, False, "bf16"),        # three slabs on 64-column workgroups, six on 128-column ones
    (128, 3584, 256, "f16", "i4", 128, True, None),           # seven / fourteen slabs; one pass: the 128-row instance
    (100, 640, 320, "bf16", "i8", 64, True, None),
    (40, 768, 256, "f16", "i8", 0, False, "f16"),
    (33, 2560, 288, "f16", "fp4", 32, False, None),
    (120, 896, 256, "bf16", "e4m3", 0, False, None),
    (256, 1536, 256, "f16", "i4", 128, True, None),           # one pass: whole rounds of the 256-row instance (512 k)
    (256, 1280, 256, "f16", "i4", 128, True, None),           # one pass: no whole rounds there, the tile kernel
])
def test_weight_only_64_column_workgroups(gpu, M, K, N, x_dt, w_dt, group, off, bias):
    """The many-rows kernel's instance whose workgroups take 64 columns (chosen when 128-column ones would number at most 128)
    against the oracle, and the same call on the 128-column instances (opsnnSetWqNarrowSlabs(0))."""
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "i8": m.ACL_INT8, "i4": m.ACL_INT4, "e4m3": m.ACL_FLOAT8_E4M3FN,
          "fp4": m.ACL_FLOAT4_E2M1, None: None}
    print(f"case wq 64-column workgroups M={M} K={K} N={N} x={x_dt} w={w_dt} g={group} off={off} bias={bias}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M * 5 + N, dt[x_dt], dt[w_dt], group, True, off, dt[bias])
    want = cases.oracle_wq(m, inp, M, K, N)
    plain(False)
    got = cases.run_wq_aclnn(m, inp, M, K, N)
    check_close(got, want, dt[x_dt], "weight-only, 64-column workgroups")
    m.lib().opsnnSetWqNarrowSlabs(0)
    try:
        wide = cases.run_wq_aclnn(m, inp, M, K, N)
    finally:
        m.lib().opsnnSetWqNarrowSlabs(1)
    check_close(wide, want, dt[x_dt], "weight-only, 128-column workgroups")


@pytest.mark.parametrize("M,K,N,x_dt,w_dt,group,off,bias", [
    # from 17 rows against a narrow N and a K of 8192 or more: K in 2 .. 8 segments over blockIdx.z (whole
    # rounds of eight chunks -- 1024 k of int4, 512 of int8 --, as equal as that allows, at least 2048 k), partial sums added
    # by a second kernel; one row slab and several, ragged last workgroup, ragged last slab, unequal segments, group counts
    # per segment that are no power of two, per-channel scales
    (64, 8192, 256, "f16", "i4", 128, True, None),            # four segments
    (49, 8192, 288, "bf16", "i4", 0, False, "bf16"),          # per-channel scale, a last workgroup of 32 columns
    (100, 8192, 256, "f16", "i8", 128, True, None),           # two slabs of 64 rows (the second with 36)
    (64, 10240, 256, "bf16", "i8", 64, True, None),           # five segments of four rounds
    (64, 14336, 256, "f16", "i4", 128, False, "f16"),         # seven segments
    (64, 11264, 256, "f16", "i4", 512, True, None),           # eleven rounds in five segments (3, 2, 2, 2, 2): six groups or four
    (200, 8192, 512, "f16", "i4", 128, True, "f16"),          # four slabs
    (300, 12288, 256, "bf16", "i4", 256, True, None),         # five slabs, six segments
    (64, 16384, 1024, "f16", "i4", 128, True, None),          # eight workgroups: eight segments
    (64, 32768, 256, "f16", "i4", 128, True, None),           # (in one piece: 256 groups per row, too many for the scale table)
    # K below 8192 where the 64-column workgroups cannot run (K no multiple of four chunks), from 33 rows
    (64, 4864, 256, "f16", "i4", 128, True, None),            # 19 x slabs in two segments (10, 9)
    (40, 6400, 288, "bf16", "i4", 256, False, "bf16"),        # 25 in three
    (128, 7424, 1024, "f16", "i4", 128, True, None),          # two row slabs, 29 in three
    # segments that are no whole rounds of the chunk pipeline
    (64, 11008, 256, "f16", "i4", 128, True, None),           # 43 x slabs in five segments (9, 9, 9, 8, 8)
    (64, 9472, 256, "bf16", "i8", 0, False, None),            # 74 in four (19, 19, 18, 18)
    (48, 8448, 256, "f16", "fp4", 32, False, None),           # 33 in four
    # 17 .. 48 rows of integer codes (in one piece the first of them runs on the streaming kernel)
    (17, 8192, 256, "bf16", "i4", 128, True, None),
    (33, 10240, 288, "f16", "i8", 0, False, "f16"),
    (48, 8192, 1024, "f16", "i4", 64, True, None),
    # floating-point codes
    (17, 8192, 256, "f16", "fp4", 32, False, None),
    (64, 14336, 288, "bf16", "fp4", 32, False, "bf16"),       # seven segments, a last workgroup of 32 columns
    (40, 11264, 256, "f16", "e4m3", 0, False, None),          # 22 rounds of 512 in five segments (5, 5, 4, 4, 4)
    (150, 8192, 256, "bf16", "fp4", 32, False, None),         # three row slabs
    (100, 9216, 512, "f16", "e4m3", 0, False, "f16"),         # two row slabs, 18 rounds in four segments
])
def test_weight_only_rows_k_segments(gpu, M, K, N, x_dt, w_dt, group, off, bias):
    """The many-rows kernel with K split over workgroups against the oracle, the same call without the split
    (opsnnSetWqNarrowSlabs(0)), and two runs of the split call bit for bit (the segments are added in a fixed order)."""
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "i8": m.ACL_INT8, "i4": m.ACL_INT4, "e4m3": m.ACL_FLOAT8_E4M3FN,
          "fp4": m.ACL_FLOAT4_E2M1, None: None}
    print(f"case wq rows K segments M={M} K={K} N={N} x={x_dt} w={w_dt} g={group} off={off} bias={bias}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M * 3 + N, dt[x_dt], dt[w_dt], group, True, off, dt[bias])
    want = cases.oracle_wq(m, inp, M, K, N)
    plain(False)
    got = cases.run_wq_aclnn(m, inp, M, K, N)
    check_close(got, want, dt[x_dt], "weight-only, K segments")
    assert np.array_equal(cases.run_wq_aclnn(m, inp, M, K, N), got), "two runs of the same call differ"
    m.lib().opsnnSetWqNarrowSlabs(0)
    try:
        whole = cases.run_wq_aclnn(m, inp, M, K, N)
    finally:
        m.lib().opsnnSetWqNarrowSlabs(1)
    check_close(whole, want, dt[x_dt], "weight-only, K in one piece")


@pytest.mark.parametrize("M,K,N,x_dt,w_dt,group,tW,off,bias", [
    # 4 .. 16 rows with K a multiple of 8 waves x 4, 8 or 16 chunks (int4: 4096, 8192; int8: 2048, 4096, 8192): groups of one
    # chunk (vector scale loads), of several chunks and per channel; with and without offset; ragged columns; fewer row
    # blocks than workgroups and more (a workgroup walks several); N-contiguous weight; bias
    (16, 8192, 256, "f16", "i4", 128, True, True, None),
    (16, 8192, 4400, "f16", "i4", 128, True, False, "f16"),    # 275 row blocks: some workgroups take two
    (5, 8192, 100, "bf16", "i4", 128, True, True, None),
    (4, 4096, 1000, "f16", "i4", 256, True, True, None),
    (9, 4096, 64, "bf16", "i4", 0, True, False, "bf16"),
    (16, 8192, 128, "f16", "i4", 1024, True, True, None),
    (16, 4096, 4096, "bf16", "i8", 0, True, False, None),
    (12, 2048, 72, "f16", "i8", 64, True, True, None),
    (16, 8192, 200, "f16", "i8", 64, True, True, "f16"),
    (7, 4096, 320, "bf16", "i8", 128, True, True, None),
    (16, 8192, 96, "bf16", "i4", 128, False, True, None),
    # floating-point weight codes (1 .. 16 rows): mxfp4 (e2m1 with one e8m0 byte per 32 K, a row's bytes contiguous) on 16 and
    # on 8 waves, both activation types; e4m3 with per-channel scales on 16 waves x 8 chunks, 16 x 4 and 8 x 4
    (16, 8192, 256, "f16", "fp4", 32, True, False, None),
    (5, 8192, 1000, "bf16", "fp4", 32, True, False, "bf16"),
    (1, 4096, 130, "bf16", "fp4", 32, True, False, None),
    (16, 4096, 4400, "f16", "fp4", 32, True, False, "f16"),
    (16, 8192, 96, "bf16", "e4m3", 0, True, False, None),
    (12, 4096, 200, "bf16", "e4m3", 0, True, False, "bf16"),
    (7, 2048, 72, "f16", "e4m3", 0, True, False, None),
    # a K of several workgroup segments (2 .. 16 of 16 x 4 chunks, else of 8 x 4): one workgroup column per segment, fp32
    # partial sums in front of the workspace (behind them the re-laid-out weight of the N-contiguous case), a reduce kernel;
    # one row (x does not fit the LDS of the few-rows kernel at this K)
    (16, 16384, 256, "f16", "i4", 128, True, True, None),
    (5, 12288, 100, "bf16", "i4", 128, True, True, "bf16"),
    (1, 28672, 264, "f16", "i4", 128, True, True, None),
    (8, 12288, 64, "f16", "i4", 128, False, True, None),
    (16, 6144, 200, "f16", "i8", 64, True, True, "f16"),
    (9, 16384, 64, "bf16", "i8", 0, True, False, None),
    (16, 16384, 256, "f16", "fp4", 32, True, False, None),
    (12, 6144, 200, "bf16", "e4m3", 0, True, False, "bf16"),
    # a K that is no whole number of segments (integer codes): the last segment's waves past the end of K stay idle --
    # 14336 = 2 x 8192 - 2048, 11008 = 3 x 4096 - 1280, 28672 = 4 x 8192 - 4096, 7168 = 8192 - 1024 in one workgroup;
    # int8: 7168 = 2 x 4096 - 1024; the last weight row's reads stay inside the row (N = 16: one row block)
    (16, 14336, 256, "f16", "i4", 128, True, True, None),
    (7, 11008, 100, "bf16", "i4", 128, True, False, "bf16"),
    (16, 28672, 64, "f16", "i4", 128, True, True, None),
    (16, 7168, 16, "f16", "i4", 128, True, True, "f16"),
    (16, 7168, 200, "bf16", "i8", 128, True, True, None),
    (4, 14336, 48, "f16", "i4", 0, True, False, None),
    (2, 14336, 72, "f16", "i4", 256, False, True, None),
    (16, 18432, 256, "f16", "i4", 128, True, True, None),      # 144 chunks in five segments of 32, vector scale loads
    (16, 13824, 256, "f16", "i4", 128, True, True, None),      # 108 chunks in four segments of 32: 20 idle, the most the plan takes
    (6, 13824, 264, "bf16", "fp4", 32, True, False, None),
    # ... floating-point codes: mxfp4 7168 = 8192 - 1024 in one workgroup, 18432 in five segments (a row's e8m0 bytes a whole
    # number of 16-byte pieces); e4m3 7168 = 4 x 2048 - 1024
    (16, 7168, 512, "f16", "fp4", 32, True, False, None),
    (9, 18432, 256, "bf16", "fp4", 32, True, False, "bf16"),
    (12, 7168, 200, "bf16", "e4m3", 0, True, False, None),
])
def test_weight_only_x_in_registers_kernel(gpu, M, K, N, x_dt, w_dt, group, tW, off, bias):
    """4 .. 16 rows of x (floating-point weight codes: 1 .. 16) with K in 8 or 16 equal ranges of whole chunks: the kernel
    that keeps x in registers."""
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "i8": m.ACL_INT8, "i4": m.ACL_INT4, "e4m3": m.ACL_FLOAT8_E4M3FN,
          "fp4": m.ACL_FLOAT4_E2M1, None: None}
    print(f"case wq x-in-registers M={M} K={K} N={N} x={x_dt} w={w_dt} g={group} tW={tW} off={off} bias={bias}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M * 3 + N, dt[x_dt], dt[w_dt], group, tW, off, dt[bias])
    want = cases.oracle_wq(m, inp, M, K, N)
    plain(False)
    got = cases.run_wq_aclnn(m, inp, M, K, N)
    check_close(got, want, dt[x_dt], "weight-only, x in registers")


@pytest.mark.parametrize("M,K,N,x_dt,w_dt,group,bias", [
    # mxfp4 (K % 1024 == 0, N % 32 == 0, N >= 256; 17 rows and more): up to 64 rows, up to 128 rows (the 8-block form), two passes of equal
    # slabs, ragged last row block of x, both activation types, a bias
    (17, 1024, 256, "bf16", "fp4", 32, None),
    (40, 2048, 256, "f16", "fp4", 32, None),
    (64, 8192, 512, "bf16", "fp4", 32, "bf16"),
    (100, 4096, 288, "f16", "fp4", 32, "f16"),
    (128, 1024, 1024, "bf16", "fp4", 32, None),
    (200, 2048, 320, "f16", "fp4", 32, None),
    # e4m3 with per-channel scales (K % 512 == 0)
    (48, 512, 256, "bf16", "e4m3", 0, None),
    (96, 4096, 544, "f16", "e4m3", 0, "f16"),
    (130, 1536, 256, "bf16", "e4m3", 0, "bf16"),
    # 129 rows and more: the 192- and 256-row instances (8-byte pieces of e2m1 codes: two lanes share an e8m0 byte), whole
    # passes of 256 rows and the rest on the instance that fits it (44, 8 and 200 rows)
    (129, 2048, 256, "bf16", "fp4", 32, None),
    (192, 1024, 288, "f16", "fp4", 32, "f16"),
    (193, 4096, 256, "f16", "fp4", 32, None),
    (256, 8192, 512, "bf16", "fp4", 32, "bf16"),
    (300, 1024, 256, "f16", "fp4", 32, None),
    (712, 2048, 320, "bf16", "fp4", 32, None),
    # K / 128 not a power of two: the scale table's rows are padded to one
    (100, 3072, 256, "bf16", "fp4", 32, None),
    (256, 3072, 288, "f16", "fp4", 32, "f16"),
    (180, 5120, 256, "bf16", "fp4", 32, None),
    # a K whose scale table does not fit beside the x buffers: a lane's e8m0 byte travels with its weight piece (8-byte
    # pieces at 129+ rows: two lanes share a byte)
    (100, 32768, 256, "bf16", "fp4", 32, None),
    (256, 12288, 288, "f16", "fp4", 32, "f16"),
    (160, 512, 256, "f16", "e4m3", 0, None),
    (250, 4096, 544, "bf16", "e4m3", 0, "bf16"),
    (256, 1024, 256, "f16", "e4m3", 0, "f16"),
    (520, 1536, 288, "bf16", "e4m3", 0, None),
])
def test_weight_only_float_codes_on_the_many_rows_kernel(gpu, M, K, N, x_dt, w_dt, group, bias):
    """17 rows of x and more against mxfp4 / e4m3 weights: the many-rows streaming kernel (two weight blocks per wave
    share every x fragment; a lane's 32 e2m1 codes of a chunk are one MX group, so its e8m0 byte travels with them)."""
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "e4m3": m.ACL_FLOAT8_E4M3FN, "fp4": m.ACL_FLOAT4_E2M1, None: None}
    print(f"case wq float codes, many rows M={M} K={K} N={N} x={x_dt} w={w_dt} g={group} bias={bias}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M * 3 + N, dt[x_dt], dt[w_dt], group, True, False, dt[bias])
    want = cases.oracle_wq(m, inp, M, K, N)
    plain(False)
    narrow = cases.run_wq_aclnn(m, inp, M, K, N)   # (narrow weights: from 65 rows equal row slabs in one launch)
    check_close(narrow, want, dt[x_dt], "weight-only float codes, row slabs in one launch")
    m.lib().opsnnSetWqNarrowSlabs(0)
    try:
        got = cases.run_wq_aclnn(m, inp, M, K, N)      # one pass of up to 256 rows per launch: the 64- .. 256-row instances
    finally:
        m.lib().opsnnSetWqNarrowSlabs(1)
    check_close(got, want, dt[x_dt], "weight-only float codes, many rows")


@pytest.mark.parametrize("M,K,N,x_dt,w_dt,tW,off,bias", [
    (16, 4096, 256, "f16", "i8", True, True, None),        # one scale and offset for the whole tensor, 16 waves x 4 chunks
    (9, 8192, 100, "f16", "i4", True, True, "f16"),        # ragged columns, per tensor, a bias
    (6, 2048, 72, "bf16", "i8", True, True, "f32"),        # fp32 bias (bf16 activations only), 8 waves x 4 chunks
    (4, 4096, 48, "bf16", "i8", False, False, "bf16"),     # N-contiguous weight (re-laid out first), three row blocks
])
def test_weight_only_x_in_registers_per_tensor_scale_and_fp32_bias(gpu, M, K, N, x_dt, w_dt, tW, off, bias):
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "f32": m.ACL_FLOAT, "i8": m.ACL_INT8, "i4": m.ACL_INT4, None: None}
    print(f"case wq x-in-registers per-tensor M={M} K={K} N={N} x={x_dt} w={w_dt} tW={tW} off={off} bias={bias}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M + N, dt[x_dt], dt[w_dt], 0, tW, off, dt[bias], per_tensor=True)
    want = cases.oracle_wq(m, inp, M, K, N)
    plain(False)
    got = cases.run_wq_aclnn(m, inp, M, K, N)
    check_close(got, want, dt[x_dt], "weight-only, x in registers, per tensor")


def test_weight_only_v3_and_per_tensor(gpu):
    m = gpu
    inp = cases.make_wq_inputs(m, 8, 256, 128, 2, m.ACL_FLOAT16, m.ACL_INT8, 0, False, True, None, per_tensor=True)
    want = cases.oracle_wq(m, inp, 8, 256, 128)
    got = cases.run_wq_aclnn(m, inp, 8, 256, 128, v3=True)
    check_close(got, want, orc.F16, "per-tensor V3")
