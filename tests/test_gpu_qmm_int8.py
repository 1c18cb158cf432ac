"""GPU parity: int8 x int8 per-token / per-channel quantized matmul (aclnnQuantMatmulV5, K-C / K-T / T-C).

Bar: bit-exact.  The int32 accumulators are exact in any order, and the epilogue is a fixed sequence of
separately rounded fp32 operations followed by one round-to-nearest-even cast, so the 16-bit outputs of the
HIP kernels must equal the oracle's bit for bit (qbmmv3_kernel_golden.py:361-387).
"""
import ctypes as C

import numpy as np
import pytest

import cases
import oracle_api as orc

pytestmark = pytest.mark.gpu


def _check_equal(got, want, what):
    if not np.array_equal(got, want):
        bad = np.argwhere(got != want)
        raise AssertionError(f"{what}: {len(bad)} of {got.size} elements differ; first at {bad[0]}: "
                             f"got {got[tuple(bad[0])]:#x} want {want[tuple(bad[0])]:#x}")


@pytest.mark.parametrize("M,K,N,tB", [
    (128, 256, 512, True),     # the reference's ST shape v3_kc_int8_fp32
    (256, 512, 384, True),
    (256, 512, 384, False),    # N-contiguous x2: re-laid out into the workspace first
    (197, 960, 854, True),     # ragged M and N, K multiple of 16
    (33, 77, 19, True),        # odd everything: plain kernel
    (1, 4096, 128, True),      # M = 1
    (300, 128, 260, False),
    # few 128 x 128 tiles against a long K: K split over 2 .. 16 workgroups per tile, int32 partial sums in the workspace
    # (behind them the re-laid-out x2 of the N-contiguous case), summed exactly: still bit-identical
    (64, 4096, 512, True),
    (200, 8192, 1000, False),
    (16, 8192, 264, True),
    (130, 4096, 130, True),    # a column count that is no multiple of 4
    # fewer than 64 x 64 outputs against a long K (one decode row against a narrow weight): the tile kernel with K split
    (1, 18944, 3584, True),
    (3, 3584, 1000, True),
])
@pytest.mark.parametrize("out_dt,bias_dt", [("bf16", "bf16"), ("bf16", None), ("f16", "f32"), ("bf16", "i32"), ("f16", "f16")])
def test_kc_matches_oracle(gpu, M, K, N, tB, out_dt, bias_dt):
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "f32": m.ACL_FLOAT, "i32": m.ACL_INT32, None: None}
    print(f"case int8 K-C M={M} K={K} N={N} tB={tB} out={out_dt} bias={bias_dt}", flush=True)
    got, want, _ = cases.run_qmm_int8_case(m, orc, M, K, N, seed=M * 31 + N, out_dtype=dt[out_dt], bias_dtype=dt[bias_dt],
                                           transpose_x2=tB)
    _check_equal(got, want, "aclnnQuantMatmulV5 K-C")


def test_kt_and_bf16_scale(gpu):
    """K-T (one x2 scale) and a bf16 per-channel scale."""
    m = gpu
    for s2_len, s2_dt in [(1, m.ACL_FLOAT), (None, m.ACL_BF16)]:
        print(f"case int8 x2s_len={s2_len} dtype={s2_dt}", flush=True)
        got, want, _ = cases.run_qmm_int8_case(m, orc, 160, 320, 272, seed=5, out_dtype=m.ACL_BF16, bias_dtype=m.ACL_BF16,
                                               transpose_x2=True, x2s_len=s2_len, x2s_dtype=s2_dt)
        _check_equal(got, want, "K-T / bf16 scale")


def test_transposed_view_equals_flag(gpu):
    """x2 given as a strided (1, K) view with transposeX2 = false must equal transposeX2 = true on [N, K]."""
    m = gpu
    M, K, N = 128, 256, 192
    inp = cases.make_qmm_int8_inputs(m, M, K, N, 3, m.ACL_BF16, True)
    a = cases.run_qmm_int8_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    b = cases.run_qmm_int8_aclnn(m, inp, M, K, N, True, m.ACL_BF16, x2_as_view=True)
    want, _ = cases.oracle_qmm_int8(m, inp, M, K, N, True, m.ACL_BF16)
    _check_equal(a, want, "flag form")
    _check_equal(b, want, "view form")


def test_batched(gpu):
    m = gpu
    print("case int8 batched", flush=True)
    got, want, _ = cases.run_qmm_int8_case(m, orc, 130, 256, 140, seed=9, out_dtype=m.ACL_BF16, bias_dtype=m.ACL_FLOAT,
                                           transpose_x2=True, batch=3)
    _check_equal(got, want, "batched K-C")
    print("case int8 batched, K split", flush=True)
    got, want, _ = cases.run_qmm_int8_case(m, orc, 130, 4096, 140, seed=10, out_dtype=m.ACL_F16 if hasattr(m, "ACL_F16") else m.ACL_FLOAT16,
                                           bias_dtype=m.ACL_INT32, transpose_x2=True, batch=3)
    _check_equal(got, want, "batched K-C with a K split")


@pytest.mark.parametrize("variant", [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11])
def test_every_kernel_variant_and_int32_accumulators(gpu, variant):
    """Each kernel variant (1 plain, 2 MFMA 256x256, 3 MFMA 128x128,
    4 MFMA 256x128 three-stage, 5-7 MFMA 256x256 eight-wave, 8-11 four-wave tiles of 256 x 32n columns) through the
    thin launcher ABI.
    With unit scales and no bias the fp32 epilogue is the identity on |acc| < 2^24, which exposes the raw
    int32 accumulators: K = 512 keeps |acc| <= 512*127*127 < 2^24."""
    m = gpu
    M, K, N = 384, 512, 640
    rng = np.random.default_rng(variant)
    inp = dict(x1=cases.gen_int8(rng, (1, M, K)), x2=cases.gen_int8(rng, (1, N, K)), s1=np.ones(M, np.float32),
               s2=np.ones(N, np.float32))
    acc = orc.qmm_int8_acc(inp["x1"][0], inp["x2"][0], M, K, N, False, True)
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items()}
    out = m.DeviceBuffer(M * N * 2)
    a = cases.qmm_args_int8(m, d, M, K, N, 1, True, out.ptr, m.ACL_FLOAT16, m.ACL_FLOAT, N, None, variant=variant)
    print(f"case int8 variant {variant}", flush=True)
    rc = m.lib().opsnnQmmInt8(C.byref(a), None)
    assert rc == 0, rc
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    got = orc.f16_to_f32(out.to_host(np.uint16, (M, N)))
    # fp16 holds integers exactly only up to 2048; compare through the same rounding instead
    want = orc.f16_to_f32(orc.f32_to_f16(acc.astype(np.float32)))
    _check_equal(got.view(np.uint32), want.view(np.uint32), f"variant {variant}")
    # and exactly, on the int32 output of the plain kernel
    if variant == 1:
        out32 = m.DeviceBuffer(M * N * 4)
        a = cases.qmm_args_int8(m, d, M, K, N, 1, True, out32.ptr, m.ACL_INT32, m.ACL_FLOAT, N, None, variant=1)
        assert m.lib().opsnnQmmInt8(C.byref(a), None) == 0
        m.check(m.lib().aclrtSynchronizeDevice(), "sync")
        _check_equal(out32.to_host(np.int32, (M, N)), acc, "int32 accumulators")


@pytest.mark.parametrize("variant", [8, 9, 10, 11])
@pytest.mark.parametrize("M,K,N,batch,bias_dt,out_dt", [
    (300, 384, 1000, 1, "bf16", "bf16"),    # ragged rows and columns, three K tiles
    (512, 128, 704, 1, "i32", "f16"),       # one K tile, int32 bias
    (256, 1024, 352, 2, "f32", "bf16"),     # batched, one tile of 352 columns
    (65, 256, 96, 1, None, "bf16"),         # far smaller than one tile
])
def test_wide_tile_variants_full_epilogue(gpu, variant, M, K, N, batch, bias_dt, out_dt):
    """The four-wave kernel with 256 x 32n tiles (n = variant): per-token and per-channel scales, every bias type,
    ragged edges and batches, bit-exact against the oracle."""
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "f32": m.ACL_FLOAT, "i32": m.ACL_INT32, None: None}
    print(f"case int8 wide variant {variant} M={M} K={K} N={N} batch={batch} bias={bias_dt} out={out_dt}", flush=True)
    inp = cases.make_qmm_int8_inputs(m, M, K, N, variant * 7 + M, dt[bias_dt], True, batch=batch)
    want, _ = cases.oracle_qmm_int8(m, inp, M, K, N, True, dt[out_dt])
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    out = m.DeviceBuffer(batch * M * N * 2)
    out.fill(0xFF)
    a = cases.qmm_args_int8(m, d, M, K, N, batch, True, out.ptr, dt[out_dt], m.ACL_FLOAT, N, dt[bias_dt], variant=variant)
    rc = m.lib().opsnnQmmInt8(C.byref(a), None)
    assert rc == 0, rc
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    _check_equal(out.to_host(np.uint16, (batch, M, N)), want, f"wide variant {variant}")


def test_config2_full_size_on_sampled_rows(gpu):
    """BASELINE config 2 at full size (M=2048, K=4096, N=11008, bf16 bias/out): every output row the oracle is
    asked for (a seeded sample of 48 rows, first and last included) must be bit-identical."""
    m = gpu
    M, K, N = 2048, 4096, 11008
    inp = cases.make_qmm_int8_inputs(m, M, K, N, 0, m.ACL_BF16, True)
    print("case int8 config 2 full size", flush=True)
    got = cases.run_qmm_int8_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    rows = np.unique(np.concatenate([[0, M - 1, 255, 256], np.random.default_rng(1).integers(0, M, 44)]))
    want, _ = cases.oracle_qmm_int8(m, inp, M, K, N, True, m.ACL_BF16, rows=rows)
    _check_equal(got[0][rows], want[0], "config 2 sampled rows")
    # size-independent property: the result is linear in x1Scale -- doubling a row's scale doubles that row exactly
    inp2 = dict(inp)
    inp2["s1"] = inp["s1"] * np.float32(2.0)
    inp2["bias"] = None
    inp2["bias_dtype"] = None
    inp1 = dict(inp, bias=None, bias_dtype=None)
    y1 = orc.bf16_to_f32(cases.run_qmm_int8_aclnn(m, inp1, M, K, N, True, m.ACL_BF16))
    y2 = orc.bf16_to_f32(cases.run_qmm_int8_aclnn(m, inp2, M, K, N, True, m.ACL_BF16))
    assert np.array_equal(y2, y1 * 2.0)


@pytest.mark.parametrize("s2_dt,bias_dt,out_dt", [("bf16", "i32", "bf16"), ("f32", "f16", "f16")])
def test_column_split_launch(gpu, s2_dt, bias_dt, out_dt):
    """A shape whose 256x256 tiles do not fill whole rounds of the chip is computed by two launches over two column
    ranges (M=4096, N=4352: 16x16 tiles in the first, the last 256 columns in the second); scales, bias and output
    of the second range start at a column offset.  Sampled rows must be bit-identical to the oracle."""
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "f32": m.ACL_FLOAT, "i32": m.ACL_INT32}
    M, K, N = 4096, 1024, 4352
    print(f"case int8 column split s2={s2_dt} bias={bias_dt}", flush=True)
    inp = cases.make_qmm_int8_inputs(m, M, K, N, 11, dt[bias_dt], True, x2s_dtype=dt[s2_dt])
    got = cases.run_qmm_int8_aclnn(m, inp, M, K, N, True, dt[out_dt])
    rows = np.unique(np.concatenate([[0, M - 1, 255, 256], np.random.default_rng(2).integers(0, M, 28)]))
    want, _ = cases.oracle_qmm_int8(m, inp, M, K, N, True, dt[out_dt], rows=rows)
    _check_equal(got[0][rows], want[0], "column split")


@pytest.mark.parametrize("out_dt,N", [("i8", 5632), ("i32", 5632), ("i8", 5630), ("i32", 5001)])
def test_integer_outputs_on_the_four_wave_kernel(gpu, out_dt, N):
    """INT8 (requantised, offset in the packed scale word) and INT32 outputs: large shapes go to the four-wave kernel, whose
    integer epilogue must give the bits of the 8-wave kernel's (forced with its variant code; that kernel is held to the oracle in
    test_tc_family.py), and a sample of rows is checked against the oracle directly."""
    import ctypes as C
    m = gpu
    M, K = 2048, 3072
    print(f"case int8 {M}x{K}x{N} out={out_dt} on the four-wave kernel", flush=True)
    rng = np.random.default_rng(N)
    x1, x2 = cases.gen_int8(rng, (1, M, K)), cases.gen_int8(rng, (1, N, K))
    sf = cases.gen_scale(rng, N, 2e-5, 2e-4)
    s2 = orc.pack_u64_scale(sf, rng.uniform(-20, 20, N).astype(np.float32))
    bias = rng.integers(-3000, 3000, size=N).astype(np.int32)
    d = {k: m.DeviceBuffer(host=v) for k, v in dict(x1=x1, x2=x2, s2=s2, bias=bias).items()}
    odt, esz, npdt = (m.ACL_INT8, 1, np.int8) if out_dt == "i8" else (m.ACL_INT32, 4, np.int32)
    outs = []
    for variant in (0, 7):   # 7: OPSNN_VARIANT_I8_256_W8_K128, the 8-wave 256 x 256 tile kernel
        d_out = m.DeviceBuffer(M * N * esz)
        d_out.fill(0x55)
        a = cases.qmm_args_int8(m, d, M, K, N, 1, True, d_out.ptr, odt, m.ACL_UINT64, N, m.ACL_INT32, variant=variant)
        assert m.lib().opsnnQmmTc(C.byref(a), None) == 0
        m.check(m.lib().aclrtSynchronizeDevice(), "sync")
        outs.append(d_out.to_host(npdt, (M, N)))
    assert np.array_equal(outs[0], outs[1]), f"{int((outs[0] != outs[1]).sum())} outputs differ between the two kernels"
    rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 6)]))
    want = orc.qmm_tc(np.ascontiguousarray(x1[0][rows]), x2[0], orc.I8, orc.I8, len(rows), K, N, False, True, s2, orc.U64, None, None, bias,
                      orc.I32, orc.I8 if out_dt == "i8" else orc.I32)
    assert np.array_equal(outs[0][rows], want)
