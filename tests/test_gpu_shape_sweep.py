"""Seeded sweeps over (M, K, N) for the modes whose kernel choice depends on the shape: few rows against many, a K that is or
is not a whole number of a kernel's units, a narrow or a wide right operand.  The single shapes of the other test files name
the case each of them is there for; these sweeps look for the combinations between them (a selector's thresholds, the K
segments, idle waves, row slabs, short last rounds).  Every case is compared with the oracle at the mode's own bar; the
shapes are small enough for the whole file to run in well under a minute.
"""
import numpy as np
import pytest

import cases
import oracle_api as orc
from test_gpu_other_modes import check_close, plain

pytestmark = pytest.mark.gpu


def _shapes(seed, count, m_max, k_unit, k_max, n_unit, n_lo, n_hi):
    """`count` shapes: M from the few-rows, many-rows and tile ranges, K in whole units, N in whole units."""
    rng = np.random.default_rng(seed)
    out = []
    for i in range(count):
        lo, hi = ((1, 17), (17, 65), (65, 257), (257, m_max + 1))[i % 4]
        hi = min(hi, m_max + 1)
        M = int(rng.integers(lo, hi)) if lo < hi else int(rng.integers(1, m_max + 1))
        K = int(rng.integers(1, k_max // k_unit + 1)) * k_unit
        N = int(rng.integers(n_lo // n_unit, n_hi // n_unit + 1)) * n_unit
        out.append((M, K, N))
    return out


def _b16_bar(got, want, code, what, K=0):
    g, w = orc.b16_to_f32(got, code), orc.b16_to_f32(want, code)
    assert np.isfinite(g).all(), what
    # (the relative error's denominator has a floor of a hundredth of the mean |want|; for fp16 outputs at least 128 steps of the
    # subnormal range, 2^-17, so that one such step on a small result is not counted as more than 2^-7)
    floor = max(float(np.mean(np.abs(w))) * 1e-2, 2.0 ** -17 if code == orc.F16 else 1e-30)
    mx, mean = orc.rel_err_stats(g, w, floor)
    if not (mx <= 2.0 ** -7 and mean <= 2.0 ** -10):
        i = np.unravel_index(np.argmax(np.abs(g - w) / np.maximum(np.abs(w), 1e-30)), g.shape)
        raise AssertionError(f"{what}: max rel {mx:.3e} mean rel {mean:.3e}; worst at {i}: got {g[i]!r} want {w[i]!r}, median |want| {np.median(np.abs(w)):.3e}")
    # 99.9 % within rtol = atol = 1e-3.  Two allowances that the single-shape tests do not need: with a few hundred outputs one
    # bf16 result an ulp off is already more than a thousandth of them; and beyond K = 8192 fp32 sums in another order than the
    # oracle's flip one bf16 result in a thousand by an ulp (four times the 1e-3), so bf16 outputs get 3e-3 there.
    allow = max(3e-3 if (K > 8192 and code == orc.BF16) else 1e-3, 2.0 / g.size)
    frac = orc.isclose_fraction(g, w)
    assert frac <= allow, f"{what}: {frac:.2e} of elements outside rtol=atol=1e-3"


# (the last six of each list: more than 128 workgroups of 128 columns, where the 192- / 256-row instances and the tiles take over)
@pytest.mark.parametrize("M,K,N", _shapes(11, 40, 400, 128, 6144, 32, 256, 1024) + _shapes(31, 6, 300, 128, 1536, 32, 16512, 20480))
@pytest.mark.parametrize("w_dt,group", [("i4", 128), ("i8", 0), ("i4", 512), ("fp4", 32)])
def test_weight_only_shapes(gpu, M, K, N, w_dt, group):
    m = gpu
    if w_dt == "i4" and K % 256:
        K += 128   # (int4 rows of whole 16-byte pieces per chunk pair keep the case on the streamlined kernels)
    if group and K <= group:
        group = 0 if w_dt != "fp4" else 32
    dt = {"i8": m.ACL_INT8, "i4": m.ACL_INT4, "fp4": m.ACL_FLOAT4_E2M1}
    x_dt = m.ACL_FLOAT16 if (M + N) % 2 else m.ACL_BF16
    print(f"case sweep weight-only M={M} K={K} N={N} w={w_dt} g={group}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M + K + N, x_dt, dt[w_dt], group, True, w_dt != "fp4", None)
    want = cases.oracle_wq(m, inp, M, K, N)
    plain(False)
    check_close(cases.run_wq_aclnn(m, inp, M, K, N), want, x_dt, "weight-only sweep")


@pytest.mark.parametrize("M,K,N", _shapes(12, 32, 300, 128, 4096, 128, 256, 1024) + _shapes(13, 8, 64, 128, 20480, 8, 256, 520) +
                         _shapes(32, 6, 300, 128, 1536, 128, 16512, 20480))
def test_fp8_block_scale_shapes(gpu, M, K, N):
    m = gpu
    gsM = 128 if (M + K) % 3 == 0 else 1
    out = (m.ACL_BF16, m.ACL_FLOAT16, m.ACL_FLOAT)[(M + N) % 3]
    print(f"case sweep fp8 block M={M} K={K} N={N} gsM={gsM} out={out}", flush=True)
    inp = cases.make_blockscale_inputs(m, M, K, N, M + N + K, True, gsM)
    want = cases.oracle_blockscale(m, inp, M, K, N, True, out)
    got = cases.run_blockscale_aclnn(m, inp, M, K, N, True, out)
    if out == m.ACL_FLOAT:
        assert np.isfinite(got).all()
        mx, mean = orc.rel_err_stats(got, want)
        assert mean <= 2.0 ** -16 and orc.isclose_fraction(got, want) == 0.0, f"max rel {mx:.3e} mean rel {mean:.3e}"
    else:
        _b16_bar(got, want, orc.BF16 if out == m.ACL_BF16 else orc.F16, "fp8 block sweep", K)


@pytest.mark.parametrize("M,K,N", _shapes(14, 24, 300, 128, 4096, 32, 256, 1024) + _shapes(15, 8, 64, 128, 20480, 8, 256, 520) +
                         _shapes(33, 6, 300, 128, 1536, 32, 16512, 20480))
def test_fp8_row_column_scale_shapes(gpu, M, K, N):
    m = gpu
    out = m.ACL_BF16 if (M + N) % 2 else m.ACL_FLOAT16
    print(f"case sweep fp8 K-C M={M} K={K} N={N}", flush=True)
    inp = cases.make_tc_inputs(m, M, K, N, M + N, m.ACL_FLOAT8_E4M3FN, m.ACL_FLOAT, N, m.ACL_FLOAT if K % 256 else None, True, pertoken="M")
    want = cases.oracle_tc(m, inp, M, K, N, out)
    _b16_bar(cases.run_tc_aclnn(m, inp, M, K, N, out), want, orc.BF16 if out == m.ACL_BF16 else orc.F16, "fp8 K-C sweep", K)


@pytest.mark.parametrize("M,K,N", _shapes(16, 24, 300, 128, 4096, 8, 256, 1024) + _shapes(17, 8, 64, 128, 20480, 8, 256, 520))
def test_int8_per_tile_shapes(gpu, M, K, N):
    m = gpu
    print(f"case sweep int8 per-tile M={M} K={K} N={N}", flush=True)
    inp = cases.make_pertile_i8_inputs(m, M, K, N, M + N, True)
    want = cases.oracle_pertile_i8(m, inp, M, K, N, True, m.ACL_BF16)
    _b16_bar(cases.run_pertile_i8_aclnn(m, inp, M, K, N, True, m.ACL_BF16), want, orc.BF16, "int8 per-tile sweep", K)


@pytest.mark.parametrize("M,K,N", _shapes(18, 24, 300, 128, 4096, 8, 256, 1024) + _shapes(19, 8, 64, 128, 20480, 8, 256, 520))
def test_fp8_fp4_mx_shapes(gpu, M, K, N):
    m = gpu
    print(f"case sweep fp8 x fp4 MX M={M} K={K} N={N}", flush=True)
    inp = cases.make_a8w4_mx_inputs(m, M, K, N, M + N, True)
    want = cases.oracle_a8w4_mx(m, inp, M, K, N, True, m.ACL_FLOAT16)
    _b16_bar(cases.run_a8w4_mx_aclnn(m, inp, M, K, N, True, m.ACL_FLOAT16), want, orc.F16, "fp8 x fp4 MX sweep", K)


@pytest.mark.parametrize("M,K,N", _shapes(20, 32, 300, 128, 4096, 32, 256, 1024) + _shapes(21, 8, 64, 128, 20480, 8, 256, 520) +
                         _shapes(34, 6, 300, 128, 1536, 32, 16512, 20480))
@pytest.mark.parametrize("fp4", [False, True])
def test_mx_shapes(gpu, M, K, N, fp4):
    m = gpu
    out = m.ACL_BF16 if (fp4 or (M + K // 128) % 2) else m.ACL_FLOAT16   # (sums of e2m1 products with these scales leave the fp16 range)
    print(f"case sweep mx M={M} K={K} N={N} fp4={fp4} out={out}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, K + N + M, True, fp4)
    bias = np.random.default_rng(M).normal(0, 1, N).astype(np.float32) if N % 64 == 0 else None
    want = cases.oracle_mx(m, inp, M, K, N, True, out, bias)
    plain(False)
    _b16_bar(cases.run_mx_aclnn(m, inp, M, K, N, True, out, bias), want, orc.BF16 if out == m.ACL_BF16 else orc.F16, "mx sweep", K)


@pytest.mark.parametrize("M,K,N", _shapes(22, 24, 300, 16, 4096, 8, 64, 1024) + _shapes(23, 8, 16, 128, 20480, 8, 256, 520))
def test_int8_shapes_are_bit_identical(gpu, M, K, N):
    m = gpu
    print(f"case sweep int8 K-C M={M} K={K} N={N}", flush=True)
    got, want, _ = cases.run_qmm_int8_case(m, orc, M, K, N, seed=M * 31 + N, out_dtype=m.ACL_BF16, bias_dtype=m.ACL_BF16 if K % 32 else None,
                                           transpose_x2=True)
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ"


# ---- few rows against a wide right operand: every stream kernel's workgroups walk several column blocks ----
def _few_rows_wide(seed, count, m_max, k_unit, k_max, n_unit):
    rng = np.random.default_rng(seed)
    return [(int(rng.integers(1, m_max + 1)), int(rng.integers(1, k_max // k_unit + 1)) * k_unit,
             int(rng.integers(8192 // n_unit, 30000 // n_unit)) * n_unit) for _ in range(count)]


@pytest.mark.parametrize("M,K,N", _few_rows_wide(41, 16, 16, 128, 8192, 16))
@pytest.mark.parametrize("w_dt,group", [("i4", 128), ("i8", 0), ("i8", 64), ("fp4", 32)])
def test_weight_only_few_rows_wide(gpu, M, K, N, w_dt, group):
    m = gpu
    if group and K <= group:
        group = 0 if w_dt != "fp4" else 32
    dt = {"i8": m.ACL_INT8, "i4": m.ACL_INT4, "fp4": m.ACL_FLOAT4_E2M1}
    x_dt = m.ACL_FLOAT16 if (M + N // 16) % 2 else m.ACL_BF16
    print(f"case sweep weight-only wide M={M} K={K} N={N} w={w_dt} g={group}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M + K + N, x_dt, dt[w_dt], group, True, w_dt != "fp4", None)
    want = cases.oracle_wq(m, inp, M, K, N)
    plain(False)
    check_close(cases.run_wq_aclnn(m, inp, M, K, N), want, x_dt, "weight-only sweep, wide")


@pytest.mark.parametrize("M,K,N", _few_rows_wide(42, 10, 32, 128, 8192, 128))
def test_fp8_block_scale_few_rows_wide(gpu, M, K, N):
    m = gpu
    print(f"case sweep fp8 block wide M={M} K={K} N={N}", flush=True)
    inp = cases.make_blockscale_inputs(m, M, K, N, M + N + K, True, 1)
    want = cases.oracle_blockscale(m, inp, M, K, N, True, m.ACL_FLOAT16)
    _b16_bar(cases.run_blockscale_aclnn(m, inp, M, K, N, True, m.ACL_FLOAT16), want, orc.F16, "fp8 block sweep, wide", K)


@pytest.mark.parametrize("M,K,N", _few_rows_wide(43, 10, 32, 128, 8192, 8))
@pytest.mark.parametrize("mode", ["kc", "pertile", "a8w4", "mxfp8", "mxfp4"])
def test_quant_modes_few_rows_wide(gpu, M, K, N, mode):
    m = gpu
    print(f"case sweep {mode} wide M={M} K={K} N={N}", flush=True)
    plain(False)
    if mode == "kc":
        inp = cases.make_tc_inputs(m, M, K, N, M + N, m.ACL_FLOAT8_E4M3FN, m.ACL_FLOAT, N, m.ACL_FLOAT, True, pertoken="M")
        want = cases.oracle_tc(m, inp, M, K, N, m.ACL_FLOAT16)
        _b16_bar(cases.run_tc_aclnn(m, inp, M, K, N, m.ACL_FLOAT16), want, orc.F16, "fp8 K-C sweep, wide", K)
    elif mode == "pertile":
        inp = cases.make_pertile_i8_inputs(m, M, K, N, M + N, True)
        want = cases.oracle_pertile_i8(m, inp, M, K, N, True, m.ACL_BF16)
        _b16_bar(cases.run_pertile_i8_aclnn(m, inp, M, K, N, True, m.ACL_BF16), want, orc.BF16, "int8 per-tile sweep, wide", K)
    elif mode == "a8w4":
        inp = cases.make_a8w4_mx_inputs(m, M, K, N, M + N, True)
        want = cases.oracle_a8w4_mx(m, inp, M, K, N, True, m.ACL_FLOAT16)
        _b16_bar(cases.run_a8w4_mx_aclnn(m, inp, M, K, N, True, m.ACL_FLOAT16), want, orc.F16, "fp8 x fp4 MX sweep, wide", K)
    else:
        fp4 = mode == "mxfp4"
        inp = cases.make_mx_inputs(m, M, K, N, K + N + M, True, fp4)
        want = cases.oracle_mx(m, inp, M, K, N, True, m.ACL_BF16)
        _b16_bar(cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16), want, orc.BF16, "mx sweep, wide", K)


# ---- an N-contiguous right operand (re-laid out into the workspace first) ----
@pytest.mark.parametrize("M,K,N", _shapes(44, 12, 300, 128, 3072, 32, 256, 1024))
@pytest.mark.parametrize("w_dt,group", [("i4", 128), ("i8", 0)])
def test_weight_only_n_contiguous_shapes(gpu, M, K, N, w_dt, group):
    m = gpu
    dt = {"i8": m.ACL_INT8, "i4": m.ACL_INT4}
    if group and K <= group:
        group = 0
    print(f"case sweep weight-only N-contiguous M={M} K={K} N={N} w={w_dt} g={group}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M + K + N, m.ACL_BF16, dt[w_dt], group, False, True, m.ACL_BF16)
    want = cases.oracle_wq(m, inp, M, K, N)
    plain(False)
    check_close(cases.run_wq_aclnn(m, inp, M, K, N), want, m.ACL_BF16, "weight-only sweep, N-contiguous")


# ---- the quantizers that prepare the operands: bit-exact, any row count and row length ----
def _mats(seed, count, rows_max, col_unit, cols_max):
    rng = np.random.default_rng(seed)
    return [(int(rng.integers(1, rows_max + 1)), int(rng.integers(1, cols_max // col_unit + 1)) * col_unit) for _ in range(count)]


@pytest.mark.parametrize("rows,cols", _mats(51, 24, 700, 2, 9000))
@pytest.mark.parametrize("y_name,symmetric", [("i8", True), ("i8", False), ("i4", True), ("e4m3", True)])
def test_dynamic_quant_shapes(gpu, rows, cols, y_name, symmetric):
    from test_dynamic_quant import _run
    m = gpu
    y_dt = {"i8": orc.I8, "i4": orc.I4, "e4m3": orc.E4M3}[y_name]
    x_dt = orc.BF16 if (rows + cols) % 2 else orc.F16
    print(f"case sweep dynamic quant {rows}x{cols} y={y_name} symmetric={symmetric}", flush=True)
    rng = np.random.default_rng(rows * 7 + cols)
    xb = orc.f32_to_b16(rng.normal(0, 2, size=(rows, cols)).astype(np.float32), x_dt)
    smb = orc.f32_to_b16(rng.uniform(0.5, 2.0, cols).astype(np.float32), x_dt) if cols % 4 == 0 else None
    want = orc.dynamic_quant(xb, x_dt, y_dt, smooth=smb, symmetric=symmetric)
    gy, gs, go = _run(m, xb, x_dt, y_dt, smb, symmetric)
    assert np.array_equal(gs.view(np.uint32), want[1].reshape(-1).view(np.uint32)), "scale differs"
    if not symmetric:
        assert np.array_equal(go.view(np.uint32), want[2].reshape(-1).view(np.uint32)), "offset differs"
    wy = want[0].reshape(-1)
    z = ((gy | wy) & 0x7f) == 0 if y_dt == orc.E4M3 else np.zeros(gy.shape, bool)   # the sign of a zero result is not pinned
    assert np.array_equal(gy[~z], wy[~z]), f"{int((gy[~z] != wy[~z]).sum())} outputs differ"


@pytest.mark.parametrize("rows,cols", _mats(52, 20, 700, 1, 3000))
@pytest.mark.parametrize("rb,cb", [(1, 128), (128, 128), (64, 192)])
def test_dynamic_block_quant_shapes(gpu, rows, cols, rb, cb):
    from test_dynamic_block_quant import _run
    m = gpu
    x_dt = orc.BF16 if (rows + cols) % 2 else orc.F16
    print(f"case sweep block quant {rows}x{cols} {rb}x{cb}", flush=True)
    rng = np.random.default_rng(rows * 5 + cols)
    xf = (rng.normal(0, 1, size=(rows, cols)) * 10.0 ** rng.integers(-3, 3, size=(rows, cols))).astype(np.float32)
    xb = orc.f32_to_b16(xf, x_dt)
    want_y, want_s = orc.dynamic_block_quant(xb, x_dt, orc.E4M3, rb, cb, 0.0)
    gy, gs = _run(m, xb, x_dt, orc.E4M3, rb, cb, 0.0)
    assert np.array_equal(gs.view(np.uint32), want_s.view(np.uint32)), "scale differs"
    z = ((gy | want_y) & 0x7f) == 0
    assert np.array_equal(gy[~z], want_y[~z]), f"{int((gy[~z] != want_y[~z]).sum())} of {want_y.size} outputs differ"


@pytest.mark.parametrize("rows,cols", _mats(53, 24, 700, 2, 9000))
@pytest.mark.parametrize("y_name", ["e2m1", "e4m3"])
def test_dynamic_mx_quant_shapes(gpu, rows, cols, y_name):
    from test_dynamic_mx_quant import _run, _codes, _same_but_zero_sign
    m = gpu
    y_dt = orc.E2M1 if y_name == "e2m1" else orc.E4M3
    x_dt = orc.BF16 if (rows + cols) % 2 else orc.F16
    print(f"case sweep mx quant {rows}x{cols} y={y_name}", flush=True)
    rng = np.random.default_rng(rows * 3 + cols)
    xf = (rng.normal(0, 1, size=(rows, cols)) * 2.0 ** rng.integers(-14, 14, size=(rows, 1))).astype(np.float32)
    xb = orc.f32_to_b16(xf, x_dt)
    want_y, want_s = orc.dynamic_mx_quant(xb, x_dt, y_dt)
    gy, gs = _run(m, xb, x_dt, y_dt)
    assert np.array_equal(gs, want_s), "scale bytes differ"
    assert _same_but_zero_sign(_codes(gy, y_dt), _codes(want_y.reshape(-1), y_dt), y_dt)


# ---- K tails: a K that is no whole number of 128-element tiles (padding pre-steps) or of 16 (int8) ----
def _tails(seed, count, m_max, k_unit, k_max, n_unit, n_hi):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        M, K, N = int(rng.integers(1, m_max + 1)), int(rng.integers(1, k_max // k_unit + 1)) * k_unit, int(rng.integers(64 // n_unit, n_hi // n_unit + 1)) * n_unit
        if K % 128:
            out.append((M, K, N))
    return out


@pytest.mark.parametrize("M,K,N", _tails(61, 16, 300, 1, 3000, 1, 600))
def test_int8_k_tail_shapes_are_bit_identical(gpu, M, K, N):
    m = gpu
    print(f"case sweep int8 K tail M={M} K={K} N={N}", flush=True)
    got, want, _ = cases.run_qmm_int8_case(m, orc, M, K, N, seed=M * 31 + N, out_dtype=m.ACL_FLOAT16, bias_dtype=m.ACL_FLOAT if K % 2 else None,
                                           transpose_x2=(M + K) % 3 != 0)
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ"


@pytest.mark.parametrize("M,K,N", _tails(62, 12, 300, 8, 3000, 8, 600))
def test_fp8_block_scale_k_tail_shapes(gpu, M, K, N):
    m = gpu
    tB = (M + N) % 4 != 0
    print(f"case sweep fp8 block K tail M={M} K={K} N={N} tB={tB}", flush=True)
    inp = cases.make_blockscale_inputs(m, M, K, N, M + N + K, tB, 1)
    want = cases.oracle_blockscale(m, inp, M, K, N, tB, m.ACL_FLOAT16)
    _b16_bar(cases.run_blockscale_aclnn(m, inp, M, K, N, tB, m.ACL_FLOAT16), want, orc.F16, "fp8 block K tail sweep", K)


@pytest.mark.parametrize("M,K,N", _tails(63, 12, 300, 32, 3000, 2, 600))
@pytest.mark.parametrize("fp4", [False, True])
def test_mx_k_tail_shapes(gpu, M, K, N, fp4):
    m = gpu
    print(f"case sweep mx K tail M={M} K={K} N={N} fp4={fp4}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, K + N + M, True, fp4)
    want = cases.oracle_mx(m, inp, M, K, N, True, m.ACL_BF16)
    plain(False)
    _b16_bar(cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16), want, orc.BF16, "mx K tail sweep", K)


@pytest.mark.parametrize("M,K,N", _tails(64, 10, 300, 32, 3000, 2, 600))
def test_fp8_fp4_mx_k_tail_shapes(gpu, M, K, N):
    m = gpu
    print(f"case sweep fp8 x fp4 MX K tail M={M} K={K} N={N}", flush=True)
    inp = cases.make_a8w4_mx_inputs(m, M, K, N, M + N, True)
    want = cases.oracle_a8w4_mx(m, inp, M, K, N, True, m.ACL_FLOAT16)
    _b16_bar(cases.run_a8w4_mx_aclnn(m, inp, M, K, N, True, m.ACL_FLOAT16), want, orc.F16, "fp8 x fp4 MX K tail sweep", K)


# ---- batched operands: every batch has its own x1 and x2; the scales, the bias and the kernel choice are shared ----
@pytest.mark.parametrize("M,K,N", _shapes(71, 12, 300, 16, 2048, 8, 64, 600) + _shapes(72, 4, 16, 128, 12288, 8, 256, 520))
def test_int8_batched_shapes_are_bit_identical(gpu, M, K, N):
    m = gpu
    batch = 2 + (M + N) % 3
    print(f"case sweep int8 batched M={M} K={K} N={N} batch={batch}", flush=True)
    got, want, _ = cases.run_qmm_int8_case(m, orc, M, K, N, seed=M * 31 + N, out_dtype=m.ACL_BF16, bias_dtype=m.ACL_FLOAT if K % 32 else None,
                                           transpose_x2=(M + K) % 3 != 0, batch=batch)
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ"


@pytest.mark.parametrize("M,K,N", _shapes(73, 12, 300, 128, 2048, 8, 64, 600) + _shapes(74, 4, 32, 128, 12288, 8, 256, 520))
@pytest.mark.parametrize("fp4", [False, True])
def test_mx_batched_shapes(gpu, M, K, N, fp4):
    m = gpu
    batch = 2 + (M + N) % 3
    print(f"case sweep mx batched M={M} K={K} N={N} fp4={fp4} batch={batch}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, K + N + M, True, fp4, batch=batch)
    want = cases.oracle_mx(m, inp, M, K, N, True, m.ACL_BF16)
    plain(False)
    _b16_bar(cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16), want, orc.BF16, "mx batched sweep", K)


# ---- the two group modes whose right operand is always stored [N, K] ----
@pytest.mark.parametrize("M,K,N", _shapes(75, 20, 300, 32, 3072, 8, 64, 600) + _shapes(76, 6, 64, 128, 12288, 8, 256, 520))
def test_fp8_fp4_group_scale_shapes(gpu, M, K, N):
    """fp8 x fp4 with 16-bit scales per 32 elements of K and a packed output scale per column."""
    m = gpu
    K = max(K, 64)   # (the mode needs more than one group)
    s_dt, out = (m.ACL_BF16, m.ACL_BF16) if (M + N) % 2 else (m.ACL_FLOAT16, m.ACL_FLOAT16)
    print(f"case sweep fp8 x fp4 group scale M={M} K={K} N={N} scale={s_dt}", flush=True)
    inp = cases.make_tcg_inputs(m, M, K, N, M + N, s_dt)
    inp["s2"] = inp["s2"] ^ ((np.arange(inp["s2"].size, dtype=np.uint32).reshape(inp["s2"].shape) % 3 == 0).astype(np.uint16) << 15)
    want = cases.oracle_tcg(m, inp, M, K, N, out)
    _b16_bar(cases.run_tcg_aclnn(m, inp, M, K, N, out), want, orc.BF16 if out == m.ACL_BF16 else orc.F16, "fp8 x fp4 group scale sweep", K)


@pytest.mark.parametrize("M,K,N", _shapes(77, 16, 300, 1024, 8192, 256, 256, 1536))
def test_int4_group_offset_shapes_are_bit_identical(gpu, M, K, N):
    """int4 x int4 with scales and offsets per 256 elements of K."""
    m = gpu
    out = m.ACL_BF16 if (M + N // 256) % 2 else m.ACL_FLOAT16
    print(f"case sweep int4 K-G M={M} K={K} N={N} out={out}", flush=True)
    inp = cases.make_i4_asym_inputs(m, M, K, N, M + N)
    want = cases.oracle_i4_asym(m, inp, M, K, N, out)
    got = cases.run_i4_asym_aclnn(m, inp, M, K, N, out)
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ"


# ---- FRACTAL_NZ right operands: the NZ entry points give bit for bit what the ND ones give on the same matrix ----
@pytest.mark.parametrize("M,K,N", _shapes(81, 16, 300, 64, 3072, 8, 64, 1024))
@pytest.mark.parametrize("w_dt,group,c0e", [("i4", 128, 16), ("i4", 0, 32), ("i8", 0, 32)])
def test_weight_only_nz_shapes_equal_nd(gpu, M, K, N, w_dt, group, c0e):
    from test_nz_entry_points import nd_to_nz
    m = gpu
    if group and K % group:
        K += group - K % group
    tW = w_dt == "i8" and (M + N) % 2 == 1
    dt = {"i8": m.ACL_INT8, "i4": m.ACL_INT4}
    x_dt = m.ACL_FLOAT16 if (M + N) % 4 < 2 else m.ACL_BF16
    print(f"case sweep weight-only NZ M={M} K={K} N={N} w={w_dt} g={group} tW={tW} c0={c0e}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M + N, x_dt, dt[w_dt], group, tW, True, None)
    plain(False)
    want = cases.run_wq_aclnn(m, inp, M, K, N)
    check_close(want, cases.oracle_wq(m, inp, M, K, N), x_dt, "weight-only NZ sweep, ND call")
    nz = nd_to_nz(inp["w"].reshape(N if tW else K, -1).view(np.uint8), c0e if w_dt == "i8" else c0e // 2)
    got = cases.run_wq_aclnn(m, dict(inp, w=nz), M, K, N, nz_storage=(nz.shape[0], nz.shape[1], 16, c0e))
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ from the ND entry point"


@pytest.mark.parametrize("M,K,N", _shapes(82, 16, 300, 4, 3072, 4, 64, 1024))
def test_int8_nz_shapes_equal_nd(gpu, M, K, N):
    from test_nz_entry_points import nd_to_nz
    m = gpu
    tB = (M + K) % 2 == 1
    print(f"case sweep int8 NZ M={M} K={K} N={N} tB={tB}", flush=True)
    inp = cases.make_qmm_int8_inputs(m, M, K, N, M + K, m.ACL_BF16, tB)
    want, _ = cases.oracle_qmm_int8(m, inp, M, K, N, tB, m.ACL_BF16)
    nz = nd_to_nz(inp["x2"][0].view(np.uint8), 32)
    got = cases.run_qmm_int8_aclnn(m, dict(inp, x2=nz[None]), M, K, N, tB, m.ACL_BF16, nz_storage=(nz.shape[0], nz.shape[1], 16, 32))
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ"


# ---- a K of one x slab on the first-generation weight-only kernel (N no multiple of 32 keeps the call there): the chunks
# past the end of K must not be multiplied at all -- their x slab in LDS was never written (found as NaN results that
# depended on the kernel that had run before; conftest fills the LDS with NaN patterns before every GPU test) ----
@pytest.mark.parametrize("M,K,N,w_dt", [(244, 192, 144, "i4"), (60, 64, 48, "i4"), (16, 512, 40, "i4"), (30, 256, 72, "i4"), (9, 96, 24, "i8"),
                                        (50, 64, 80, "i8"), (32, 208, 56, "i8"), (128, 128, 16, "i8")])
def test_weight_only_one_slab_of_k(gpu, M, K, N, w_dt):
    m = gpu
    dt = {"i8": m.ACL_INT8, "i4": m.ACL_INT4}
    for x_dt in (m.ACL_FLOAT16, m.ACL_BF16):
        print(f"case weight-only one slab M={M} K={K} N={N} w={w_dt} x={x_dt}", flush=True)
        inp = cases.make_wq_inputs(m, M, K, N, M + N, x_dt, dt[w_dt], 0, True, True, None)
        plain(False)
        m.check(m.lib().opsnnDebugFillLds(None), "opsnnDebugFillLds")
        check_close(cases.run_wq_aclnn(m, inp, M, K, N), cases.oracle_wq(m, inp, M, K, N), x_dt, "weight-only, one slab of K")


# ---- int8 epilogues: output, bias and x2-scale forms picked per shape ----
_EPILOGUES = [("bf16", "bf16", "f32", None), ("bf16", None, "f32", 1), ("f16", "f32", "f32", None), ("bf16", "i32", "bf16", None),
              ("f16", "f16", "f32", 1), ("bf16", "bf16", "bf16", None)]


@pytest.mark.parametrize("M,K,N", _shapes(91, 36, 400, 8, 4096, 1, 32, 1100) + _shapes(92, 6, 32, 64, 16384, 4, 128, 600))
def test_int8_epilogue_forms_are_bit_identical(gpu, M, K, N):
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "f32": m.ACL_FLOAT, "i32": m.ACL_INT32, None: None}
    out_dt, bias_dt, s2_dt, s2_len = _EPILOGUES[(M + K + N) % len(_EPILOGUES)]
    tB = (M + N) % 3 != 0
    print(f"case sweep int8 epilogue M={M} K={K} N={N} tB={tB} out={out_dt} bias={bias_dt} s2={s2_dt} x{s2_len}", flush=True)
    got, want, _ = cases.run_qmm_int8_case(m, orc, M, K, N, seed=M * 31 + N, out_dtype=dt[out_dt], bias_dtype=dt[bias_dt], transpose_x2=tB,
                                           x2s_len=s2_len, x2s_dtype=dt[s2_dt])
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ"


# ---- weight-only forms: bias (x's dtype or fp32), no offset, one scale for the whole weight, the V3 entry point, e4m3 weights ----
_WQ_FORMS = [dict(w="i4", group=128, off=True, bias="x", pt=False, v3=False), dict(w="i8", group=0, off=False, bias="f32", pt=False, v3=False),
             dict(w="i4", group=0, off=False, bias=None, pt=True, v3=False), dict(w="i8", group=0, off=True, bias="x", pt=True, v3=True),
             dict(w="i8", group=128, off=True, bias="f32", pt=False, v3=True), dict(w="i4", group=64, off=False, bias="x", pt=False, v3=False),
             dict(w="e4m3", group=0, off=False, bias=None, pt=False, v3=False)]


@pytest.mark.parametrize("M,K,N", _shapes(93, 44, 400, 128, 6144, 32, 256, 1024) + _shapes(94, 12, 64, 128, 16384, 8, 64, 520))
def test_weight_only_forms(gpu, M, K, N):
    m = gpu
    f = _WQ_FORMS[(M + K // 128 + N // 8) % len(_WQ_FORMS)]
    if f["w"] == "i4" and K % 256:
        K += 128
    x_dt = m.ACL_FLOAT16 if (M + N) % 2 else m.ACL_BF16
    if f["w"] == "e4m3":
        x_dt = m.ACL_BF16 if K > 4096 else x_dt
    group = f["group"] if K > f["group"] else 0
    w_dt = {"i8": m.ACL_INT8, "i4": m.ACL_INT4, "e4m3": m.ACL_FLOAT8_E4M3FN}[f["w"]]
    bias_dt = {"x": x_dt, "f32": m.ACL_FLOAT, None: None}[f["bias"]]
    if bias_dt == m.ACL_FLOAT and x_dt != m.ACL_BF16:
        bias_dt = x_dt   # (an fp32 bias goes with bf16 x)
    tW = (M + K // 128) % 3 != 0
    print(f"case sweep weight-only forms M={M} K={K} N={N} tW={tW} x={x_dt} {f}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M + K + N, x_dt, w_dt, group, tW, f["off"], bias_dt, per_tensor=f["pt"] and group == 0)
    want = cases.oracle_wq(m, inp, M, K, N)
    plain(False)
    check_close(cases.run_wq_aclnn(m, inp, M, K, N, v3=f["v3"]), want, x_dt, "weight-only forms sweep")


# ---- int8 without a per-token scale: packed, fp32 and bf16 scales, int8 / int32 / 16-bit outputs, offsets ----
_TC_FORMS = [("u64", "N", "i32", "f16", 0), ("u64", 1, "i32", "i8", 1), ("u64", "N", "i32", "i8", "N"), ("u64", "N", None, "i8", 0),
             ("f32", 1, "i32", "bf16", 0), ("f32", 1, "f32", "bf16", 0), ("bf16", 1, None, "bf16", 0), ("f32", "N", "i32", "i32", 0),
             ("bf16", "N", "bf16", "bf16", 0)]


@pytest.mark.parametrize("M,K,N", _shapes(95, 36, 400, 8, 4096, 1, 32, 1100) + _shapes(96, 9, 32, 64, 16384, 4, 128, 600))
def test_int8_static_forms_are_bit_identical(gpu, M, K, N):
    m = gpu
    dt = {"u64": m.ACL_UINT64, "f32": m.ACL_FLOAT, "bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "i32": m.ACL_INT32, "i8": m.ACL_INT8, None: None}
    s_dt, s_len, bias_dt, out_dt, off_len = _TC_FORMS[(M + K + N) % len(_TC_FORMS)]
    tB = (M + N) % 3 != 0
    print(f"case sweep int8 static M={M} K={K} N={N} tB={tB} scale={s_dt}/{s_len} bias={bias_dt} out={out_dt} off={off_len}", flush=True)
    inp = cases.make_tc_inputs(m, M, K, N, M + N, m.ACL_INT8, dt[s_dt], 1 if s_len == 1 else N, dt[bias_dt], tB, pertoken=False,
                               offset_len=N if off_len == "N" else off_len)
    want = cases.oracle_tc(m, inp, M, K, N, dt[out_dt])
    got = cases.run_tc_aclnn(m, inp, M, K, N, dt[out_dt])
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ"


# ---- fp8 with per-row, one-element or no x1 scale; e4m3 and e5m2; fp32 and packed x2 scales; K tails and N-contiguous x2 ----
_F8_FORMS = [("e4m3", "f32", "N", "f32", "M"), ("e5m2", "f32", "N", "f32", True), ("e4m3", "u64", "N", None, False), ("e4m3", "u64", 1, "f32", False),
             ("e4m3", "f32", 1, None, "M"), ("e4m3", "f32", 1, None, True), ("e5m2", "f32", "N", None, "M")]


@pytest.mark.parametrize("M,K,N", _shapes(97, 35, 400, 8, 4096, 8, 64, 1100) + _shapes(98, 7, 32, 128, 16384, 8, 128, 600))
def test_fp8_scale_forms(gpu, M, K, N):
    m = gpu
    dt = {"e4m3": m.ACL_FLOAT8_E4M3FN, "e5m2": m.ACL_FLOAT8_E5M2, "u64": m.ACL_UINT64, "f32": m.ACL_FLOAT, None: None}
    in_dt, s_dt, s_len, bias_dt, pt = _F8_FORMS[(M + K // 8 + N // 8) % len(_F8_FORMS)]
    out = m.ACL_BF16 if (M + N) % 2 else m.ACL_FLOAT16
    tB = (M + N) % 3 != 0
    print(f"case sweep fp8 forms M={M} K={K} N={N} tB={tB} in={in_dt} scale={s_dt}/{s_len} bias={bias_dt} pt={pt}", flush=True)
    inp = cases.make_tc_inputs(m, M, K, N, M + N, dt[in_dt], dt[s_dt], 1 if s_len == 1 else N, dt[bias_dt], tB, pertoken=pt, e5m2=in_dt == "e5m2")
    want = cases.oracle_tc(m, inp, M, K, N, out)
    _b16_bar(cases.run_tc_aclnn(m, inp, M, K, N, out), want, orc.BF16 if out == m.ACL_BF16 else orc.F16, "fp8 forms sweep", K)


# ---- fp8 block scales with N-contiguous and batched operands, int8 per-tile with N-contiguous x2 ----
@pytest.mark.parametrize("M,K,N", _shapes(99, 20, 300, 128, 4096, 128, 128, 1024) + _shapes(100, 4, 32, 128, 12288, 128, 256, 640))
def test_fp8_block_scale_n_contiguous_and_batched(gpu, M, K, N):
    m = gpu
    batch, tB = 1 + (M + N // 128) % 3, (M + K // 128) % 2 == 0
    gsM = 128 if (M + K) % 3 == 0 else 1
    out = m.ACL_BF16 if (M + N // 128) % 2 else m.ACL_FLOAT16
    print(f"case sweep fp8 block M={M} K={K} N={N} tB={tB} batch={batch} gsM={gsM}", flush=True)
    inp = cases.make_blockscale_inputs(m, M, K, N, M + N + K, tB, gsM, batch=batch)
    want = cases.oracle_blockscale(m, inp, M, K, N, tB, out)
    _b16_bar(cases.run_blockscale_aclnn(m, inp, M, K, N, tB, out), want, orc.BF16 if out == m.ACL_BF16 else orc.F16, "fp8 block sweep, layouts", K)


@pytest.mark.parametrize("M,K,N", _shapes(101, 16, 300, 128, 4096, 8, 128, 1024))
def test_int8_per_tile_n_contiguous(gpu, M, K, N):
    m = gpu
    print(f"case sweep int8 per-tile N-contiguous M={M} K={K} N={N}", flush=True)
    inp = cases.make_pertile_i8_inputs(m, M, K, N, M + N, False)
    want = cases.oracle_pertile_i8(m, inp, M, K, N, False, m.ACL_BF16)
    _b16_bar(cases.run_pertile_i8_aclnn(m, inp, M, K, N, False, m.ACL_BF16), want, orc.BF16, "int8 per-tile N-contiguous sweep", K)


# ---- weight-only with any N and a short or ragged K: the first-generation kernel and the plain one behind the streamlined ones ----
@pytest.mark.parametrize("M,K,N", _shapes(102, 40, 300, 8, 2048, 1, 8, 700))
@pytest.mark.parametrize("w_dt", ["i4", "i8"])
def test_weight_only_ragged_shapes(gpu, M, K, N, w_dt):
    m = gpu
    dt = {"i8": m.ACL_INT8, "i4": m.ACL_INT4}
    x_dt = m.ACL_FLOAT16 if (M + N) % 2 else m.ACL_BF16
    group = (0, 32, 64, 128)[(M + K // 8) % 4]
    if group and (K % group or K <= group):
        group = 0
    tW = (M + N + K // 8) % 3 != 0
    if w_dt == "i4" and not tW and N % 2:
        N += 1   # (packed nibbles: whole bytes per stored row)
    print(f"case sweep weight-only ragged M={M} K={K} N={N} w={w_dt} g={group} tW={tW}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M + K + N, x_dt, dt[w_dt], group, tW, (M + N) % 4 != 0, x_dt if N % 3 == 0 else None)
    want = cases.oracle_wq(m, inp, M, K, N)
    plain(False)
    check_close(cases.run_wq_aclnn(m, inp, M, K, N), want, x_dt, "weight-only ragged sweep")


# ---- the re-layout behind N-contiguous right operands (aclnnPrepackMatmulWeight), bytes and nibbles, any K and N ----
@pytest.mark.parametrize("K,N", _mats(110, 30, 3000, 1, 3000) + [(1, 1), (2, 4097), (4097, 2), (64, 64), (33, 31)])
@pytest.mark.parametrize("bits", [8, 4])
def test_prepack_shapes(gpu, K, N, bits):
    m = gpu
    if bits == 4:
        K, N = K + K % 2, N + N % 2   # whole bytes per row on both sides
    B = 1 + (K + N) % 2
    print(f"case sweep prepack K={K} N={N} bits={bits} batch={B}", flush=True)
    rng = np.random.default_rng(K * 7 + N)
    if bits == 8:
        src = rng.integers(-128, 128, size=(B, K, N), dtype=np.int8)
        want = np.ascontiguousarray(src.transpose(0, 2, 1)).view(np.uint8)
        adt = m.ACL_INT8
    else:
        codes = rng.integers(0, 16, size=(B, K, N), dtype=np.uint8)
        src = orc.pack_nibbles(codes)
        want = orc.pack_nibbles(np.ascontiguousarray(codes.transpose(0, 2, 1)))
        adt = m.ACL_INT4
    d_src = m.DeviceBuffer(host=src)
    d_dst = cases.guarded_out(m, want.nbytes, 0xEE)
    rc, ws = m.prepack_matmul_weight(m.Tensor((B, K, N), adt, d_src), m.Tensor((B, N, K), adt, d_dst))
    assert rc == 0, m.err_msg()
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    got = d_dst.to_host(np.uint8, want.shape)
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {want.size} bytes differ"


# ---- operands at element offsets inside their storage: pointers that are not 16-byte (or even 4-byte) aligned ----
def _at_offset(m, shape, dtype, host, off, elem_bytes, strides=None, storage_cols=None):
    """A tensor whose data starts `off` elements into its storage (junk in front); returns (tensor, buffer).  storage_cols: the
    storage is declared as rows of that many elements (for operands whose storage must have two dimensions)."""
    raw = np.ascontiguousarray(host).view(np.uint8).reshape(-1)
    n = off + raw.size // elem_bytes
    if storage_cols:
        rows = -(-n // storage_cols)
        sshape, tail = (rows, storage_cols), (rows * storage_cols - n) * elem_bytes
    else:
        sshape, tail = (n,), 0
    buf = m.DeviceBuffer(host=np.concatenate([np.full(off * elem_bytes, 0x5A, np.uint8), raw, np.full(tail, 0x5A, np.uint8)]))
    return m.Tensor(shape, dtype, buf, strides=strides, offset=off, storage_shape=sshape), buf


@pytest.mark.parametrize("M,K,N", _shapes(120, 24, 400, 16, 4096, 8, 64, 1100))
def test_int8_operands_at_odd_offsets_are_bit_identical(gpu, M, K, N):
    m = gpu
    tB = (M + N) % 3 != 0
    o = [(1, 3, 1, 1, 1, 1), (4, 8, 2, 0, 1, 2), (16, 1, 0, 1, 0, 4), (0, 16, 1, 1, 1, 0), (5, 0, 0, 0, 0, 1)][(M + K + N) % 5]
    print(f"case sweep int8 offsets M={M} K={K} N={N} tB={tB} offsets={o}", flush=True)
    inp = cases.make_qmm_int8_inputs(m, M, K, N, M * 31 + N, m.ACL_BF16, tB)
    want, _ = cases.oracle_qmm_int8(m, inp, M, K, N, tB, m.ACL_BF16)
    x1, b1 = _at_offset(m, (M, K), m.ACL_INT8, inp["x1"][0], o[0], 1)
    x2, b2 = _at_offset(m, (N, K) if tB else (K, N), m.ACL_INT8, inp["x2"][0], o[1], 1, storage_cols=K if tB else N)
    s1, b3 = _at_offset(m, (M,), m.ACL_FLOAT, inp["s1"], o[2], 4)
    s2, b4 = _at_offset(m, (N,), m.ACL_FLOAT, inp["s2"], o[3], 4)
    bias, b5 = _at_offset(m, (N,), m.ACL_BF16, inp["bias"], o[4], 2)
    d_out = cases.guarded_out(m, (M * N + o[5]) * 2)
    out = m.Tensor((M, N), m.ACL_BF16, d_out, offset=o[5], storage_shape=(M * N + o[5],))
    ws = m.quant_matmul_v5(x1, x2, s1, s2, out, bias=bias, transpose_x2=tB)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    del ws
    got = d_out.to_host(np.uint16, (M * N + o[5],))
    assert (got[:o[5]] == 0xFFFF).all(), "wrote in front of the output view"
    got = got[o[5]:].reshape(M, N)
    assert np.array_equal(got, want[0]), f"{int((got != want[0]).sum())} of {got.size} outputs differ"


@pytest.mark.parametrize("M,K,N", _shapes(121, 24, 300, 128, 4096, 32, 256, 1024))
def test_weight_only_operands_at_odd_offsets(gpu, M, K, N):
    m = gpu
    o = [(1, 1, 1, 1), (8, 16, 0, 2), (3, 0, 1, 0), (0, 4, 2, 4), (2, 3, 1, 1)][(M + K // 128 + N // 32) % 5]
    x_dt = m.ACL_FLOAT16 if (M + N) % 2 else m.ACL_BF16
    group = 128 if (M + K // 128) % 2 and K > 128 else 0
    G = K // group if group else 1
    print(f"case sweep weight-only offsets M={M} K={K} N={N} g={group} offsets={o}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M + K + N, x_dt, m.ACL_INT8, group, True, True, None)
    want = cases.oracle_wq(m, inp, M, K, N)
    x, b1 = _at_offset(m, (M, K), x_dt, inp["x"], o[0], 2)
    w, b2 = _at_offset(m, (K, N), m.ACL_INT8, inp["w"], o[1], 1, strides=(1, K))
    sshape, sst = ((G, N), (1, G)) if group else ((N,), None)
    sc, b3 = _at_offset(m, sshape, x_dt, inp["scale"], o[2], 2, strides=sst)
    off, b4 = _at_offset(m, sshape, x_dt, inp["offset"], o[2], 2, strides=sst)
    d_y = cases.guarded_out(m, (M * N + o[3]) * 2)
    y = m.Tensor((M, N), x_dt, d_y, offset=o[3], storage_shape=(M * N + o[3],))
    plain(False)
    ws = m.weight_quant_batch_matmul(x, w, sc, y, offset=off, group_size=group)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    del ws
    got = d_y.to_host(np.uint16, (M * N + o[3],))
    assert (got[:o[3]] == 0xFFFF).all(), "wrote in front of the output view"
    check_close(got[o[3]:].reshape(M, N), want, x_dt, "weight-only at odd offsets")


@pytest.mark.parametrize("M,K,N", _shapes(122, 20, 300, 128, 4096, 128, 128, 1024))
@pytest.mark.parametrize("mode", ["block", "mxfp8"])
def test_fp8_operands_at_odd_offsets(gpu, M, K, N, mode):
    m = gpu
    o = [(1, 3, 1, 1, 1), (4, 8, 2, 0, 2), (16, 1, 0, 1, 4), (0, 16, 1, 1, 0), (5, 0, 0, 0, 1)][(M + K // 128 + N // 128) % 5]
    print(f"case sweep fp8 offsets {mode} M={M} K={K} N={N} offsets={o}", flush=True)
    if mode == "block":
        inp = cases.make_blockscale_inputs(m, M, K, N, M + N + K, True, 1)
        want = cases.oracle_blockscale(m, inp, M, K, N, True, m.ACL_BF16)[0]
        sdt, sb, gs = m.ACL_FLOAT, 4, (1 << 32) | (128 << 16) | 128
    else:
        inp = cases.make_mx_inputs(m, M, K, N, M + N + K, True, False)
        want = cases.oracle_mx(m, inp, M, K, N, True, m.ACL_BF16)[0]
        sdt, sb, gs = m.ACL_FLOAT8_E8M0, 1, (1 << 32) | (1 << 16) | 32
    x1, b1 = _at_offset(m, (M, K), m.ACL_FLOAT8_E4M3FN, inp["x1"][0], o[0], 1)
    x2, b2 = _at_offset(m, (N, K), m.ACL_FLOAT8_E4M3FN, inp["x2"][0], o[1], 1, storage_cols=K)
    s1, b3 = _at_offset(m, inp["s1"].shape[1:], sdt, inp["s1"][0], o[2], sb, storage_cols=inp["s1"].shape[-1] * (inp["s1"].shape[-2] if mode != "block" else 1))
    s2, b4 = _at_offset(m, inp["s2"].shape[1:], sdt, inp["s2"][0], o[3], sb, storage_cols=inp["s2"].shape[-1] * (inp["s2"].shape[-2] if mode != "block" else 1))
    d_out = cases.guarded_out(m, (M * N + o[4]) * 2)
    out = m.Tensor((M, N), m.ACL_BF16, d_out, offset=o[4], storage_shape=(M * N + o[4],))
    plain(False)
    ws = m.quant_matmul_v5(x1, x2, s1, s2, out, transpose_x2=True, group_size=gs)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    del ws
    got = d_out.to_host(np.uint16, (M * N + o[4],))
    assert (got[:o[4]] == 0xFFFF).all(), "wrote in front of the output view"
    _b16_bar(got[o[4]:].reshape(M, N), want, orc.BF16, f"fp8 {mode} at odd offsets", K)


# ---- a NaN row of x stays in its row: no kernel may multiply another row's x (a K tail read from the next row, a padded row
# block) into a result, not even with a zero weight ----
@pytest.mark.parametrize("M,K,N", _shapes(130, 28, 300, 8, 4096, 8, 64, 1024) + _shapes(131, 8, 300, 128, 8192, 32, 256, 1024))
@pytest.mark.parametrize("w_dt", ["i4", "i8"])
def test_weight_only_nan_row_stays_in_its_row(gpu, M, K, N, w_dt):
    m = gpu
    if M < 2:
        M = 2
    if w_dt == "i4":
        K += K % 2
    dt = {"i8": m.ACL_INT8, "i4": m.ACL_INT4}
    x_dt = m.ACL_FLOAT16 if (M + N) % 2 else m.ACL_BF16
    group = 128 if (M + K // 8) % 2 and K % 128 == 0 and K > 128 else 0
    print(f"case sweep weight-only NaN row M={M} K={K} N={N} w={w_dt} g={group}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M + K + N, x_dt, dt[w_dt], group, True, True, None)
    bad = sorted({M // 2, M - 1})
    clean = [r for r in range(M) if r not in bad]
    inp["x"][bad] = 0x7E00 if x_dt == m.ACL_FLOAT16 else 0x7FC0
    plain(False)
    got = cases.run_wq_aclnn(m, inp, M, K, N)
    g = orc.b16_to_f32(got, x_dt)
    assert np.isnan(g[bad]).all(), "a NaN row of x gave finite results"
    if clean:
        want = cases.oracle_wq(m, inp, M, K, N, rows=clean)
        check_close(got[clean], want, x_dt, "rows next to a NaN row")


@pytest.mark.parametrize("M,K,N", _shapes(132, 24, 300, 32, 4096, 8, 64, 1024) + _shapes(133, 6, 64, 128, 16384, 8, 256, 520))
@pytest.mark.parametrize("mode", ["block", "mxfp8", "mxfp4"])
def test_quant_modes_nan_row_stays_in_its_row(gpu, M, K, N, mode):
    m = gpu
    M = max(M, 2)
    bad = sorted({M // 2, M - 1})
    clean = [r for r in range(M) if r not in bad]
    print(f"case sweep {mode} NaN row M={M} K={K} N={N}", flush=True)
    plain(False)
    if mode == "block":
        inp = cases.make_blockscale_inputs(m, M, K, N, M + N + K, True, 1)
        inp["x1"][0, bad] = 0x7F   # e4m3 NaN
        got = cases.run_blockscale_aclnn(m, inp, M, K, N, True, m.ACL_BF16)[0]
        want = cases.oracle_blockscale(m, inp, M, K, N, True, m.ACL_BF16, rows=clean)[0] if clean else None
    else:
        inp = cases.make_mx_inputs(m, M, K, N, M + N + K, True, mode == "mxfp4")
        # MXFP4: an e8m0 NaN scale makes the whole block NaN (e2m1 has no NaN code of its own).  MXFP8: NaN elements (a NaN
        # scale would also send the whole call from the exact products to the scaled 8-bit instruction, whose bar is another)
        if mode == "mxfp4":
            inp["s1"][0, bad] = 0xFF
        else:
            inp["x1"][0, bad] = 0x7F
        got = cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16)[0]
        want = cases.oracle_mx(m, inp, M, K, N, True, m.ACL_BF16, rows=clean)[0] if clean else None
    g = orc.b16_to_f32(got, orc.BF16)
    assert np.isnan(g[bad]).all(), "a NaN row of x1 gave finite results"
    if clean:
        _b16_bar(got[clean], want, orc.BF16, f"{mode}: rows next to a NaN row", K)


@pytest.mark.parametrize("M,K,N", _shapes(134, 24, 300, 8, 4096, 8, 64, 1024) + _shapes(135, 8, 300, 128, 8192, 32, 256, 1024))
def test_weight_only_nan_scale_stays_in_its_column(gpu, M, K, N):
    """A NaN scale of one output column (all its groups) makes that column NaN and no other."""
    m = gpu
    x_dt = m.ACL_FLOAT16 if (M + N) % 2 else m.ACL_BF16
    w_dt = m.ACL_INT8 if (M + K // 8) % 2 else m.ACL_INT4
    if w_dt == m.ACL_INT4:
        K += K % 2
    group = 128 if (M + N // 8) % 2 and K % 128 == 0 and K > 128 else 0
    print(f"case sweep weight-only NaN scale column M={M} K={K} N={N} w={w_dt} g={group}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M + K + N, x_dt, w_dt, group, True, True, None)
    want = cases.oracle_wq(m, inp, M, K, N)
    bad = sorted({0, N // 3, N - 1})
    inp["scale"][bad] = 0x7E00 if x_dt == m.ACL_FLOAT16 else 0x7FC0
    plain(False)
    got = cases.run_wq_aclnn(m, inp, M, K, N)
    g = orc.b16_to_f32(got, x_dt)
    assert np.isnan(g[:, bad]).all(), "a NaN scale column gave finite results"
    keep = np.ones(N, bool); keep[bad] = False
    check_close(np.ascontiguousarray(got[:, keep]), np.ascontiguousarray(want[:, keep]), x_dt, "columns next to a NaN scale column")


@pytest.mark.parametrize("M,K,N", _shapes(136, 20, 300, 128, 4096, 8, 64, 1024) + _shapes(137, 6, 64, 128, 16384, 8, 256, 520))
@pytest.mark.parametrize("mode", ["int8", "fp8_kc", "pertile", "a8w4"])
def test_scaled_modes_nan_row_scale_stays_in_its_row(gpu, M, K, N, mode):
    """A NaN x1 scale of one row (a NaN x1 element for fp8 x fp4) makes that output row NaN and no other."""
    m = gpu
    M = max(M, 2)
    bad = sorted({M // 2, M - 1})
    clean = [r for r in range(M) if r not in bad]
    print(f"case sweep {mode} NaN row scale M={M} K={K} N={N}", flush=True)
    if mode == "int8":
        inp = cases.make_qmm_int8_inputs(m, M, K, N, M * 31 + N, m.ACL_BF16, True)
        inp["s1"][bad] = np.nan
        got = cases.run_qmm_int8_aclnn(m, inp, M, K, N, True, m.ACL_BF16)[0]
        want = cases.oracle_qmm_int8(m, inp, M, K, N, True, m.ACL_BF16)[0][0]
    elif mode == "fp8_kc":
        inp = cases.make_tc_inputs(m, M, K, N, M + N, m.ACL_FLOAT8_E4M3FN, m.ACL_FLOAT, N, m.ACL_FLOAT, True, pertoken="M")
        inp["pt"][bad] = np.nan
        got = cases.run_tc_aclnn(m, inp, M, K, N, m.ACL_BF16)
        want = cases.oracle_tc(m, inp, M, K, N, m.ACL_BF16)
    elif mode == "pertile":
        inp = cases.make_pertile_i8_inputs(m, M, K, N, M + N, True)
        inp["s1"][bad] = np.nan
        got = cases.run_pertile_i8_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
        want = cases.oracle_pertile_i8(m, inp, M, K, N, True, m.ACL_BF16)
    else:
        inp = cases.make_a8w4_mx_inputs(m, M, K, N, M + N, True)
        inp["x1"][bad] = 0x7F
        got = cases.run_a8w4_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16, bias_dt=orc.BF16)
        want = cases.oracle_a8w4_mx(m, inp, M, K, N, True, m.ACL_BF16, bias_dt=orc.BF16)
    g = orc.b16_to_f32(got, orc.BF16)
    assert np.isnan(g[bad]).all(), "a NaN row gave finite results"
    assert np.isnan(orc.b16_to_f32(want, orc.BF16)[bad]).all()
    if mode == "int8":
        assert np.array_equal(got[clean], want[clean]), f"{int((got[clean] != want[clean]).sum())} outputs of the other rows differ"
    else:
        _b16_bar(np.ascontiguousarray(got[clean]), np.ascontiguousarray(want[clean]), orc.BF16, f"{mode}: rows next to a NaN row", K)


# ---- the same call three times gives the same bits: partial sums are added in a fixed order, and a race (a missing barrier or
# wait) would show as a result that changes between runs while staying inside the tolerance of the comparisons above ----
@pytest.mark.parametrize("M,K,N", _shapes(140, 16, 300, 128, 4096, 32, 256, 1024) + _shapes(141, 8, 64, 128, 20480, 32, 256, 1024) +
                         _shapes(142, 4, 300, 128, 1536, 128, 16512, 20480))
@pytest.mark.parametrize("mode", ["wq_i4", "wq_i8", "wq_fp4", "block", "fp8_kc", "pertile", "a8w4", "mxfp8", "mxfp4", "tcg"])
def test_repeated_calls_are_bit_identical(gpu, M, K, N, mode):
    m = gpu
    print(f"case sweep repeat {mode} M={M} K={K} N={N}", flush=True)
    plain(False)
    if mode.startswith("wq_"):
        w_dt, group, off = {"wq_i4": (m.ACL_INT4, 128, True), "wq_i8": (m.ACL_INT8, 0, True), "wq_fp4": (m.ACL_FLOAT4_E2M1, 32, False)}[mode]
        if mode == "wq_i4" and K % 256:
            K += 128
        inp = cases.make_wq_inputs(m, M, K, N, M + K + N, m.ACL_BF16 if (M + N) % 2 else m.ACL_FLOAT16, w_dt, group if K > group else 0, True, off, None)
        run = lambda: cases.run_wq_aclnn(m, inp, M, K, N)
    elif mode == "block":
        inp = cases.make_blockscale_inputs(m, M, K, N, M + N + K, True, 1)
        run = lambda: cases.run_blockscale_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    elif mode == "fp8_kc":
        inp = cases.make_tc_inputs(m, M, K, N, M + N, m.ACL_FLOAT8_E4M3FN, m.ACL_FLOAT, N, m.ACL_FLOAT, True, pertoken="M")
        run = lambda: cases.run_tc_aclnn(m, inp, M, K, N, m.ACL_BF16)
    elif mode == "pertile":
        inp = cases.make_pertile_i8_inputs(m, M, K, N, M + N, True)
        run = lambda: cases.run_pertile_i8_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    elif mode == "a8w4":
        inp = cases.make_a8w4_mx_inputs(m, M, K, N, M + N, True)
        run = lambda: cases.run_a8w4_mx_aclnn(m, inp, M, K, N, True, m.ACL_FLOAT16)
    elif mode == "tcg":
        inp = cases.make_tcg_inputs(m, M, K, N, M + N, m.ACL_BF16)
        run = lambda: cases.run_tcg_aclnn(m, inp, M, K, N, m.ACL_BF16)
    else:
        inp = cases.make_mx_inputs(m, M, K, N, K + N + M, True, mode == "mxfp4")
        run = lambda: cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    first = run()
    for rep in (1, 2):
        m.check(m.lib().opsnnDebugFillLds(None), "opsnnDebugFillLds")
        again = run()
        assert np.array_equal(first.view(np.uint16), again.view(np.uint16)), f"run {rep + 1}: {int((first.view(np.uint16) != again.view(np.uint16)).sum())} of {first.size} outputs differ from the first run"
