"""aclnnDynamicMxQuant (MX quantizer of the fp4 / fp8 MX matmuls): oracle pins, phase-1 status cases, device parity.

The golden (quant/dynamic_mx_quant/tests/assets/golden.py:140-330) states the OCP MX conversion: shared exponent
floor(log2 max|x|) - emax, elements rounded to nearest even on the element grid and saturated.  The pins recompute that from
the definition -- torch's fp8 casts, and a brute-force nearest-grid-point search for e2m1 -- and add known answers.
Device bar: bit-identical elements (the sign of a zero result aside) and scale bytes.
"""
import numpy as np
import pytest

import oracle_api as orc

torch = pytest.importorskip("torch")
EMAX = {orc.E2M1: 2, orc.E4M3: 8, orc.E5M2: 15}
TMAX = {orc.E2M1: 6.0, orc.E4M3: 448.0, orc.E5M2: 57344.0}
GRID4 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])


def _codes(y, y_dt):
    return orc.unpack_nibbles(y) if y_dt == orc.E2M1 else y


def _definition(xf, y_dt):
    """[rows, cols] float32 (cols % 32 == 0) -> (element codes, scale bytes) from the MX definition, in float64."""
    rows, cols = xf.shape
    blk = xf.reshape(rows, cols // 32, 32).astype(np.float64)
    amax = np.abs(blk).max(axis=-1)
    with np.errstate(divide="ignore"):
        share = np.where(amax > 0, np.floor(np.log2(np.where(amax > 0, amax, 1.0))) - EMAX[y_dt], -127.0)
    share = np.maximum(share, -127.0)
    q = np.clip(blk / 2.0 ** share[..., None], -TMAX[y_dt], TMAX[y_dt]).reshape(rows, cols)
    if y_dt == orc.E2M1:
        # nearest grid point, ties to the even code (codes 0, 2, 4, 6 have a zero mantissa bit)
        d = np.abs(np.abs(q)[..., None] - GRID4)
        best = d.min(axis=-1, keepdims=True)
        cand = d == best
        code = np.where(cand.sum(-1) == 1, cand.argmax(-1), np.where(cand[..., ::2].any(-1), 2 * cand[..., ::2].argmax(-1), cand.argmax(-1)))
        codes = (code | np.where(np.signbit(q), 8, 0)).astype(np.uint8)
    else:
        tdt = torch.float8_e4m3fn if y_dt == orc.E4M3 else torch.float8_e5m2
        codes = torch.from_numpy(q.astype(np.float32)).to(tdt).view(torch.uint8).numpy()
    return codes, (share + 127).astype(np.uint8)


def _same_but_zero_sign(a, b, y_dt):
    mag = 0x7 if y_dt == orc.E2M1 else 0x7f
    z = ((a | b) & mag) == 0
    return np.array_equal(a[~z], b[~z])


# ------------------------------------------------------------------------------------------------ oracle pins (CPU)
@pytest.mark.parametrize("x_dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("y_dt", [orc.E2M1, orc.E4M3, orc.E5M2])
def test_against_the_mx_definition(x_dt, y_dt):
    rng = np.random.default_rng(y_dt)
    shape = (48, 256)
    xf = (rng.normal(0, 1, size=shape) * 2.0 ** rng.integers(-12, 12, size=(48, 8)).repeat(32, axis=1)).astype(np.float32)
    xb = orc.f32_to_b16(xf, x_dt)
    want_codes, want_scale = _definition(orc.b16_to_f32(xb, x_dt), y_dt)
    y, s = orc.dynamic_mx_quant(xb, x_dt, y_dt)
    assert np.array_equal(s.reshape(48, -1), want_scale)
    assert _same_but_zero_sign(_codes(y, y_dt), want_codes, y_dt)


def test_known_answers():
    """Block max 6 -> share_exp 0, scale byte 127, and the fp4 ties go to even: 0.25 -> 0, 0.75 -> 1, 1.25 -> 1, 1.75 -> 2,
    2.5 -> 2, 3.5 -> 4, 5 -> 4.  Block max 7 -> floor(log2 7) = 2, same scale, 7 saturates to 6.  Block max 448 * 2^-20 with e4m3:
    byte 107.  A zero block: byte 0 and zeros.  An odd number of blocks pads the scale row with byte 0.  A block with an infinity
    or a NaN: byte 0xFF and zeros."""
    x = np.zeros((1, 96), np.float32)
    x[0, :9] = [6.0, 0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.75]
    x[0, 32:34] = [7.0, -7.0]
    y, s = orc.dynamic_mx_quant(orc.f32_to_bf16(x), orc.BF16, orc.E2M1)
    c = orc.unpack_nibbles(y)[0]
    assert list(c[:9]) == [7, 0, 2, 2, 4, 4, 6, 6, 10] and list(c[32:34]) == [7, 15]
    assert s.shape == (1, 2, 2) and list(s.reshape(-1)) == [127, 127, 0, 0]
    x8 = np.zeros((2, 64), np.float32)
    x8[0, 0] = 448.0 * 2.0 ** -20
    x8[0, 32], x8[1, 5], x8[1, 40] = np.inf, np.nan, 3.0
    y, s = orc.dynamic_mx_quant(orc.f32_to_bf16(x8), orc.BF16, orc.E4M3)
    assert list(s.reshape(2, 2)[0]) == [107, 0xFF] and list(s.reshape(2, 2)[1]) == [0xFF, 127 + 1 - 8]
    assert y[0, 0] == 0x7e and not (y[0, 32:] & 0x7f).any() and not (y[1, :32] & 0x7f).any()
    assert y[1, 40] == orc.f32_to_e4m3(np.float32([3.0 * 2.0 ** 7]))[0]


def test_larger_blocks_take_the_larger_scale():
    """floor(log2 max) is monotone: a block of 64 has the larger of the scale bytes of its two halves, and the half that had
    that byte keeps its element codes."""
    rng = np.random.default_rng(4)
    xf = (rng.normal(0, 1, size=(32, 256)) * 2.0 ** rng.integers(-6, 6, size=(32, 8)).repeat(32, axis=1)).astype(np.float32)
    xb = orc.f32_to_bf16(xf)
    y32, s32 = orc.dynamic_mx_quant(xb, orc.BF16, orc.E4M3, block=32)
    y64, s64 = orc.dynamic_mx_quant(xb, orc.BF16, orc.E4M3, block=64)
    b32 = s32.reshape(32, 8)
    assert s64.shape == (32, 2, 2) and np.array_equal(s64.reshape(32, 4), np.maximum(b32[:, 0::2], b32[:, 1::2]))
    same = np.repeat(b32 == np.repeat(s64.reshape(32, 4), 2, axis=1), 32, axis=1)
    assert same.any() and np.array_equal(y32[same], y64[same])


def test_scale_algorithm_1_is_the_smallest_power_of_two_that_avoids_saturation():
    """max / 448 rounded up to a power of two: every scaled element fits (no code reaches beyond 448 and the block maximum is
    above 224 unless max / 448 is itself a power of two), and half the scale would not fit."""
    rng = np.random.default_rng(5)
    xf = (rng.normal(0, 1, size=(64, 128)) * 2.0 ** rng.integers(-10, 10, size=(64, 4)).repeat(32, axis=1)).astype(np.float32)
    xf[0, :32] = 0.0
    xf[1, :32] = 448.0 * 2.0 ** -3 * np.linspace(0, 1, 32)        # max / 448 is exactly a power of two: not rounded up
    xb = orc.f32_to_bf16(xf)
    xf = orc.b16_to_f32(xb, orc.BF16).astype(np.float64)
    y, s = orc.dynamic_mx_quant(xb, orc.BF16, orc.E4M3, scale_alg=1)
    scale = 2.0 ** (s.reshape(64, 4).astype(np.float64) - 127)
    amax = np.abs(xf).reshape(64, 4, 32).max(axis=-1)
    assert s.reshape(64, 4)[0, 0] == 0 and s.reshape(64, 4)[1, 0] == 127 - 3
    nz = amax > 0
    assert (amax[nz] <= 448.0 * scale[nz]).all() and (amax[nz] > 448.0 * scale[nz] / 2).all()
    deq = orc.e4m3_to_f32(y).astype(np.float64) * np.repeat(scale, 32, axis=1)
    assert (np.abs(deq - xf) <= np.maximum(np.abs(xf) * 2.0 ** -4, 2.0 ** -10 * np.repeat(scale, 32, axis=1))).all()   # never saturates


def test_dequantised_values_are_within_half_a_grid_step():
    """Relative 2^-4 (half a step of three mantissa bits), or 2^-3 where the block maximum saturates: a block maximum in
    (448, 512) * scale comes back as 448 * scale."""
    rng = np.random.default_rng(9)
    xb = orc.f32_to_bf16(rng.normal(0, 1, size=(64, 512)).astype(np.float32))
    xf = orc.b16_to_f32(xb, orc.BF16).astype(np.float64)
    y, s = orc.dynamic_mx_quant(xb, orc.BF16, orc.E4M3)
    deq = orc.e4m3_to_f32(y).astype(np.float64) * np.repeat(2.0 ** (s.reshape(64, -1).astype(np.float64) - 127), 32, axis=1)
    assert (np.abs(deq - xf) <= np.maximum(np.abs(xf) * 2.0 ** -3, 2.0 ** -9 * np.repeat(2.0 ** (s.reshape(64, -1).astype(np.float64) - 127), 32, axis=1))).all()


# ------------------------------------------------------------------------------------------- status cases (no GPU)
def _t(m, shape, dt):
    return m.Tensor(shape, dt, None)


def _status(m, x, y, sc, **kw):
    rc, ws, ex = m.dynamic_mx_quant_get_workspace(x, y, sc, **kw)
    if ex:
        m.lib().aclDestroyAclOpExecutor(ex)
    return rc


# ---- the general form: another axis, fp32 input, e1m2 elements, the other rounding modes
GRID_E1M2 = np.arange(8) / 4.0


def _nearest_on_grid(q, grid, mode):
    """q float64 inside the grid's range -> index of the grid point that `mode` selects, from the definition of the mode on
    the explicit list of magnitudes (floor / ceil / trunc: the neighbouring grid point in that direction; rint: nearest, ties to
    the even mantissa, i.e. the even index; round: nearest, ties away from zero).  Returns signed values."""
    full = np.concatenate([-grid[:0:-1], grid])   # ascending signed grid
    out = np.empty_like(q)
    for i, v in enumerate(q.reshape(-1)):
        lo = full[full <= v].max(); hi = full[full >= v].min()
        if mode == "floor": r = lo
        elif mode == "ceil": r = hi
        elif mode == "trunc": r = lo if v >= 0 else hi
        elif lo == hi: r = lo
        elif v - lo < hi - v: r = lo
        elif v - lo > hi - v: r = hi
        elif mode == "round": r = hi if v > 0 else lo
        else:   # rint: the candidate with an even index in the magnitude grid
            r = lo if int(np.where(grid == abs(lo))[0][0]) % 2 == 0 else hi
        out.reshape(-1)[i] = r
    return out


@pytest.mark.parametrize("y_dt,grid", [(orc.E2M1, GRID4), (orc.E1M2, GRID_E1M2)])
@pytest.mark.parametrize("mode", ["rint", "round", "floor", "ceil", "trunc"])
def test_round_modes_select_the_grid_point_their_definition_names(y_dt, grid, mode):
    """One block whose maximum is the format's largest power-of-two binade (share_exp 0, scale byte 127), so q = x: every
    element must land on the grid point that the mode's definition selects, ties included (multiples of 1/8 hit every tie)."""
    top = 6.0 if y_dt == orc.E2M1 else 1.75
    vals = np.concatenate([np.arange(-48, 49) / 8.0 * (top / 6.0), [top, -top, 0.3, -0.3, 0.26, -0.26, 0.74]]).astype(np.float32)
    vals = vals[np.abs(vals) <= top]
    for start in range(0, len(vals), 31):
        blk = np.zeros(32, np.float32)
        part = vals[start:start + 31]
        blk[:len(part)] = part
        blk[31] = top
        y, sc = orc.dynamic_mx_quant_general(blk, orc.F32, y_dt, round_mode=mode)
        assert sc.reshape(-1)[0] == 127
        codes = orc.unpack_nibbles(y)
        got = np.where(codes & 8, -1.0, 1.0) * grid[codes & 7]
        want = _nearest_on_grid(blk.astype(np.float64), grid, mode)
        assert np.array_equal(np.abs(got), np.abs(want)) and np.array_equal(got[want != 0], want[want != 0]), (mode, blk, got, want)


def test_e1m2_share_exponent_and_saturation():
    """e1m2: emax 0, so a block maximum in [2^k, 2^(k+1)) gives scale byte 127 + k; 1.9 * 2^k saturates at code 7 (1.75)."""
    for k in (-3, 0, 5):
        blk = np.zeros(32, np.float32); blk[0] = 1.9 * 2.0 ** k; blk[1] = -1.0 * 2.0 ** k; blk[2] = 0.13 * 2.0 ** k
        y, sc = orc.dynamic_mx_quant_general(blk, orc.F32, orc.E1M2)
        codes = orc.unpack_nibbles(y)
        assert sc.reshape(-1)[0] == 127 + k and codes[0] == 7 and codes[1] == (8 | 4) and codes[2] == 1   # 0.13 -> 0.25 (nearest)


@pytest.mark.parametrize("y_dt", [orc.E2M1, orc.E4M3])
def test_another_axis_is_the_last_axis_of_the_transposed_tensor(y_dt):
    rng = np.random.default_rng(5)
    x = (rng.normal(0, 1, size=(3, 70, 6)) * 2.0 ** rng.integers(-6, 6, size=(3, 1, 6))).astype(np.float32)
    xb = orc.f32_to_b16(x, orc.BF16)
    y, sc = orc.dynamic_mx_quant_general(xb, orc.BF16, y_dt, axis=1)
    xt = np.ascontiguousarray(xb.transpose(0, 2, 1))                         # [3, 6, 70]
    yt, sct = orc.dynamic_mx_quant(xt, orc.BF16, y_dt)                       # the pinned last-axis form
    ct = _codes(yt.reshape(-1), y_dt).reshape(3, 6, 70)
    assert np.array_equal(_codes(y.reshape(-1), y_dt).reshape(3, 70, 6), ct.transpose(0, 2, 1))
    assert sc.shape == (3, 2, 6, 2)                                          # 3 blocks of 32 -> 2 pairs; the pair's two bytes last
    assert np.array_equal(sc.transpose(0, 2, 1, 3).reshape(3, 6, 4), sct.reshape(3, 6, 4))
    # axis 0 as well, with a block of 64
    y0, sc0 = orc.dynamic_mx_quant_general(xb, orc.BF16, y_dt, axis=0, block=64)
    x0 = np.ascontiguousarray(xb.transpose(1, 2, 0))                         # [70, 6, 3]
    y0t, sc0t = orc.dynamic_mx_quant(np.concatenate([x0, np.zeros((70, 6, 1), np.uint16)], axis=-1) if y_dt == orc.E2M1 else x0, orc.BF16, y_dt, block=64)
    c0t = _codes(y0t.reshape(-1), y_dt).reshape(70, 6, -1)[..., :3]
    assert np.array_equal(_codes(y0.reshape(-1), y_dt).reshape(3, 70, 6), c0t.transpose(2, 0, 1))
    assert np.array_equal(sc0.reshape(70, 6, 2), sc0t.reshape(70, 6, 2))


@pytest.mark.parametrize("y_dt", [orc.E2M1, orc.E4M3, orc.E5M2])
def test_fp32_input_equals_the_16_bit_input_it_came_from(y_dt):
    rng = np.random.default_rng(8)
    xf = (rng.normal(0, 1, size=(9, 96)) * 2.0 ** rng.integers(-10, 10, size=(9, 1))).astype(np.float32)
    xh = orc.f32_to_b16(xf, orc.F16)
    y16, s16 = orc.dynamic_mx_quant(xh, orc.F16, y_dt)
    y32, s32 = orc.dynamic_mx_quant_general(orc.b16_to_f32(xh, orc.F16), orc.F32, y_dt)
    assert np.array_equal(y16, y32) and np.array_equal(s16, s32)


def test_status_rules(opsnn):
    """The documented rules (docs/aclnnDynamicMxQuant.md:99-260, 312-320) and its example call (:428-454: axis -1, rint,
    dstType 36, blocksize 32)."""
    m = opsnn
    bad, null, not_run = m.ACLNN_ERR_PARAM_INVALID, m.ACLNN_ERR_PARAM_NULLPTR, 561002
    f4, f8, e8 = m.ACL_FLOAT4_E2M1, m.ACL_FLOAT8_E4M3FN, m.ACL_FLOAT8_E8M0
    x, y, sc = _t(m, (4, 6, 320), m.ACL_BF16), _t(m, (4, 6, 320), f8), _t(m, (4, 6, 5, 2), e8)
    assert _status(m, x, y, sc) == 0 and _status(m, x, y, sc, round_mode=None) == 0
    assert _status(m, x, _t(m, (4, 6, 320), f4), sc) == 0
    assert _status(m, _t(m, (96,), m.ACL_FLOAT16), _t(m, (96,), m.ACL_FLOAT8_E5M2), _t(m, (2, 2), e8)) == 0
    assert _status(m, None, y, sc) == null and _status(m, x, None, sc) == null and _status(m, x, y, None) == null
    assert _status(m, _t(m, (4, 6, 320), m.ACL_INT8), y, sc) == bad
    assert _status(m, x, y, sc, dst_type=35) == bad and _status(m, x, _t(m, (4, 6, 320), m.ACL_INT8), sc, dst_type=2) == bad
    assert _status(m, x, y, _t(m, (4, 6, 5, 2), m.ACL_UINT8 if hasattr(m, "ACL_UINT8") else 4)) == bad
    assert _status(m, x, y, sc, round_mode=b"floor") == bad and _status(m, x, y, sc, round_mode=b"up") == bad
    assert _status(m, x, y, sc, blocksize=48) == bad and _status(m, x, y, sc, blocksize=2048) == bad and _status(m, x, y, sc, blocksize=0) == bad
    assert _status(m, x, y, sc, scale_alg=2) == bad and _status(m, x, _t(m, (4, 6, 320), f4), sc, scale_alg=1) == bad
    assert _status(m, x, y, sc, axis=3) == bad and _status(m, x, y, sc, axis=-4) == bad
    assert _status(m, x, _t(m, (4, 6, 160), f8), sc) == bad
    assert _status(m, _t(m, (4, 31), m.ACL_BF16), _t(m, (4, 31), f4), _t(m, (4, 1, 2), e8)) == bad     # fp4 needs an even last dim
    assert _status(m, x, y, _t(m, (4, 6, 10), e8)) == bad and _status(m, x, y, _t(m, (4, 6, 6, 2), e8)) == bad
    # V2 / V3: the added arguments at 0 are the first version
    assert _status(m, x, y, sc, dst_type_max=0.0) == 0 and _status(m, x, y, sc, dst_type_max=0.0, max_low_bound=0.0) == 0
    assert _status(m, x, y, sc, dst_type_max=6.0) == not_run and _status(m, x, y, sc, dst_type_max=0.0, max_low_bound=1.0) == not_run
    assert _status(m, x, y, sc, dst_type_max=0.0, scale_alg=2) == not_run and _status(m, x, y, sc, dst_type_max=0.0, blocksize=48) == bad
    # another axis, a FLOAT x, e1m2 elements and the fp4 rounding modes run on the general kernel
    assert _status(m, x, y, _t(m, (4, 1, 320, 2), e8), axis=1) == 0
    assert _status(m, x, y, _t(m, (4, 6, 3, 2), e8), blocksize=64) == 0
    assert _status(m, x, y, _t(m, (4, 6, 1, 2), e8), blocksize=1024) == 0
    assert _status(m, _t(m, (4, 6, 320), m.ACL_FLOAT), y, sc) == 0
    assert _status(m, _t(m, (4, 6, 320), m.ACL_FLOAT), y, _t(m, (4, 6, 3, 2), e8), blocksize=64) == bad     # FLOAT x: blocks of 32 only
    assert _status(m, x, _t(m, (4, 6, 320), m.ACL_FLOAT4_E1M2), sc) == 0
    assert _status(m, x, _t(m, (4, 6, 320), f4), sc, round_mode=b"floor") == 0
    assert _status(m, x, _t(m, (4, 6, 320), f4), sc, round_mode=b"round") == 0
    assert _status(m, x, _t(m, (4, 6, 320), f4), sc, round_mode=b"ceil") == bad
    assert _status(m, x, y, sc, scale_alg=1) == 0


# --------------------------------------------------------------------------------------------------- device parity
ACL_OF = {orc.E2M1: "ACL_FLOAT4_E2M1", orc.E4M3: "ACL_FLOAT8_E4M3FN", orc.E5M2: "ACL_FLOAT8_E5M2"}


def _run(m, xb, x_dt, y_dt, block=32, scale_alg=0):
    cols = xb.shape[-1]
    nblk = -(-cols // block)
    ybytes = xb.size // 2 if y_dt == orc.E2M1 else xb.size
    sbytes = xb.size // cols * ((nblk + 1) // 2) * 2
    d_x, d_y, d_s = m.DeviceBuffer(host=xb), m.DeviceBuffer(ybytes + 16), m.DeviceBuffer(sbytes + 16)
    d_y.fill(0xEE); d_s.fill(0xEE)
    adt = m.ACL_FLOAT16 if x_dt == orc.F16 else m.ACL_BF16
    sshape = xb.shape[:-1] + ((nblk + 1) // 2, 2)
    m.dynamic_mx_quant(m.Tensor(xb.shape, adt, d_x), m.Tensor(xb.shape, m.DTYPE_BY_NAME[ACL_OF[y_dt]], d_y), m.Tensor(sshape, m.ACL_FLOAT8_E8M0, d_s),
                       blocksize=block, scale_alg=scale_alg)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    gy, gs = d_y.to_host(np.uint8, (ybytes + 16,)), d_s.to_host(np.uint8, (sbytes + 16,))
    assert (gy[ybytes:] == 0xEE).all() and (gs[sbytes:] == 0xEE).all(), "wrote past an output"
    return gy[:ybytes], gs[:sbytes].reshape(sshape)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(16, 64), (33, 1024), (4, 8192), (3, 5, 320), (7, 40), (6, 1000), (5, 30), (2, 3, 4, 96), (4096,)])
@pytest.mark.parametrize("x_dt,y_dt", [(orc.BF16, orc.E2M1), (orc.F16, orc.E2M1), (orc.BF16, orc.E4M3), (orc.F16, orc.E5M2)])
def test_gpu_mx_quant_is_bit_identical(gpu, shape, x_dt, y_dt):
    m = gpu
    print(f"case mx quant {shape} x={x_dt} y={y_dt}", flush=True)
    rng = np.random.default_rng(sum(shape) + y_dt)
    xf = (rng.normal(0, 1, size=shape) * 2.0 ** rng.integers(-14, 14, size=shape[:-1] + (1,))).astype(np.float32)
    flat = xf.reshape(-1)
    flat[:min(40, flat.size // 2)] = 0.0
    flat[-1] = np.inf
    if flat.size > 200:
        flat[100] = np.nan
    xb = orc.f32_to_b16(xf, x_dt)
    want_y, want_s = orc.dynamic_mx_quant(xb, x_dt, y_dt)
    gy, gs = _run(m, xb, x_dt, y_dt)
    assert np.array_equal(gs, want_s), "scale bytes differ"
    assert _same_but_zero_sign(_codes(gy, y_dt), _codes(want_y.reshape(-1), y_dt), y_dt)


@pytest.mark.gpu
@pytest.mark.parametrize("fp4", [True, False])
def test_gpu_mx_quantised_operands_feed_the_mx_matmul(gpu, fp4):
    """bf16 activation and weight -> aclnnDynamicMxQuant -> aclnnQuantMatmulV5 (MX mode): the operands and the [.., K/64, 2]
    scale tensors are passed on as they come out; the product is the oracle's on the oracle's quantised operands (fp4
    products are exact in the matrix core, so identical; fp8 to the MX kernel's bar)."""
    import cases
    m = gpu
    M, K, N = 128, 512, 256
    y_dt = orc.E2M1 if fp4 else orc.E4M3
    rng = np.random.default_rng(12)
    xb = orc.f32_to_bf16(rng.normal(0, 1, size=(M, K)).astype(np.float32))
    wb = orc.f32_to_bf16(rng.normal(0, 0.05, size=(N, K)).astype(np.float32))
    gx, sx = _run(m, xb, orc.BF16, y_dt)
    gw, sw = _run(m, wb, orc.BF16, y_dt)
    ox, osx = orc.dynamic_mx_quant(xb, orc.BF16, y_dt)
    ow, osw = orc.dynamic_mx_quant(wb, orc.BF16, y_dt)
    assert np.array_equal(sx, osx) and np.array_equal(sw, osw)
    kb = K // 2 if fp4 else K
    inp = dict(x1=gx.reshape(1, M, kb), x2=gw.reshape(1, N, kb), s1=sx[None], s2=sw[None], fp4=fp4)
    want = cases.oracle_mx(m, dict(inp, x1=ox[None], x2=ow[None]), M, K, N, True, m.ACL_BF16)
    got = cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    g, w = orc.b16_to_f32(got, orc.BF16), orc.b16_to_f32(want, orc.BF16)
    mx, mean = orc.rel_err_stats(g, w)
    assert mx <= 2.0 ** -7 and mean <= 2.0 ** -10, f"max rel {mx:.3e} mean rel {mean:.3e}"


@pytest.mark.gpu
@pytest.mark.parametrize("shape,block,alg,y_dt", [((33, 1024), 64, 0, orc.E2M1), ((7, 1000), 128, 0, orc.E4M3), ((5, 4096), 1024, 0, orc.E5M2),
                                                  ((33, 1024), 32, 1, orc.E4M3), ((6, 1000), 32, 1, orc.E5M2), ((9, 520), 256, 1, orc.E4M3),
                                                  # the wave-per-512-elements kernel: several waves per row, a ragged last wave and
                                                  # block, an odd number of blocks, two pieces per lane (1024); a block that is not a
                                                  # power of two stays on the one-thread-per-block kernel
                                                  ((3, 2048), 512, 0, orc.E2M1), ((4, 1544), 64, 0, orc.E4M3), ((2, 3072), 1024, 0, orc.E2M1),
                                                  ((5, 2200), 1024, 1, orc.E4M3), ((6, 960), 96, 0, orc.E4M3)])
def test_gpu_block_sizes_and_scale_algorithm_1(gpu, shape, block, alg, y_dt):
    m = gpu
    print(f"case mx quant {shape} block={block} scale_alg={alg} y={y_dt}", flush=True)
    rng = np.random.default_rng(sum(shape) + block + alg)
    xf = (rng.normal(0, 1, size=shape) * 2.0 ** rng.integers(-14, 14, size=shape[:-1] + (1,))).astype(np.float32)
    xf.reshape(-1)[:40] = 0.0
    xf.reshape(-1)[-1] = np.inf
    xb = orc.f32_to_b16(xf, orc.BF16)
    want_y, want_s = orc.dynamic_mx_quant(xb, orc.BF16, y_dt, block=block, scale_alg=alg)
    gy, gs = _run(m, xb, orc.BF16, y_dt, block=block, scale_alg=alg)
    assert np.array_equal(gs, want_s), "scale bytes differ"
    assert _same_but_zero_sign(_codes(gy, y_dt), _codes(want_y.reshape(-1), y_dt), y_dt)


def _run_general(m, x, x_dt, y_dt, axis, block=32, scale_alg=0, round_mode="rint"):
    """x: uint16 bits or float32, any shape -> (y bytes flat, scale bytes in the API's shape) from the device."""
    ax = axis % x.ndim
    nblk = -(-x.shape[ax] // block)
    fp4 = y_dt in (orc.E2M1, orc.E1M2)
    ybytes = x.size // 2 if fp4 else x.size
    sshape = x.shape[:ax] + ((nblk + 1) // 2,) + x.shape[ax + 1:] + (2,)
    sbytes = int(np.prod(sshape))
    d_x, d_y, d_s = m.DeviceBuffer(host=x), m.DeviceBuffer(ybytes + 16), m.DeviceBuffer(sbytes + 16)
    d_y.fill(0xEE); d_s.fill(0xEE)
    adt = {orc.F16: m.ACL_FLOAT16, orc.BF16: m.ACL_BF16, orc.F32: m.ACL_FLOAT}[x_dt]
    ydt = {orc.E2M1: m.ACL_FLOAT4_E2M1, orc.E1M2: m.ACL_FLOAT4_E1M2, orc.E4M3: m.ACL_FLOAT8_E4M3FN, orc.E5M2: m.ACL_FLOAT8_E5M2}[y_dt]
    m.dynamic_mx_quant(m.Tensor(x.shape, adt, d_x), m.Tensor(x.shape, ydt, d_y), m.Tensor(sshape, m.ACL_FLOAT8_E8M0, d_s),
                       axis=axis, blocksize=block, scale_alg=scale_alg, round_mode=round_mode.encode())
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    gy, gs = d_y.to_host(np.uint8, (ybytes + 16,)), d_s.to_host(np.uint8, (sbytes + 16,))
    assert (gy[ybytes:] == 0xEE).all() and (gs[sbytes:] == 0xEE).all(), "wrote past an output"
    return gy[:ybytes], gs[:sbytes].reshape(sshape)


@pytest.mark.gpu
@pytest.mark.parametrize("shape,axis,x_dt,y_dt,block,alg,mode", [
    ((3, 70, 6), 1, orc.BF16, orc.E2M1, 32, 0, "rint"),        # a middle axis, three blocks (one pair and a half), fp4 pairs along the last axis
    ((100, 40), 0, orc.F16, orc.E4M3, 32, 0, "rint"),          # the first axis
    ((100, 40), 0, orc.BF16, orc.E5M2, 64, 1, "rint"),         # larger blocks and the second scale algorithm on another axis
    ((2, 96, 4, 10), -3, orc.BF16, orc.E2M1, 32, 0, "floor"),
    ((5, 320), -1, orc.F32, orc.E4M3, 32, 0, "rint"),          # FLOAT x
    ((5, 320), -1, orc.F32, orc.E2M1, 32, 0, "round"),
    ((7, 40), -1, orc.BF16, orc.E1M2, 32, 0, "rint"),          # e1m2 elements, a ragged last block
    ((7, 40), -1, orc.F16, orc.E1M2, 32, 0, "floor"),
    ((6, 1000), -1, orc.BF16, orc.E2M1, 32, 0, "floor"),       # the rounding modes of the 4-bit types on the last axis
    ((6, 1000), -1, orc.F16, orc.E2M1, 128, 0, "round"),
    ((64, 33, 2), 0, orc.F32, orc.E1M2, 32, 0, "round"),
    # inner extents of whole 16-byte pieces of a 16-bit x (the vector kernel: 8 columns and a pair of blocks per thread):
    # an odd number of blocks with a ragged last one, two outer slices, 4-bit and 8-bit elements
    ((130, 64), 0, orc.BF16, orc.E2M1, 32, 0, "rint"),
    ((2, 70, 16), 1, orc.F16, orc.E1M2, 32, 0, "round"),
    ((3, 200, 8), -2, orc.BF16, orc.E4M3, 64, 1, "rint"),
])
def test_gpu_general_form_is_bit_identical(gpu, shape, axis, x_dt, y_dt, block, alg, mode):
    """Blocks along another axis, fp32 input, e1m2 elements and the floor / round modes (the one-thread-per-block kernel)
    against the oracle, scale bytes and element codes (the sign of a zero aside).  fp32 inputs keep 12 mantissa bits, away
    from the values just below a power of two where numpy's float32 log2 rounds up to the next integer."""
    m = gpu
    print(f"case mx quant general {shape} axis={axis} x={x_dt} y={y_dt} block={block} alg={alg} mode={mode}", flush=True)
    rng = np.random.default_rng(sum(shape) + y_dt + block)
    ax = axis % len(shape)
    sc_shape = tuple(1 if i == ax else d for i, d in enumerate(shape))
    xf = (rng.normal(0, 1, size=shape) * 2.0 ** rng.integers(-14, 14, size=sc_shape)).astype(np.float32)
    flat = xf.reshape(-1)
    flat[:min(40, flat.size // 4)] = 0.0
    flat[-1] = np.inf
    flat[flat.size // 2] = np.nan
    if x_dt == orc.F32:
        x = (xf.view(np.uint32) & np.uint32(0xFFFFF800)).view(np.float32)
    else:
        x = orc.f32_to_b16(xf, x_dt)
    want_y, want_s = orc.dynamic_mx_quant_general(x, x_dt, y_dt, axis=axis, block=block, scale_alg=alg, round_mode=mode)
    gy, gs = _run_general(m, x, x_dt, y_dt, axis, block, alg, mode)
    assert np.array_equal(gs, want_s), "scale bytes differ"
    fp4 = y_dt in (orc.E2M1, orc.E1M2)
    a, b = (orc.unpack_nibbles(gy), orc.unpack_nibbles(want_y.reshape(-1))) if fp4 else (gy, want_y.reshape(-1))
    mag = 0x7 if fp4 else 0x7f
    z = ((a | b) & mag) == 0
    assert np.array_equal(a[~z], b[~z]), f"{int((a[~z] != b[~z]).sum())} element codes differ"
