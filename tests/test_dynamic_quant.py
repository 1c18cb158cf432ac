"""aclnnDynamicQuant / aclnnDynamicQuantV2 (per-token activation quantizer): oracle pins, phase-1 status cases, device parity.

Status cases: quant/dynamic_quant/tests/ut/op_host/op_api/test_aclnn_dynamic_quant.cpp:70-121 (the newest-SoC rows) plus the
rules of aclnn_dynamic_quant.cpp:136-328 one by one.  The golden (quant/dynamic_quant/tests/assets/golden.py:17-122) is numpy
float32 arithmetic, so the pins below are numpy float32 evaluations and hand-derived known answers that a plausible wrong
reading of it fails.  Device bar: bit-identical y, scale and offset.
"""
import numpy as np
import pytest

import oracle_api as orc

torch = pytest.importorskip("torch")


def _f16(a):
    return orc.f32_to_f16(np.asarray(a, np.float32))


# ------------------------------------------------------------------------------------------------ oracle pins (CPU)
def test_e5m2_encode_matches_torch():
    rng = np.random.default_rng(3)
    f = np.concatenate([rng.normal(0, 1, 50000) * 10.0 ** rng.integers(-6, 5, 50000), np.linspace(-60000, 60000, 100001),
                        [57344.0, 61439.9, 2.0 ** -16, 2.0 ** -17 * 1.001, 2.0 ** -17, 3 * 2.0 ** -17, 2.0 ** -14, 0.0]]).astype(np.float32)
    f = f[np.abs(f) < 61440.0]
    ref = torch.from_numpy(f).to(torch.float8_e5m2).view(torch.uint8).numpy()
    got = np.array([orc.lib().orc_e5m2_from_f32(float(v)) for v in f], np.uint8)
    assert np.array_equal(got & 0x7f, ref & 0x7f)
    nz = (got & 0x7f) != 0
    assert np.array_equal(got[nz] & 0x80, ref[nz] & 0x80)
    assert orc.lib().orc_e5m2_from_f32(61440.0) == 0x7c and orc.lib().orc_e5m2_from_f32(-1e9) == 0xfc   # overflow: infinity


def test_scale_is_max_times_the_fp32_reciprocal():
    """max|x| = 13: 13 * fp32(1/127) = 0x3dd1a346, whereas 13 / 127 = 0x3dd1a347.  max|x| = 127: the scale is exactly 1, so
    the row is rounded as it stands -- half to even: 2.5 -> 2, 3.5 -> 4, 0.5 -> 0, -0.5 -> 0, 126.5 -> 126, -1.5 -> -2."""
    x = _f16([[13.0, 1.0, -2.0, 0.0, 0, 0, 0, 0], [127.0, 2.5, 3.5, 0.5, -0.5, 126.5, -1.5, -127.0]])
    y, scale = orc.dynamic_quant(x, orc.F16, orc.I8)
    assert scale.view(np.uint32)[0] == 0x3dd1a346 and scale[1] == 1.0
    assert list(y[1].view(np.int8)) == [127, 2, 4, 0, 0, 126, -2, -127]
    assert list(y[0].view(np.int8)) == [127, 10, -20, 0, 0, 0, 0, 0]   # 1 / (13 * r) = 9.77, 2 / (13 * r) = 19.54


def test_smooth_product_is_fp32():
    """(1 + 2^-10)^2 = 1 + 2^-9 + 2^-20 needs 21 bits: exact in fp32, rounded to 1 + 2^-9 in fp16.  The scale tells."""
    a = np.float32(1 + 2.0 ** -10)
    x, sm = _f16([[a, 0.5]]), _f16([a, 1.0])
    _, scale = orc.dynamic_quant(x, orc.F16, orc.I8, smooth=sm)
    r = np.float32(1.0) / np.float32(127.0)
    assert scale[0] == np.float32(1 + 2.0 ** -9 + 2.0 ** -20) * r != np.float32(1 + 2.0 ** -9) * r


def _numpy_golden(xf, smooth, tmax, tmax2, symmetric):
    """The golden's float32 steps for the integer types, written with numpy float32 arrays (its own arithmetic)."""
    v = xf * smooth if smooth is not None else xf
    if symmetric:
        scale = np.max(np.abs(v), axis=-1, keepdims=True) * (np.float32(1.0) / np.float32(tmax))
        return np.round(v / scale), scale.squeeze(-1), None
    vmax, vmin = np.max(v, axis=-1, keepdims=True), np.min(v, axis=-1, keepdims=True)
    scale = (vmax - vmin) * (np.float32(1.0) / np.float32(tmax2))
    offset = np.float32(tmax) - vmax / scale
    return np.round(v / scale + offset), scale.squeeze(-1), offset.squeeze(-1)


@pytest.mark.parametrize("x_dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("y_dt,tmax,tmax2", [(orc.I8, 127, 255), (orc.I4, 7, 15)])
@pytest.mark.parametrize("symmetric,with_smooth", [(True, False), (True, True), (False, False), (False, True)])
def test_integer_outputs_against_numpy_float32(x_dt, y_dt, tmax, tmax2, symmetric, with_smooth):
    rng = np.random.default_rng(11)
    xb = orc.f32_to_b16(rng.normal(0, 2, size=(3, 17, 96)).astype(np.float32), x_dt)
    smb = orc.f32_to_b16(rng.uniform(0.5, 2.0, 96).astype(np.float32), x_dt) if with_smooth else None
    xf = orc.b16_to_f32(xb, x_dt)
    want_y, want_s, want_o = _numpy_golden(xf, orc.b16_to_f32(smb, x_dt) if with_smooth else None, tmax, tmax2, symmetric)
    out = orc.dynamic_quant(xb, x_dt, y_dt, smooth=smb, symmetric=symmetric)
    y = out[0].view(np.int8).astype(np.int32) if y_dt == orc.I8 else orc.unpack_nibbles(out[0]).astype(np.int32)
    if y_dt == orc.I4:
        y = np.where(y >= 8, y - 16, y)
    assert np.array_equal(y, want_y.astype(np.int32))
    assert np.array_equal(out[1].view(np.uint32), want_s.view(np.uint32))
    if not symmetric:
        assert np.array_equal(out[2].view(np.uint32), want_o.view(np.uint32))
        assert y.min() == -tmax - 1 and y.max() == tmax            # the row's extremes land on the type's


@pytest.mark.parametrize("y_dt,tdt", [(orc.E4M3, "float8_e4m3fn"), (orc.E5M2, "float8_e5m2")])
def test_fp8_outputs_against_torch_cast(y_dt, tdt):
    rng = np.random.default_rng(5)
    xb = orc.f32_to_b16(rng.normal(0, 1, size=(40, 64)).astype(np.float32), orc.BF16)
    xf = orc.b16_to_f32(xb, orc.BF16)
    tmax = np.float32(448.0 if y_dt == orc.E4M3 else 57344.0)
    scale = np.max(np.abs(xf), axis=-1, keepdims=True) * (np.float32(1.0) / tmax)
    want = torch.from_numpy(xf / scale).to(getattr(torch, tdt)).view(torch.uint8).numpy()
    y, s = orc.dynamic_quant(xb, orc.BF16, y_dt)
    assert np.array_equal(s.view(np.uint32), scale.squeeze(-1).view(np.uint32))
    assert np.array_equal(y & 0x7f, want & 0x7f) and (y & 0x7f).max() == (0x7e if y_dt == orc.E4M3 else 0x7b)


def test_dequantised_rows_are_within_half_a_step():
    rng = np.random.default_rng(2)
    xb = orc.f32_to_b16(rng.normal(0, 3, size=(64, 200)).astype(np.float32), orc.F16)
    xf = orc.b16_to_f32(xb, orc.F16).astype(np.float64)
    y, s = orc.dynamic_quant(xb, orc.F16, orc.I8)
    assert (np.abs(y.view(np.int8) * s[:, None].astype(np.float64) - xf) <= 0.5001 * s[:, None]).all()
    y, s, o = orc.dynamic_quant(xb, orc.F16, orc.I8, symmetric=False)
    assert (np.abs((y.view(np.int8) - o[:, None].astype(np.float64)) * s[:, None] - xf) <= 0.51 * s[:, None]).all()


def test_group_index_selects_the_smooth_row():
    """Rows [0, 3) use expert 0's factors, expert 1 owns no rows (its end equals expert 0's), rows [3, 7) use expert 2's: equal to
    quantising each slice with its own smooth vector.  Rows from 7 on are left untouched."""
    rng = np.random.default_rng(8)
    xb = orc.f32_to_b16(rng.normal(0, 1, size=(9, 64)).astype(np.float32), orc.F16)
    smb = orc.f32_to_b16(rng.uniform(0.5, 2.0, size=(3, 64)).astype(np.float32), orc.F16)
    y, s = orc.dynamic_quant(xb, orc.F16, orc.I8, smooth=smb, group_end=[3, 3, 7], fill=0xEE)
    y0, s0 = orc.dynamic_quant(xb[:3], orc.F16, orc.I8, smooth=smb[0])
    y2, s2 = orc.dynamic_quant(xb[3:7], orc.F16, orc.I8, smooth=smb[2])
    assert np.array_equal(y[:3], y0) and np.array_equal(y[3:7], y2) and np.array_equal(s[:3], s0) and np.array_equal(s[3:7], s2)
    assert (y[7:] == 0xEE).all() and (s[7:].view(np.uint8) == 0xEE).all()


@pytest.mark.parametrize("mode", ["pertensor", "perchannel"])
@pytest.mark.parametrize("symmetric,with_smooth", [(True, False), (False, True)])
def test_wide_modes_against_numpy_float32(mode, symmetric, with_smooth):
    """quant/dynamic_quant/tests/assets/golden.py:66-94 with quant_mode "pertensor" (the maxima over everything) and :125-176
    (_dynamic_quant_perchannel: maxima over axis -2, smooth_scales[:, None]), in numpy float32 as the golden computes them."""
    rng = np.random.default_rng(13)
    shape = (3, 20, 48)
    xb = orc.f32_to_b16(rng.normal(0, 2, size=shape).astype(np.float32), orc.BF16)
    xf = orc.b16_to_f32(xb, orc.BF16)
    n_sm = 48 if mode == "pertensor" else 20
    smb = orc.f32_to_b16(rng.uniform(0.5, 2.0, n_sm).astype(np.float32), orc.BF16) if with_smooth else None
    smf = orc.b16_to_f32(smb, orc.BF16) if with_smooth else None
    v = xf if smf is None else (xf * smf if mode == "pertensor" else xf * smf[:, None])
    red = dict(axis=None) if mode == "pertensor" else dict(axis=-2, keepdims=True)
    if symmetric:
        scale = np.max(np.abs(v), **red) * (np.float32(1.0) / np.float32(127.0))
        want_y, want_o = np.round(v / scale), None
    else:
        vmax, vmin = np.max(v, **red), np.min(v, **red)
        scale = (vmax - vmin) * (np.float32(1.0) / np.float32(255.0))
        want_o = np.float32(127.0) - vmax / scale
        want_y = np.round(v / scale + want_o)
    out = orc.dynamic_quant_wide(xb, orc.BF16, orc.I8, mode, smooth=smb, symmetric=symmetric)
    assert np.array_equal(out[0].view(np.int8).astype(np.int32), want_y.astype(np.int32))
    assert np.array_equal(out[1].reshape(-1).view(np.uint32), np.asarray(scale, np.float32).reshape(-1).view(np.uint32))
    if not symmetric:
        assert np.array_equal(out[2].reshape(-1).view(np.uint32), np.asarray(want_o, np.float32).reshape(-1).view(np.uint32))


def test_rows_without_range_give_zeros():
    """Not the golden's behaviour (it divides by zero there): the convention of this build, see the oracle's header."""
    x = _f16([[0.0] * 8, [1.0] * 8])
    y, s = orc.dynamic_quant(x, orc.F16, orc.I8)
    assert s[0] == 0 and not y[0].any() and (y[1].view(np.int8) == 127).all()
    y, s, o = orc.dynamic_quant(x, orc.F16, orc.I8, symmetric=False)
    assert not s.any() and not o.any() and not y.any()


# ------------------------------------------------------------------------------------------- status cases (no GPU)
def _t(m, shape, dt):
    return m.Tensor(shape, dt, None)


def _status(m, x, y, sc, **kw):
    rc, ws, ex = m.dynamic_quant_get_workspace(x, y, sc, **kw)
    if ex:
        m.lib().aclDestroyAclOpExecutor(ex)
    return rc


def test_status_cases_of_the_reference_unit_test(opsnn):
    m = opsnn
    ok, bad = m.ACLNN_SUCCESS, m.ACLNN_ERR_PARAM_INVALID
    # fp16 -> int8 with smooth scales: success (:70-81)
    assert _status(m, _t(m, (16, 32), m.ACL_FLOAT16), _t(m, (16, 32), m.ACL_INT8), _t(m, (16,), m.ACL_FLOAT),
                   smooth=_t(m, (32,), m.ACL_FLOAT16)) == ok
    # bf16 -> int4 with an odd last dim: invalid (:96-107)
    assert _status(m, _t(m, (16, 31), m.ACL_BF16), _t(m, (16, 31), m.ACL_INT4), _t(m, (16,), m.ACL_FLOAT),
                   smooth=_t(m, (31,), m.ACL_BF16)) == bad
    # bf16 -> int32 carrier [16, 4]: success (:110-121)
    assert _status(m, _t(m, (16, 32), m.ACL_BF16), _t(m, (16, 4), m.ACL_INT32), _t(m, (16,), m.ACL_FLOAT),
                   smooth=_t(m, (32,), m.ACL_BF16)) == ok


def test_status_rules_one_by_one(opsnn):
    m = opsnn
    bad, null = m.ACLNN_ERR_PARAM_INVALID, m.ACLNN_ERR_PARAM_NULLPTR
    x, y, sc = _t(m, (4, 6, 32), m.ACL_BF16), _t(m, (4, 6, 32), m.ACL_INT8), _t(m, (4, 6), m.ACL_FLOAT)
    assert _status(m, x, y, sc) == 0
    assert _status(m, None, y, sc) == null and _status(m, x, None, sc) == null and _status(m, x, y, None) == null
    assert _status(m, _t(m, (4, 6, 32), m.ACL_FLOAT), y, sc) == bad                                   # x dtype
    assert _status(m, x, y, sc, smooth=_t(m, (32,), m.ACL_FLOAT16)) == bad                            # smooth dtype != x dtype
    assert _status(m, x, y, sc, smooth=_t(m, (1, 32), m.ACL_BF16)) == bad                             # smooth rank
    assert _status(m, x, y, sc, smooth=_t(m, (16,), m.ACL_BF16)) == bad                               # smooth length
    assert _status(m, x, _t(m, (4, 6, 32), m.DTYPE_BY_NAME["ACL_INT16"]), sc) == bad                                   # y dtype
    assert _status(m, x, _t(m, (4, 6, 16), m.ACL_INT8), sc) == bad                                    # y shape
    assert _status(m, x, _t(m, (4, 6, 8), m.ACL_INT32), sc) == bad                                    # int32 carrier: 32 / 8 = 4
    assert _status(m, x, y, _t(m, (4, 6), m.ACL_FLOAT16)) == bad                                      # scale dtype
    assert _status(m, x, y, _t(m, (24,), m.ACL_FLOAT)) == bad                                         # scale shape
    assert _status(m, _t(m, (32,), m.ACL_BF16), _t(m, (32,), m.ACL_INT8), _t(m, (1,), m.ACL_FLOAT)) == bad   # 1-D x
    assert _status(m, x, y, sc, offset=_t(m, (4, 6), m.ACL_FLOAT)) == 0                               # V2, asymmetric
    assert _status(m, x, y, sc, offset=_t(m, (4, 6), m.ACL_FLOAT16)) == bad
    assert _status(m, x, y, sc, offset=_t(m, (6, 4), m.ACL_FLOAT)) == bad
    for dt in (m.ACL_INT4, m.ACL_FLOAT8_E4M3FN, m.ACL_FLOAT8_E5M2):
        assert _status(m, x, _t(m, (4, 6, 32), dt), sc) == 0
    # empty x: success, nothing to run (:366-371)
    assert _status(m, _t(m, (0, 32), m.ACL_BF16), _t(m, (0, 32), m.ACL_INT8), _t(m, (0,), m.ACL_FLOAT)) == 0
    # accepted by the reference, no kernel here
    assert _status(m, x, _t(m, (4, 6, 32), m.ACL_HIFLOAT8), sc) == m.STATUS_BY_NAME.get("ACLNN_ERR_INNER_TILING_ERROR", 561002)
    # per-expert smooth scales (V2): smoothScales [experts, cols] with groupIndex [experts]
    assert _status(m, x, y, sc, smooth=_t(m, (2, 32), m.ACL_BF16), group_index=_t(m, (2,), m.ACL_INT32)) == 0
    assert _status(m, x, y, sc, smooth=_t(m, (2, 32), m.ACL_BF16), group_index=_t(m, (2,), m.ACL_INT64)) == 0
    assert _status(m, x, y, sc, smooth=_t(m, (2, 32), m.ACL_BF16), group_index=_t(m, (2,), m.ACL_FLOAT)) == bad
    assert _status(m, x, y, sc, smooth=_t(m, (2, 32), m.ACL_BF16), group_index=_t(m, (1, 2), m.ACL_INT32)) == bad
    assert _status(m, x, y, sc, smooth=_t(m, (3, 32), m.ACL_BF16), group_index=_t(m, (2,), m.ACL_INT32)) == bad
    assert _status(m, x, y, sc, smooth=_t(m, (32,), m.ACL_BF16), group_index=_t(m, (2,), m.ACL_INT32)) == bad
    assert _status(m, x, y, sc, group_index=_t(m, (2,), m.ACL_INT32)) == bad                        # groupIndex needs smoothScales


def test_v3_v4_attribute_rules(opsnn):
    """aclnn_dynamic_quant.cpp:171-189 and the mode-dependent scale shapes :258-284; (quant/dynamic_quant/tests/ut/op_host/op_api/test_aclnn_dynamic_quant_v3.cpp:71-90
    is the per-tensor shape of scale and offset)."""
    m = opsnn
    bad, not_run = m.ACLNN_ERR_PARAM_INVALID, 561002
    x, y, sc, off = _t(m, (16, 32), m.ACL_BF16), _t(m, (16, 32), m.ACL_INT8), _t(m, (16,), m.ACL_FLOAT), _t(m, (16,), m.ACL_FLOAT)
    assert _status(m, x, y, sc, quant_mode=b"pertoken") == 0
    assert _status(m, x, y, sc, offset=off, quant_mode=b"pertoken") == 0
    assert _status(m, x, y, sc, quant_mode=b"pertoken", dst_type_max=0.0) == 0
    assert _status(m, x, y, sc, offset=off, quant_mode=b"pertoken", is_symmetrical=True) == bad
    assert _status(m, x, y, sc, quant_mode=b"pertoken", is_symmetrical=False) == bad
    assert _status(m, x, y, sc, quant_mode=b"perrow") == bad
    one = _t(m, (1,), m.ACL_FLOAT)
    assert _status(m, x, y, one, offset=_t(m, (1,), m.ACL_FLOAT), quant_mode=b"pertensor") == 0
    assert _status(m, x, y, sc, quant_mode=b"pertensor") == bad                                            # scale must be [1]
    assert _status(m, x, y, _t(m, (32,), m.ACL_FLOAT), quant_mode=b"perchannel") == 0
    assert _status(m, x, y, sc, quant_mode=b"perchannel") == bad                                           # scale must be [32]
    assert _status(m, x, y, _t(m, (32,), m.ACL_FLOAT), quant_mode=b"perchannel", smooth=_t(m, (16,), m.ACL_BF16)) == 0
    assert _status(m, x, y, one, quant_mode=b"pertensor", smooth=_t(m, (2, 32), m.ACL_BF16), group_index=_t(m, (2,), m.ACL_INT32)) == not_run
    assert _status(m, x, y, _t(m, (32,), m.ACL_FLOAT), quant_mode=b"perchannel", smooth=_t(m, (32,), m.ACL_BF16)) == bad
    assert _status(m, x, y, _t(m, (32,), m.ACL_FLOAT), quant_mode=b"perchannel", smooth=_t(m, (2, 32), m.ACL_BF16),
                   group_index=_t(m, (2,), m.ACL_INT32)) == bad
    assert _status(m, x, y, sc, quant_mode=b"pertoken", dst_type_max=100.0) == not_run


# --------------------------------------------------------------------------------------------------- device parity
ACL_OF = {orc.I8: "ACL_INT8", orc.I4: "ACL_INT4", orc.E4M3: "ACL_FLOAT8_E4M3FN", orc.E5M2: "ACL_FLOAT8_E5M2"}


def _run(m, xb, x_dt, y_dt, smb, symmetric, carrier_int32=False):
    shape = xb.shape
    cols = shape[-1]
    d_x = m.DeviceBuffer(host=xb)
    d_sm = m.DeviceBuffer(host=smb) if smb is not None else None
    ybytes = xb.size // 2 if y_dt == orc.I4 else xb.size
    d_y, d_s, d_o = m.DeviceBuffer(ybytes + 16), m.DeviceBuffer(xb.size // cols * 4 + 16), m.DeviceBuffer(xb.size // cols * 4 + 16)
    for b in (d_y, d_s, d_o):
        b.fill(0xEE)
    adt = m.ACL_FLOAT16 if x_dt == orc.F16 else m.ACL_BF16
    x = m.Tensor(shape, adt, d_x)
    if carrier_int32:
        y = m.Tensor(shape[:-1] + (cols // 8,), m.ACL_INT32, d_y)
    else:
        y = m.Tensor(shape, m.DTYPE_BY_NAME[ACL_OF[y_dt]], d_y)
    sc = m.Tensor(shape[:-1], m.ACL_FLOAT, d_s)
    off = None if symmetric else m.Tensor(shape[:-1], m.ACL_FLOAT, d_o)
    sm = m.Tensor((cols,), adt, d_sm) if smb is not None else None
    m.dynamic_quant(x, y, sc, smooth=sm, offset=off)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    nrow = xb.size // cols
    gy = d_y.to_host(np.uint8, (ybytes + 16,))
    gs = d_s.to_host(np.uint8, (nrow * 4 + 16,))
    go = d_o.to_host(np.uint8, (nrow * 4 + 16,))
    assert (gy[ybytes:] == 0xEE).all() and (gs[nrow * 4:] == 0xEE).all(), "wrote past an output"
    return gy[:ybytes], gs[:nrow * 4].view(np.float32), go[:nrow * 4].view(np.float32)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(16, 32), (5, 7, 256), (33, 2048), (9, 4096), (3, 16384), (6, 31), (4, 20000), (2, 3, 1000)])
@pytest.mark.parametrize("x_dt,y_dt,symmetric,with_smooth", [
    (orc.F16, orc.I8, True, False), (orc.BF16, orc.I8, True, True), (orc.BF16, orc.I8, False, True), (orc.F16, orc.I4, True, True),
    (orc.BF16, orc.I4, False, False), (orc.BF16, orc.E4M3, True, False), (orc.F16, orc.E5M2, True, True), (orc.F16, orc.E4M3, False, False)])
def test_gpu_dynamic_quant_is_bit_identical(gpu, shape, x_dt, y_dt, symmetric, with_smooth):
    m = gpu
    if y_dt == orc.I4 and shape[-1] % 2:
        pytest.skip("INT4 needs an even last dim")
    print(f"case dynamic quant {shape} x={x_dt} y={y_dt} symmetric={symmetric} smooth={with_smooth}", flush=True)
    rng = np.random.default_rng(sum(shape) + y_dt)
    xf = rng.normal(0, 2, size=shape).astype(np.float32)
    xf.reshape(-1, shape[-1])[0] = 0.0                         # a row without range
    xb = orc.f32_to_b16(xf, x_dt)
    smb = orc.f32_to_b16(rng.uniform(0.5, 2.0, shape[-1]).astype(np.float32), x_dt) if with_smooth else None
    want = orc.dynamic_quant(xb, x_dt, y_dt, smooth=smb, symmetric=symmetric)
    gy, gs, go = _run(m, xb, x_dt, y_dt, smb, symmetric)
    assert np.array_equal(gs.view(np.uint32), want[1].reshape(-1).view(np.uint32)), "scale differs"
    if not symmetric:
        assert np.array_equal(go.view(np.uint32), want[2].reshape(-1).view(np.uint32)), "offset differs"
    wy = want[0].reshape(-1)
    if y_dt in (orc.E4M3, orc.E5M2):                            # the sign of a zero result is not pinned
        z = ((gy | wy) & 0x7f) == 0
        assert np.array_equal(gy[~z], wy[~z]), f"{int((gy[~z] != wy[~z]).sum())} outputs differ"
    else:
        assert np.array_equal(gy, wy), f"{int((gy != wy).sum())} of {wy.size} outputs differ"


@pytest.mark.gpu
def test_gpu_int32_carrier_holds_the_int4_bytes(gpu):
    m = gpu
    rng = np.random.default_rng(1)
    xb = orc.f32_to_b16(rng.normal(0, 1, size=(12, 64)).astype(np.float32), orc.BF16)
    want = orc.dynamic_quant(xb, orc.BF16, orc.I4)
    gy, gs, _ = _run(m, xb, orc.BF16, orc.I4, None, True, carrier_int32=True)
    assert np.array_equal(gy, want[0].reshape(-1)) and np.array_equal(gs, want[1])


@pytest.mark.gpu
def test_gpu_quantised_activation_feeds_the_int8_matmul(gpu):
    """The chain the op exists for: bf16 activation -> aclnnDynamicQuant -> aclnnQuantMatmulV5 (K-C: x1Scale = the per-token
    scale) equals the oracle's matmul on the oracle's quantised activation, bit for bit."""
    import cases
    m = gpu
    M, K, N = 96, 512, 256
    rng = np.random.default_rng(4)
    xb = orc.f32_to_b16(rng.normal(0, 1, size=(M, K)).astype(np.float32), orc.BF16)
    q, s1 = orc.dynamic_quant(xb, orc.BF16, orc.I8)
    inp = cases.make_qmm_int8_inputs(m, M, K, N, 3, m.ACL_BF16, True)
    inp = dict(inp, x1=q.view(np.int8).reshape(1, M, K), s1=s1)
    want, _ = cases.oracle_qmm_int8(m, inp, M, K, N, True, m.ACL_BF16)
    d_x, d_q, d_s = m.DeviceBuffer(host=xb), m.DeviceBuffer(M * K), m.DeviceBuffer(M * 4)
    m.dynamic_quant(m.Tensor((M, K), m.ACL_BF16, d_x), m.Tensor((M, K), m.ACL_INT8, d_q), m.Tensor((M,), m.ACL_FLOAT, d_s))
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    inp_dev = dict(inp, x1=d_q.to_host(np.int8, (1, M, K)), s1=d_s.to_host(np.float32, (M,)))
    got = cases.run_qmm_int8_aclnn(m, inp_dev, M, K, N, True, m.ACL_BF16)
    assert np.array_equal(got, want)


@pytest.mark.gpu
def test_gpu_v3_and_v4_pertoken_equal_v1(gpu):
    m = gpu
    rng = np.random.default_rng(6)
    xb = orc.f32_to_b16(rng.normal(0, 1, size=(40, 512)).astype(np.float32), orc.F16)
    want_y, want_s = orc.dynamic_quant(xb, orc.F16, orc.I8)
    d_x = m.DeviceBuffer(host=xb)
    for kw in (dict(quant_mode=b"pertoken"), dict(quant_mode=b"pertoken", dst_type_max=0.0)):
        d_y, d_s = m.DeviceBuffer(xb.size), m.DeviceBuffer(40 * 4)
        m.dynamic_quant(m.Tensor((40, 512), m.ACL_FLOAT16, d_x), m.Tensor((40, 512), m.ACL_INT8, d_y), m.Tensor((40,), m.ACL_FLOAT, d_s), **kw)
        m.check(m.lib().aclrtSynchronizeDevice(), "sync")
        assert np.array_equal(d_y.to_host(np.uint8, (40, 512)), want_y) and np.array_equal(d_s.to_host(np.float32, (40,)), want_s)


@pytest.mark.gpu
@pytest.mark.parametrize("shape,ends,gi_dt,symmetric", [((40, 256), [5, 5, 17, 40], "i32", True), ((3, 11, 4096), [10, 20, 30], "i64", False),
                                                       ((9, 1000), [2, 9], "i32", True), ((6, 20000), [1, 4], "i64", True)])
def test_gpu_group_index(gpu, shape, ends, gi_dt, symmetric):
    """aclnnDynamicQuantV2 with per-expert smooth scales, on the register-resident and the two-pass kernels; rows past the last
    expert's end keep what was in the output buffers."""
    m = gpu
    print(f"case dynamic quant groups {shape} ends={ends} {gi_dt} symmetric={symmetric}", flush=True)
    rng = np.random.default_rng(sum(shape))
    cols, rows = shape[-1], int(np.prod(shape[:-1]))
    xb = orc.f32_to_b16(rng.normal(0, 2, size=shape).astype(np.float32), orc.BF16)
    smb = orc.f32_to_b16(rng.uniform(0.5, 2.0, size=(len(ends), cols)).astype(np.float32), orc.BF16)
    want = orc.dynamic_quant(xb, orc.BF16, orc.I8, smooth=smb, symmetric=symmetric, group_end=ends, fill=0xEE)
    gi = np.array(ends, np.int32 if gi_dt == "i32" else np.int64)
    d_x, d_sm, d_gi = m.DeviceBuffer(host=xb), m.DeviceBuffer(host=smb), m.DeviceBuffer(host=gi)
    d_y, d_s, d_o = m.DeviceBuffer(xb.size), m.DeviceBuffer(rows * 4), m.DeviceBuffer(rows * 4)
    for b in (d_y, d_s, d_o):
        b.fill(0xEE)
    off = None if symmetric else m.Tensor(shape[:-1], m.ACL_FLOAT, d_o)
    m.dynamic_quant(m.Tensor(shape, m.ACL_BF16, d_x), m.Tensor(shape, m.ACL_INT8, d_y), m.Tensor(shape[:-1], m.ACL_FLOAT, d_s),
                    smooth=m.Tensor((len(ends), cols), m.ACL_BF16, d_sm), offset=off,
                    group_index=m.Tensor((len(ends),), m.ACL_INT32 if gi_dt == "i32" else m.ACL_INT64, d_gi))
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    assert np.array_equal(d_y.to_host(np.uint8, shape), want[0])
    assert np.array_equal(d_s.to_host(np.uint32, shape[:-1]), want[1].view(np.uint32))
    if not symmetric:
        assert np.array_equal(d_o.to_host(np.uint32, shape[:-1]), want[2].view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("mode,shape", [("pertensor", (16, 32)), ("pertensor", (3, 70, 500)), ("pertensor", (1000, 257)),
                                        ("perchannel", (16, 32)), ("perchannel", (3, 70, 500)), ("perchannel", (2, 200, 1001)), ("perchannel", (130, 64)),
                                        # rows of whole 16-byte pieces (the vector kernels): several row chunks per batch, a ragged
                                        # last chunk, more than one block of 64 pieces, fewer pieces than a block
                                        ("pertensor", (1000, 256)), ("pertensor", (2, 70, 1032)), ("perchannel", (3, 200, 512)),
                                        ("perchannel", (5, 64, 1032)), ("perchannel", (300, 8))])
@pytest.mark.parametrize("y_dt,symmetric,with_smooth", [(orc.I8, True, False), (orc.I8, False, True), (orc.I4, True, True), (orc.E4M3, True, False)])
def test_gpu_per_tensor_and_per_channel_modes(gpu, mode, shape, y_dt, symmetric, with_smooth):
    m = gpu
    if y_dt == orc.I4 and shape[-1] % 2:
        pytest.skip("INT4 needs an even last dim")
    print(f"case dynamic quant {mode} {shape} y={y_dt} symmetric={symmetric} smooth={with_smooth}", flush=True)
    rng = np.random.default_rng(sum(shape) + y_dt)
    xb = orc.f32_to_b16(rng.normal(0, 2, size=shape).astype(np.float32), orc.BF16)
    n_sm = shape[-1] if mode == "pertensor" else shape[-2]
    smb = orc.f32_to_b16(rng.uniform(0.5, 2.0, n_sm).astype(np.float32), orc.BF16) if with_smooth else None
    want = orc.dynamic_quant_wide(xb, orc.BF16, y_dt, mode, smooth=smb, symmetric=symmetric)
    sshape = (1,) if mode == "pertensor" else shape[:-2] + (shape[-1],)
    nsc = int(np.prod(sshape))
    d_x, d_sm = m.DeviceBuffer(host=xb), (m.DeviceBuffer(host=smb) if with_smooth else None)
    d_y, d_s, d_o = m.DeviceBuffer(want[0].nbytes), m.DeviceBuffer(nsc * 4), m.DeviceBuffer(nsc * 4)
    yt = m.Tensor(shape, m.DTYPE_BY_NAME[ACL_OF[y_dt]], d_y)
    m.dynamic_quant(m.Tensor(shape, m.ACL_BF16, d_x), yt, m.Tensor(sshape, m.ACL_FLOAT, d_s),
                    smooth=m.Tensor((n_sm,), m.ACL_BF16, d_sm) if with_smooth else None,
                    offset=None if symmetric else m.Tensor(sshape, m.ACL_FLOAT, d_o), quant_mode=mode.encode())
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    assert np.array_equal(d_s.to_host(np.uint32, sshape), want[1].view(np.uint32)), "scale differs"
    if not symmetric:
        assert np.array_equal(d_o.to_host(np.uint32, sshape), want[2].view(np.uint32)), "offset differs"
    gy, wy = d_y.to_host(np.uint8, want[0].shape), want[0]
    if y_dt == orc.E4M3:
        z = ((gy | wy) & 0x7f) == 0
        assert np.array_equal(gy[~z], wy[~z])
    else:
        assert np.array_equal(gy, wy), f"{int((gy != wy).sum())} of {wy.size} outputs differ"
