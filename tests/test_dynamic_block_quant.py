"""aclnnDynamicBlockQuant (fp8 quantizer of the block-scale matmul): oracle pins, phase-1 status cases, device parity.

The golden (quant/dynamic_block_quant/tests/assets/golden.py:95-222) is numpy float32 arithmetic followed by an ml_dtypes fp8
cast; the pins are a numpy float32 recomputation with torch's fp8 casts (the same round-to-nearest-even), known answers,
and the golden's stated rules for infinities and NaN.  Device bar: bit-identical y (the sign of a zero result aside) and scale.
"""
import numpy as np
import pytest

import oracle_api as orc

torch = pytest.importorskip("torch")
TORCH_FP8 = {orc.E4M3: "float8_e4m3fn", orc.E5M2: "float8_e5m2"}
TMAX = {orc.E4M3: 448.0, orc.E5M2: 57344.0}


def _numpy_golden(xf, rb, cb, y_dt, min_scale=0.0):
    rows, cols = xf.shape
    tmax = np.float32(TMAX[y_dt])
    clean = np.where(np.isfinite(xf), xf, np.float32(0))
    nrb, ncb = -(-rows // rb), -(-cols // cb)
    scale = np.zeros((nrb, ncb), np.float32)
    q = np.empty_like(xf)
    for i in range(nrb):
        for j in range(ncb):
            blk = (slice(i * rb, (i + 1) * rb), slice(j * cb, (j + 1) * cb))
            s = np.max(np.abs(clean[blk])).astype(np.float32) / tmax
            if min_scale:
                s = np.minimum(s, np.float32(1.0 / min_scale))
            scale[i, j] = s
            with np.errstate(all="ignore"):
                q[blk] = xf[blk] / s
    q = np.where(np.isfinite(xf), q, xf)
    q = np.clip(q, -tmax, tmax)
    with np.errstate(all="ignore"):
        q = np.round(q, 8)
    q = np.nan_to_num(q, nan=0.0, posinf=None, neginf=None)
    y = torch.from_numpy(q.astype(np.float32)).to(getattr(torch, TORCH_FP8[y_dt])).view(torch.uint8).numpy()
    return y, scale


def _same_but_zero_sign(a, b):
    z = ((a | b) & 0x7f) == 0
    return np.array_equal(a[~z], b[~z])


# ------------------------------------------------------------------------------------------------ oracle pins (CPU)
@pytest.mark.parametrize("x_dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("y_dt", [orc.E4M3, orc.E5M2])
@pytest.mark.parametrize("rb,cb,shape", [(1, 128, (9, 384)), (128, 128, (200, 300)), (64, 192, (70, 200)), (1, 64, (5, 100))])
def test_against_numpy_float32(x_dt, y_dt, rb, cb, shape):
    rng = np.random.default_rng(rb + cb)
    xb = orc.f32_to_b16((rng.normal(0, 1, size=shape) * 10.0 ** rng.integers(-3, 3, size=shape)).astype(np.float32), x_dt)
    xf = orc.b16_to_f32(xb, x_dt)
    want_y, want_s = _numpy_golden(xf, rb, cb, y_dt)
    y, s = orc.dynamic_block_quant(xb, x_dt, y_dt, rb, cb)
    assert np.array_equal(s.view(np.uint32), want_s.view(np.uint32))
    assert _same_but_zero_sign(y, want_y)


def test_known_answers():
    """A block whose max is 448 has scale 1: y is fp8(x), e.g. 3.3 -> 3.25 (0x45), 0.3 -> 0.3125 (0x2a).  A block of zeros has
    scale 0 and zeros.  min_scale = 4 caps the scale at 0.25: 448 / 0.25 is clipped to 448 (0x7e), 1 / 0.25 = 4 (0x48).
    Infinity counts as 0 for the max and comes out as +-448; NaN comes out as +0."""
    x = np.zeros((2, 256), np.float32)
    x[0, :4] = [448.0, 3.3, 0.3, -448.0]
    xb = orc.f32_to_f16(x)
    y, s = orc.dynamic_block_quant(xb, orc.F16, orc.E4M3, 1, 128)
    assert s[0, 0] == 1.0 and list(y[0, :4]) == [0x7e, 0x45, 0x2a, 0xfe]
    assert not s[0, 1] and not s[1].any() and not (y[1] & 0x7f).any()
    y, s = orc.dynamic_block_quant(xb, orc.F16, orc.E4M3, 1, 128, min_scale=4.0)
    assert s[0, 0] == 0.25 and y[0, 0] == 0x7e
    x[0, :4] = [np.inf, 1.0, np.nan, -np.inf]
    y, s = orc.dynamic_block_quant(orc.f32_to_f16(x), orc.F16, orc.E4M3, 1, 128)
    assert s[0, 0] == np.float32(1.0) / np.float32(448.0) and list(y[0, :4]) == [0x7e, 0x7e, 0x00, 0xfe]


def test_decimal_rounding_is_part_of_the_formula():
    """round(q, 8) in float32 moves q before the fp8 cast; the oracle must agree with numpy's own float32 round on values
    where rint(q * 1e8) / 1e8 != q."""
    rng = np.random.default_rng(0)
    q = rng.uniform(0.001, 0.08, 4096).astype(np.float32)
    moved = np.round(q, 8)
    assert (moved != q).any()
    x = np.zeros((1, 4096 + 128), np.float32)
    xb = orc.f32_to_bf16(np.concatenate([q, np.full(128, 448.0, np.float32)])[None, :])
    xf = orc.b16_to_f32(xb, orc.BF16)
    want_y, _ = _numpy_golden(xf, 1, 4096 + 128, orc.E4M3)
    y, s = orc.dynamic_block_quant(xb, orc.BF16, orc.E4M3, 1, 4096 + 128)
    assert s[0, 0] == 1.0 and _same_but_zero_sign(y, want_y)


# ------------------------------------------------------------------------------------------- status cases (no GPU)
def _t(m, shape, dt):
    return m.Tensor(shape, dt, None)


def _status(m, x, y, sc, **kw):
    rc, ws, ex = m.dynamic_block_quant_get_workspace(x, y, sc, **kw)
    if ex:
        m.lib().aclDestroyAclOpExecutor(ex)
    return rc


def test_status_rules(opsnn):
    """The documented rules (docs/aclnnDynamicBlockQuant.md:95-220) and the example calls of that file (:423-427 INT8 with
    1 x 128 blocks; :581-584 FLOAT8_E5M2, minScale 0.1)."""
    m = opsnn
    bad, null = m.ACLNN_ERR_PARAM_INVALID, m.ACLNN_ERR_PARAM_NULLPTR
    f8, f5 = m.ACL_FLOAT8_E4M3FN, m.ACL_FLOAT8_E5M2
    x, y, sc = _t(m, (256, 512), m.ACL_BF16), _t(m, (256, 512), f8), _t(m, (256, 4), m.ACL_FLOAT)
    assert _status(m, x, y, sc) == 0
    assert _status(m, x, _t(m, (256, 512), f5), sc, min_scale=0.1) == 0
    assert _status(m, x, y, _t(m, (2, 4), m.ACL_FLOAT), row_block=128) == 0
    assert _status(m, _t(m, (3, 256, 512), m.ACL_FLOAT16), _t(m, (3, 256, 512), f8), _t(m, (3, 4, 3), m.ACL_FLOAT), row_block=64, col_block=192) == 0
    assert _status(m, None, y, sc) == null and _status(m, x, None, sc) == null and _status(m, x, y, None) == null
    assert _status(m, _t(m, (256, 512), m.ACL_FLOAT), y, sc) == bad
    assert _status(m, x, y, sc, dst_type=f5) == bad                                  # dstType != yOut dtype
    assert _status(m, x, _t(m, (256, 512), m.ACL_INT32), sc) == bad
    assert _status(m, x, y, _t(m, (256, 4), m.ACL_FLOAT16)) == bad
    assert _status(m, x, y, sc, round_mode=b"round") == bad and _status(m, x, y, sc, round_mode=None) == 0
    assert _status(m, x, y, sc, row_block=2) == bad and _status(m, x, y, sc, col_block=32) == bad
    assert _status(m, x, y, sc, min_scale=-1.0) == bad
    assert _status(m, _t(m, (512,), m.ACL_BF16), _t(m, (512,), f8), _t(m, (4,), m.ACL_FLOAT)) == bad
    assert _status(m, x, _t(m, (256, 256), f8), sc) == bad
    assert _status(m, x, y, _t(m, (256, 5), m.ACL_FLOAT)) == bad
    # V2: the same with a dstTypeMax, which only 0 is run for
    assert _status(m, x, y, sc, dst_type_max=0.0) == 0 and _status(m, x, y, sc, dst_type_max=100.0) == 561002
    assert _status(m, x, y, sc, dst_type_max=0.0, row_block=2) == bad
    # accepted by the reference, no kernel here
    assert _status(m, x, _t(m, (256, 512), m.ACL_INT8), sc) == 561002
    assert _status(m, x, _t(m, (256, 512), m.ACL_HIFLOAT8), sc, round_mode=b"round") == 561002


# --------------------------------------------------------------------------------------------------- device parity
def _run(m, xb, x_dt, y_dt, rb, cb, min_scale=0.0):
    d_x = m.DeviceBuffer(host=xb)
    nsc = int(np.prod(xb.shape[:-2], dtype=np.int64)) * -(-xb.shape[-2] // rb) * -(-xb.shape[-1] // cb)
    d_y, d_s = m.DeviceBuffer(xb.size + 16), m.DeviceBuffer(nsc * 4 + 16)
    d_y.fill(0xEE); d_s.fill(0xEE)
    adt = m.ACL_FLOAT16 if x_dt == orc.F16 else m.ACL_BF16
    ydt = m.ACL_FLOAT8_E4M3FN if y_dt == orc.E4M3 else m.ACL_FLOAT8_E5M2
    sshape = xb.shape[:-2] + (-(-xb.shape[-2] // rb), -(-xb.shape[-1] // cb))
    m.dynamic_block_quant(m.Tensor(xb.shape, adt, d_x), m.Tensor(xb.shape, ydt, d_y), m.Tensor(sshape, m.ACL_FLOAT, d_s),
                          row_block=rb, col_block=cb, min_scale=min_scale)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    gy, gs = d_y.to_host(np.uint8, (xb.size + 16,)), d_s.to_host(np.uint8, (nsc * 4 + 16,))
    assert (gy[xb.size:] == 0xEE).all() and (gs[nsc * 4:] == 0xEE).all(), "wrote past an output"
    return gy[:xb.size].reshape(xb.shape), gs[:nsc * 4].view(np.float32).reshape(sshape)


@pytest.mark.gpu
@pytest.mark.parametrize("shape,rb,cb", [((64, 512), 1, 128), ((33, 1000), 1, 128), ((7, 7168), 1, 128), ((2, 50, 448), 1, 64),
                                         ((40, 600), 1, 192), ((20, 520), 1, 256), ((300, 500), 128, 128), ((2, 130, 260), 64, 192),
                                         ((700, 300), 512, 256), ((5, 131), 1, 128), ((256, 256), 128, 128)])
@pytest.mark.parametrize("x_dt,y_dt,min_scale", [(orc.BF16, orc.E4M3, 0.0), (orc.F16, orc.E5M2, 0.0), (orc.F16, orc.E4M3, 300.0)])
def test_gpu_block_quant_is_bit_identical(gpu, shape, rb, cb, x_dt, y_dt, min_scale):
    m = gpu
    print(f"case block quant {shape} {rb}x{cb} x={x_dt} y={y_dt} min_scale={min_scale}", flush=True)
    rng = np.random.default_rng(sum(shape) + rb)
    xf = (rng.normal(0, 1, size=shape) * 10.0 ** rng.integers(-3, 3, size=shape)).astype(np.float32)
    flat = xf.reshape(-1)
    flat[:shape[-1]] = 0.0                                     # a run of zeros (whole blocks of them when rb == 1)
    flat[-3:] = [np.inf, np.nan, -np.inf]
    xb = orc.f32_to_b16(xf, x_dt)
    want_y, want_s = orc.dynamic_block_quant(xb, x_dt, y_dt, rb, cb, min_scale)
    gy, gs = _run(m, xb, x_dt, y_dt, rb, cb, min_scale)
    assert np.array_equal(gs.view(np.uint32), want_s.view(np.uint32)), "scale differs"
    z = ((gy | want_y) & 0x7f) == 0
    assert np.array_equal(gy[~z], want_y[~z]), f"{int((gy[~z] != want_y[~z]).sum())} of {want_y.size} outputs differ"


@pytest.mark.gpu
def test_gpu_block_quantised_operands_feed_the_block_scale_matmul(gpu):
    """bf16 activation -> aclnnDynamicBlockQuant (1 x 128) and bf16 weight -> aclnnDynamicBlockQuant (128 x 128) give exactly the
    operands and scale tensors aclnnQuantMatmulV5's G-B mode takes; the product is the oracle's on the oracle's quantised
    operands, to the block-scale kernel's bar."""
    import cases
    m = gpu
    M, K, N = 128, 512, 256
    rng = np.random.default_rng(8)
    xb = orc.f32_to_bf16(rng.normal(0, 1, size=(M, K)).astype(np.float32))
    wb = orc.f32_to_bf16(rng.normal(0, 0.05, size=(N, K)).astype(np.float32))
    x8, s1 = _run(m, xb, orc.BF16, orc.E4M3, 1, 128)
    w8, s2 = _run(m, wb, orc.BF16, orc.E4M3, 128, 128)
    ox8, os1 = orc.dynamic_block_quant(xb, orc.BF16, orc.E4M3, 1, 128)
    ow8, os2 = orc.dynamic_block_quant(wb, orc.BF16, orc.E4M3, 128, 128)
    assert np.array_equal(s1, os1) and np.array_equal(s2, os2)
    inp = dict(x1=x8[None], x2=w8[None], s1=s1[None], s2=s2[None], gsM=1)     # [batch, ...]; x2 and its scales are [N, K]-major
    want = cases.oracle_blockscale(m, dict(inp, x1=ox8[None], x2=ow8[None]), M, K, N, True, m.ACL_BF16)
    got = cases.run_blockscale_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    g, w = orc.b16_to_f32(got, orc.BF16), orc.b16_to_f32(want, orc.BF16)
    mx, mean = orc.rel_err_stats(g, w)
    assert mx <= 2.0 ** -7 and mean <= 2.0 ** -10, f"max rel {mx:.3e} mean rel {mean:.3e}"


@pytest.mark.gpu
def test_gpu_v2_entry_point(gpu):
    m = gpu
    xb = orc.f32_to_bf16(np.random.default_rng(3).normal(0, 1, size=(64, 256)).astype(np.float32))
    want_y, want_s = orc.dynamic_block_quant(xb, orc.BF16, orc.E4M3, 1, 128)
    d_x, d_y, d_s = m.DeviceBuffer(host=xb), m.DeviceBuffer(xb.size), m.DeviceBuffer(64 * 2 * 4)
    m.dynamic_block_quant(m.Tensor((64, 256), m.ACL_BF16, d_x), m.Tensor((64, 256), m.ACL_FLOAT8_E4M3FN, d_y),
                          m.Tensor((64, 2), m.ACL_FLOAT, d_s), dst_type_max=0.0)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    gy = d_y.to_host(np.uint8, (64, 256))
    z = ((gy | want_y) & 0x7f) == 0
    assert np.array_equal(gy[~z], want_y[~z]) and np.array_equal(d_s.to_host(np.float32, (64, 2)), want_s)
