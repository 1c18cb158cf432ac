"""aclnnTransQuantParamV2 / V3 (fp32 scale + offset -> the packed 64-bit quantisation parameter): oracle pins, the reference's
status rules, device parity, and the chain into aclnnQuantMatmulV5's per-channel mode.

Reference: checks quant/trans_quant_param_v2/op_host/op_api/aclnn_trans_quant_param_v2.cpp:36-127, arithmetic
op_kernel/trans_quant_param_v2.h:224-300, system-test formula tests/st/aclnnTransQuantParamV2/executor_aclnnTransQuantParamV2.py:24-80.
"""
import numpy as np
import pytest

import oracle_api as orc


def _bits(f):
    return int(np.float32(f).view(np.uint32))


# ------------------------------------------------------------------------------------------------ oracle pins (CPU)
def test_truncating_mode_is_the_golden_utility_with_19_bits():
    rng = np.random.default_rng(0)
    s = rng.uniform(1e-4, 1.0, 300).astype(np.float32) * rng.choice([-1, 1], 300).astype(np.float32)
    o = rng.uniform(-300, 300, 300).astype(np.float32)
    want = orc.pack_u64_scale((s.view(np.uint32) & np.uint32(0xFFFFE000)).view(np.float32), o)
    assert np.array_equal(orc.trans_quant_param(s, o), want)
    # the system test's formula, written out: 19 bits of the scale, bit 46, the clipped and rounded offset at bit 37
    st = (s.view(np.uint32) & np.uint32(0xFFFFE000)).astype(np.uint64) | np.uint64(1 << 46)
    st |= (np.clip(np.round(np.clip(o, -256, 255)).astype(np.int64), -256, 255).astype(np.uint64) & np.uint64(0x1FF)) << np.uint64(37)
    assert np.array_equal(orc.trans_quant_param(s, o), st)
    # and what the matmul golden reads back is the truncated scale
    back = np.array([orc.lib().orc_u64_to_deq_scale(int(v)) for v in orc.trans_quant_param(s)], np.float32)
    assert np.array_equal(back.view(np.uint32), s.view(np.uint32) & np.uint32(0xFFFFE000))


def test_broadcast_of_one_element_inputs():
    s, o = np.float32([0.5]), np.float32([1, -2, 300, -300])
    got = orc.trans_quant_param(s, o)
    assert got.size == 4 and all(int(v) & 0xFFFFFFFF == _bits(0.5) for v in got)
    assert [(int(v) >> 37) & 0x1FF for v in got] == [1, 0x1FE, 255, 0x100]
    got = orc.trans_quant_param(np.float32([0.5, 0.25, 2.0]), np.float32([7]))
    assert [(int(v) >> 37) & 0x1FF for v in got] == [7, 7, 7] and [int(v) & 0xFFFFFFFF for v in got] == [_bits(0.5), _bits(0.25), _bits(2.0)]
    assert all((int(v) >> 46) & 1 for v in got)


def test_rounding_mode_known_answers():
    """13 mantissa bits are dropped.  Below half: down.  Above half: up.  Exactly half: to the even 10-bit mantissa.  A carry out
    of an all-ones mantissa raises the exponent; out of exponent 254 it gives infinity.  Subnormals and zero: signed zero.
    Infinity and NaN keep their truncated bits."""
    cases = [
        (0x3F800FFF, 0x3F800000), (0x3F801001, 0x3F802000), (0x3F801000, 0x3F800000), (0x3F803000, 0x3F804000),
        (0x3FFFF000, 0x40000000), (0x3FFFEFFF, 0x3FFFE000), (0xBF801001, 0xBF802000), (0x7F7FF000, 0x7F800000),
        (0x00400000, 0x00000000), (0x80000001, 0x80000000), (0x7F800000, 0x7F800000), (0x7FC01234, 0x7FC00000),
    ]
    s = np.array([c[0] for c in cases], np.uint32).view(np.float32)
    got = orc.trans_quant_param(s, round_mode=1)
    assert [hex(int(v) & 0xFFFFFFFF) for v in got] == [hex(c[1]) for c in cases]
    # random scales: numpy float64 recomputation of round-to-nearest-even at 10 mantissa bits
    rng = np.random.default_rng(1)
    r = rng.uniform(1e-6, 10, 2000).astype(np.float32)
    m, e = np.frexp(r.astype(np.float64))
    want = (np.rint(m * 2048) / 2048 * 2.0 ** e).astype(np.float32)
    assert np.array_equal((orc.trans_quant_param(r, round_mode=1) & np.uint64(0xFFFFFFFF)).astype(np.uint32), want.view(np.uint32))


# ------------------------------------------------------------------------------------------- status cases (no GPU)
def _t(m, shape, dt):
    return m.Tensor(shape, dt, None)


def _status(m, s, o, out, rm=None):
    rc, ws, ex = m.trans_quant_param_get_workspace(s, o, out, rm)
    if ex:
        m.lib().aclDestroyAclOpExecutor(ex)
    return rc


def test_status_rules(opsnn):
    m = opsnn
    bad, null = m.ACLNN_ERR_PARAM_INVALID, m.ACLNN_ERR_PARAM_NULLPTR
    f, u64, i64 = m.ACL_FLOAT, m.ACL_UINT64, m.ACL_INT64
    assert _status(m, _t(m, (64,), f), None, _t(m, (64,), u64)) == 0
    assert _status(m, _t(m, (64,), f), _t(m, (64,), f), _t(m, (64,), i64)) == 0
    assert _status(m, _t(m, (1, 64), f), _t(m, (1, 64), f), _t(m, (1, 64), u64)) == 0
    assert _status(m, _t(m, (4, 16), f), None, _t(m, (4, 16), u64)) == 0                      # [g, n] on the newest SoC
    assert _status(m, _t(m, (1,), f), _t(m, (64,), f), _t(m, (64,), u64)) == 0
    assert _status(m, _t(m, (64,), f), _t(m, (1,), f), _t(m, (64,), u64), rm=1) == 0
    assert _status(m, None, None, _t(m, (64,), u64)) == null and _status(m, _t(m, (64,), f), None, None) == null
    assert _status(m, _t(m, (64,), m.ACL_FLOAT16), None, _t(m, (64,), u64)) == bad
    assert _status(m, _t(m, (64,), f), _t(m, (64,), m.ACL_FLOAT16), _t(m, (64,), u64)) == bad
    assert _status(m, _t(m, (64,), f), None, _t(m, (64,), m.ACL_INT32)) == bad
    assert _status(m, _t(m, (2, 3, 4), f), None, _t(m, (24,), u64)) == bad
    assert _status(m, _t(m, (64,), f), _t(m, (2, 32), f), _t(m, (64,), u64)) == bad            # offset [g, n] with g > 1
    assert _status(m, _t(m, (64,), f), _t(m, (32,), f), _t(m, (64,), u64)) == bad              # lengths differ, both > 1
    assert _status(m, _t(m, (64,), f), None, _t(m, (64,), u64), rm=2) == bad
    assert _status(m, _t(m, (64,), f), None, _t(m, (32,), u64)) == bad                         # out too small


# --------------------------------------------------------------------------------------------------- device parity
@pytest.mark.gpu
@pytest.mark.parametrize("ns,no,rm", [(1000, 1000, None), (1, 777, None), (513, 1, 0), (4096, None, 1), (300, 300, 1), (1, 1, 1)])
def test_gpu_trans_quant_param_is_bit_identical(gpu, ns, no, rm):
    m = gpu
    print(f"case trans quant param scale {ns} offset {no} round mode {rm}", flush=True)
    rng = np.random.default_rng(ns + (no or 0))
    s = (rng.uniform(1e-5, 4.0, ns) * rng.choice([-1, 1], ns)).astype(np.float32)
    s.view(np.uint32)[:: 7] |= 0x1000                           # some exact ties for the rounding mode
    o = rng.uniform(-400, 400, no).astype(np.float32) if no else None
    want = orc.trans_quant_param(s, o, rm or 0)
    n = want.size
    d_s, d_o, d_out = m.DeviceBuffer(host=s), (m.DeviceBuffer(host=o) if no else None), m.DeviceBuffer(n * 8 + 16)
    d_out.fill(0xEE)
    m.trans_quant_param(m.Tensor((ns,), m.ACL_FLOAT, d_s), m.Tensor((no,), m.ACL_FLOAT, d_o) if no else None,
                        m.Tensor((n,), m.ACL_UINT64, d_out), rm)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    got = d_out.to_host(np.uint8, (n * 8 + 16,))
    assert (got[n * 8:] == 0xEE).all(), "wrote past out"
    assert np.array_equal(got[:n * 8].view(np.uint64), want)


@pytest.mark.gpu
def test_gpu_packed_scale_feeds_the_per_channel_matmul(gpu):
    """fp32 per-channel scale -> aclnnTransQuantParamV2 -> x2Scale (UINT64) of aclnnQuantMatmulV5 with int8 operands and an int32
    bias: the product equals the one with the scale packed on the host."""
    import cases
    m = gpu
    M, K, N = 64, 256, 192
    inp = cases.make_tc_inputs(m, M, K, N, 5, m.ACL_INT8, m.ACL_UINT64, N, m.ACL_INT32, True)
    want = cases.run_tc_aclnn(m, inp, M, K, N, m.ACL_FLOAT16)
    packed_host = np.ascontiguousarray(inp["scale"]).view(np.uint64).reshape(-1)
    s = (packed_host & np.uint64(0xFFFFFFFF)).astype(np.uint32).view(np.float32)
    d_s, d_out = m.DeviceBuffer(host=s), m.DeviceBuffer(N * 8)
    m.trans_quant_param(m.Tensor((N,), m.ACL_FLOAT, d_s), None, m.Tensor((N,), m.ACL_UINT64, d_out))
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    dev = d_out.to_host(np.uint64, (N,))
    assert np.array_equal(dev & np.uint64(0xFFFFE000), packed_host & np.uint64(0xFFFFE000))
    got = cases.run_tc_aclnn(m, dict(inp, scale=dev.reshape(inp["scale"].shape)), M, K, N, m.ACL_FLOAT16)
    assert np.array_equal(got, want)
