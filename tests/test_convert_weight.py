"""aclnnConvertWeightToINT4Pack: oracle pins, the reference's phase-1 status cases, device parity.

Status rows: the parameter table and the extra invalid cases of the reference's API unit test
(matmul/convert_weight_to_int4_pack/tests/ut/op_host/op_api/test_aclnn_convert_weight_to_int4_pack.cpp:70-151, 208-218,
285-301), written out as data in tests/golden/aclnn_convert_weight_to_int4_pack_cases.csv.  That test asserts no status for
its valid cases (its host implementation cannot run there), so the valid cases here are the device parity tests.
"""
import csv
import os

import numpy as np
import pytest

import oracle_api as orc

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "aclnn_convert_weight_to_int4_pack_cases.csv"), newline="") as f:
    ROWS = list(csv.DictReader(f))

E2M1_VALUES = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]


# ------------------------------------------------------------------------------------------------ oracle pins (CPU)
def test_int32_carriers_pack_like_the_golden_utility():
    """The low four bits of each carrier, even element in the low nibble: the bytes of the golden utility's
    eight-per-int32 packing (orc_pack_int4_to_int32) read as little-endian bytes."""
    rng = np.random.default_rng(0)
    vals = rng.integers(-8, 8, size=(6, 48)).astype(np.int8)
    got = orc.convert_weight_b4(vals.astype(np.int32))
    ref = np.empty(vals.size // 8, np.int32)
    orc.lib().orc_pack_int4_to_int32(np.ascontiguousarray(vals).ctypes.data, ref.ctypes.data, ref.size)
    assert np.array_equal(got.reshape(-1), ref.view(np.uint8))
    # carriers with bits above the nibble: only the low four bits count
    noisy = (vals.astype(np.int32) & 15) | (rng.integers(0, 2 ** 20, size=vals.shape).astype(np.int32) << 4)
    assert np.array_equal(orc.convert_weight_b4(noisy), got)
    assert np.array_equal(got, orc.pack_nibbles(vals.astype(np.uint8) & 15))


def test_fp32_carriers_give_the_fp4_code_of_their_value():
    """Each of the 16 fp4 e2m1 values comes back through the decoder; +0 and -0 keep their codes 0 and 8."""
    vals = np.array(E2M1_VALUES + [-v for v in E2M1_VALUES], np.float32)
    codes = orc.unpack_nibbles(orc.convert_weight_b4(vals))
    assert list(codes) == list(range(16))
    back = np.array([orc.lib().orc_e2m1_to_f32(int(c)) for c in codes], np.float32)
    assert np.array_equal(back.view(np.uint32), vals.view(np.uint32))


def test_fp32_carriers_off_the_table():
    """The reference cuts the bits to sign, exponent and one mantissa bit before its table lookup, so a value is
    truncated toward zero onto the half-step grid of its binade first: 1.25 -> 1.0, 1.75 -> 1.5, 3.5 -> 3.0, 5.0 -> 4.0,
    7.9 -> 6.0.  What is then not one of the 16 values gives code 0 without the sign: 0.75 (0.5-binade, mantissa bit set),
    0.25, 8.0, a subnormal, infinity, NaN, and their negatives."""
    on = np.array([1.25, 1.75, 3.5, 5.0, 7.9, -1.25, -5.0, 0.5 + 2 ** -10, 1e-39, -1e-39], np.float32)
    want_on = [2, 3, 5, 6, 7, 10, 14, 1, 0, 8]
    # 1e-39 is a subnormal below 2^-127 * 0.5: its exponent and first mantissa bit are zero, so it reads as (signed) zero
    assert list(orc.unpack_nibbles(orc.convert_weight_b4(on))) == want_on
    off = np.array([0.75, -0.75, 0.25, -0.25, 8.0, -8.0, 12.0, np.inf, -np.inf, np.nan, 2 ** -127 * 1.5, 100.0], np.float32)
    assert not orc.unpack_nibbles(orc.convert_weight_b4(off)).any()


# ------------------------------------------------------------------------------------------- status cases (no GPU)
def _tensor(m, shape_s, dtype_s, fmt_s, strides_s="", storage_s=""):
    shape = [int(v) for v in shape_s.split()]
    strides = [int(v) for v in strides_s.split()] or None
    storage = [int(v) for v in storage_s.split()] or None
    return m.Tensor(shape, m.DTYPE_BY_NAME["ACL_" + dtype_s], None, strides=strides, fmt=m.FORMAT_BY_NAME["ACL_FORMAT_" + fmt_s],
                    storage_shape=storage)


@pytest.mark.parametrize("row", ROWS, ids=[r["caseName"] for r in ROWS])
def test_status_matches_reference_table(opsnn, row):
    m = opsnn
    w = _tensor(m, row["weight"], row["weightType"], row["weightFormat"], row["weightStrides"], row["weightStorage"])
    p = _tensor(m, row["weightInt4Pack"], row["weightInt4PackType"], row["weightInt4PackFormat"])
    assert m.convert_weight_to_int4_pack(w, p) == int(row["expect"]), m.err_msg()


def test_null_arguments(opsnn):
    m = opsnn
    w = _tensor(m, "32 64", "INT32", "ND")
    assert m.convert_weight_to_int4_pack(None, w) == m.ACLNN_ERR_PARAM_NULLPTR
    assert m.convert_weight_to_int4_pack(w, None) == m.ACLNN_ERR_PARAM_NULLPTR


def test_leading_dims_must_agree(opsnn):
    """The reference compares the last two dims only and sizes its buffers from weight; a pack tensor with fewer
    groups would be overrun, so it is refused here."""
    m = opsnn
    w, p = _tensor(m, "3 32 64", "INT32", "ND"), _tensor(m, "2 32 8", "INT32", "ND")
    assert m.convert_weight_to_int4_pack(w, p) == m.ACLNN_ERR_PARAM_INVALID


# --------------------------------------------------------------------------------------------------- device parity
def _carriers(rng, shape, fp):
    if fp:
        vals = np.array(E2M1_VALUES + [-v for v in E2M1_VALUES] + [0.75, 1.25, 5.0, 8.0, -0.25, np.nan, np.inf, 1e-39], np.float32)
        return vals[rng.integers(0, vals.size, size=shape)]
    return rng.integers(-8, 8, size=shape).astype(np.int32) | (rng.integers(0, 2, size=shape).astype(np.int32) << 9)


@pytest.mark.gpu
@pytest.mark.parametrize("shape,fp,pack_dt", [((32, 64), False, "INT4"), ((32, 64), False, "INT32"), ((32, 64), True, "FLOAT4_E2M1"),
                                              ((32, 64), True, "FLOAT"), ((1, 2), False, "INT4"), ((3, 5, 14), False, "INT4"),
                                              ((3, 40, 24), True, "FLOAT"), ((1000, 1048), False, "INT32"), ((2048, 4096), True, "FLOAT4_E2M1")])
def test_gpu_pack_is_bit_identical(gpu, shape, fp, pack_dt):
    m = gpu
    print(f"case convert weight {shape} fp32={fp} -> {pack_dt}", flush=True)
    rng = np.random.default_rng(sum(shape))
    w = _carriers(rng, shape, fp)
    want = orc.convert_weight_b4(w)
    d_w, d_p = m.DeviceBuffer(host=w), m.DeviceBuffer(want.nbytes + 16)
    d_p.fill(0xEE)
    pshape = shape if pack_dt in ("INT4", "FLOAT4_E2M1") else shape[:-1] + (shape[-1] // 8,)
    tw = m.Tensor(shape, m.ACL_FLOAT if fp else m.ACL_INT32, d_w)
    tp = m.Tensor(pshape, m.DTYPE_BY_NAME["ACL_" + pack_dt], d_p)
    assert m.convert_weight_to_int4_pack(tw, tp) == 0, m.err_msg()
    got = d_p.to_host(np.uint8, (want.nbytes + 16,))   # no synchronisation call: the result is in place on return
    assert np.array_equal(got[:want.nbytes].reshape(want.shape), want)
    assert (got[want.nbytes:] == 0xEE).all(), "wrote past the packed weight"


@pytest.mark.gpu
@pytest.mark.parametrize("x_dt,M,K,N,group", [("f16", 16, 1024, 512, 128), ("bf16", 4, 512, 256, 0)])
def test_gpu_packed_weight_feeds_the_weight_only_matmul(gpu, x_dt, M, K, N, group):
    """The call sequence of the reference's example (matmul/convert_weight_to_int4_pack/examples/
    test_aclnn_convert_weight_to_int4_pack.cpp:137-300): int32 carriers -> aclnnConvertWeightToINT4Pack into an INT32 tensor
    [K, N / 8] -> aclnnWeightQuantBatchMatmulV2.  The product must equal the one on the same weight packed on the host."""
    import cases
    m = gpu
    print(f"case convert weight -> wqbmm {x_dt} {M}x{K}x{N} group={group}", flush=True)
    dt = m.ACL_FLOAT16 if x_dt == "f16" else m.ACL_BF16
    inp = cases.make_wq_inputs(m, M, K, N, 7, dt, m.ACL_INT4, group, False)
    want = cases.run_wq_aclnn(m, inp, M, K, N)
    nib = orc.unpack_nibbles(inp["w"]).astype(np.int32)            # [K, N] values 0..15
    carriers = np.where(nib >= 8, nib - 16, nib).astype(np.int32)  # one signed int4 per int32
    d_w, d_p = m.DeviceBuffer(host=carriers), m.DeviceBuffer(K * N // 2)
    assert m.convert_weight_to_int4_pack(m.Tensor((K, N), m.ACL_INT32, d_w), m.Tensor((K, N // 8), m.ACL_INT32, d_p)) == 0, m.err_msg()
    assert np.array_equal(d_p.to_host(np.uint8, inp["w"].shape), inp["w"])
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray) and k != "w"}
    d_y = m.DeviceBuffer(M * N * 2)
    G = -(-K // group) if group > 0 else 1
    sshape = (G, N) if group > 0 else (N,)
    x, w = m.Tensor((M, K), dt, d["x"]), m.Tensor((K, N // 8), m.ACL_INT32, d_p)
    sc, off = m.Tensor(sshape, dt, d["scale"]), m.Tensor(sshape, dt, d["offset"])
    ws = m.weight_quant_batch_matmul(x, w, sc, m.Tensor((M, N), dt, d_y), offset=off, group_size=group)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    del ws
    assert np.array_equal(d_y.to_host(np.uint16, (M, N)), want)
