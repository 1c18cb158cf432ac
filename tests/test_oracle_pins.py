"""Pins for the CPU oracle (oracle/oracle.c): every function is checked against something that does not
restate its formula -- format definitions and torch's CPU dtypes for the codecs, the reference's own constants
and all-ones example, exact integer / float64 arithmetic where power-of-two operands make the result
order-independent, numpy's own float16 arithmetic for the double rounding of the weight-only path, and
hand-built cases that a dropped term, a swapped operand order or a wrong index would fail.
"""
import numpy as np
import pytest

import oracle_api as orc

torch = pytest.importorskip("torch")


# ------------------------------------------------------------------ codecs
def test_bf16_and_f16_decode_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    t = torch.from_numpy(bits.view(np.int16).copy())
    ref_bf = t.view(torch.bfloat16).float().numpy()
    ref_h = t.view(torch.float16).float().numpy()
    assert np.array_equal(orc.bf16_to_f32(bits).view(np.uint32), ref_bf.view(np.uint32))
    got = orc.f16_to_f32(bits)
    nan = np.isnan(ref_h)
    assert np.array_equal(got[~nan].view(np.uint32), ref_h[~nan].view(np.uint32)) and np.isnan(got[nan]).all()


def _interesting_floats(rng, n):
    u = rng.integers(0, 2 ** 32, size=n, dtype=np.uint64).astype(np.uint32)
    f = u.view(np.float32)
    f = f[np.isfinite(f)]
    # every 16-bit value, its neighbours and exact midpoints (ties)
    b = np.arange(0, 0x7f80, dtype=np.uint32) << 16
    ties = np.concatenate([b | 0x8000, b | 0x7fff, b | 0x8001, b]).view(np.float32)
    h = np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float32)
    hn = np.nextafter(h, np.float32(np.inf))
    hmid = ((h.astype(np.float64) + hn.astype(np.float64)) / 2).astype(np.float32)  # halfway points where representable
    small = np.array([0.0, -0.0, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -26, 65504.0, 65519.9, 65520.0,
                      65536.0, 1e30, -1e30, 448.0, 464.0, 465.0, 479.9, 480.0, 2.0 ** -9, 2.0 ** -10, 2.0 ** -10 * 1.01],
                     dtype=np.float32)
    return np.concatenate([f, ties, h, hmid, -hmid, small, -small]).astype(np.float32)


def test_bf16_and_f16_encode_match_torch_rne():
    f = _interesting_floats(np.random.default_rng(0), 400000)
    t = torch.from_numpy(f)
    assert np.array_equal(orc.f32_to_bf16(f), t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16))
    assert np.array_equal(orc.f32_to_f16(f), t.to(torch.float16).view(torch.int16).numpy().view(np.uint16))
    # and numpy's independent float16 conversion
    assert np.array_equal(orc.f32_to_f16(f), f.astype(np.float16).view(np.uint16))


def test_fp8_tables_match_ocp_and_torch():
    codes = np.arange(256, dtype=np.uint8)
    t = torch.from_numpy(codes)
    ref = t.view(torch.float8_e4m3fn).float().numpy()
    got = orc.e4m3_to_f32(codes)
    nan = np.isnan(ref)
    assert nan.sum() == 2 and np.isnan(got[nan]).all()
    assert np.array_equal(got[~nan].view(np.uint32), ref[~nan].view(np.uint32))
    ref5 = t.view(torch.float8_e5m2).float().numpy()
    got5 = orc.e5m2_to_f32(codes)
    nan5 = np.isnan(ref5)
    assert np.array_equal(got5[~nan5].view(np.uint32), ref5[~nan5].view(np.uint32)) and np.isnan(got5[nan5]).all()
    # OCP landmarks: max 448, min subnormal 2^-9; the reference example's constant 0b00111000 == 1.0
    assert got[0x7E] == 448.0 and got[0x01] == 2.0 ** -9 and got[0b00111000] == 1.0
    # (matmul/quant_batch_matmul_v4/examples/arch35/test_aclnn_quant_matmul_v5_f8f4_nd.cpp:129-131)


def test_e4m3_encode_matches_torch_in_range():
    f = _interesting_floats(np.random.default_rng(1), 200000)
    f = f[np.abs(f) <= 448.0]
    fine = np.linspace(-448, 448, 200001).astype(np.float32)
    f = np.concatenate([f, fine, np.float32([464.0, -464.0, 463.9, 2.0 ** -10, 3 * 2.0 ** -10, 2.0 ** -9 * 1.5])])
    ref = torch.from_numpy(f).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = orc.f32_to_e4m3(f)
    assert np.array_equal(got & 0x7f, ref & 0x7f)          # magnitude code
    nz = (got & 0x7f) != 0
    assert np.array_equal(got[nz] & 0x80, ref[nz] & 0x80)  # sign (the sign of a zero result is not pinned)


def test_e4m3_encode_out_of_range_matches_torch():
    """The cast does not saturate: whatever rounds above 448 -- everything above the tie 464 -- becomes NaN, as in
    torch.float8_e4m3fn (the cast the golden delegates to its dtype package inside compute_t_cg,
    qbmmv4_kernel_golden.py:239).  Every 4097th fp32 bit pattern of the whole range plus a dense sweep of 440..500."""
    bits = np.arange(0, 2 ** 32, 4097, dtype=np.uint64).astype(np.uint32)
    f = np.concatenate([bits.view(np.float32), np.linspace(440, 500, 60001).astype(np.float32),
                        -np.linspace(440, 500, 60001).astype(np.float32),
                        np.float32([464.0, np.nextafter(np.float32(464), np.float32(500)), 480.0, np.inf, -np.inf, np.nan])])
    ref = torch.from_numpy(f).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = orc.f32_to_e4m3(f)
    assert np.array_equal(got & 0x7f, ref & 0x7f)
    nz = ((got & 0x7f) != 0) & ((got & 0x7f) != 0x7f)
    assert np.array_equal(got[nz] & 0x80, ref[nz] & 0x80)


def test_e8m0_and_fp4_tables():
    codes = np.arange(256, dtype=np.uint8)
    got = orc.e8m0_to_f32(codes)
    assert np.isnan(got[255]) and got[127] == 1.0 and got[128] == 2.0 and got[126] == 0.5
    assert np.array_equal(got[:255].astype(np.float64), 2.0 ** (codes[:255].astype(np.float64) - 127))
    if hasattr(torch, "float8_e8m0fnu"):
        ref = torch.from_numpy(codes).view(torch.float8_e8m0fnu).float().numpy()
        assert np.array_equal(got[:255], ref[:255])
    # FP4_E2M1_TABLE of the reference (matmul_quant_util.py:329-346); 0b0010 == 1.0 in its fp4 example
    table = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]
    got4 = np.array([orc.lib().orc_e2m1_to_f32(i) for i in range(16)], np.float32)
    assert np.array_equal(got4.view(np.uint32), np.float32(table).view(np.uint32)) and got4[0b0010] == 1.0
    assert np.array_equal(orc.E2M1_VALUES.view(np.uint32), np.float32(table).view(np.uint32))


def test_group_size_codec_documented_constants():
    import ctypes as C
    for gs, want in [(4303356032, (1, 128, 128)), (549764202624, (128, 128, 128)), (4295032864, (1, 1, 32)), (0, (1, 1, 1)),
                     (32, (1, 1, 32))]:
        a, b, c = C.c_int64(), C.c_int64(), C.c_int64()
        orc.lib().orc_unpack_groupsize(gs, C.byref(a), C.byref(b), C.byref(c))
        assert (a.value, b.value, c.value) == want  # aclnnQuantMatmulV5.md:900-901, 929


def test_int4_pack_roundtrip_and_nibble_order():
    rng = np.random.default_rng(0)
    v = rng.integers(-8, 8, size=64).astype(np.int8)
    packed = np.empty(8, np.int32)
    orc.lib().orc_pack_int4_to_int32(v.ctypes.data, packed.ctypes.data, 8)
    # element i sits in bits 4i..4i+3 (matmul_quant_util.py:228-273)
    assert packed.view(np.uint32)[0] == sum((int(v[i]) & 15) << (4 * i) for i in range(8))
    back = np.empty(64, np.int8)
    orc.lib().orc_unpack_int32_to_int4(packed.ctypes.data, back.ctypes.data, 8)
    assert np.array_equal(back, v)
    # the same bytes read as a 4-bit tensor: low nibble = even index
    nib = orc.unpack_nibbles(packed.view(np.uint8))
    assert np.array_equal(np.where(nib >= 8, nib.astype(np.int16) - 16, nib), v)


def test_scale_truncation_helpers():
    s = np.float32(1.2345678)
    t = orc.lib().orc_scale_generate(s)
    assert np.float32(t).view(np.uint32) == (s.view(np.uint32) & 0xFFFFE000)
    assert orc.lib().orc_u64_to_deq_scale(int(s.view(np.uint32)) | (1 << 46)) == t


# ------------------------------------------------------------------ int8 GEMM + per-token epilogue
def test_int8_acc_brute_force_and_transposes():
    rng = np.random.default_rng(2)
    M, K, N = 7, 19, 11
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    b = rng.integers(-128, 128, (K, N), dtype=np.int8)
    want = np.zeros((M, N), np.int64)
    for i in range(M):
        for j in range(N):
            for k in range(K):
                want[i, j] += int(a[i, k]) * int(b[k, j])
    assert np.array_equal(orc.qmm_int8_acc(a, b, M, K, N), want)
    assert np.array_equal(orc.qmm_int8_acc(a, np.ascontiguousarray(b.T), M, K, N, tB=True), want)
    assert np.array_equal(orc.qmm_int8_acc(np.ascontiguousarray(a.T), b, M, K, N, tA=True), want)
    eye = np.eye(K, dtype=np.int8)
    assert np.array_equal(orc.qmm_int8_acc(a, eye, M, K, K), a.astype(np.int32))
    # extreme values: K * (-128)^2 fits int32 for K = 4096
    big = orc.qmm_int8_acc(np.full((1, 4096), -128, np.int8), np.full((4096, 1), -128, np.int8), 1, 4096, 1)
    assert big[0, 0] == 4096 * 16384


def test_pertoken_operation_order_and_bias_placement():
    # acc * s2 * s1 is evaluated left to right in fp32; choose values where the other association differs
    rng = np.random.default_rng(3)
    found = False
    for _ in range(2000):
        acc = np.int32(rng.integers(1, 1 << 26))
        s1, s2 = np.float32(rng.uniform(1e-3, 1e-2)), np.float32(rng.uniform(1e-3, 1e-2))
        left = np.float32(np.float32(np.float32(acc) * s2) * s1)
        right = np.float32(np.float32(acc) * np.float32(s2 * s1))
        if left != right:
            found = True
            break
    assert found
    y = np.empty((1, 1), np.float32)
    a = np.array([[acc]], np.int32)
    s1a, s2a = np.float32([s1]), np.float32([s2])   # keep the buffers alive across the ctypes calls
    epi = orc.lib().orc_qmm_pertoken_epilogue
    epi(a.ctypes.data, 1, 1, s1a.ctypes.data, s2a.ctypes.data, 1, None, 0, orc.F32, y.ctypes.data)
    assert y[0, 0] == left and y[0, 0] != right
    # int32 bias is added before scaling, float bias after (qbmmv3_kernel_golden.py:372-383)
    ib = np.int32([1000])
    epi(a.ctypes.data, 1, 1, s1a.ctypes.data, s2a.ctypes.data, 1, ib.ctypes.data, orc.I32, orc.F32, y.ctypes.data)
    assert y[0, 0] == np.float32(np.float32(np.float32(acc + 1000) * s2) * s1)
    fb = np.float32([0.125])
    epi(a.ctypes.data, 1, 1, s1a.ctypes.data, s2a.ctypes.data, 1, fb.ctypes.data, orc.F32, orc.F32, y.ctypes.data)
    assert y[0, 0] == np.float32(left + np.float32(0.125))


def test_pertoken_against_float64():
    rng = np.random.default_rng(4)
    M, K, N = 24, 200, 40
    a = rng.integers(-127, 128, (M, K), dtype=np.int8)
    b = rng.integers(-127, 128, (K, N), dtype=np.int8)
    s1, s2 = rng.uniform(1e-3, 1e-2, M).astype(np.float32), rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    bias = rng.normal(0, 0.1, N).astype(np.float32)
    y = orc.qmm_pertoken(a, b, M, K, N, False, False, s1, s2, bias, orc.F32, orc.F32)
    ref = (a.astype(np.float64) @ b.astype(np.float64)) * s2[None, :].astype(np.float64) * s1[:, None].astype(np.float64) + bias
    assert np.max(np.abs(y - ref) / np.maximum(np.abs(ref), 1e-3)) < 4e-7
    yb = orc.qmm_pertoken(a, b, M, K, N, False, False, s1, s2, bias, orc.F32, orc.BF16)
    assert np.array_equal(yb, orc.f32_to_bf16(y))


# ------------------------------------------------------------------ block scale
def test_perblock_all_ones_example():
    # the reference's per-block example: M=128 K=4096 N=512, all ones, unit scales -> every output is 4096
    # (matmul/quant_batch_matmul_v4/examples/test_aclnn_quant_matmul_v5_perblock.cpp:99-158)
    M, K, N = 128, 4096, 512
    x1, x2 = np.ones((M, K), np.int8), np.ones((N, K), np.int8)
    s1, s2 = np.ones((M, 32), np.float32), np.ones((4, 32), np.float32)
    y = orc.qmm_perblock(x1, x2, orc.I8, orc.I8, M, K, N, False, True, s1, s2, 1, 128, 128, np.zeros(N, np.float32), orc.BF16)
    assert (orc.bf16_to_f32(y) == 4096.0).all()


def test_perblock_power_of_two_scales_are_exact_and_indexing_is_right():
    rng = np.random.default_rng(5)
    M, K, N = 70, 300, 200   # ragged in every direction
    for tB in (False, True):
        for gsM in (1, 128):
            x1 = orc.f32_to_e4m3(rng.integers(-8, 9, (M, K)).astype(np.float32))
            x2f = rng.integers(-8, 9, (K, N)).astype(np.float32)
            x2 = orc.f32_to_e4m3(np.ascontiguousarray(x2f.T) if tB else x2f)
            KB, NB, MB = 3, 2, -(-M // gsM)
            e1 = rng.integers(-3, 4, (MB, KB))
            e2 = rng.integers(-3, 4, (KB, NB))
            s1 = (2.0 ** e1).astype(np.float32)
            s2l = (2.0 ** e2).astype(np.float32)
            s2 = np.ascontiguousarray(s2l.T) if tB else s2l
            y = orc.qmm_perblock(x1, x2, orc.E4M3, orc.E4M3, M, K, N, False, tB, s1, s2, gsM, 128, 128, None, orc.F32)
            a = orc.e4m3_to_f32(x1).astype(np.float64)
            ref = np.zeros((M, N))
            for kb in range(KB):
                k0, k1 = kb * 128, min(K, kb * 128 + 128)
                sc = np.repeat(s1[:, kb], gsM)[:M, None].astype(np.float64) * np.repeat(s2l[kb], 128)[None, :N]
                ref += (a[:, k0:k1] @ x2f[k0:k1].astype(np.float64)) * sc
            assert np.array_equal(y, ref.astype(np.float32))   # all sums are small integers times powers of two: exact


def test_perblock_single_block_equals_scaled_gemm_in_float64():
    rng = np.random.default_rng(6)
    M, K, N = 16, 128, 128
    x1 = orc.f32_to_e4m3(rng.normal(0, 1, (M, K)).astype(np.float32))
    x2 = orc.f32_to_e4m3(rng.normal(0, 1, (K, N)).astype(np.float32))
    s1, s2 = rng.uniform(1e-3, 1e-2, (M, 1)).astype(np.float32), rng.uniform(1e-3, 1e-2, (1, 1)).astype(np.float32)
    y = orc.qmm_perblock(x1, x2, orc.E4M3, orc.E4M3, M, K, N, False, False, s1, s2, 1, 128, 128, None, orc.F32)
    ref = (orc.e4m3_to_f32(x1).astype(np.float64) @ orc.e4m3_to_f32(x2).astype(np.float64)) * np.float64(np.float32(s1 * s2[0, 0]))
    assert np.max(np.abs(y - ref) / np.maximum(np.abs(ref), 1e-6)) < 2e-5
    # linear in the scales
    y2 = orc.qmm_perblock(x1, x2, orc.E4M3, orc.E4M3, M, K, N, False, False, s1 * np.float32(4), s2, 1, 128, 128, None, orc.F32)
    assert np.array_equal(y2, y * np.float32(4))


# ------------------------------------------------------------------ MX
def _mx_reference(c1, c2_kn, s1_mk, s2_kn):
    """float64 evaluation with fully expanded per-element scales."""
    a = orc.E2M1_VALUES[c1].astype(np.float64) * np.repeat(2.0 ** (s1_mk.astype(np.float64) - 127), 32, axis=1)[:, :c1.shape[1]]
    b = orc.E2M1_VALUES[c2_kn].astype(np.float64) * np.repeat(2.0 ** (s2_kn.astype(np.float64) - 127), 32, axis=0)[:c2_kn.shape[0]]
    return a @ b


def test_mx_exact_and_scale_layouts():
    rng = np.random.default_rng(7)
    M, K, N = 9, 192, 14          # ceil(K/32) = 6, K64 = 3
    c1 = rng.integers(0, 16, (M, K), dtype=np.uint8)
    c2 = rng.integers(0, 16, (K, N), dtype=np.uint8)
    s1 = (127 + rng.integers(-2, 3, (M, 6))).astype(np.uint8)        # logical [M, K/32]
    s2 = (127 + rng.integers(-2, 3, (6, N))).astype(np.uint8)        # logical [K/32, N]
    ref = _mx_reference(c1, c2, s1, s2)                              # exact: small dyadic rationals
    x1 = orc.pack_nibbles(c1)
    s1_store = s1.reshape(M, 3, 2)                                   # [M, K64, 2]
    # x2 not transposed: data [K, N] packed along N; scale stored [K64, N, 2]
    s2_store = np.ascontiguousarray(s2.reshape(3, 2, N).transpose(0, 2, 1))
    y = orc.qmm_mx(x1, orc.pack_nibbles(c2), orc.E2M1, orc.E2M1, M, K, N, False, False, s1_store, s2_store, None, orc.F32)
    assert np.array_equal(y, ref.astype(np.float32))
    # x2 transposed: data [N, K] packed along K; scale stored [N, K64, 2]
    s2_store_t = np.ascontiguousarray(s2.T).reshape(N, 3, 2)
    yt = orc.qmm_mx(x1, orc.pack_nibbles(np.ascontiguousarray(c2.T)), orc.E2M1, orc.E2M1, M, K, N, False, True, s1_store,
                    s2_store_t, None, orc.F32)
    assert np.array_equal(yt, ref.astype(np.float32))
    # bias is added in fp32 before the cast
    bias = rng.normal(0, 1, N).astype(np.float32)
    yb = orc.qmm_mx(x1, orc.pack_nibbles(c2), orc.E2M1, orc.E2M1, M, K, N, False, False, s1_store, s2_store, bias, orc.BF16)
    assert np.array_equal(yb, orc.f32_to_bf16(ref.astype(np.float32) + bias))


def test_mx_odd_block_count_ignores_the_pad_scale():
    # K = 96: three 32-blocks, scale arrays hold four entries; the fourth is padding and may hold anything
    rng = np.random.default_rng(8)
    M, K, N = 4, 96, 6
    c1 = rng.integers(0, 16, (M, K), dtype=np.uint8)
    c2 = rng.integers(0, 16, (N, K), dtype=np.uint8)
    s1 = np.full((M, 2, 2), 127, np.uint8)
    s2 = np.full((N, 2, 2), 128, np.uint8)
    s1[:, 1, 1] = 0xFF   # NaN in the pad slot
    s2[:, 1, 1] = 0xFF
    y = orc.qmm_mx(orc.pack_nibbles(c1), orc.pack_nibbles(c2), orc.E2M1, orc.E2M1, M, K, N, False, True, s1, s2, None, orc.F32)
    ref = (orc.E2M1_VALUES[c1].astype(np.float64) @ orc.E2M1_VALUES[c2].astype(np.float64).T) * 2.0
    assert np.array_equal(y, ref.astype(np.float32))


# ------------------------------------------------------------------ weight-only
def _np_dequant_f16(w_int, off16, s16, g):
    """numpy's own float16 arithmetic (computes in float32, rounds to float16 after every operation)."""
    K, N = w_int.shape
    out = np.empty((K, N), np.float16)
    for k in range(K):
        gi = k // g
        t = w_int[k].astype(np.float16)
        if off16 is not None:
            t = t + off16[gi]
        out[k] = t * s16[gi]
    return out


@pytest.mark.parametrize("w_bits", [8, 4])
def test_weight_only_dequant_double_rounding_matches_numpy_float16(w_bits):
    # x = identity makes y equal the dequantised weight exactly, exposing both b16 roundings
    rng = np.random.default_rng(9)
    K, N, g = 64, 48, 32
    lo, hi = (-127, 128) if w_bits == 8 else (-8, 8)
    w_int = rng.integers(lo, hi, (K, N))
    off16 = rng.uniform(-1, 1, (2, N)).astype(np.float16)
    s16 = rng.uniform(0.005, 0.02, (2, N)).astype(np.float16)
    want = _np_dequant_f16(w_int, off16, s16, g)
    single = (w_int.astype(np.float32) + np.repeat(off16.astype(np.float32), g, 0)) * np.repeat(s16.astype(np.float32), g, 0)
    assert (single.astype(np.float16) != want).any(), "the case must distinguish one rounding from two"
    x = orc.f32_to_f16(np.eye(K, dtype=np.float32))
    w = w_int.astype(np.int8) if w_bits == 8 else orc.pack_nibbles((w_int & 15).astype(np.uint8))
    y = orc.wqbmm(x, orc.F16, w, orc.I8 if w_bits == 8 else orc.I4, K, K, N, False, s16.view(np.uint16), orc.F16, N,
                  off16.view(np.uint16), g, None, 0)
    assert np.array_equal(y, want.view(np.uint16))
    # transposed storage of weight, scale and offset gives the same result
    wt = np.ascontiguousarray(w_int.T)
    wt = wt.astype(np.int8) if w_bits == 8 else orc.pack_nibbles((wt & 15).astype(np.uint8))
    yt = orc.wqbmm(x, orc.F16, wt, orc.I8 if w_bits == 8 else orc.I4, K, K, N, True,
                   np.ascontiguousarray(s16.T).view(np.uint16), orc.F16, N, np.ascontiguousarray(off16.T).view(np.uint16), g, None, 0)
    assert np.array_equal(yt, y)


def _mx_weight_case(rng, K, N, exps):
    codes = rng.integers(0, 16, (K, N)).astype(np.uint8)
    G = -(-K // 32)
    e = rng.choice(np.asarray(exps), size=(G, N)).astype(np.int64)
    return codes, (e + 127).astype(np.uint8), e


def test_weight_only_mx_fp16_matches_numpy_float16_closed_form():
    """_compute_mx (wqbmmv2_kernel_golden.py:300-352) with fp16 x: w = f16(fp4 * f16(2^e)) per 32 K.  x = identity makes
    y the dequantised weight itself.  Exponents reach the fp16 subnormals (2^-24 is the smallest, 2^-25 and below round the
    SCALE to zero; 0.5 * 2^-24 ties to zero, 1.5 * 2^-24 ties to 2 * 2^-24) and the largest scale that keeps 6 * 2^e
    finite; three blocks (an odd count) along K."""
    rng = np.random.default_rng(21)
    K, N = 96, 40
    codes, sbytes, e = _mx_weight_case(rng, K, N, list(range(-27, 14)))
    s16 = np.ldexp(np.float32(1), e).astype(np.float32).astype(np.float16)             # the scale through fp16
    want = (orc.E2M1_VALUES[codes] * np.repeat(s16.astype(np.float32), 32, 0)).astype(np.float16)
    assert (s16 == 0).any() and (np.abs(want.astype(np.float32)) < 2.0 ** -14).any()   # flushed scales and subnormal weights occur
    x = orc.f32_to_f16(np.eye(K, dtype=np.float32))
    y = orc.wqbmm(x, orc.F16, orc.pack_nibbles(codes), orc.E2M1, K, K, N, False, sbytes, orc.E8M0, N, None, 32, None, 0)
    z = want.view(np.uint16)
    zero = ((y | z) & 0x7fff) == 0
    assert np.array_equal(y[~zero], z[~zero])
    # [N, K] storage of the weight with [N, K/32] scales gives the same result
    yt = orc.wqbmm(x, orc.F16, orc.pack_nibbles(np.ascontiguousarray(codes.T)), orc.E2M1, K, K, N, True,
                   np.ascontiguousarray(sbytes.T), orc.E8M0, N, None, 32, None, 0)
    assert np.array_equal(yt, y)


def test_weight_only_mx_fp16_scale_overflow():
    """2^16 is not an fp16 number: the scale becomes infinity, every non-zero weight +-inf and a zero weight NaN; 2^14 keeps
    4 * 2^14 = 65536 > 65504 -> inf but 3 * 2^14 finite.  One K element, x = 1, so nothing else enters the sum."""
    codes = np.arange(16, dtype=np.uint8).reshape(1, 16)
    x = orc.f32_to_f16(np.ones((1, 1), np.float32))
    for e in (14, 16):
        s16 = np.float32(2.0 ** e).astype(np.float16)
        with np.errstate(over="ignore", invalid="ignore"):
            want = (orc.E2M1_VALUES[codes] * np.float32(s16)).astype(np.float16)
        y = orc.wqbmm(x, orc.F16, orc.pack_nibbles(codes), orc.E2M1, 1, 1, 16, False, np.full((1, 16), 127 + e, np.uint8),
                      orc.E8M0, 16, None, 32, None, 0).view(np.float16)
        assert np.array_equal(np.isnan(y), np.isnan(want))
        ok = ~np.isnan(want)
        assert np.array_equal(y[ok], want[ok])
        assert np.isinf(want[0, 7]) and (e == 16 or np.isfinite(want[0, 5]))


def test_weight_only_mx_bf16_matches_torch_bfloat16():
    """bf16 x: the scale is NOT rounded (2^e is a bf16 number for every e8m0 byte but 0xFF) and fp4 * 2^e is exact in bf16
    down to its subnormals; byte 0 is 2^-127."""
    rng = np.random.default_rng(22)
    K, N = 64, 24
    codes, sbytes, e = _mx_weight_case(rng, K, N, [-127, -126, -100, -3, 0, 5, 60, 120])
    prod = orc.E2M1_VALUES[codes].astype(np.float64) * np.repeat(np.ldexp(1.0, e), 32, 0)
    want = torch.from_numpy(prod.astype(np.float32)).to(torch.bfloat16)
    assert np.array_equal(want.float().numpy().astype(np.float64), prod)      # exact: nothing is rounded on this path
    x = orc.f32_to_bf16(np.eye(K, dtype=np.float32))
    y = orc.wqbmm(x, orc.BF16, orc.pack_nibbles(codes), orc.E2M1, K, K, N, False, sbytes, orc.E8M0, N, None, 32, None, 0)
    z = want.view(torch.int16).numpy().view(np.uint16)
    zero = ((y | z) & 0x7fff) == 0
    assert np.array_equal(y[~zero], z[~zero])


def test_weight_only_mx_full_product_against_float64():
    """With power-of-two scales in a narrow band every product and partial sum of x (small integers) times the weight is
    exact in fp32, so the result must equal the float64 matmul rounded once to the output type, whatever the order."""
    rng = np.random.default_rng(23)
    M, K, N = 7, 128, 20
    codes, sbytes, e = _mx_weight_case(rng, K, N, [-2, -1, 0, 1, 2])
    xi = rng.integers(-4, 5, (M, K)).astype(np.float32)
    w = orc.E2M1_VALUES[codes].astype(np.float64) * np.repeat(np.ldexp(1.0, e), 32, 0)
    want = (xi.astype(np.float64) @ w)
    for dt, enc in ((orc.F16, orc.f32_to_f16), (orc.BF16, orc.f32_to_bf16)):
        y = orc.wqbmm(enc(xi), dt, orc.pack_nibbles(codes), orc.E2M1, M, K, N, False, sbytes, orc.E8M0, N, None, 32, None, 0)
        assert np.array_equal(y, enc(want.astype(np.float32)))


def test_weight_only_bf16_dequant_matches_torch_bfloat16():
    rng = np.random.default_rng(10)
    K, N = 32, 40
    w_int = rng.integers(-127, 128, (K, N))
    off = torch.from_numpy(rng.uniform(-1, 1, (1, N)).astype(np.float32)).to(torch.bfloat16)
    sc = torch.from_numpy(rng.uniform(0.005, 0.02, (1, N)).astype(np.float32)).to(torch.bfloat16)
    want = ((torch.from_numpy(w_int.astype(np.float32)).to(torch.bfloat16) + off) * sc)  # torch rounds to bf16 after each op
    x = orc.f32_to_bf16(np.eye(K, dtype=np.float32))
    y = orc.wqbmm(x, orc.BF16, w_int.astype(np.int8), orc.I8, K, K, N, False, sc.view(torch.int16).numpy().view(np.uint16),
                  orc.BF16, N, off.view(torch.int16).numpy().view(np.uint16), 0, None, 0)
    assert np.array_equal(y, want.view(torch.int16).numpy().view(np.uint16))


def test_weight_only_reductions():
    rng = np.random.default_rng(11)
    M, K, N = 5, 128, 24
    x = orc.f32_to_f16(rng.normal(0, 1, (M, K)).astype(np.float32))
    w = rng.integers(-127, 128, (K, N), dtype=np.int8)
    s = orc.f32_to_f16(rng.uniform(0.005, 0.02, (1, N)).astype(np.float32))
    z = orc.f32_to_f16(np.zeros((1, N), np.float32))
    base = orc.wqbmm(x, orc.F16, w, orc.I8, M, K, N, False, s, orc.F16, N, None, 0, None, 0)
    # zero offset == no offset; one group spanning K-ish == per-channel (two groups with equal scales)
    assert np.array_equal(orc.wqbmm(x, orc.F16, w, orc.I8, M, K, N, False, s, orc.F16, N, z, 0, None, 0), base)
    s2 = np.repeat(s, 2, 0)
    assert np.array_equal(orc.wqbmm(x, orc.F16, w, orc.I8, M, K, N, False, s2, orc.F16, N, None, 64, None, 0), base)
    # against float64 on the dequantised weight
    wd = (w.astype(np.float32) * orc.f16_to_f32(s)).astype(np.float16).astype(np.float64)
    ref = orc.f16_to_f32(x).astype(np.float64) @ wd
    got = orc.f16_to_f32(base)
    assert np.max(np.abs(got - ref) / np.maximum(np.abs(ref), 0.05)) < 2e-3
    # bias is added in fp32 before the final cast; bf16 outputs take one extra rounding through bf16 (a no-op on bits)
    bias = rng.normal(0, 0.1, N).astype(np.float32)
    yb = orc.f16_to_f32(orc.wqbmm(x, orc.F16, w, orc.I8, M, K, N, False, s, orc.F16, N, None, 0, bias, orc.F32))
    assert np.max(np.abs(yb - (ref + bias)) / np.maximum(np.abs(ref + bias), 0.05)) < 2e-3
