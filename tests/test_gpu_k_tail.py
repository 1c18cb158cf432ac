"""K that is not a multiple of the matrix-core kernels' K tile (128 bytes; int8: 16): both operands are first copied into
zero-padded K-contiguous rows in the workspace, then the matrix-core kernels run -- not the one-thread-per-output kernel.

The evidence that the padded route is the one taken: phase 1 asks for a workspace of exactly the two padded copies
(a K-contiguous right operand with K % 128 == 0 needs none).  Results: int8 bit-identical to the oracle (integer sums, the
same epilogue), fp8 at the bar of the matrix-core path.
"""
import numpy as np
import pytest

import cases
import oracle_api as orc
from test_gpu_other_modes import check_close

pytestmark = pytest.mark.gpu


def _pad_bytes(M, K, N, batch=1):
    Kp = -(-K // 128) * 128
    return -(-(batch * M * Kp) // 256) * 256 + batch * N * Kp


@pytest.mark.parametrize("M,K,N,tB,bias,out", [
    (256, 4100, 512, True, "bf16", "bf16"),     # K % 16 = 4, K-contiguous x2
    (130, 1001, 264, False, None, "f16"),       # odd K, N-contiguous x2 (gathered, not transposed), ragged tiles
    (64, 24, 64, True, "f32", "bf16"),          # one padded K tile
])
def test_int8_k_tail(gpu, M, K, N, tB, bias, out):
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "f32": m.ACL_FLOAT, None: None}
    print(f"case int8 K tail M={M} K={K} N={N} tB={tB} bias={bias} out={out}", flush=True)
    inp = cases.make_qmm_int8_inputs(m, M, K, N, K, dt[bias], tB)
    want, _ = cases.oracle_qmm_int8(m, inp, M, K, N, tB, dt[out])
    got = cases.run_qmm_int8_aclnn(m, inp, M, K, N, tB, dt[out])
    assert np.array_equal(got, want), "int8 with a K tail must stay bit-identical"
    # phase 1 plans the padded copies
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    x1 = m.Tensor((M, K), m.ACL_INT8, d["x1"])
    x2 = m.Tensor((N, K) if tB else (K, N), m.ACL_INT8, d["x2"])
    s1 = m.Tensor((M,), m.ACL_FLOAT, d["s1"]) if inp["s1"] is not None else None
    s2 = m.Tensor((inp["s2"].size,), inp["s2_dtype"], d["s2"])
    o = m.Tensor((M, N), dt[out], m.DeviceBuffer(M * N * 2))
    b = m.Tensor((N,), inp["bias_dtype"], d["bias"]) if inp["bias"] is not None else None
    rc, ws, ex = m.quant_matmul_v5_get_workspace(x1, x2, s1, s2, o, bias=b, transpose_x2=tB)
    assert rc == 0 and ws == _pad_bytes(M, K, N)
    m.lib().aclDestroyAclOpExecutor(ex)


@pytest.mark.parametrize("fast", [False, True])
@pytest.mark.parametrize("M,K,N,tB,gsM", [
    (256, 1000, 384, True, 1),        # G-B, 7 full K groups + 104
    (300, 200, 260, False, 1),        # N-contiguous x2, ragged everywhere
    (256, 448, 256, True, 128),       # B-B, K = 3.5 groups
])
def test_fp8_blockscale_k_tail(gpu, M, K, N, tB, gsM, fast):
    m = gpu
    print(f"case fp8 block K tail M={M} K={K} N={N} tB={tB} gsM={gsM} fast={fast}", flush=True)
    inp = cases.make_blockscale_inputs(m, M, K, N, K + N, tB, gsM)
    want = cases.oracle_blockscale(m, inp, M, K, N, tB, m.ACL_BF16)
    m.lib().opsnnSetFp8Fast(1 if fast else 0)
    try:
        got = cases.run_blockscale_aclnn(m, inp, M, K, N, tB, m.ACL_BF16)
    finally:
        m.lib().opsnnSetFp8Fast(0)
    check_close(got, want, orc.BF16, "fp8 block scale with a K tail", fp8_mfma=fast)
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    x1 = m.Tensor((M, K), m.ACL_FLOAT8_E4M3FN, d["x1"])
    x2 = m.Tensor((N, K) if tB else (K, N), m.ACL_FLOAT8_E4M3FN, d["x2"])
    s1 = m.Tensor(inp["s1"].shape[1:], m.ACL_FLOAT, d["s1"])
    s2 = m.Tensor(inp["s2"].shape[1:], m.ACL_FLOAT, d["s2"])
    o = m.Tensor((M, N), m.ACL_BF16, m.DeviceBuffer(M * N * 2))
    rc, ws, ex = m.quant_matmul_v5_get_workspace(x1, x2, s1, s2, o, transpose_x2=tB, group_size=(gsM << 32) | (128 << 16) | 128)
    assert rc == 0 and ws == _pad_bytes(M, K, N)
    m.lib().aclDestroyAclOpExecutor(ex)


def _splitk_bytes(M, K, N, bm, bn, batch=1, tile_us=1.4, kunit=128, bytes_per_us=5.0e6):
    """The partial sums that phase 1 puts in front of the workspace when a call of a mode that can split K has few tiles
    against a long K (splitk_factor in launch.h): at most 128 tiles, K >= 1024, 2 .. 16 splits of at least four K tiles, the
    count with the largest estimated gain (loop time saved less a launch and the partial sums' traffic), if at least 3 us.
    bm x bn: the mode's tile; tile_us: one K tile of its kernel (1.4 the exact fp8 kernel, 1.8 fp8 x fp4 MX and int8
    per-tile, 0.55 int8 per-token / per-channel on 128 x 128 tiles -- that one with bytes_per_us = 2.4e6)."""
    if (M <= 32 and bm != 128) or M * N < 64 * 64 or K < 1024:
        return 0
    tiles = -(-M // bm) * -(-N // bn) * batch
    if tiles > 128:
        return 0
    kt = -(-K // kunit)
    best, best_gain = 1, 3.0
    for s in range(2, min(256 // tiles, kt // 4, 16) + 1):
        gain = kt * tile_us * (1.0 - 1.0 / s) - 4.0 - 2.0 * s * (M * N * batch) * 4.0 / bytes_per_us
        if gain > best_gain:
            best, best_gain = s, gain
    return -(-(best * batch * M * N * 4) // 256) * 256 if best >= 2 else 0


def _mx_pad_bytes(M, K, N, fp4, batch=1):
    Kp, epb = -(-K // 128) * 128, 2 if fp4 else 1
    up = lambda v: -(-v // 256) * 256
    return up(batch * M * Kp // epb) + up(batch * N * Kp // epb) + up(batch * M * (Kp // 64) * 2) + up(batch * N * (Kp // 64) * 2)


def _mx_exact_bytes(M, K, N, batch=1):
    """What the exact route of MXFP8 puts in front of the workspace: 127 - base and 2^(base - 127) per row of both
    operands and one flag per 64 rows (+ 2)."""
    up = lambda v: -(-v // 256) * 256
    rows = batch * (M + N)
    return up(rows * 8) + up((-(-rows // 64) + 2) * 4)


@pytest.mark.parametrize("M,K,N,fp4,batch,bias", [
    (197, 960, 854, True, 1, True),      # MXFP4, 7.5 K tiles, ragged rows and columns
    (256, 1472, 384, False, 1, False),   # MXFP8, 11.5 K tiles
    (128, 192, 256, True, 2, True),      # batched, 1.5 K tiles
    (64, 64, 64, False, 1, False),       # half a K tile
    (384, 544, 512, True, 1, True),      # K % 64 == 32: the last scale pair is half used
    (200, 96, 320, False, 2, True),      # the same for MXFP8, batched, three quarters of a K tile
    (130, 32, 70, True, 1, False),       # one MX block
])
def test_mx_k_tail(gpu, M, K, N, fp4, batch, bias):
    """MX operands with K % 128 != 0 (whole 32-element blocks): both operands and both scale tables are copied with K
    rounded up to 128 (zero elements; their scales repeat the row's last one, also in the unused half of a half-used
    pair, which the caller may have left at any value), then the matrix-core kernels run."""
    m = gpu
    print(f"case mx K tail M={M} K={K} N={N} fp4={fp4} batch={batch} bias={bias}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, K + N, True, fp4, batch=batch)
    if K % 64:   # the byte behind the last block scales nothing: a NaN code there must not reach any sum
        inp["s1"][..., -1, 1] = 0xFF
        inp["s2"][..., -1, 1] = 0xFF
    b = np.random.default_rng(3).normal(0, 1, N).astype(np.float32) if bias else None
    want = cases.oracle_mx(m, inp, M, K, N, True, m.ACL_BF16, b)
    got = cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16, b)
    check_close(got, want, orc.BF16, "mx with a K tail")   # fp8: the exact route behind the padded copies
    # phase 1 plans the four padded copies
    adt = m.ACL_FLOAT4_E2M1 if fp4 else m.ACL_FLOAT8_E4M3FN
    bs = (batch,) if batch > 1 else ()
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    x1 = m.Tensor(bs + (M, K), adt, d["x1"]); x2 = m.Tensor(bs + (N, K), adt, d["x2"])
    s1 = m.Tensor(bs + inp["s1"].shape[1:], m.ACL_FLOAT8_E8M0, d["s1"]); s2 = m.Tensor(bs + inp["s2"].shape[1:], m.ACL_FLOAT8_E8M0, d["s2"])
    o = m.Tensor(bs + (M, N), m.ACL_BF16, m.DeviceBuffer(batch * M * N * 2))
    rc, ws, ex = m.quant_matmul_v5_get_workspace(x1, x2, s1, s2, o, transpose_x2=True, group_size=(1 << 32) | (1 << 16) | 32)
    plan = _mx_pad_bytes(M, K, N, fp4, batch) + (0 if fp4 else _mx_exact_bytes(M, K, N, batch) + _splitk_bytes(M, K, N, 256, 128, batch))
    assert rc == 0 and ws == plan, (rc, ws, plan)
    m.lib().aclDestroyAclOpExecutor(ex)


@pytest.mark.parametrize("M,K,N,fp4,batch", [
    (197, 960, 854, True, 1),      # MXFP4, ragged rows and columns
    (256, 1472, 384, False, 1),    # MXFP8
    (128, 192, 256, True, 2),      # batched
    (64, 64, 128, False, 3),       # half a K tile, batched
    (384, 544, 512, True, 1),      # K % 64 == 32
    (96, 96, 192, False, 2),       # the same for MXFP8, batched
])
def test_mx_k_tail_n_contiguous_x2(gpu, M, K, N, fp4, batch):
    """K % 128 != 0 with x2 stored [K, N] (N contiguous, scales [K/64, N, 2]): x2 and its scales are first re-laid out
    K-contiguous, then all four operands are padded as for K-contiguous callers; the matrix-core kernels run (the log line
    of a plain-kernel landing must not appear: checked through the workspace plan, which is zero for the plain route)."""
    m = gpu
    print(f"case mx K tail, N-contiguous x2 M={M} K={K} N={N} fp4={fp4} batch={batch}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, K + N + 1, False, fp4, batch=batch)
    b = np.random.default_rng(5).normal(0, 1, N).astype(np.float32)
    want = cases.oracle_mx(m, inp, M, K, N, False, m.ACL_BF16, b)
    got = cases.run_mx_aclnn(m, inp, M, K, N, False, m.ACL_BF16, b)
    check_close(got, want, orc.BF16, "mx with a K tail, N-contiguous x2")
    adt = m.ACL_FLOAT4_E2M1 if fp4 else m.ACL_FLOAT8_E4M3FN
    bs = (batch,) if batch > 1 else ()
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    x1 = m.Tensor(bs + (M, K), adt, d["x1"]); x2 = m.Tensor(bs + (K, N), adt, d["x2"])
    s1 = m.Tensor(bs + inp["s1"].shape[1:], m.ACL_FLOAT8_E8M0, d["s1"]); s2 = m.Tensor(bs + inp["s2"].shape[1:], m.ACL_FLOAT8_E8M0, d["s2"])
    o = m.Tensor(bs + (M, N), m.ACL_BF16, m.DeviceBuffer(batch * M * N * 2))
    rc, ws, ex = m.quant_matmul_v5_get_workspace(x1, x2, s1, s2, o, transpose_x2=False, group_size=(1 << 32) | (1 << 16) | 32)
    up = lambda v: -(-v // 256) * 256
    relaid = up(batch * up(N * K // (2 if fp4 else 1)) + batch * up(N * -(-K // 64) * 2))
    plan = relaid + _mx_pad_bytes(M, K, N, fp4, batch) + (0 if fp4 else _mx_exact_bytes(M, K, N, batch) + _splitk_bytes(M, K, N, 256, 128, batch))
    assert rc == 0 and ws == plan, (rc, ws, plan)
    m.lib().aclDestroyAclOpExecutor(ex)


@pytest.mark.parametrize("M,K,N", [(300, 960, 260), (128, 192, 256), (16, 1984, 512), (96, 544, 320)])
def test_mx_fp8_fp4_k_tail(gpu, M, K, N):
    """fp8 x fp4 MX with K % 128 != 0: the same padded copies (x1 rows of K + 64 bytes, x2 rows of half that), then the
    matrix-core kernel of the mode (the stream kernel with 16 rows): the stated bar."""
    m = gpu
    print(f"case fp8 x fp4 mx K tail M={M} K={K} N={N}", flush=True)
    inp = cases.make_a8w4_mx_inputs(m, M, K, N, K + N, True)
    want = cases.oracle_a8w4_mx(m, inp, M, K, N, True, m.ACL_FLOAT16)
    got = cases.run_a8w4_mx_aclnn(m, inp, M, K, N, True, m.ACL_FLOAT16)
    check_close(got, want, orc.F16, "fp8 x fp4 mx with a K tail")
    # phase 1 plans the four padded copies
    up = lambda v: -(-v // 256) * 256
    Kp = -(-K // 128) * 128
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items()}
    x1 = m.Tensor((M, K), m.ACL_FLOAT8_E4M3FN, d["x1"]); x2 = m.Tensor((N, K), m.ACL_FLOAT4_E2M1, d["x2"])
    s1 = m.Tensor(inp["s1"].shape, m.ACL_FLOAT8_E8M0, d["s1"]); s2 = m.Tensor(inp["s2"].shape, m.ACL_FLOAT8_E8M0, d["s2"])
    bias = m.Tensor((1, N), m.ACL_FLOAT16, d["bias"])
    o = m.Tensor((M, N), m.ACL_FLOAT16, m.DeviceBuffer(M * N * 2))
    rc, ws, ex = m.quant_matmul_v5_get_workspace(x1, x2, s1, s2, o, bias=bias, transpose_x2=True, group_size=32)
    assert rc == 0 and ws == up(M * Kp) + up(N * Kp // 2) + up(M * (Kp // 64) * 2) + up(N * (Kp // 64) * 2) + _splitk_bytes(M, K, N, 256, 256, tile_us=1.8), (rc, ws)
    m.lib().aclDestroyAclOpExecutor(ex)
    m.lib().opsnnSetForcePlain(1)
    try:
        exact = cases.run_a8w4_mx_aclnn(m, inp, M, K, N, True, m.ACL_FLOAT16)
    finally:
        m.lib().opsnnSetForcePlain(0)
    assert np.array_equal(exact, want)


@pytest.mark.parametrize("M,K,N,s_len,pt", [(256, 1000, 264, "N", "M"), (128, 72, 512, "N", True)])
def test_fp8_row_and_column_scales_k_tail(gpu, M, K, N, s_len, pt):
    m = gpu
    print(f"case fp8 row/col scale K tail M={M} K={K} N={N} s_len={s_len} pertoken={pt}", flush=True)
    inp = cases.make_tc_inputs(m, M, K, N, K, m.ACL_FLOAT8_E4M3FN, m.ACL_FLOAT, N if s_len == "N" else 1, None, True, pertoken=pt)
    want = cases.oracle_tc(m, inp, M, K, N, m.ACL_BF16)
    got = cases.run_tc_aclnn(m, inp, M, K, N, m.ACL_BF16)
    check_close(got, want, orc.BF16, "fp8 row and column scales with a K tail")


def _strided_case(m, M, K, N, x1_pad, x2_step, batch=1):
    """int8 operands as regular strided views: x1 rows of K inside storage rows of K + x1_pad, x2 [K, N] as every
    x2_step-th column of a [K, N * x2_step] storage.  Returns (logical inputs, device tensors, storages kept alive)."""
    inp = cases.make_qmm_int8_inputs(m, M, K, N, M + K, m.ACL_BF16, False, batch=batch)
    rng = np.random.default_rng(5)
    s1 = rng.integers(-128, 128, size=(batch, M, K + x1_pad), dtype=np.int8)
    s1[:, :, :K] = inp["x1"]
    s2 = rng.integers(-128, 128, size=(batch, K, N * x2_step), dtype=np.int8)
    s2[:, :, ::x2_step] = inp["x2"]
    d1, d2 = m.DeviceBuffer(host=s1), m.DeviceBuffer(host=s2)
    bshape = (batch,) if batch > 1 else ()
    bs1 = (M * (K + x1_pad),) if batch > 1 else ()
    bs2 = (K * N * x2_step,) if batch > 1 else ()
    x1 = m.Tensor(bshape + (M, K), m.ACL_INT8, d1, strides=bs1 + (K + x1_pad, 1), storage_shape=bshape + (M, K + x1_pad))
    x2 = m.Tensor(bshape + (K, N), m.ACL_INT8, d2, strides=bs2 + (N * x2_step, x2_step), storage_shape=bshape + (K, N * x2_step))
    return inp, x1, x2, (d1, d2)


@pytest.mark.parametrize("M,K,N,x1_pad,x2_step,batch", [
    (256, 512, 384, 48, 2, 1),     # x1 rows 16-byte aligned but not dense (taken as it lies), x2 every other column (gathered)
    (130, 1000, 264, 7, 3, 1),     # nothing aligned, a K tail on top
    (128, 256, 192, 16, 2, 3),     # batched
])
def test_int8_regular_strided_views(gpu, M, K, N, x1_pad, x2_step, batch):
    """Views that are neither dense nor a dense transpose (the reference copies them contiguous; here they are gathered
    into the workspace on the way to the matrix cores): same bits as the dense call."""
    m = gpu
    print(f"case int8 strided views M={M} K={K} N={N} x1_pad={x1_pad} x2_step={x2_step} batch={batch}", flush=True)
    inp, x1, x2, keep = _strided_case(m, M, K, N, x1_pad, x2_step, batch)
    want, _ = cases.oracle_qmm_int8(m, inp, M, K, N, False, m.ACL_BF16)
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray) and k not in ("x1", "x2")}
    bshape = (batch,) if batch > 1 else ()
    d_out = m.DeviceBuffer(batch * M * N * 2)
    d_out.fill(0xFF)
    s1 = m.Tensor((M,), m.ACL_FLOAT, d["s1"])
    s2 = m.Tensor((inp["s2"].size,), inp["s2_dtype"], d["s2"])
    b = m.Tensor((N,), inp["bias_dtype"], d["bias"])
    out = m.Tensor(bshape + (M, N), m.ACL_BF16, d_out)
    rc, ws, ex = m.quant_matmul_v5_get_workspace(x1, x2, s1, s2, out, bias=b)
    assert rc == 0 and ws == _pad_bytes(M, K, N, batch), (rc, ws)
    m.lib().aclDestroyAclOpExecutor(ex)
    wbuf = m.quant_matmul_v5(x1, x2, s1, s2, out, bias=b)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    got = d_out.to_host(np.uint16, (batch, M, N))
    assert np.array_equal(got, want)
    # and on the plain kernels, which index the views directly
    m.lib().opsnnSetForcePlain(1)
    try:
        d_out.fill(0xFF)
        wbuf = m.quant_matmul_v5(x1, x2, s1, s2, out, bias=b)
        m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    finally:
        m.lib().opsnnSetForcePlain(0)
    assert np.array_equal(d_out.to_host(np.uint16, (batch, M, N)), want)


@pytest.mark.parametrize("M,K,N,x1_off,x1_pad,x2_step,batch", [
    (256, 512, 384, 0, 64, 2, 1),    # x1 rows byte-aligned but not dense, x2 every other stored row
    (130, 320, 264, 3, 10, 3, 1),    # x1 starts on an odd nibble, its row pitch is 5 bytes more than the row; a K tail on top
    (128, 256, 192, 2, 32, 2, 3),    # batched
])
def test_fp4_strided_views(gpu, M, K, N, x1_off, x1_pad, x2_step, batch):
    """Strided views of 4-bit operands (MXFP4): the reference copies any non-contiguous operand contiguous first
    (quant_matmul_common_check.cpp:106-123); here phase 2 gathers them nibble by nibble into dense copies at the front of the
    workspace, then the call goes on as the dense one: same bits as the dense call."""
    m = gpu
    print(f"case fp4 strided views M={M} K={K} N={N} x1_off={x1_off} x1_pad={x1_pad} x2_step={x2_step} batch={batch}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, M + K, True, True, batch=batch)
    b = np.random.default_rng(8).normal(0, 1, N).astype(np.float32)
    want = cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16, b)
    check_close(want, cases.oracle_mx(m, inp, M, K, N, True, m.ACL_BF16, b), orc.BF16, "mxfp4 dense")
    rng = np.random.default_rng(9)
    # nibble images: x1 rows of K + x1_pad nibbles behind x1_off nibbles; x2 rows at every x2_step-th stored row
    n1 = rng.integers(0, 16, size=(batch, M * (K + x1_pad) + x1_off + 1), dtype=np.uint8)
    c1 = orc.unpack_nibbles(inp["x1"]).reshape(batch, M, K)
    for r in range(M):
        n1[:, x1_off + r * (K + x1_pad): x1_off + r * (K + x1_pad) + K] = c1[:, r]
    if n1.shape[1] % 2:
        n1 = n1[:, :-1]
    n2 = rng.integers(0, 16, size=(batch, N * x2_step, K), dtype=np.uint8)
    n2[:, ::x2_step] = orc.unpack_nibbles(inp["x2"]).reshape(batch, N, K)
    d1, d2 = m.DeviceBuffer(host=orc.pack_nibbles(n1)), m.DeviceBuffer(host=orc.pack_nibbles(n2))
    bs = (batch,) if batch > 1 else ()
    x1 = m.Tensor(bs + (M, K), m.ACL_FLOAT4_E2M1, d1, strides=((n1.shape[1],) if batch > 1 else ()) + (K + x1_pad, 1), offset=x1_off,
                  storage_shape=(batch * n1.shape[1],))
    x2 = m.Tensor(bs + (N, K), m.ACL_FLOAT4_E2M1, d2, strides=((N * x2_step * K,) if batch > 1 else ()) + (K * x2_step, 1),
                  storage_shape=bs + (N * x2_step, K))
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray) and k in ("s1", "s2")}
    s1 = m.Tensor(bs + inp["s1"].shape[1:], m.ACL_FLOAT8_E8M0, d["s1"]); s2 = m.Tensor(bs + inp["s2"].shape[1:], m.ACL_FLOAT8_E8M0, d["s2"])
    d_out = m.DeviceBuffer(batch * M * N * 2); d_out.fill(0xFF)
    out = m.Tensor(bs + (M, N), m.ACL_BF16, d_out)
    d_b = m.DeviceBuffer(host=b); t_b = m.Tensor((N,), m.ACL_FLOAT, d_b)
    gs = (1 << 32) | (1 << 16) | 32
    rc, ws, ex = m.quant_matmul_v5_get_workspace(x1, x2, s1, s2, out, bias=t_b, transpose_x2=True, group_size=gs)
    up = lambda v: -(-v // 256) * 256
    assert rc == 0 and ws >= up(batch * M * K // 2) + up(batch * N * K // 2), (rc, ws, m.err_msg())
    m.lib().aclDestroyAclOpExecutor(ex)
    wbuf = m.quant_matmul_v5(x1, x2, s1, s2, out, bias=t_b, transpose_x2=True, group_size=gs)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    assert np.array_equal(d_out.to_host(np.uint16, (batch, M, N)), want)
    del wbuf


@pytest.mark.parametrize("mode", ["mxfp8", "blockscale"])
@pytest.mark.parametrize("M,K,N,x1_off,x1_pad,x2_step,batch,expand", [
    (256, 512, 384, 0, 64, 2, 1, False),
    (130, 320, 264, 3, 5, 3, 1, False),     # nothing aligned, a K tail (MX) / a ragged last K block (block scales) on top
    (128, 256, 192, 16, 32, 2, 3, True),    # batched, x2 one matrix expanded over the batch (batch stride 0)
])
def test_fp8_strided_views_mx_and_blockscale(gpu, mode, M, K, N, x1_off, x1_pad, x2_step, batch, expand):
    """Strided views of fp8 operands in the MX mode (gathered by phase 2 into the front of the workspace) and in the
    block-scale mode (gathered by its launcher): same bits as the dense call; a batch dim of stride 0 included."""
    m = gpu
    print(f"case fp8 strided views {mode} M={M} K={K} N={N} x1_off={x1_off} x1_pad={x1_pad} x2_step={x2_step} batch={batch} expand={expand}", flush=True)
    if mode == "mxfp8":
        inp = cases.make_mx_inputs(m, M, K, N, M + K + 1, True, False, batch=batch)
        sdt, gs = m.ACL_FLOAT8_E8M0, (1 << 32) | (1 << 16) | 32
    else:
        inp = cases.make_blockscale_inputs(m, M, K, N, M + K + 2, True, batch=batch)
        sdt, gs = m.ACL_FLOAT, (1 << 32) | (128 << 16) | 128
    if expand:
        inp["x2"][1:] = inp["x2"][0]
        inp["s2"][1:] = inp["s2"][0]
    if mode == "mxfp8":
        want = cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    else:
        want = cases.run_blockscale_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    rng = np.random.default_rng(10)
    L1 = M * (K + x1_pad) + x1_off
    b1 = rng.integers(0, 120, size=(batch, L1), dtype=np.uint8)
    for r in range(M):
        b1[:, x1_off + r * (K + x1_pad): x1_off + r * (K + x1_pad) + K] = inp["x1"][:, r]
    nb2 = 1 if expand else batch
    b2 = rng.integers(0, 120, size=(nb2, N * x2_step, K), dtype=np.uint8)
    b2[:, ::x2_step] = inp["x2"][:nb2]
    d1, d2 = m.DeviceBuffer(host=b1), m.DeviceBuffer(host=b2)
    bs = (batch,) if batch > 1 else ()
    x1 = m.Tensor(bs + (M, K), m.ACL_FLOAT8_E4M3FN, d1, strides=((L1,) if batch > 1 else ()) + (K + x1_pad, 1), offset=x1_off, storage_shape=(batch * L1,))
    x2 = m.Tensor(bs + (N, K), m.ACL_FLOAT8_E4M3FN, d2, strides=((0 if expand else N * x2_step * K,) if batch > 1 else ()) + (K * x2_step, 1),
                  storage_shape=(nb2, N * x2_step, K))
    ds1, ds2 = m.DeviceBuffer(host=inp["s1"]), m.DeviceBuffer(host=inp["s2"])
    s1 = m.Tensor(bs + inp["s1"].shape[1:], sdt, ds1); s2 = m.Tensor(bs + inp["s2"].shape[1:], sdt, ds2)
    d_out = m.DeviceBuffer(batch * M * N * 2); d_out.fill(0xFF)
    out = m.Tensor(bs + (M, N), m.ACL_BF16, d_out)
    wbuf = m.quant_matmul_v5(x1, x2, s1, s2, out, transpose_x2=True, group_size=gs)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    assert np.array_equal(d_out.to_host(np.uint16, (batch, M, N)), want)
    del wbuf


def test_irregular_views_are_still_rejected(gpu):
    m = gpu
    d = m.DeviceBuffer(4096 * 16)
    x1 = m.Tensor((2, 2, 16, 32), m.ACL_INT8, d, strides=(4096, 1000, 64, 1), storage_shape=(16, 4096))   # batch dims do not collapse
    x2 = m.Tensor((32, 16), m.ACL_INT8, d)
    s2 = m.Tensor((16,), m.ACL_FLOAT, d)
    out = m.Tensor((2, 2, 16, 16), m.ACL_BF16, d)
    rc, ws, ex = m.quant_matmul_v5_get_workspace(x1, x2, None, s2, out)
    assert rc == 161002
