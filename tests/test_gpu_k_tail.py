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


@pytest.mark.parametrize("M,K,N,s_len,pt", [(256, 1000, 264, "N", "M"), (128, 72, 512, "N", True)])
def test_fp8_row_and_column_scales_k_tail(gpu, M, K, N, s_len, pt):
    m = gpu
    print(f"case fp8 row/col scale K tail M={M} K={K} N={N} s_len={s_len} pertoken={pt}", flush=True)
    inp = cases.make_tc_inputs(m, M, K, N, K, m.ACL_FLOAT8_E4M3FN, m.ACL_FLOAT, N if s_len == "N" else 1, None, True, pertoken=pt)
    want = cases.oracle_tc(m, inp, M, K, N, m.ACL_BF16)
    got = cases.run_tc_aclnn(m, inp, M, K, N, m.ACL_BF16)
    check_close(got, want, orc.BF16, "fp8 row and column scales with a K tail")
