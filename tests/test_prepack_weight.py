"""aclnnPrepackMatmulWeight: the one-time [k, n] -> K-contiguous [n, k] re-layout (with the scales that run along k).

After it, the matmul entry points take the packed tensor with transposeX2 = true (or as a transposed view), report a zero
workspace, and must give bit for bit what they give on the [k, n] operand they would otherwise re-lay out per call.
"""
import numpy as np
import pytest

import cases
import oracle_api as orc
from test_nz_entry_points import NZ, nd_to_nz


def test_prepack_argument_rules(opsnn):
    m = opsnn
    K, N = 64, 48
    invalid, null = m.STATUS_BY_NAME["ACLNN_ERR_PARAM_INVALID"], m.STATUS_BY_NAME["ACLNN_ERR_PARAM_NULLPTR"]
    w = m.Tensor((K, N), m.ACL_INT8)
    assert m.prepack_matmul_weight(w, None)[0] == null
    assert m.prepack_matmul_weight(w, m.Tensor((K, N), m.ACL_INT8))[0] == invalid           # not swapped
    assert m.prepack_matmul_weight(w, m.Tensor((N, K), m.ACL_FLOAT8_E4M3FN))[0] == invalid    # dtype differs
    assert m.prepack_matmul_weight(w, m.Tensor((N, K), m.ACL_INT8), scale=m.Tensor((1, N, 2), m.ACL_FLOAT8_E8M0))[0] == null   # scale without its output
    assert m.prepack_matmul_weight(m.Tensor((63, N), m.ACL_INT4), m.Tensor((N, 63), m.ACL_INT4))[0] == invalid   # odd k, 4-bit
    assert m.prepack_matmul_weight(w, m.Tensor((N, K), m.ACL_INT8), scale=m.Tensor((2, N, 2), m.ACL_FLOAT8_E8M0),
                                   scale_packed=m.Tensor((N, 2, 2), m.ACL_FLOAT8_E8M0))[0] == invalid   # ceil(64 / 64) = 1 scale pair per column


@pytest.mark.gpu
@pytest.mark.parametrize("from_nz", [False, True])
def test_gpu_prepacked_int8_matches_per_call_relayout(gpu, from_nz):
    m = gpu
    M, K, N = 300, 512, 712
    inp = cases.make_qmm_int8_inputs(m, M, K, N, 3, m.ACL_BF16, False)
    want = cases.run_qmm_int8_aclnn(m, inp, M, K, N, False, m.ACL_BF16)                      # [k, n]: re-laid out inside the call
    x2 = inp["x2"][0]
    d_packed = m.DeviceBuffer(N * K)
    d_packed.fill(0xEE)
    if from_nz:
        nz = nd_to_nz(x2.view(np.uint8), 32)
        d_src = m.DeviceBuffer(host=nz)
        t_src = m.Tensor((K, N), m.ACL_INT8, d_src, fmt=NZ, storage_shape=(nz.shape[0], nz.shape[1], 16, 32))
    else:
        d_src = m.DeviceBuffer(host=x2)
        t_src = m.Tensor((K, N), m.ACL_INT8, d_src)
    rc, ws = m.prepack_matmul_weight(t_src, m.Tensor((N, K), m.ACL_INT8, d_packed))
    assert rc == 0, m.err_msg()
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    packed = d_packed.to_host(np.int8, (N, K))
    assert np.array_equal(packed, x2.T)
    got = cases.run_qmm_int8_aclnn(m, dict(inp, x2=packed[None]), M, K, N, True, m.ACL_BF16)
    assert np.array_equal(got, want)
    # and that call needs no workspace any more
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray) and k != "x2"}
    rc, wsz, ex = m.quant_matmul_v5_get_workspace(m.Tensor((M, K), m.ACL_INT8, d["x1"]), m.Tensor((N, K), m.ACL_INT8, d_packed),
                                                  m.Tensor((M,), m.ACL_FLOAT, d["s1"]), m.Tensor((N,), m.ACL_FLOAT, d["s2"]),
                                                  m.Tensor((M, N), m.ACL_BF16, m.DeviceBuffer(M * N * 2)), transpose_x2=True)
    assert rc == 0 and wsz == 0
    m.lib().aclDestroyAclOpExecutor(ex)


@pytest.mark.gpu
def test_gpu_prepacked_mxfp4_with_scales(gpu):
    m = gpu
    M, K, N, B = 128, 512, 256, 2
    inp = cases.make_mx_inputs(m, M, K, N, 7, False, True, batch=B)             # x2 [B, K, N / 2] bytes, s2 [B, K/64, N, 2]
    want = cases.run_mx_aclnn(m, inp, M, K, N, False, m.ACL_BF16)
    KS = K // 64
    d_x2, d_s2 = m.DeviceBuffer(host=inp["x2"]), m.DeviceBuffer(host=inp["s2"])
    d_px, d_ps = m.DeviceBuffer(B * N * K // 2), m.DeviceBuffer(B * N * KS * 2)
    rc, ws = m.prepack_matmul_weight(m.Tensor((B, K, N), m.ACL_FLOAT4_E2M1, d_x2), m.Tensor((B, N, K), m.ACL_FLOAT4_E2M1, d_px),
                                     scale=m.Tensor((B, KS, N, 2), m.ACL_FLOAT8_E8M0, d_s2),
                                     scale_packed=m.Tensor((B, N, KS, 2), m.ACL_FLOAT8_E8M0, d_ps))
    assert rc == 0, m.err_msg()
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    px, ps = d_px.to_host(np.uint8, (B, N, K // 2)), d_ps.to_host(np.uint8, (B, N, KS, 2))
    assert np.array_equal(ps, inp["s2"].transpose(0, 2, 1, 3))
    assert np.array_equal(orc.unpack_nibbles(px).reshape(B, N, K), orc.unpack_nibbles(inp["x2"]).reshape(B, K, N).transpose(0, 2, 1))
    got = cases.run_mx_aclnn(m, dict(inp, x2=px, s2=ps), M, K, N, True, m.ACL_BF16)
    assert np.array_equal(got, want)


@pytest.mark.gpu
def test_gpu_prepacked_w4a16_group_scales(gpu):
    """Weight-only: pack the int4 [k, n] weight with its [G, n] scale, then the offset by a second call; the packed tensors
    go to aclnnWeightQuantBatchMatmulV2 as transposed views."""
    m = gpu
    M, K, N, g = 16, 1024, 512, 128
    inp = cases.make_wq_inputs(m, M, K, N, 9, m.ACL_FLOAT16, m.ACL_INT4, g, False, True, None)
    want = cases.run_wq_aclnn(m, inp, M, K, N)
    G = K // g
    d_w, d_s, d_o = m.DeviceBuffer(host=inp["w"]), m.DeviceBuffer(host=inp["scale"]), m.DeviceBuffer(host=inp["offset"])
    d_pw, d_ps, d_po = m.DeviceBuffer(N * K // 2), m.DeviceBuffer(N * G * 2), m.DeviceBuffer(N * G * 2)
    t_w, t_pw = m.Tensor((K, N), m.ACL_INT4, d_w), m.Tensor((N, K), m.ACL_INT4, d_pw)
    assert m.prepack_matmul_weight(t_w, t_pw, scale=m.Tensor((G, N), m.ACL_FLOAT16, d_s), scale_packed=m.Tensor((N, G), m.ACL_FLOAT16, d_ps))[0] == 0
    assert m.prepack_matmul_weight(t_w, t_pw, scale=m.Tensor((G, N), m.ACL_FLOAT16, d_o), scale_packed=m.Tensor((N, G), m.ACL_FLOAT16, d_po))[0] == 0
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    packed = dict(inp, w=d_pw.to_host(np.uint8, (N, K // 2)), scale=d_ps.to_host(np.uint16, (N, G)), offset=d_po.to_host(np.uint16, (N, G)), tW=True)
    assert np.array_equal(packed["scale"], inp["scale"].T)
    got = cases.run_wq_aclnn(m, packed, M, K, N)
    assert np.array_equal(got, want)
