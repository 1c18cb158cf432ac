"""FRACTAL_NZ right operands: opsnnNzToNd / opsnnNdToNz, aclnnConvertWeightToINT4Pack with an NZ output,
aclnnWeightQuantBatchMatmulNz and aclnnQuantMatmulWeightNz.

The layout is the reference's: nz[b // c0][r // 16][r % 16][b % c0] = nd[r][b] over the bytes of the stored matrix, padding
zero (matmul/common/tests/st/arch35/matmul_golden_util.py:76-114 nz_to_nd, :284-313 nd_to_nz;
aclnn_convert_weight_to_int4_pack.cpp:318-366).  The numpy form used here is checked against that element formula written
out as loops; the NZ entry points must then give bit for bit what the ND entry points give on the same matrix.
"""
import ctypes as C

import numpy as np
import pytest

import cases
import oracle_api as orc

NZ = 29


def nd_to_nz(nd, c0):
    """[rows, row_bytes] uint8 -> [ceil(row_bytes / c0), ceil(rows / 16), 16, c0] uint8, zero padded."""
    rows, rb = nd.shape
    x1, y1 = -(-rb // c0), -(-rows // 16)
    pad = np.zeros((y1 * 16, x1 * c0), np.uint8)
    pad[:rows, :rb] = nd
    return np.ascontiguousarray(pad.reshape(y1, 16, x1, c0).transpose(2, 0, 1, 3))


def test_numpy_nz_form_equals_the_element_formula():
    rng = np.random.default_rng(0)
    for rows, rb, c0 in ((37, 50, 8), (16, 32, 32), (5, 9, 16)):
        nd = rng.integers(1, 256, (rows, rb), dtype=np.uint8)
        want = np.zeros((-(-rb // c0), -(-rows // 16), 16, c0), np.uint8)
        for i in range(rows):
            for j in range(rb):
                want[j // c0, i // 16, i % 16, j % c0] = nd[i, j]
        assert np.array_equal(nd_to_nz(nd, c0), want)


def test_nz_entry_points_reject_nd_and_bad_storage(opsnn):
    m = opsnn
    M, K, N = 8, 64, 48
    x1, s2, out = m.Tensor((M, K), m.ACL_INT8), m.Tensor((N,), m.ACL_FLOAT), m.Tensor((M, N), m.ACL_BF16)
    invalid = m.STATUS_BY_NAME["ACLNN_ERR_PARAM_INVALID"]
    rc, _, ex = m.quant_matmul_v5_get_workspace(x1, m.Tensor((K, N), m.ACL_INT8), None, s2, out, weight_nz=True)
    assert rc == invalid and "FRACTAL_NZ" in m.err_msg()
    bad = m.Tensor((K, N), m.ACL_INT8, fmt=NZ, storage_shape=(2, 4, 16, 16))        # 16-byte c0 for an 8-bit type, wrong counts
    rc, _, ex = m.quant_matmul_v5_get_workspace(x1, bad, None, s2, out, weight_nz=True)
    assert rc == invalid and "storage shape" in m.err_msg()
    good = m.Tensor((K, N), m.ACL_INT8, fmt=NZ, storage_shape=(2, 4, 16, 32))
    rc, ws, ex = m.quant_matmul_v5_get_workspace(x1, good, None, s2, out, weight_nz=True)
    assert rc == 0, m.err_msg()
    assert ws >= K * N
    m.lib().aclDestroyAclOpExecutor(ex)
    # the ND entry point keeps refusing NZ (aclnn_quant_matmul_v5.cpp:1201-1205)
    rc, _, ex = m.quant_matmul_v5_get_workspace(x1, good, None, s2, out)
    assert rc == invalid
    x, y = m.Tensor((M, K), m.ACL_FLOAT16), m.Tensor((M, N), m.ACL_FLOAT16)
    sc = m.Tensor((N,), m.ACL_FLOAT16)
    rc, _, ex = m.weight_quant_batch_matmul_get_workspace(x, m.Tensor((K, N), m.ACL_INT8), sc, y, weight_nz=True)
    assert rc == invalid and "FRACTAL_NZ" in m.err_msg()
    rc, ws, ex = m.weight_quant_batch_matmul_get_workspace(x, good, sc, y, weight_nz=True)
    assert rc == 0 and ws >= K * N, m.err_msg()
    m.lib().aclDestroyAclOpExecutor(ex)


@pytest.mark.gpu
@pytest.mark.parametrize("rows,rb,c0,batch", [(37, 50, 8, 1), (256, 512, 32, 2), (16, 32, 32, 1), (5, 9, 16, 3), (1000, 264, 8, 1)])
def test_gpu_relayout_kernels(gpu, rows, rb, c0, batch):
    m = gpu
    rng = np.random.default_rng(rows)
    nd = rng.integers(1, 256, (batch, rows, rb), dtype=np.uint8)
    nz = np.stack([nd_to_nz(nd[b], c0) for b in range(batch)])
    d_nd, d_nz = m.DeviceBuffer(host=nd), m.DeviceBuffer(nz.nbytes)
    d_nz.fill(0xAB)
    assert m.lib().opsnnNdToNz(d_nd.ptr, d_nz.ptr, rows, rb, c0, batch, None) == 0
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    assert np.array_equal(d_nz.to_host(np.uint8, nz.shape), nz)
    d_back = m.DeviceBuffer(nd.nbytes)
    d_back.fill(0xCD)
    assert m.lib().opsnnNzToNd(d_nz.ptr, d_back.ptr, rows, rb, c0, batch, None) == 0
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    assert np.array_equal(d_back.to_host(np.uint8, nd.shape), nd)


@pytest.mark.gpu
@pytest.mark.parametrize("K,N,pack_dt,c0e", [(64, 128, "i4", 16), (100, 72, "i4", 32), (64, 128, "i32", 2), (48, 64, "f4", 16)])
def test_gpu_convert_weight_to_nz(gpu, K, N, pack_dt, c0e):
    """The packed bytes of the ND result (pinned against the oracle in test_convert_weight.py), in fractal order."""
    m = gpu
    rng = np.random.default_rng(K + N)
    if pack_dt == "f4":
        w = orc.E2M1_VALUES[rng.integers(0, 16, (K, N))].astype(np.float32)
        w_dt, p_dt, shape = m.ACL_FLOAT, m.ACL_FLOAT4_E2M1, (K, N)
    else:
        w = rng.integers(-8, 8, (K, N)).astype(np.int32)
        w_dt = m.ACL_INT32
        p_dt, shape = (m.ACL_INT4, (K, N)) if pack_dt == "i4" else (m.ACL_INT32, (K, N // 8))
    nd_bytes = orc.convert_weight_b4(w)                                      # [K, N / 2]
    c0 = c0e * (4 if pack_dt == "i32" else 1) // (1 if pack_dt == "i32" else 2)   # bytes per fractal row
    want = nd_to_nz(nd_bytes, c0)
    d_w, d_p = m.DeviceBuffer(host=w), m.DeviceBuffer(want.nbytes)
    d_p.fill(0xEE)
    t_p = m.Tensor(shape, p_dt, d_p, fmt=NZ, storage_shape=(want.shape[0], want.shape[1], 16, c0e))
    assert m.convert_weight_to_int4_pack(m.Tensor((K, N), w_dt, d_w), t_p) == 0, m.err_msg()
    assert np.array_equal(d_p.to_host(np.uint8, want.shape), want)


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N,x_dt,w_dt,group,tW,off,c0e", [
    (16, 1024, 512, "f16", "i4", 128, False, True, 16),     # the documented form: [ceil(n/16), ceil(k/16), 16, 16]
    (1, 4096, 264, "f16", "i4", 128, False, True, 32),      # 32 elements per fractal row, ragged fractal count
    (33, 300, 100, "bf16", "i8", 0, False, False, 32),      # INT8 [k, n], ragged rows and columns
    (9, 256, 96, "f16", "i8", 0, True, True, 32),           # INT8 as the transposed view of an [n, k] matrix
    (4, 128, 64, "bf16", "fp4", 32, False, False, 16),      # mxfp4
])
def test_gpu_weight_quant_nz_equals_nd(gpu, M, K, N, x_dt, w_dt, group, tW, off, c0e):
    m = gpu
    dt = {"bf16": m.ACL_BF16, "f16": m.ACL_FLOAT16, "i8": m.ACL_INT8, "i4": m.ACL_INT4, "fp4": m.ACL_FLOAT4_E2M1}
    print(f"case wq nz M={M} K={K} N={N} x={x_dt} w={w_dt} g={group} tW={tW} c0={c0e}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M + N, dt[x_dt], dt[w_dt], group, tW, off, None)
    want = cases.run_wq_aclnn(m, inp, M, K, N)
    stored = inp["w"].reshape(N if tW else K, -1).view(np.uint8)             # the stored matrix's bytes
    c0 = c0e if w_dt == "i8" else c0e // 2
    nz = nd_to_nz(stored, c0)
    got = cases.run_wq_aclnn(m, dict(inp, w=nz), M, K, N, nz_storage=(nz.shape[0], nz.shape[1], 16, c0e))
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} outputs differ from the ND entry point"


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N,tB", [(128, 512, 256, False), (300, 384, 200, True), (64, 100, 72, False)])
def test_gpu_quant_matmul_weight_nz_int8_equals_nd(gpu, M, K, N, tB):
    m = gpu
    print(f"case qmm nz int8 M={M} K={K} N={N} tB={tB}", flush=True)
    inp = cases.make_qmm_int8_inputs(m, M, K, N, M + K, m.ACL_BF16, tB)
    want = cases.run_qmm_int8_aclnn(m, inp, M, K, N, tB, m.ACL_BF16)
    ref, _ = cases.oracle_qmm_int8(m, inp, M, K, N, tB, m.ACL_BF16)
    assert np.array_equal(want, ref)
    nz = nd_to_nz(inp["x2"][0].view(np.uint8), 32)
    got = cases.run_qmm_int8_aclnn(m, dict(inp, x2=nz[None]), M, K, N, tB, m.ACL_BF16, nz_storage=(nz.shape[0], nz.shape[1], 16, 32))
    assert np.array_equal(got, want)


@pytest.mark.gpu
def test_gpu_quant_matmul_weight_nz_mxfp4_equals_nd(gpu):
    """fp4 x2 in fractals of 32 elements (16 bytes) per row (ACL_FORMAT_FRACTAL_NZ_C0_32 in the reference's example,
    aclnnQuantMatmulWeightNz.md:850): the MX result must be bit for bit the ND one."""
    m = gpu
    M, K, N = 128, 512, 256
    inp = cases.make_mx_inputs(m, M, K, N, 5, True, True)
    want = cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    nz = nd_to_nz(inp["x2"][0].view(np.uint8).reshape(N, K // 2), 16)
    got = cases.run_mx_aclnn(m, dict(inp, x2=nz[None]), M, K, N, True, m.ACL_BF16, nz_storage=(nz.shape[0], nz.shape[1], 16, 32))
    assert np.array_equal(got, want)
