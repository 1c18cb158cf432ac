"""Batch dims of x1 and x2 that broadcast against each other in any numpy pattern (qbmmv3_kernel_golden.py:288-330), not
only "no batch" or "equal batch": phase 1 splits the out batch into one launch per combination of the outer batch dims."""
import numpy as np
import pytest

import cases
import oracle_api as orc
from test_gpu_other_modes import check_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("b1,b2,M,K,N", [
    ((2, 1), (1, 3), 128, 256, 192),      # both operands broadcast, on different dims
    ((2, 3), (3,), 64, 128, 64),          # x2 has fewer batch dims and is reused for every outer index
    ((1, 2), (4, 1), 96, 512, 136),
    ((2,), (2,), 64, 4096, 256),          # equal batches, few tiles against a long K: the K split inside a batched launch
    ((2, 1), (1, 2), 48, 8192, 136),      # and inside the launches of a broadcast pattern (they share the partial sums' buffer, in stream order)
])
def test_int8_partial_batch_broadcast(gpu, b1, b2, M, K, N):
    m = gpu
    print(f"case int8 batch broadcast x1 {b1} x2 {b2} M={M} K={K} N={N}", flush=True)
    n1, n2 = int(np.prod(b1)), int(np.prod(b2))
    rng = np.random.default_rng(M + N)
    x1 = cases.gen_int8(rng, (n1, M, K))
    x2 = cases.gen_int8(rng, (n2, N, K))
    s1 = cases.gen_scale(rng, M)
    s2 = cases.gen_scale(rng, N)
    bias = cases.gen_bias(rng, N, m.ACL_BF16, m)
    ob = np.broadcast_shapes(b1, b2)
    i1 = np.broadcast_to(np.arange(n1).reshape(b1), ob).reshape(-1)
    i2 = np.broadcast_to(np.arange(n2).reshape(b2), ob).reshape(-1)
    want = np.stack([orc.qmm_pertoken(x1[a], x2[b], M, K, N, False, True, s1, s2, bias, m.ACL_BF16, m.ACL_BF16) for a, b in zip(i1, i2)])
    d = {k: m.DeviceBuffer(host=v) for k, v in dict(x1=x1, x2=x2, s1=s1, s2=s2, bias=bias).items()}
    d_out = m.DeviceBuffer(want.size * 2)
    d_out.fill(0xFF)
    t1 = m.Tensor(tuple(b1) + (M, K), m.ACL_INT8, d["x1"])
    t2 = m.Tensor(tuple(b2) + (N, K), m.ACL_INT8, d["x2"])
    out = m.Tensor(tuple(ob) + (M, N), m.ACL_BF16, d_out)
    ws = m.quant_matmul_v5(t1, t2, m.Tensor((M,), m.ACL_FLOAT, d["s1"]), m.Tensor((N,), m.ACL_FLOAT, d["s2"]), out,
                           bias=m.Tensor((N,), m.ACL_BF16, d["bias"]), transpose_x2=True)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    got = d_out.to_host(np.uint16, want.shape)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("M,K,N", [(128, 256, 256), (256, 2048, 256)])   # (the second: the exact kernel's K split in every launch)
def test_fp8_blockscale_partial_batch_broadcast(gpu, M, K, N):
    """The scale tables carry their operand's batch dims: they are offset with it."""
    m = gpu
    b1, b2 = (2, 1), (3,)
    n1, n2 = 2, 3
    inp1 = cases.make_blockscale_inputs(m, M, K, N, 3, True, 1, batch=n1)
    inp2 = cases.make_blockscale_inputs(m, M, K, N, 4, True, 1, batch=n2)
    ob = (2, 3)
    want = []
    for a in range(2):
        for b in range(3):
            one = dict(x1=inp1["x1"][a:a + 1], s1=inp1["s1"][a:a + 1], x2=inp2["x2"][b:b + 1], s2=inp2["s2"][b:b + 1], gsM=1)
            want.append(cases.oracle_blockscale(m, one, M, K, N, True, m.ACL_BF16)[0])
    want = np.stack(want)
    d = {k: m.DeviceBuffer(host=v) for k, v in dict(x1=inp1["x1"], s1=inp1["s1"], x2=inp2["x2"], s2=inp2["s2"]).items()}
    d_out = m.DeviceBuffer(want.size * 2)
    d_out.fill(0xFF)
    t1 = m.Tensor(b1 + (M, K), m.ACL_FLOAT8_E4M3FN, d["x1"])
    t2 = m.Tensor(b2 + (N, K), m.ACL_FLOAT8_E4M3FN, d["x2"])
    s1 = m.Tensor(b1 + inp1["s1"].shape[1:], m.ACL_FLOAT, d["s1"])
    s2 = m.Tensor(b2 + inp2["s2"].shape[1:], m.ACL_FLOAT, d["s2"])
    out = m.Tensor(ob + (M, N), m.ACL_BF16, d_out)
    ws = m.quant_matmul_v5(t1, t2, s1, s2, out, transpose_x2=True, group_size=(1 << 32) | (128 << 16) | 128)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    got = d_out.to_host(np.uint16, want.shape)
    check_close(got, want, orc.BF16, "fp8 block scale, partial batch broadcast")
