"""Calls in flight on two streams at once: every call has its own workspace and output, so calls on different streams share
nothing but the library's read-only state, and each must give the bits it gives alone.  Three multi-kernel routes (a K split
with partial sums, a widening pre-step, a re-layout) are enqueued alternately on two streams, ten rounds, without a
synchronisation in between."""
import numpy as np
import pytest

import cases

pytestmark = pytest.mark.gpu


def _weight_only(m, M, K, N, tW):
    inp = cases.make_wq_inputs(m, M, K, N, M + N, m.ACL_FLOAT16, m.ACL_INT4, 128, tW, True, None)
    want = cases.run_wq_aclnn(m, inp, M, K, N)
    d = {k: m.DeviceBuffer(host=inp[k]) for k in ("x", "w", "scale", "offset")}
    G = K // 128

    def enqueue(stream, out):
        sst = (1, G) if tW else None
        t = (m.Tensor((M, K), m.ACL_FLOAT16, d["x"]), m.Tensor((K, N), m.ACL_INT4, d["w"], strides=(1, K) if tW else None),
             m.Tensor((G, N), m.ACL_FLOAT16, d["scale"], strides=sst), m.Tensor((G, N), m.ACL_FLOAT16, d["offset"], strides=sst),
             m.Tensor((M, N), m.ACL_FLOAT16, out))
        ws = m.weight_quant_batch_matmul(t[0], t[1], t[2], t[4], offset=t[3], group_size=128, stream=stream)
        return out, (ws, t)
    return enqueue, want, (M, N), d


def _v5(m, kind, M, K, N):
    if kind == "block":
        inp = cases.make_blockscale_inputs(m, M, K, N, M + N, True, 1)
        want = cases.run_blockscale_aclnn(m, inp, M, K, N, True, m.ACL_BF16)[0]
        adt, sdt, gs = m.ACL_FLOAT8_E4M3FN, m.ACL_FLOAT, (1 << 32) | (128 << 16) | 128
    else:
        inp = cases.make_mx_inputs(m, M, K, N, M + N, True, False)
        want = cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16)[0]
        adt, sdt, gs = m.ACL_FLOAT8_E4M3FN, m.ACL_FLOAT8_E8M0, (1 << 32) | (1 << 16) | 32
    d = {k: m.DeviceBuffer(host=inp[k]) for k in ("x1", "x2", "s1", "s2")}

    def enqueue(stream, out):
        t = (m.Tensor((M, K), adt, d["x1"]), m.Tensor((N, K), adt, d["x2"]), m.Tensor(inp["s1"].shape[1:], sdt, d["s1"]),
             m.Tensor(inp["s2"].shape[1:], sdt, d["s2"]), m.Tensor((M, N), m.ACL_BF16, out))
        ws = m.quant_matmul_v5(t[0], t[1], t[2], t[3], t[4], transpose_x2=True, group_size=gs, stream=stream)
        return out, (ws, t)
    return enqueue, want, (M, N), d


def test_calls_on_two_streams_do_not_disturb_each_other(gpu):
    m = gpu
    print("case two streams: weight-only K split / re-layout, fp8 block K split, MXFP8 widening pre-step", flush=True)
    calls = [_weight_only(m, 8, 8192, 1024, True), _v5(m, "block", 16, 18432, 512), _weight_only(m, 4, 2048, 4096, False),
             _v5(m, "mxfp8", 64, 8192, 1024), _weight_only(m, 64, 8192, 1024, True), _v5(m, "block", 64, 18432, 1024)]
    s = [m.Stream(), m.Stream()]
    import opsnn.binding as binding
    fill, binding.FILL_NEW_WORKSPACE = binding.FILL_NEW_WORKSPACE, None   # (a memset on the default stream would wait for both streams)
    try:
        outs, keep = [], []
        for rnd in range(10):
            for i, c in enumerate(calls):
                out = m.DeviceBuffer(c[2][0] * c[2][1] * 2)
                out.fill(0xEE)
                outs.append((i, rnd, out))
        m.check(m.lib().aclrtSynchronizeDevice(), "sync")
        for i, rnd, out in outs:
            keep.append(calls[i][0](s[(i + rnd) % 2], out))
        s[0].sync()
        s[1].sync()
        for i, rnd, out in outs:
            got = out.to_host(np.uint16, calls[i][2])
            want = calls[i][1]
            assert np.array_equal(got, want), f"call {i}, round {rnd}: {int((got != want).sum())} of {got.size} outputs differ from the call alone"
    finally:
        binding.FILL_NEW_WORKSPACE = fill
        m.check(m.lib().aclrtSynchronizeDevice(), "sync")
        for st in s:
            st.destroy()
