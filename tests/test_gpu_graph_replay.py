"""The second phase of a call recorded into a HIP graph and replayed: the calls whose route has more than one kernel (a
re-layout or widening pre-step, partial sums of a K split and the kernel that adds them) must give on every replay what the
eager call gives on the same inputs.  The graph is replayed several times with eager work and synchronisations in between,
and x is overwritten between replays so that a replay that did not run all of its kernels would show.

torch is used for the capture only (its stream handle goes to the library as the aclrtStream) and for the device memory that
the captured call reads and writes; the first phase and the workspace allocation stay outside the capture.  torch brings its
own copy of the HIP runtime, which has to be the first one loaded in a process, so the cases run in a child process that
imports torch before the library: the test starts this file as a script.
"""
import ctypes as C
import os
import subprocess
import sys

import numpy as np
import pytest

WQ_CASES = [(8, 8192, 1024, True),     # x in registers, K split across workgroup columns, partial sums added
            (64, 8192, 1024, True),    # the many-rows kernel with K in segments
            (4, 2048, 4096, False),    # N-contiguous weight: re-laid out into the workspace first
            (200, 1024, 768, True)]    # row slabs in one launch
FP8_CASES = [(16, 18432, 512, True),   # few rows: K in segments, partial sums, a kernel that adds them
             (64, 18432, 1024, True),  # the many-rows kernel with K in segments
             (300, 1024, 640, False)]  # tiles, N-contiguous x2 re-laid out into the workspace
MX_CASES = [(64, 8192, 1024, False),   # MXFP8, 17 .. 256 rows: x1 widened into the workspace, the many-rows kernel
            (16, 8192, 512, False),    # MXFP8, few rows, K in segments
            (16, 8192, 512, True),     # MXFP4, few rows
            (300, 1024, 640, True)]    # MXFP4 tiles
INT8_CASES = [(64, 8192, 512, True),   # few tiles against a long K: integer partial sums in the workspace
              (300, 1024, 640, False)] # N-contiguous x2 re-laid out into the workspace


@pytest.mark.gpu
def test_calls_recorded_into_a_graph_replay_like_eager_calls():
    r = subprocess.run([sys.executable, "-u", os.path.abspath(__file__)], capture_output=True, text=True, timeout=600)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert r.stdout.count("replays ok") == len(WQ_CASES) + len(FP8_CASES) + len(MX_CASES) + len(INT8_CASES)


def _dev(torch, arr):
    return torch.from_numpy(np.ascontiguousarray(arr).view(np.uint8).reshape(-1).copy()).cuda()


def _replay_check(torch, record, eager, x_dev, x_variants, out_dev, out_shape):
    """record(stream_handle): phase 2 on that stream; eager(): the same call on the default stream, returns the output bytes."""
    want = []
    for xv in x_variants:
        x_dev.copy_(xv)
        torch.cuda.synchronize()
        want.append(eager())
    x_dev.copy_(x_variants[0])
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        record(C.c_void_p(torch.cuda.current_stream().cuda_stream))
    for rep in range(4):
        i = rep % len(x_variants)
        x_dev.copy_(x_variants[i])
        out_dev.fill_(0xEE)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = out_dev.cpu().numpy().view(np.uint16).reshape(out_shape)
        assert np.array_equal(got, want[i]), f"replay {rep}: {int((got != want[i]).sum())} of {got.size} outputs differ from the eager call"
        junk = torch.rand(1 << 20, device="cuda").sum().item()   # eager work between the replays
        assert junk > 0


def _weight_only_case(m, torch, cases, orc, M, K, N, tW):
    print(f"case graph replay weight-only M={M} K={K} N={N} tW={tW}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, M + N, m.ACL_FLOAT16, m.ACL_INT4, 128, tW, True, None)
    rng = np.random.default_rng(M)
    xs = [_dev(torch, inp["x"]), _dev(torch, orc.f32_to_b16(rng.normal(0, 1, size=(M, K)).astype(np.float32), m.ACL_FLOAT16))]
    G = K // 128
    t = {k: _dev(torch, inp[k]) for k in ("w", "scale", "offset")}
    x_dev, y_dev = xs[0].clone(), torch.empty(M * N * 2, dtype=torch.uint8, device="cuda")

    def tensors():
        x = m.Tensor((M, K), m.ACL_FLOAT16, x_dev.data_ptr())
        w = m.Tensor((K, N), m.ACL_INT4, t["w"].data_ptr(), strides=(1, K) if tW else None)
        sst = (1, G) if tW else None
        sc = m.Tensor((G, N), m.ACL_FLOAT16, t["scale"].data_ptr(), strides=sst)
        off = m.Tensor((G, N), m.ACL_FLOAT16, t["offset"].data_ptr(), strides=sst)
        return x, w, sc, off, m.Tensor((M, N), m.ACL_FLOAT16, y_dev.data_ptr())

    def phase1():
        x, w, sc, off, y = tensors()
        rc, ws, ex = m.weight_quant_batch_matmul_get_workspace(x, w, sc, y, offset=off, group_size=128)
        m.check(rc, "phase 1")
        return ws, ex, (x, w, sc, off, y)

    ws_bytes, _, _ = phase1()
    ws_dev = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")

    def run(stream):
        ws, ex, keep = phase1()
        m.check(m.lib().aclnnWeightQuantBatchMatmulV2(C.c_void_p(ws_dev.data_ptr()) if ws else None, C.c_uint64(ws), C.c_void_p(ex), stream), "phase 2")
        return keep

    def eager():
        y_dev.fill_(0xEE)
        torch.cuda.synchronize()
        keep = run(None)
        torch.cuda.synchronize()
        del keep
        return y_dev.cpu().numpy().view(np.uint16).reshape(M, N).copy()

    first = eager()
    want = cases.oracle_wq(m, inp, M, K, N)
    g, w = orc.b16_to_f32(first, orc.F16), orc.b16_to_f32(want, orc.F16)
    mx, mean = orc.rel_err_stats(g, w)
    assert mx <= 2.0 ** -7 and mean <= 2.0 ** -10, f"eager call before the capture: max rel {mx:.3e} mean rel {mean:.3e}"
    kept = []
    _replay_check(torch, lambda s: kept.append(run(s)), eager, x_dev, xs, y_dev, (M, N))
    print("replays ok", flush=True)


def _fp8_block_scale_case(m, torch, cases, orc, M, K, N, tB):
    print(f"case graph replay fp8 block M={M} K={K} N={N} tB={tB}", flush=True)
    inp = cases.make_blockscale_inputs(m, M, K, N, M + N, tB, 1)
    other = cases.make_blockscale_inputs(m, M, K, N, M + N + 1, tB, 1)
    xs = [_dev(torch, inp["x1"]), _dev(torch, other["x1"])]
    t = {k: _dev(torch, inp[k]) for k in ("x2", "s1", "s2")}
    x_dev, y_dev = xs[0].clone(), torch.empty(M * N * 2, dtype=torch.uint8, device="cuda")

    def phase1():
        x1 = m.Tensor((M, K), m.ACL_FLOAT8_E4M3FN, x_dev.data_ptr())
        x2 = m.Tensor((N, K) if tB else (K, N), m.ACL_FLOAT8_E4M3FN, t["x2"].data_ptr())
        s1 = m.Tensor(inp["s1"].shape[1:], m.ACL_FLOAT, t["s1"].data_ptr())
        s2 = m.Tensor(inp["s2"].shape[1:], m.ACL_FLOAT, t["s2"].data_ptr())
        out = m.Tensor((M, N), m.ACL_BF16, y_dev.data_ptr())
        rc, ws, ex = m.quant_matmul_v5_get_workspace(x1, x2, s1, s2, out, transpose_x2=tB, group_size=(1 << 32) | (128 << 16) | 128)
        m.check(rc, "phase 1")
        return ws, ex, (x1, x2, s1, s2, out)

    ws_bytes, _, _ = phase1()
    ws_dev = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")

    def run(stream):
        ws, ex, keep = phase1()
        m.check(m.lib().aclnnQuantMatmulV5(C.c_void_p(ws_dev.data_ptr()) if ws else None, C.c_uint64(ws), C.c_void_p(ex), stream), "phase 2")
        return keep

    def eager():
        y_dev.fill_(0xEE)
        torch.cuda.synchronize()
        keep = run(None)
        torch.cuda.synchronize()
        del keep
        return y_dev.cpu().numpy().view(np.uint16).reshape(M, N).copy()

    first = eager()
    want = cases.oracle_blockscale(m, inp, M, K, N, tB, m.ACL_BF16)[0]
    g, w = orc.b16_to_f32(first, orc.BF16), orc.b16_to_f32(want, orc.BF16)
    mx, mean = orc.rel_err_stats(g, w)
    assert mx <= 2.0 ** -7 and mean <= 2.0 ** -10, f"eager call before the capture: max rel {mx:.3e} mean rel {mean:.3e}"
    kept = []
    _replay_check(torch, lambda s: kept.append(run(s)), eager, x_dev, xs, y_dev, (M, N))
    print("replays ok", flush=True)


def _v5_case(m, torch, orc, what, M, N, x_key, inp, other_x, make_tensors, kw, want, code):
    """A quant_matmul_v5 call whose left operand is inp[x_key]; make_tensors(ptr of each array) -> (x1, x2, s1, s2)."""
    xs = [_dev(torch, inp[x_key]), _dev(torch, other_x)]
    t = {k: _dev(torch, v) for k, v in inp.items() if isinstance(v, np.ndarray) and k != x_key}
    x_dev, y_dev = xs[0].clone(), torch.empty(M * N * 2, dtype=torch.uint8, device="cuda")

    def phase1():
        ptrs = {k: v.data_ptr() for k, v in t.items()}
        ptrs[x_key] = x_dev.data_ptr()
        x1, x2, s1, s2, extra = make_tensors(ptrs)
        out = m.Tensor((M, N), m.ACL_BF16, y_dev.data_ptr())
        rc, ws, ex = m.quant_matmul_v5_get_workspace(x1, x2, s1, s2, out, **kw, **extra)
        m.check(rc, "phase 1")
        return ws, ex, (x1, x2, s1, s2, out, extra)

    ws_bytes, _, _ = phase1()
    ws_dev = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")

    def run(stream):
        ws, ex, keep = phase1()
        m.check(m.lib().aclnnQuantMatmulV5(C.c_void_p(ws_dev.data_ptr()) if ws else None, C.c_uint64(ws), C.c_void_p(ex), stream), "phase 2")
        return keep

    def eager():
        y_dev.fill_(0xEE)
        torch.cuda.synchronize()
        keep = run(None)
        torch.cuda.synchronize()
        del keep
        return y_dev.cpu().numpy().view(np.uint16).reshape(M, N).copy()

    first = eager()
    if code is None:
        assert np.array_equal(first, want), f"{what}: eager call before the capture differs from the oracle"
    else:
        mx, mean = orc.rel_err_stats(orc.b16_to_f32(first, code), orc.b16_to_f32(want, code))
        assert mx <= 2.0 ** -7 and mean <= 2.0 ** -10, f"{what}: eager call before the capture: max rel {mx:.3e} mean rel {mean:.3e}"
    kept = []
    _replay_check(torch, lambda s: kept.append(run(s)), eager, x_dev, xs, y_dev, (M, N))
    print("replays ok", flush=True)


def _mx_case(m, torch, cases, orc, M, K, N, fp4):
    print(f"case graph replay mx M={M} K={K} N={N} fp4={fp4}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, M + N, True, fp4)
    other = cases.make_mx_inputs(m, M, K, N, M + N + 1, True, fp4)["x1"]
    adt = m.ACL_FLOAT4_E2M1 if fp4 else m.ACL_FLOAT8_E4M3FN
    inp = {k: (v[0] if isinstance(v, np.ndarray) else v) for k, v in inp.items()}

    def tensors(p):
        return (m.Tensor((M, K), adt, p["x1"]), m.Tensor((N, K), adt, p["x2"]), m.Tensor(inp["s1"].shape, m.ACL_FLOAT8_E8M0, p["s1"]),
                m.Tensor(inp["s2"].shape, m.ACL_FLOAT8_E8M0, p["s2"]), {})
    want = cases.oracle_mx(m, {k: (v[None] if isinstance(v, np.ndarray) else v) for k, v in inp.items()}, M, K, N, True, m.ACL_BF16)[0]
    _v5_case(m, torch, orc, "mx", M, N, "x1", inp, other[0], tensors, dict(transpose_x2=True, group_size=(1 << 32) | (1 << 16) | 32), want, orc.BF16)


def _int8_case(m, torch, cases, orc, M, K, N, tB):
    print(f"case graph replay int8 M={M} K={K} N={N} tB={tB}", flush=True)
    inp = cases.make_qmm_int8_inputs(m, M, K, N, M + N, m.ACL_BF16, tB)
    other = cases.make_qmm_int8_inputs(m, M, K, N, M + N + 1, m.ACL_BF16, tB)["x1"][0]
    want = cases.oracle_qmm_int8(m, inp, M, K, N, tB, m.ACL_BF16)[0][0]
    flat = dict(x1=inp["x1"][0], x2=inp["x2"][0], s1=inp["s1"], s2=inp["s2"], bias=inp["bias"])

    def tensors(p):
        return (m.Tensor((M, K), m.ACL_INT8, p["x1"]), m.Tensor((N, K) if tB else (K, N), m.ACL_INT8, p["x2"]), m.Tensor((M,), m.ACL_FLOAT, p["s1"]),
                m.Tensor((N,), m.ACL_FLOAT, p["s2"]), dict(bias=m.Tensor((N,), m.ACL_BF16, p["bias"])))
    _v5_case(m, torch, orc, "int8", M, N, "x1", flat, other, tensors, dict(transpose_x2=tB), want, None)


if __name__ == "__main__":
    import torch   # first: its HIP runtime must be the one the library binds to
    assert torch.cuda.is_available()
    torch.zeros(1, device="cuda")
    here = os.path.dirname(os.path.abspath(__file__))
    sys.path.insert(0, os.path.join(os.path.dirname(here), "ops-nn_amd"))
    sys.path.insert(0, here)
    import opsnn
    import cases as _cases
    import oracle_api as _orc
    opsnn.check(opsnn.lib().aclInit(None), "aclInit")
    opsnn.check(opsnn.lib().aclrtSetDevice(0), "aclrtSetDevice")
    for c in WQ_CASES:
        _weight_only_case(opsnn, torch, _cases, _orc, *c)
    for c in FP8_CASES:
        _fp8_block_scale_case(opsnn, torch, _cases, _orc, *c)
    for c in MX_CASES:
        _mx_case(opsnn, torch, _cases, _orc, *c)
    for c in INT8_CASES:
        _int8_case(opsnn, torch, _cases, _orc, *c)
