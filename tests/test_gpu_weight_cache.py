"""The opt-in cache of re-laid-out right operands (opsnnSetWeightCache): an N-contiguous weight / x2 is re-laid out once, later
calls with the same operand find the K-contiguous copy; results are those of the uncached path."""
import ctypes as C

import numpy as np
import pytest

import cases
import oracle_api as orc

pytestmark = pytest.mark.gpu


def _stats(m):
    v = [C.c_int64(0) for _ in range(4)]
    m.lib().opsnnWeightCacheStats(*[C.byref(x) for x in v])
    return tuple(x.value for x in v)   # entries, bytes, hits, misses


@pytest.fixture
def cache(gpu):
    m = gpu
    m.lib().opsnnSetWeightCache(256 << 20)
    try:
        yield m
    finally:
        m.lib().opsnnSetWeightCache(0)


def _wq_call(m, inp, d, d_y, M, K, N):
    group = inp["group"]
    G = K // group
    x = m.Tensor((M, K), inp["x_dt"], d["x"])
    w = m.Tensor((K, N), inp["w_dt"], d["w"])                       # [K, N] storage, N contiguous
    sc = m.Tensor((G, N), inp["x_dt"], d["scale"])
    off = m.Tensor((G, N), inp["x_dt"], d["offset"])
    y = m.Tensor((M, N), inp["x_dt"], d_y)
    ws = m.weight_quant_batch_matmul(x, w, sc, y, offset=off, group_size=group)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    del ws
    return d_y.to_host(np.uint16, (M, N))


def test_weight_only_weight_is_re_laid_out_once(cache):
    m = cache
    M, K, N = 16, 1024, 512
    print(f"case weight cache, weight-only int4 {M}x{K}x{N}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, 3, m.ACL_FLOAT16, m.ACL_INT4, 128, False, True, None)
    want = cases.oracle_wq(m, inp, M, K, N)
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    d_y = m.DeviceBuffer(M * N * 2)
    e0, _, h0, m0 = _stats(m)
    first = _wq_call(m, inp, d, d_y, M, K, N)
    second = _wq_call(m, inp, d, d_y, M, K, N)
    third = _wq_call(m, inp, d, d_y, M, K, N)
    e1, b1, h1, m1 = _stats(m)
    assert (e1 - e0, m1 - m0, h1 - h0) == (1, 1, 2) and b1 >= K * N // 2
    assert np.array_equal(first, second) and np.array_equal(first, third)
    g, w = orc.b16_to_f32(first, orc.F16), orc.b16_to_f32(want, orc.F16)
    mx, mean = orc.rel_err_stats(g, w)
    assert mx <= 2.0 ** -7 and mean <= 2.0 ** -10
    # a new weight in the same memory: the caller clears the cache, and the next call re-lays the new bytes out
    inp2 = cases.make_wq_inputs(m, M, K, N, 4, m.ACL_FLOAT16, m.ACL_INT4, 128, False, True, None)
    m.lib().opsnnWeightCacheClear()
    assert _stats(m)[0] == 0
    d["w"].upload(inp2["w"])
    inp2 = dict(inp2, x=inp["x"], scale=inp["scale"], offset=inp["offset"])
    got2 = _wq_call(m, inp2, d, d_y, M, K, N)
    want2 = cases.oracle_wq(m, inp2, M, K, N)
    mx, mean = orc.rel_err_stats(orc.b16_to_f32(got2, orc.F16), orc.b16_to_f32(want2, orc.F16))
    assert mx <= 2.0 ** -7 and mean <= 2.0 ** -10
    assert not np.array_equal(got2, first)


def test_weight_overwritten_in_place_is_stale_until_invalidated(cache):
    """The documented limit of the cache and its per-weight remedy: a weight overwritten in place keeps giving the old
    weight's results (the cache keys on the address), opsnnWeightCacheInvalidate(ptr, bytes) drops exactly that operand's
    entry -- another cached weight stays -- and the next call re-lays the new bytes out."""
    m = cache
    M, K, N = 16, 1024, 512
    print(f"case weight cache, in-place overwrite {M}x{K}x{N}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, 5, m.ACL_FLOAT16, m.ACL_INT4, 128, False, True, None)
    other = cases.make_wq_inputs(m, M, K, N, 6, m.ACL_FLOAT16, m.ACL_INT4, 128, False, True, None)
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    d_other = {k: m.DeviceBuffer(host=v) for k, v in other.items() if isinstance(v, np.ndarray)}
    d_y = m.DeviceBuffer(M * N * 2)
    e0 = _stats(m)[0]
    first = _wq_call(m, inp, d, d_y, M, K, N)
    _wq_call(m, other, d_other, d_y, M, K, N)
    assert _stats(m)[0] - e0 == 2
    inp2 = cases.make_wq_inputs(m, M, K, N, 7, m.ACL_FLOAT16, m.ACL_INT4, 128, False, True, None)
    inp2 = dict(inp2, x=inp["x"], scale=inp["scale"], offset=inp["offset"])
    d["w"].upload(inp2["w"])
    stale = _wq_call(m, inp2, d, d_y, M, K, N)
    assert np.array_equal(stale, first), "the cache is expected to serve the old copy until it is told"
    assert m.lib().opsnnWeightCacheInvalidate(d["w"].ptr, K * N // 2) == 1
    assert _stats(m)[0] - e0 == 1   # the other weight's entry is still there
    fresh = _wq_call(m, inp2, d, d_y, M, K, N)
    want2 = cases.oracle_wq(m, inp2, M, K, N)
    mx, mean = orc.rel_err_stats(orc.b16_to_f32(fresh, orc.F16), orc.b16_to_f32(want2, orc.F16))
    assert mx <= 2.0 ** -7 and mean <= 2.0 ** -10 and not np.array_equal(fresh, first)
    assert m.lib().opsnnWeightCacheInvalidate(d["w"].ptr, 0) == 1 and m.lib().opsnnWeightCacheInvalidate(d["w"].ptr, 0) == 0


def test_int8_x2_is_re_laid_out_once_and_the_limit_evicts(cache):
    m = cache
    M, K, N = 128, 512, 384
    print(f"case weight cache, int8 {M}x{K}x{N}", flush=True)
    inp = cases.make_qmm_int8_inputs(m, M, K, N, 5, m.ACL_BF16, False)
    want, _ = cases.oracle_qmm_int8(m, inp, M, K, N, False, m.ACL_BF16)
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    d_out = m.DeviceBuffer(M * N * 2)
    a = cases.qmm_args_int8(m, d, M, K, N, 1, False, d_out.ptr, m.ACL_BF16, inp["s2_dtype"], N, inp["bias_dtype"])
    e0, _, h0, m0 = _stats(m)
    outs = []
    for _ in range(3):                      # no workspace at all: only the cache can serve the matrix-core kernel
        d_out.fill(0xFF)
        assert m.lib().opsnnQmmInt8(a, None) == 0
        m.check(m.lib().aclrtSynchronizeDevice(), "sync")
        outs.append(d_out.to_host(np.uint16, (1, M, N)))
    e1, _, h1, m1 = _stats(m)
    assert (e1 - e0, m1 - m0, h1 - h0) == (1, 1, 2)
    assert all(np.array_equal(o, want) for o in outs)
    # a limit below the entry's size evicts it; with the cache off the same call (still no workspace) takes the plain kernel
    m.lib().opsnnSetWeightCache(1024)
    assert _stats(m)[0] == 0
    d_out.fill(0xFF)
    assert m.lib().opsnnQmmInt8(a, None) == 0
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    assert np.array_equal(d_out.to_host(np.uint16, (1, M, N)), want) and _stats(m)[0] == 0


def test_mx_operand_and_its_scales_are_re_laid_out_once(cache):
    """MXFP4 with x2 stored [K, N]: data and the [K/64, N, 2] scales go into one cached buffer; the product stays the oracle's."""
    m = cache
    M, K, N = 128, 512, 256
    print(f"case weight cache, mxfp4 {M}x{K}x{N}", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, 7, False, True)
    want = cases.oracle_mx(m, inp, M, K, N, False, m.ACL_BF16)
    e0, _, h0, m0 = _stats(m)
    first = cases.run_mx_aclnn(m, inp, M, K, N, False, m.ACL_BF16)       # fresh device buffers: a miss
    assert np.array_equal(first, want)
    e1, _, h1, m1 = _stats(m)
    assert (m1 - m0, h1 - h0) == (1, 0) and e1 - e0 == 1


def test_int4_group_mode_x2_blocks_are_written_once(cache):
    """int4 x int4 with group scales and offsets: the x2 half of the pre-step (e4m3 blocks with their scales and offsets)
    is kept; x1 is rewritten by every call, so a second call with other activations is still right."""
    m = cache
    M, K, N = 130, 1024, 512
    print(f"case weight cache, int4 K-G {M}x{K}x{N}", flush=True)
    inp = cases.make_i4_asym_inputs(m, M, K, N, 5)
    want = cases.oracle_i4_asym(m, inp, M, K, N, m.ACL_BF16)
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items()}
    d_out = m.DeviceBuffer(M * N * 2)
    t = dict(x1=m.Tensor((M, K), m.ACL_INT4, d["x1"]), x2=m.Tensor((N, K), m.ACL_INT4, d["x2"]),
             s1=m.Tensor(inp["s1"].shape, m.ACL_FLOAT, d["s1"]), s2=m.Tensor(inp["s2"].shape, m.ACL_FLOAT, d["s2"]),
             off=m.Tensor(inp["off"].shape, m.ACL_FLOAT16, d["off"]), out=m.Tensor((M, N), m.ACL_BF16, d_out))

    def call():
        ws = m.quant_matmul_v5(t["x1"], t["x2"], t["s1"], t["s2"], t["out"], x2_offset=t["off"], transpose_x2=True, group_size=256)
        m.check(m.lib().aclrtSynchronizeDevice(), "sync")
        del ws
        return d_out.to_host(np.uint16, (M, N))

    e0, _, h0, m0 = _stats(m)
    first = call()
    second = call()
    e1, _, h1, m1 = _stats(m)
    assert (e1 - e0, m1 - m0, h1 - h0) == (1, 1, 1)
    assert np.array_equal(first, want) and np.array_equal(second, want)
    # other activations against the kept x2 blocks
    inp2 = cases.make_i4_asym_inputs(m, M, K, N, 6)
    d["x1"].upload(inp2["x1"])
    inp2.update(x2=inp["x2"], s2=inp["s2"], off=inp["off"], s1=inp["s1"])
    third = call()
    assert np.array_equal(third, cases.oracle_i4_asym(m, inp2, M, K, N, m.ACL_BF16))
    assert _stats(m)[2] - h0 == 2


def test_fp8_fp4_group_mode_requantised_weight_is_written_once(cache):
    """fp8 x fp4 with 16-bit group scales: the re-quantised e4m3 weight with the decoded output scales is kept, keyed
    by x2, its scales and the output scale; a second call with other activations is still right (few rows: the
    streaming kernel reads the kept bytes)."""
    m = cache
    M, K, N = 40, 2048, 512
    print(f"case weight cache, fp8 x fp4 T-CG {M}x{K}x{N}", flush=True)
    inp = cases.make_tcg_inputs(m, M, K, N, 5, m.ACL_BF16)
    want = cases.oracle_tcg(m, inp, M, K, N, m.ACL_BF16)
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    d_out = m.DeviceBuffer(M * N * 2)
    t = dict(x1=m.Tensor((M, K), m.ACL_FLOAT8_E4M3FN, d["x1"]), x2=m.Tensor((N, K), m.ACL_FLOAT4_E2M1, d["x2"]),
             s2=m.Tensor((N, K // 32), m.ACL_BF16, d["s2"]), ys=m.Tensor((1, N), m.ACL_UINT64, d["ys"]),
             out=m.Tensor((M, N), m.ACL_BF16, d_out))

    def call():
        ws = m.quant_matmul_v5(t["x1"], t["x2"], None, t["s2"], t["out"], y_scale=t["ys"], transpose_x2=True, group_size=32)
        m.check(m.lib().aclrtSynchronizeDevice(), "sync")
        del ws
        return d_out.to_host(np.uint16, (M, N))

    def close(got, want):
        g, w = orc.b16_to_f32(got, orc.BF16), orc.b16_to_f32(want, orc.BF16)
        mx, mean = orc.rel_err_stats(g, w)
        return mx <= 2.0 ** -7 and mean <= 2.0 ** -10 and orc.isclose_fraction(g, w) <= 1e-3

    e0, _, h0, m0 = _stats(m)
    first = call()
    second = call()
    e1, _, h1, m1 = _stats(m)
    assert (e1 - e0, m1 - m0, h1 - h0) == (1, 1, 1)
    assert close(first, want) and np.array_equal(first, second)
    inp2 = cases.make_tcg_inputs(m, M, K, N, 6, m.ACL_BF16)
    d["x1"].upload(inp2["x1"])
    inp2.update(x2=inp["x2"], s2=inp["s2"], ys=inp["ys"])
    third = call()
    assert close(third, cases.oracle_tcg(m, inp2, M, K, N, m.ACL_BF16))
    assert _stats(m)[2] - h0 == 2


def test_nz_entry_points_do_not_key_the_cache_on_the_workspace(cache):
    """A FRACTAL_NZ weight is first written as the ND matrix into the front of the caller's workspace.  Two weights of one
    shape that share one workspace (as the layers of a model do) would meet under one cache key; the NZ entry points
    therefore leave the cache alone: both results equal the ND entry point's, and the cache holds nothing afterwards."""
    from test_nz_entry_points import nd_to_nz
    m = cache
    M, K, N = 16, 512, 256
    print(f"case weight cache with FRACTAL_NZ weights sharing a workspace, int8 {M}x{K}x{N}", flush=True)
    e0 = _stats(m)[0]
    inps = [cases.make_qmm_int8_inputs(m, M, K, N, seed, m.ACL_BF16, False) for seed in (21, 22)]
    wants = [cases.oracle_qmm_int8(m, inp, M, K, N, False, m.ACL_BF16)[0][0] for inp in inps]
    m.lib().opsnnSetWeightCache(0)
    nd = [cases.run_qmm_int8_aclnn(m, inp, M, K, N, False, m.ACL_BF16)[0] for inp in inps]
    m.lib().opsnnSetWeightCache(256 << 20)
    assert all(np.array_equal(a, b) for a, b in zip(nd, wants))
    shared_ws = None
    got = []
    for inp in inps:
        nz = nd_to_nz(inp["x2"][0].view(np.uint8), 32)
        d = {k: m.DeviceBuffer(host=v) for k, v in dict(inp, x2=nz[None]).items() if isinstance(v, np.ndarray)}
        d_out = m.DeviceBuffer(M * N * 2)
        d_out.fill(0xFF)
        x1 = m.Tensor((M, K), m.ACL_INT8, d["x1"])
        x2 = m.Tensor((K, N), m.ACL_INT8, d["x2"], fmt=29, storage_shape=(nz.shape[0], nz.shape[1], 16, 32))
        s1, s2 = m.Tensor((M,), m.ACL_FLOAT, d["s1"]), m.Tensor((N,), m.ACL_FLOAT, d["s2"])
        bias = m.Tensor((N,), m.ACL_BF16, d["bias"])
        out = m.Tensor((M, N), m.ACL_BF16, d_out)
        rc, ws, ex = m.quant_matmul_v5_get_workspace(x1, x2, s1, s2, out, bias=bias, weight_nz=True)
        assert rc == 0 and ws > 0, m.err_msg()
        if shared_ws is None:
            shared_ws = m.DeviceBuffer(ws)
        m.check(m.lib().aclnnQuantMatmulWeightNz(shared_ws.ptr, ws, ex, None), "aclnnQuantMatmulWeightNz")
        m.check(m.lib().aclrtSynchronizeDevice(), "sync")
        got.append(d_out.to_host(np.uint16, (M, N)))
    assert np.array_equal(got[0], wants[0]), "first NZ weight"
    assert np.array_equal(got[1], wants[1]), "second NZ weight through the same workspace: a stale cached copy was used"
    assert _stats(m)[0] == e0, "the NZ entry point put its workspace address into the cache"


def test_static_entry_point_leaves_the_cache_alone(cache):
    """opsnnQmmInt8Static promises no allocation: with the cache on it must not look the operand up (a miss allocates)."""
    m = cache
    M, K, N = 128, 256, 192
    inp = cases.make_qmm_int8_inputs(m, M, K, N, 5, m.ACL_BF16, False)
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    out = m.DeviceBuffer(M * N * 2)
    before = _stats(m)
    a = cases.qmm_args_int8(m, d, M, K, N, 1, False, out.ptr, m.ACL_BF16, m.ACL_FLOAT, N, m.ACL_BF16)
    assert m.lib().opsnnQmmInt8Static(C.byref(a), None) == 0, m.err_msg()
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    assert _stats(m) == before, (before, _stats(m))
    want, _ = cases.oracle_qmm_int8(m, inp, M, K, N, False, m.ACL_BF16)
    assert np.array_equal(out.to_host(np.uint16, (M, N)), want[0])
