"""The BASELINE configurations at their full sizes, through the aclnn C ABI.

The CPU oracle is asked for a seeded sample of output rows (first and last included) -- enough to finish in
seconds -- and every sampled row must meet the bar of its kernel class (see test_gpu_other_modes.py).  On top
of that, a size-independent property is checked on the whole output: scaling by a power of two is exact in
every format on the path, so doubling one operand's scales must double every output bit for bit.
"""
import numpy as np
import pytest

import cases
import oracle_api as orc
from test_gpu_other_modes import check_close

pytestmark = pytest.mark.gpu


def _rows(M, n, seed):
    return np.unique(np.concatenate([[0, M - 1], np.random.default_rng(seed).integers(0, M, n)]))


def _double_exactly(a_bits, b_bits, dt, tiny=0.0):
    a, b = orc.b16_to_f32(a_bits, dt), orc.b16_to_f32(b_bits, dt)
    assert np.isfinite(a).all() and np.isfinite(b).all()
    ok = (b == a * np.float32(2.0)) | (np.abs(a) < tiny)   # rounding in the subnormal range is not scale invariant
    assert ok.all(), f"{int((~ok).sum())} of {a.size} outputs did not double exactly"


def test_config1_w8a16_per_channel_full(gpu):
    m = gpu
    M, K, N = 16, 4096, 4096
    print("case config 1 full size", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, 0, m.ACL_BF16, m.ACL_INT8, 0, True, False, None, 1e-4, 0.06)
    got = cases.run_wq_aclnn(m, inp, M, K, N)
    check_close(got, cases.oracle_wq(m, inp, M, K, N), m.ACL_BF16, "config 1")
    # N-contiguous weight (the literal [K, N] storage of the config): re-laid out inside the call
    inp_nd = dict(inp, w=np.ascontiguousarray(inp["w"].T), tW=False)
    got_nd = cases.run_wq_aclnn(m, inp_nd, M, K, N)
    assert np.array_equal(got_nd, got), "both weight layouts must give the same bits"


@pytest.mark.parametrize("M", [1, 16, 64])
def test_config3_w4a16_per_group_full(gpu, M):
    m = gpu
    K, N = 8192, 28672
    print(f"case config 3 full size M={M}", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, 0, m.ACL_FLOAT16, m.ACL_INT4, 128, True, True, None)
    got = cases.run_wq_aclnn(m, inp, M, K, N)
    rows = _rows(M, 6, 3)
    want = cases.oracle_wq(m, inp, M, K, N, rows=rows)
    check_close(got[rows], want, m.ACL_FLOAT16, f"config 3 M={M}")
    # doubling x (exact in fp16, subnormals included) doubles every product, every partial sum and every output
    # exactly, except outputs so small that fp16 rounds them on the subnormal grid
    inp2 = dict(inp, x=orc.f32_to_b16(orc.b16_to_f32(inp["x"], m.ACL_FLOAT16) * np.float32(2.0), m.ACL_FLOAT16))
    _double_exactly(got, cases.run_wq_aclnn(m, inp2, M, K, N), m.ACL_FLOAT16, tiny=2.0 ** -13)


def test_config3_m256_sampled(gpu):
    m = gpu
    M, K, N = 256, 8192, 28672
    print("case config 3 full size M=256", flush=True)
    inp = cases.make_wq_inputs(m, M, K, N, 0, m.ACL_FLOAT16, m.ACL_INT4, 128, True, True, None)
    got = cases.run_wq_aclnn(m, inp, M, K, N)
    rows = _rows(M, 6, 4)
    check_close(got[rows], cases.oracle_wq(m, inp, M, K, N, rows=rows), m.ACL_FLOAT16, "config 3 M=256")


def test_config4_fp8_block_scale_full(gpu):
    m = gpu
    M, K, N = 4096, 7168, 18432
    print("case config 4 full size", flush=True)
    inp = cases.make_blockscale_inputs(m, M, K, N, 0, True, 1)
    got = cases.run_blockscale_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    rows = _rows(M, 10, 5)
    want = cases.oracle_blockscale(m, inp, M, K, N, True, m.ACL_BF16, rows=rows)
    check_close(got[0][rows], want[0], m.ACL_BF16, "config 4", fp8_mfma=True)
    inp2 = dict(inp, s1=inp["s1"] * np.float32(2.0))
    _double_exactly(got, cases.run_blockscale_aclnn(m, inp2, M, K, N, True, m.ACL_BF16), m.ACL_BF16)


def test_config5_mxfp4_batched_full(gpu):
    m = gpu
    B, M, K, N = 8, 4096, 8192, 8192
    print("case config 5 full size", flush=True)
    inp = cases.make_mx_inputs(m, M, K, N, 0, True, True, batch=B)
    got = cases.run_mx_aclnn(m, inp, M, K, N, True, m.ACL_BF16)
    rows = _rows(M, 4, 6)
    for b in (0, B - 1):
        one = {k: (v[b:b + 1] if isinstance(v, np.ndarray) else v) for k, v in inp.items()}
        want = cases.oracle_mx(m, one, M, K, N, True, m.ACL_BF16, rows=rows)
        # fp4 products and their partial sums are exact in the matrix unit: the bar is the ordinary one
        check_close(got[b][rows], want[0], m.ACL_BF16, f"config 5 batch {b}")
    # one more on every x1 exponent doubles every output exactly
    inp2 = dict(inp, s1=(inp["s1"] + 1).astype(np.uint8))
    _double_exactly(got, cases.run_mx_aclnn(m, inp2, M, K, N, True, m.ACL_BF16), m.ACL_BF16)
