"""Seeded input generators and case runners shared by the GPU parity tests, smoke() and bench.py.
Every runner feeds identical bytes to the HIP path (through the C ABI) and to the CPU oracle."""
import ctypes as C

import numpy as np

import oracle_api as orc


def gen_int8(rng, shape):
    return rng.integers(-127, 128, size=shape, dtype=np.int8)


def gen_scale(rng, n, lo=1e-3, hi=1e-2):
    return rng.uniform(lo, hi, size=n).astype(np.float32)


def gen_bias(rng, n, dt, m):
    """Bias ~N(0, 0.1) in the requested dtype; returns (host array as stored, None if dt is None)."""
    if dt is None:
        return None
    v = rng.normal(0.0, 0.1, size=n).astype(np.float32)
    if dt == m.ACL_FLOAT:
        return v
    if dt == m.ACL_BF16:
        return orc.f32_to_bf16(v)
    if dt == m.ACL_FLOAT16:
        return orc.f32_to_f16(v)
    if dt == m.ACL_INT32:
        return rng.integers(-1000, 1000, size=n, dtype=np.int32)
    raise ValueError(dt)


def as_f32(arr, dt, m):
    if dt == m.ACL_BF16:
        return orc.bf16_to_f32(arr)
    if dt == m.ACL_FLOAT16:
        return orc.f16_to_f32(arr)
    return np.asarray(arr, np.float32)


def make_qmm_int8_inputs(m, M, K, N, seed, bias_dtype, transpose_x2, x2s_dtype=None, x2s_len=None, batch=1, x1s=True):
    rng = np.random.default_rng(seed)
    x1 = gen_int8(rng, (batch, M, K))
    x2 = gen_int8(rng, (batch, N, K) if transpose_x2 else (batch, K, N))
    s1 = gen_scale(rng, M) if x1s else None
    s2f = gen_scale(rng, N if x2s_len is None else x2s_len)
    x2s_dtype = m.ACL_FLOAT if x2s_dtype is None else x2s_dtype
    s2 = orc.f32_to_bf16(s2f) if x2s_dtype == m.ACL_BF16 else s2f
    bias = gen_bias(rng, N, bias_dtype, m)
    return dict(x1=x1, x2=x2, s1=s1, s2=s2, s2_dtype=x2s_dtype, bias=bias, bias_dtype=bias_dtype)


def oracle_qmm_int8(m, inp, M, K, N, transpose_x2, out_dtype, rows=None):
    """Oracle output [batch, M', N] (M' = len(rows) if a row subset is given) and int32 accumulators."""
    batch = inp["x1"].shape[0]
    s2f = as_f32(inp["s2"], inp["s2_dtype"], m)
    outs, accs = [], []
    for b in range(batch):
        x1 = inp["x1"][b]
        s1 = inp["s1"]
        if rows is not None:
            x1 = np.ascontiguousarray(x1[rows])
            s1 = np.ascontiguousarray(s1[rows]) if s1 is not None else None
        y, acc = orc.qmm_pertoken(x1, inp["x2"][b], x1.shape[0], K, N, False, transpose_x2, s1, s2f, inp["bias"],
                                  inp["bias_dtype"] if inp["bias_dtype"] is not None else 0, out_dtype, want_acc=True)
        outs.append(y)
        accs.append(acc)
    return np.stack(outs), np.stack(accs)


def run_qmm_int8_aclnn(m, inp, M, K, N, transpose_x2, out_dtype, x2_as_view=False):
    """aclnnQuantMatmulV5 on the device.  x2_as_view: pass x2 [N,K] storage as a transposed view of logical [K,N]
    with transposeX2 = false (the reference treats both spellings alike)."""
    batch = inp["x1"].shape[0]
    bshape = (batch,) if batch > 1 else ()
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    out_np = orc.out_array((batch, M, N), out_dtype)
    d_out = m.DeviceBuffer(out_np.nbytes)
    d_out.fill(0xFF)
    x1 = m.Tensor(bshape + (M, K), m.ACL_INT8, d["x1"])
    if transpose_x2 and x2_as_view:
        assert batch == 1
        x2 = m.Tensor((K, N), m.ACL_INT8, d["x2"], strides=(1, K))
        tflag = False
    else:
        x2 = m.Tensor(bshape + ((N, K) if transpose_x2 else (K, N)), m.ACL_INT8, d["x2"])
        tflag = transpose_x2
    s1 = m.Tensor((M,), m.ACL_FLOAT, d["s1"]) if inp["s1"] is not None else None
    s2 = m.Tensor((inp["s2"].size,), inp["s2_dtype"], d["s2"])
    bias = m.Tensor((N,), inp["bias_dtype"], d["bias"]) if inp["bias"] is not None else None
    out = m.Tensor(bshape + (M, N), out_dtype, d_out)
    ws = m.quant_matmul_v5(x1, x2, s1, s2, out, bias=bias, transpose_x2=tflag)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    del ws
    return d_out.to_host(out_np.dtype, out_np.shape)


def run_qmm_int8_case(m, orc_mod, M, K, N, seed, out_dtype, bias_dtype, transpose_x2, **kw):
    inp = make_qmm_int8_inputs(m, M, K, N, seed, bias_dtype, transpose_x2, **kw)
    got = run_qmm_int8_aclnn(m, inp, M, K, N, transpose_x2, out_dtype)
    want, acc = oracle_qmm_int8(m, inp, M, K, N, transpose_x2, out_dtype)
    return got, want, acc


def qmm_args_int8(m, d, M, K, N, batch, transpose_x2, out_ptr, out_dtype, s2_dtype, s2_len, bias_dtype, variant=0, ws=None):
    a = m.OpsnnQmmArgs()
    a.M, a.N, a.K, a.batch = M, N, K, batch
    a.x1 = m.OpsnnMat(d["x1"].ptr, K, 1, M * K if batch > 1 else 0)
    if transpose_x2:
        a.x2 = m.OpsnnMat(d["x2"].ptr, 1, K, N * K if batch > 1 else 0)
    else:
        a.x2 = m.OpsnnMat(d["x2"].ptr, N, 1, N * K if batch > 1 else 0)
    a.x1_dtype = a.x2_dtype = m.ACL_INT8
    a.out, a.out_dtype = out_ptr, out_dtype
    a.x1_scale = d["s1"].ptr if "s1" in d else None
    a.x2_scale, a.x2_scale_dtype, a.x2_scale_len = d["s2"].ptr, s2_dtype, s2_len
    if "bias" in d:
        a.bias, a.bias_dtype = d["bias"].ptr, bias_dtype
    a.force_variant = variant
    a.workspace = ws.ptr if ws is not None else None
    return a
