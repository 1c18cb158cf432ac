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


GUARD = 4096


def guarded_out(m, nbytes, fill=0xFF):
    """An output allocation with GUARD bytes in front of and behind the nbytes the call may write, all filled with `fill`;
    to_host checks that both guards still hold the fill (a store outside the output would otherwise land in whatever the
    allocator has placed next to it, unseen)."""
    class _Guarded(m.DeviceBuffer):
        def __init__(self):
            self.whole = m.DeviceBuffer(nbytes + 2 * GUARD)
            self.whole.fill(fill)
            self.nbytes, self.ptr = int(nbytes), self.whole.ptr + GUARD

        def fill(self, byte):
            pass   # (already filled; the guards must keep their byte)

        def free(self):
            self.ptr = None

        def to_host(self, dtype, shape):
            raw = self.whole.to_host(np.uint8, (self.nbytes + 2 * GUARD,))
            front, back = raw[:GUARD], raw[GUARD + self.nbytes:]
            assert (front == fill).all(), f"{int((front != fill).sum())} bytes written in front of the output"
            assert (back == fill).all(), f"{int((back != fill).sum())} bytes written behind the output, first at +{int(np.argmax(back != fill))}"
            out = np.empty(shape, dtype=dtype)
            assert out.nbytes <= self.nbytes
            return raw[GUARD:GUARD + out.nbytes].view(out.dtype).reshape(shape).copy()
    return _Guarded()


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


def run_qmm_int8_aclnn(m, inp, M, K, N, transpose_x2, out_dtype, x2_as_view=False, nz_storage=None):
    """aclnnQuantMatmulV5 on the device.  x2_as_view: pass x2 [N,K] storage as a transposed view of logical [K,N]
    with transposeX2 = false (the reference treats both spellings alike)."""
    batch = inp["x1"].shape[0]
    bshape = (batch,) if batch > 1 else ()
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    out_np = orc.out_array((batch, M, N), out_dtype)
    d_out = guarded_out(m, out_np.nbytes)
    x1 = m.Tensor(bshape + (M, K), m.ACL_INT8, d["x1"])
    if transpose_x2 and x2_as_view:
        assert batch == 1
        x2 = m.Tensor((K, N), m.ACL_INT8, d["x2"], strides=(1, K))
        tflag = False
    else:
        # nz_storage: inp["x2"] holds the FRACTAL_NZ bytes of the stored matrix and the call goes to aclnnQuantMatmulWeightNz
        x2 = m.Tensor(bshape + ((N, K) if transpose_x2 else (K, N)), m.ACL_INT8, d["x2"], fmt=29 if nz_storage else m.ACL_FORMAT_ND,
                      storage_shape=nz_storage)
        tflag = transpose_x2
    s1 = m.Tensor((M,), m.ACL_FLOAT, d["s1"]) if inp["s1"] is not None else None
    s2 = m.Tensor((inp["s2"].size,), inp["s2_dtype"], d["s2"])
    bias = m.Tensor((N,), inp["bias_dtype"], d["bias"]) if inp["bias"] is not None else None
    out = m.Tensor(bshape + (M, N), out_dtype, d_out)
    ws = m.quant_matmul_v5(x1, x2, s1, s2, out, bias=bias, transpose_x2=tflag, weight_nz=bool(nz_storage))
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


# --------------------------------------------------------------------------------------------------
# fp8 block scale (G-B / B-B)
# --------------------------------------------------------------------------------------------------
def gen_fp8(rng, shape):
    v = np.clip(rng.normal(0.0, 1.0, size=shape), -448.0, 448.0).astype(np.float32)
    return orc.f32_to_e4m3(v)


def make_blockscale_inputs(m, M, K, N, seed, tB, gsM=1, batch=1):
    rng = np.random.default_rng(seed)
    KB, NB, MB = -(-K // 128), -(-N // 128), -(-M // gsM)
    x1 = gen_fp8(rng, (batch, M, K))
    x2 = gen_fp8(rng, (batch, N, K) if tB else (batch, K, N))
    s1 = gen_scale(rng, batch * MB * KB).reshape(batch, MB, KB)
    s2 = gen_scale(rng, batch * KB * NB).reshape((batch, NB, KB) if tB else (batch, KB, NB))
    return dict(x1=x1, x2=x2, s1=s1, s2=s2, gsM=gsM)


def oracle_blockscale(m, inp, M, K, N, tB, out_dtype, rows=None):
    outs = []
    gsM = inp["gsM"]
    for b in range(inp["x1"].shape[0]):
        x1, s1 = inp["x1"][b], inp["s1"][b]
        Mr = M
        if rows is not None:
            assert gsM == 1
            x1, s1, Mr = np.ascontiguousarray(x1[rows]), np.ascontiguousarray(s1[rows]), len(rows)
        outs.append(orc.qmm_perblock(x1, inp["x2"][b], orc.E4M3, orc.E4M3, Mr, K, N, False, tB, s1,
                                     np.ascontiguousarray(inp["s2"][b]), gsM, 128, 128, None, out_dtype))
    return np.stack(outs)


def run_blockscale_aclnn(m, inp, M, K, N, tB, out_dtype, group_size=None):
    batch = inp["x1"].shape[0]
    bshape = (batch,) if batch > 1 else ()
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    out_np = orc.out_array((batch, M, N), out_dtype)
    d_out = guarded_out(m, out_np.nbytes)
    x1 = m.Tensor(bshape + (M, K), m.ACL_FLOAT8_E4M3FN, d["x1"])
    x2 = m.Tensor(bshape + ((N, K) if tB else (K, N)), m.ACL_FLOAT8_E4M3FN, d["x2"])
    s1 = m.Tensor(bshape + inp["s1"].shape[1:], m.ACL_FLOAT, d["s1"])
    s2 = m.Tensor(bshape + inp["s2"].shape[1:], m.ACL_FLOAT, d["s2"])
    out = m.Tensor(bshape + (M, N), out_dtype, d_out)
    gs = (inp["gsM"] << 32) | (128 << 16) | 128 if group_size is None else group_size
    ws = m.quant_matmul_v5(x1, x2, s1, s2, out, transpose_x2=tB, group_size=gs)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    del ws
    return d_out.to_host(out_np.dtype, out_np.shape)


# --------------------------------------------------------------------------------------------------
# per-tensor / per-channel family (T-T, T-C; 64-bit packed scales, int8 requantisation, fp8 double scale)
# --------------------------------------------------------------------------------------------------
def make_tc_inputs(m, M, K, N, seed, in_dt, scale_dt, scale_len, bias_dt, tB, pertoken=False, offset_len=0, e5m2=False):
    """in_dt: ACL_INT8 or an fp8 type; scale_dt: ACL_FLOAT / ACL_BF16 / ACL_UINT64; offset_len: 0 (none), 1 or N."""
    rng = np.random.default_rng(seed)
    if in_dt == m.ACL_INT8:
        x1, x2 = gen_int8(rng, (M, K)), gen_int8(rng, (N, K) if tB else (K, N))
    else:
        x1, x2 = gen_fp8(rng, (M, K)), gen_fp8(rng, (N, K) if tB else (K, N))
        if e5m2:   # any byte pattern below infinity is a finite e5m2 value
            x1, x2 = (x1 & 0xBB).astype(np.uint8), (x2 & 0xBB).astype(np.uint8)
    sf = gen_scale(rng, N if scale_len != 1 else 1, 1e-3, 1e-2) if in_dt == m.ACL_INT8 else gen_scale(rng, N if scale_len != 1 else 1, 0.05, 0.5)
    if scale_dt == m.ACL_UINT64:
        scale = orc.pack_u64_scale(sf)
    elif scale_dt == m.ACL_BF16:
        scale = orc.f32_to_bf16(sf)
    else:
        scale = sf
    pt = gen_scale(rng, M if pertoken == "M" else 1, 0.5, 2.0) if pertoken else None   # "M": one scale per row (K-C / K-T)
    off = rng.uniform(-20, 20, size=offset_len).astype(np.float32) if offset_len else None
    bias = gen_bias(rng, N, bias_dt, m)
    if bias_dt == m.ACL_INT32 and bias is not None:
        bias = rng.integers(-3000, 3000, size=N).astype(np.int32)
    return dict(x1=x1, x2=x2, scale=scale, scale_dt=scale_dt, pt=pt, off=off, bias=bias, bias_dt=bias_dt, in_dt=in_dt, tB=tB,
                x2_dt=in_dt)


def oracle_tc(m, inp, M, K, N, out_dt):
    if inp["pt"] is not None and inp["pt"].size > 1:   # fp8 with a per-row scale: compute_pertoken
        return orc.qmm_pertoken_f8(inp["x1"], inp["x2"], inp["in_dt"], inp["x2_dt"], M, K, N, False, inp["tB"], inp["pt"],
                                   inp["scale"], inp["bias"], out_dt)
    return orc.qmm_tc(inp["x1"], inp["x2"], inp["in_dt"], inp["x2_dt"], M, K, N, False, inp["tB"], inp["scale"], inp["scale_dt"],
                      inp["pt"], inp["off"], inp["bias"], inp["bias_dt"] or 0, out_dt)


def run_tc_aclnn(m, inp, M, K, N, out_dt):
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    out_np = orc.out_array((M, N), out_dt)
    d_out = guarded_out(m, out_np.nbytes, 0x7F)
    tB = inp["tB"]
    x1 = m.Tensor((M, K), inp["in_dt"], d["x1"])
    x2 = m.Tensor((N, K) if tB else (K, N), inp["x2_dt"], d["x2"])
    s2 = m.Tensor((inp["scale"].size,), inp["scale_dt"], d["scale"])
    s1 = m.Tensor((inp["pt"].size,), m.ACL_FLOAT, d["pt"]) if inp["pt"] is not None else None
    off = m.Tensor((inp["off"].size,), m.ACL_FLOAT, d["off"]) if inp["off"] is not None else None
    bias = m.Tensor((N,), inp["bias_dt"], d["bias"]) if inp["bias"] is not None else None
    out = m.Tensor((M, N), out_dt, d_out)
    ws = m.quant_matmul_v5(x1, x2, s1, s2, out, bias=bias, x2_offset=off, transpose_x2=tB)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    del ws
    return d_out.to_host(out_np.dtype, out_np.shape)


# --------------------------------------------------------------------------------------------------
# MX (fp4 / fp8 with e8m0 scales per 32 K)
# --------------------------------------------------------------------------------------------------
def make_mx_inputs(m, M, K, N, seed, tB, fp4=True, batch=1, exp_range=4):
    rng = np.random.default_rng(seed)
    KS = -(-K // 64)
    if fp4:
        c1 = rng.integers(0, 16, size=(batch, M, K), dtype=np.uint8)
        c2 = rng.integers(0, 16, size=(batch, N, K) if tB else (batch, K, N), dtype=np.uint8)
        x1, x2 = orc.pack_nibbles(c1), orc.pack_nibbles(c2)
    else:
        x1 = gen_fp8(rng, (batch, M, K))
        x2 = gen_fp8(rng, (batch, N, K) if tB else (batch, K, N))
    s1 = (127 + rng.integers(-exp_range, exp_range + 1, size=(batch, M, KS, 2))).astype(np.uint8)
    s2 = (127 + rng.integers(-exp_range, exp_range + 1, size=(batch, N, KS, 2) if tB else (batch, KS, N, 2))).astype(np.uint8)
    return dict(x1=x1, x2=x2, s1=s1, s2=s2, fp4=fp4)


def oracle_mx(m, inp, M, K, N, tB, out_dtype, bias=None, rows=None):
    dt = orc.E2M1 if inp["fp4"] else orc.E4M3
    outs = []
    for b in range(inp["x1"].shape[0]):
        x1, s1, Mr = inp["x1"][b], inp["s1"][b], M
        if rows is not None:
            x1, s1, Mr = np.ascontiguousarray(x1[rows]), np.ascontiguousarray(s1[rows]), len(rows)
        outs.append(orc.qmm_mx(x1, inp["x2"][b], dt, dt, Mr, K, N, False, tB, s1, np.ascontiguousarray(inp["s2"][b]), bias, out_dtype))
    return np.stack(outs)


def run_mx_aclnn(m, inp, M, K, N, tB, out_dtype, bias=None, nz_storage=None):
    batch = inp["x1"].shape[0]
    bshape = (batch,) if batch > 1 else ()
    adt = m.ACL_FLOAT4_E2M1 if inp["fp4"] else m.ACL_FLOAT8_E4M3FN
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    out_np = orc.out_array((batch, M, N), out_dtype)
    d_out = guarded_out(m, out_np.nbytes)
    x1 = m.Tensor(bshape + (M, K), adt, d["x1"])
    x2 = m.Tensor(bshape + ((N, K) if tB else (K, N)), adt, d["x2"], fmt=29 if nz_storage else m.ACL_FORMAT_ND, storage_shape=nz_storage)
    s1 = m.Tensor(bshape + inp["s1"].shape[1:], m.ACL_FLOAT8_E8M0, d["s1"])
    s2 = m.Tensor(bshape + inp["s2"].shape[1:], m.ACL_FLOAT8_E8M0, d["s2"])
    out = m.Tensor(bshape + (M, N), out_dtype, d_out)
    d_bias = m.DeviceBuffer(host=bias) if bias is not None else None
    t_bias = m.Tensor((N,), m.ACL_FLOAT, d_bias) if bias is not None else None
    ws = m.quant_matmul_v5(x1, x2, s1, s2, out, bias=t_bias, transpose_x2=tB, group_size=(1 << 32) | (1 << 16) | 32,
                           weight_nz=bool(nz_storage))
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    del ws
    return d_out.to_host(out_np.dtype, out_np.shape)


# --------------------------------------------------------------------------------------------------
# weight-only (aclnnWeightQuantBatchMatmulV2)
# --------------------------------------------------------------------------------------------------
def make_wq_inputs(m, M, K, N, seed, x_dt, w_dt, group, tW, with_offset=True, bias_dt=None, scale_lo=0.005, scale_hi=0.02,
                   per_tensor=False, mx_exp=(-6, 2)):
    """x ~N(0,1) in x_dt; weight int8 [-127,127], int4 [-8,7], e4m3 ~N(0,1) or the 16 fp4 e2m1 codes; scale U(lo,hi) and
    offset U(-1,1) in x_dt -- or, for fp4 weights, one e8m0 byte per 32 K with the exponent uniform in mx_exp (no offset)."""
    rng = np.random.default_rng(seed)
    x = orc.f32_to_b16(rng.normal(0, 1, size=(M, K)).astype(np.float32), x_dt)
    wshape = (N, K) if tW else (K, N)
    if w_dt == m.ACL_INT8:
        w = rng.integers(-127, 128, size=wshape, dtype=np.int8)
    elif w_dt == m.ACL_INT4:
        w = orc.pack_nibbles((rng.integers(-8, 8, size=wshape) & 15).astype(np.uint8))
    elif w_dt == m.ACL_FLOAT8_E4M3FN:
        w = gen_fp8(rng, wshape)
    elif w_dt == m.ACL_FLOAT4_E2M1:
        w = orc.pack_nibbles(rng.integers(0, 16, size=wshape, dtype=np.uint8))
    else:
        raise ValueError(w_dt)
    G = -(-K // group) if group > 0 else 1
    sshape = (1,) if per_tensor else ((N, G) if tW else (G, N))
    bias = gen_bias(rng, N, bias_dt, m)
    if w_dt == m.ACL_FLOAT4_E2M1:   # MX: e8m0 scales, group 32, no offset
        assert group == 32 and not with_offset
        scale = (127 + rng.integers(mx_exp[0], mx_exp[1] + 1, size=sshape)).astype(np.uint8)
        return dict(x=x, w=w, scale=scale, offset=None, bias=bias, bias_dt=bias_dt, x_dt=x_dt, w_dt=w_dt, group=group, tW=tW,
                    per_tensor=False, scale_dt=m.ACL_FLOAT8_E8M0)
    scale = orc.f32_to_b16(rng.uniform(scale_lo, scale_hi, size=sshape).astype(np.float32), x_dt)
    offset = orc.f32_to_b16(rng.uniform(-1, 1, size=sshape).astype(np.float32), x_dt) if with_offset else None
    return dict(x=x, w=w, scale=scale, offset=offset, bias=bias, bias_dt=bias_dt, x_dt=x_dt, w_dt=w_dt, group=group, tW=tW,
                per_tensor=per_tensor, scale_dt=x_dt)


def oracle_wq(m, inp, M, K, N, rows=None):
    x = inp["x"] if rows is None else np.ascontiguousarray(inp["x"][rows])
    return orc.wqbmm(x, inp["x_dt"], inp["w"], inp["w_dt"], x.shape[0], K, N, inp["tW"], inp["scale"], inp.get("scale_dt", inp["x_dt"]),
                     1 if inp["per_tensor"] else N, inp["offset"], inp["group"], inp["bias"], inp["bias_dt"] or 0)


def run_wq_aclnn(m, inp, M, K, N, v3=False, scale_2d=None, nz_storage=None):
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    d_y = guarded_out(m, M * N * 2)
    tW, group = inp["tW"], inp["group"]
    G = -(-K // group) if group > 0 else 1
    x = m.Tensor((M, K), inp["x_dt"], d["x"])
    # the weight view is always the logical [K, N]; [N, K] storage is expressed through strides (1, K)
    # nz_storage: inp["w"] holds the FRACTAL_NZ bytes of the stored matrix and the call goes to aclnnWeightQuantBatchMatmulNz
    w = m.Tensor((K, N), inp["w_dt"], d["w"], strides=(1, K) if tW else None, fmt=29 if nz_storage else m.ACL_FORMAT_ND,
                 storage_shape=nz_storage)
    if inp["per_tensor"]:
        sshape, sst = (1,), None
    elif group > 0 or scale_2d:
        sshape, sst = (G, N), ((1, G) if tW else None)
    else:
        sshape, sst = (N,), None
    sc = m.Tensor(sshape, inp.get("scale_dt", inp["x_dt"]), d["scale"], strides=sst)
    off = m.Tensor(sshape, inp["x_dt"], d["offset"], strides=sst) if inp["offset"] is not None else None
    bias = m.Tensor((N,), inp["bias_dt"], d["bias"]) if inp["bias"] is not None else None
    y = m.Tensor((M, N), inp["x_dt"], d_y)
    ws = m.weight_quant_batch_matmul(x, w, sc, y, offset=off, bias=bias, group_size=group, inner_precise=0 if v3 else None,
                                     weight_nz=bool(nz_storage))
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    del ws
    return d_y.to_host(np.uint16, (M, N))


# --------------------------------------------------------------------------------------------------
# K-group modes of quant_batch_matmul_v4: fp8 x fp4 MX, fp8 x fp4 with 16-bit group scales (T-CG), int8 per-tile,
# int4 x int4 with per-group scales and offsets
# --------------------------------------------------------------------------------------------------
FP4_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0], np.float32)


def make_a8w4_mx_inputs(m, M, K, N, seed, tB):
    rng = np.random.default_rng(seed)
    KS = -(-K // 64)
    x1 = gen_fp8(rng, (M, K))
    x2 = orc.pack_nibbles(rng.integers(0, 16, size=(N, K) if tB else (K, N), dtype=np.uint8))
    s1 = (127 + rng.integers(-3, 4, size=(M, KS, 2))).astype(np.uint8)
    s2 = (127 + rng.integers(-3, 4, size=(N, KS, 2) if tB else (KS, N, 2))).astype(np.uint8)
    bias = orc.f32_to_f16(rng.normal(0, 1, N).astype(np.float32))
    return dict(x1=x1, x2=x2, s1=s1, s2=s2, bias=bias)


def oracle_a8w4_mx(m, inp, M, K, N, tB, out_dt, bias_dt=None):
    """inp["bias"] holds 16-bit patterns: fp16 unless bias_dt says bf16 (the mode wants the bias in the output's type)."""
    bias = orc.bf16_to_f32(inp["bias"]) if bias_dt == orc.BF16 else orc.f16_to_f32(inp["bias"])
    return orc.qmm_mx(inp["x1"], inp["x2"], orc.E4M3, orc.E2M1, M, K, N, False, tB, inp["s1"], inp["s2"], bias, out_dt)


def run_a8w4_mx_aclnn(m, inp, M, K, N, tB, out_dt, bias_dt=None):
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items()}
    out_np = orc.out_array((M, N), out_dt)
    d_out = guarded_out(m, out_np.nbytes)
    x1 = m.Tensor((M, K), m.ACL_FLOAT8_E4M3FN, d["x1"])
    x2 = m.Tensor((N, K) if tB else (K, N), m.ACL_FLOAT4_E2M1, d["x2"])
    s1 = m.Tensor(inp["s1"].shape, m.ACL_FLOAT8_E8M0, d["s1"])
    s2 = m.Tensor(inp["s2"].shape, m.ACL_FLOAT8_E8M0, d["s2"])
    bias = m.Tensor((1, N), bias_dt if bias_dt is not None else m.ACL_FLOAT16, d["bias"])
    out = m.Tensor((M, N), out_dt, d_out)
    ws = m.quant_matmul_v5(x1, x2, s1, s2, out, bias=bias, transpose_x2=tB, group_size=32)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    del ws
    return d_out.to_host(out_np.dtype, out_np.shape)


def make_tcg_inputs(m, M, K, N, seed, s_dt):
    """x2 stored [N, K] (the mode requires transposeX2), scales [N, K/32] in s_dt, yScale uint64 [1, N].
    Scales stay below 64 so that 6 * scale fits e4m3 (the cast's overflow behaviour is not pinned)."""
    rng = np.random.default_rng(seed)
    x1 = gen_fp8(rng, (M, K))
    x2 = orc.pack_nibbles(rng.integers(0, 16, size=(N, K), dtype=np.uint8))
    sf = rng.uniform(0.05, 60.0, size=(N, K // 32)).astype(np.float32)
    s2 = orc.f32_to_bf16(sf) if s_dt == m.ACL_BF16 else orc.f32_to_f16(sf)
    ys = orc.pack_u64_scale(rng.uniform(1e-3, 1e-2, N).astype(np.float32)).reshape(1, N)
    return dict(x1=x1, x2=x2, s2=s2, ys=ys, s_dt=s_dt)


def oracle_tcg(m, inp, M, K, N, out_dt):
    return orc.qmm_tcg(inp["x1"], inp["x2"], M, K, N, True, inp["s2"], inp["s_dt"], 32, inp["ys"], None, out_dt)


def run_tcg_aclnn(m, inp, M, K, N, out_dt, ys_dt=None):
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    out_np = orc.out_array((M, N), out_dt)
    d_out = guarded_out(m, out_np.nbytes)
    x1 = m.Tensor((M, K), m.ACL_FLOAT8_E4M3FN, d["x1"])
    x2 = m.Tensor((N, K), m.ACL_FLOAT4_E2M1, d["x2"])
    s2 = m.Tensor((N, K // 32), inp["s_dt"], d["s2"])
    ys = m.Tensor((1, N), ys_dt or m.ACL_UINT64, d["ys"])
    out = m.Tensor((M, N), out_dt, d_out)
    ws = m.quant_matmul_v5(x1, x2, None, s2, out, y_scale=ys, transpose_x2=True, group_size=32)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    del ws
    return d_out.to_host(out_np.dtype, out_np.shape)


def make_pertile_i8_inputs(m, M, K, N, seed, tB):
    rng = np.random.default_rng(seed)
    KB, NB = -(-K // 128), -(-N // 128)
    x1, x2 = gen_int8(rng, (M, K)), gen_int8(rng, (N, K) if tB else (K, N))
    s1 = gen_scale(rng, (M, KB), 1e-3, 1e-2)
    s2 = gen_scale(rng, (NB, KB) if tB else (KB, NB), 1e-3, 1e-2)
    bias = rng.normal(0, 1, N).astype(np.float32)
    return dict(x1=x1, x2=x2, s1=s1, s2=s2, bias=bias)


def oracle_pertile_i8(m, inp, M, K, N, tB, out_dt):
    return orc.qmm_perblock(inp["x1"], inp["x2"], orc.I8, orc.I8, M, K, N, False, tB, inp["s1"], inp["s2"], 1, 128, 128, inp["bias"], out_dt)


def run_pertile_i8_aclnn(m, inp, M, K, N, tB, out_dt):
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items()}
    out_np = orc.out_array((M, N), out_dt)
    d_out = guarded_out(m, out_np.nbytes)
    x1 = m.Tensor((M, K), m.ACL_INT8, d["x1"])
    x2 = m.Tensor((N, K) if tB else (K, N), m.ACL_INT8, d["x2"])
    s1 = m.Tensor(inp["s1"].shape, m.ACL_FLOAT, d["s1"])
    s2 = m.Tensor(inp["s2"].shape, m.ACL_FLOAT, d["s2"])
    bias = m.Tensor((N,), m.ACL_FLOAT, d["bias"])
    out = m.Tensor((M, N), out_dt, d_out)
    ws = m.quant_matmul_v5(x1, x2, s1, s2, out, bias=bias, transpose_x2=tB, group_size=(1 << 32) | (128 << 16) | 128)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    del ws
    return d_out.to_host(out_np.dtype, out_np.shape)


def make_i4_asym_inputs(m, M, K, N, seed):
    """x2 stored [N, K] (the mode requires transposeX2); scales fp32 and offsets fp16 [K/256, N]; x1Scale fp32 [M, 1]."""
    rng = np.random.default_rng(seed)
    x1 = orc.pack_nibbles(rng.integers(0, 16, size=(M, K), dtype=np.uint8))
    x2 = orc.pack_nibbles(rng.integers(0, 16, size=(N, K), dtype=np.uint8))
    G = -(-K // 256)
    s1 = gen_scale(rng, (M, 1), 1e-2, 1e-1)
    s2 = gen_scale(rng, (G, N), 1e-2, 1e-1)
    off = orc.f32_to_f16(rng.uniform(-8, 8, size=(G, N)).astype(np.float32))
    return dict(x1=x1, x2=x2, s1=s1, s2=s2, off=off)


def oracle_i4_asym(m, inp, M, K, N, out_dt):
    return orc.qmm_i4_asym(inp["x1"], inp["x2"], M, K, N, True, inp["s1"], inp["s2"], inp["off"], out_dt)


def run_i4_asym_aclnn(m, inp, M, K, N, out_dt):
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items()}
    out_np = orc.out_array((M, N), out_dt)
    d_out = guarded_out(m, out_np.nbytes)
    x1 = m.Tensor((M, K), m.ACL_INT4, d["x1"])
    x2 = m.Tensor((N, K), m.ACL_INT4, d["x2"])
    s1 = m.Tensor(inp["s1"].shape, m.ACL_FLOAT, d["s1"])
    s2 = m.Tensor(inp["s2"].shape, m.ACL_FLOAT, d["s2"])
    off = m.Tensor(inp["off"].shape, m.ACL_FLOAT16, d["off"])
    out = m.Tensor((M, N), out_dt, d_out)
    ws = m.quant_matmul_v5(x1, x2, s1, s2, out, x2_offset=off, transpose_x2=True, group_size=256)
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    del ws
    return d_out.to_host(out_np.dtype, out_np.shape)
