"""Workloads of bench.py: the five BASELINE configs with inputs resident on the device.
Lives beside the test helpers because it shares their seeded generators and, for the CPU-baseline leg only,
the oracle."""
import os
import time

import numpy as np

import cases
import oracle_api as orc


# HBM-side traffic per step in bytes (read + written), from the hardware counters FETCH_SIZE and WRITE_SIZE of the
# very same bench command, each scaled by what the counter reads for a byte transpose of known size; the runs and the
# figures are in profiles/<kernel>_<workload>.txt.  Keyed by (config, M of the weight-only configs).
MEASURED_TRAFFIC = {
    (2, None): 104.5e6, (4, None): 824.4e6, (5, None): 1802.2e6,
    (3, 1): 67.2e6, (3, 16): 69.2e6, (1, None): 9.2e6,
    (6, None): 583.0e6, (7, None): 132.4e6, (8, None): 260.2e6, (9, None): 405.9e6,
}


class Workload:
    metric = "quant_gemm_throughput"
    bound = "mfma"
    peak_key = "int8"
    kernel = ""
    dtype = ""
    flop = 0
    bytes = 0
    config = {}

    def step(self, stream):
        raise NotImplementedError

    def cpu_baseline(self):
        return None


def _cores():
    try:
        return len(os.sched_getaffinity(0))
    except Exception:
        return os.cpu_count() or 1


class Config2(Workload):
    """aclnnQuantMatmulV5, int8 x int8, per-token x per-channel fp32 scales, bf16 bias and output."""
    peak_key, dtype = "int8", "int8"
    kernel = "qgemm_i8_wide_kernel<FN=11> (256 x 352 tiles, one round of 256 workgroups)"

    def __init__(self, m, args, M=2048, K=4096, N=11008):
        self.m, self.M, self.K, self.N = m, M, K, N
        self.packed = args.layout == "packed"
        self.inp = cases.make_qmm_int8_inputs(m, M, K, N, 0, m.ACL_BF16, self.packed)
        r = getattr(args, "int8_range", None)
        if r:   # operands uniform in [-r, r] instead of the full int8 range (the sustained clock depends on the data)
            rng = np.random.default_rng(1)
            self.inp["x1"] = rng.integers(-r, r + 1, size=self.inp["x1"].shape, dtype=np.int8)
            self.inp["x2"] = rng.integers(-r, r + 1, size=self.inp["x2"].shape, dtype=np.int8)
        self.d = {k: m.DeviceBuffer(host=v) for k, v in self.inp.items() if isinstance(v, np.ndarray)}
        self.d_out = m.DeviceBuffer(M * N * 2)
        self.t_x1 = m.Tensor((M, K), m.ACL_INT8, self.d["x1"])
        # "packed": x2 is the logical [K, N] matrix stored K-contiguous (strides (1, K)), i.e. pre-packed offline
        if self.packed:
            self.t_x2 = m.Tensor((K, N), m.ACL_INT8, self.d["x2"], strides=(1, K))
        else:
            self.t_x2 = m.Tensor((K, N), m.ACL_INT8, self.d["x2"])
        self.t_s1 = m.Tensor((M,), m.ACL_FLOAT, self.d["s1"])
        self.t_s2 = m.Tensor((N,), m.ACL_FLOAT, self.d["s2"])
        self.t_bias = m.Tensor((N,), m.ACL_BF16, self.d["bias"])
        self.t_out = m.Tensor((M, N), m.ACL_BF16, self.d_out)
        rc, ws, ex = m.quant_matmul_v5_get_workspace(self.t_x1, self.t_x2, self.t_s1, self.t_s2, self.t_out, bias=self.t_bias)
        m.check(rc, "phase 1")
        m.lib().aclDestroyAclOpExecutor(ex)
        self.ws = m.DeviceBuffer(ws) if ws else None
        self.ws_size = ws
        self.flop = 2 * M * N * K
        self.bytes = M * K + K * N + 4 * M + 4 * N + 2 * N + 2 * M * N
        self.config = {"workload": "config2: aclnnQuantMatmulV5 W8A8 int8 K-C, bf16 bias/out", "M": M, "K": K, "N": N,
                       "x2_layout": "K-contiguous (pre-packed offline)" if self.packed else "N-contiguous (re-laid out per call)"}

    def step(self, stream):
        m = self.m
        rc, ws, ex = m.quant_matmul_v5_get_workspace(self.t_x1, self.t_x2, self.t_s1, self.t_s2, self.t_out, bias=self.t_bias)
        m.check(rc, "phase 1")
        m.check(m.lib().aclnnQuantMatmulV5(self.ws.ptr if self.ws else None, self.ws_size, ex, stream.ptr), "phase 2")

    def cpu_baseline(self):
        # bounded sample: the first R rows of x1 against the full x2 (same K, N), sized for roughly 10 s
        m = self.m
        s2f = cases.as_f32(self.inp["s2"], self.inp["s2_dtype"], m)

        def run(rows):
            x1 = np.ascontiguousarray(self.inp["x1"][0][:rows])
            t0 = time.perf_counter()
            orc.qmm_pertoken(x1, self.inp["x2"][0], rows, self.K, self.N, False, self.packed,
                             np.ascontiguousarray(self.inp["s1"][:rows]), s2f, self.inp["bias"], m.ACL_BF16, m.ACL_BF16)
            return time.perf_counter() - t0

        t = run(16)
        rows = int(min(self.M, max(16, 16 * (10.0 / max(t, 1e-3)) // 16 * 16)))
        t = run(rows)
        return {"value": 2.0 * rows * self.K * self.N / t / 1e12, "unit": "TFLOP/s", "cores": _cores(), "kind": "port",
                "sample": f"first {rows} of {self.M} rows of x1 against the full x2 (oracle/liboracle.so, OpenMP), {t:.2f} s"}


class Config4(Workload):
    """aclnnQuantMatmulV5, fp8 e4m3 x e4m3, G-B block scales (1x128 on x1, 128x128 on x2), bf16 output."""
    peak_key, dtype = "fp8", "fp8_e4m3"
    kernel = "qmm_fp8_block_kernel"

    def __init__(self, m, args, M=4096, K=7168, N=18432):
        self.m, self.M, self.K, self.N = m, M, K, N
        self.packed = args.layout == "packed"
        self.inp = cases.make_blockscale_inputs(m, M, K, N, 0, self.packed, 1)
        self.d = {k: m.DeviceBuffer(host=v) for k, v in self.inp.items() if isinstance(v, np.ndarray)}
        self.d_out = m.DeviceBuffer(M * N * 2)
        KB, NB = K // 128, N // 128
        self.t_x1 = m.Tensor((M, K), m.ACL_FLOAT8_E4M3FN, self.d["x1"])
        if self.packed:   # logical [K, N] stored K-contiguous; its block scales [KB, NB] stored [NB, KB] likewise
            self.t_x2 = m.Tensor((K, N), m.ACL_FLOAT8_E4M3FN, self.d["x2"], strides=(1, K))
            self.t_s2 = m.Tensor((KB, NB), m.ACL_FLOAT, self.d["s2"], strides=(1, KB))
        else:
            self.t_x2 = m.Tensor((K, N), m.ACL_FLOAT8_E4M3FN, self.d["x2"])
            self.t_s2 = m.Tensor((KB, NB), m.ACL_FLOAT, self.d["s2"])
        self.t_s1 = m.Tensor((M, KB), m.ACL_FLOAT, self.d["s1"])
        self.t_out = m.Tensor((M, N), m.ACL_BF16, self.d_out)
        self.gs = (1 << 32) | (128 << 16) | 128
        rc, ws, ex = m.quant_matmul_v5_get_workspace(self.t_x1, self.t_x2, self.t_s1, self.t_s2, self.t_out, group_size=self.gs)
        m.check(rc, "phase 1")
        m.lib().aclDestroyAclOpExecutor(ex)
        self.ws = m.DeviceBuffer(ws) if ws else None
        self.ws_size = ws
        self.flop = 2 * M * N * K
        self.bytes = M * K + K * N + 4 * M * KB + 4 * KB * NB + 2 * M * N
        self.config = {"workload": "config4: aclnnQuantMatmulV5 fp8 e4m3 G-B (1x128 / 128x128 scales), bf16 out", "M": M, "K": K,
                       "N": N, "x2_layout": "K-contiguous (pre-packed offline)" if self.packed else "N-contiguous (re-laid out per call)"}

    def step(self, stream):
        m = self.m
        rc, ws, ex = m.quant_matmul_v5_get_workspace(self.t_x1, self.t_x2, self.t_s1, self.t_s2, self.t_out, group_size=self.gs)
        m.check(rc, "phase 1")
        m.check(m.lib().aclnnQuantMatmulV5(self.ws.ptr if self.ws else None, self.ws_size, ex, stream.ptr), "phase 2")

    def cpu_baseline(self):
        rows = 64
        x1 = np.ascontiguousarray(self.inp["x1"][0][:rows])
        s1 = np.ascontiguousarray(self.inp["s1"][0][:rows])
        t0 = time.perf_counter()
        orc.qmm_perblock(x1, self.inp["x2"][0], orc.E4M3, orc.E4M3, rows, self.K, self.N, False, self.packed, s1,
                         np.ascontiguousarray(self.inp["s2"][0]), 1, 128, 128, None, orc.BF16)
        t = time.perf_counter() - t0
        return {"value": 2.0 * rows * self.K * self.N / t / 1e12, "unit": "TFLOP/s", "cores": _cores(), "kind": "port",
                "sample": f"first {rows} of {self.M} rows of x1 against the full x2 (oracle/liboracle.so, OpenMP), {t:.2f} s"}


class Config5(Workload):
    """aclnnQuantMatmulV5, MXFP4 (e2m1 with e8m0 scale per 32 K), batch 8, bf16 output."""
    peak_key, dtype = "fp4", "fp4_e2m1"
    kernel = "qgemm_kernel<mxfp4, 256x256x128B>"

    def __init__(self, m, args, B=8, M=4096, K=8192, N=8192):
        self.m, self.B, self.M, self.K, self.N = m, B, M, K, N
        self.packed = args.layout == "packed"
        self.inp = cases.make_mx_inputs(m, M, K, N, 0, self.packed, True, batch=B)
        self.d = {k: m.DeviceBuffer(host=v) for k, v in self.inp.items() if isinstance(v, np.ndarray)}
        self.d_out = m.DeviceBuffer(B * M * N * 2)
        KS = K // 64
        self.t_x1 = m.Tensor((B, M, K), m.ACL_FLOAT4_E2M1, self.d["x1"])
        self.t_s1 = m.Tensor((B, M, KS, 2), m.ACL_FLOAT8_E8M0, self.d["s1"])
        if self.packed:
            self.t_x2 = m.Tensor((B, K, N), m.ACL_FLOAT4_E2M1, self.d["x2"], strides=(K * N, 1, K))
            self.t_s2 = m.Tensor((B, KS, N, 2), m.ACL_FLOAT8_E8M0, self.d["s2"], strides=(N * KS * 2, 2, KS * 2, 1))
        else:
            self.t_x2 = m.Tensor((B, K, N), m.ACL_FLOAT4_E2M1, self.d["x2"])
            self.t_s2 = m.Tensor((B, KS, N, 2), m.ACL_FLOAT8_E8M0, self.d["s2"])
        self.t_out = m.Tensor((B, M, N), m.ACL_BF16, self.d_out)
        self.gs = (1 << 32) | (1 << 16) | 32
        rc, ws, ex = m.quant_matmul_v5_get_workspace(self.t_x1, self.t_x2, self.t_s1, self.t_s2, self.t_out, group_size=self.gs)
        m.check(rc, "phase 1")
        m.lib().aclDestroyAclOpExecutor(ex)
        self.ws = m.DeviceBuffer(ws) if ws else None
        self.ws_size = ws
        self.flop = 2 * B * M * N * K
        self.bytes = B * (M * K // 2 + K * N // 2 + M * K // 32 + N * K // 32 + 2 * M * N)
        self.config = {"workload": "config5: aclnnQuantMatmulV5 MXFP4 batched, bf16 out", "B": B, "M": M, "K": K, "N": N,
                       "x2_layout": "K-contiguous (pre-packed offline)" if self.packed else "N-contiguous (re-laid out per call)"}

    def step(self, stream):
        m = self.m
        rc, ws, ex = m.quant_matmul_v5_get_workspace(self.t_x1, self.t_x2, self.t_s1, self.t_s2, self.t_out, group_size=self.gs)
        m.check(rc, "phase 1")
        m.check(m.lib().aclnnQuantMatmulV5(self.ws.ptr if self.ws else None, self.ws_size, ex, stream.ptr), "phase 2")

    def cpu_baseline(self):
        rows = 64
        x1 = np.ascontiguousarray(self.inp["x1"][0][:rows])
        s1 = np.ascontiguousarray(self.inp["s1"][0][:rows])
        t0 = time.perf_counter()
        orc.qmm_mx(x1, self.inp["x2"][0], orc.E2M1, orc.E2M1, rows, self.K, self.N, False, self.packed, s1,
                   np.ascontiguousarray(self.inp["s2"][0]), None, orc.BF16)
        t = time.perf_counter() - t0
        return {"value": 2.0 * rows * self.K * self.N / t / 1e12, "unit": "TFLOP/s", "cores": _cores(), "kind": "port",
                "sample": f"first {rows} of {self.M} rows of batch slice 0 against its full x2 (oracle/liboracle.so, OpenMP), {t:.2f} s"}


class ConfigWQ(Workload):
    """aclnnWeightQuantBatchMatmulV2: config 1 (W8A16 per-channel bf16, M=16) and config 3 (W4A16 per-group fp16 decode)."""
    bound = "hbm"

    def __init__(self, m, args, config):
        self.m = m
        self.packed = args.layout == "packed"
        if config == 1:
            M, K, N, x_dt, w_dt, group, off = 16, 4096, 4096, m.ACL_BF16, m.ACL_INT8, 0, False
            self.dtype, lo, hi = "bf16 (int8 weights)", 1e-4, 0.06
            name = "config1: aclnnWeightQuantBatchMatmulV2 W8A16 per-channel bf16"
        else:
            M, K, N, x_dt, w_dt, group, off = (args.m or 16), 8192, 28672, m.ACL_FLOAT16, m.ACL_INT4, 128, True
            self.dtype, lo, hi = "f16 (int4 weights)", 0.005, 0.02
            name = "config3: aclnnWeightQuantBatchMatmulV2 W4A16 per-group(128) fp16 decode"
        self.M, self.K, self.N, self.group = M, K, N, group
        self.kernel = "wqmm_resx_kernel" if (config == 3 and M <= 3) else ("wqmm_rows_kernel" if M > 48 else "wqmm_stream_kernel")
        self.inp = cases.make_wq_inputs(m, M, K, N, 0, x_dt, w_dt, group, self.packed, off, None, lo, hi)
        inp = self.inp
        self.ncopies = 1
        wbytes = inp["w"].nbytes
        if args.cold:   # rotate through enough weight copies to exceed the 256 MB last-level cache
            self.ncopies = max(2, int(np.ceil(600e6 / wbytes)))
        self.d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray) and k != "w"}
        self.d_w = [m.DeviceBuffer(host=inp["w"]) for _ in range(self.ncopies)]
        self.d_y = m.DeviceBuffer(M * N * 2)
        G = -(-K // group) if group > 0 else 1
        self.t_x = m.Tensor((M, K), x_dt, self.d["x"])
        self.t_w = [m.Tensor((K, N), w_dt, d, strides=(1, K) if self.packed else None) for d in self.d_w]
        if group > 0:
            sshape, sst = (G, N), ((1, G) if self.packed else None)
        else:
            sshape, sst = (N,), None
        self.t_sc = m.Tensor(sshape, x_dt, self.d["scale"], strides=sst)
        self.t_off = m.Tensor(sshape, x_dt, self.d["offset"], strides=sst) if off else None
        self.t_y = m.Tensor((M, N), x_dt, self.d_y)
        rc, ws, ex = m.weight_quant_batch_matmul_get_workspace(self.t_x, self.t_w[0], self.t_sc, self.t_y, offset=self.t_off,
                                                               group_size=group)
        m.check(rc, "phase 1")
        m.lib().aclDestroyAclOpExecutor(ex)
        self.ws = m.DeviceBuffer(ws) if ws else None
        self.ws_size = ws
        self.flop = 2 * M * N * K
        wb = K * N * (1 if w_dt == m.ACL_INT8 else 0.5)
        self.bytes = int(wb + 2 * M * K + 2 * M * N + 2 * G * N * (2 if off else 1))
        self.config = {"workload": name, "M": M, "K": K, "N": N, "group": group, "weight_copies_rotated": self.ncopies,
                       "weight_layout": "K-contiguous (pre-packed offline)" if self.packed else "N-contiguous (re-laid out per call)"}
        self.i = 0

    def step(self, stream):
        m = self.m
        w = self.t_w[self.i % self.ncopies]
        self.i += 1
        rc, ws, ex = m.weight_quant_batch_matmul_get_workspace(self.t_x, w, self.t_sc, self.t_y, offset=self.t_off,
                                                               group_size=self.group)
        m.check(rc, "phase 1")
        m.check(m.lib().aclnnWeightQuantBatchMatmulV2(self.ws.ptr if self.ws else None, self.ws_size, ex, stream.ptr), "phase 2")

    def cpu_baseline(self):
        t0 = time.perf_counter()
        cases.oracle_wq(self.m, self.inp, self.M, self.K, self.N)
        t = time.perf_counter() - t0
        return {"value": self.bytes / t / 1e9, "unit": "GB/s", "cores": _cores(), "kind": "port",
                "sample": f"the whole workload once (oracle/liboracle.so, OpenMP), {t:.2f} s"}


class PrepOp(Workload):
    """The operators either side of the matmuls, each on the tensor of the BASELINE config it prepares (HBM-bound):
    6 aclnnConvertWeightToINT4Pack on config 3's weight; 7 aclnnDynamicQuant (int8) on config 2's activation, 8 batches of it;
    8 aclnnDynamicBlockQuant (e4m3, 128 x 128) on config 4's weight; 9 aclnnDynamicMxQuant (e2m1) on config 5's activation."""
    metric = "prep_op_bandwidth"
    bound = "hbm"

    def __init__(self, m, args, config):
        self.m, self.op = m, config
        rng = np.random.default_rng(0)
        if config == 6:
            K, N = 8192, 28672
            self.host = rng.integers(-8, 8, size=(K, N)).astype(np.int32)
            self.d_in, self.d_out = m.DeviceBuffer(host=self.host), m.DeviceBuffer(K * N // 2)
            self.count = K * N
            self.bytes = K * N * 4 + K * N // 2
            self.kernel, self.dtype = "pack_b4_kernel", "u32"
            self.config = {"workload": "aclnnConvertWeightToINT4Pack on config 3's weight", "K": K, "N": N}
            return
        rows, cols = {7: (8 * 2048, 4096), 8: (18432, 7168), 9: (8 * 4096, 8192)}[config]
        self.rows, self.cols = rows, cols
        self.xb = orc.f32_to_bf16(rng.normal(0, 1, size=(rows, cols)).astype(np.float32))
        self.d_in = m.DeviceBuffer(host=self.xb)
        x = m.Tensor((rows, cols), m.ACL_BF16, self.d_in)
        if config == 7:
            self.d_out, self.d_sc = m.DeviceBuffer(rows * cols), m.DeviceBuffer(rows * 4)
            self.tensors = (x, m.Tensor((rows, cols), m.ACL_INT8, self.d_out), m.Tensor((rows,), m.ACL_FLOAT, self.d_sc))
            self.bytes = rows * cols * 3 + rows * 4
            self.kernel, self.dtype = "dynamic_quant_rows_kernel", "f32"
            self.config = {"workload": "aclnnDynamicQuant (int8, per token) on 8 batches of config 2's activation", "rows": rows, "cols": cols}
        elif config == 8:
            self.d_out, self.d_sc = m.DeviceBuffer(rows * cols), m.DeviceBuffer(rows // 128 * (cols // 128) * 4)
            self.tensors = (x, m.Tensor((rows, cols), m.ACL_FLOAT8_E4M3FN, self.d_out), m.Tensor((rows // 128, cols // 128), m.ACL_FLOAT, self.d_sc))
            self.bytes = rows * cols * 3 + rows // 128 * (cols // 128) * 4
            self.kernel, self.dtype = "block_quant_tile_kernel", "f32"
            self.config = {"workload": "aclnnDynamicBlockQuant (e4m3, 128 x 128 blocks) on config 4's weight", "rows": rows, "cols": cols}
        else:
            self.d_out, self.d_sc = m.DeviceBuffer(rows * cols // 2), m.DeviceBuffer(rows * cols // 32)
            self.tensors = (x, m.Tensor((rows, cols), m.ACL_FLOAT4_E2M1, self.d_out), m.Tensor((rows, cols // 64, 2), m.ACL_FLOAT8_E8M0, self.d_sc))
            self.bytes = rows * cols * 2 + rows * cols // 2 + rows * cols // 32
            self.kernel, self.dtype = "mx_quant_kernel", "f32"
            self.config = {"workload": "aclnnDynamicMxQuant (e2m1, blocks of 32) on config 5's activation, all 8 batches", "rows": rows, "cols": cols}

    def step(self, stream):
        m = self.m
        if self.op == 6:   # the aclnn entry point of this op works on the null stream and waits; the stream form is timed
            m.check(m.lib().opsnnPackB4(self.d_in.ptr, 0, self.d_out.ptr, self.count, stream.ptr), "opsnnPackB4")
        elif self.op == 7:
            m.dynamic_quant(*self.tensors, stream=stream)
        elif self.op == 8:
            m.dynamic_block_quant(*self.tensors, stream=stream, row_block=128, col_block=128)
        else:
            m.dynamic_mx_quant(*self.tensors, stream=stream)

    def cpu_baseline(self):
        t0 = time.perf_counter()
        if self.op == 6:
            orc.convert_weight_b4(self.host)
        elif self.op == 7:
            orc.dynamic_quant(self.xb, orc.BF16, orc.I8)
        elif self.op == 8:
            orc.dynamic_block_quant(self.xb, orc.BF16, orc.E4M3, 128, 128)
        else:
            orc.dynamic_mx_quant(self.xb, orc.BF16, orc.E2M1)
        t = time.perf_counter() - t0
        return {"value": self.bytes / t / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"the whole workload once (oracle/liboracle.so, one thread), {t:.2f} s"}


def make_workload(m, config, args):
    if config in (6, 7, 8, 9):
        return PrepOp(m, args, config)
    if config in (1, 3):
        return ConfigWQ(m, args, config)
    if config == 2:
        return Config2(m, args)
    if config == 4:
        return Config4(m, args)
    if config == 5:
        return Config5(m, args)
    raise SystemExit(f"bench.py: config {config} is not wired up yet")
