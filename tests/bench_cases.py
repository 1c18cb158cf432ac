"""Workloads of bench.py: the five BASELINE configs with inputs resident on the device.
Lives beside the test helpers because it shares their seeded generators and, for the CPU-baseline leg only,
the oracle."""
import os
import time

import numpy as np

import cases
import oracle_api as orc


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
    kernel = "qmm_i8_mfma"

    def __init__(self, m, args, M=2048, K=4096, N=11008):
        self.m, self.M, self.K, self.N = m, M, K, N
        self.packed = args.layout == "packed"
        self.inp = cases.make_qmm_int8_inputs(m, M, K, N, 0, m.ACL_BF16, self.packed)
        if os.environ.get("OPSNN_BENCH_ZERO"):   # experiment: data-dependent power
            self.inp["x1"][:] = 0
            self.inp["x2"][:] = 0
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


def make_workload(m, config, args):
    if config == 2:
        return Config2(m, args)
    raise SystemExit(f"bench.py: config {config} is not wired up yet")
