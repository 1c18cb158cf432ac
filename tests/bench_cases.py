"""Workloads of bench.py: the five BASELINE configs with inputs resident on the device.
Lives beside the test helpers because it shares their seeded generators and, for the CPU-baseline leg only,
the oracle."""
import os
import time

import numpy as np

import cases
import oracle_api as orc


# HBM-side traffic per step in bytes (read + written) as the memory-side request counters of an EARLIER profiling run of
# the same bench command gave it (profiles/<file>: TCC_EA0_RDREQ / _32B and TCC_EA0_WRREQ / _64B, with the bytes per
# request taken from two kernels of known size in the same run: a 16-byte-per-lane streaming read and a byte transpose).
# bench.py does not measure it; it copies the figure and names the file.  A figure below the algorithmic bytes would not
# be evidence and is reported as null.  Keyed by (config, M of the weight-only configs, variant).
PROFILED_TRAFFIC = {
    (1, None, "warm"): (20.7e6, "profiles/wqmm_decode_w8a16_m16_k4096_n4096.txt"),
    (1, None, "cold"): (20.5e6, "profiles/wqmm_decode_w8a16_m16_k4096_n4096_cold.txt"),
    (2, None, None): (162.5e6, "profiles/qgemm_int8_w8a8_m2048_k4096_n11008.txt"),
    (3, 1, "warm"): (144.0e6, "profiles/wqmm_decode_w4a16_m1_k8192_n28672.txt"),
    (3, 1, "cold"): (140.9e6, "profiles/wqmm_decode_w4a16_m1_k8192_n28672_cold.txt"),
    (3, 16, "warm"): (132.5e6, "profiles/wqmm_decode_w4a16_m16_k8192_n28672.txt"),
    (3, 16, "cold"): (132.7e6, "profiles/wqmm_decode_w4a16_m16_k8192_n28672_cold.txt"),
    (3, 64, "warm"): (137.8e6, "profiles/wqmm_decode_w4a16_m64_k8192_n28672.txt"),
    (3, 64, "cold"): (137.9e6, "profiles/wqmm_decode_w4a16_m64_k8192_n28672_cold.txt"),
    (3, 256, "warm"): (196.9e6, "profiles/wqmm_decode_w4a16_m256_k8192_n28672.txt"),
    (3, 256, "cold"): (193.0e6, "profiles/wqmm_decode_w4a16_m256_k8192_n28672_cold.txt"),
    (4, None, "exact"): (1220.1e6, "profiles/qmm_fp8_exact_m4096_k7168_n18432.txt"),
    (4, None, "fast"): (1502.5e6, "profiles/qmm_fp8_block_m4096_k7168_n18432.txt"),
    (5, None, None): (2229.7e6, "profiles/qgemm_mxfp4_b8_m4096_k8192_n8192.txt"),
    (6, None, None): (1052.7e6, "profiles/pack_b4_k8192_n28672.txt"),
    (7, None, None): (199.4e6, "profiles/dynamic_quant_int8_16384x4096.txt"),
    (8, None, None): (392.1e6, "profiles/block_quant_e4m3_128x128_18432x7168.txt"),
    (9, None, None): (674.5e6, "profiles/mx_quant_e2m1_32768x8192.txt"),
    (10, None, None): (290.3e6, "profiles/qmm_i4_kg_m4096_k4096_n4096.txt"),
    (12, 16, "exact"): (136.9e6, "profiles/qmm_fp8_block_decode_m16_k7168_n18432.txt"),
    (12, 64, "exact"): (143.5e6, "profiles/qmm_fp8_block_rows_m64_k7168_n18432.txt"),
    (12, 128, "exact"): (154.8e6, "profiles/qmm_fp8_block_rows_m128_k7168_n18432.txt"),
    (13, 16, None): (131.0e6, "profiles/qmm_mx_a8w4_decode_m16_k8192_n28672.txt"),
    (14, 16, None): (244.0e6, "profiles/qmm_i8_pertile_decode_m16_k8192_n28672.txt"),
    (11, 16, "warm"): (133.5e6, "profiles/wqmm_decode_mxfp4_m16_k8192_n28672.txt"),
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

    variant = None
    instr_peak_key = None   # matrix instruction actually issued, when it is not the operand dtype's

    def begin(self):
        pass

    def end(self):
        pass

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
    """aclnnQuantMatmulV5, fp8 e4m3 x e4m3, G-B block scales (1x128 on x1, 128x128 on x2), bf16 output.
    Default arithmetic: e4m3 widened exactly to fp16 in registers, fp16 matrix instruction (exact products); `fast`
    selects the 8-bit matrix instruction (opsnnSetFp8Fast)."""
    peak_key = "fp8"

    def __init__(self, m, args, M=4096, K=7168, N=18432):
        self.m, self.M, self.K, self.N = m, M, K, N
        self.packed = args.layout == "packed"
        self.fast = bool(getattr(args, "fp8_fast", False))
        if self.fast:
            self.dtype, self.kernel, self.instr_peak_key = "fp8_e4m3", "qmm_fp8_block_kernel (v_mfma_scale_f32_16x16x128_f8f6f4)", "fp8"
        else:
            self.dtype = "f16 products of e4m3 operands (widened exactly in registers), fp32 sums"
            self.kernel, self.instr_peak_key = "qmm_fp8_exact_kernel (v_mfma_f32_16x16x32_f16)", "f16"
        self.variant = "fast" if self.fast else "exact"
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
                       "N": N, "arithmetic": "8-bit matrix instruction (opsnnSetFp8Fast(1))" if self.fast else "exact fp16 products (default)",
                       "x2_layout": "K-contiguous (pre-packed offline)" if self.packed else "N-contiguous (re-laid out per call)"}

    def begin(self):
        self.m.lib().opsnnSetFp8Fast(1 if self.fast else 0)

    def end(self):
        self.m.lib().opsnnSetFp8Fast(0)

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


class Config4Rows(Config4):
    """Not a BASELINE config: config 4's operator, K and N with the few rows of x1 of a decode step (--m, default 16).  The
    call is a stream over x2: reported against the HBM roofline (bytes of both operands, scales and the output per step)."""
    metric = "quant_gemm_stream_bandwidth"
    bound = "hbm"

    def __init__(self, m, args):
        M = args.m or 16
        super().__init__(m, args, M=M)
        self.instr_peak_key = None
        self.kernel = "fp8_block_decode_kernel" if M <= 16 else "wqmm_rows_kernel<f16, e4m3, block scales> (+ widen_e4m3_f16_kernel)" if M <= 128 else self.kernel
        self.config = dict(self.config, workload="aclnnQuantMatmulV5 fp8 e4m3 G-B (1x128 / 128x128 scales), bf16 out, decode rows")


class ConfigA8W4Rows(Workload):
    """Not a BASELINE config: the fp8 x fp4 MX mode of aclnnQuantMatmulV5 (e8m0 scales per 32 elements of K) at config 3's
    K and N with the few rows of x1 of a decode step (--m, default 16): a stream over the 4-bit x2, reported against the
    HBM roofline (both operands, both scale tables, bias and output per step)."""
    metric = "quant_gemm_stream_bandwidth"
    bound = "hbm"
    peak_key = "fp8"
    dtype = "fp8_e4m3 x fp4_e2m1, e8m0 scales inside the matrix instruction, fp32 sums"
    kernel = "mx_a8w4_decode_kernel (v_mfma_scale_f32_16x16x128_f8f6f4)"

    def __init__(self, m, args, K=8192, N=28672):
        M = args.m or 16
        self.m, self.M, self.K, self.N = m, M, K, N
        self.inp = cases.make_a8w4_mx_inputs(m, M, K, N, 0, True)
        self.d = {k: m.DeviceBuffer(host=v) for k, v in self.inp.items()}
        self.d_out = m.DeviceBuffer(M * N * 2)
        self.t_x1 = m.Tensor((M, K), m.ACL_FLOAT8_E4M3FN, self.d["x1"])
        self.t_x2 = m.Tensor((N, K), m.ACL_FLOAT4_E2M1, self.d["x2"])
        self.t_s1 = m.Tensor(self.inp["s1"].shape, m.ACL_FLOAT8_E8M0, self.d["s1"])
        self.t_s2 = m.Tensor(self.inp["s2"].shape, m.ACL_FLOAT8_E8M0, self.d["s2"])
        self.t_bias = m.Tensor((1, N), m.ACL_FLOAT16, self.d["bias"])
        self.t_out = m.Tensor((M, N), m.ACL_FLOAT16, self.d_out)
        rc, ws, ex = m.quant_matmul_v5_get_workspace(self.t_x1, self.t_x2, self.t_s1, self.t_s2, self.t_out, bias=self.t_bias,
                                                     transpose_x2=True, group_size=32)
        m.check(rc, "phase 1")
        m.lib().aclDestroyAclOpExecutor(ex)
        self.ws = m.DeviceBuffer(ws) if ws else None
        self.ws_size = ws
        self.flop = 2 * M * N * K
        self.bytes = M * K + N * K // 2 + M * K // 32 + N * K // 32 + 2 * N + 2 * M * N
        self.config = {"workload": "aclnnQuantMatmulV5 fp8 e4m3 x fp4 e2m1 MX, fp16 bias and out, decode rows", "M": M, "K": K, "N": N,
                       "x2_layout": "K-contiguous (transposeX2)"}

    def step(self, stream):
        m = self.m
        rc, ws, ex = m.quant_matmul_v5_get_workspace(self.t_x1, self.t_x2, self.t_s1, self.t_s2, self.t_out, bias=self.t_bias,
                                                     transpose_x2=True, group_size=32)
        m.check(rc, "phase 1")
        m.check(m.lib().aclnnQuantMatmulV5(self.ws.ptr if self.ws else None, self.ws_size, ex, stream.ptr), "phase 2")

    def cpu_baseline(self):
        rows = min(self.M, 16)
        t0 = time.perf_counter()
        orc.qmm_mx(np.ascontiguousarray(self.inp["x1"][:rows]), self.inp["x2"], orc.E4M3, orc.E2M1, rows, self.K, self.N, False, True,
                   np.ascontiguousarray(self.inp["s1"][:rows]), self.inp["s2"], orc.f16_to_f32(self.inp["bias"]), orc.F16)
        t = time.perf_counter() - t0
        return {"value": self.bytes * rows / self.M / t / 1e9, "unit": "GB/s", "cores": _cores(), "kind": "port",
                "sample": f"first {rows} of {self.M} rows of x1 against the full x2 (oracle/liboracle.so, OpenMP), {t:.2f} s"}


class ConfigPerTileRows(Workload):
    """Not a BASELINE config: the int8 per-tile mode of aclnnQuantMatmulV5 (1x128 scales on x1, 128x128 on x2, fp32 bias) at
    config 3's K and N with the few rows of x1 of a decode step (--m, default 16): a stream over x2 against the HBM roofline."""
    metric = "quant_gemm_stream_bandwidth"
    bound = "hbm"
    peak_key = "int8"
    dtype = "int8 x int8, exact int32 sums per 128-block, fp32 fold"
    kernel = "fp8_block_decode_kernel<int8> (v_mfma_i32_16x16x64_i8)"

    def __init__(self, m, args, K=8192, N=28672):
        M = args.m or 16
        self.m, self.M, self.K, self.N = m, M, K, N
        self.inp = cases.make_pertile_i8_inputs(m, M, K, N, 0, True)
        self.d = {k: m.DeviceBuffer(host=v) for k, v in self.inp.items()}
        self.d_out = m.DeviceBuffer(M * N * 2)
        self.t_x1 = m.Tensor((M, K), m.ACL_INT8, self.d["x1"])
        self.t_x2 = m.Tensor((N, K), m.ACL_INT8, self.d["x2"])
        self.t_s1 = m.Tensor(self.inp["s1"].shape, m.ACL_FLOAT, self.d["s1"])
        self.t_s2 = m.Tensor(self.inp["s2"].shape, m.ACL_FLOAT, self.d["s2"])
        self.t_bias = m.Tensor((N,), m.ACL_FLOAT, self.d["bias"])
        self.t_out = m.Tensor((M, N), m.ACL_BF16, self.d_out)
        self.gs = (1 << 32) | (128 << 16) | 128
        rc, ws, ex = self._phase1()
        m.lib().aclDestroyAclOpExecutor(ex)
        self.ws = m.DeviceBuffer(ws) if ws else None
        self.ws_size = ws
        self.flop = 2 * M * N * K
        self.bytes = M * K + N * K + 4 * M * (K // 128) + 4 * (N // 128) * (K // 128) + 4 * N + 2 * M * N
        self.config = {"workload": "aclnnQuantMatmulV5 int8 per-tile (1x128 / 128x128 scales), fp32 bias, bf16 out, decode rows", "M": M, "K": K,
                       "N": N, "x2_layout": "K-contiguous (transposeX2)"}

    def _phase1(self):
        m = self.m
        rc, ws, ex = m.quant_matmul_v5_get_workspace(self.t_x1, self.t_x2, self.t_s1, self.t_s2, self.t_out, bias=self.t_bias,
                                                     transpose_x2=True, group_size=self.gs)
        m.check(rc, "phase 1")
        return rc, ws, ex

    def step(self, stream):
        m = self.m
        rc, ws, ex = self._phase1()
        m.check(m.lib().aclnnQuantMatmulV5(self.ws.ptr if self.ws else None, self.ws_size, ex, stream.ptr), "phase 2")

    def cpu_baseline(self):
        rows = min(self.M, 16)
        t0 = time.perf_counter()
        orc.qmm_perblock(np.ascontiguousarray(self.inp["x1"][:rows]), self.inp["x2"], orc.I8, orc.I8, rows, self.K, self.N, False, True,
                         np.ascontiguousarray(self.inp["s1"][:rows]), self.inp["s2"], 1, 128, 128, self.inp["bias"], orc.BF16)
        t = time.perf_counter() - t0
        return {"value": self.bytes * rows / self.M / t / 1e9, "unit": "GB/s", "cores": _cores(), "kind": "port",
                "sample": f"first {rows} of {self.M} rows of x1 against the full x2 (oracle/liboracle.so, OpenMP), {t:.2f} s"}


class ConfigMxfp8Rows(Workload):
    """Not a BASELINE config: MXFP8 (e4m3 x e4m3, e8m0 scales per 32 elements of K on both operands) at config 3's K and N with
    the few rows of x1 of a decode step (--m, default 16): a stream over x2 against the HBM roofline."""
    metric = "quant_gemm_stream_bandwidth"
    bound = "hbm"
    peak_key = "fp8"
    dtype = "fp8_e4m3 x fp8_e4m3, both widened to bf16 with their e8m0 block scales (exact), fp32 sums"
    kernel = "mx8_decode_kernel (v_mfma_f32_16x16x32_bf16); from 17 rows wqmm_rows_kernel on e4m3 codes with e8m0 scales"

    def __init__(self, m, args, K=8192, N=28672):
        M = args.m or 16
        self.m, self.M, self.K, self.N = m, M, K, N
        self.inp = cases.make_mx_inputs(m, M, K, N, 0, True, False)
        self.d = {k: m.DeviceBuffer(host=v) for k, v in self.inp.items() if isinstance(v, np.ndarray)}
        self.d_out = m.DeviceBuffer(M * N * 2)
        KS = K // 64
        self.t_x1 = m.Tensor((M, K), m.ACL_FLOAT8_E4M3FN, self.d["x1"])
        self.t_x2 = m.Tensor((N, K), m.ACL_FLOAT8_E4M3FN, self.d["x2"])
        self.t_s1 = m.Tensor((M, KS, 2), m.ACL_FLOAT8_E8M0, self.d["s1"])
        self.t_s2 = m.Tensor((N, KS, 2), m.ACL_FLOAT8_E8M0, self.d["s2"])
        self.t_out = m.Tensor((M, N), m.ACL_BF16, self.d_out)
        self.gs = (1 << 32) | (1 << 16) | 32
        rc, ws, ex = self._phase1()
        m.lib().aclDestroyAclOpExecutor(ex)
        self.ws = m.DeviceBuffer(ws) if ws else None
        self.ws_size = ws
        self.flop = 2 * M * N * K
        self.bytes = M * K + N * K + M * K // 32 + N * K // 32 + 2 * M * N
        self.config = {"workload": "aclnnQuantMatmulV5 MXFP8 (e8m0 scales per 32 K), bf16 out, decode rows", "M": M, "K": K, "N": N,
                       "x2_layout": "K-contiguous (transposeX2)"}

    def _phase1(self):
        m = self.m
        rc, ws, ex = m.quant_matmul_v5_get_workspace(self.t_x1, self.t_x2, self.t_s1, self.t_s2, self.t_out, transpose_x2=True, group_size=self.gs)
        m.check(rc, "phase 1")
        return rc, ws, ex

    def step(self, stream):
        m = self.m
        rc, ws, ex = self._phase1()
        m.check(m.lib().aclnnQuantMatmulV5(self.ws.ptr if self.ws else None, self.ws_size, ex, stream.ptr), "phase 2")

    def cpu_baseline(self):
        rows = min(self.M, 16)
        t0 = time.perf_counter()
        orc.qmm_mx(np.ascontiguousarray(self.inp["x1"][0][:rows]), self.inp["x2"][0], orc.E4M3, orc.E4M3, rows, self.K, self.N, False, True,
                   np.ascontiguousarray(self.inp["s1"][0][:rows]), np.ascontiguousarray(self.inp["s2"][0]), None, orc.BF16)
        t = time.perf_counter() - t0
        return {"value": self.bytes * rows / self.M / t / 1e9, "unit": "GB/s", "cores": _cores(), "kind": "port",
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
    """aclnnWeightQuantBatchMatmulV2: config 1 (W8A16 per-channel bf16, M=16) and config 3 (W4A16 per-group fp16 decode).
    One object serves every M of config 3 (set_m) and both cache states (set_cold): the weight copies stay on the device."""
    bound = "hbm"

    def __init__(self, m, args, config, max_m=None):
        self.m = m
        self.packed = args.layout == "packed"
        if config == 1:
            M, K, N, x_dt, w_dt, group, off = 16, 4096, 4096, m.ACL_BF16, m.ACL_INT8, 0, False
            self.dtype, lo, hi = "bf16 (int8 weights)", 1e-4, 0.06
            self.name = "config1: aclnnWeightQuantBatchMatmulV2 W8A16 per-channel bf16"
        elif config == 11:   # not a BASELINE config: config 3's shape with mxfp4 weights (e2m1, one e8m0 scale per 32 K, no offset)
            M, K, N, x_dt, w_dt, group, off = (max_m or args.m or 16), 8192, 28672, m.ACL_FLOAT16, m.ACL_FLOAT4_E2M1, 32, False
            self.dtype, lo, hi = "f16 (mxfp4 weights)", 0.005, 0.02
            self.name = "aclnnWeightQuantBatchMatmulV2 mxfp4 weights (e2m1, e8m0 per 32 K), fp16 decode, config 3's shape"
        else:
            M, K, N, x_dt, w_dt, group, off = (max_m or args.m or 16), 8192, 28672, m.ACL_FLOAT16, m.ACL_INT4, 128, True
            self.dtype, lo, hi = "f16 (int4 weights)", 0.005, 0.02
            self.name = "config3: aclnnWeightQuantBatchMatmulV2 W4A16 per-group(128) fp16 decode"
        self.cfg, self.K, self.N, self.group, self.x_dt, self.w_dt, self.off = config, K, N, group, x_dt, w_dt, off
        self.inp_full = cases.make_wq_inputs(m, M, K, N, 0, x_dt, w_dt, group, self.packed, off, None, lo, hi)
        inp = self.inp_full
        self.d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray) and k != "w"}
        self.d_w = [m.DeviceBuffer(host=inp["w"])]
        self.d_y = m.DeviceBuffer(M * N * 2)
        self.G = -(-K // group) if group > 0 else 1
        if group > 0:
            sshape, sst = (self.G, N), ((1, self.G) if self.packed else None)
        else:
            sshape, sst = (N,), None
        self.scale_dt = inp.get("scale_dt", x_dt)
        self.t_sc = m.Tensor(sshape, self.scale_dt, self.d["scale"], strides=sst)
        self.t_off = m.Tensor(sshape, x_dt, self.d["offset"], strides=sst) if off else None
        self.ncopies = 1
        self.i = 0
        self.set_cold(bool(getattr(args, "cold", False)))
        self.set_m(M)

    def set_cold(self, cold):
        """cold: rotate through enough weight copies to exceed the 256 MB last-level cache between two uses of one copy."""
        m = self.m
        want = max(2, int(np.ceil(600e6 / self.inp_full["w"].nbytes))) if cold else 1
        while len(self.d_w) < want:
            self.d_w.append(m.DeviceBuffer(host=self.inp_full["w"]))
        self.ncopies = want
        self.t_w = [m.Tensor((self.K, self.N), self.w_dt, d, strides=(1, self.K) if self.packed else None) for d in self.d_w[:want]]
        if hasattr(self, "M"):
            self.set_m(self.M)

    def set_m(self, M):
        m, K, N = self.m, self.K, self.N
        self.M = M
        self.inp = dict(self.inp_full, x=np.ascontiguousarray(self.inp_full["x"][:M]))
        self.kernel = ("wqmm_resx_kernel" if (self.cfg == 3 and M <= 3) else "wqmm_xreg_kernel" if M <= 16 else
                       "wqmm_decode_kernel" if self.cfg == 11 else
                       "wqmm_rows_kernel<256 or 192 rows>" if M > 128 else "wqmm_rows_kernel" if M > 48 else "wqmm_stream_kernel")
        self.t_x = m.Tensor((M, K), self.x_dt, self.d["x"])
        self.t_y = m.Tensor((M, N), self.x_dt, self.d_y)
        rc, ws, ex = m.weight_quant_batch_matmul_get_workspace(self.t_x, self.t_w[0], self.t_sc, self.t_y, offset=self.t_off,
                                                               group_size=self.group)
        m.check(rc, "phase 1")
        m.lib().aclDestroyAclOpExecutor(ex)
        self.ws = m.DeviceBuffer(ws) if ws else None
        self.ws_size = ws
        self.flop = 2 * M * N * K
        wb = K * N * (1 if self.w_dt == m.ACL_INT8 else 0.5)
        sb = 1 if self.scale_dt == m.ACL_FLOAT8_E8M0 else 2
        self.bytes = int(wb + 2 * M * K + 2 * M * N + sb * self.G * N * (2 if self.off else 1))
        self.variant = "cold" if self.ncopies > 1 else "warm"
        self.config = {"workload": self.name, "M": M, "K": K, "N": N, "group": self.group,
                       "cache": "cold (weight copies rotated, %d x %.0f MB)" % (self.ncopies, self.inp_full["w"].nbytes / 1e6)
                                if self.ncopies > 1 else "warm (one weight copy, resident in the 256 MB last-level cache between steps)",
                       "weight_copies_rotated": self.ncopies,
                       "weight_layout": "K-contiguous (pre-packed offline)" if self.packed else "N-contiguous (re-laid out per call)"}

    def step(self, stream):
        m = self.m
        w = self.t_w[self.i % self.ncopies]
        self.i += 1
        rc, ws, ex = m.weight_quant_batch_matmul_get_workspace(self.t_x, w, self.t_sc, self.t_y, offset=self.t_off,
                                                               group_size=self.group)
        m.check(rc, "phase 1")
        m.check(m.lib().aclnnWeightQuantBatchMatmulV2(self.ws.ptr if self.ws else None, self.ws_size, ex, stream.ptr), "phase 2")

    def cpu_baseline(self):
        # bounded sample: at most the first 16 rows of x against the whole weight (the weight dequantisation dominates)
        rows = min(self.M, 16)
        inp = dict(self.inp, x=np.ascontiguousarray(self.inp["x"][:rows]))
        t0 = time.perf_counter()
        cases.oracle_wq(self.m, inp, rows, self.K, self.N)
        t = time.perf_counter() - t0
        nbytes = self.bytes - (self.M - rows) * 2 * (self.K + self.N)
        what = "the whole workload once" if rows == self.M else f"the first {rows} of {self.M} rows of x against the whole weight"
        return {"value": nbytes / t / 1e9, "unit": "GB/s", "cores": _cores(), "kind": "port",
                "sample": f"{what} (oracle/liboracle.so, OpenMP), {t:.2f} s"}


class ConfigKG(Workload):
    """Not a BASELINE config: aclnnQuantMatmulV5 in the int4 x int4 mode with per-group (256 K) scales and offsets of x2
    ("K-G" of quant_batch_matmul_v4), 4096 x 4096 x 4096, bf16 output.  Every call rewrites the operands as e4m3 bytes
    in the workspace (one kernel before the matrix kernel; with --weight-cache the x2 half of it only on the first call):
    that is inside the timed step."""
    peak_key, dtype = "fp8", "fp8 e4m3 (int4 operands, exact)"
    kernel = "kg_gemm_kernel (+ kg_prepare_kernel)"

    def __init__(self, m, args, M=4096, K=4096, N=4096):
        self.m, self.M, self.K, self.N = m, M, K, N
        self.inp = cases.make_i4_asym_inputs(m, M, K, N, 0)
        self.d = {k: m.DeviceBuffer(host=v) for k, v in self.inp.items()}
        self.d_out = m.DeviceBuffer(M * N * 2)
        G = K // 256
        self.t = dict(x1=m.Tensor((M, K), m.ACL_INT4, self.d["x1"]), x2=m.Tensor((N, K), m.ACL_INT4, self.d["x2"]),
                      s1=m.Tensor((M, 1), m.ACL_FLOAT, self.d["s1"]), s2=m.Tensor((G, N), m.ACL_FLOAT, self.d["s2"]),
                      off=m.Tensor((G, N), m.ACL_FLOAT16, self.d["off"]), out=m.Tensor((M, N), m.ACL_BF16, self.d_out))
        rc, ws, ex = self._phase1()
        m.lib().aclDestroyAclOpExecutor(ex)
        self.ws = m.DeviceBuffer(ws) if ws else None
        self.ws_size = ws
        self.flop = 2 * M * N * K
        self.bytes = M * K // 2 + K * N // 2 + 4 * M + 6 * G * N + 2 * M * N
        self.config = {"workload": "aclnnQuantMatmulV5 int4 x int4 K-G (groups of 256, fp32 scale + fp16 offset per group and column), bf16 out",
                       "M": M, "K": K, "N": N, "x2_layout": "K-contiguous (transposeX2, as the mode requires)"}

    def _phase1(self):
        m, t = self.m, self.t
        rc, ws, ex = m.quant_matmul_v5_get_workspace(t["x1"], t["x2"], t["s1"], t["s2"], t["out"], x2_offset=t["off"], transpose_x2=True,
                                                     group_size=256)
        m.check(rc, "phase 1")
        return rc, ws, ex

    def step(self, stream):
        m = self.m
        rc, ws, ex = self._phase1()
        m.check(m.lib().aclnnQuantMatmulV5(self.ws.ptr if self.ws else None, self.ws_size, ex, stream.ptr), "phase 2")

    def cpu_baseline(self):
        rows = 64
        inp = self.inp
        x1 = np.ascontiguousarray(inp["x1"][:rows]); s1 = np.ascontiguousarray(inp["s1"][:rows])
        t0 = time.perf_counter()
        orc.qmm_i4_asym(x1, inp["x2"], rows, self.K, self.N, True, s1, inp["s2"], inp["off"], self.m.ACL_BF16)
        t = time.perf_counter() - t0
        return {"value": 2.0 * rows * self.K * self.N / t / 1e12, "unit": "TFLOP/s", "cores": _cores(), "kind": "port",
                "sample": f"first {rows} of {self.M} rows of x1 against the full x2 (oracle/liboracle.so, OpenMP), {t:.2f} s"}


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
    if config in (1, 3, 11):
        return ConfigWQ(m, args, config)
    if config == 10:
        return ConfigKG(m, args)
    shape = getattr(args, "shape", None)
    if shape and config in (2, 4, 5):   # the same operator at another shape (not the BASELINE workload)
        M, K, N = (int(v) for v in shape.split(","))
        wl = Config2(m, args, M, K, N) if config == 2 else Config4(m, args, M, K, N) if config == 4 else Config5(m, args, 1, M, K, N)
        wl.kernel = "the selector's choice for this shape (tile kernel, with a K split where the tiles are few)"
        wl.config = dict(wl.config, workload=wl.config["workload"].split(":")[-1].strip() + f" at {M} x {K} x {N} (not a BASELINE shape)")
        return wl
    if config == 2:
        return Config2(m, args)
    if config == 4:
        return Config4(m, args)
    if config == 12:
        return Config4Rows(m, args)
    if config == 13:
        return ConfigA8W4Rows(m, args)
    if config == 14:
        return ConfigPerTileRows(m, args)
    if config == 15:
        return ConfigMxfp8Rows(m, args)
    if config == 5:
        return Config5(m, args)
    raise SystemExit(f"bench.py: config {config} is not wired up yet")
