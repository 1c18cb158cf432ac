#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 1..5] [--m M] [--no-cpu] [--cold] [--calib-copy]

A step is one pass of the operator (both aclnn phases) over one batch of synthetic, seeded input that is
already resident in HBM.  The default workload is BASELINE config 2 (aclnnQuantMatmulV5, int8 per-token x
per-channel, M=2048 K=4096 N=11008, bf16 bias and output); --config selects the other four.
One JSON line is printed: whole-job throughput, the roofline record of the dominant kernel (algorithmic
work / HIP-event time measured here on the launch stream) and a CPU baseline (the C oracle on a bounded
sample of the same workload, on this host's cores).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "ops-nn_amd"))
sys.path.insert(0, os.path.join(ROOT, "tests"))

import numpy as np  # noqa: E402

PEAK = {"int8": 5000.0, "fp8": 5000.0, "fp4": 10100.0, "f16": 2500.0, "bf16": 2500.0}  # dense TFLOP/s, MI355X
PEAK_HBM = 8000.0  # GB/s


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", type=int, default=2,
                    help="1-5: the BASELINE configs; 6-9: the pre-pack / quantizer operators that prepare their tensors")
    ap.add_argument("--m", type=int, default=None, help="M for config 3 (1, 16, 64 or 256)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--int8-range", type=int, default=None,
                    help="config 2: operands uniform in [-R, R] (default: the full int8 range, the most power-hungry data)")
    ap.add_argument("--cold", action="store_true", help="rotate through weight copies larger than the 256 MB cache")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run a byte transpose of an 8192x8192 matrix (64 MiB read, 64 MiB written) three times "
                         "before the timed loop: the known-size kernel that hardware traffic counters are scaled by")
    ap.add_argument("--layout", default="packed", choices=["packed", "nd"],
                    help="packed: right operand K-contiguous (offline pre-pack, [N,K] storage); nd: [K,N] storage, "
                         "re-laid out inside every call")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU; --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import opsnn as m
    import bench_cases

    if not m.gpu_available():
        print("bench.py: no HIP device visible", file=sys.stderr)
        sys.exit(3)
    m.check(m.lib().aclInit(None), "aclInit")
    m.check(m.lib().aclrtSetDevice(0), "aclrtSetDevice")
    wl = bench_cases.make_workload(m, args.config, args)
    stream = m.Stream()

    if args.calib_copy:
        src, dst = m.DeviceBuffer(8192 * 8192), m.DeviceBuffer(8192 * 8192)
        src.fill(1)
        for _ in range(3):
            m.check(m.lib().opsnnTranspose8(src.ptr, dst.ptr, 8192, 8192, 1, stream.ptr), "opsnnTranspose8")
        stream.sync()
    for _ in range(args.warmup):
        wl.step(stream)
    stream.sync()
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    ev0, ev1 = m.Event(), m.Event()
    t0 = time.perf_counter()
    ev0.record(stream)
    for _ in range(args.steps):
        wl.step(stream)
    ev1.record(stream)
    stream.sync()
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    t1 = time.perf_counter()
    wall_ms = (t1 - t0) * 1e3 / args.steps
    dev_ms = ev0.elapsed_ms(ev1) / args.steps

    tflops = wl.flop / (wall_ms * 1e-3) / 1e12
    gbps = wl.bytes / (wall_ms * 1e-3) / 1e9
    if wl.bound == "mfma":
        value, unit = tflops, "TFLOP/s"
        roof = {"bound": "mfma", "achieved": wl.flop / (dev_ms * 1e-3) / 1e12, "peak": PEAK[wl.peak_key], "unit": "TFLOP/s"}
    else:
        value, unit = gbps, "GB/s"
        roof = {"bound": "hbm", "achieved": wl.bytes / (dev_ms * 1e-3) / 1e9, "peak": PEAK_HBM, "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    key = (args.config, (args.m or 16) if args.config == 3 else None)
    roof["traffic"] = bench_cases.MEASURED_TRAFFIC.get(key) if args.layout == "packed" and not args.cold else None
    roof["kernel"] = wl.kernel
    roof["kernel_ms"] = dev_ms

    rec = {
        "metric": wl.metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": wl.dtype,
        "data": "synthetic", "config": wl.config, "roofline": roof,
        "tflops": tflops, "gbps": gbps, "device": m.device_info(),
    }
    if not args.no_cpu:
        rec["cpu_baseline"] = wl.cpu_baseline()
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
