#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 1..15] [--shape M,K,N] [--m M] [--cold] [--fp8-fast] [--no-cpu] [--calib-copy] [--layout packed|nd] [--weight-cache MB]

A step is one pass of the operator (both aclnn phases) over one batch of synthetic, seeded input that is already
resident in HBM.  One JSON line is printed.

Without --config the headline record is BASELINE config 2 (aclnnQuantMatmulV5, int8 per-token x per-channel, M=2048
K=4096 N=11008, bf16 bias and output), timed with exactly --steps steps after --warmup ("ms_per_step_sustained" and
"roofline.frac_sustained" repeat it over at least 50 steps, where the power-limited clock has settled), and "configs" holds one record
for every BASELINE config -- 1 (warm and cold), 2, 3 with M = 1, 16, 64, 256 (each warm and cold), 4 (the default exact
arithmetic and the opt-in 8-bit matrix instruction), 5, and configs 2 and 3 (16 rows) once more with the right operand in
the literal [K, N] storage and the library's weight cache on -- each with its own roofline record (algorithmic work / HIP-event
time measured here on the launch stream) and CPU baseline (the C oracle on a bounded sample of the same workload, on this
host's cores).  "cold" rotates through weight copies larger than the 256 MB last-level cache, so the weight really comes
from HBM; "warm" re-reads one copy.  With --config N only that workload runs (what the rocprofv3 commands in profiles/ use).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "ops-nn_amd"))
sys.path.insert(0, os.path.join(ROOT, "tests"))

import numpy as np  # noqa: E402,F401

PEAK = {"int8": 5000.0, "fp8": 5000.0, "fp4": 10100.0, "f16": 2500.0, "bf16": 2500.0}  # dense TFLOP/s, MI355X
PEAK_HBM = 8000.0  # GB/s


def run_workload(m, bench_cases, wl, stream, steps, warmup, with_cpu):
    """warmup untimed steps, then exactly `steps` steps between two events on the launch stream; one record."""
    wl.begin()
    try:
        for _ in range(warmup):
            wl.step(stream)
        stream.sync()
        m.check(m.lib().aclrtSynchronizeDevice(), "sync")
        ev0, ev1 = m.Event(), m.Event()
        t0 = time.perf_counter()
        ev0.record(stream)
        for _ in range(steps):
            wl.step(stream)
        ev1.record(stream)
        stream.sync()
        m.check(m.lib().aclrtSynchronizeDevice(), "sync")
        t1 = time.perf_counter()
    finally:
        wl.end()
    wall_ms = (t1 - t0) * 1e3 / steps
    dev_ms = ev0.elapsed_ms(ev1) / steps
    tflops = wl.flop / (wall_ms * 1e-3) / 1e12
    gbps = wl.bytes / (wall_ms * 1e-3) / 1e9
    if wl.bound == "mfma":
        value, unit = tflops, "TFLOP/s"
        roof = {"bound": "mfma", "achieved": wl.flop / (dev_ms * 1e-3) / 1e12, "peak": PEAK[wl.peak_key], "unit": "TFLOP/s"}
    else:
        value, unit = gbps, "GB/s"
        roof = {"bound": "hbm", "achieved": wl.bytes / (dev_ms * 1e-3) / 1e9, "peak": PEAK_HBM, "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    if wl.bound == "mfma" and wl.instr_peak_key and wl.instr_peak_key != wl.peak_key:
        # the operands' dtype sets `peak`; the instruction actually issued has a lower one
        roof["instruction_peak"] = PEAK[wl.instr_peak_key]
        roof["frac_of_instruction_peak"] = roof["achieved"] / PEAK[wl.instr_peak_key]
    if wl.bound == "hbm" and wl.flop:
        roof["tflops"] = wl.flop / (dev_ms * 1e-3) / 1e12
    key = (wl.key[0], wl.key[1], wl.variant)
    traffic = bench_cases.PROFILED_TRAFFIC.get(key)
    if traffic and traffic[0] >= 0.95 * wl.bytes:   # (a calibrated counter reading can fall a percent short of the truth)
        roof["traffic"] = max(traffic[0], float(wl.bytes))
        roof["traffic_source"] = traffic[1] + " (hardware counters of an earlier profiling run of this workload; not measured by this run)"
    else:
        roof["traffic"] = None
    roof["algorithmic_bytes"] = wl.bytes
    roof["kernel"] = wl.kernel
    roof["kernel_ms"] = dev_ms
    rec = {"metric": wl.metric, "value": value, "unit": unit, "steps": steps, "warmup": warmup, "ms_per_step": wall_ms,
           "dtype": wl.dtype, "config": wl.config, "roofline": roof, "tflops": tflops, "gbps": gbps}
    if with_cpu:
        rec["cpu_baseline"] = wl.cpu_baseline()
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", type=int, default=0,
                    help="0 (default): every BASELINE config, headline config 2; 1-5: that BASELINE config only; 6-9: the "
                         "pre-pack / quantizer operators that prepare their tensors; 10: the int4 x int4 K-G mode at 4096^3; "
                         "11: config 3's shape with mxfp4 weights; 12: config 4's operator with the --m rows of a decode step; "
                         "13 / 14 / 15: the fp8 x fp4 MX mode / the int8 per-tile mode / MXFP8 at config 3's K and N with the --m rows of a decode step")
    ap.add_argument("--m", type=int, default=None, help="M for config 3 (1, 16, 64 or 256) and configs 11 to 15 (default 16)")
    ap.add_argument("--shape", default=None, metavar="M,K,N",
                    help="configs 2, 4 and 5 (one batch) at another shape, e.g. --config 4 --shape 512,7168,2048: the mid-size "
                         "calls whose few tiles split K (not a BASELINE workload; the record says so)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--int8-range", type=int, default=None,
                    help="config 2: operands uniform in [-R, R] (default: the full int8 range, the most power-hungry data)")
    ap.add_argument("--cold", action="store_true", help="configs 1 and 3: rotate through weight copies larger than the 256 MB cache")
    ap.add_argument("--fp8-fast", action="store_true", help="config 4: the 8-bit matrix instruction instead of exact fp16 products")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run, three times each before the timed loop, a byte transpose of an 8192x8192 matrix (64 MiB read, "
                         "64 MiB written) and the 4-bit pack of 16 Mi carriers (64 MiB read in 16-byte pieces per lane, 8 MiB "
                         "written): the known-size kernels that hardware traffic counters are scaled by")
    ap.add_argument("--weight-cache", type=int, default=0, metavar="MB",
                    help="switch on the library's cache of re-laid-out right operands with this limit (only matters with --layout nd: "
                         "the first call re-lays the operand out, the timed ones find the copy)")
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
    stream = m.Stream()
    with_cpu = not args.no_cpu
    if args.weight_cache:
        m.lib().opsnnSetWeightCache(args.weight_cache << 20)

    def top(rec):
        rec.update({"n_gpus": 1, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "data": "synthetic",
                    "device": m.device_info()})
        if args.weight_cache:
            rec["config"]["weight_cache_MB"] = args.weight_cache
        return rec

    if args.config:
        wl = bench_cases.make_workload(m, args.config, args)
        wl.key = (args.config, (args.m or 16) if args.config in (3, 11, 12, 13, 14) else None)
        if args.calib_copy:
            src, dst = m.DeviceBuffer(8192 * 8192), m.DeviceBuffer(8192 * 8192)
            src.fill(1)
            for _ in range(3):
                m.check(m.lib().opsnnTranspose8(src.ptr, dst.ptr, 8192, 8192, 1, stream.ptr), "opsnnTranspose8")
            # and a 16-byte-per-lane stream of known size (the access pattern of the decode and quantizer kernels):
            # the 4-bit pack kernel reads 64 MiB of 32-bit carriers and writes 8 MiB
            for _ in range(3):
                m.check(m.lib().opsnnPackB4(src.ptr, 0, dst.ptr, 8192 * 8192 // 4, stream.ptr), "opsnnPackB4")
            stream.sync()
        print(json.dumps(top(run_workload(m, bench_cases, wl, stream, args.steps, args.warmup, with_cpu))))
        return

    # every BASELINE config; the headline (config 2) first, with exactly the requested step counts
    records = []
    wl = bench_cases.make_workload(m, 2, args)
    wl.key = (2, None)
    head = run_workload(m, bench_cases, wl, stream, args.steps, args.warmup, with_cpu)
    # the same workload over a run long enough for the power-limited clock to settle (short bursts run faster):
    # "value", "ms_per_step" and "roofline" above are the requested --steps; the *_sustained fields are this run
    if args.steps >= 50:
        sus = head
    else:
        sus = run_workload(m, bench_cases, wl, stream, 60, 10, False)
    head["ms_per_step_sustained"] = sus["ms_per_step"]
    head["value_sustained"] = sus["value"]
    head["steps_sustained"] = sus["steps"]
    head["roofline"]["frac_sustained"] = sus["roofline"]["frac"]
    head["roofline"]["kernel_ms_sustained"] = sus["roofline"]["kernel_ms"]
    del wl

    def sub(wl, key, steps, warmup):
        wl.key = key
        r = run_workload(m, bench_cases, wl, stream, steps, warmup, with_cpu)
        print(f"bench.py: {r['config']['workload']} {wl.variant or ''} M={r['config'].get('M')}: {r['ms_per_step'] * 1e3:.1f} us/step, "
              f"roofline {r['roofline']['frac']:.3f}", file=sys.stderr, flush=True)
        records.append(r)

    wq = bench_cases.ConfigWQ(m, args, 1)
    for cold in (False, True):
        wq.set_cold(cold)
        sub(wq, (1, None), 50, 10)
    del wq
    records.append({k: v for k, v in head.items()})
    wq = bench_cases.ConfigWQ(m, args, 3, max_m=256)
    for M in (1, 16, 64, 256):
        for cold in (False, True):
            wq.set_cold(cold)
            wq.set_m(M)
            sub(wq, (3, M), 30, 6)
    del wq
    for fast in (False, True):
        args.fp8_fast = fast
        wl = bench_cases.make_workload(m, 4, args)
        sub(wl, (4, None), 10, 3)
        del wl
    wl = bench_cases.make_workload(m, 5, args)
    sub(wl, (5, None), 6, 2)
    del wl
    # the literal [K, N] storage of the reference's callers with the library's weight cache on: the re-layout is paid by the
    # first (warm-up) call, the timed calls find the K-contiguous copy (configs 2 and 3; cold rotation would only measure
    # the cache's eviction, so warm only)
    if args.layout == "packed":
        args.layout = "nd"
        m.lib().opsnnSetWeightCache(1024 << 20)
        wl = bench_cases.make_workload(m, 2, args)
        sub(wl, (2, None), 30, 6)
        records[-1]["config"].update({"weight_cache_MB": 1024, "x2_layout": "N-contiguous, the literal [K, N] storage (re-laid out once: weight cache)"})
        del wl
        wq = bench_cases.ConfigWQ(m, args, 3, max_m=16)
        wq.set_cold(False)
        wq.set_m(16)
        sub(wq, (3, 16), 30, 6)
        records[-1]["config"].update({"weight_cache_MB": 1024, "weight_layout": "N-contiguous, the literal [K, N] storage (re-laid out once: weight cache)"})
        del wq
        m.lib().opsnnSetWeightCache(0)
        args.layout = "packed"
    head["configs"] = records
    print(json.dumps(top(head)))


if __name__ == "__main__":
    main()
