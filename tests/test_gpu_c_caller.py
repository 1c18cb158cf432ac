"""The C++ callers under ops-nn_amd/examples, built against the public headers only, run end to end on the GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "ops-nn_amd", "lib", "examples", "quant_matmul_v5_int8")


@pytest.mark.gpu
def test_cpp_caller_runs_and_verifies():
    assert os.path.exists(BIN), "example not built: run make -C ops-nn_amd/csrc"
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "worst relative error" in r.stdout


@pytest.mark.gpu
def test_cpp_chain_of_prepack_quantizer_and_matmuls():
    """int32 carriers -> ConvertWeightToINT4Pack -> WeightQuantBatchMatmulV2, and fp16 -> DynamicQuant -> QuantMatmulV5."""
    exe = os.path.join(ROOT, "ops-nn_amd", "lib", "examples", "w4_pack_and_dynamic_quant_chain")
    assert os.path.exists(exe), "example not built: run make -C ops-nn_amd/csrc"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ConvertWeightToINT4Pack" in r.stdout and "DynamicQuant" in r.stdout


@pytest.mark.gpu
def test_cpp_decode_call_cost_is_reported():
    """Config 1's shape from a C++ serving loop: both phases per call, 500 calls back to back; the example prints the host
    time per call and the end-to-end time per call.  The host side must stay below the kernel time it feeds (about 10 us)."""
    exe = os.path.join(ROOT, "ops-nn_amd", "lib", "examples", "decode_call_cost")
    assert os.path.exists(exe), "example not built: run make -C ops-nn_amd/csrc"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    line = [l for l in r.stdout.splitlines() if l.startswith("decode call cost")][0]
    host_us = float(line.split("host ")[1].split(" us")[0])
    assert host_us < 10.0, line
