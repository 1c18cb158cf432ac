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
