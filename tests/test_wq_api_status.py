"""Phase-1 status table of aclnnWeightQuantBatchMatmulV2/V3, and the exported-symbol check.

The ten cases are the newest-SoC rows of the reference's own API unit test
(matmul/weight_quant_batch_matmul_v2/tests/ut/op_host/op_api/test_aclnn_weight_quant_batch_matmul_v2_api.cpp:2471-2752),
written out as data in tests/golden/aclnn_weight_quant_batch_matmul_v2_api_cases.csv.  Tensors are built the way
that harness builds them (same file, :190-236 and :238-282): null data pointers; CONTIGUOUS = dense strides,
TRANSPOSE_LAST_TWO_DIMS = the last two strides swapped and the storage shape transposed; an optional argument
whose "NotNull" flag is false is passed as a null pointer.  No GPU is needed.
"""
import csv
import ctypes
import os
import re

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSV = os.path.join(HERE, "golden", "aclnn_weight_quant_batch_matmul_v2_api_cases.csv")

with open(CSV, newline="") as f:
    ROWS = list(csv.DictReader(f))


def _tensor(m, shape_s, dtype_s, fmt_s, ctgs):
    shape = [int(v) for v in shape_s.split()]
    dtype, fmt = m.DTYPE_BY_NAME["ACL_" + dtype_s], m.FORMAT_BY_NAME["ACL_FORMAT_" + fmt_s]
    if ctgs == "CONTIGUOUS":
        return m.Tensor(shape, dtype, None, fmt=fmt)
    assert ctgs == "TRANSPOSE_LAST_TWO_DIMS" and len(shape) >= 2
    strides = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        strides[i] = strides[i + 1] * shape[i + 1]
    strides[-1], strides[-2] = strides[-2], strides[-1]
    storage = list(shape)
    storage[-1], storage[-2] = storage[-2], storage[-1]
    return m.Tensor(shape, dtype, None, strides=strides, fmt=fmt, storage_shape=storage)


def run_case(m, r, v3=False):
    x = _tensor(m, r["x"], r["xType"], r["xFormat"], r["ctgsX"])
    w = _tensor(m, r["weight"], r["weightType"], r["weightFormat"], r["ctgsWeight"])
    sc = _tensor(m, r["antiquantScale"], r["scaleType"], r["xFormat"], r["ctgsScale"])
    off = _tensor(m, r["antiquantOffset"], r["offsetType"], r["xFormat"], "CONTIGUOUS") if r["offsetNotNull"] == "true" else None
    qs = _tensor(m, r["quantScale"], r["quantScaleType"], r["xFormat"], "CONTIGUOUS") if r["quantScaleNotNull"] == "true" else None
    qo = _tensor(m, r["quantOffset"], r["quantOffsetType"], r["xFormat"], "CONTIGUOUS") if r["quantOffsetNotNull"] == "true" else None
    bias = _tensor(m, r["bias"], r["biasType"], r["xFormat"], "CONTIGUOUS") if r["biasNotNull"] == "true" else None
    y = _tensor(m, r["y"], r["yType"], r["xFormat"], "CONTIGUOUS")
    rc, ws, ex = m.weight_quant_batch_matmul_get_workspace(x, w, sc, y, offset=off, quant_scale=qs, quant_offset=qo, bias=bias,
                                                           group_size=int(r["groupSize"]), inner_precise=0 if v3 else None)
    if ex:
        m.lib().aclDestroyAclOpExecutor(ex)
    return rc


@pytest.mark.parametrize("v3", [False, True], ids=["V2", "V3"])
@pytest.mark.parametrize("row", ROWS, ids=[r["caseName"] for r in ROWS])
def test_status_matches_reference_table(opsnn, row, v3):
    rc = run_case(opsnn, row, v3)
    want = opsnn.STATUS_BY_NAME[row["expectRet"]]
    assert rc == want, f"{row['caseName']}: got {rc} ({opsnn.err_msg()}), reference expects {row['expectRet']}"
    if rc != 0:
        assert opsnn.err_msg()


def test_table_size():
    assert len(ROWS) == 10
    assert sum(r["expectRet"] == "ACLNN_SUCCESS" for r in ROWS) == 2


def test_v3_inner_precise_must_be_0_or_1(opsnn):
    # aclnn_weight_quant_batch_matmul_v2.cpp:283-291
    r = ROWS[3]
    x = _tensor(opsnn, r["x"], r["xType"], "ND", "CONTIGUOUS")
    w = _tensor(opsnn, r["weight"], r["weightType"], "ND", "CONTIGUOUS")
    sc = _tensor(opsnn, r["antiquantScale"], r["scaleType"], "ND", "CONTIGUOUS")
    y = _tensor(opsnn, r["y"], r["yType"], "ND", "CONTIGUOUS")
    for ip, want in ((0, 0), (1, 0), (2, 161002), (-1, 161002)):
        rc, ws, ex = opsnn.weight_quant_batch_matmul_get_workspace(x, w, sc, y, group_size=32, inner_precise=ip)
        if ex:
            opsnn.lib().aclDestroyAclOpExecutor(ex)
        assert rc == want, (ip, rc, opsnn.err_msg())


def _declared_symbols():
    """Every function the public headers declare (ACLNN_API / ACL_FUNC_VISIBILITY / OPSNN_API)."""
    names = set()
    inc = os.path.join(ROOT, "include")
    for d, _, files in os.walk(inc):
        for fn in files:
            if fn.endswith(".h"):
                text = open(os.path.join(d, fn)).read()
                text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
                text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
                for mt in re.finditer(r"\b(?:ACLNN_API|ACL_FUNC_VISIBILITY|OPSNN_API)\b[^;{]*?\b(\w+)\s*\(", text):
                    names.add(mt.group(1))
    return names


def test_library_exports_every_declared_symbol(opsnn):
    lib = ctypes.CDLL(opsnn.LIB_PATH)
    declared = _declared_symbols()
    assert {"aclnnQuantMatmulV5GetWorkspaceSize", "aclnnQuantMatmulV5", "aclnnWeightQuantBatchMatmulV2GetWorkspaceSize",
            "aclnnWeightQuantBatchMatmulV2", "aclnnWeightQuantBatchMatmulV3GetWorkspaceSize", "aclnnWeightQuantBatchMatmulV3",
            "aclnnConvertWeightToINT4PackGetWorkspaceSize", "aclnnConvertWeightToINT4Pack", "opsnnPackB4",
            "aclnnDynamicQuantGetWorkspaceSize", "aclnnDynamicQuant", "aclnnDynamicQuantV2GetWorkspaceSize", "aclnnDynamicQuantV2",
            "aclnnDynamicQuantV3GetWorkspaceSize", "aclnnDynamicQuantV3", "aclnnDynamicQuantV4GetWorkspaceSize", "aclnnDynamicQuantV4",
            "opsnnDynamicQuant", "aclnnDynamicBlockQuantGetWorkspaceSize", "aclnnDynamicBlockQuant",
            "aclnnDynamicBlockQuantV2GetWorkspaceSize", "aclnnDynamicBlockQuantV2", "opsnnDynamicBlockQuant",
            "aclnnDynamicMxQuantGetWorkspaceSize", "aclnnDynamicMxQuant", "opsnnDynamicMxQuant",
            "aclnnDynamicMxQuantV2GetWorkspaceSize", "aclnnDynamicMxQuantV2", "aclnnDynamicMxQuantV3GetWorkspaceSize", "aclnnDynamicMxQuantV3",
            "aclnnTransQuantParamV2GetWorkspaceSize", "aclnnTransQuantParamV2", "aclnnTransQuantParamV3GetWorkspaceSize",
            "aclnnTransQuantParamV3", "opsnnTransQuantParam",
            "opsnnQmmInt8", "opsnnWqmm", "aclCreateTensor"} <= declared
    missing = [n for n in sorted(declared) if not hasattr(lib, n)]
    assert not missing, f"declared in include/ but not exported by the library: {missing}"
    # and the binding's own list is covered by the headers
    assert set(opsnn.EXPORTED_SYMBOLS) <= declared
