"""Phase-1 status table of aclnnQuantMatmulV5.

The cases are the reference's own API unit-test table
(matmul/quant_batch_matmul_v4/tests/ut/op_host/test_aclnn_quant_matmul_v5_api.csv, committed unchanged as
tests/golden/aclnn_quant_matmul_v5_api_cases.csv) restricted to its newest SoC generation; tensors are built
the way that harness builds them (test_aclnn_quant_matmul_v5_api.cpp:187-273): null data pointers, strides
only for x1/x2, empty shape column = argument absent.  No GPU is needed: phase 1 never touches data.
"""
import csv
import os
import threading

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CSV = os.path.join(HERE, "golden", "aclnn_quant_matmul_v5_api_cases.csv")


def _rows():
    with open(CSV, newline="") as f:
        return [r for r in csv.DictReader(f) if r["socVersion"] == "Ascend950"]


def _ints(s):
    return [int(v) for v in s.split()] if s.strip() else None


def run_case(m, r):
    def mk(shape_col, type_col, stride_col=None, fmt_col=None, storage_col=None):
        shape = _ints(r[shape_col])
        if shape is None:
            return None
        strides = _ints(r[stride_col]) if stride_col else None
        if strides is not None and len(strides) != len(shape):
            strides = None
        storage = _ints(r[storage_col]) if storage_col else None
        fmt = m.FORMAT_BY_NAME[r[fmt_col]] if fmt_col else m.ACL_FORMAT_ND
        return m.Tensor(shape, m.DTYPE_BY_NAME[r[type_col]], None, strides=strides, fmt=fmt, storage_shape=storage)

    x1 = mk("x1Shape", "x1Type", "x1Stride", "x1Format", "x1StorageShape")
    x2 = mk("x2Shape", "x2Type", "x2Stride", "x2Format", "x2StorageShape")
    rc, ws, ex = m.quant_matmul_v5_get_workspace(
        x1, x2, mk("pertokenScaleShape", "pertokenType"), mk("scaleShape", "scaleType"), mk("outShape", "outType"),
        y_scale=mk("yScaleShape", "yScaleType"), x1_offset=mk("x1OffsetShape", "x1OffsetType"),
        x2_offset=mk("offsetShape", "offsetType"), y_offset=mk("yOffsetShape", "yOffsetType"),
        bias=mk("biasShape", "biasType"), transpose_x1=r["transposeX1"] == "true", transpose_x2=r["transposeX2"] == "true",
        group_size=int(r["groupSize"]))
    if ex:
        m.lib().aclDestroyAclOpExecutor(ex)
    return rc


ROWS = _rows()
# Modes that validate like the reference but have no kernel here yet: phase 1 reports them with an
# inner "no kernel" status instead of SUCCESS (fp8 x fp4, int4 K-G, 64-bit packed scales, int8 requant).
NO_KERNEL = 561002


@pytest.mark.parametrize("row", ROWS, ids=[r["caseName"] for r in ROWS])
def test_status_matches_reference_table(opsnn, row):
    rc = run_case(opsnn, row)
    want = opsnn.STATUS_BY_NAME[row["expectRet"]]
    if want == 0 and rc == NO_KERNEL:
        pytest.xfail("validated, but this quant mode has no gfx950 kernel yet: " + opsnn.err_msg())
    assert rc == want, f"{row['caseName']}: got {rc} ({opsnn.err_msg()}), reference expects {row['expectRet']}"
    if rc != 0:
        assert opsnn.err_msg(), "a failing status must leave a message for aclGetRecentErrMsg"


def test_table_has_the_expected_size():
    assert len(ROWS) == 84
    counts = {}
    for r in ROWS:
        counts[r["expectRet"]] = counts.get(r["expectRet"], 0) + 1
    assert counts == {"ACLNN_SUCCESS": 24, "ACLNN_ERR_PARAM_INVALID": 56, "ACLNN_ERR_PARAM_NULLPTR": 4}


def test_phase1_is_thread_safe(opsnn):
    # the reference runs its table from three threads (test_aclnn_quant_matmul_v5_api.cpp:302-325)
    errors = []

    def worker():
        for r in ROWS:
            rc = run_case(opsnn, r)
            want = opsnn.STATUS_BY_NAME[r["expectRet"]]
            if rc != want and not (want == 0 and rc == NO_KERNEL):
                errors.append((r["caseName"], rc))

    ts = [threading.Thread(target=worker) for _ in range(3)]
    [t.start() for t in ts]
    [t.join() for t in ts]
    assert not errors, errors[:5]


def test_executor_is_single_use_and_destroy_after_run_is_harmless(opsnn):
    """An empty output (M == 0) validates and yields an executor with nothing to launch, so both phases run without a
    GPU.  Phase 2 consumes the executor (two_phase_api.md:17-24): a second phase 2 with the same handle is refused with
    161002, and aclDestroyAclOpExecutor on a consumed or already destroyed handle does nothing -- the library recognises
    such handles by address, without reading the freed object."""
    m = opsnn
    K, N = 64, 32
    x1 = m.Tensor((0, K), m.ACL_INT8, None)
    x2 = m.Tensor((K, N), m.ACL_INT8, None)
    s2 = m.Tensor((N,), m.ACL_FLOAT, None)
    out = m.Tensor((0, N), m.ACL_BF16, None)
    rc, ws, ex = m.quant_matmul_v5_get_workspace(x1, x2, None, s2, out)
    assert rc == 0 and ex, m.err_msg()
    assert m.lib().aclnnQuantMatmulV5(None, 0, ex, None) == 0
    # garbage churn on the heap between the calls: the freed block is likely to be handed out again
    junk = [m.quant_matmul_v5_get_workspace(x1, x2, None, s2, out) for _ in range(8)]
    assert m.lib().aclnnQuantMatmulV5(None, 0, ex, None) == m.STATUS_BY_NAME["ACLNN_ERR_PARAM_INVALID"] or any(j[2] == ex for j in junk)
    for rc_j, _, ex_j in junk:
        assert rc_j == 0
        assert m.lib().aclDestroyAclOpExecutor(ex_j) == 0
        assert m.lib().aclDestroyAclOpExecutor(ex_j) == 0   # twice: the second call finds nothing to do
