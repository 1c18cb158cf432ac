"""opsnnQmmInt8Static (the entry point that allocates nothing) against opsnnQmmInt8 with a caller-allocated workspace.

x2 is stored [K, N] with N contiguous, so both entry points first re-lay it out K-contiguous: opsnnQmmInt8 into the
workspace the caller passes, opsnnQmmInt8Static into the array inside the library's device image.  Outputs must be
bit-identical (int8 products are exact and both run the same kernels), on two calls in a row, the second with a
smaller input that leaves most of the array holding the first call's bytes.
"""
import ctypes as C

import numpy as np
import pytest

import cases
from test_gpu_k_tail import _splitk_bytes

pytestmark = pytest.mark.gpu


def _run_pair(m, M, K, N, seed):
    inp = cases.make_qmm_int8_inputs(m, M, K, N, seed, m.ACL_BF16, False)
    d = {k: m.DeviceBuffer(host=v) for k, v in inp.items() if isinstance(v, np.ndarray)}
    out_ws, out_st = m.DeviceBuffer(M * N * 2), m.DeviceBuffer(M * N * 2)
    out_ws.fill(0xFF)
    out_st.fill(0xEE)
    a = cases.qmm_args_int8(m, d, M, K, N, 1, False, out_ws.ptr, m.ACL_BF16, m.ACL_FLOAT, N, m.ACL_BF16)
    need = m.lib().opsnnQmmWorkspace(C.byref(a), 0)
    # the fast path applies: the re-laid-out operand is the scratch buffer in question; opsnnQmmInt8 also gets room for the
    # integer partial sums of a K split when the call has few tiles (the no-alloc entry point runs unsplit: same bits)
    assert need == N * K + _splitk_bytes(M, K, N, 128, 128, tile_us=0.55, bytes_per_us=2.4e6), need
    ws = m.DeviceBuffer(need)
    a.workspace = ws.ptr
    assert m.lib().opsnnQmmInt8(C.byref(a), None) == 0
    b = cases.qmm_args_int8(m, d, M, K, N, 1, False, out_st.ptr, m.ACL_BF16, m.ACL_FLOAT, N, m.ACL_BF16)
    rc = m.lib().opsnnQmmInt8Static(C.byref(b), None)
    assert rc == 0, (rc, m.err_msg())
    m.check(m.lib().aclrtSynchronizeDevice(), "sync")
    got_ws, got_st = out_ws.to_host(np.uint16, (M, N)), out_st.to_host(np.uint16, (M, N))
    want, _ = cases.oracle_qmm_int8(m, inp, M, K, N, False, m.ACL_BF16)
    assert np.array_equal(got_ws, want[0]), "opsnnQmmInt8 with a workspace differs from the oracle"
    assert np.array_equal(got_st, got_ws), f"{int((got_st != got_ws).sum())} of {got_st.size} outputs differ"


def test_static_scratch_entry_point_matches_workspace_entry_point_twice(gpu):
    m = gpu
    print("case no-alloc int8: 512x1024x768, then 200x256x328", flush=True)
    _run_pair(m, 512, 1024, 768, 1)
    _run_pair(m, 200, 256, 328, 2)   # smaller: the scratch array still holds most of the first call's operand


def test_static_scratch_entry_point_rejects_oversize(gpu):
    m = gpu
    M, K, N = 64, 8192, 8200   # N * K = 67,174,400 bytes > 64 MiB; nothing is launched, no buffer is touched
    a = m.OpsnnQmmArgs()
    a.M, a.N, a.K, a.batch = M, N, K, 1
    dummy = m.DeviceBuffer(256)
    a.x1 = m.OpsnnMat(dummy.ptr, K, 1, 0)
    a.x2 = m.OpsnnMat(dummy.ptr, N, 1, 0)
    a.x1_dtype = a.x2_dtype = m.ACL_INT8
    a.out, a.out_dtype = dummy.ptr, m.ACL_BF16
    a.x2_scale, a.x2_scale_dtype, a.x2_scale_len = dummy.ptr, m.ACL_FLOAT, N
    rc = m.lib().opsnnQmmInt8Static(C.byref(a), None)
    assert rc == -6, rc
    assert "scratch" in m.err_msg()
