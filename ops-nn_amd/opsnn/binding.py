"""Thin ctypes layer over include/acl/acl.h, include/aclnnop/*.h and include/opsnn_kernels.h."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "..", "lib", "libopsnn_amd.so")

# aclDataType values (include/acl/acl.h)
ACL_FLOAT, ACL_FLOAT16, ACL_INT8, ACL_INT32, ACL_UINT8 = 0, 1, 2, 3, 4
ACL_INT64, ACL_UINT64, ACL_BF16, ACL_INT4 = 9, 10, 27, 29
ACL_HIFLOAT8, ACL_FLOAT8_E5M2, ACL_FLOAT8_E4M3FN, ACL_FLOAT8_E8M0 = 34, 35, 36, 37
ACL_FLOAT4_E2M1, ACL_FLOAT4_E1M2 = 40, 41
ACL_FORMAT_ND, ACL_FORMAT_FRACTAL_NZ = 2, 29
DTYPE_BY_NAME = {
    "ACL_FLOAT": 0, "ACL_FLOAT16": 1, "ACL_INT8": 2, "ACL_INT32": 3, "ACL_UINT8": 4, "ACL_INT16": 6,
    "ACL_UINT16": 7, "ACL_UINT32": 8, "ACL_INT64": 9, "ACL_UINT64": 10, "ACL_DOUBLE": 11, "ACL_BOOL": 12,
    "ACL_BF16": 27, "ACL_INT4": 29, "ACL_HIFLOAT8": 34, "ACL_FLOAT8_E5M2": 35, "ACL_FLOAT8_E4M3FN": 36,
    "ACL_FLOAT8_E8M0": 37, "ACL_FLOAT4_E2M1": 40, "ACL_FLOAT4_E1M2": 41,
}
FORMAT_BY_NAME = {"ACL_FORMAT_ND": 2, "ACL_FORMAT_FRACTAL_NZ": 29, "ACL_FORMAT_NCHW": 0, "ACL_FORMAT_NHWC": 1}
ACLNN_SUCCESS, ACLNN_ERR_PARAM_NULLPTR, ACLNN_ERR_PARAM_INVALID, ACLNN_ERR_RUNTIME_ERROR = 0, 161001, 161002, 361001
STATUS_BY_NAME = {"ACLNN_SUCCESS": 0, "ACLNN_ERR_PARAM_NULLPTR": 161001, "ACLNN_ERR_PARAM_INVALID": 161002,
                  "ACLNN_ERR_RUNTIME_ERROR": 361001}
H2D, D2H, D2D = 1, 2, 3
VARIANT_AUTO, VARIANT_PLAIN = 0, 1

DTYPE_BITS = {0: 32, 1: 16, 2: 8, 3: 32, 4: 8, 9: 64, 10: 64, 27: 16, 29: 4, 34: 8, 35: 8, 36: 8, 37: 8, 40: 4, 41: 4}


class OpsnnMat(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("row_stride", C.c_int64), ("col_stride", C.c_int64), ("batch_stride", C.c_int64)]


class OpsnnQmmArgs(C.Structure):
    _fields_ = [
        ("M", C.c_int64), ("N", C.c_int64), ("K", C.c_int64), ("batch", C.c_int64),
        ("x1", OpsnnMat), ("x2", OpsnnMat), ("x1_dtype", C.c_int), ("x2_dtype", C.c_int),
        ("out", C.c_void_p), ("out_dtype", C.c_int),
        ("x1_scale", C.c_void_p), ("x2_scale", C.c_void_p), ("x2_scale_dtype", C.c_int), ("x2_scale_len", C.c_int64),
        ("bias", C.c_void_p), ("bias_dtype", C.c_int), ("bias_batch_stride", C.c_int64),
        ("gsM", C.c_int64), ("gsN", C.c_int64), ("gsK", C.c_int64),
        ("x1_scale_mat", OpsnnMat), ("x2_scale_mat", OpsnnMat),
        ("workspace", C.c_void_p), ("force_variant", C.c_int),
        ("x1_scale_len", C.c_int64), ("x2_offset", C.c_void_p), ("x2_offset_len", C.c_int64),
        ("y_scale", C.c_void_p), ("y_scale_len", C.c_int64), ("x2_offset_mat", OpsnnMat), ("x2_scale_trunc", C.c_int),
    ]


class OpsnnWqmmArgs(C.Structure):
    _fields_ = [
        ("M", C.c_int64), ("N", C.c_int64), ("K", C.c_int64),
        ("x", C.c_void_p), ("x_dtype", C.c_int),
        ("w", OpsnnMat), ("w_dtype", C.c_int),
        ("scale", OpsnnMat), ("scale_dtype", C.c_int), ("scale_n", C.c_int64),
        ("offset", C.c_void_p), ("group", C.c_int64),
        ("bias", C.c_void_p), ("bias_dtype", C.c_int),
        ("y", C.c_void_p), ("workspace", C.c_void_p), ("force_variant", C.c_int),
    ]


class OpsnnDynQuantArgs(C.Structure):
    _fields_ = [
        ("x", C.c_void_p), ("x_dtype", C.c_int),
        ("smooth", C.c_void_p),
        ("y", C.c_void_p), ("y_dtype", C.c_int),
        ("scale", C.c_void_p), ("offset", C.c_void_p),
        ("rows", C.c_int64), ("cols", C.c_int64),
        ("force_variant", C.c_int),
        ("group_index", C.c_void_p), ("group_index_dtype", C.c_int),
        ("groups", C.c_int64),
        ("quant_mode", C.c_int), ("chan_rows", C.c_int64),
    ]


class OpsnnBlockQuantArgs(C.Structure):
    _fields_ = [
        ("x", C.c_void_p), ("x_dtype", C.c_int),
        ("y", C.c_void_p), ("y_dtype", C.c_int),
        ("scale", C.c_void_p),
        ("batch", C.c_int64), ("rows", C.c_int64), ("cols", C.c_int64),
        ("row_block", C.c_int64), ("col_block", C.c_int64),
        ("min_scale", C.c_double),
        ("force_variant", C.c_int),
    ]


class OpsnnMxQuantArgs(C.Structure):
    _fields_ = [
        ("x", C.c_void_p), ("x_dtype", C.c_int),
        ("y", C.c_void_p), ("y_dtype", C.c_int),
        ("scale", C.c_void_p),
        ("rows", C.c_int64), ("cols", C.c_int64),
        ("force_variant", C.c_int),
        ("block", C.c_int64), ("scale_alg", C.c_int),
        ("outer", C.c_int64), ("axis_len", C.c_int64), ("inner", C.c_int64), ("round_mode", C.c_int),
    ]


_T = C.c_void_p  # aclTensor*
_SIGS = {
    "aclInit": (C.c_int, [C.c_char_p]),
    "aclFinalize": (C.c_int, []),
    "aclrtSetDevice": (C.c_int, [C.c_int32]),
    "aclrtResetDevice": (C.c_int, [C.c_int32]),
    "aclrtGetDeviceCount": (C.c_int, [C.POINTER(C.c_uint32)]),
    "aclrtSynchronizeDevice": (C.c_int, []),
    "aclGetRecentErrMsg": (C.c_char_p, []),
    "aclrtCreateStream": (C.c_int, [C.POINTER(C.c_void_p)]),
    "aclrtDestroyStream": (C.c_int, [C.c_void_p]),
    "aclrtSynchronizeStream": (C.c_int, [C.c_void_p]),
    "aclrtCreateEvent": (C.c_int, [C.POINTER(C.c_void_p)]),
    "aclrtDestroyEvent": (C.c_int, [C.c_void_p]),
    "aclrtRecordEvent": (C.c_int, [C.c_void_p, C.c_void_p]),
    "aclrtSynchronizeEvent": (C.c_int, [C.c_void_p]),
    "aclrtEventElapsedTime": (C.c_int, [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]),
    "aclrtMalloc": (C.c_int, [C.POINTER(C.c_void_p), C.c_size_t, C.c_int]),
    "aclrtFree": (C.c_int, [C.c_void_p]),
    "aclrtMallocHost": (C.c_int, [C.POINTER(C.c_void_p), C.c_size_t]),
    "aclrtFreeHost": (C.c_int, [C.c_void_p]),
    "aclrtMemcpy": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_int]),
    "aclrtMemcpyAsync": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]),
    "aclrtMemset": (C.c_int, [C.c_void_p, C.c_size_t, C.c_int32, C.c_size_t]),
    "aclCreateTensor": (_T, [C.POINTER(C.c_int64), C.c_uint64, C.c_int, C.POINTER(C.c_int64), C.c_int64, C.c_int,
                             C.POINTER(C.c_int64), C.c_uint64, C.c_void_p]),
    "aclDestroyTensor": (C.c_int32, [_T]),
    "aclGetViewShape": (C.c_int32, [_T, C.POINTER(C.POINTER(C.c_int64)), C.POINTER(C.c_uint64)]),
    "aclGetDataType": (C.c_int32, [_T, C.POINTER(C.c_int)]),
    "aclGetFormat": (C.c_int32, [_T, C.POINTER(C.c_int)]),
    "aclDestroyAclOpExecutor": (C.c_int32, [C.c_void_p]),
    "aclnnQuantMatmulV5GetWorkspaceSize": (C.c_int32, [_T] * 9 + [C.c_bool, C.c_bool, C.c_int64, _T,
                                                              C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnQuantMatmulV5": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "aclnnQuantMatmulWeightNzGetWorkspaceSize": (C.c_int32, [_T] * 9 + [C.c_bool, C.c_bool, C.c_int64, _T,
                                                                    C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnQuantMatmulWeightNz": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "aclnnWeightQuantBatchMatmulNzGetWorkspaceSize": (C.c_int32, [_T] * 7 + [C.c_int, _T, C.POINTER(C.c_uint64),
                                                                         C.POINTER(C.c_void_p)]),
    "aclnnWeightQuantBatchMatmulNz": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "aclnnPrepackMatmulWeightGetWorkspaceSize": (C.c_int32, [_T, _T, _T, _T, C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnPrepackMatmulWeight": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "opsnnTranspose16": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_void_p]),
    "opsnnNzToNd": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int, C.c_int64, C.c_void_p]),
    "opsnnNdToNz": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int, C.c_int64, C.c_void_p]),
    "aclnnWeightQuantBatchMatmulV2GetWorkspaceSize": (C.c_int32, [_T] * 7 + [C.c_int, _T, C.POINTER(C.c_uint64),
                                                                         C.POINTER(C.c_void_p)]),
    "aclnnWeightQuantBatchMatmulV2": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "aclnnWeightQuantBatchMatmulV3GetWorkspaceSize": (C.c_int32, [_T] * 7 + [C.c_int, C.c_int, _T, C.POINTER(C.c_uint64),
                                                                         C.POINTER(C.c_void_p)]),
    "aclnnWeightQuantBatchMatmulV3": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "aclnnConvertWeightToINT4PackGetWorkspaceSize": (C.c_int32, [_T, _T, C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnConvertWeightToINT4Pack": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "aclnnDynamicQuantGetWorkspaceSize": (C.c_int32, [_T] * 4 + [C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnDynamicQuant": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "aclnnDynamicQuantV2GetWorkspaceSize": (C.c_int32, [_T] * 3 + [C.c_int64] + [_T] * 3 + [C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnDynamicQuantV2": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "aclnnDynamicQuantV3GetWorkspaceSize": (C.c_int32, [_T] * 3 + [C.c_int64, C.c_bool, C.c_char_p] + [_T] * 3 + [C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnDynamicQuantV3": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "aclnnDynamicQuantV4GetWorkspaceSize": (C.c_int32, [_T] * 3 + [C.c_int64, C.c_bool, C.c_char_p, C.c_float] + [_T] * 3 + [C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnDynamicQuantV4": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "opsnnDynamicQuant": (C.c_int, [C.POINTER(OpsnnDynQuantArgs), C.c_void_p]),
    "aclnnDynamicBlockQuantGetWorkspaceSize": (C.c_int32, [_T, C.c_double, C.c_char_p, C.c_int64, C.c_int64, C.c_int64, _T, _T,
                                                          C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnDynamicBlockQuant": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "aclnnDynamicBlockQuantV2GetWorkspaceSize": (C.c_int32, [_T, C.c_double, C.c_char_p, C.c_int64, C.c_int64, C.c_int64, C.c_double, _T, _T,
                                                            C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnDynamicBlockQuantV2": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "opsnnDynamicBlockQuant": (C.c_int, [C.POINTER(OpsnnBlockQuantArgs), C.c_void_p]),
    "aclnnDynamicMxQuantGetWorkspaceSize": (C.c_int32, [_T, C.c_int64, C.c_char_p, C.c_int64, C.c_int64, C.c_int64, _T, _T,
                                                       C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnDynamicMxQuant": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "aclnnDynamicMxQuantV2GetWorkspaceSize": (C.c_int32, [_T, C.c_int64, C.c_char_p, C.c_int64, C.c_int64, C.c_int64, C.c_double, _T, _T,
                                                         C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnDynamicMxQuantV2": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "aclnnDynamicMxQuantV3GetWorkspaceSize": (C.c_int32, [_T, C.c_int64, C.c_char_p, C.c_int64, C.c_int64, C.c_int64, C.c_double, C.c_double, _T, _T,
                                                         C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnDynamicMxQuantV3": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "opsnnDynamicMxQuant": (C.c_int, [C.POINTER(OpsnnMxQuantArgs), C.c_void_p]),
    "aclnnTransQuantParamV2GetWorkspaceSize": (C.c_int32, [_T, _T, _T, C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnTransQuantParamV2": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "aclnnTransQuantParamV3GetWorkspaceSize": (C.c_int32, [_T, _T, C.c_int64, _T, C.POINTER(C.c_uint64), C.POINTER(C.c_void_p)]),
    "aclnnTransQuantParamV3": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]),
    "opsnnTransQuantParam": (C.c_int, [C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_int, C.c_void_p, C.c_void_p]),
    "opsnnPackB4": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_int64, C.c_void_p]),
    "opsnnSetWeightCache": (None, [C.c_int64]),
    "opsnnWeightCacheClear": (None, []),
    "opsnnWeightCacheInvalidate": (C.c_int, [C.c_void_p, C.c_uint64]),
    "opsnnWeightCacheStats": (None, [C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
    "opsnnQmmInt8": (C.c_int, [C.POINTER(OpsnnQmmArgs), C.c_void_p]),
    "opsnnQmmInt8Static": (C.c_int, [C.POINTER(OpsnnQmmArgs), C.c_void_p]),
    "opsnnQmmBlockScale": (C.c_int, [C.POINTER(OpsnnQmmArgs), C.c_void_p]),
    "opsnnQmmMx": (C.c_int, [C.POINTER(OpsnnQmmArgs), C.c_void_p]),
    "opsnnQmmTc": (C.c_int, [C.POINTER(OpsnnQmmArgs), C.c_void_p]),
    "opsnnQmmGroup": (C.c_int, [C.POINTER(OpsnnQmmArgs), C.c_void_p]),
    "opsnnQmmWorkspace": (C.c_uint64, [C.POINTER(OpsnnQmmArgs), C.c_int]),
    "opsnnWqmm": (C.c_int, [C.POINTER(OpsnnWqmmArgs), C.c_void_p]),
    "opsnnWqmmWorkspace": (C.c_uint64, [C.POINTER(OpsnnWqmmArgs)]),
    "opsnnTranspose8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_void_p]),
    "opsnnTranspose4": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_void_p]),
    "opsnnSetFp8Fast": (None, [C.c_int]),
    "opsnnSetForcePlain": (None, [C.c_int]),
    "opsnnSetMx8Wide": (None, [C.c_int]),
    "opsnnSetWqTileMin": (None, [C.c_int]),
    "opsnnGetFp8Fast": (C.c_int, []),
    "opsnnDeviceInfo": (C.c_int, [C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int64), C.c_char_p, C.c_int]),
}
EXPORTED_SYMBOLS = sorted(_SIGS)

_lib = None


def lib():
    """The loaded shared library.  There is no fallback: a missing build is an error."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
        _lib = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGS.items():
            fn = getattr(_lib, name)
            fn.restype, fn.argtypes = res, args
    return _lib


def err_msg():
    return lib().aclGetRecentErrMsg().decode("utf-8", "replace")


def check(rc, what="call"):
    if rc != 0:
        raise RuntimeError(f"{what} failed with status {rc}: {err_msg()}")


def gpu_available():
    n = C.c_uint32(0)
    try:
        lib().aclrtGetDeviceCount(C.byref(n))
    except Exception:
        return False
    return n.value > 0


class DeviceBuffer:
    """A device allocation, optionally initialised from a numpy array (any dtype; bytes are copied)."""

    def __init__(self, nbytes=None, host=None):
        if host is not None:
            host = np.ascontiguousarray(host)
            nbytes = host.nbytes
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(lib().aclrtMalloc(C.byref(p), max(self.nbytes, 16), 0), "aclrtMalloc")
        self.ptr = p.value
        if host is not None and self.nbytes:
            check(lib().aclrtMemcpy(self.ptr, self.nbytes, host.ctypes.data, self.nbytes, H2D), "aclrtMemcpy H2D")

    def to_host(self, dtype, shape):
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes, (out.nbytes, self.nbytes)
        if out.nbytes:
            check(lib().aclrtMemcpy(out.ctypes.data, out.nbytes, self.ptr, out.nbytes, D2H), "aclrtMemcpy D2H")
        return out

    def fill(self, byte):
        check(lib().aclrtMemset(self.ptr, self.nbytes, byte, self.nbytes), "aclrtMemset")

    def upload(self, host):
        """Overwrite the allocation's first bytes with a numpy array's."""
        host = np.ascontiguousarray(host)
        assert host.nbytes <= self.nbytes, (host.nbytes, self.nbytes)
        if host.nbytes:
            check(lib().aclrtMemcpy(self.ptr, host.nbytes, host.ctypes.data, host.nbytes, H2D), "aclrtMemcpy H2D")

    def free(self):
        if self.ptr:
            lib().aclrtFree(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _i64(seq):
    seq = list(seq)
    return (C.c_int64 * max(len(seq), 1))(*seq), len(seq)


class Tensor:
    """An aclTensor handle.  shape/strides/offset are in elements (also for 4-bit types)."""

    def __init__(self, shape, dtype, data=None, strides=None, offset=0, fmt=ACL_FORMAT_ND, storage_shape=None):
        self.shape, self.dtype, self.buf = tuple(shape), dtype, data
        dims, n = _i64(shape)
        st = _i64(strides)[0] if strides is not None else None
        sdims, sn = _i64(storage_shape if storage_shape is not None else shape)
        ptr = data.ptr if isinstance(data, DeviceBuffer) else data
        self.handle = lib().aclCreateTensor(dims, n, dtype, st, offset, fmt, sdims, sn, ptr)
        if not self.handle:
            raise RuntimeError("aclCreateTensor failed: " + err_msg())

    def destroy(self):
        if self.handle:
            lib().aclDestroyTensor(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def _h(t):
    return t.handle if t is not None else None


class Stream:
    def __init__(self):
        p = C.c_void_p()
        check(lib().aclrtCreateStream(C.byref(p)), "aclrtCreateStream")
        self.ptr = p.value

    def sync(self):
        check(lib().aclrtSynchronizeStream(self.ptr), "aclrtSynchronizeStream")

    def destroy(self):
        if self.ptr:
            lib().aclrtDestroyStream(self.ptr)
            self.ptr = None


class Event:
    def __init__(self):
        p = C.c_void_p()
        check(lib().aclrtCreateEvent(C.byref(p)), "aclrtCreateEvent")
        self.ptr = p.value

    def record(self, stream):
        check(lib().aclrtRecordEvent(self.ptr, stream.ptr if stream else None), "aclrtRecordEvent")

    def sync(self):
        check(lib().aclrtSynchronizeEvent(self.ptr), "aclrtSynchronizeEvent")

    def elapsed_ms(self, end):
        ms = C.c_float()
        check(lib().aclrtEventElapsedTime(C.byref(ms), self.ptr, end.ptr), "aclrtEventElapsedTime")
        return ms.value


def quant_matmul_v5_get_workspace(x1, x2, x1_scale, x2_scale, out, *, y_scale=None, x1_offset=None, x2_offset=None,
                                  y_offset=None, bias=None, transpose_x1=False, transpose_x2=False, group_size=0,
                                  ws_ptr=True, ex_ptr=True, weight_nz=False):
    """Phase 1 (of aclnnQuantMatmulWeightNz when weight_nz).  Returns (status, workspace_size, executor)."""
    ws, ex = C.c_uint64(0), C.c_void_p()
    fn = lib().aclnnQuantMatmulWeightNzGetWorkspaceSize if weight_nz else lib().aclnnQuantMatmulV5GetWorkspaceSize
    rc = fn(
        _h(x1), _h(x2), _h(x1_scale), _h(x2_scale), _h(y_scale), _h(x1_offset), _h(x2_offset), _h(y_offset), _h(bias),
        transpose_x1, transpose_x2, group_size, _h(out), C.byref(ws) if ws_ptr else None, C.byref(ex) if ex_ptr else None)
    return rc, ws.value, ex.value


# A byte (0 .. 255) to fill every workspace with that the two-phase helpers below allocate, or None.  The parity tests set 0xFF
# (NaN in every floating-point format used here): a kernel that reads workspace bytes no kernel of the call has written then
# shows in the results.
FILL_NEW_WORKSPACE = None


def _new_workspace(nbytes):
    if not nbytes:
        return None
    buf = DeviceBuffer(nbytes)
    if FILL_NEW_WORKSPACE is not None:
        buf.fill(FILL_NEW_WORKSPACE)
    return buf


def quant_matmul_v5(x1, x2, x1_scale, x2_scale, out, stream=None, **kw):
    """Both phases; allocates the workspace the first phase asks for.  Asynchronous on `stream`."""
    rc, ws, ex = quant_matmul_v5_get_workspace(x1, x2, x1_scale, x2_scale, out, **kw)
    check(rc, "aclnnQuantMatmulV5GetWorkspaceSize")
    wbuf = _new_workspace(ws)
    run = lib().aclnnQuantMatmulWeightNz if kw.get("weight_nz") else lib().aclnnQuantMatmulV5
    check(run(wbuf.ptr if wbuf else None, ws, ex, stream.ptr if stream else None), "aclnnQuantMatmulV5")
    return wbuf  # keep alive until the stream has been synchronised


def prepack_matmul_weight(weight, packed, scale=None, scale_packed=None, stream=None):
    """Both phases of aclnnPrepackMatmulWeight; returns (status of phase 1, workspace buffer kept alive)."""
    ws, ex = C.c_uint64(0), C.c_void_p()
    rc = lib().aclnnPrepackMatmulWeightGetWorkspaceSize(_h(weight), _h(scale), _h(packed), _h(scale_packed), C.byref(ws), C.byref(ex))
    if rc != 0:
        return rc, None
    wbuf = _new_workspace(ws.value)
    check(lib().aclnnPrepackMatmulWeight(wbuf.ptr if wbuf else None, ws.value, ex, stream.ptr if stream else None), "aclnnPrepackMatmulWeight")
    return 0, wbuf


def weight_quant_batch_matmul_get_workspace(x, weight, scale, y, *, offset=None, quant_scale=None, quant_offset=None,
                                            bias=None, group_size=0, inner_precise=None, weight_nz=False):
    ws, ex = C.c_uint64(0), C.c_void_p()
    if weight_nz:
        rc = lib().aclnnWeightQuantBatchMatmulNzGetWorkspaceSize(_h(x), _h(weight), _h(scale), _h(offset), _h(quant_scale),
                                                                 _h(quant_offset), _h(bias), group_size, _h(y),
                                                                 C.byref(ws), C.byref(ex))
    elif inner_precise is None:
        rc = lib().aclnnWeightQuantBatchMatmulV2GetWorkspaceSize(_h(x), _h(weight), _h(scale), _h(offset), _h(quant_scale),
                                                                 _h(quant_offset), _h(bias), group_size, _h(y),
                                                                 C.byref(ws), C.byref(ex))
    else:
        rc = lib().aclnnWeightQuantBatchMatmulV3GetWorkspaceSize(_h(x), _h(weight), _h(scale), _h(offset), _h(quant_scale),
                                                                 _h(quant_offset), _h(bias), group_size, inner_precise,
                                                                 _h(y), C.byref(ws), C.byref(ex))
    return rc, ws.value, ex.value


def weight_quant_batch_matmul(x, weight, scale, y, stream=None, **kw):
    v3 = kw.get("inner_precise") is not None
    rc, ws, ex = weight_quant_batch_matmul_get_workspace(x, weight, scale, y, **kw)
    check(rc, "aclnnWeightQuantBatchMatmulGetWorkspaceSize")
    wbuf = _new_workspace(ws)
    run = lib().aclnnWeightQuantBatchMatmulV3 if v3 else lib().aclnnWeightQuantBatchMatmulV2
    if kw.get("weight_nz"):
        run = lib().aclnnWeightQuantBatchMatmulNz
    check(run(wbuf.ptr if wbuf else None, ws, ex, stream.ptr if stream else None), "aclnnWeightQuantBatchMatmul")
    return wbuf


def dynamic_quant_get_workspace(x, y, scale, *, smooth=None, offset=None, group_index=None, v2=False, dst_type=2, quant_mode=None,
                                is_symmetrical=None, dst_type_max=None):
    """Phase 1 of aclnnDynamicQuant; V2 when v2 / offset / group_index is given; V3 when quant_mode is given; V4 when dst_type_max
    is given too.  Returns (status, workspace, executor)."""
    ws, ex = C.c_uint64(0), C.c_void_p()
    if quant_mode is not None:
        sym = (offset is None) if is_symmetrical is None else is_symmetrical
        if dst_type_max is None:
            rc = lib().aclnnDynamicQuantV3GetWorkspaceSize(_h(x), _h(smooth), _h(group_index), dst_type, sym, quant_mode, _h(y), _h(scale),
                                                           _h(offset), C.byref(ws), C.byref(ex))
        else:
            rc = lib().aclnnDynamicQuantV4GetWorkspaceSize(_h(x), _h(smooth), _h(group_index), dst_type, sym, quant_mode, dst_type_max, _h(y),
                                                           _h(scale), _h(offset), C.byref(ws), C.byref(ex))
    elif v2 or offset is not None or group_index is not None:
        rc = lib().aclnnDynamicQuantV2GetWorkspaceSize(_h(x), _h(smooth), _h(group_index), dst_type, _h(y), _h(scale), _h(offset),
                                                       C.byref(ws), C.byref(ex))
    else:
        rc = lib().aclnnDynamicQuantGetWorkspaceSize(_h(x), _h(smooth), _h(y), _h(scale), C.byref(ws), C.byref(ex))
    return rc, ws.value, ex.value


def dynamic_quant(x, y, scale, stream=None, **kw):
    """Both phases; asynchronous on `stream`."""
    v2 = kw.get("v2") or kw.get("offset") is not None or kw.get("group_index") is not None
    rc, ws, ex = dynamic_quant_get_workspace(x, y, scale, **kw)
    check(rc, "aclnnDynamicQuantGetWorkspaceSize")
    run = lib().aclnnDynamicQuantV2 if v2 else lib().aclnnDynamicQuant
    if kw.get("quant_mode") is not None:
        run = lib().aclnnDynamicQuantV4 if kw.get("dst_type_max") is not None else lib().aclnnDynamicQuantV3
    check(run(None, ws, ex, stream.ptr if stream else None), "aclnnDynamicQuant")


def dynamic_block_quant_get_workspace(x, y, scale, *, dst_type=None, row_block=1, col_block=128, min_scale=0.0, round_mode=b"rint",
                                      dst_type_max=None):
    ws, ex = C.c_uint64(0), C.c_void_p()
    dst = dst_type if dst_type is not None else (y.dtype if y is not None else 36)
    if dst_type_max is not None:   # V2
        rc = lib().aclnnDynamicBlockQuantV2GetWorkspaceSize(_h(x), min_scale, round_mode, dst, row_block, col_block, dst_type_max, _h(y),
                                                            _h(scale), C.byref(ws), C.byref(ex))
        return rc, ws.value, ex.value
    rc = lib().aclnnDynamicBlockQuantGetWorkspaceSize(_h(x), min_scale, round_mode, dst, row_block, col_block, _h(y), _h(scale),
                                                      C.byref(ws), C.byref(ex))
    return rc, ws.value, ex.value


def dynamic_block_quant(x, y, scale, stream=None, **kw):
    rc, ws, ex = dynamic_block_quant_get_workspace(x, y, scale, **kw)
    check(rc, "aclnnDynamicBlockQuantGetWorkspaceSize")
    run = lib().aclnnDynamicBlockQuantV2 if kw.get("dst_type_max") is not None else lib().aclnnDynamicBlockQuant
    check(run(None, ws, ex, stream.ptr if stream else None), "aclnnDynamicBlockQuant")


def dynamic_mx_quant_get_workspace(x, y, scale, *, axis=-1, round_mode=b"rint", dst_type=None, blocksize=32, scale_alg=0, dst_type_max=None,
                                   max_low_bound=None):
    """aclnnDynamicMxQuant; V2 when dst_type_max is given, V3 when max_low_bound is given too."""
    ws, ex = C.c_uint64(0), C.c_void_p()
    dst = dst_type if dst_type is not None else (y.dtype if y is not None else 40)
    if max_low_bound is not None:
        rc = lib().aclnnDynamicMxQuantV3GetWorkspaceSize(_h(x), axis, round_mode, dst, blocksize, scale_alg, dst_type_max or 0.0, max_low_bound,
                                                         _h(y), _h(scale), C.byref(ws), C.byref(ex))
        return rc, ws.value, ex.value
    if dst_type_max is not None:
        rc = lib().aclnnDynamicMxQuantV2GetWorkspaceSize(_h(x), axis, round_mode, dst, blocksize, scale_alg, dst_type_max, _h(y), _h(scale),
                                                         C.byref(ws), C.byref(ex))
        return rc, ws.value, ex.value
    rc = lib().aclnnDynamicMxQuantGetWorkspaceSize(_h(x), axis, round_mode, dst, blocksize, scale_alg, _h(y), _h(scale),
                                                   C.byref(ws), C.byref(ex))
    return rc, ws.value, ex.value


def dynamic_mx_quant(x, y, scale, stream=None, **kw):
    rc, ws, ex = dynamic_mx_quant_get_workspace(x, y, scale, **kw)
    check(rc, "aclnnDynamicMxQuantGetWorkspaceSize")
    run = lib().aclnnDynamicMxQuant
    if kw.get("max_low_bound") is not None:
        run = lib().aclnnDynamicMxQuantV3
    elif kw.get("dst_type_max") is not None:
        run = lib().aclnnDynamicMxQuantV2
    check(run(None, ws, ex, stream.ptr if stream else None), "aclnnDynamicMxQuant")


def trans_quant_param_get_workspace(scale, offset, out, round_mode=None):
    """Phase 1 of aclnnTransQuantParamV2, or V3 when round_mode is given."""
    ws, ex = C.c_uint64(0), C.c_void_p()
    if round_mode is None:
        rc = lib().aclnnTransQuantParamV2GetWorkspaceSize(_h(scale), _h(offset), _h(out), C.byref(ws), C.byref(ex))
    else:
        rc = lib().aclnnTransQuantParamV3GetWorkspaceSize(_h(scale), _h(offset), round_mode, _h(out), C.byref(ws), C.byref(ex))
    return rc, ws.value, ex.value


def trans_quant_param(scale, offset, out, round_mode=None, stream=None):
    rc, ws, ex = trans_quant_param_get_workspace(scale, offset, out, round_mode)
    check(rc, "aclnnTransQuantParamGetWorkspaceSize")
    run = lib().aclnnTransQuantParamV2 if round_mode is None else lib().aclnnTransQuantParamV3
    check(run(None, ws, ex, stream.ptr if stream else None), "aclnnTransQuantParam")


def convert_weight_to_int4_pack(weight, weight_int4_pack):
    """Both phases of aclnnConvertWeightToINT4Pack; returns the first phase's status (the second does nothing)."""
    ws, ex = C.c_uint64(0), C.c_void_p()
    rc = lib().aclnnConvertWeightToINT4PackGetWorkspaceSize(_h(weight), _h(weight_int4_pack), C.byref(ws), C.byref(ex))
    if rc == 0:
        check(lib().aclnnConvertWeightToINT4Pack(None, ws.value, ex, None), "aclnnConvertWeightToINT4Pack")
    return rc


def device_info():
    cu, clk, mem = C.c_int(), C.c_int(), C.c_int64()
    arch = C.create_string_buffer(64)
    check(lib().opsnnDeviceInfo(C.byref(cu), C.byref(clk), C.byref(mem), arch, 64), "opsnnDeviceInfo")
    return {"cu": cu.value, "clock_khz": clk.value, "hbm_bytes": mem.value, "arch": arch.value.decode()}
