"""ctypes access to oracle/liboracle.so (the CPU restatement of the reference goldens) plus numpy-side
helpers for the narrow float formats.  Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "oracle", "liboracle.so")

F32, F16, I8, I32, BF16, I4, E5M2, E4M3, E8M0, E2M1, E1M2 = 0, 1, 2, 3, 27, 29, 35, 36, 37, 40, 41
U64 = 10
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True)
        _lib = C.CDLL(LIB)
        L = _lib
        vp, i64, ci = C.c_void_p, C.c_int64, C.c_int
        L.orc_qmm_int8_acc.argtypes = [vp, vp, i64, i64, i64, ci, ci, vp]
        L.orc_qmm_pertoken_epilogue.argtypes = [vp, i64, i64, vp, vp, i64, vp, ci, ci, vp]
        L.orc_qmm_pertoken.argtypes = [vp, vp, i64, i64, i64, ci, ci, vp, vp, i64, vp, ci, ci, vp, vp]
        L.orc_qmm_perblock.argtypes = [vp, vp, ci, ci, i64, i64, i64, ci, ci, vp, vp, i64, i64, i64, vp, ci, vp]
        L.orc_qmm_tc.argtypes = [vp, vp, ci, ci, i64, i64, i64, ci, ci, vp, ci, i64, vp, vp, i64, vp, ci, ci, vp]
        L.orc_qmm_pertoken_f8.argtypes = [vp, vp, ci, ci, i64, i64, i64, ci, ci, vp, vp, i64, vp, ci, vp]
        L.orc_qmm_mx.argtypes = [vp, vp, ci, ci, i64, i64, i64, ci, ci, vp, vp, vp, ci, vp]
        L.orc_wqbmm.argtypes = [vp, ci, vp, ci, i64, i64, i64, ci, vp, ci, i64, vp, i64, vp, ci, vp]
        L.orc_qmm_tcg.argtypes = [vp, vp, i64, i64, i64, ci, vp, ci, i64, vp, i64, vp, ci, vp]
        L.orc_qmm_i4_asym.argtypes = [vp, vp, i64, i64, i64, ci, vp, vp, vp, ci, vp]
        for n in ("orc_vec_f32_to_bf16", "orc_vec_bf16_to_f32", "orc_vec_f32_to_f16", "orc_vec_f16_to_f32",
                  "orc_vec_f32_to_e4m3", "orc_vec_e4m3_to_f32", "orc_vec_e5m2_to_f32", "orc_vec_e8m0_to_f32"):
            getattr(L, n).argtypes = [vp, vp, C.c_size_t]
        L.orc_unpack_groupsize.argtypes = [i64, C.POINTER(i64), C.POINTER(i64), C.POINTER(i64)]
        L.orc_pack_int4_to_int32.argtypes = [vp, vp, C.c_size_t]
        L.orc_unpack_int32_to_int4.argtypes = [vp, vp, C.c_size_t]
        L.orc_convert_weight_b4.argtypes = [vp, i64, C.c_int, vp]
        L.orc_convert_weight_b4.restype = None
        L.orc_dynamic_quant.argtypes = [vp, C.c_int, i64, i64, vp, C.c_int, C.c_int, vp, vp, vp]
        L.orc_dynamic_quant.restype = C.c_int
        L.orc_dynamic_quant_grouped.argtypes = [vp, C.c_int, i64, i64, vp, vp, i64, C.c_int, C.c_int, vp, vp, vp]
        L.orc_dynamic_quant_grouped.restype = C.c_int
        L.orc_dynamic_quant_wide.argtypes = [vp, C.c_int, i64, i64, i64, C.c_int, vp, C.c_int, C.c_int, vp, vp, vp]
        L.orc_dynamic_quant_wide.restype = C.c_int
        L.orc_e5m2_from_f32.argtypes = [C.c_float]
        L.orc_e5m2_from_f32.restype = C.c_uint8
        L.orc_dynamic_block_quant.argtypes = [vp, C.c_int, i64, i64, i64, i64, i64, C.c_double, C.c_int, vp, vp]
        L.orc_dynamic_block_quant.restype = C.c_int
        L.orc_dynamic_mx_quant_alg.argtypes = [vp, C.c_int, i64, i64, i64, C.c_int, C.c_int, vp, vp]
        L.orc_dynamic_mx_quant_alg.restype = C.c_int
        L.orc_dynamic_mx_quant.argtypes = [vp, C.c_int, i64, i64, i64, C.c_int, vp, vp]
        L.orc_dynamic_mx_quant.restype = C.c_int
        L.orc_dynamic_mx_quant_general.argtypes = [vp, C.c_int, i64, i64, i64, i64, C.c_int, C.c_int, C.c_int, vp, vp]
        L.orc_dynamic_mx_quant_general.restype = C.c_int
        L.orc_trans_quant_param.argtypes = [vp, i64, vp, i64, C.c_int, vp]
        L.orc_trans_quant_param.restype = None
        L.orc_scale_generate.argtypes = [C.c_float]
        L.orc_scale_generate.restype = C.c_float
        L.orc_u64_to_deq_scale.argtypes = [C.c_uint64]
        L.orc_u64_to_deq_scale.restype = C.c_float
        L.orc_e2m1_to_f32.argtypes = [C.c_uint8]
        L.orc_e2m1_to_f32.restype = C.c_float
    return _lib


def _p(a):
    return a.ctypes.data if a is not None else None


def _conv(name, src, out_dtype):
    src = np.ascontiguousarray(src)
    out = np.empty(src.shape, dtype=out_dtype)
    getattr(lib(), name)(_p(src), _p(out), src.size)
    return out


def f32_to_bf16(a): return _conv("orc_vec_f32_to_bf16", np.asarray(a, np.float32), np.uint16)
def bf16_to_f32(a): return _conv("orc_vec_bf16_to_f32", np.asarray(a, np.uint16), np.float32)
def f32_to_f16(a): return _conv("orc_vec_f32_to_f16", np.asarray(a, np.float32), np.uint16)
def f16_to_f32(a): return _conv("orc_vec_f16_to_f32", np.asarray(a, np.uint16), np.float32)
def f32_to_e4m3(a): return _conv("orc_vec_f32_to_e4m3", np.asarray(a, np.float32), np.uint8)
def e4m3_to_f32(a): return _conv("orc_vec_e4m3_to_f32", np.asarray(a, np.uint8), np.float32)
def e5m2_to_f32(a): return _conv("orc_vec_e5m2_to_f32", np.asarray(a, np.uint8), np.float32)
def e8m0_to_f32(a): return _conv("orc_vec_e8m0_to_f32", np.asarray(a, np.uint8), np.float32)


E2M1_VALUES = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6], np.float32)


def dynamic_quant(x, x_dt, y_dt, smooth=None, symmetric=True, group_end=None, fill=0):
    """x: uint16 bits [..., cols] of x_dt.  Returns (y bytes, scale[, offset]); int4 results are packed two per byte.
    group_end: per-expert row ends (then smooth is [experts, cols]); rows past the last end keep the byte `fill`."""
    x = np.ascontiguousarray(x, np.uint16)
    cols = x.shape[-1]
    rows = x.size // cols
    y = np.zeros(x.shape[:-1] + ((cols // 2) if y_dt == I4 else cols,), np.uint8)
    scale = np.zeros(x.shape[:-1], np.float32)
    offset = np.zeros(x.shape[:-1], np.float32)
    sm = None if smooth is None else np.ascontiguousarray(smooth, np.uint16)
    ge = None if group_end is None else np.ascontiguousarray(group_end, np.int64)
    if fill:
        y[...] = fill
        scale.view(np.uint8)[...] = fill
        offset.view(np.uint8)[...] = fill
    rc = lib().orc_dynamic_quant_grouped(x.ctypes.data, x_dt, rows, cols, sm.ctypes.data if sm is not None else None,
                                         ge.ctypes.data if ge is not None else None, ge.size if ge is not None else 0, y_dt, int(symmetric),
                                         y.ctypes.data, scale.ctypes.data, offset.ctypes.data)
    assert rc == 0, rc
    return (y, scale) if symmetric else (y, scale, offset)


def dynamic_block_quant(x, x_dt, y_dt, rb, cb, min_scale=0.0):
    """x: uint16 bits [rows, cols] or [batch, rows, cols].  Returns (y bytes of x's shape, scale [.., ceil(rows/rb), ceil(cols/cb)])."""
    x = np.ascontiguousarray(x, np.uint16)
    rows, cols = x.shape[-2:]
    batch = x.shape[0] if x.ndim == 3 else 1
    y = np.zeros(x.shape, np.uint8)
    scale = np.zeros(x.shape[:-2] + (-(-rows // rb), -(-cols // cb)), np.float32)
    rc = lib().orc_dynamic_block_quant(x.ctypes.data, x_dt, batch, rows, cols, rb, cb, float(min_scale), y_dt, y.ctypes.data, scale.ctypes.data)
    assert rc == 0, rc
    return y, scale


def dynamic_mx_quant(x, x_dt, y_dt, block=32, scale_alg=0):
    """x: uint16 bits [..., cols].  Returns (y bytes [..., cols] or [..., cols / 2] for e2m1, e8m0 bytes [..., ceil(nblk / 2), 2])."""
    x = np.ascontiguousarray(x, np.uint16)
    cols = x.shape[-1]
    rows = x.size // cols
    nblk = -(-cols // block)
    y = np.zeros(x.shape[:-1] + ((cols // 2) if y_dt == E2M1 else cols,), np.uint8)
    scale = np.zeros(x.shape[:-1] + ((nblk + 1) // 2, 2), np.uint8)
    rc = lib().orc_dynamic_mx_quant_alg(x.ctypes.data, x_dt, rows, cols, block, scale_alg, y_dt, y.ctypes.data, scale.ctypes.data)
    assert rc == 0, rc
    return y, scale


ROUND_MODES = {"rint": 0, "round": 1, "floor": 2, "ceil": 3, "trunc": 4}


def dynamic_mx_quant_general(x, x_dt, y_dt, axis=-1, block=32, scale_alg=0, round_mode="rint"):
    """x: uint16 bits (fp16 / bf16) or float32, any shape; blocks along `axis`.  Returns (y bytes with x's shape, the last dim
    halved for the 4-bit types, e8m0 bytes with x's shape where the axis holds ceil(nblk / 2) and a trailing 2)."""
    x = np.ascontiguousarray(x, np.float32 if x_dt == F32 else np.uint16)
    ax = axis % x.ndim
    A = x.shape[ax]
    outer = int(np.prod(x.shape[:ax], dtype=np.int64))
    inner = int(np.prod(x.shape[ax + 1:], dtype=np.int64))
    nblk = -(-A // block)
    fp4 = y_dt in (E2M1, E1M2)
    y = np.zeros(x.shape[:-1] + ((x.shape[-1] // 2) if fp4 else x.shape[-1],), np.uint8)
    scale = np.zeros(x.shape[:ax] + ((nblk + 1) // 2,) + x.shape[ax + 1:] + (2,), np.uint8)
    rc = lib().orc_dynamic_mx_quant_general(x.ctypes.data, x_dt, outer, A, inner, block, scale_alg, ROUND_MODES[round_mode], y_dt,
                                            y.ctypes.data, scale.ctypes.data)
    assert rc == 0, rc
    return y, scale


def trans_quant_param(scale, offset=None, round_mode=0):
    scale = np.ascontiguousarray(scale, np.float32).reshape(-1)
    off = None if offset is None else np.ascontiguousarray(offset, np.float32).reshape(-1)
    n = max(scale.size, off.size if off is not None else 0)
    out = np.zeros(n, np.uint64)
    lib().orc_trans_quant_param(scale.ctypes.data, scale.size, off.ctypes.data if off is not None else None,
                                off.size if off is not None else 0, round_mode, out.ctypes.data)
    return out


def dynamic_quant_wide(x, x_dt, y_dt, mode, smooth=None, symmetric=True):
    """mode "pertensor": one scale; "perchannel": x [..., R, C], one scale per leading index and column.  Returns (y, scale[, offset])."""
    x = np.ascontiguousarray(x, np.uint16)
    cols = x.shape[-1]
    rows = x.size // cols
    per_tensor = mode == "pertensor"
    chan_rows = rows if per_tensor else x.shape[-2]
    sshape = (1,) if per_tensor else x.shape[:-2] + (cols,)
    y = np.zeros(x.shape[:-1] + ((cols // 2) if y_dt == I4 else cols,), np.uint8)
    scale, offset = np.zeros(sshape, np.float32), np.zeros(sshape, np.float32)
    sm = None if smooth is None else np.ascontiguousarray(smooth, np.uint16)
    rc = lib().orc_dynamic_quant_wide(x.ctypes.data, x_dt, rows, cols, chan_rows, 1 if per_tensor else 2, sm.ctypes.data if sm is not None else None,
                                      y_dt, int(symmetric), y.ctypes.data, scale.ctypes.data, offset.ctypes.data)
    assert rc == 0, rc
    return (y, scale) if symmetric else (y, scale, offset)


def convert_weight_b4(w):
    """int32 or float32 carrier array (one 4-bit value per element) -> uint8 array with half the last dim."""
    w = np.ascontiguousarray(w)
    assert w.dtype in (np.int32, np.float32) and w.shape[-1] % 2 == 0
    out = np.empty(w.shape[:-1] + (w.shape[-1] // 2,), np.uint8)
    lib().orc_convert_weight_b4(w.ctypes.data, w.size, int(w.dtype == np.float32), out.ctypes.data)
    return out


def pack_nibbles(codes):
    """[.., C] values 0..15 -> [.., C/2] bytes, even index in the low nibble."""
    codes = np.asarray(codes, np.uint8)
    return (codes[..., 0::2] & 15) | ((codes[..., 1::2] & 15) << 4)


def unpack_nibbles(b):
    b = np.asarray(b, np.uint8)
    out = np.empty(b.shape[:-1] + (b.shape[-1] * 2,), np.uint8)
    out[..., 0::2] = b & 15
    out[..., 1::2] = b >> 4
    return out


def b16_to_f32(bits, dt):
    return bf16_to_f32(bits) if dt == BF16 else f16_to_f32(bits)


def f32_to_b16(v, dt):
    return f32_to_bf16(v) if dt == BF16 else f32_to_f16(v)


def out_array(shape, dt):
    return np.empty(shape, {F32: np.float32, I32: np.int32, I8: np.int8}.get(dt, np.uint16))


def qmm_pertoken(x1, x2, M, K, N, tA, tB, x1s, x2s, bias, bias_dt, y_dt, want_acc=False):
    y = out_array((M, N), y_dt)
    acc = np.empty((M, N), np.int32) if want_acc else None
    x2s = np.ascontiguousarray(x2s, np.float32)
    rc = lib().orc_qmm_pertoken(_p(x1), _p(x2), M, K, N, int(tA), int(tB), _p(x1s), _p(x2s), x2s.size, _p(bias), bias_dt, y_dt,
                                _p(y), _p(acc))
    assert rc == 0
    return (y, acc) if want_acc else y


def qmm_int8_acc(x1, x2, M, K, N, tA=False, tB=False):
    acc = np.empty((M, N), np.int32)
    assert lib().orc_qmm_int8_acc(_p(x1), _p(x2), M, K, N, int(tA), int(tB), _p(acc)) == 0
    return acc


def qmm_perblock(x1, x2, dt1, dt2, M, K, N, tA, tB, x1s, x2s, gsM, gsN, gsK, bias, y_dt):
    y = out_array((M, N), y_dt)
    rc = lib().orc_qmm_perblock(_p(x1), _p(x2), dt1, dt2, M, K, N, int(tA), int(tB), _p(x1s), _p(x2s), gsM, gsN, gsK, _p(bias),
                                y_dt, _p(y))
    assert rc == 0
    return y


def qmm_tc(x1, x2, dt1, dt2, M, K, N, tA, tB, scale, scale_dt, pertoken, offset, bias, bias_dt, y_dt):
    """Per-tensor / per-channel family; scale is float32 / bf16 bits / uint64 words according to scale_dt."""
    y = out_array((M, N), y_dt)
    scale = np.ascontiguousarray(scale)
    offset = None if offset is None else np.ascontiguousarray(offset, np.float32)
    pertoken = None if pertoken is None else np.ascontiguousarray(pertoken, np.float32)
    rc = lib().orc_qmm_tc(_p(x1), _p(x2), dt1, dt2, M, K, N, int(tA), int(tB), _p(scale), scale_dt, scale.size, _p(pertoken),
                          _p(offset), 0 if offset is None else offset.size, _p(bias), bias_dt, y_dt, _p(y))
    assert rc == 0
    return y


def qmm_pertoken_f8(x1, x2, dt1, dt2, M, K, N, tA, tB, x1s, x2s, bias, y_dt):
    """fp8 operands with one fp32 scale per row of x1 and one or N for x2 (K-C / K-T through compute_pertoken)."""
    y = out_array((M, N), y_dt)
    x1s = np.ascontiguousarray(x1s, np.float32); x2s = np.ascontiguousarray(x2s, np.float32)
    bias = None if bias is None else np.ascontiguousarray(bias, np.float32)
    rc = lib().orc_qmm_pertoken_f8(_p(x1), _p(x2), dt1, dt2, M, K, N, int(tA), int(tB), _p(x1s), _p(x2s), x2s.size, _p(bias), y_dt, _p(y))
    assert rc == 0
    return y


def pack_u64_scale(scale_f32, offset_f32=None):
    """The 64-bit packed scale of the static modes: fp32 bits in the low word, bit 46 set, the offset as a signed
    9-bit integer at bits 37..45 (layout read by u64_to_deq_scale / u64_to_offset, matmul_quant_util.py:129-158)."""
    u = np.ascontiguousarray(scale_f32, np.float32).view(np.uint32).astype(np.uint64)
    u |= np.uint64(1 << 46)
    if offset_f32 is not None:
        s9 = np.clip(np.rint(np.asarray(offset_f32, np.float32)), -256, 255).astype(np.int64)
        u |= (s9.astype(np.uint64) & np.uint64(0x1FF)) << np.uint64(37)
    return u


def qmm_mx(x1, x2, dt1, dt2, M, K, N, tA, tB, x1s, x2s, bias, y_dt):
    y = out_array((M, N), y_dt)
    rc = lib().orc_qmm_mx(_p(x1), _p(x2), dt1, dt2, M, K, N, int(tA), int(tB), _p(x1s), _p(x2s), _p(bias), y_dt, _p(y))
    assert rc == 0
    return y


def qmm_tcg(x1, x2, M, K, N, tB, x2s, s_dt, gs, yscale, bias, y_dt):
    """fp8 e4m3 x fp4 with 16-bit group scales and a packed 64-bit output scale (compute_t_cg)."""
    y = out_array((M, N), y_dt)
    x2s = np.ascontiguousarray(x2s)
    yscale = None if yscale is None else np.ascontiguousarray(yscale, np.uint64)
    bias = None if bias is None else np.ascontiguousarray(bias, np.float32)
    rc = lib().orc_qmm_tcg(_p(x1), _p(x2), M, K, N, int(tB), _p(x2s), s_dt, gs, _p(yscale), 0 if yscale is None else yscale.size,
                           _p(bias), y_dt, _p(y))
    assert rc == 0
    return y


def qmm_i4_asym(x1, x2, M, K, N, tB, x1s, x2s, x2o, y_dt):
    """int4 x int4 with per-256-K scales and fp16 offsets (compute_int4_asymmetrical)."""
    y = out_array((M, N), y_dt)
    x1s = np.ascontiguousarray(x1s, np.float32); x2s = np.ascontiguousarray(x2s, np.float32); x2o = np.ascontiguousarray(x2o, np.uint16)
    rc = lib().orc_qmm_i4_asym(_p(x1), _p(x2), M, K, N, int(tB), _p(x1s), _p(x2s), _p(x2o), y_dt, _p(y))
    assert rc == 0
    return y


def wqbmm(x, x_dt, w, w_dt, M, K, N, tW, scale, scale_dt, scale_n, offset, group, bias, bias_dt):
    y = np.empty((M, N), np.uint16)
    rc = lib().orc_wqbmm(_p(x), x_dt, _p(w), w_dt, M, K, N, int(tW), _p(scale), scale_dt, scale_n, _p(offset), group, _p(bias),
                         bias_dt, _p(y))
    assert rc == 0
    return y


def rel_err_stats(got_f32, want_f32, floor=None):
    """max and mean relative error with an absolute floor on the denominator."""
    got = np.asarray(got_f32, np.float64)
    want = np.asarray(want_f32, np.float64)
    if floor is None:
        floor = max(float(np.mean(np.abs(want))) * 1e-2, 1e-30)
    rel = np.abs(got - want) / np.maximum(np.abs(want), floor)
    return float(rel.max()), float(rel.mean())


def isclose_fraction(got_f32, want_f32, rtol=1e-3, atol=1e-3):
    """The reference's ST acceptance (matmul_golden_util.py:340-380): fraction of elements outside isclose."""
    ok = np.isclose(got_f32, want_f32, rtol=rtol, atol=atol, equal_nan=True)
    return 1.0 - ok.sum() / ok.size
