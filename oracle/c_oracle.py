"""ctypes front end of oracle/rtn_oracle.c (test infrastructure only).

build() runs oracle/Makefile; load() returns the library or raises.  The
wrappers take and return numpy arrays with the same conventions as
oracle/rtn_oracle.py so the two restatements can be compared directly.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "librtn_oracle.so")
_lib = None


def build():
    subprocess.run(["make", "-B", "-C", _HERE], check=True, capture_output=True)
    return _SO


def load():
    global _lib
    if _lib is None:
        src = os.path.join(_HERE, "rtn_oracle.c")
        if not os.path.exists(_SO) or (os.path.exists(src) and os.path.getmtime(src) > os.path.getmtime(_SO)):
            build()
        lib = ctypes.CDLL(_SO)
        i64, i32, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
        lib.orc_quantize_rtn_f32.argtypes = [vp, i64, i64, i32, i32, vp, vp, vp]
        lib.orc_quantize_rtn_f32_div.argtypes = [vp, i64, i64, i32, i32, i32, vp, vp, vp]
        lib.orc_quantize_rtn_f32_div.restype = ctypes.c_int
        lib.orc_dequantize_f32.argtypes = [vp, vp, vp, i64, i64, i32, i32, vp]
        lib.orc_dequantize_f16.argtypes = [vp, vp, vp, i64, i64, i32, i32, vp]
        lib.orc_qlinear_forward.argtypes = [vp, i64, i64, vp, vp, vp, vp, i64, i32, i32, vp]
        for f in (lib.orc_quantize_rtn_f32, lib.orc_dequantize_f32, lib.orc_dequantize_f16, lib.orc_qlinear_forward):
            f.restype = ctypes.c_int
        _lib = lib
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def quantize_rtn_f32(w, bits, group_size, scale_div="ieee"):
    w = np.ascontiguousarray(w, np.float32)
    n, k = w.shape
    qw = np.empty((n, k * bits // 32), np.int32)
    s = np.empty((n, k // group_size), np.float32)
    z = np.empty((n, k // group_size), np.int32)
    rc = load().orc_quantize_rtn_f32_div(_p(w), n, k, bits, group_size, int(scale_div == "reciprocal"), _p(qw), _p(s), _p(z))
    if rc:
        raise ValueError("orc_quantize_rtn_f32 rejected its arguments")
    return qw, s, z


def dequantize_f32(qweight, scale, zp, group_size, bits):
    qweight = np.ascontiguousarray(qweight, np.int32)
    n, words = qweight.shape
    k = words * 32 // bits
    s = np.ascontiguousarray(np.asarray(scale).astype(np.float32))
    z = np.ascontiguousarray(np.asarray(zp).astype(np.float32))
    w = np.empty((n, k), np.float32)
    rc = load().orc_dequantize_f32(_p(qweight), _p(s), _p(z), n, k, bits, group_size, _p(w))
    if rc:
        raise ValueError("orc_dequantize_f32 rejected its arguments")
    return w


def dequantize_f16(qweight, scale16, zp16, group_size, bits):
    qweight = np.ascontiguousarray(qweight, np.int32)
    n, words = qweight.shape
    k = words * 32 // bits
    s = np.ascontiguousarray(scale16, np.float16)
    z = np.ascontiguousarray(zp16, np.float16)
    w = np.empty((n, k), np.float16)
    rc = load().orc_dequantize_f16(_p(qweight), _p(s), _p(z), n, k, bits, group_size, _p(w))
    if rc:
        raise ValueError("orc_dequantize_f16 rejected its arguments")
    return w


def qlinear_forward(x16, qweight, scale16, zp16, bias16, bits, group_size):
    x16 = np.ascontiguousarray(x16, np.float16)
    m, k = x16.shape
    qweight = np.ascontiguousarray(qweight, np.int32)
    n = qweight.shape[0]
    s = np.ascontiguousarray(scale16, np.float16)
    z = np.ascontiguousarray(zp16, np.float16)
    b = None if bias16 is None else np.ascontiguousarray(bias16, np.float16)
    y = np.empty((m, n), np.float16)
    rc = load().orc_qlinear_forward(_p(x16), m, k, _p(qweight), _p(s), _p(z), None if b is None else _p(b), n,
                                    bits, group_size, _p(y))
    if rc:
        raise ValueError("orc_qlinear_forward rejected its arguments")
    return y
