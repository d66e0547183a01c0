"""ctypes front-end to the plain-C oracle (oracle/duq_oracle.c).

TEST INFRASTRUCTURE ONLY.  Arrays go in and out as NumPy; binary16 travels as uint16
bit patterns (``arr.view(np.uint16)``).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libduq_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile oracle/duq_oracle.c with gcc (see oracle/Makefile)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.duqo_h2f.restype = ctypes.c_float
        _lib.duqo_h2f.argtypes = [ctypes.c_uint16]
        _lib.duqo_f2h.restype = ctypes.c_uint16
        _lib.duqo_f2h.argtypes = [ctypes.c_float]
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _h(a):
    a = np.ascontiguousarray(np.asarray(a, dtype=np.float16))
    return a


def _u32(v):
    return ctypes.c_uint32(int(v))


def sym_scales(x, clip=1.0):
    x = _h(x)
    rows, cols = x.shape
    s = np.empty((rows, 1), np.float16)
    lib().duqo_sym_scales(_p(x), _u32(rows), _u32(cols), ctypes.c_float(clip), _p(s))
    return s


def asym_scales_zeros(x):
    x = _h(x)
    rows, cols = x.shape
    s = np.empty((rows, 1), np.float16)
    z = np.empty((rows, 1), np.float16)
    lib().duqo_asym_scales_zeros(_p(x), _u32(rows), _u32(cols), _p(s), _p(z))
    return s, z


def sym_quant(x, scale, qmax=6):
    x = _h(x)
    scale = _h(scale).reshape(-1)
    rows, cols = x.shape
    cd = (cols + 1) // 2
    q = np.empty((rows, cd), np.uint8)
    lib().duqo_sym_quant(_p(x), _p(scale), _u32(rows), _u32(cols), _u32(cd), ctypes.c_int32(qmax), _p(q))
    return q


def sym_dual_quant(x, s1, s2, qmax=6):
    x = _h(x)
    s1 = _h(s1).reshape(-1)
    s2 = _h(s2).reshape(-1)
    rows, cols = x.shape
    cd = (cols + 1) // 2
    q = np.empty((rows, cd), np.uint8)
    lib().duqo_sym_dual_quant(_p(x), _p(s1), _p(s2), _u32(rows), _u32(cols), _u32(cd), ctypes.c_int32(qmax), _p(q))
    return q


def asym_quant(x, scale, zero):
    x = _h(x)
    scale = _h(scale).reshape(-1)
    zero = _h(zero).reshape(-1)
    rows, cols = x.shape
    cd = (cols + 1) // 2
    q = np.empty((rows, cd), np.uint8)
    lib().duqo_asym_quant(_p(x), _p(scale), _p(zero), _u32(rows), _u32(cols), _u32(cd), _p(q))
    return q


def asym_dual_quant(x, s1, z1, s2, z2):
    x = _h(x)
    s1, z1, s2, z2 = (_h(v).reshape(-1) for v in (s1, z1, s2, z2))
    rows, cols = x.shape
    cd = (cols + 1) // 2
    q = np.empty((rows, cd), np.uint8)
    lib().duqo_asym_dual_quant(_p(x), _p(s1), _p(z1), _p(s2), _p(z2), _u32(rows), _u32(cols), _u32(cd), _p(q))
    return q


def matmul_s4(a, b):
    a = np.ascontiguousarray(a, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.uint8)
    m, kb = a.shape
    n = b.shape[0]
    assert b.shape[1] == kb
    c = np.empty((m, n), np.int32)
    lib().duqo_matmul_s4(_p(a), _p(b), _u32(m), _u32(n), _u32(kb * 2), _p(c))
    return c


def sym_dequant(acc, sr, sc):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    sr = _h(sr).reshape(-1)
    sc = _h(sc).reshape(-1)
    rows, cols = acc.shape
    y = np.empty((rows, cols), np.float16)
    lib().duqo_sym_dequant(_p(acc), _p(sr), _p(sc), _u32(rows), _u32(cols), _p(y))
    return y


def sym_dual_dequant(acc, sr, sc1, sc2):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    sr, sc1, sc2 = (_h(v).reshape(-1) for v in (sr, sc1, sc2))
    rows, cols = acc.shape
    y = np.empty((rows, cols), np.float16)
    lib().duqo_sym_dual_dequant(_p(acc), _p(sr), _p(sc1), _p(sc2), _u32(rows), _u32(cols), _p(y))
    return y


def asym_dequant(acc, sr, zr, sc, zc):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    sr, zr, sc, zc = (_h(v).reshape(-1) for v in (sr, zr, sc, zc))
    rows, cols = acc.shape
    y = np.empty((rows, cols), np.float16)
    lib().duqo_asym_dequant(_p(acc), _p(sr), _p(zr), _p(sc), _p(zc), _u32(rows), _u32(cols), _p(y))
    return y


def asym_dual_dequant(acc, sr, zr, sc1, zc1, sc2, zc2):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    sr, zr, sc1, zc1, sc2, zc2 = (_h(v).reshape(-1) for v in (sr, zr, sc1, zc1, sc2, zc2))
    rows, cols = acc.shape
    y = np.empty((rows, cols), np.float16)
    lib().duqo_asym_dual_dequant(_p(acc), _p(sr), _p(zr), _p(sc1), _p(zc1), _p(sc2), _p(zc2), _u32(rows), _u32(cols), _p(y))
    return y


def add_bias(y, bias):
    y = np.array(_h(y), copy=True)
    bias = _h(bias).reshape(-1)
    rows, cols = y.shape
    lib().duqo_add_bias(_p(y), _p(bias), _u32(rows), _u32(cols))
    return y


# ---- 8-bit asymmetric layer ------------------------------------------------------------------

def _f32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def asym8_scales_zeros(x, device_division=True):
    x = _f32(x)
    rows, cols = x.shape
    s = np.empty((rows, 1), np.float32)
    z = np.empty((rows, 1), np.float32)
    lib().duqo_asym8_scales_zeros(_p(x), _u32(rows), _u32(cols), ctypes.c_int(1 if device_division else 0), _p(s), _p(z))
    return s, z


def asym_quant_8bit(x, scale, zeros):
    x = _f32(x)
    scale, zeros = _f32(scale).reshape(-1), _f32(zeros).reshape(-1)
    rows, cols = x.shape
    q = np.empty((rows, cols), np.int8)
    lib().duqo_asym_quant_8bit(_p(x), _p(scale), _p(zeros), _u32(rows), _u32(cols), _p(q))
    return q


def matmul_s8(a, b):
    a = np.ascontiguousarray(a, dtype=np.int8)
    b = np.ascontiguousarray(b, dtype=np.int8)
    c = np.empty((a.shape[0], b.shape[0]), np.int32)
    lib().duqo_matmul_s8(_p(a), _p(b), _u32(a.shape[0]), _u32(b.shape[0]), _u32(a.shape[1]), _p(c))
    return c


def asym_dequant_hprec(acc, sr, zr, sc, zc):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    sr, zr, sc, zc = (_f32(v).reshape(-1) for v in (sr, zr, sc, zc))
    rows, cols = acc.shape
    y = np.empty((rows, cols), np.float32)
    lib().duqo_asym_dequant_hprec(_p(acc), _p(sr), _p(zr), _p(sc), _p(zc), _u32(rows), _u32(cols), _p(y))
    return y
