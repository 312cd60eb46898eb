"""ctypes access to the C restatement in ``hqq_oracle.c`` (test infrastructure).

Loads ``oracle/_build/libhqq_oracle.so``; ``build()`` runs the Makefile."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libhqq_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "hqq_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "_build/libhqq_oracle.so"], stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.oracle_h2f.restype = ctypes.c_float
        _lib.oracle_h2f.argtypes = [ctypes.c_uint16]
        _lib.oracle_f2h.restype = ctypes.c_uint16
        _lib.oracle_f2h.argtypes = [ctypes.c_float]
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _i64(v):
    return ctypes.c_int64(int(v))


def pack(q: np.ndarray, nbits: int) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.uint8)
    h, w = q.shape
    if nbits == 4:
        out = np.empty((h // 2, w), np.uint8)
        lib().oracle_pack_4bit_u8(_p(q), _i64(h), _i64(w), _p(out))
    elif nbits == 2:
        out = np.empty((h // 4, w), np.uint8)
        lib().oracle_pack_2bit_u8(_p(q), _i64(h), _i64(w), _p(out))
    else:
        out = np.empty(((h + 9) // 10, w), np.int32)
        lib().oracle_pack_3bit_i32(_p(q), _i64(h), _i64(w), _p(out))
    return out


def unpack(p: np.ndarray, nbits: int) -> np.ndarray:
    p = np.ascontiguousarray(p)
    hp, w = p.shape
    f = {4: 2, 2: 4, 3: 10}[nbits]
    out = np.empty((hp * f, w), np.uint8)
    fn = {4: "oracle_unpack_4bit_u8", 2: "oracle_unpack_2bit_u8", 3: "oracle_unpack_3bit_i32"}[nbits]
    getattr(lib(), fn)(_p(p), _i64(hp), _i64(w), _p(out))
    return out


def meta_dequant(q: np.ndarray, ms, mz) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.uint8)
    rows, cols = q.shape
    ms = np.ascontiguousarray(np.asarray(ms, dtype=np.float16).reshape(-1))
    mz = np.ascontiguousarray(np.asarray(mz, dtype=np.float16).reshape(-1))
    scalar = int(ms.size == 1)
    assert scalar or ms.size == cols
    out = np.empty((rows, cols), np.float16)
    lib().oracle_meta_dequant(_p(q), _i64(rows), _i64(cols), _p(ms), _p(mz), ctypes.c_int(scalar), _p(out))
    return out


def dequantize(codes: np.ndarray, nbits: int, n: int, k: int, gs: int, scale: np.ndarray, zero: np.ndarray) -> np.ndarray:
    codes = np.ascontiguousarray(codes)
    scale = np.ascontiguousarray(scale, dtype=np.float16)
    zero = np.ascontiguousarray(zero, dtype=np.float16)
    out = np.empty((n, k), np.float16)
    lib().oracle_dequantize(_p(codes), ctypes.c_int(nbits), _i64(n), _i64(k), _i64(gs), _p(scale), _p(zero), _p(out))
    return out


def matmul_transpose(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float16)
    w = np.ascontiguousarray(w, dtype=np.float16)
    m, k = x.shape
    n = w.shape[0]
    y = np.empty((m, n), np.float16)
    lib().oracle_matmul_transpose(_p(x), _i64(m), _p(w), _i64(n), _i64(k), _p(y))
    return y
