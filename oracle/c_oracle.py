"""ctypes face of oracle_c.c (test infrastructure only).

Builds `oracle/_build/liboracle_c.so` with the Makefile beside this file when
it is missing, then exposes NumPy-friendly wrappers.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "liboracle_c.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "all"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        u8p, u16p = ctypes.POINTER(ctypes.c_uint8), ctypes.POINTER(ctypes.c_uint16)
        i64, ci = ctypes.c_int64, ctypes.c_int
        L.matgptq_oracle_slice.argtypes = [u8p, u8p, i64, ci, ci]
        L.matgptq_oracle_slice.restype = None
        L.matgptq_oracle_dequantize.argtypes = [u8p, u16p, u16p, u16p, i64, i64, ci, ci, ci]
        L.matgptq_oracle_dequantize.restype = None
        L.matgptq_oracle_linear.argtypes = [u16p, u16p, u16p, i64, i64, i64]
        L.matgptq_oracle_linear.restype = None
        L.matgptq_oracle_forward.argtypes = [u8p, u16p, u16p, u16p, u16p, i64, i64, i64, ci, ci, ci]
        L.matgptq_oracle_forward.restype = None
        L.matgptq_oracle_f64_to_f16.argtypes = [ctypes.c_double]
        L.matgptq_oracle_f64_to_f16.restype = ctypes.c_uint16
        L.matgptq_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.matgptq_oracle_f16_to_f32.restype = ctypes.c_float
        _lib = L
    return _lib


def _p8(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8))


def _p16(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16))


def slice_codes(q: np.ndarray, slice_bits: int, master_bits: int = 8) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.uint8)
    out = np.empty_like(q)
    lib().matgptq_oracle_slice(_p8(q), _p8(out), q.size, slice_bits, master_bits)
    return out


def dequantize(q, scale, zero, slice_bits, group_size, master_bits: int = 8) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.uint8)
    n, k = q.shape
    s = np.ascontiguousarray(scale, dtype=np.float16).view(np.uint16)
    z = np.ascontiguousarray(zero, dtype=np.float16).view(np.uint16)
    w = np.empty((n, k), dtype=np.uint16)
    lib().matgptq_oracle_dequantize(_p8(q), _p16(s), _p16(z), _p16(w), n, k, group_size,
                                    slice_bits, master_bits)
    return w.view(np.float16)


def forward(x, q, scale, zero, slice_bits, group_size, master_bits: int = 8) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.uint8)
    n, k = q.shape
    x = np.ascontiguousarray(x, dtype=np.float16)
    m = x.shape[0]
    s = np.ascontiguousarray(scale, dtype=np.float16).view(np.uint16)
    z = np.ascontiguousarray(zero, dtype=np.float16).view(np.uint16)
    y = np.empty((m, n), dtype=np.uint16)
    lib().matgptq_oracle_forward(_p8(q), _p16(s), _p16(z), _p16(x.view(np.uint16)), _p16(y),
                                 m, n, k, group_size, slice_bits, master_bits)
    return y.view(np.float16)
