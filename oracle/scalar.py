"""ctypes loader for oracle/ref_scalar.c (test infrastructure only)."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

from . import mx_oracle as mo

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_scalar.so")
_lib = None


def build(force: bool = False) -> str:
    if force:
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle_scalar.so"], stdout=subprocess.DEVNULL)
    elif not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "liboracle_scalar.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        _lib.orc_f32_to_exmy.restype = ctypes.c_uint8
        _lib.orc_f32_to_exmy.argtypes = [ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_float]
        _lib.orc_scale_exponent.restype = ctypes.c_int
        _lib.orc_scale_exponent.argtypes = [ctypes.c_float, ctypes.c_float]
        p = ctypes.c_void_p
        for fn in (_lib.orc_quantize_x, _lib.orc_quantize_w):
            fn.restype = None
            fn.argtypes = [p, p] + [ctypes.c_int] * 5 + [p] * 6
    return _lib


def f32_to_exmy(v: float, fmt: str) -> int:
    ebits, mbits, bias, maxv = mo.FORMATS[fmt]
    return int(lib().orc_f32_to_exmy(float(v), ebits, mbits, bias, maxv))


def scale_exponent(amax: float, fmt: str) -> int:
    return int(lib().orc_scale_exponent(float(amax), mo.FORMATS[fmt][3]))


def _quantize(fn, operand, x_bits: np.ndarray, idx: np.ndarray, kn: int, ks: int, ko: int) -> dict:
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    idx = np.ascontiguousarray(idx, dtype=np.int16)
    rows, k = x_bits.shape
    assert k == kn + ks + ko and idx.shape == (k,)
    w = operand == "b"
    out = {
        "qn": np.zeros((rows, kn // 2), np.uint8),
        "qs": np.zeros((rows, ks // 2 if w else ks // 4 * 3), np.uint8),
        "qo": np.zeros((rows, ko // 2 if w else ko), np.uint8),
        "sfn": np.zeros(mo.sf_bytes(rows, kn, operand), np.uint8),
        "sfs": np.zeros(mo.sf_bytes(rows, ks, operand), np.uint8),
        "sfo": np.zeros(mo.sf_bytes(rows, ko, operand), np.uint8),
    }
    ptr = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    fn(ptr(x_bits), ptr(idx), rows, k, kn, ks, ko,
       *(ptr(out[n]) for n in ("qn", "qs", "qo", "sfn", "sfs", "sfo")))
    return out


def quantize_x(x_bits, idx, kn, ks, ko) -> dict:
    """x_bits: uint16 [M, K] bf16 bit patterns."""
    return _quantize(lib().orc_quantize_x, "a", x_bits, idx, kn, ks, ko)


def quantize_w(w_bits, idx, kn, ks, ko) -> dict:
    return _quantize(lib().orc_quantize_w, "b", w_bits, idx, kn, ks, ko)
