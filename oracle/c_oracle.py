"""ctypes front end of oracle/gptq_oracle.c.  TEST INFRASTRUCTURE ONLY (see that file's header)."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libgptq_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "gptq_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libgptq_oracle.so"])
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.oracle_half_to_float.restype = ctypes.c_float
        _lib.oracle_half_to_float.argtypes = [ctypes.c_uint16]
        _lib.oracle_float_to_half.restype = ctypes.c_uint16
        _lib.oracle_float_to_half.argtypes = [ctypes.c_float]
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _i32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a), dtype=np.int32)


def _u16(a) -> np.ndarray:
    a = np.ascontiguousarray(np.asarray(a))
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    return np.ascontiguousarray(a, dtype=np.uint16)


def unpack_rows(qweight, bits: int) -> np.ndarray:
    qweight = _i32(qweight)
    k = qweight.shape[0] * 32 // bits
    n = qweight.shape[1]
    out = np.empty((k, n), dtype=np.int32)
    rc = lib().oracle_unpack_rows(_p(qweight), k, n, bits, _p(out))
    if rc != 0:
        raise ValueError(f"oracle_unpack_rows failed: {rc}")
    return out


def unpack_zeros(qzeros, bits: int) -> np.ndarray:
    qzeros = _i32(qzeros)
    g = qzeros.shape[0]
    n = qzeros.shape[1] * 32 // bits
    out = np.empty((g, n), dtype=np.int32)
    rc = lib().oracle_unpack_zeros(_p(qzeros), g, n, bits, _p(out))
    if rc != 0:
        raise ValueError(f"oracle_unpack_zeros failed: {rc}")
    return out


def dequant(qweight, qzeros, scales, g_idx, bits: int) -> np.ndarray:
    qweight, qzeros, scales, g_idx = _i32(qweight), _i32(qzeros), _u16(scales), _i32(g_idx)
    k = qweight.shape[0] * 32 // bits
    n = qweight.shape[1]
    g = scales.shape[0]
    out = np.empty((k, n), dtype=np.uint16)
    rc = lib().oracle_dequant(_p(qweight), _p(qzeros), _p(scales), _p(g_idx), k, n, g, bits, _p(out))
    if rc != 0:
        raise ValueError(f"oracle_dequant failed: {rc}")
    return out.view(np.float16)


def forward(x, qweight, qzeros, scales, g_idx, bias, bits: int) -> np.ndarray:
    x = _u16(x)
    x = x.reshape(-1, x.shape[-1])
    qweight, qzeros, scales, g_idx = _i32(qweight), _i32(qzeros), _u16(scales), _i32(g_idx)
    m, k = x.shape
    n = qweight.shape[1]
    g = scales.shape[0]
    b = _u16(bias) if bias is not None else None
    out = np.empty((m, n), dtype=np.float32)
    rc = lib().oracle_forward(_p(x), _p(qweight), _p(qzeros), _p(scales), _p(g_idx),
                              _p(b) if b is not None else None, m, k, n, g, bits, _p(out))
    if rc != 0:
        raise ValueError(f"oracle_forward failed: {rc}")
    return out
