"""ctypes loader of oracle/_build/libhfrk_oracle.so (built from oracle/c/hfrk_oracle.c by its Makefile).
Test infrastructure only (see __init__.py)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_build", "libhfrk_oracle.so")
_lib = None


def build():
    subprocess.run(["make", "-C", os.path.join(_HERE, "c")], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return LIB_PATH


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        lib = ctypes.CDLL(LIB_PATH)
        lib.hfrk_oracle_decode_e4m3fn.restype = ctypes.c_double
        lib.hfrk_oracle_decode_e4m3fn.argtypes = [ctypes.c_uint8]
        lib.hfrk_oracle_encode_e4m3fn.restype = ctypes.c_uint8
        lib.hfrk_oracle_encode_e4m3fn.argtypes = [ctypes.c_double]
        p = ctypes.c_void_p
        i = ctypes.c_int
        lib.hfrk_oracle_gemm_int.restype = None
        lib.hfrk_oracle_gemm_int.argtypes = [p, p, i, i, i, i, p]
        lib.hfrk_oracle_gemm_f32.restype = None
        lib.hfrk_oracle_gemm_f32.argtypes = [p, p, p, i, p, i, p, i, i, i, i, p]
        lib.hfrk_oracle_rms_row.restype = None
        lib.hfrk_oracle_rms_row.argtypes = [p, p, ctypes.c_double, i, p]
        lib.hfrk_oracle_swiglu.restype = None
        lib.hfrk_oracle_swiglu.argtypes = [p, i, i, p]
        _lib = lib
    return _lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def gemm_int(a_codes: np.ndarray, w_codes: np.ndarray) -> np.ndarray:
    """a_codes [m,k] uint8, w_codes [n,k] uint8 -> exact int64 [m,n] dot products in units of 2^-18."""
    a = np.ascontiguousarray(a_codes, dtype=np.uint8)
    w = np.ascontiguousarray(w_codes, dtype=np.uint8)
    m, k = a.shape
    n = w.shape[0]
    out = np.empty((m, n), dtype=np.int64)
    load().hfrk_oracle_gemm_int(_ptr(a), _ptr(w), m, n, k, k, _ptr(out))
    return out


def gemm_f32(a_codes, w_codes, sa, sw, bias=None) -> np.ndarray:
    a = np.ascontiguousarray(a_codes, dtype=np.uint8)
    w = np.ascontiguousarray(w_codes, dtype=np.uint8)
    m, k = a.shape
    n = w.shape[0]
    sa = np.ascontiguousarray(np.asarray(sa, dtype=np.float32).reshape(-1))
    sw = np.ascontiguousarray(np.asarray(sw, dtype=np.float32).reshape(-1))
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    out = np.empty((m, n), dtype=np.float32)
    load().hfrk_oracle_gemm_f32(_ptr(a), _ptr(w), _ptr(sa), 0 if sa.size == 1 else 1, _ptr(sw), 0 if sw.size == 1 else 1,
                                None if b is None else _ptr(b), m, n, k, k, _ptr(out))
    return out


def rms_row(z: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    z = np.ascontiguousarray(z, dtype=np.float64)
    w = np.ascontiguousarray(w, dtype=np.float64)
    y = np.empty_like(z)
    load().hfrk_oracle_rms_row(_ptr(z), _ptr(w), float(eps), z.size, _ptr(y))
    return y


def swiglu(gate_up: np.ndarray) -> np.ndarray:
    gu = np.ascontiguousarray(gate_up, dtype=np.float64)
    rows, two_n = gu.shape
    out = np.empty((rows, two_n // 2), dtype=np.float64)
    load().hfrk_oracle_swiglu(_ptr(gu), rows, two_n // 2, _ptr(out))
    return out
