"""ctypes front end of oracle/w4a16_oracle.c (test infrastructure: see that file's header).

``load()`` returns the library, building it with ``make -C oracle`` if the shared object is
missing.  The array helpers take and return numpy arrays (fp16 as ``np.float16``).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libw4a16_oracle.so")
_lib = None

_P = ctypes.c_void_p
_I64 = ctypes.c_int64


def build() -> str:
    subprocess.check_call(["make", "-C", _HERE, "-s", "-B"])
    return _SO


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        lib = ctypes.CDLL(_SO)
        lib.oracle_h2f.restype = ctypes.c_float
        lib.oracle_h2f.argtypes = [ctypes.c_uint16]
        lib.oracle_f2h.restype = ctypes.c_uint16
        lib.oracle_f2h.argtypes = [ctypes.c_float]
        lib.oracle_unpack_u4.argtypes = [_P, _I64, _I64, _I64, _P]
        for name in ("oracle_gemv_f32acc", "oracle_gemm_deq_f32acc", "oracle_linear_f64"):
            getattr(lib, name).argtypes = [_P, _P, _P, _P, _P, _I64, _I64, _I64, ctypes.c_int, _I64, _I64, _I64]
        lib.oracle_dequant_f16.argtypes = [_P, _P, _P, _P, _I64, _I64, ctypes.c_int, _I64, _I64, _I64]
        lib.oracle_shared_proj.argtypes = [_P, _P, _P, _I64, _I64, _I64]
        lib.oracle_add_correction.argtypes = [_P, _P, _P, ctypes.c_float, _I64, _I64, _I64]
        _lib = lib
    return _lib


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def _ptr(a):
    return a.ctypes.data_as(_P)


def dequant(qweight, scales, qzeros, K: int, group_size: int) -> np.ndarray:
    lib = load()
    qw, sc, qz = _c(qweight, np.int32), _c(scales, np.float16), _c(qzeros, np.int32)
    N = qw.shape[0]
    out = np.empty((N, K), dtype=np.float16)
    lib.oracle_dequant_f16(_ptr(qw), _ptr(sc), _ptr(qz), _ptr(out), N, K, group_size, qw.shape[1], sc.shape[1], qz.shape[1])
    return out


def _linear(fn, out_dtype, x, qweight, scales, qzeros, group_size):
    lib = load()
    x = _c(x, np.float16)
    qw, sc, qz = _c(qweight, np.int32), _c(scales, np.float16), _c(qzeros, np.int32)
    M, K = x.shape
    N = qw.shape[0]
    y = np.empty((M, N), dtype=out_dtype)
    getattr(lib, fn)(_ptr(x), _ptr(qw), _ptr(sc), _ptr(qz), _ptr(y), M, K, N, group_size, qw.shape[1], sc.shape[1], qz.shape[1])
    return y


def gemv_f32acc(x, qweight, scales, qzeros, group_size):
    return _linear("oracle_gemv_f32acc", np.float16, x, qweight, scales, qzeros, group_size)


def gemm_deq_f32acc(x, qweight, scales, qzeros, group_size):
    return _linear("oracle_gemm_deq_f32acc", np.float16, x, qweight, scales, qzeros, group_size)


def linear_f64(x, qweight, scales, qzeros, group_size):
    return _linear("oracle_linear_f64", np.float64, x, qweight, scales, qzeros, group_size)


def shared_proj(x, R) -> np.ndarray:
    lib = load()
    x, R = _c(x, np.float16), _c(R, np.float16)
    M, K = x.shape
    rank = R.shape[0]
    r = np.empty((M, rank), dtype=np.float16)
    lib.oracle_shared_proj(_ptr(x), _ptr(R), _ptr(r), M, K, rank)
    return r


def add_correction(z, r, L, alpha: float) -> np.ndarray:
    lib = load()
    z = np.array(z, dtype=np.float16, order="C", copy=True)
    r, L = _c(r, np.float16), _c(L, np.float16)
    M, N = z.shape
    lib.oracle_add_correction(_ptr(z), _ptr(r), _ptr(L), alpha, M, N, r.shape[1])
    return z
