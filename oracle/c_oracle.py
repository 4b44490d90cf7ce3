"""ctypes view of gemm_oracle.c (test infrastructure). `load()` builds the library on first use."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build() -> str:
    subprocess.check_call(['make', '-s', '-C', _HERE, 'liboracle.so'])
    return os.path.join(_HERE, 'liboracle.so')


def load():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, 'liboracle.so')
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
    return _LIB


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def gemm_bf16_tn(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    a_bits, b_bits = np.ascontiguousarray(a_bits, np.uint16), np.ascontiguousarray(b_bits, np.uint16)
    (m, k), n = a_bits.shape, b_bits.shape[0]
    c = np.empty((m, n), np.float64)
    load().oracle_gemm_bf16_tn(ctypes.c_int(m), ctypes.c_int(n), ctypes.c_int(k), _ptr(a_bits), _ptr(b_bits), _ptr(c))
    return c


def gemm_fp8_nt(a: np.ndarray, sa: np.ndarray, b: np.ndarray, sb: np.ndarray) -> np.ndarray:
    a, b = np.ascontiguousarray(a, np.uint8), np.ascontiguousarray(b, np.uint8)
    sa, sb = np.asarray(sa, np.float32), np.ascontiguousarray(sb, np.float32)
    (m, k), n = a.shape, b.shape[0]
    c = np.empty((m, n), np.float64)
    load().oracle_gemm_fp8_nt(ctypes.c_int(m), ctypes.c_int(n), ctypes.c_int(k), _ptr(a), _ptr(sa),
                              ctypes.c_long(sa.strides[0] // 4), ctypes.c_long(sa.strides[1] // 4),
                              _ptr(b), _ptr(sb), _ptr(c))
    return c


def gemm_float_nt(m: int, n: int, k: int, alpha: float, a_buf: np.ndarray, lda: int, b_buf: np.ndarray, ldb: int,
                  beta: float, c_buf: np.ndarray, ldc: int) -> np.ndarray:
    """Raw fp32 buffers in the C-ABI's memory convention; returns a float64 buffer shaped like `c_buf` (elements
    outside the m x n window are left as zeros)."""
    a_buf, b_buf = np.ascontiguousarray(a_buf, np.float32).ravel(), np.ascontiguousarray(b_buf, np.float32).ravel()
    c_in = np.ascontiguousarray(c_buf, np.float32).ravel()
    assert a_buf.size >= (k - 1) * lda + m and b_buf.size >= (k - 1) * ldb + n and c_in.size >= (m - 1) * ldc + n
    c_out = np.zeros(c_in.size, np.float64)
    load().oracle_gemm_float_nt(ctypes.c_int(m), ctypes.c_int(n), ctypes.c_int(k), ctypes.c_double(alpha), _ptr(a_buf),
                                ctypes.c_int(lda), _ptr(b_buf), ctypes.c_int(ldb), ctypes.c_double(beta), _ptr(c_in),
                                _ptr(c_out), ctypes.c_int(ldc))
    return c_out
