"""ctypes access to oracle/kernels_ref.c.  TEST INFRASTRUCTURE ONLY."""

import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "liboracle_kernels.so")
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            raise RuntimeError(f"{LIB} not built: make -C oracle")
        _lib = ctypes.CDLL(LIB)
        _lib.oracle_triad_f32.argtypes = [ctypes.c_void_p, ctypes.c_void_p,
                                          ctypes.c_void_p, ctypes.c_float,
                                          ctypes.c_size_t]
        _lib.oracle_gemm_bf16_nt.argtypes = [ctypes.c_void_p, ctypes.c_void_p,
                                             ctypes.c_void_p] + [ctypes.c_int] * 5
        _lib.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib.oracle_f32_to_bf16.restype = ctypes.c_uint16
    return _lib


def triad(b, c, s):
    b = np.ascontiguousarray(b, dtype=np.float32)
    c = np.ascontiguousarray(c, dtype=np.float32)
    a = np.empty_like(b)
    lib().oracle_triad_f32(a.ctypes.data, b.ctypes.data, c.ctypes.data,
                           ctypes.c_float(s), b.size)
    return a


def gemm_bf16_nt(a_bits, b_bits, row_begin=0, row_end=None):
    """a_bits[M,K], b_bits[N,K]: uint16 bf16 patterns -> float64 rows."""
    a_bits = np.ascontiguousarray(a_bits, dtype=np.uint16)
    b_bits = np.ascontiguousarray(b_bits, dtype=np.uint16)
    m, k = a_bits.shape
    n = b_bits.shape[0]
    row_end = m if row_end is None else row_end
    out = np.empty((row_end - row_begin, n), dtype=np.float64)
    lib().oracle_gemm_bf16_nt(a_bits.ctypes.data, b_bits.ctypes.data,
                              out.ctypes.data, m, n, k, row_begin, row_end)
    return out


def f32_to_bf16_bits(x):
    """Round-to-nearest-even fp32 -> bf16 bit patterns (numpy restatement)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7fffffff) > 0x7f800000
    r = (u + 0x7fff + ((u >> 16) & 1)) >> 16
    r = np.where(nan, (u >> 16) | 0x40, r)
    return r.astype(np.uint16)


def bf16_bits_to_f32(bits):
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
