"""ctypes/numpy front end of the CPU checker in intgemm16_oracle.c (Marian's 16-bit intgemm path).

TEST INFRASTRUCTURE ONLY: imported by tests/.  The shipped HIP path never imports this module.

A 16-bit quantized tensor (reference src/common/types.cpp:32-34, src/tensors/cpu/integer_common.h:
101-106) is `elements` int16 values followed by the fp32 quantMult: here a flat int16 array of
``elements + 2`` entries whose last two hold the bits of 1024.0f.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_intgemm16.so")
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            subprocess.check_call(["make", "-C", _HERE, "-s", "-B", "liboracle_intgemm16.so"])
        L = ctypes.CDLL(_LIB_PATH)
        c = ctypes
        fp, i16p, i32p = c.POINTER(c.c_float), c.POINTER(c.c_int16), c.POINTER(c.c_int32)
        L.oracle16_quant_mult.restype = c.c_float
        L.oracle16_quantize.restype = None
        L.oracle16_quantize.argtypes = [fp, i16p, c.c_float, c.c_size_t]
        L.oracle16_prepare_a.restype = None
        L.oracle16_prepare_a.argtypes = [fp, i16p, c.c_int64, c.c_int64]
        L.oracle16_prepare_b.restype = None
        L.oracle16_prepare_b.argtypes = [fp, i16p, c.c_int64, c.c_int64]
        L.oracle16_multiply_i32.restype = None
        L.oracle16_multiply_i32.argtypes = [i16p, i16p, i32p, c.c_int64, c.c_int64, c.c_int64]
        L.oracle16_affine.restype = None
        L.oracle16_affine.argtypes = [i16p, i16p, fp, fp, i32p, c.c_int64, c.c_int64, c.c_int64, c.c_float, c.c_int]
        _lib = L
    return _lib


def _p(a, ty):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(ty))


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def quantize(x, qm=1024.0):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.int16)
    lib().oracle16_quantize(_p(x, ctypes.c_float), _p(out, ctypes.c_int16), np.float32(qm), x.size)
    return out


def tail(q, elements):
    return q[elements:elements + 2].view(np.float32)[0]


def prepare_a(A):
    A = _f32(A)
    K = A.shape[-1]
    M = A.size // K
    out = np.zeros(M * K + 2, dtype=np.int16)
    lib().oracle16_prepare_a(_p(A, ctypes.c_float), _p(out, ctypes.c_int16), M, K)
    return out


def prepare_b(W):
    W = _f32(W)
    K, N = W.shape
    out = np.zeros(K * N + 2, dtype=np.int16)
    lib().oracle16_prepare_b(_p(W, ctypes.c_float), _p(out, ctypes.c_int16), K, N)
    return out


def multiply_i32(Aq, Bq, M, K, N):
    acc = np.empty((M, N), dtype=np.int32)
    lib().oracle16_multiply_i32(_p(Aq, ctypes.c_int16), _p(Bq, ctypes.c_int16), _p(acc, ctypes.c_int32), M, K, N)
    return acc


def affine(Aq, Bq, bias, M, K, N, scale=1.0, relu=False):
    """Returns (out fp32 [M, N], acc int32 [M, N]) for quantized operands with tails."""
    b = _f32(bias).ravel() if bias is not None else None
    out = np.empty((M, N), dtype=np.float32)
    acc = np.empty((M, N), dtype=np.int32)
    lib().oracle16_affine(_p(Aq, ctypes.c_int16), _p(Bq, ctypes.c_int16), _p(b, ctypes.c_float),
                          _p(out, ctypes.c_float), _p(acc, ctypes.c_int32), M, K, N, np.float32(scale), int(relu))
    return out, acc
