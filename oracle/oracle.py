"""ctypes/numpy front end of the CPU checker in intgemm8_oracle.c.

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke check and the cpu_baseline leg of
the benchmark.  The shipped HIP path never imports this module.

Tensor conventions follow Marian's intgemm8 types (reference src/common/types.cpp:32-34,
src/tensors/cpu/integer_common.h:101-106): a quantized tensor is a flat int8 array of
``elements + 4`` bytes whose last four bytes hold the fp32 quantMult.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_intgemm8.so")
_lib = None


def build(force=False):
    """Compile the checker with gcc (no reference sources are involved)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-s", "-B", "liboracle_intgemm8.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        c = ctypes
        fp, i8p, i32p, u32p = (c.POINTER(c.c_float), c.POINTER(c.c_int8),
                               c.POINTER(c.c_int32), c.POINTER(c.c_uint32))
        L.oracle_max_abs.restype = c.c_float
        L.oracle_max_abs.argtypes = [fp, c.c_size_t]
        L.oracle_quant_mult.restype = c.c_float
        L.oracle_quant_mult.argtypes = [c.c_float]
        L.oracle_unquant_mult.restype = c.c_float
        L.oracle_unquant_mult.argtypes = [c.c_float, c.c_float, c.c_float]
        L.oracle_quantize.restype = None
        L.oracle_quantize.argtypes = [fp, i8p, c.c_float, c.c_size_t]
        L.oracle_prepare_a.restype = None
        L.oracle_prepare_a.argtypes = [fp, i8p, c.c_int64, c.c_int64]
        L.oracle_prepare_b.restype = None
        L.oracle_prepare_b.argtypes = [fp, i8p, c.c_int64, c.c_int64]
        for name in ("oracle_multiply_i32", "oracle_multiply_i32_scalar"):
            f = getattr(L, name)
            f.restype = None
            f.argtypes = [i8p, i8p, i32p, c.c_int64, c.c_int64, c.c_int64]
        L.oracle_unquantize.restype = None
        L.oracle_unquantize.argtypes = [i32p, c.c_float, fp, c.c_int, fp, c.c_int64, c.c_int64]
        L.oracle_affine.restype = None
        L.oracle_affine.argtypes = [i8p, i8p, fp, fp, i32p, i32p, c.c_int64, c.c_int64,
                                    c.c_int64, c.c_float, c.c_int]
        L.oracle_affine_shortlist.restype = None
        L.oracle_affine_shortlist.argtypes = [i8p, i8p, fp, u32p, c.c_int64, fp, i32p,
                                              c.c_int64, c.c_int64, c.c_int64, c.c_float,
                                              c.c_int]
        L.oracle_affine_f32.restype = None
        L.oracle_affine_f32.argtypes = [fp, i8p, fp, fp, i8p, i32p, c.c_int64, c.c_int64,
                                        c.c_int64, c.c_float, c.c_int]
        L.oracle_has_vnni.restype = c.c_int
        L.oracle_has_vnni.argtypes = []
        _lib = L
    return _lib


def _p(a, ty):
    return a.ctypes.data_as(ctypes.POINTER(ty)) if a is not None else None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def max_abs(x):
    x = _f32(x).ravel()
    return float(lib().oracle_max_abs(_p(x, ctypes.c_float), x.size))


def quant_mult(maxabs):
    return np.float32(lib().oracle_quant_mult(np.float32(maxabs)))


def unquant_mult(aqm, bqm, scale=1.0):
    return np.float32(lib().oracle_unquant_mult(np.float32(aqm), np.float32(bqm),
                                                np.float32(scale)))


def quantize(x, qm):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.int8)
    lib().oracle_quantize(_p(x, ctypes.c_float), _p(out, ctypes.c_int8), np.float32(qm), x.size)
    return out


def tail(q, elements):
    """fp32 quantMult stored after `elements` int8 values."""
    return q[elements:elements + 4].view(np.float32)[0]


def prepare_a(A):
    """A fp32 [M, K] -> flat int8 [M*K + 4] (payload + quantMult tail)."""
    A = _f32(A)
    K = A.shape[-1]
    M = A.size // K
    out = np.zeros(M * K + 4, dtype=np.int8)
    lib().oracle_prepare_a(_p(A, ctypes.c_float), _p(out, ctypes.c_int8), M, K)
    return out


def prepare_b(W):
    """W fp32 [K, N] -> flat int8 [N*K + 4]: quantized transpose [N, K] + quantMult tail."""
    W = _f32(W)
    K, N = W.shape
    out = np.zeros(K * N + 4, dtype=np.int8)
    lib().oracle_prepare_b(_p(W, ctypes.c_float), _p(out, ctypes.c_int8), K, N)
    return out


def multiply_i32(Aq, Bq, M, K, N, scalar=False):
    acc = np.empty((M, N), dtype=np.int32)
    f = lib().oracle_multiply_i32_scalar if scalar else lib().oracle_multiply_i32
    f(_p(Aq, ctypes.c_int8), _p(Bq, ctypes.c_int8), _p(acc, ctypes.c_int32), M, K, N)
    return acc


def unquantize(acc, unquant, bias=None, relu=False):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    M, N = acc.shape
    b = _f32(bias).ravel() if bias is not None else None
    out = np.empty((M, N), dtype=np.float32)
    lib().oracle_unquantize(_p(acc, ctypes.c_int32), np.float32(unquant),
                            _p(b, ctypes.c_float), int(relu), _p(out, ctypes.c_float), M, N)
    return out


def affine(Aq, Bq, bias, M, K, N, scale=1.0, relu=False):
    """Returns (out fp32 [M,N], acc int32 [M,N]) for quantized operands with tails."""
    b = _f32(bias).ravel() if bias is not None else None
    out = np.empty((M, N), dtype=np.float32)
    acc = np.empty((M, N), dtype=np.int32)
    lib().oracle_affine(_p(Aq, ctypes.c_int8), _p(Bq, ctypes.c_int8), _p(b, ctypes.c_float),
                        _p(out, ctypes.c_float), _p(acc, ctypes.c_int32), None, M, K, N,
                        np.float32(scale), int(relu))
    return out, acc


def affine_shortlist(Aq, Bq, bias, idx, M, K, N, scale=1.0, relu=False):
    idx = np.ascontiguousarray(idx, dtype=np.uint32)
    b = _f32(bias).ravel() if bias is not None else None
    n_idx = idx.size
    out = np.empty((M, n_idx), dtype=np.float32)
    acc = np.empty((M, n_idx), dtype=np.int32)
    lib().oracle_affine_shortlist(_p(Aq, ctypes.c_int8), _p(Bq, ctypes.c_int8),
                                  _p(b, ctypes.c_float), _p(idx, ctypes.c_uint32), n_idx,
                                  _p(out, ctypes.c_float), _p(acc, ctypes.c_int32), M, K, N,
                                  np.float32(scale), int(relu))
    return out, acc


class AffineF32:
    """Reusable scratch for timing the whole CPU sequence (prepareA + multiply + ReLU)."""

    def __init__(self, M, K, N):
        self.M, self.K, self.N = M, K, N
        self.Aq = np.zeros(M * K + 4, dtype=np.int8)
        self.acc = np.empty((M, N), dtype=np.int32)
        self.out = np.empty((M, N), dtype=np.float32)

    def __call__(self, A, Bq, bias, scale=1.0, relu=False):
        b = _f32(bias).ravel() if bias is not None else None
        A = _f32(A)
        lib().oracle_affine_f32(_p(A, ctypes.c_float), _p(Bq, ctypes.c_int8),
                                _p(b, ctypes.c_float), _p(self.out, ctypes.c_float),
                                _p(self.Aq, ctypes.c_int8), _p(self.acc, ctypes.c_int32),
                                self.M, self.K, self.N, np.float32(scale), int(relu))
        return self.out


def has_vnni():
    return bool(lib().oracle_has_vnni())
