"""ctypes/numpy front end of the CPU checker in decode_ops_oracle.c.

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke check and the cpu_baseline leg of the
benchmark.  The shipped HIP path never imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_decode_ops.so")
_lib = None


def build(force=False):
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-s", "-B", "liboracle_decode_ops.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        c = ctypes
        fp, i64 = c.POINTER(c.c_float), c.c_int64
        L.oracle_layer_norm.restype = None
        L.oracle_layer_norm.argtypes = [fp, fp, fp, fp, c.c_int, fp, c.c_int, c.c_float, i64, i64]
        L.oracle_softmax.restype = None
        L.oracle_softmax.argtypes = [fp, fp, fp, i64, i64, i64, i64]
        L.oracle_logsoftmax.restype = None
        L.oracle_logsoftmax.argtypes = [fp, fp, i64, i64]
        L.oracle_transpose0213.restype = None
        L.oracle_transpose0213.argtypes = [fp, fp, i64, i64, i64, i64]
        L.oracle_bdot_legacy.restype = None
        L.oracle_bdot_legacy.argtypes = [fp, fp, fp, i64, i64, i64, i64, i64, c.c_int, c.c_int,
                                         c.c_float]
        L.oracle_nbest.restype = None
        L.oracle_nbest.argtypes = [fp, i64, i64, i64, fp, c.POINTER(c.c_uint32)]
        L.oracle_embed.restype = None
        L.oracle_embed.argtypes = [fp, fp, c.POINTER(c.c_uint32), i64, i64, c.c_float, fp, i64, i64]
        L.oracle_sinusoidal_position_embeddings.restype = None
        L.oracle_sinusoidal_position_embeddings.argtypes = [fp, i64, i64, c.c_int]
        _lib = L
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def layer_norm(x, gamma, beta=None, eps=1e-9, add=None):
    x = _f32(x)
    cols = x.shape[-1]
    rows = x.size // cols
    gamma = _f32(gamma).ravel()
    beta = None if beta is None else _f32(beta).ravel()
    add = None if add is None else _f32(add)
    out = np.empty_like(x)
    lib().oracle_layer_norm(_p(out), _p(x), _p(add), _p(gamma), int(gamma.size > 1), _p(beta),
                            int(beta is not None and beta.size > 1), np.float32(eps), rows, cols)
    return out


def softmax(x, mask=None, rows_per_mask=1):
    x = _f32(x)
    cols = x.shape[-1]
    rows = x.size // cols
    n_masks = 1
    if mask is not None:
        mask = _f32(mask).reshape(-1, cols)
        n_masks = mask.shape[0]
    out = np.empty_like(x)
    lib().oracle_softmax(_p(out), _p(x), _p(mask), rows, cols, rows_per_mask, n_masks)
    return out


def logsoftmax(x):
    x = _f32(x)
    cols = x.shape[-1]
    out = np.empty_like(x)
    lib().oracle_logsoftmax(_p(out), _p(x), x.size // cols, cols)
    return out


def transpose0213(x):
    x = _f32(x)
    d0, d1, d2, d3 = x.shape
    out = np.empty((d0, d2, d1, d3), dtype=np.float32)
    lib().oracle_transpose0213(_p(out), _p(x), d0, d1, d2, d3)
    return out


def bdot_legacy(a, b, transA=False, transB=False, scalar=1.0):
    a, b = _f32(a), _f32(b)
    batchA = a.size // (a.shape[-1] * a.shape[-2])
    batchB = b.size // (b.shape[-1] * b.shape[-2])
    m, k = a.shape[-2], a.shape[-1]
    if transA:
        m, k = k, m
    l, n = b.shape[-2], b.shape[-1]
    if transB:
        l, n = n, l
    assert l == k
    batchC = max(batchA, batchB)
    lead = a.shape[:-2] if batchA >= batchB else b.shape[:-2]
    out = np.empty(tuple(lead) + (m, n), dtype=np.float32)
    assert out.size == batchC * m * n
    lib().oracle_bdot_legacy(_p(out), _p(a), _p(b), batchA, batchB, m, n, k, int(transA),
                             int(transB), np.float32(scalar))
    return out


def nbest(scores, N):
    scores = _f32(scores)
    dimBatch = scores.shape[0]
    rowLen = scores.size // dimBatch
    vals = np.empty(dimBatch * N, dtype=np.float32)
    keys = np.empty(dimBatch * N, dtype=np.uint32)
    lib().oracle_nbest(_p(scores), dimBatch, rowLen, N, _p(vals),
                       keys.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32)))
    return vals, keys


def embed(E, ids, scale=1.0, signal=None, rows_per_signal=1):
    """scale * E[ids] (+ the position signal: row (r // rows_per_signal) % n_signals for output row r)"""
    E = _f32(E)
    ids = np.ascontiguousarray(ids, dtype=np.uint32).ravel()
    d = E.shape[-1]
    n_signals = 1
    if signal is not None:
        signal = _f32(signal).reshape(-1, d)
        n_signals = signal.shape[0]
    out = np.empty((ids.size, d), dtype=np.float32)
    lib().oracle_embed(_p(out), _p(E), ids.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32)), ids.size, d,
                       np.float32(scale), _p(signal), rows_per_signal, n_signals)
    return out


def sinusoidal_position_embeddings(dimWords, dimEmb, start=0):
    out = np.empty((dimWords, dimEmb), dtype=np.float32)
    lib().oracle_sinusoidal_position_embeddings(_p(out), dimWords, dimEmb, int(start))
    return out
