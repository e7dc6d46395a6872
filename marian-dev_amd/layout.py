"""Host-side description of the prepared ("K-blocked") order of int8 weights.

The kernels read the K*N int8 values of W^T in the order marian_hip_int8_prepare_b and
marian_hip_int8_prepare_b_quantized_transposed write (include/marian_hip_int8.h):

    byte of B[k, n] = (k // 32) * 32 * N + n * 32 + k % 32

A Marian `.bin` file holds the same values as plain rows [N, K] (reference
src/tensors/cpu/expression_graph_packable.h:160-201).  The functions here convert between the two on
the host with numpy, for tools and tests; the device conversion is the C entry point.
"""
import numpy as np


def prepared_offsets(K, N):
    """int64 [N, K]: byte offset of B[k, n] (file order: row n, position k) in prepared order."""
    assert K % 64 == 0 and N % 8 == 0, (K, N)
    n = np.arange(N, dtype=np.int64)[:, None]
    k = np.arange(K, dtype=np.int64)[None, :]
    return (k // 32) * (32 * N) + n * 32 + k % 32


def to_prepared(flat, K, N):
    """File-order bytes (payload [N, K] then whatever follows, e.g. the quantMult tail) -> prepared."""
    flat = np.ascontiguousarray(flat).view(np.uint8).ravel()
    out = flat.copy()
    out[prepared_offsets(K, N).ravel()] = flat[: K * N]
    return out


def from_prepared(flat, K, N):
    """Prepared-order bytes -> file order (payload [N, K] row-major); bytes past K*N are kept."""
    flat = np.ascontiguousarray(flat).view(np.uint8).ravel()
    out = flat.copy()
    out[: K * N] = flat[prepared_offsets(K, N).ravel()]
    return out
