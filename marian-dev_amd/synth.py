"""Deterministic synthetic inputs shared by the parity tests and the benchmark.

Counter-based generator: every element is a pure function of (seed, stream, index), so any
slice of any tensor can be regenerated anywhere (CPU checker, GPU path, another process)
without carrying state.  splitmix64 mixes the counter, Box-Muller (in float64) turns pairs of
uniforms into normals, and the result is cast to fp32 once.

Streams used by the workloads: A = 0, W = 1, bias = 2, shortlist ids = 3, lengths = 4.
"""
import numpy as np

STREAM_A, STREAM_W, STREAM_BIAS, STREAM_IDX, STREAM_LEN = 0, 1, 2, 3, 4

_U64 = np.uint64


def _splitmix64(x):
    x = (x + _U64(0x9E3779B97F4A7C15))
    x = (x ^ (x >> _U64(30))) * _U64(0xBF58476D1CE4E5B9)
    x = (x ^ (x >> _U64(27))) * _U64(0x94D049BB133111EB)
    return x ^ (x >> _U64(31))


def uniform_u64(seed, stream, n, offset=0):
    """n 64-bit words for counters offset .. offset+n-1 of (seed, stream)."""
    with np.errstate(over="ignore"):
        base = _splitmix64(_U64(seed) * _U64(0x100000001B3) + _U64(stream))
        ctr = np.arange(offset, offset + n, dtype=np.uint64)
        return _splitmix64(base ^ _splitmix64(ctr))


def normal(seed, stream, shape, std=1.0, mean=0.0):
    """fp32 N(mean, std^2) tensor of the given shape."""
    n = int(np.prod(shape))
    half = (n + 1) // 2
    w = uniform_u64(seed, stream, 2 * half)
    # 53-bit uniforms in (0, 1]
    u1 = ((w[:half] >> _U64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
    u2 = (w[half:] >> _U64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
    r = np.sqrt(-2.0 * np.log(u1))
    z = np.concatenate([r * np.cos(2.0 * np.pi * u2), r * np.sin(2.0 * np.pi * u2)])[:n]
    return (z * std + mean).astype(np.float32).reshape(shape)


def randint(seed, stream, low, high, n=1):
    """n integers uniform in [low, high)."""
    w = uniform_u64(seed, stream, n)
    return (low + (w % _U64(high - low)).astype(np.int64))


def shortlist(seed, vocab, n_min=500, n_max=2000, stream=STREAM_IDX):
    """Sorted unique uint32 ids, count uniform in [n_min, n_max] rounded up to a multiple of 8
    (the shortlist generators pad to x8 for intgemm, reference src/data/shortlist.cpp:513-520)."""
    n = int(randint(seed, stream, n_min, n_max + 1)[0])
    n = (n + 7) // 8 * 8
    keys = uniform_u64(seed, stream + 100, vocab)
    ids = np.argsort(keys, kind="stable")[:n]
    return np.sort(ids).astype(np.uint32)
