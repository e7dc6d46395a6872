"""The prepared ("K-blocked") order of int8 weights, host side: the index formula against a loop that
follows the description in words, the properties the kernels rely on, and the two conversions."""
import numpy as np
import pytest

from conftest import load


def offsets_by_description(K, N):
    """K in sub-steps of 32; per sub-step the columns one after the other, 32 bytes each."""
    off = np.empty((N, K), dtype=np.int64)
    pos = 0
    for s in range(K // 32):
        for n in range(N):
            for b in range(32):
                off[n, s * 32 + b] = pos
                pos += 1
    assert pos == K * N
    return off


@pytest.mark.parametrize("K,N", [(64, 8), (64, 32), (128, 24), (192, 136), (256, 1000)])
def test_offsets_follow_the_description(K, N):
    L = load("layout")
    got = L.prepared_offsets(K, N)
    assert np.array_equal(got, offsets_by_description(K, N))
    assert np.array_equal(np.sort(got.ravel()), np.arange(K * N))          # a permutation of the payload


@pytest.mark.parametrize("K,N", [(64, 32), (128, 96), (256, 1000)])
def test_operand_blocks_are_contiguous(K, N):
    """32 consecutive columns x one sub-step = 1 KB of consecutive bytes (what one wave loads for one
    32x32x32 matrix instruction); 16 columns x one sub-step = 512 bytes; a step along K is 32 * N
    bytes for every column; a column's 32 values of a sub-step stay together (shortlist gathers)."""
    L = load("layout")
    off = L.prepared_offsets(K, N)
    for n0 in range(0, N - 31, 32):
        for s in range(K // 32):
            blk = off[n0:n0 + 32, s * 32:(s + 1) * 32].ravel()
            assert blk.min() == s * 32 * N + n0 * 32 and blk.max() - blk.min() == 1023
    for n0 in range(0, N - 15, 16):
        blk = off[n0:n0 + 16, 0:32].ravel()
        assert blk.max() - blk.min() == 511
    assert np.array_equal(off[:, 32:] - off[:, :-32], np.full((N, K - 32), 32 * N))
    assert np.array_equal(off[:, 31::32] - off[:, 0::32], np.full((N, K // 32), 31))


def test_conversions_are_inverse_and_keep_the_tail():
    L = load("layout")
    K, N = 128, 40
    rng = np.random.default_rng(3)
    flat = rng.integers(-128, 128, size=K * N + 4 + 252, dtype=np.int8)      # payload, tail, allocation padding
    prepared = L.to_prepared(flat, K, N)
    assert np.array_equal(prepared[K * N:], flat.view(np.uint8)[K * N:])
    assert not np.array_equal(prepared[: K * N], flat.view(np.uint8)[: K * N])
    assert np.array_equal(L.from_prepared(prepared, K, N), flat.view(np.uint8))
    # B[k, n] of the file order sits where the formula says
    rows = flat[: K * N].reshape(N, K)
    off = L.prepared_offsets(K, N)
    for n, k in [(0, 0), (7, 15), (8, 16), (39, 127), (13, 77)]:
        assert prepared[off[n, k]] == rows[n, k].view(np.uint8)
