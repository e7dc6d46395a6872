"""Tied int8 output layer and shortlist plumbing (marian-dev_amd/output.py).

CPU part: the id maps and the multiple-of-eight padding of reference src/data/shortlist.cpp.
GPU part: the quantized tied matrix equals what the weight packer writes for the logical
[D x V] weight, logits match the CPU checker, shortlisted logits are the column pick of the
dense ones, and best words come back as vocabulary ids."""
import numpy as np
import pytest

from conftest import load

f32 = np.float32


def test_shortlist_maps():
    out = load("output")
    sl = out.Shortlist([3, 7, 8, 100, 31999, 32000 - 8, 5, 6][:5])
    assert sl.reverseMap(0, 0, 0) == 3 and sl.reverseMap(2, 1, 4) == 31999
    assert sl.tryForwardMap(100) == 3 and sl.tryForwardMap(3) == 0
    assert sl.tryForwardMap(4) == out.npos and sl.tryForwardMap(40000) == out.npos
    for j, w in enumerate(sl.indices()):
        assert sl.tryForwardMap(int(w)) == j and sl.reverseMap(0, 0, j) == int(w)
    with pytest.raises(Exception):
        out.Shortlist([5, 4])


@pytest.mark.parametrize("n,first", [(1, 0), (7, 0), (8, 0), (13, 100), (500, 0)])
def test_shortlist_padding_rule(n, first):
    """reference src/data/shortlist.cpp:513-520: lowest unselected ids >= firstNum are added
    until the count is a multiple of eight; selected ids stay."""
    out = load("output")
    rng = np.random.default_rng(n)
    V = 2000
    ids = np.sort(rng.choice(V, size=n, replace=False))
    sl = out.Shortlist.padToMultipleOfEight(ids, V, first)
    got = sl.indices()
    assert got.size % 8 == 0 and got.size - n < 8
    assert set(ids.tolist()) <= set(got.tolist())
    added = sorted(set(got.tolist()) - set(ids.tolist()))
    # brute force: walk up from firstNum
    want, have, i = [], set(ids.tolist()), first
    while (n + len(want)) % 8 != 0:
        if i not in have:
            want.append(i)
        i += 1
    assert added == want


@pytest.mark.gpu
def test_tied_output_layer(integer, orc, synth):
    import torch
    out_mod = load("output")
    V, D, M = 4000, 256, 12
    Wt = synth.normal(901, synth.STREAM_W, (V, D), 0.05)       # tied embedding matrix [V x D]
    b = synth.normal(901, synth.STREAM_BIAS, (V,), 0.01)
    x = synth.normal(901, synth.STREAM_A, (M, D), 1.0)
    layer = out_mod.Output(torch.from_numpy(Wt).cuda(), torch.from_numpy(b).cuda())

    # the quantized tied matrix is byte for byte what the packer writes for W = Wt^T [D x V]
    Bq_h = orc.prepare_b(np.ascontiguousarray(Wt.T))
    assert np.array_equal(layer.WtQuant_.file_bytes()[:V * D + 4], Bq_h[:V * D + 4])
    assert layer.WtQuant_.shape == (D, V)

    # embedding lookup keeps the fp32 rows
    ids = [0, 17, V - 1, 17]
    assert np.array_equal(layer.embed(ids).cpu().numpy(), Wt[ids])

    Aq_h = orc.prepare_a(x)
    dense_want, _ = orc.affine(Aq_h, Bq_h, b, M, D, V)
    dense = layer.applyAsLogits(torch.from_numpy(x).cuda()).cpu().numpy()
    assert np.array_equal(dense, dense_want)

    sl = out_mod.Shortlist.padToMultipleOfEight(synth.shortlist(902, V, 100, 300)[:-3], V)
    layer.setShortlist(sl)
    short = layer.applyAsLogits(torch.from_numpy(x).cuda()).cpu().numpy()
    assert short.shape == (M, sl.indices().size)
    assert np.array_equal(short, dense[:, sl.indices()])
    scores, words = layer.bestWords(torch.from_numpy(x).cuda(), k=3)
    words = words.cpu().numpy()
    order = np.argsort(-short, axis=1, kind="stable")[:, :3]
    assert np.array_equal(np.sort(words, axis=1), np.sort(sl.indices()[order].astype(np.int64), axis=1))
    assert np.allclose(scores.cpu().numpy(), np.take_along_axis(short, order, axis=1))
    for w in words.ravel():
        assert sl.tryForwardMap(int(w)) != out_mod.npos
    layer.clear()
    assert layer.applyAsLogits(torch.from_numpy(x).cuda()).shape[-1] == V
