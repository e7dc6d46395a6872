"""Pins the CPU checker of the decode-step float operators (oracle/decode_ops_oracle.c) against
float64 closed forms and against invariants that a dropped term, a wrong sign or a wrong index
would break.  No GPU."""
import numpy as np
import pytest

f64 = np.float64


@pytest.fixture(scope="module")
def ops():
    from oracle import decode_ops
    decode_ops.lib()
    return decode_ops


def close(a, b, rel=2e-6, floor=2e-6):
    a, b = np.asarray(a, f64), np.asarray(b, f64)
    return np.all(np.abs(a - b) <= rel * np.abs(b) + floor)


@pytest.mark.parametrize("rows,cols", [(1, 8), (5, 64), (128, 1024), (3, 1000)])
def test_layer_norm_closed_form(ops, rows, cols):
    rng = np.random.default_rng(rows * cols)
    x = rng.normal(0.3, 2.0, (rows, cols)).astype(np.float32)
    g = rng.normal(1.0, 0.2, cols).astype(np.float32)
    b = rng.normal(0.0, 0.5, cols).astype(np.float32)
    add = rng.normal(0, 1, (rows, cols)).astype(np.float32)
    for eps in (1e-9, 1e-6, 1e-3):
        for a in (None, add):
            xs = x.astype(f64) if a is None else (x + a).astype(f64)   # the skip add is an fp32 add
            mean = xs.mean(-1, keepdims=True)
            var = ((xs - mean) ** 2).mean(-1, keepdims=True)
            want = g.astype(f64) * (xs - mean) / np.sqrt(var + eps) + b.astype(f64)
            assert close(ops.layer_norm(x, g, b, eps, add=a), want, 5e-6, 5e-6)
    # no beta; broadcast gamma (a single value)
    xs = x.astype(f64)
    mean = xs.mean(-1, keepdims=True)
    var = ((xs - mean) ** 2).mean(-1, keepdims=True)
    assert close(ops.layer_norm(x, np.array([2.0], np.float32), None, 1e-9),
                 2.0 * (xs - mean) / np.sqrt(var + 1e-9), 5e-6, 5e-6)


def test_layer_norm_invariants(ops):
    rng = np.random.default_rng(1)
    x = rng.normal(5.0, 3.0, (16, 512)).astype(np.float32)
    y = ops.layer_norm(x, np.full(512, 3.0, np.float32), np.full(512, -1.0, np.float32), 1e-9)
    assert np.allclose(y.mean(-1), -1.0, atol=1e-4) and np.allclose(y.std(-1), 3.0, atol=1e-3)
    # shift of the input leaves the output unchanged (a wrong mean term would not)
    y2 = ops.layer_norm(x + np.float32(8.0), np.full(512, 3.0, np.float32), np.full(512, -1.0, np.float32), 1e-9)
    assert np.allclose(y, y2, atol=2e-5)


@pytest.mark.parametrize("rows,cols", [(1, 1), (7, 5), (64, 40), (4, 32000)])
def test_softmax_and_logsoftmax(ops, rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = rng.normal(0, 3.0, (rows, cols)).astype(np.float32)
    xs = x.astype(f64)
    e = np.exp(xs - xs.max(-1, keepdims=True))
    want = e / e.sum(-1, keepdims=True)
    # the checker sums sequentially in float like the reference loop: its error grows with cols
    rel = 5e-6 * max(1.0, cols / 500.0)
    got = ops.softmax(x)
    assert close(got, want, rel, 1e-9)
    assert np.allclose(got.astype(f64).sum(-1), 1.0, atol=2 * rel)
    assert close(ops.softmax(x + np.float32(11.0)), want, 4 * rel, 1e-9)      # shift invariance
    lwant = xs - xs.max(-1, keepdims=True) - np.log(e.sum(-1, keepdims=True))
    assert close(ops.logsoftmax(x), lwant, rel, 5e-6 * max(1.0, cols / 500.0))
    assert close(np.exp(ops.logsoftmax(x).astype(f64)), want, 4 * rel, 1e-9)


def test_softmax_mask_rows(ops):
    """mask row = (row / rows_per_mask) % n_masks: scores [beam*batch, heads, 1, len] against a
    [batch, 1, 1, len] mask repeated over the beam."""
    beam, batch, heads, L = 2, 3, 4, 9
    rng = np.random.default_rng(3)
    z = rng.normal(0, 1, (beam * batch, heads, 1, L)).astype(np.float32)
    keep = (rng.random((batch, L)) > 0.3)
    keep[:, 0] = True
    mask = ((1 - keep) * -99999999.0).astype(np.float32)
    got = ops.softmax(z, mask, rows_per_mask=heads)
    zz = z.astype(f64) + np.tile(mask.astype(np.float32), (beam, 1))[:, None, None, :]
    e = np.exp(zz - zz.max(-1, keepdims=True))
    want = e / e.sum(-1, keepdims=True)
    assert close(got, want, 5e-6, 1e-9)
    assert np.all(got.reshape(beam, batch, heads, L).transpose(1, 3, 0, 2)[~keep] == 0)


def test_transpose0213(ops):
    rng = np.random.default_rng(4)
    x = rng.normal(0, 1, (3, 5, 7, 4)).astype(np.float32)
    y = ops.transpose0213(x)
    assert np.array_equal(y, x.transpose(0, 2, 1, 3))
    assert np.array_equal(ops.transpose0213(y), x)
    # split heads then join heads (reference src/models/transformer.h:145-170) is the identity
    q = rng.normal(0, 1, (6, 1, 8, 16)).astype(np.float32)
    assert np.array_equal(ops.transpose0213(ops.transpose0213(q)), q)


@pytest.mark.parametrize("tA,tB", [(False, False), (False, True), (True, False), (True, True)])
def test_bdot_legacy(ops, tA, tB):
    rng = np.random.default_rng(5 + tA + 2 * tB)
    batch, m, n, k = 6, 3, 5, 8
    a = rng.normal(0, 1, (batch, k, m) if tA else (batch, m, k)).astype(np.float32)
    b = rng.normal(0, 1, (batch, n, k) if tB else (batch, k, n)).astype(np.float32)
    A = a.transpose(0, 2, 1) if tA else a
    B = b.transpose(0, 2, 1) if tB else b
    want = 0.125 * np.matmul(A.astype(f64), B.astype(f64))
    assert close(ops.bdot_legacy(a, b, tA, tB, 0.125), want, 1e-5, 1e-6)
    # batch broadcast: B has two batch entries, used as i % 2
    b2 = b[:2]
    B2 = b2.transpose(0, 2, 1) if tB else b2
    want2 = np.stack([A[i].astype(f64) @ B2[i % 2].astype(f64) for i in range(batch)])
    assert close(ops.bdot_legacy(a, b2, tA, tB, 1.0), want2, 1e-5, 1e-6)
    # a single A against all B
    a1 = a[:1]
    A1 = a1.transpose(0, 2, 1) if tA else a1
    want3 = np.stack([A1[0].astype(f64) @ B[i].astype(f64) for i in range(batch)])
    assert close(ops.bdot_legacy(a1, b, tA, tB, 1.0), want3, 1e-5, 1e-6)


def test_nbest_against_full_sort(ops):
    rng = np.random.default_rng(9)
    x = rng.normal(0, 1, (5, 1, 3, 400)).astype(np.float32)
    vals, keys = ops.nbest(x, 6)
    flat = x.reshape(5, -1)
    order = np.argsort(-flat, axis=1, kind="stable")[:, :6]
    assert np.array_equal(vals.reshape(5, 6), np.take_along_axis(flat, order, 1))
    assert np.array_equal(keys.reshape(5, 6).astype(np.int64), order + np.arange(5)[:, None] * flat.shape[1])
    # equal scores: lowest index first
    t = np.zeros((1, 10), np.float32)
    t[0, [7, 2, 5]] = 1.0
    v, k = ops.nbest(t, 4)
    assert k.tolist() == [2, 5, 7, 0] and v.tolist() == [1.0, 1.0, 1.0, 0.0]


# ---- the reference's own operator-test vectors (tests/golden/operator_vectors.json) -------------

def reference_vectors():
    import json
    import os
    return json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "operator_vectors.json")))


def test_reference_softmax_logsoftmax_vectors(ops):
    v = reference_vectors()["softmax_logsoftmax"]
    x = np.array(v["in"], np.float32).reshape(v["shape"])
    assert np.all(np.abs(ops.softmax(x).ravel() - np.array(v["softmax"])) <= v["margin"])
    assert np.all(np.abs(ops.logsoftmax(x).ravel() - np.array(v["logsoftmax"])) <= v["margin"])


def test_reference_layer_norm_vector(ops):
    v = reference_vectors()["layer_norm"]
    x = np.array(v["in"], np.float32).reshape(v["shape"])
    g, b = np.array(v["gamma"], np.float32), np.array(v["beta"], np.float32)
    xs = x.astype(f64)
    num = xs - xs.mean(-1, keepdims=True)
    want = g.astype(f64) * (num / np.sqrt((num ** 2).mean(-1, keepdims=True) + v["eps"])) + b.astype(f64)
    got = ops.layer_norm(x, g, b, v["eps"])
    assert np.all(np.abs(got - want) <= v["margin"]) and close(got, want, 5e-6, 5e-6)


def test_reference_bdot_vectors(ops):
    """bdot broadcasts [2,1] x [1,3] batches; the legacy batched product pairs batch entries by
    modulo (reference src/tensors/cpu/prod.cpp:233-330), so entry i of A meets all of B in a call."""
    v = reference_vectors()["bdot"]
    A = np.array(v["A"], np.float32).reshape(v["A_shape"])
    B = np.array(v["B"], np.float32).reshape(v["B_shape"])
    C = np.array(v["C"], np.float32).reshape(v["C_shape"])
    Ct = np.array(v["C_transB"], np.float32).reshape(v["C_shape"])
    for i in range(2):
        assert np.array_equal(ops.bdot_legacy(A[i], B[0]), C[i])
        assert np.array_equal(ops.bdot_legacy(A[i], B[0], transB=True), Ct[i])


def test_reference_topk_vectors(ops):
    v = reference_vectors()["topk"]
    x = np.array(v["in"], np.float32).reshape(-1, v["shape"][-1])
    vals, keys = ops.nbest(x, v["k"])
    assert np.array_equal(vals, np.array(v["values"], np.float32))
    rows = np.repeat(np.arange(x.shape[0]), v["k"])
    assert np.array_equal(keys - rows * x.shape[1], np.array(v["indices"], np.uint32))


def test_reference_rows_vectors(ops):
    v = reference_vectors()["rows"]
    A = np.array(v["A"], np.float32).reshape(v["A_shape"])
    for case in v["cases"]:
        got = ops.embed(A, case["indices"])
        assert got.shape == (len(case["indices"]), 3)
        assert np.array_equal(got.ravel(), np.array(case["out"], np.float32))


def test_embed_scale_and_signal(ops):
    """scale * E[ids] + signal[(r // rows_per_signal) % n]: against numpy indexing in float64, where
    the product of two floats is exact and the sum rounds once, so float32(float32(s * e) + g) is what
    two separate float operations give; a fused multiply-add, a signal row picked by r % n instead
    of r // rows_per_signal, or a missing scale fail it."""
    rng = np.random.default_rng(5)
    E = rng.standard_normal((50, 24)).astype(np.float32)
    ids = rng.integers(0, 50, 12)
    sig = rng.standard_normal((4, 24)).astype(np.float32)
    scale = np.float32(np.sqrt(24.0))
    prod = (E[ids].astype(f64) * f64(scale)).astype(np.float32)
    assert np.array_equal(ops.embed(E, ids, scale), prod)
    want = (prod.astype(f64) + sig[(np.arange(12) // 3) % 4].astype(f64)).astype(np.float32)
    got = ops.embed(E, ids, scale, sig, rows_per_signal=3)
    assert np.array_equal(got, want)
    fused = (E[ids].astype(f64) * f64(scale) + sig[(np.arange(12) // 3) % 4].astype(f64)).astype(np.float32)
    assert not np.array_equal(fused, want)     # the case does tell one rounding from two
    wrapped = ops.embed(E, ids, scale, sig[:2], rows_per_signal=3)     # 4 groups of rows, 2 signal rows
    assert np.array_equal(wrapped[6:], (prod[6:].astype(f64) + sig[(np.arange(6) // 3) % 2].astype(f64)).astype(np.float32))


def test_sinusoidal_position_embeddings(ops):
    """sin / cos of position * 10000^(-i / (d/2 - 1)): float64 closed form within float rounding of
    the argument (position * 1e-7 relative), zeros and ones at position 0, the two halves of a row
    a quarter turn apart, `start` a shift of the rows."""
    d, n = 64, 40
    t = ops.sinusoidal_position_embeddings(n, d)
    assert np.array_equal(t[0, :d // 2], np.zeros(d // 2, np.float32)) and np.array_equal(t[0, d // 2:], np.ones(d // 2, np.float32))
    pos = np.arange(n, dtype=f64)[:, None]
    freq = 10000.0 ** (-(np.arange(d // 2, dtype=f64)) / (d // 2 - 1))
    want = np.concatenate([np.sin(pos * freq), np.cos(pos * freq)], axis=1)
    assert np.all(np.abs(t - want) <= 4e-7 * np.tile(1 + pos * freq, (1, 2)))
    assert close(t[:, :d // 2] ** 2 + t[:, d // 2:] ** 2, np.ones((n, d // 2)), 1e-6, 0)
    assert np.array_equal(ops.sinusoidal_position_embeddings(5, d, start=7), t[7:12])
    assert abs(t[1, 0] - np.sin(1.0)) < 6e-8 and abs(t[1, d // 2 - 1] - 1e-4) < 1e-9
