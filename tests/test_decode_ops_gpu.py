"""GPU parity of the float operators of include/marian_hip_ops.h (through the C ABI, via the host
mirror marian-dev_amd/ops.py) against the CPU checker and against float64 closed forms.

Bar: 1e-5 relative plus a small absolute floor.  These are floating-point reductions whose
summation order differs between the reference's own builds (SIMD width, fast-math), the checker
(sequential) and the kernels (wave trees); the kernels are held to the float64 value within the
bar, and to the checker within the bar widened by the checker's own sequential-sum error on long
rows."""
import numpy as np
import pytest

from conftest import load

pytestmark = pytest.mark.gpu
f64 = np.float64
REL = 1e-5


@pytest.fixture(scope="module")
def ops(integer):
    return load("ops")


@pytest.fixture(scope="module")
def chk():
    from oracle import decode_ops
    decode_ops.lib()
    return decode_ops


def dev(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def close(got, want, rel=REL, floor=1e-6):
    got, want = np.asarray(got, f64), np.asarray(want, f64)
    err = np.abs(got - want)
    ok = err <= rel * np.abs(want) + floor
    assert ok.all(), "max err %g (rel %g) at %s" % (err.max(), (err / (np.abs(want) + floor)).max(),
                                                    np.argwhere(~ok)[:3].tolist())


@pytest.mark.parametrize("rows,cols", [(1, 8), (5, 64), (128, 1024), (3, 1000), (7, 4096), (2, 5000),
                                       (4, 1023), (3, 8192), (2, 8196)])
@pytest.mark.parametrize("with_add,with_beta", [(False, True), (True, True), (True, False)])
def test_layer_norm(ops, chk, synth, rows, cols, with_add, with_beta):
    x = synth.normal(rows * 7 + cols, 0, (rows, cols), 2.0) + np.float32(0.3)
    add = synth.normal(rows * 7 + cols, 1, (rows, cols), 1.0) if with_add else None
    g = synth.normal(cols, 2, (cols,), 0.2) + np.float32(1.0)
    b = synth.normal(cols, 3, (cols,), 0.5) if with_beta else None
    for eps in (1e-9, 1e-6):
        got = ops.layerNorm(dev(x), dev(g), None if b is None else dev(b), eps,
                            None if add is None else dev(add)).cpu().numpy()
        xs = (x if add is None else x + add).astype(f64)
        mean = xs.mean(-1, keepdims=True)
        var = ((xs - mean) ** 2).mean(-1, keepdims=True)
        want = g.astype(f64) * (xs - mean) / np.sqrt(var + eps) + (0 if b is None else b.astype(f64))
        close(got, want, REL, 2e-6)
        close(got, chk.layer_norm(x, g, b, eps, add=add), 2 * REL, 4e-6)
    # a single broadcast gamma/beta value (reference alphaStride/betaStride = 0)
    got = ops.layerNorm(dev(x), dev(np.array([2.0], np.float32)), dev(np.array([-1.0], np.float32)), 1e-9).cpu().numpy()
    close(got, chk.layer_norm(x, np.array([2.0], np.float32), np.array([-1.0], np.float32), 1e-9), 2 * REL, 4e-6)


def test_layer_norm_4d_and_inplace_shapes(ops, chk, synth):
    x = synth.normal(11, 0, (4, 32, 1, 1024), 1.0)
    g = synth.normal(11, 2, (1, 1024), 0.1) + np.float32(1.0)
    b = synth.normal(11, 3, (1, 1024), 0.1)
    got = ops.layerNorm(dev(x), dev(g), dev(b), 1e-6, dev(x)).cpu().numpy()
    assert got.shape == x.shape
    close(got, chk.layer_norm(x, g, b, 1e-6, add=x), 2 * REL, 4e-6)


@pytest.mark.parametrize("rows,cols", [(1, 1), (7, 5), (2048, 40), (4096, 64), (33, 2048), (5, 2049),
                                       (128, 32000), (3, 32768), (2, 32772), (3, 8190), (4, 4100),
                                       (5, 50000), (2, 65536), (2, 65540), (300, 512)])
def test_softmax_and_logsoftmax(ops, chk, synth, rows, cols):
    x = synth.normal(rows + cols, 0, (rows, cols), 3.0)
    xs = x.astype(f64)
    e = np.exp(xs - xs.max(-1, keepdims=True))
    want = e / e.sum(-1, keepdims=True)
    got = ops.softmax(dev(x)).cpu().numpy()
    close(got, want, REL, 1e-10)
    assert np.allclose(got.astype(f64).sum(-1), 1.0, atol=1e-5)
    lwant = xs - xs.max(-1, keepdims=True) - np.log(e.sum(-1, keepdims=True))
    lgot = ops.logsoftmax(dev(x)).cpu().numpy()
    close(lgot, lwant, REL, 1e-5)
    if rows * cols <= 1 << 20:   # against the checker, widened by its sequential-sum error
        wide = REL * max(1.0, cols / 250.0)
        close(got, chk.softmax(x), wide, 1e-10)
        close(lgot, chk.logsoftmax(x), wide, 1e-5 * max(1.0, cols / 250.0))


def test_softmax_with_attention_mask(ops, chk, synth):
    """scores [beam*batch, heads, 1, len] + log-mask [batch, 1, 1, len] repeated over the beam"""
    beam, batch, heads, L = 4, 8, 16, 37
    z = synth.normal(21, 0, (beam * batch, heads, 1, L), 1.0)
    lens = 1 + (np.arange(batch) * 5) % L
    keep = (np.arange(L)[None, :] < lens[:, None])
    mask = ((1 - keep) * -99999999.0).astype(np.float32)
    got = ops.softmax(dev(z), dev(mask), rowsPerMask=heads).cpu().numpy()
    close(got, chk.softmax(z, mask, rows_per_mask=heads), REL, 1e-10)
    g4 = got.reshape(beam, batch, heads, L)
    for bi in range(batch):
        assert np.all(g4[:, bi, :, lens[bi]:] == 0) and np.allclose(g4[:, bi].sum(-1), 1.0, atol=1e-5)


@pytest.mark.parametrize("L", [300, 1000, 4100, 258])
def test_softmax_with_mask_on_long_rows(ops, chk, synth, L):
    """Masked rows of more than 256 scores (long source sentences): the register-resident kernels
    add the mask row as they load."""
    batch, heads = 6, 4
    z = synth.normal(22 + L, 0, (batch, heads, 3, L), 1.0)
    lens = 1 + (np.arange(batch) * 97) % L
    mask = ((np.arange(L)[None, :] >= lens[:, None]) * -99999999.0).astype(np.float32)
    got = ops.softmax(dev(z), dev(mask), rowsPerMask=heads * 3).cpu().numpy()
    zs = z.astype(f64) + mask.astype(f64)[:, None, None, :]
    e = np.exp(zs - zs.max(-1, keepdims=True))
    close(got, e / e.sum(-1, keepdims=True), REL, 1e-10)
    close(got, chk.softmax(z, mask, rows_per_mask=heads * 3), REL * max(1.0, L / 250.0), 1e-10)


@pytest.mark.parametrize("shape", [(3, 5, 7, 4), (128, 1, 16, 64), (128, 16, 1, 64), (32, 40, 16, 64),
                                   (2, 3, 4, 5), (1, 2, 2, 1)])
def test_transpose0213(ops, chk, synth, shape):
    x = synth.normal(sum(shape), 0, shape, 1.0)
    y = ops.transpose0213(dev(x))
    assert np.array_equal(y.cpu().numpy(), chk.transpose0213(x))
    assert np.array_equal(ops.transpose0213(y).cpu().numpy(), x)


def test_split_and_join_heads(ops, synth):
    beam, batch, steps, heads, depth = 4, 8, 1, 16, 64
    x = synth.normal(31, 0, (beam, batch, steps, heads * depth), 1.0)
    q = ops.SplitHeads(dev(x), heads)
    assert tuple(q.shape) == (beam * batch, heads, steps, depth)
    want = x.reshape(beam * batch, steps, heads, depth).transpose(0, 2, 1, 3)
    assert np.array_equal(q.cpu().numpy(), want)
    assert np.array_equal(ops.JoinHeads(q, beam).cpu().numpy(), x)


@pytest.mark.parametrize("tA,tB", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("batch,m,n,k", [(6, 3, 5, 8), (2048, 1, 40, 64), (2048, 1, 64, 40), (8, 33, 70, 65),
                                         (4, 64, 64, 64), (3, 70, 100, 36), (2, 9, 8, 8), (16, 40, 44, 64),
                                         (64, 64, 64, 64)])
def test_bdot_legacy(ops, chk, synth, tA, tB, batch, m, n, k):
    a = synth.normal(batch + m, 0, (batch, k, m) if tA else (batch, m, k), 1.0)
    b = synth.normal(batch + n, 1, (batch, n, k) if tB else (batch, k, n), 1.0)
    got = ops.bdot_legacy(dev(a), dev(b), tA, tB, 0.125).cpu().numpy()
    A = a.transpose(0, 2, 1) if tA else a
    B = b.transpose(0, 2, 1) if tB else b
    want = 0.125 * np.matmul(A.astype(f64), B.astype(f64))
    floor = 2e-6 * np.sqrt(k)   # cancellation in sums of k products of unit-variance values
    close(got, want, REL, floor)
    if batch * m * n * k <= 1 << 22:
        close(got, chk.bdot_legacy(a, b, tA, tB, 0.125), REL, 2 * floor)
    # batch broadcast i % batchB
    b2 = np.ascontiguousarray(b[:2])
    got2 = ops.bdot_legacy(dev(a), dev(b2), tA, tB, 1.0).cpu().numpy()
    B2 = b2.transpose(0, 2, 1) if tB else b2
    want2 = np.stack([A[i].astype(f64) @ B2[i % 2].astype(f64) for i in range(batch)])
    close(got2, want2, REL, 8 * floor)


def _random_row_cases(n):
    rng = np.random.default_rng(20261128)
    cases = []
    for i in range(n):
        cols = int(rng.choice([1, 3, 64, 100, 255, 256, 260, 1024, 2047, 2052, 4096, 4104, 8192, 9000,
                               32768, 40000, 65536, 66000]))
        rows = int(rng.integers(1, 600)) if cols <= 4104 else int(rng.integers(1, 12))
        cases.append((i, rows, cols))
    return cases


@pytest.mark.parametrize("i,rows,cols", _random_row_cases(28))
def test_row_operators_random_shapes(ops, synth, i, rows, cols):
    """Seeded random shapes through softmax (plain and with a mask per group of rows), log-softmax
    and layer norm (with the skip input), against float64: every column-count range of the
    kernel choice, aligned and unaligned row lengths."""
    x = synth.normal(9500 + i, 0, (rows, cols), 2.5)
    xs = x.astype(f64)
    e = np.exp(xs - xs.max(-1, keepdims=True))
    close(ops.softmax(dev(x)).cpu().numpy(), e / e.sum(-1, keepdims=True), REL, 1e-10)
    close(ops.logsoftmax(dev(x)).cpu().numpy(), xs - xs.max(-1, keepdims=True) - np.log(e.sum(-1, keepdims=True)),
          REL, 1e-5)
    # mask rows shared by rpm consecutive score rows
    rpm = [r for r in (1, 2, 3, 4, 5) if rows % r == 0][-1]
    lens = 1 + (np.arange(rows // rpm) * 37) % cols
    mask = ((np.arange(cols)[None, :] >= lens[:, None]) * -99999999.0).astype(np.float32)
    zs = xs.reshape(rows // rpm, rpm, cols) + mask.astype(f64)[:, None, :]
    em = np.exp(zs - zs.max(-1, keepdims=True))
    got = ops.softmax(dev(x.reshape(rows // rpm, rpm, 1, cols)), dev(mask), rowsPerMask=rpm).cpu().numpy()
    close(got.reshape(rows // rpm, rpm, cols), em / em.sum(-1, keepdims=True), REL, 1e-10)
    g = synth.normal(9500 + i, 2, (cols,), 0.2) + np.float32(1.0)
    b = synth.normal(9500 + i, 3, (cols,), 0.5)
    add = synth.normal(9500 + i, 1, (rows, cols), 1.0)
    ys = xs + add.astype(f64)
    mean = ys.mean(-1, keepdims=True)
    var = ((ys - mean) ** 2).mean(-1, keepdims=True)
    want = g.astype(f64) * (ys - mean) / np.sqrt(var + 1e-6) + b.astype(f64)
    # x + add is rounded to float32 before the mean is taken off: rows whose values nearly coincide
    # amplify that rounding by max|y| / sigma, in any float32 implementation
    floor = 2e-6 + 4 * 2.0 ** -24 * np.abs(ys).max(-1, keepdims=True) / np.sqrt(var + 1e-6) * np.abs(g).max()
    close(ops.layerNorm(dev(x), dev(g), dev(b), 1e-6, dev(add)).cpu().numpy(), want, REL, floor)


def _random_bdot_cases(n):
    rng = np.random.default_rng(20261129)
    return [(i, int(rng.integers(1, 40)), int(rng.integers(1, 100)), int(rng.integers(1, 100)),
             int(rng.choice([1, 4, 8, 20, 36, 64, 65, 128])), bool(rng.integers(2)), bool(rng.integers(2)))
            for i in range(n)]


@pytest.mark.parametrize("i,batch,m,n,k,tA,tB", _random_bdot_cases(24))
def test_bdot_random_shapes(ops, synth, i, batch, m, n, k, tA, tB):
    a = synth.normal(9700 + i, 0, (batch, k, m) if tA else (batch, m, k), 1.0)
    b = synth.normal(9700 + i, 1, (batch, n, k) if tB else (batch, k, n), 1.0)
    got = ops.bdot_legacy(dev(a), dev(b), tA, tB, 0.5).cpu().numpy()
    A = a.transpose(0, 2, 1) if tA else a
    B = b.transpose(0, 2, 1) if tB else b
    close(got, 0.5 * np.matmul(A.astype(f64), B.astype(f64)), REL, 2e-6 * np.sqrt(k))


def test_attention_products_of_a_decode_step(ops, chk, synth):
    """q [B*H, 1, dk] . k^T [B*H, len, dk] * 1/sqrt(dk), softmax, . v [B*H, len, dk]
    (reference src/models/transformer.h:258-277) against the checker, op by op."""
    BH, L, dk = 128 * 16, 40, 64
    q = synth.normal(41, 0, (BH, 1, dk), 1.0)
    k = synth.normal(41, 1, (BH, L, dk), 1.0)
    v = synth.normal(41, 2, (BH, L, dk), 1.0)
    z = ops.bdot_legacy(dev(q), dev(k), False, True, 1.0 / np.sqrt(dk))
    w = ops.softmax(z)
    o = ops.bdot_legacy(w, dev(v))
    zc = chk.bdot_legacy(q, k, False, True, 1.0 / np.sqrt(dk))
    wc = chk.softmax(zc)
    oc = chk.bdot_legacy(wc, v)
    close(z.cpu().numpy(), zc, REL, 1e-5)
    close(w.cpu().numpy(), wc, 4 * REL, 1e-8)
    close(o.cpu().numpy(), oc, 4 * REL, 1e-5)


@pytest.mark.parametrize("BQ,BKV,m,L,dk,masked", [(2048, 2048, 1, 21, 64, False), (2048, 512, 1, 40, 64, True),
                                                  (24, 24, 3, 130, 64, False), (8, 4, 2, 7, 20, True),
                                                  (16, 16, 1, 1, 64, False)])
def test_one_launch_attention_equals_the_three_operators(ops, chk, synth, BQ, BKV, m, L, dk, masked):
    """marian_hip_attention against bdot_legacy + (mask) softmax + bdot_legacy of the same library:
    bit for bit where it sums in their order (head sizes other than 64), within the bar for the
    head size 64, whose dot products are summed sixteen lanes wide and whose weighted values four
    positions wide; and against the checker within the bar."""
    heads = 4
    q = synth.normal(BQ + L, 0, (BQ, m, dk), 1.0)
    k = synth.normal(BQ + L, 1, (BKV, L, dk), 1.0)
    v = synth.normal(BQ + L, 2, (BKV, L, dk), 1.0)
    mask = None
    rpm = 1
    if masked:
        n_masks = BKV // heads
        lens = 1 + (np.arange(n_masks) * 3) % L
        mask = ((np.arange(L)[None, :] >= lens[:, None]) * -99999999.0).astype(np.float32)
        rpm = heads * m
    scale = 1.0 / float(dk) ** 0.5
    z = ops.bdot_legacy(dev(q), dev(k), False, True, scale)
    w = ops.softmax(z, None if mask is None else dev(mask), rpm)
    want = ops.bdot_legacy(w, dev(v)).cpu().numpy()
    got = ops.Attention(dev(q), dev(k), dev(v), None if mask is None else dev(mask), rpm).cpu().numpy()
    if dk == 64:
        close(got, want, 4 * REL, 2e-5)
    else:
        assert np.array_equal(got, want)
    zc = chk.bdot_legacy(q, k, False, True, scale)
    wc = chk.softmax(zc, mask, rows_per_mask=rpm)
    close(got, chk.bdot_legacy(wc, v), 4 * REL, 2e-5)


def test_absmax_outputs_of_layer_norm_and_attention(ops, integer, synth):
    """The abs-max slots a producer leaves have max|out| as their maximum, and an affine call that
    takes them gives the bits of the call that scans the tensor itself."""
    x = synth.normal(51, 0, (128, 1024), 1.0)
    g = synth.normal(51, 2, (1024,), 0.1) + np.float32(1.0)
    b = synth.normal(51, 3, (1024,), 0.1)
    y, ymax = ops.layerNorm(dev(x), dev(g), dev(b), 1e-6, dev(x), want_absmax=True)
    assert np.array_equal(y.cpu().numpy(), ops.layerNorm(dev(x), dev(g), dev(b), 1e-6, dev(x)).cpu().numpy())
    assert float(ymax.data.max()) == float(y.abs().max())
    q = synth.normal(52, 0, (2048, 1, 64), 1.0)
    k = synth.normal(52, 1, (2048, 21, 64), 1.0)
    v = synth.normal(52, 2, (2048, 21, 64), 1.0)
    o, omax = ops.Attention(dev(q), dev(k), dev(v), want_absmax=True)
    assert np.array_equal(o.cpu().numpy(), ops.Attention(dev(q), dev(k), dev(v)).cpu().numpy())
    assert float(omax.data.max()) == float(o.abs().max())
    import torch
    W = torch.randn(1024, 1024, device="cuda") * 0.02
    Bq = integer.prepareB(W)
    for t, tmax in ((y, ymax), (o.view(128, 1024), omax)):
        got, aq = integer.affine_f32(t, Bq, None, absmax=tmax)
        want, aq_ref = integer.affine_f32(t, Bq, None)
        assert np.array_equal(aq.numpy(), aq_ref.numpy()) and np.array_equal(got.cpu().numpy(), want.cpu().numpy())


@pytest.mark.parametrize("beam,entries,L,masked,rows_per_mask", [(4, 512, 60, True, 16), (4, 512, 21, False, 1),
                                                               (2, 48, 130, True, 16), (3, 16, 7, True, 1),
                                                               (6, 32, 64, True, 16), (12, 8, 1, False, 1),
                                                               (8, 5, 1024, True, 1),
                                                               # around the lengths up to which the rows of an entry
                                                               # share its keys and values through LDS (32, 64, 96)
                                                               (4, 64, 96, True, 16), (5, 16, 97, True, 1),
                                                               (2, 32, 33, False, 1), (9, 4, 32, True, 1), (4, 32, 65, True, 16)])
def test_attention_rows_that_share_keys_and_values(ops, synth, beam, entries, L, masked, rows_per_mask):
    """hypotheses of a sentence over the encoder's keys and values: the call that names the shared
    cache once (batchKV = batchQ / beam, query row i reads entry i % batchKV) gives the bits of the
    call on a cache that holds a copy per query row; the abs-max slots agree too"""
    import torch
    dk = 64
    BQ = beam * entries
    q = dev(synth.normal(BQ + L, 0, (BQ, 1, dk), 1.0))
    k = dev(synth.normal(BQ + L, 1, (entries, L, dk), 1.0))
    v = dev(synth.normal(BQ + L, 2, (entries, L, dk), 1.0))
    mask = None
    if masked:
        n_masks = max(1, entries // rows_per_mask)
        lens = 1 + (np.arange(n_masks) * 7) % L
        mask = dev(((np.arange(L)[None, :] >= lens[:, None]) * -99999999.0).astype(np.float32))
    got, gmax = ops.Attention(q, k, v, mask, rowsPerMask=rows_per_mask, want_absmax=BQ <= 2048) if BQ <= 2048 else \
        (ops.Attention(q, k, v, mask, rowsPerMask=rows_per_mask), None)
    want = ops.Attention(q, k.repeat(beam, 1, 1), v.repeat(beam, 1, 1), mask, rowsPerMask=rows_per_mask, want_absmax=BQ <= 2048)
    if BQ <= 2048:
        want, wmax = want
        assert torch.equal(gmax.data, wmax.data)
    assert torch.equal(got, want)


@pytest.mark.parametrize("BQ,BKV,m,L,dk,masked", [(24, 24, 40, 40, 64, True), (16, 8, 9, 33, 32, False)])
def test_attention_with_many_query_positions(ops, synth, BQ, BKV, m, L, dk, masked):
    """Encoder-size use (many query positions per head; the host mirror runs the three operators):
    against the float64 closed form."""
    q = synth.normal(BQ + m, 0, (BQ, m, dk), 1.0)
    k = synth.normal(BQ + m, 1, (BKV, L, dk), 1.0)
    v = synth.normal(BQ + m, 2, (BKV, L, dk), 1.0)
    mask = None
    heads = 4
    if masked:   # one mask row per sentence, shared by its heads and query positions
        mask = np.zeros((BQ // heads, L), np.float32)
        mask[:, L - 5:] = -np.inf
    got = ops.Attention(dev(q), dev(k), dev(v), None if mask is None else dev(mask), heads * m).cpu().numpy()
    z = np.einsum("bmd,bld->bml", q.astype(f64), k.astype(f64)[np.arange(BQ) % BKV]) / np.sqrt(dk)
    if masked:
        z = z + mask.astype(f64)[np.arange(BQ) // heads][:, None, :]
    w = np.exp(z - z.max(-1, keepdims=True))
    w = w / w.sum(-1, keepdims=True)
    want = np.einsum("bml,bld->bmd", w, v.astype(f64)[np.arange(BQ) % BKV])
    close(got, want, 4 * REL, 2e-5)


def _random_attention_cases(n):
    rng = np.random.default_rng(20261130)
    cases = []
    for i in range(n):
        heads = int(rng.choice([1, 2, 4, 8]))
        batch = int(rng.integers(1, 7))
        beam = int(rng.integers(1, 5))
        cases.append((i, beam, batch, heads, int(rng.choice([1, 1, 1, 2, 7, 8, 9, 20])),
                      int(rng.choice([1, 2, 15, 16, 17, 40, 63, 64, 65, 130, 300, 1000])),
                      int(rng.choice([8, 20, 32, 64, 64, 128])), bool(rng.integers(2)), bool(rng.integers(2))))
    return cases


@pytest.mark.parametrize("i,beam,batch,heads,m,L,dk,masked,shared", _random_attention_cases(32))
def test_attention_random_shapes(ops, synth, i, beam, batch, heads, m, L, dk, masked, shared):
    """Seeded random shapes against the float64 closed form: one and many query positions, keys and
    values per beam entry or shared by the beam (i % batchKV), a mask row per sentence."""
    BQ = beam * batch * heads
    BKV = batch * heads if shared else BQ
    q = synth.normal(9800 + i, 0, (BQ, m, dk), 1.0)
    k = synth.normal(9800 + i, 1, (BKV, L, dk), 1.0)
    v = synth.normal(9800 + i, 2, (BKV, L, dk), 1.0)
    mask = None
    if masked:
        lens = 1 + (np.arange(batch) * 7 + i) % L
        mask = ((np.arange(L)[None, :] >= lens[:, None]) * -99999999.0).astype(np.float32)
    got = ops.Attention(dev(q), dev(k), dev(v), None if mask is None else dev(mask), heads * m).cpu().numpy()
    z = np.einsum("bmd,bld->bml", q.astype(f64), k.astype(f64)[np.arange(BQ) % BKV]) / np.sqrt(dk)
    if masked:
        z = z + mask.astype(f64)[(np.arange(BQ) // heads) % batch][:, None, :]
    w = np.exp(z - z.max(-1, keepdims=True))
    w = w / w.sum(-1, keepdims=True)
    want = np.einsum("bml,bld->bmd", w, v.astype(f64)[np.arange(BQ) % BKV])
    close(got, want, 4 * REL, 2e-5)


@pytest.mark.parametrize("BH,T,dk", [(2048, 21, 64), (64, 1, 64), (48, 70, 20), (16, 9, 64)])
def test_attention_with_cache_append(ops, synth, BH, T, dk):
    """kNew / vNew stand for the last cached position and are stored there: same output bits as
    appending by hand first, and the cache ends up holding the new rows."""
    q = synth.normal(61 + T, 0, (BH, 1, dk), 1.0)
    k = synth.normal(61 + T, 1, (BH, T, dk), 1.0)
    v = synth.normal(61 + T, 2, (BH, T, dk), 1.0)
    kn = synth.normal(61 + T, 3, (BH, dk), 1.0)
    vn = synth.normal(61 + T, 4, (BH, dk), 1.0)
    k2, v2 = k.copy(), v.copy()
    k2[:, T - 1, :] = kn
    v2[:, T - 1, :] = vn
    want = ops.Attention(dev(q), dev(k2), dev(v2)).cpu().numpy()
    kc, vc = dev(k), dev(v)
    got = ops.Attention(dev(q), kc, vc, kNew=dev(kn), vNew=dev(vn)).cpu().numpy()
    assert np.array_equal(got, want)
    assert np.array_equal(kc.cpu().numpy(), k2) and np.array_equal(vc.cpu().numpy(), v2)


@pytest.mark.parametrize("batch,beam,V,N", [(32, 4, 32000, 4), (1, 1, 32000, 12), (7, 6, 1000, 6), (3, 1, 20, 16),
                                            (2, 2, 8, 16), (5, 4, 3000, 1)])
def test_nbest(ops, chk, synth, batch, beam, V, N):
    x = synth.normal(71 + V, 0, (batch, 1, beam, V), 2.0)
    vals, keys = ops.getNBestList(dev(x), N)
    flat = x.reshape(batch, -1)
    order = np.argsort(-flat, axis=1, kind="stable")[:, :N]
    assert np.array_equal(vals.cpu().numpy().reshape(batch, N), np.take_along_axis(flat, order, 1))
    want_keys = order + np.arange(batch)[:, None] * flat.shape[1]
    assert np.array_equal(keys.cpu().numpy().view(np.uint32).reshape(batch, N).astype(np.int64), want_keys)
    if batch * beam * V <= 20000:
        cv, ck = chk.nbest(x, N)
        assert np.array_equal(vals.cpu().numpy(), cv) and np.array_equal(keys.cpu().numpy().view(np.uint32), ck)


@pytest.mark.parametrize("batch,beam,V,N", [(32, 4, 32000, 4), (1, 1, 32000, 12), (7, 6, 1000, 6), (3, 1, 20, 16),
                                            (2, 2, 8, 16), (5, 4, 3000, 1), (2, 3, 8195, 5), (300, 2, 4099, 2),
                                            (1, 12, 50001, 16), (4, 64, 512, 16)])
def test_nbest_of_beams(ops, chk, synth, batch, beam, V, N):
    """Beam-major scores [beam, 1, batch, V] in one call = the transposition followed by the n-best
    of the rows (the separate entry point and a stable sort), several slices per beam entry, ragged
    last slices, rows not 16-byte aligned (odd V), slices shorter than N, equal scores across
    slices and beam entries."""
    x = synth.normal(91 + V, 0, (beam, 1, batch, V), 2.0)
    if V >= 4099:
        x[:, 0, 0, ::997] = np.float32(7.5)       # ties across slices and beam entries
        x[0, 0, -1, :] = np.float32(-np.inf)
    vals, keys = ops.getNBestListOfBeams(dev(x), N)
    swapped = np.ascontiguousarray(np.swapaxes(x, 0, 2))       # [batch, 1, beam, V]
    flat = swapped.reshape(batch, -1)
    order = np.argsort(-flat, axis=1, kind="stable")[:, :N]
    assert np.array_equal(vals.cpu().numpy().reshape(batch, N), np.take_along_axis(flat, order, 1))
    want_keys = order + np.arange(batch)[:, None] * flat.shape[1]
    assert np.array_equal(keys.cpu().numpy().view(np.uint32).reshape(batch, N).astype(np.int64), want_keys)
    v1, k1 = ops.getNBestList(dev(swapped), N)
    assert np.array_equal(vals.cpu().numpy(), v1.cpu().numpy()) and np.array_equal(keys.cpu().numpy(), k1.cpu().numpy())
    if batch * beam * V <= 20000:
        cv, ck = chk.nbest(swapped, N)
        assert np.array_equal(vals.cpu().numpy(), cv) and np.array_equal(keys.cpu().numpy().view(np.uint32), ck)


@pytest.mark.parametrize("batch,beam,V,N,with_scores", [(32, 4, 32000, 4, False), (32, 4, 32000, 4, True), (1, 1, 32000, 12, True),
                                                        (7, 6, 5000, 6, True), (9, 3, 8196, 5, True), (40, 2, 4100, 2, False),
                                                        (2, 12, 32768, 16, True), (3, 64, 4104, 16, False), (1, 2, 6000, 8, True),
                                                        # sizes the one-launch form does not take: the mirror falls back
                                                        (3, 1, 20, 16, False), (2, 2, 8, 8, True), (5, 4, 3000, 1, False),
                                                        (2, 2, 4098, 3, True), (1, 2, 40000, 4, False)])
def test_logsoftmax_nbest_of_beams_is_the_separate_calls(ops, chk, synth, batch, beam, V, N, with_scores):
    """The end of a beam-search step in one launch: bit for bit the log-softmax entry point, the
    addition of the path scores and the n-best over beams one after the other; the log-probabilities
    it writes on request are those of the separate call; and for sizes the CPU checker finishes
    quickly, its n-best of its own log-softmax (values within the float bar of that operator, keys
    equal wherever the checker's values are not tied within that bar)."""
    import torch
    x = synth.normal(77 + V + beam, 0, (beam, 1, batch, V), 3.0)
    if V >= 1000:
        x[:, 0, 0, ::499] = np.float32(6.25)      # equal logits inside a row and across the beam
        x[0, 0, -1, :] = np.float32(0.5)          # a constant row
    path = synth.normal(5 + beam, 1, (beam, batch), 1.5) if with_scores else None
    dx = dev(x)
    lp_sep = ops.logsoftmax(dx)
    scored = lp_sep if path is None else lp_sep + dev(path).view(beam, 1, batch, 1)
    want_v, want_k = ops.getNBestListOfBeams(scored, N)
    vals, keys, lp = ops.logsoftmaxNBestOfBeams(dx, N, None if path is None else dev(path), want_logprobs=True)
    assert torch.equal(lp, lp_sep)
    assert torch.equal(vals, want_v) and torch.equal(keys, want_k)
    vals2, keys2 = ops.logsoftmaxNBestOfBeams(dx, N, None if path is None else dev(path))      # without the copy
    assert torch.equal(vals2, want_v) and torch.equal(keys2, want_k)
    if batch * beam * V <= 60000:
        ref = chk.logsoftmax(x.reshape(beam * batch, V)).reshape(beam, 1, batch, V)
        if path is not None:
            ref = ref + path.reshape(beam, 1, batch, 1)
        flat = np.ascontiguousarray(np.swapaxes(ref, 0, 2)).reshape(batch, -1)
        got_v = vals.cpu().numpy().reshape(batch, N)
        got_k = keys.cpu().numpy().view(np.uint32).reshape(batch, N).astype(np.int64) - np.arange(batch)[:, None] * flat.shape[1]
        assert np.allclose(got_v, np.take_along_axis(flat, got_k, 1), rtol=2e-5, atol=4e-6)
        order = np.argsort(-flat, axis=1, kind="stable")[:, :N]
        assert np.allclose(got_v, np.take_along_axis(flat, order, 1), rtol=2e-5, atol=4e-6)


@pytest.mark.parametrize("batch,beam,V,N", [(32, 4, 32000, 4), (32, 4, 32000, 8), (64, 6, 8196, 6), (300, 2, 4100, 2)])
def test_nbest_hand_over_with_and_without_fences(ops, synth, batch, beam, V, N):
    """The hand-over of candidates between workgroups relies on device-scope stores and a wait for
    their acknowledgement instead of the fences the language's memory model asks for.  The tuning
    build holds both forms: same values and keys from both, for both entry points that use the
    hand-over, at the size of a beam-search step and with many sentences, twenty calls each (a stale
    candidate would show as a different n-best)."""
    import torch
    L = load("_lib")
    x = dev(synth.normal(313 + V + N, 0, (beam, 1, batch, V), 3.0))
    path = dev(synth.normal(314 + V, 1, (beam, batch), 1.0))
    with L.forced_kernel(0) as T:
        results = {}
        for fenced in (0, 1):
            prev = T.marian_hip_nbest_set_fenced(fenced)
            try:
                runs = []
                for _ in range(20):
                    v, k = ops.getNBestListOfBeams(x, N)
                    v2, k2 = ops.logsoftmaxNBestOfBeams(x, N, pathScores=path)
                    runs.append((v, k, v2, k2))
                torch.cuda.synchronize()
                results[fenced] = [[t.cpu().numpy() for t in r] for r in runs]
            finally:
                assert T.marian_hip_nbest_set_fenced(prev) == fenced
    first = results[0][0]
    for fenced in (0, 1):
        for r in results[fenced]:
            for got, want in zip(r, first):
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_logsoftmax_nbest_of_beams_argument_checks(ops):
    import torch
    from conftest import load
    L = load("_lib")
    lib = L.lib()
    x = torch.zeros(1, 1, 40000, device="cuda")
    need = lib.marian_hip_nbest_beams_workspace_bytes(1, 1, 5000, 4)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    out = torch.zeros(64, device="cuda")
    call = lambda beam, batch, V, N, wb: lib.marian_hip_logsoftmax_nbest_beams(
        x.data_ptr(), None, None, beam, batch, V, N, out.data_ptr(), out.data_ptr(), ws.data_ptr(), wb, None)
    assert call(1, 1, 5000, 4, need) == L.OK
    assert call(1, 1, 5000, 4, 16) == L.ERR_WORKSPACE
    assert call(4, 2, 100, 4, need) == L.ERR_SHAPE            # short rows: the separate calls
    assert call(1, 1, 5002, 4, need) == L.ERR_SHAPE           # rows of whole 16-byte units only
    assert call(1, 1, 40000, 4, need) == L.ERR_SHAPE          # longer than a workgroup's registers hold
    assert call(1, 1, 5000, 17, need) == L.ERR_SHAPE
    assert call(4, 0, 5000, 4, 0) == L.OK
    torch.cuda.synchronize()


def _random_nbest_cases(n):
    rng = np.random.default_rng(20261127)
    cases = []
    for i in range(n):
        V = int(rng.choice([8, 20, 63, 64, 65, 257, 1000, 4096, 8191, 32000, 50001, 70003]))
        beam = int(rng.integers(1, 13))
        batch = int(rng.integers(1, 41)) if V <= 8191 else int(rng.integers(1, 9))
        N = int(min(rng.integers(1, 17), beam * V))
        cases.append((i, batch, beam, V, N, bool(rng.integers(2))))
    return cases


@pytest.mark.parametrize("i,batch,beam,V,N,coarse", _random_nbest_cases(32))
def test_nbest_random_shapes(ops, synth, i, batch, beam, V, N, coarse):
    """Seeded random shapes through both n-best entry points against a stable sort; 'coarse' rounds
    the scores to one decimal, so that equal scores are everywhere (lowest index first)."""
    x = synth.normal(9000 + i, 0, (beam, 1, batch, V), 2.0)
    if coarse:
        x = np.round(x, 1).astype(np.float32)
    swapped = np.ascontiguousarray(np.swapaxes(x, 0, 2))
    flat = swapped.reshape(batch, -1)
    order = np.argsort(-flat, axis=1, kind="stable")[:, :N]
    want_vals = np.take_along_axis(flat, order, 1)
    want_keys = order + np.arange(batch)[:, None] * flat.shape[1]
    for vals, keys in (ops.getNBestListOfBeams(dev(x), N), ops.getNBestList(dev(swapped), N)):
        assert np.array_equal(vals.cpu().numpy().reshape(batch, N), want_vals)
        assert np.array_equal(keys.cpu().numpy().view(np.uint32).reshape(batch, N).astype(np.int64), want_keys)


def test_nbest_of_beams_argument_checks(ops):
    import torch
    from conftest import load
    lib = load("_lib").lib()
    x = torch.zeros(4, 2, 100, device="cuda")
    out = torch.zeros(8, device="cuda")
    keys = torch.zeros(8, dtype=torch.int32, device="cuda")
    need = lib.marian_hip_nbest_beams_workspace_bytes(4, 2, 100, 4)
    assert need == 4096 * 256 + 2 * 4 * 4 * 8
    ws = torch.full((need,), 255, dtype=torch.uint8, device="cuda")
    assert lib.marian_hip_nbest_beams_workspace_init(ws.data_ptr(), need, None) == 0
    torch.cuda.synchronize()
    assert int(ws.to(torch.int64).sum()) == 0
    call = lambda beam, batch, V, N, w, wb: lib.marian_hip_nbest_beams(x.data_ptr(), beam, batch, V, N, out.data_ptr(),
                                                                       keys.data_ptr(), w, wb, None)
    assert call(4, 2, 100, 4, ws.data_ptr(), need) == 0
    assert call(4, 2, 100, 4, ws.data_ptr(), need - 1) == 4        # workspace too small
    assert call(4, 2, 100, 4, None, need) == 1                     # null workspace
    assert call(4, 2, 100, 17, ws.data_ptr(), need) == 2           # N > 16
    assert call(0, 2, 100, 4, ws.data_ptr(), need) == 2
    assert call(4, 0, 100, 4, ws.data_ptr(), need) == 0            # empty batch: nothing is touched
    torch.cuda.synchronize()


def test_nbest_ties_lowest_index_first(ops):
    t = np.zeros((2, 5000), np.float32)
    t[0, [4000, 17, 2048]] = 3.0
    t[1, :] = -1.0
    vals, keys = ops.getNBestList(dev(t), 4)
    k = keys.cpu().numpy().view(np.uint32).reshape(2, 4)
    assert k[0].tolist() == [17, 2048, 4000, 0] and k[1].tolist() == [5000, 5001, 5002, 5003]


@pytest.mark.parametrize("N", [3, 8, 16])
def test_nbest_when_one_thread_holds_the_best_elements(ops, synth, N):
    """Every 1024th element is large (the kernel gives those to one thread), so the bound taken
    from per-thread bests is loose and many candidates pass; and a row of equal scores, where all
    elements pass.  Results still equal a full sort."""
    x = synth.normal(81, 0, (3, 1, 1, 40000), 1.0)
    x[0, 0, 0, ::1024] += np.float32(50.0)
    x[1, 0, 0, 5::1024] += np.float32(50.0)
    x[2] = np.float32(0.25)
    vals, keys = ops.getNBestList(dev(x), N)
    flat = x.reshape(3, -1)
    order = np.argsort(-flat, axis=1, kind="stable")[:, :N]
    assert np.array_equal(vals.cpu().numpy().reshape(3, N), np.take_along_axis(flat, order, 1))
    assert np.array_equal(keys.cpu().numpy().view(np.uint32).reshape(3, N).astype(np.int64),
                          order + np.arange(3)[:, None] * flat.shape[1])


# ---- the reference's own operator-test vectors (tests/golden/operator_vectors.json): at the
#      margin the reference test allows, and at this file's own bar against float64 ----------------

def reference_vectors():
    import json
    import os
    return json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "operator_vectors.json")))


def test_reference_softmax_logsoftmax_vectors(ops):
    v = reference_vectors()["softmax_logsoftmax"]
    x = np.array(v["in"], np.float32).reshape(v["shape"])
    sm = ops.softmax(dev(x)).cpu().numpy()
    lsm = ops.logsoftmax(dev(x)).cpu().numpy()
    assert sm.shape == tuple(v["shape"]) and lsm.shape == tuple(v["shape"])
    assert np.all(np.abs(sm.ravel() - np.array(v["softmax"])) <= v["margin"])
    assert np.all(np.abs(lsm.ravel() - np.array(v["logsoftmax"])) <= v["margin"])
    xs = x.astype(f64)
    e = np.exp(xs - xs.max(-1, keepdims=True))
    close(sm, e / e.sum(-1, keepdims=True), REL, 1e-7)
    close(lsm, xs - xs.max(-1, keepdims=True) - np.log(e.sum(-1, keepdims=True)), REL, 1e-6)


def test_reference_layer_norm_vector(ops):
    v = reference_vectors()["layer_norm"]
    x = np.array(v["in"], np.float32).reshape(v["shape"])
    g, b = np.array(v["gamma"], np.float32), np.array(v["beta"], np.float32)
    xs = x.astype(f64)
    num = xs - xs.mean(-1, keepdims=True)
    want = g.astype(f64) * (num / np.sqrt((num ** 2).mean(-1, keepdims=True) + v["eps"])) + b.astype(f64)
    got = ops.layerNorm(dev(x), dev(g), dev(b), v["eps"]).cpu().numpy()
    assert got.shape == tuple(v["shape"])
    assert np.all(np.abs(got - want) <= v["margin"])
    close(got, want, REL, 2e-6)


def test_reference_bdot_vectors(ops):
    v = reference_vectors()["bdot"]
    A = np.array(v["A"], np.float32).reshape(v["A_shape"])
    B = np.array(v["B"], np.float32).reshape(v["B_shape"])
    C = np.array(v["C"], np.float32).reshape(v["C_shape"])
    Ct = np.array(v["C_transB"], np.float32).reshape(v["C_shape"])
    for i in range(2):   # (the legacy product pairs batch entries by modulo: entry i of A meets all of B)
        assert np.array_equal(ops.bdot_legacy(dev(A[i]), dev(B[0])).cpu().numpy(), C[i])
        assert np.array_equal(ops.bdot_legacy(dev(A[i]), dev(B[0]), transB=True).cpu().numpy(), Ct[i])


def test_reference_topk_vectors(ops):
    v = reference_vectors()["topk"]
    x = np.array(v["in"], np.float32).reshape(-1, v["shape"][-1])
    vals, keys = ops.getNBestList(dev(x), v["k"])
    assert np.array_equal(vals.cpu().numpy(), np.array(v["values"], np.float32))
    rows = np.repeat(np.arange(x.shape[0]), v["k"])
    assert np.array_equal(keys.cpu().numpy().astype(np.int64) - rows * x.shape[1], np.array(v["indices"]))
    # the same rows as the beam-major form sees them: beam 1, batch 4, vocabulary 3
    vals2, keys2 = ops.getNBestListOfBeams(dev(x.reshape(1, 1, 4, 3)), v["k"])
    assert np.array_equal(vals2.cpu().numpy(), vals.cpu().numpy())
    assert np.array_equal(keys2.cpu().numpy(), keys.cpu().numpy())


def test_reference_rows_vectors(ops):
    import torch
    v = reference_vectors()["rows"]
    A = np.array(v["A"], np.float32).reshape(v["A_shape"])
    for case in v["cases"]:
        ids = torch.tensor(case["indices"], dtype=torch.int32, device="cuda")
        got = ops.rows(dev(A), ids).cpu().numpy()
        assert got.shape == (len(case["indices"]), 3)
        assert np.array_equal(got.ravel(), np.array(case["out"], np.float32))


@pytest.mark.parametrize("vocab,d,shape,n_sig,rps", [(32000, 1024, (128,), 1, 1), (32000, 1024, (21, 32), 21, 32),
                                                     (500, 1023, (7, 3), 7, 3), (77, 6, (40,), 3, 8),
                                                     (1000, 512, (2048,), 4, 1), (64, 8196, (5,), 0, 1),
                                                     (9, 64, (3000,), 2, 1500)])
def test_scaled_embeddings_bit_for_bit(ops, chk, integer, synth, vocab, d, shape, n_sig, rps):
    """the embedding step through the library equals the checker's two float operations per value
    bit for bit, for decoding-step and whole-sentence shapes, rows that are not a multiple of four
    wide (the scalar kernel), int32 and int64 indices, ids past the table clamped to its last row;
    the abs-max slots it leaves are those of a scan of its output"""
    import torch
    E = synth.normal(vocab + d, 0, (vocab, d), 0.05)
    n = int(np.prod(shape))
    ids = (synth.normal(n, 1, (n,), 1e4).astype(np.int64) % vocab).astype(np.int64)
    ids[::5] = vocab - 1
    sig = chk.sinusoidal_position_embeddings(n_sig, d, 3) if n_sig else None
    scale = np.float32(np.sqrt(np.float32(d)))
    want = chk.embed(E, ids, scale, sig, rps)
    dE, dsig = dev(E), (None if sig is None else dev(sig))
    for dtype in (torch.int32, torch.int64):
        got = ops.scaledEmbeddings(dE, torch.from_numpy(ids).to(dtype).cuda().reshape(shape), scale, dsig, rps)
        assert tuple(got.shape) == tuple(shape) + (d,)
        assert np.array_equal(got.cpu().numpy().reshape(n, d), want)
    chunks = (d + 4095) // 4096     # a slot per 4096 values of a row
    if n * chunks <= 2048:
        got, gmax = ops.scaledEmbeddings(dE, torch.from_numpy(ids).cuda(), scale, dsig, rps, want_absmax=True)
        assert np.array_equal(got.cpu().numpy(), want)
        slots = gmax.data.cpu().numpy()
        padded = np.zeros((n, chunks * 4096), np.float32)
        padded[:, :d] = np.abs(want)
        assert np.array_equal(slots[:n * chunks], padded.reshape(n * chunks, 4096).max(-1)) and not slots[n * chunks:].any()
    far = torch.tensor([vocab, 2 ** 31 - 1, 0], dtype=torch.int64, device="cuda")
    got = ops.scaledEmbeddings(dE, far, 1.0).cpu().numpy()
    assert np.array_equal(got, E[[vocab - 1, vocab - 1, 0]])


@pytest.mark.parametrize("hyps,row", [(128, 16 * 21 * 64), (12, 4096 * 3 + 4), (40, 8193), (5, 4096), (3, 70001)])
def test_rows_of_a_decoder_state(ops, synth, hyps, row):
    """rows() as the beam search uses it between two steps: the cached positions of the surviving
    hypotheses, one long row each (split over several workgroups), picked by their back-pointers -
    a pure copy, so the result is the numpy gather bit for bit"""
    import torch
    state = synth.normal(hyps + row, 0, (hyps, row), 1.0)
    back = (synth.normal(hyps, 1, (hyps,), 1e3).astype(np.int64) % hyps)
    got = ops.rows(dev(state), torch.from_numpy(back).cuda())
    assert tuple(got.shape) == (hyps, row)
    assert np.array_equal(got.cpu().numpy(), state[back])


def test_scaled_embeddings_feed_the_first_affine_call(ops, integer, synth):
    """an affine call that takes the abs-max the embedding step leaves gives the bits of the call
    that scans the embeddings itself"""
    import torch
    E = dev(synth.normal(61, 0, (4000, 1024), 0.05))
    ids = torch.arange(0, 128 * 31, 31, dtype=torch.int32, device="cuda")
    sig = ops.sinusoidalPositionEmbeddings(1, 1024, 9, device="cuda")
    x, xmax = ops.scaledEmbeddings(E, ids, 32.0, sig, 128, want_absmax=True)
    Bq = integer.prepareB(torch.randn(1024, 1024, device="cuda") * 0.02)
    got, aq = integer.affine_f32(x, Bq, None, absmax=xmax)
    want, aq_ref = integer.affine_f32(x, Bq, None)
    assert np.array_equal(aq.numpy(), aq_ref.numpy()) and np.array_equal(got.cpu().numpy(), want.cpu().numpy())


def test_scaled_embeddings_argument_checks(ops):
    import torch
    mh = load("_lib").MarianHipError
    E = torch.zeros(10, 8, device="cuda")
    with pytest.raises(mh):
        ops.scaledEmbeddings(E, torch.zeros(3, device="cuda"))             # float indices
    with pytest.raises(mh):
        ops.scaledEmbeddings(E.view(2, 5, 8), torch.zeros(3, dtype=torch.int32, device="cuda"))
    with pytest.raises(mh):
        ops.scaledEmbeddings(E, torch.zeros(3, dtype=torch.int32))           # indices on the host
    assert tuple(ops.scaledEmbeddings(E, torch.zeros(0, dtype=torch.int32, device="cuda")).shape) == (0, 8)


@pytest.mark.parametrize("rows,cols", [(3000, 512), (300, 768), (70, 1024), (2048, 256), (9, 4)])
def test_layer_norm_one_wave_per_row(ops, chk, synth, rows, cols):
    """rows of up to 1024 values take the kernel that gives a row to one wave: scale and shift as
    vectors, as single values and from addresses that are not 16-byte aligned (the workgroup-per-row
    kernel behind the same entry point), with and without the skip input; the abs-max slots are
    those of a scan of the output, zero past the last row"""
    import torch
    x = synth.normal(rows + cols, 0, (rows, cols), 1.5) - np.float32(0.2)
    add = synth.normal(rows + cols, 1, (rows, cols), 0.7)
    g = synth.normal(cols, 2, (cols + 1,), 0.2) + np.float32(1.0)
    b = synth.normal(cols, 3, (cols + 1,), 0.5)

    def want(g_, b_, add_):
        xs = (x if add_ is None else x + add_).astype(f64)
        mean = xs.mean(-1, keepdims=True)
        var = ((xs - mean) ** 2).mean(-1, keepdims=True)
        return g_.astype(f64) * (xs - mean) / np.sqrt(var + 1e-6) + (0 if b_ is None else b_.astype(f64))
    dg, db = dev(g), dev(b)
    for g_, b_, add_, dg_, db_ in ((g[:cols], b[:cols], add, dg[:cols], db[:cols]),
                                   (g[1:], b[1:], None, dg[1:], db[1:]),            # 4 bytes off a 16-byte boundary
                                   (g[:1], None, add, dg[:1], None),
                                   (g[:cols], b[:1], None, dg[:cols], db[:1])):
        got = ops.layerNorm(dev(x), dg_, db_, 1e-6, None if add_ is None else dev(add_))
        close(got.cpu().numpy(), want(g_, b_, add_), REL, 2e-6)
        close(got.cpu().numpy(), chk.layer_norm(x, g_, b_, 1e-6, add=add_), 2 * REL, 4e-6)
    if rows <= 2048:
        y, ymax = ops.layerNorm(dev(x), dg[:cols], db[:cols], 1e-6, dev(add), want_absmax=True)
        slots = ymax.data.cpu().numpy()
        assert np.array_equal(slots[:rows], np.abs(y.cpu().numpy()).max(-1)) and not slots[rows:].any()
    # in place: the output may be the input
    xin = dev(x)
    ref = ops.layerNorm(xin, dg[:cols], db[:cols], 1e-6).cpu().numpy()
    L = load("_lib")
    st = L.lib().marian_hip_layer_norm(xin.data_ptr(), None, dg.data_ptr(), cols, db.data_ptr(), cols, xin.data_ptr(),
                                       rows, cols, 1e-6, None, None)
    torch.cuda.synchronize()
    assert st == 0 and np.array_equal(xin.cpu().numpy(), ref)


@pytest.mark.parametrize("BQ,BKV,L,cap,dk,masked,append", [(2048, 2048, 21, 32, 64, False, True), (96, 24, 40, 64, 64, True, False),
                                                           (30, 30, 7, 7, 64, False, True), (16, 16, 5, 9, 32, False, True),
                                                           (12, 4, 70, 100, 20, True, False), (8, 8, 1, 4, 64, False, True)])
def test_attention_on_caches_with_room_to_grow(ops, synth, BQ, BKV, L, cap, dk, masked, append):
    """keys and values in [entries, capacity, dk] tensors of which the first L positions are in use
    give the bits of the call on [entries, L, dk] tensors, whatever the rest of the cache holds;
    the appended position lands at L - 1 of the roomy cache and nothing else in it changes"""
    import torch
    q = dev(synth.normal(BQ + L, 0, (BQ, 1, dk), 1.0))
    k = synth.normal(BQ + L, 1, (BKV, L, dk), 1.0)
    v = synth.normal(BQ + L, 2, (BKV, L, dk), 1.0)
    roomy_k = synth.normal(BQ + L, 3, (BKV, cap, dk), 50.0)
    roomy_v = synth.normal(BQ + L, 4, (BKV, cap, dk), 50.0)
    roomy_k[:, :L], roomy_v[:, :L] = k, v
    mask = None
    if masked:
        lens = 1 + (np.arange(BKV) * 5) % L
        mask = dev(((np.arange(L)[None, :] >= lens[:, None]) * -99999999.0).astype(np.float32))
    kn = dev(synth.normal(BQ + L, 5, (BQ, dk), 1.0)) if append else None
    vn = dev(synth.normal(BQ + L, 6, (BQ, dk), 1.0)) if append else None
    dk_, dv_ = dev(k), dev(v)
    want = ops.Attention(q, dk_, dv_, mask, kNew=kn, vNew=vn)
    rk, rv = dev(roomy_k), dev(roomy_v)
    got = ops.Attention(q, rk, rv, mask, kNew=kn, vNew=vn, kvLen=L)
    assert torch.equal(got, want)
    if append:
        roomy_k[:, L - 1], roomy_v[:, L - 1] = kn.cpu().numpy(), vn.cpu().numpy()
        assert np.array_equal(rk.cpu().numpy(), roomy_k) and np.array_equal(rv.cpu().numpy(), roomy_v)
        assert torch.equal(dk_[:, L - 1], kn) and torch.equal(dv_[:, L - 1], vn)


@pytest.mark.parametrize("entries,rows,segs,cap,used", [(1536, 1536, 16, 21 * 64, 20 * 64), (30, 45, 4, 8 * 64, 3 * 64),
                                                        (7, 7, 3, 10, 7), (12, 5, 2, 5000 * 4, 4097 * 4), (9, 9, 16, 64, 0),
                                                        (4, 6, 1, 4096, 4096)])
def test_select_state_copies_the_positions_in_use(ops, synth, entries, rows, segs, cap, used):
    """the state selection between two beam-search steps on states with room to grow: the values in
    use of every segment of the chosen entries, bit for bit; what lies behind them in the output is
    left as it was"""
    import torch
    state = synth.normal(entries + cap, 0, (entries, segs, cap), 1.0)
    back = synth.normal(rows, 1, (rows,), 1e3).astype(np.int64) % entries
    old = synth.normal(entries + cap, 2, (rows, segs, cap), 1.0)
    out = dev(old)
    ops.selectState(dev(state), torch.from_numpy(back).cuda(), out, used=used)
    want = old.copy()
    want[:, :, :used] = state[back][:, :, :used]
    assert np.array_equal(out.cpu().numpy(), want)
    L = load("_lib")
    s = dev(state)
    assert L.lib().marian_hip_select_state(s.data_ptr(), s.data_ptr(), 1, entries, segs, cap, used, s.data_ptr(), None) == (L.ERR_ALIAS if used else L.OK)


@pytest.mark.parametrize("hyps,heads,L,cap", [(128, 16, 21, 21), (128, 16, 21, 40), (12, 4, 70, 100), (6, 2, 1, 3),
                                              (9, 3, 64, 64), (5, 8, 65, 66), (20, 1, 130, 140)])
def test_attention_by_ancestors_is_attention_on_gathered_caches(ops, synth, hyps, heads, L, cap):
    """caches that are never moved: cached position p of hypothesis h read from the entry of
    hypothesis ancestors[h, p] gives the bits of the call on caches into which those rows were
    copied first; the new position lands in the hypothesis's own entry and nothing else changes"""
    import torch
    dk, E = 64, hyps * heads
    q = dev(synth.normal(E + L, 0, (E, 1, dk), 1.0))
    k = synth.normal(E + L, 1, (E, cap, dk), 1.0)
    v = synth.normal(E + L, 2, (E, cap, dk), 1.0)
    kn, vn = synth.normal(E + L, 3, (E, dk), 1.0), synth.normal(E + L, 4, (E, dk), 1.0)
    anc = (synth.normal(E + L, 5, (hyps, cap), 1e3).astype(np.int64) % hyps).astype(np.int32)
    anc[:, L - 1] = np.arange(hyps)
    # gathered caches: entry (h, head), position p <- entry (anc[h, p], head), position p
    kg, vg = k.copy().reshape(hyps, heads, cap, dk), v.copy().reshape(hyps, heads, cap, dk)
    k4, v4 = k.reshape(hyps, heads, cap, dk), v.reshape(hyps, heads, cap, dk)
    for p in range(L - 1):
        kg[:, :, p] = k4[anc[:, p], :, p]
        vg[:, :, p] = v4[anc[:, p], :, p]
    want, wmax = ops.Attention(q, dev(kg.reshape(E, cap, dk)), dev(vg.reshape(E, cap, dk)), kNew=dev(kn), vNew=dev(vn),
                               kvLen=L, want_absmax=E <= 2048) if E <= 2048 else (None, None)
    dk_, dv_ = dev(k), dev(v)
    got, gmax = ops.AttentionByAncestors(q, dk_, dv_, dev(anc), L, dev(kn), dev(vn), want_absmax=True)
    assert torch.equal(got, want) and torch.equal(gmax.data, wmax.data)
    k[:, L - 1], v[:, L - 1] = kn, vn
    assert np.array_equal(dk_.cpu().numpy(), k) and np.array_equal(dv_.cpu().numpy(), v)


def test_advance_ancestors(ops, synth):
    import torch
    hyps, cap = 37, 19
    L = load("_lib")
    for len_prev in (0, 1, 7, 18):
        prev = (synth.normal(len_prev, 0, (hyps, cap), 1e3).astype(np.int64) % hyps).astype(np.int32)
        parents = (synth.normal(len_prev, 1, (hyps,), 1e3).astype(np.int64) % hyps).astype(np.int32)
        old = np.full((hyps, cap), -5, np.int32)
        out = dev(old)
        ops.advanceAncestors(dev(prev), dev(parents), len_prev, out)
        want = old.copy()
        want[:, :len_prev] = prev[parents][:, :len_prev]
        want[:, len_prev] = np.arange(hyps)
        assert np.array_equal(out.cpu().numpy(), want)
    t = dev(prev)
    assert L.lib().marian_hip_ancestors_advance(t.data_ptr(), t.data_ptr(), hyps, cap, 3, t.data_ptr(), None) == L.ERR_ALIAS
    assert L.lib().marian_hip_ancestors_advance(t.data_ptr(), t.data_ptr(), hyps, cap, cap, out.data_ptr(), None) == L.ERR_SHAPE
