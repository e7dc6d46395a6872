"""The library's calls recorded into a HIP graph: every replay gives the eager result.

The calls allocate nothing and clear what must start from zero with kernels (abs-max slots, the
counters of the split n-best), so a captured sequence is replayable as often as wanted.  The graph
is replayed several times with eager work of the same library and synchronisations in between,
and every replay is compared with the eager results, bit for bit."""
import numpy as np
import pytest

from conftest import load

pytestmark = pytest.mark.gpu


def test_decoder_tail_replays(integer, synth):
    import torch
    ops = load("ops")
    M, K, V, beam, batch = 32, 512, 4104, 4, 8
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    x = torch.randn(M, K, device="cuda", generator=g)
    skip = torch.randn(M, K, device="cuda", generator=g)
    gamma = torch.randn(K, device="cuda", generator=g) * 0.1 + 1.0
    beta = torch.randn(K, device="cuda", generator=g) * 0.1
    W1 = integer.prepareB(torch.randn(K, K, device="cuda", generator=g) * 0.02)
    b1 = torch.randn(K, device="cuda", generator=g) * 0.01
    Wv = integer.prepareB(torch.randn(K, V, device="cuda", generator=g) * 0.02)
    bv = torch.randn(V, device="cuda", generator=g) * 0.01

    def step():
        # layer norm (leaves the abs-max of its output) -> chained affine + ReLU -> affine over the
        # vocabulary -> log-softmax -> transposition + n-best of the beam
        h, hmax = ops.layerNorm(x, gamma, beta, 1e-6, skip, want_absmax=True)
        h1, _, h1max = integer.affine_f32(h, W1, b1, relu=True, absmax=hmax, want_absmax=True)
        logits, _ = integer.affine_f32(h1, Wv, bv, absmax=h1max)
        lp = ops.logsoftmax(logits)
        vals, keys = ops.getNBestListOfBeams(lp.view(beam, 1, batch, V), beam)
        # ... and log-softmax + n-best once more as one launch (the same workspace, the same counters)
        vals1, keys1 = ops.logsoftmaxNBestOfBeams(logits.view(beam, 1, batch, V), beam)
        return lp, vals, keys, vals1, keys1

    want = [t.clone() for t in step()]
    assert torch.equal(want[1], want[3]) and torch.equal(want[2], want[4])
    torch.cuda.synchronize()

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        step()   # warm up on the capture stream (module load, workspaces)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for replay in range(4):
        for t in outs:
            t.fill_(float("nan")) if t.is_floating_point() else t.fill_(-1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, w in zip(outs, want):
            assert torch.equal(got, w), "replay %d differs from the eager result" % replay
        # eager work of the same kind between the replays (shares the n-best workspace)
        other = step()
        torch.cuda.synchronize()
        for got, w in zip(other, want):
            assert torch.equal(got, w)


def test_one_pass_prepare_a_replays_with_new_inputs(integer, orc, synth):
    """The one-pass prepareA hands the abs-max between its workgroups through tagged words in the
    workspace.  A recorded graph repeats the host's part of the tag on every replay, so words left
    by the previous replay must not be taken for this one's: the input changes between replays
    (another abs-max, at another place) and every replay must give the checker's bytes.  The same
    workspace also serves eager calls in between."""
    import torch
    from conftest import load
    T = load("types")
    M, K = 4096, 1024     # 4 M values: the one-pass form, all CUs
    inputs = []
    for r in range(4):
        A = synth.normal(70 + r, synth.STREAM_A, (M, K), 1.0 + r)
        A.flat[(r * 7919 + 13) % A.size] = np.float32(50.0 * (r + 1)) * (-1 if r % 2 else 1)
        inputs.append(A)
    want = [orc.prepare_a(A) for A in inputs]
    dA = torch.from_numpy(inputs[0]).cuda()
    out = integer.QTensor.empty((M, K), T.Type.intgemm8, "cuda")
    be = integer.Backend.get(dA.device)

    def call():
        st = be.lib.marian_hip_int8_prepare_a(dA.data_ptr(), out.data_ptr(), M, K, be.workspace.data_ptr(),
                                              be.workspace_bytes, be.stream())
        assert st == 0

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        call()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for replay in range(8):
        r = replay % 4
        dA.copy_(torch.from_numpy(inputs[r]).cuda())
        out.data.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.numpy(), want[r]), "replay %d" % replay
        if replay % 2:    # an eager call on another input, same workspace
            other = integer.prepareA(torch.from_numpy(inputs[(r + 1) % 4]).cuda())
            assert np.array_equal(other.numpy(), want[(r + 1) % 4])


def test_beam_step_on_unmoved_caches_replays(integer, synth):
    """embedding -> table of ancestors advanced -> self-attention that follows it (appending the
    new position) -> the copy form of the same selection, recorded once: every replay gives the
    eager results, with eager calls of the same kind in between.  (The replays start from the same
    caches: the appended position is rewritten with the same values.)"""
    import torch
    ops = load("ops")
    hyps, heads, cap, L, dk, vocab = 12, 4, 9, 6, 64, 300
    g = torch.Generator(device="cuda")
    g.manual_seed(9)
    E = torch.randn(vocab, heads * dk, device="cuda", generator=g)
    words = torch.randint(0, vocab, (hyps,), device="cuda", generator=g).to(torch.int32)
    signal = ops.sinusoidalPositionEmbeddings(1, heads * dk, L - 1, device="cuda")
    k = torch.randn(hyps * heads, cap, dk, device="cuda", generator=g)
    v = torch.randn(hyps * heads, cap, dk, device="cuda", generator=g)
    prev = torch.randint(0, hyps, (hyps, cap), device="cuda", generator=g).to(torch.int32)
    parents = torch.randint(0, hyps, (hyps,), device="cuda", generator=g).to(torch.int32)
    nxt = torch.empty_like(prev)
    k2, v2 = torch.empty_like(k), torch.empty_like(v)

    def step():
        x, xmax = ops.scaledEmbeddings(E, words, 16.0, signal, hyps, want_absmax=True)
        q = x.view(hyps * heads, 1, dk)
        ops.advanceAncestors(prev, parents, L - 1, nxt)
        o = ops.AttentionByAncestors(q, k, v, nxt, L, x.view(hyps * heads, dk), x.view(hyps * heads, dk))
        ops.selectState(k.view(hyps, heads, cap * dk), parents, k2.view(hyps, heads, cap * dk), used=(L - 1) * dk)
        ops.selectState(v.view(hyps, heads, cap * dk), parents, v2.view(hyps, heads, cap * dk), used=(L - 1) * dk)
        return x, xmax.data, o, nxt, k2, v2

    k2.zero_(); v2.zero_()
    want = [t.clone() for t in step()]
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        step()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for replay in range(4):
        for t in outs[:3]:
            t.fill_(float("nan"))
        nxt.fill_(-1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, (got, w) in enumerate(zip(outs, want)):
            if i == 3:   # (the table's columns past the positions in use are not written)
                assert torch.equal(got[:, :L], w[:, :L])
            else:
                assert torch.equal(got, w), "replay %d, output %d differs from the eager result" % (replay, i)
        other = step()
        torch.cuda.synchronize()
        assert torch.equal(other[2], want[2])
