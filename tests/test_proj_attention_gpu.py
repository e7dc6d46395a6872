"""Projection + attention in one launch (marian_hip_int8_proj_attention): against the separate
calls - the grouped int8 affine for q, k, v (or the single one for q), then the attention on the
caches - bit for bit, and the projections against the CPU checker of the int8 path."""
import sys

import numpy as np
import pytest

from conftest import load

pytestmark = pytest.mark.gpu
f32 = np.float32


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def make_weights(integer, orc, synth, torch, seed, K, N, n):
    T = load("types")
    out = []
    for g in range(n):
        W = synth.normal(seed + g, synth.STREAM_W, (K, N), 0.02)
        Bh = orc.prepare_b(W)
        Bq = integer.prepareAndTransposeB(integer.QTensor.from_numpy(Bh, (K, N), T.Type.intgemm8, "cuda"))
        bias = synth.normal(seed + 10 + g, synth.STREAM_BIAS, (N,), 0.01) if g != 1 else None   # (one without bias)
        out.append((Bh, Bq, bias, None if bias is None else torch.from_numpy(bias).cuda()))
    return out


@pytest.mark.parametrize("M,K,heads,T,cap,chained", [(128, 1024, 16, 21, 21, True), (128, 1024, 16, 21, 40, False),
                                                     (37, 512, 8, 1, 4, True), (9, 128, 2, 70, 100, False),
                                                     (64, 256, 4, 130, 130, True)])
def test_self_attention_form_equals_the_separate_calls(integer, orc, synth, M, K, heads, T, cap, chained):
    import torch
    ops = load("ops")
    say("proj + self-attention", M, K, heads, T, cap, chained)
    N = heads * 64
    X = synth.normal(6100 + M, synth.STREAM_A, (M, K), 1.0)
    ws = make_weights(integer, orc, synth, torch, 6200 + M, K, N, 3)
    g = torch.Generator(device="cuda")
    g.manual_seed(6300 + M)
    kc = torch.randn(M * heads, cap, 64, device="cuda", generator=g)
    vc = torch.randn(M * heads, cap, 64, device="cuda", generator=g)
    kc2, vc2 = kc.clone(), vc.clone()
    x = torch.from_numpy(X).cuda()
    xmax = None
    if chained:
        xmax = integer.AbsMax(x.device)
        xmax.data.zero_()
        xmax.data[5] = x.abs().max()
    # separate calls
    (q, k, v), Aq_ref = integer.affine_f32_grouped(x, [(w[1], w[3]) for w in ws], absmax=xmax)
    o_ref, omax_ref = ops.Attention(q.view(M * heads, 1, 64), kc, vc, want_absmax=True, kNew=k.view(M * heads, 64),
                                    vNew=v.view(M * heads, 64), kvLen=T)
    # one launch
    o, Aq, omax, proj = ops.ProjectedAttention(x, [(w[1], w[3]) for w in ws], kc2, vc2, heads, kvLen=T, absmax=xmax,
                                               want_absmax=True, want_projections=True)
    torch.cuda.synchronize()
    assert np.array_equal(Aq.numpy(), Aq_ref.numpy()) and np.array_equal(Aq.numpy(), orc.prepare_a(X))
    for name, got, want in (("q", proj[0], q), ("k", proj[1], k), ("v", proj[2], v)):
        assert torch.equal(got, want), name
    # the projections against the checker
    Aq_h = orc.prepare_a(X)
    for i in range(3):
        want, _ = orc.affine(Aq_h, ws[i][0], ws[i][2], M, K, N, 1.0, False)
        assert np.array_equal(proj[i].cpu().numpy(), np.asarray(want, dtype=f32).reshape(M, N))
    assert torch.equal(kc2, kc) and torch.equal(vc2, vc), "caches after the append"
    assert torch.equal(o.view(-1), o_ref.view(-1)), "attention output"
    assert torch.equal(omax.data, omax_ref.data)
    # without asking for the projections: the same output
    kc3, vc3 = kc.clone(), vc.clone()
    o3, _ = ops.ProjectedAttention(x, [(w[1], w[3]) for w in ws], kc3, vc3, heads, kvLen=T, absmax=xmax)
    assert torch.equal(o3, o) and torch.equal(kc3, kc)


@pytest.mark.parametrize("M,K,heads,batch,L,masked,chained", [(128, 1024, 16, 32, 60, True, True), (128, 1024, 16, 32, 21, False, False),
                                                              (30, 512, 8, 10, 7, True, True), (12, 256, 4, 12, 200, True, False),
                                                              # hypotheses of a sentence in one workgroup: 8, 4, 2 of them; lengths
                                                              # at and past what is staged in LDS; an odd number of sentences
                                                              (64, 256, 4, 8, 96, True, True), (64, 256, 4, 8, 97, True, False),
                                                              (32, 256, 4, 16, 33, True, True), (48, 128, 2, 12, 50, False, True),
                                                              (40, 128, 2, 10, 64, True, False), (20, 128, 2, 5, 30, True, True),
                                                              (128, 1024, 16, 16, 1, True, True),
                                                              # the most LDS the staged form asks for
                                                              (128, 1024, 16, 32, 96, True, False),
                                                              # more workgroups than CUs
                                                              (256, 256, 4, 64, 40, True, True), (512, 128, 2, 64, 20, True, False)])
def test_context_attention_form_equals_the_separate_calls(integer, orc, synth, M, K, heads, batch, L, masked, chained):
    import torch
    ops = load("ops")
    say("proj + context attention", M, K, heads, batch, L, masked, chained)
    N = heads * 64
    X = synth.normal(6500 + M, synth.STREAM_A, (M, K), 1.0)
    ws = make_weights(integer, orc, synth, torch, 6600 + M, K, N, 1)
    g = torch.Generator(device="cuda")
    g.manual_seed(6700 + M)
    kc = torch.randn(batch * heads, L, 64, device="cuda", generator=g)
    vc = torch.randn(batch * heads, L, 64, device="cuda", generator=g)
    kc0, vc0 = kc.clone(), vc.clone()
    mask = None
    if masked:
        lens = torch.randint(max(1, L // 3), L + 1, (batch,), device="cuda", generator=g)
        mask = (torch.arange(L, device="cuda")[None, :] >= lens[:, None]).float() * -99999999.0
    x = torch.from_numpy(X).cuda()
    xmax = None
    if chained:
        xmax = integer.AbsMax(x.device)
        xmax.data.zero_()
        xmax.data[2047] = x.abs().max()
    q, Aq_ref = integer.affine_f32(x, ws[0][1], ws[0][3], absmax=xmax)
    o_ref, omax_ref = ops.Attention(q.view(M * heads, 1, 64), kc, vc, mask, rowsPerMask=heads, want_absmax=True)
    o, Aq, omax, proj = ops.ProjectedAttention(x, [(ws[0][1], ws[0][3])], kc, vc, heads, mask=mask, absmax=xmax,
                                               want_absmax=True, want_projections=True)
    torch.cuda.synchronize()
    assert np.array_equal(Aq.numpy(), Aq_ref.numpy())
    assert torch.equal(proj[0], q)
    want, _ = orc.affine(orc.prepare_a(X), ws[0][0], ws[0][2], M, K, N, 1.0, False)
    assert np.array_equal(q.cpu().numpy(), np.asarray(want, dtype=f32).reshape(M, N))
    assert torch.equal(kc, kc0) and torch.equal(vc, vc0), "complete caches are not written"
    assert torch.equal(o.view(-1), o_ref.view(-1))
    assert torch.equal(omax.data, omax_ref.data)


def _random_context_cases(n, seed):
    rng = np.random.RandomState(seed)
    cases = []
    for i in range(n):
        hyps = int(rng.choice([1, 2, 3, 4, 4, 5, 6, 7, 8, 10, 12]))
        sentences = int(rng.choice([1, 2, 3, 4, 6, 7, 16, 24]))
        heads = int(rng.choice([1, 2, 4]))
        K = int(rng.choice([128, 256, 384]))
        L = int(rng.choice([1, 2, 15, 16, 17, 31, 32, 33, 47, 63, 64, 65, 80, 95, 96, 97, 120]))
        cases.append((i, hyps, sentences, heads, K, L, L + int(rng.randint(0, 5)), bool(rng.randint(0, 2))))
    return cases


@pytest.mark.parametrize("i,hyps,sentences,heads,K,L,cap,masked", _random_context_cases(36, 77))
def test_context_attention_form_random_shapes(integer, orc, synth, i, hyps, sentences, heads, K, L, cap, masked):
    """hypotheses x sentences in every combination the row plan distinguishes (eight, four, two, one
    hypotheses of a sentence per workgroup; staged in LDS or not; caches with room to grow): the one
    launch against Wq's affine call followed by the attention, bit for bit"""
    import torch
    ops = load("ops")
    M = hyps * sentences
    say("proj + context attention, random", i, hyps, sentences, heads, K, L, cap, masked)
    N = heads * 64
    X = synth.normal(7100 + i, synth.STREAM_A, (M, K), 1.0)
    ws = make_weights(integer, orc, synth, torch, 7200 + i, K, N, 1)
    g = torch.Generator(device="cuda")
    g.manual_seed(7300 + i)
    kc = torch.randn(sentences * heads, cap, 64, device="cuda", generator=g)
    vc = torch.randn(sentences * heads, cap, 64, device="cuda", generator=g)
    mask = None
    if masked:
        lens = torch.randint(1, L + 1, (sentences,), device="cuda", generator=g)
        mask = (torch.arange(L, device="cuda")[None, :] >= lens[:, None]).float() * -99999999.0
    x = torch.from_numpy(X).cuda()
    q, Aq_ref = integer.affine_f32(x, ws[0][1], ws[0][3])
    o_ref, omax_ref = ops.Attention(q.view(M * heads, 1, 64), kc, vc, mask, rowsPerMask=heads, want_absmax=True, kvLen=L)
    o, Aq, omax = ops.ProjectedAttention(x, [(ws[0][1], ws[0][3])], kc, vc, heads, kvLen=L, mask=mask, want_absmax=True)
    torch.cuda.synchronize()
    assert np.array_equal(Aq.numpy(), Aq_ref.numpy())
    assert torch.equal(o.view(-1), o_ref.view(-1))
    assert torch.equal(omax.data, omax_ref.data)
    # and the attention alone against the same rows on a cache with a copy per query row (the
    # general kernel: nothing is shared there)
    o_rep = ops.Attention(q.view(M * heads, 1, 64), kc.repeat(hyps, 1, 1), vc.repeat(hyps, 1, 1), mask, rowsPerMask=heads, kvLen=L)
    assert torch.equal(o_rep.view(-1), o_ref.view(-1))


def test_proj_attention_argument_checks(integer):
    import ctypes
    L = load("_lib")
    lib = L.lib()
    buf = 0x10000
    one = (ctypes.c_void_p * 3)(buf, buf, buf)
    call = lambda n, M, K, heads, bkv, ln, cap: lib.marian_hip_int8_proj_attention(
        buf, buf, n, one, None, None, M, K, heads, buf, buf, bkv, ln, cap, None, 0, 0.125, buf, buf, None, None, 0, None)
    assert call(2, 8, 128, 2, 16, 1, 1) == L.ERR_SHAPE        # one or three projections
    assert call(3, 8, 192, 2, 16, 1, 1) == L.ERR_SHAPE        # K % 128
    assert call(3, 8, 2048, 2, 16, 1, 1) == L.ERR_SHAPE       # K <= 1024
    assert call(3, 8, 128, 2, 16, 600, 600) == L.ERR_SHAPE    # len <= 512
    assert call(3, 8, 128, 2, 16, 5, 4) == L.ERR_SHAPE        # capacity < len
    assert call(3, 8, 128, 2, 8, 1, 1) == L.ERR_SHAPE         # self-attention: an entry per query row
    assert call(3, 0, 128, 2, 16, 1, 1) == L.OK               # empty batch
