"""Two host threads, two streams, one device: the library is re-entrant and takes its stream per
call (reference src/translator/translator.h:158-164: one graph and backend per worker thread,
several workers may share a device).  Each thread runs 200 mixed calls on a stream and workspace
of its own - fused small-M, grouped, the one-pass prepareA at 4096 x 1024, a large-M GEMM, a
shortlisted output layer, log-softmax + n-best - while the other does the same, and every result
is compared with the CPU checker's (n-best: with the separate calls' result taken beforehand);
the run stops at the first mismatch."""
import sys
import threading

import numpy as np
import pytest

from conftest import load

pytestmark = pytest.mark.gpu
f32 = np.float32


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def build_cases(integer, ops, orc, synth, torch, seed):
    """A thread's pool of calls: (name, run() -> list of device tensors, expected host arrays)."""
    T = load("types")
    dev = lambda x: torch.from_numpy(np.ascontiguousarray(x)).cuda()
    cases = []

    def weights(s, K, N):
        W = synth.normal(s, synth.STREAM_W, (K, N), 0.02)
        Bh = orc.prepare_b(W)
        return Bh, integer.prepareAndTransposeB(integer.QTensor.from_numpy(Bh, (K, N), T.Type.intgemm8, "cuda"))

    # fused small-M calls (one kernel) and a quantize-on-stage one
    for i, (M, K, N, relu) in enumerate([(1, 512, 512, False), (16, 512, 1536, True), (64, 512, 2048, False),
                                        (4, 2048, 512, True), (128, 1024, 1024, False)]):
        s = seed + 10 * i
        A = synth.normal(s, synth.STREAM_A, (M, K), 1.0)
        bias = synth.normal(s, synth.STREAM_BIAS, (N,), 0.01)
        Bh, Bq = weights(s, K, N)
        want, _ = orc.affine(orc.prepare_a(A), Bh, bias, M, K, N, 1.0, relu)
        dA, db = dev(A), dev(bias)
        cases.append(("affine_f32 %dx%dx%d" % (M, K, N),
                      (lambda dA=dA, Bq=Bq, db=db, relu=relu: [integer.affine_f32(dA, Bq, db, relu=relu)[0]]),
                      [np.asarray(want, dtype=f32).reshape(M, N)]))
    # three matrices behind one input in one call
    M, K, N = 128, 1024, 1024
    A = synth.normal(seed + 71, synth.STREAM_A, (M, K), 1.0)
    ws3 = [weights(seed + 72 + g, K, N) for g in range(3)]
    b3 = [synth.normal(seed + 75 + g, synth.STREAM_BIAS, (N,), 0.01) for g in range(3)]
    Aq_h = orc.prepare_a(A)
    want3 = [np.asarray(orc.affine(Aq_h, ws3[g][0], b3[g], M, K, N, 1.0, False)[0], dtype=f32).reshape(M, N) for g in range(3)]
    dA, db3 = dev(A), [dev(b) for b in b3]
    cases.append(("grouped 128x1024x3x1024",
                  (lambda dA=dA, ws3=ws3, db3=db3: integer.affine_f32_grouped(dA, [(ws3[g][1], db3[g]) for g in range(3)])[0]),
                  want3))
    # the one-pass prepareA (4 Mi values: all CUs, workgroups exchange their abs-max through the workspace)
    A = synth.normal(seed + 81, synth.STREAM_A, (4096, 1024), 1.0)
    dA = dev(A)
    cases.append(("prepareA 4096x1024",
                  (lambda dA=dA: [integer.prepareA(dA).data[: 4096 * 1024 + 4]]),
                  [orc.prepare_a(A).view(np.int8)]))
    # a large-M GEMM from float32 input (prepareA + tile kernel), ragged on both sides
    M, K, N = 1100, 1024, 1032
    A = synth.normal(seed + 91, synth.STREAM_A, (M, K), 1.0)
    bias = synth.normal(seed + 92, synth.STREAM_BIAS, (N,), 0.01)
    Bh, Bq = weights(seed + 93, K, N)
    want, _ = orc.affine(orc.prepare_a(A), Bh, bias, M, K, N, 1.0, True)
    dA, db = dev(A), dev(bias)
    cases.append(("affine_f32 1100x1024x1032",
                  (lambda dA=dA, Bq=Bq, db=db: [integer.affine_f32(dA, Bq, db, relu=True)[0]]),
                  [np.asarray(want, dtype=f32).reshape(M, N)]))
    # shortlisted output layer
    M, K, N = 64, 512, 8000
    A = synth.normal(seed + 101, synth.STREAM_A, (M, K), 1.0)
    bias = synth.normal(seed + 102, synth.STREAM_BIAS, (N,), 0.01)
    Bh, Bq = weights(seed + 103, K, N)
    idx = synth.shortlist(seed + 104, N, 504, 504)
    want, _ = orc.affine_shortlist(orc.prepare_a(A), Bh, bias, idx, M, K, N, 1.0, False)
    dA, db, didx = dev(A), dev(bias), torch.from_numpy(idx.view(np.int32)).cuda()
    cases.append(("shortlist 64x512x504 of 8000",
                  (lambda dA=dA, Bq=Bq, db=db, didx=didx: [integer.affine_f32(dA, Bq, db, shortlist=didx)[0]]),
                  [np.asarray(want, dtype=f32).reshape(M, idx.size)]))
    # the end of a beam-search step in one launch (workgroups hand candidates over through the n-best
    # workspace of the stream): expected = the separate calls' result, taken before the threads start
    beam, batch, vocab, nb = 4, 8, 8000, 4
    logits = synth.normal(seed + 111, synth.STREAM_A, (beam, 1, batch, vocab), 3.0)
    dl = dev(logits)
    lp = ops.logsoftmax(dl)
    v, k = ops.getNBestListOfBeams(lp, nb)
    torch.cuda.synchronize()
    cases.append(("logsoftmax + n-best 4x8x8000",
                  (lambda dl=dl, nb=nb: list(ops.logsoftmaxNBestOfBeams(dl, nb))),
                  [v.cpu().numpy(), k.cpu().numpy()]))
    return cases


def worker(name, torch, cases, order, stream, failures, burst=8):
    try:
        with torch.cuda.stream(stream):
            done = 0
            while done < len(order) and not failures:
                chunk = order[done: done + burst]
                outs = [(c, cases[c][1]()) for c in chunk]
                stream.synchronize()
                for c, got in outs:
                    for g, want in zip(got, cases[c][2]):
                        gh = g.cpu().numpy().reshape(want.shape)
                        if not np.array_equal(gh.view(np.uint8), want.view(np.uint8)):
                            failures.append("%s: call %d (%s) differs from the checker" % (name, done, cases[c][0]))
                            return
                done += len(chunk)
    except Exception as e:   # noqa: BLE001 - reported by the main thread
        failures.append("%s: %r" % (name, e))


def test_two_threads_two_streams_one_device(integer, orc, synth):
    import torch
    ops = load("ops")
    pools = [build_cases(integer, ops, orc, synth, torch, 31000 + 500 * t) for t in range(2)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    failures = []
    threads = []
    for t in range(2):
        rng = np.random.default_rng(77 + t)
        order = [int(x) for x in rng.integers(len(pools[t]), size=200)]
        say("thread", t, "runs", len(order), "calls over", len(pools[t]), "kinds")
        threads.append(threading.Thread(target=worker, args=("thread %d" % t, torch, pools[t], order, streams[t], failures)))
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=150)
    assert not any(th.is_alive() for th in threads), "a worker did not finish"
    assert not failures, failures[0]
    # the two streams did not share a workspace
    be = integer.Backend.get("cuda:0")
    with torch.cuda.stream(streams[0]):
        w0 = be.workspace.data_ptr()
    with torch.cuda.stream(streams[1]):
        w1 = be.workspace.data_ptr()
    assert w0 != w1
