"""The entry point that allocates nothing (marian_hip_int8_affine_f32_static): its output equals
that of marian_hip_int8_affine_f32, bit for bit, and the CPU checker's, on two calls in a row that
share the library's static scratch - the second with a smaller input, so that stale bytes of the
first call lie behind the ones it uses."""
import ctypes
import sys

import numpy as np
import pytest

from conftest import load

f32 = np.float32


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def test_static_limit_is_refused_before_any_device_work():
    L = load("_lib")
    lib = L.lib()
    buf = 0x1000   # never dereferenced
    too_many = L.STATIC_MAX_ELEMS // 64 + 1
    assert lib.marian_hip_int8_affine_f32_static(buf, buf, None, None, 0, buf, too_many, 64, 8, 1.0, 0, None) == L.ERR_STATIC_LIMIT
    assert lib.marian_hip_int8_affine_f32_static(buf, buf, None, None, 0, buf, 4, 100, 8, 1.0, 0, None) == L.ERR_SHAPE
    assert lib.marian_hip_int8_affine_f32_static(buf, buf, None, None, 0, buf, 0, 64, 8, 1.0, 0, None) == L.OK
    assert b"MARIAN_HIP_STATIC_MAX_ELEMS" in lib.marian_hip_status_string(L.ERR_STATIC_LIMIT)


CASES = [
    # (first call, then a smaller one): M, K, N, bias, relu, shortlist length
    ((300, 1024, 512, True, True, 0), (16, 256, 64, True, False, 0)),       # two launches, then one fused kernel
    ((128, 1024, 1024, True, False, 0), (64, 512, 2048, False, True, 0)),   # abs-max launch + quantize-on-stage, then fused
    ((1024, 2048, 1024, True, True, 0), (256, 1024, 32000, True, False, 1000)),   # large-M kernel, then shortlisted output layer
    # 4 Mi values and more: the one-pass prepareA, whose workgroups exchange their abs-max through
    # words of the static workspace that persist from call to call (arrival slots, generation word,
    # mailboxes) - twice in a row on different inputs, a two-set input, then a small call
    ((4096, 1024, 256, True, True, 0), (4096, 1024, 264, True, False, 0), (2048, 4096, 128, False, True, 0),
     (64, 512, 512, True, False, 0)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("calls", CASES)
def test_static_entry_point_matches_affine_f32(integer, orc, synth, calls):
    import torch
    L = load("_lib")
    T = load("types")
    lib = L.lib()
    be = integer.Backend.get(torch.device("cuda", torch.cuda.current_device()))
    for call, (M, K, N, bias_on, relu, n_sl) in enumerate(calls):
        say("static affine call", call, M, K, N, bias_on, relu, n_sl)
        seed = 4100 + M + N + 7 * call
        A = synth.normal(seed, synth.STREAM_A, (M, K), 1.0)
        W = synth.normal(seed, synth.STREAM_W, (K, N), 0.02)
        bias = synth.normal(seed, synth.STREAM_BIAS, (N,), 0.01) if bias_on else None
        idx = None
        if n_sl:
            idx = np.sort(np.random.default_rng(seed).choice(N, size=n_sl, replace=False)).astype(np.uint32)
        n_out = n_sl if n_sl else N
        Bq_h = orc.prepare_b(W)
        Bq = integer.prepareAndTransposeB(integer.QTensor.from_numpy(Bq_h, (K, N), T.Type.intgemm8, "cuda"))
        dA = torch.from_numpy(A).cuda()
        dbias = None if bias is None else torch.from_numpy(bias).cuda()
        didx = None if idx is None else torch.from_numpy(idx.view(np.int32)).cuda()
        want_dev, _ = integer.affine_f32(dA, Bq, dbias, relu=relu, shortlist=didx)
        got = torch.full((M, n_out), float("nan"), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        st = lib.marian_hip_int8_affine_f32_static(
            dA.data_ptr(), Bq.data_ptr(), None if dbias is None else dbias.data_ptr(),
            None if didx is None else didx.data_ptr(), n_sl, got.data_ptr(), M, K, N, 1.0, int(relu),
            be.stream())
        L.check(st, "affine_f32_static")
        torch.cuda.synchronize()
        got_h, want_h = got.cpu().numpy(), want_dev.cpu().numpy()
        assert np.array_equal(got_h.view(np.uint32), want_h.view(np.uint32)), "differs from affine_f32"
        Aq_h = orc.prepare_a(A)
        if idx is None:
            ref, _ = orc.affine(Aq_h, Bq_h, bias, M, K, N, 1.0, relu)
        else:
            ref, _ = orc.affine_shortlist(Aq_h, Bq_h, bias, idx, M, K, N, 1.0, relu)
        assert np.array_equal(got_h.view(np.uint32), np.asarray(ref, dtype=f32).reshape(M, n_out).view(np.uint32)), "differs from the CPU checker"
