"""Degenerate inputs through the HIP path and the CPU checker: all-zero activations (quantMult =
inf, every product NaN), NaN and +-Inf among the activations, abs-max so small that the quantMult
overflows, all-zero weights.  What the real intgemm binary does with them is not pinned (its
source is absent); the checker follows the x86 conversions (cvtps2dq gives "integer indefinite"
for NaN and out-of-range, the saturating packs and max(-127) turn that into -127), and the HIP
kernels have to agree with the checker bit for bit: quantized operands, quantMult tails, int32
accumulators, and the fp32 outputs (NaN against NaN by position, everything else by bit pattern)."""
import contextlib
import sys

import numpy as np
import pytest

from conftest import load

pytestmark = pytest.mark.gpu
f32 = np.float32


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def dev(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def forced(kernel):
    return load("_lib").forced_kernel(kernel) if kernel else contextlib.nullcontext()


def make_a(kind, M, K, seed):
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((M, K)).astype(f32)
    at = lambda: int(rng.integers(A.size))
    if kind == "zeros":
        A[:] = 0.0
    elif kind == "negzeros":
        A[:] = -0.0
    elif kind == "nan":
        A.flat[at()] = np.nan
    elif kind == "pinf":
        A.flat[at()] = np.inf
    elif kind == "ninf":
        A.flat[at()] = -np.inf
    elif kind == "nan_inf":
        A.flat[at()] = np.nan
        A.flat[at()] = -np.inf
        A.flat[at()] = np.inf
    elif kind == "tiny":        # abs-max below 127 / FLT_MAX: the quantMult overflows to inf
        A *= f32(1e-39)
        A.flat[at()] = 0.0
    elif kind == "huge":        # near FLT_MAX: the quantMult is tiny but normal
        A *= f32(5e37)
    elif kind == "allnan":
        A[:] = np.nan
    else:
        raise ValueError(kind)
    return A


A_KINDS = ["zeros", "negzeros", "nan", "pinf", "ninf", "nan_inf", "tiny", "huge", "allnan"]


def same_bits_or_both_nan(got, want):
    got, want = np.asarray(got, dtype=f32), np.asarray(want, dtype=f32)
    gn, wn = np.isnan(got), np.isnan(want)
    assert np.array_equal(gn, wn), "NaN positions differ: %d vs %d, first %s" % (
        gn.sum(), wn.sum(), np.argwhere(gn != wn)[:3].tolist())
    assert np.array_equal(got.view(np.uint32)[~gn], want.view(np.uint32)[~wn]), "values differ"


def same_qtensor(got, want, what):
    """payload bytes and the quantMult tail (inf, 0 and denormals included) bit for bit"""
    assert np.array_equal(got[:-4], want[:-4]), what + ": payload"
    same_bits_or_both_nan(got[-4:].view(f32), want[-4:].view(f32))


@pytest.mark.parametrize("kind", A_KINDS)
@pytest.mark.parametrize("M,K", [(1, 64), (16, 512), (100, 320), (300, 1024), (2048, 1024)])
def test_prepare_a_degenerate(integer, orc, kind, M, K):
    say("degenerate prepare_a", kind, M, K)
    A = make_a(kind, M, K, 31 + M)
    same_qtensor(integer.prepareA(dev(A)).numpy(), orc.prepare_a(A), "prepareA " + kind)


@pytest.mark.parametrize("kernel", [700, 701])
@pytest.mark.parametrize("kind", A_KINDS)
def test_prepare_a_degenerate_both_forms(integer, orc, kind, kernel):
    """the two-pass and the one-pass form of prepareA at a size both take"""
    say("degenerate prepare_a forms", kind, kernel)
    A = make_a(kind, 1024, 1024, 99)
    with forced(kernel):
        got = integer.prepareA(dev(A)).numpy()
    same_qtensor(got, orc.prepare_a(A), "prepareA %s id %d" % (kind, kernel))


@pytest.mark.parametrize("kind", A_KINDS)
@pytest.mark.parametrize("K,N", [(64, 8), (512, 264), (1024, 1024)])
def test_prepare_b_degenerate(integer, orc, kind, K, N):
    say("degenerate prepare_b", kind, K, N)
    W = make_a(kind, K, N, 57 + N)
    same_qtensor(integer.prepareB(dev(W)).file_bytes(), orc.prepare_b(W), "prepareB " + kind)


# fused call: 0 = shipped library; 600 = separate launches; 611..618 one fused kernel with that K
# split; 620..628 abs-max launch + quantize-on-stage kernel
FUSED_IDS = [0, 600, 611, 612, 614, 618, 620, 621, 622, 624, 628]
FUSED_SHAPES = [(4, 256, 64), (16, 512, 1536), (64, 512, 2048), (128, 1024, 1024), (100, 2048, 512)]


@pytest.mark.parametrize("kernel", FUSED_IDS)
@pytest.mark.parametrize("kind", A_KINDS)
def test_fused_affine_degenerate_activations(integer, orc, synth, kind, kernel):
    T = load("types")
    for (M, K, N) in FUSED_SHAPES:
        say("degenerate fused", kind, kernel, M, K, N)
        A = make_a(kind, M, K, 77 + M + kernel)
        W = synth.normal(91, synth.STREAM_W, (K, N), 0.02)
        bias = synth.normal(91, synth.STREAM_BIAS, (N,), 0.01)
        Aq_h, Bq_h = orc.prepare_a(A), orc.prepare_b(W)
        Bq = integer.prepareAndTransposeB(integer.QTensor.from_numpy(Bq_h, (K, N), T.Type.intgemm8, "cuda"))
        for relu in (False, True):
            want, _ = orc.affine(Aq_h, Bq_h, bias, M, K, N, 0.5, relu)
            with forced(kernel):
                out, Aq = integer.affine_f32(dev(A), Bq, dev(bias), scale=0.5, relu=relu)
                out, got_aq = out.cpu().numpy(), Aq.numpy()
            same_qtensor(got_aq, Aq_h, "fused Aq")
            same_bits_or_both_nan(out, want)


# pre-quantized operands: small-M families, the large-M tiles, the tile-pair kernel
MULT_CASES = [(0, 8, 256, 64), (101, 8, 256, 64), (102, 16, 512, 512), (501, 64, 512, 2048),
              (0, 300, 1024, 512), (301, 512, 1024, 512), (307, 300, 320, 264), (312, 512, 2048, 1024),
              (313, 640, 1024, 1024), (330, 512, 1024, 512), (331, 256, 1280, 512), (0, 4096, 1024, 1024),
              (372, 512, 1024, 512), (376, 300, 1024, 264)]


@pytest.mark.parametrize("kernel,M,K,N", MULT_CASES)
@pytest.mark.parametrize("kind", ["zeros", "nan", "pinf", "nan_inf", "tiny", "allnan"])
def test_multiply_degenerate_activations(integer, orc, synth, kind, kernel, M, K, N):
    """The multiply node on operands whose tails are inf / 0 / NaN-producing: accumulators exact,
    fp32 outputs (inf, NaN, or the bias alone when the unquantization factor is 0) as the checker's."""
    T = load("types")
    say("degenerate multiply", kind, kernel, M, K, N)
    A = make_a(kind, M, K, 13 + M + kernel)
    W = synth.normal(92, synth.STREAM_W, (K, N), 0.02)
    bias = synth.normal(92, synth.STREAM_BIAS, (N,), 0.01)
    Aq_h, Bq_h = orc.prepare_a(A), orc.prepare_b(W)
    Aq = integer.QTensor.from_numpy(Aq_h, (M, K), T.Type.intgemm8, "cuda")
    Bq = integer.prepareAndTransposeB(integer.QTensor.from_numpy(Bq_h, (K, N), T.Type.intgemm8, "cuda"))
    for relu, use_bias in ((False, True), (True, True), (False, False), (True, False)):
        want, want_acc = orc.affine(Aq_h, Bq_h, bias if use_bias else None, M, K, N, 1.0, relu)
        with forced(kernel):
            acc = integer.multiply_i32(Aq, Bq).cpu().numpy()
            out = integer.multiply(Aq, Bq, dev(bias) if use_bias else None, relu=relu).cpu().numpy()
        assert np.array_equal(acc, want_acc)
        same_bits_or_both_nan(out, want)


@pytest.mark.parametrize("kernel,M,K,N", [(0, 16, 512, 512), (620, 128, 1024, 1024), (0, 512, 1024, 512), (330, 512, 1024, 512)])
@pytest.mark.parametrize("wkind", ["zeros", "nan", "pinf", "tiny"])
def test_degenerate_weights(integer, orc, synth, wkind, kernel, M, K, N):
    """All-zero weights (quantMult inf, payload -127 everywhere, unquantization factor 0: the
    output is the bias), NaN/Inf/tiny weights, with ordinary and with all-zero activations."""
    say("degenerate weights", wkind, kernel, M, K, N)
    W = make_a(wkind, K, N, 201 + N)
    bias = synth.normal(93, synth.STREAM_BIAS, (N,), 0.01)
    Bq_h = orc.prepare_b(W)
    Bq = integer.prepareB(dev(W))
    same_qtensor(Bq.file_bytes(), Bq_h, "prepareB " + wkind)
    for akind in ("normal", "zeros"):
        A = synth.normal(94, synth.STREAM_A, (M, K), 1.0) if akind == "normal" else np.zeros((M, K), f32)
        Aq_h = orc.prepare_a(A)
        want, _ = orc.affine(Aq_h, Bq_h, bias, M, K, N, 1.0, False)
        with forced(kernel):
            out, Aq = integer.affine_f32(dev(A), Bq, dev(bias))
            out = out.cpu().numpy()
        same_bits_or_both_nan(out, want)
        if wkind == "zeros":
            assert np.array_equal(out, np.broadcast_to(bias, (M, N))), "zero weights: output is the bias"
