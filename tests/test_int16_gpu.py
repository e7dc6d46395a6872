"""GPU parity of the 16-bit intgemm path (Type::intgemm16, include/marian_hip_int16.h) against its
CPU checker: quantized operands and quantMult tails bit for bit, int32 accumulators bit for bit
(sums mod 2^32, like pmaddwd + paddd), fp32 outputs bit-identical (two roundings, as on the CPU)."""
import os
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


@pytest.fixture(scope="module")
def o16():
    from oracle import oracle16
    oracle16.lib()
    return oracle16


def qbytes(q16):
    return np.ascontiguousarray(q16).view(np.int8)


@pytest.mark.parametrize("M,K", [(1, 32), (3, 64), (16, 512), (100, 448), (128, 1024), (1000, 1024)])
def test_prepare_a16_bit_exact(integer, o16, synth, M, K):
    T = load("types")
    say("prepare_a16", M, K)
    A = synth.normal(160 + M, synth.STREAM_A, (M, K), 4.0)
    A.flat[0], A.flat[-1] = 40.0, -40.0                       # saturate at both ends of int16
    A.flat[1:4] = [0.5 / 1024, 1.5 / 1024, -2.5 / 1024]        # ties to even
    got = integer.prepareA(dev(A), T.Type.intgemm16)
    assert got.type == T.Type.intgemm16 and got.shape == (M, K)
    assert np.array_equal(got.numpy(), qbytes(o16.prepare_a(A)))
    assert integer.getQuantMult(got) == 1024.0


@pytest.mark.parametrize("K,N", [(32, 8), (64, 24), (512, 2048), (2048, 512), (1024, 1000)])
def test_prepare_b16_bit_exact(integer, o16, synth, K, N):
    T = load("types")
    say("prepare_b16", K, N)
    W = synth.normal(170 + N, synth.STREAM_W, (K, N), 0.5)
    W.flat[5] = 77.0
    got = integer.prepareB(dev(W), T.Type.intgemm16)
    assert np.array_equal(got.numpy(), qbytes(o16.prepare_b(W)))


@pytest.mark.parametrize("kind", ["nan", "pinf", "ninf", "huge"])
def test_prepare_a16_degenerate(integer, o16, kind):
    T = load("types")
    rng = np.random.default_rng(3)
    A = rng.standard_normal((33, 96)).astype(f32)
    A.flat[17] = {"nan": np.nan, "pinf": np.inf, "ninf": -np.inf, "huge": 3e38}[kind]
    A.flat[40] = -3e38
    assert np.array_equal(integer.prepareA(dev(A), T.Type.intgemm16).numpy(), qbytes(o16.prepare_a(A)))


CASES = [(1, 32, 8), (5, 128, 24), (16, 512, 512), (33, 192, 136), (64, 512, 2048), (128, 1024, 1024),
         (100, 2048, 512), (129, 64, 8), (300, 320, 1000), (513, 96, 264), (1024, 1024, 1024)]


@pytest.mark.parametrize("M,K,N", CASES)
def test_affine16_bit_exact(integer, o16, synth, M, K, N):
    T = load("types")
    say("affine16", M, K, N)
    A = synth.normal(180 + M + N, synth.STREAM_A, (M, K), 1.0)
    W = synth.normal(180 + M + N, synth.STREAM_W, (K, N), 0.02)
    bias = synth.normal(180 + M + N, synth.STREAM_BIAS, (N,), 0.01)
    Aq_h, Bq_h = o16.prepare_a(A), o16.prepare_b(W)
    Bq = integer.QTensor.from_numpy(qbytes(Bq_h), (K, N), T.Type.intgemm16, "cuda")
    Aq = integer.QTensor.from_numpy(qbytes(Aq_h), (M, K), T.Type.intgemm16, "cuda")
    relu = M % 2 == 1
    want, want_acc = o16.affine(Aq_h, Bq_h, bias, M, K, N, 0.5, relu)
    assert np.array_equal(integer.multiply_i32(Aq, Bq).cpu().numpy(), want_acc)
    assert np.array_equal(integer.multiply(Aq, Bq, dev(bias), scale=0.5, relu=relu).cpu().numpy(), want)
    # the operator: prepareA node + multiply node, selected by the weight's type
    out = integer.affineOrDot(dev(A), Bq, dev(bias), scale=0.5, relu=relu)
    assert np.array_equal(out.cpu().numpy(), want)
    want_dot, _ = o16.affine(Aq_h, Bq_h, None, M, K, N, 1.0, False)
    assert np.array_equal(integer.dot(dev(A), Bq).cpu().numpy(), want_dot)


def test_multiply16_wraps_like_the_cpu(integer, o16):
    """accumulators beyond int32: the sum is taken mod 2^32, in any order"""
    T = load("types")
    rng = np.random.default_rng(8)
    M, K, N = 70, 256, 72
    A = rng.integers(-32768, 32768, (M, K), dtype=np.int16)
    Bt = rng.integers(-32768, 32768, (N, K), dtype=np.int16)
    A[0, :] = -32768
    Bt[0, :] = -32768
    tail = np.frombuffer(f32(1024.0).tobytes(), np.int16)
    Aq_h, Bq_h = np.concatenate([A.ravel(), tail]), np.concatenate([Bt.ravel(), tail])
    Aq = integer.QTensor.from_numpy(qbytes(Aq_h), (M, K), T.Type.intgemm16, "cuda")
    Bq = integer.QTensor.from_numpy(qbytes(Bq_h), (K, N), T.Type.intgemm16, "cuda")
    assert np.array_equal(integer.multiply_i32(Aq, Bq).cpu().numpy(), o16.multiply_i32(Aq_h, Bq_h, M, K, N))


def test_marian_operator_vectors_through_the_16_bit_path(integer, o16):
    """reference src/tests/units/operator_tests.cpp:618-659 padded to the shape rules (K = 32,
    N = 8): small integers are exact at a multiplier of 1024."""
    T = load("types")
    vA = np.zeros((4, 32), f32)
    vA[:, :3] = np.arange(1, 13, dtype=f32).reshape(4, 3)
    vB = np.zeros((32, 8), f32)
    vB[:3, :2] = np.array([[1, -2], [3, 4], [-5, 6]], f32)
    bias = np.zeros(8, f32)
    bias[:2] = 2.0
    Bq = integer.prepareB(dev(vB), T.Type.intgemm16)
    out = integer.affine(dev(vA), Bq, dev(bias)).cpu().numpy()
    assert np.array_equal(out[:, :2], np.array([-6, 26, -9, 50, -12, 74, -15, 98], f32).reshape(4, 2))
    relu = integer.affineWithReluDropout(dev(vA), Bq, dev(bias)).cpu().numpy()
    assert np.array_equal(relu[:, :2], np.array([0, 26, 0, 50, 0, 74, 0, 98], f32).reshape(4, 2))


def test_model_file_item_runs_verbatim(integer, o16, synth, tmp_path):
    """A Type::intgemm16 item of a .bin file goes to the device as stored and multiplies."""
    B = load("binary")
    T = load("types")
    K, N, M = 256, 120, 9
    W = synth.normal(191, synth.STREAM_W, (K, N), 0.02)
    A = synth.normal(191, synth.STREAM_A, (M, K), 1.0)
    path = os.path.join(tmp_path, "m16.bin")
    B.save_items(path, [B.intgemm16_item("decoder_l1_ffn_W1", o16.prepare_b(W), (K, N))])
    (item,) = B.load_items(path)
    Bq = integer.QTensor.from_numpy(item.bytes, item.shape, item.type, "cuda")
    want, _ = o16.affine(o16.prepare_a(A), o16.prepare_b(W), None, M, K, N)
    assert np.array_equal(integer.dot(dev(A), Bq).cpu().numpy(), want)


def test_16_bit_argument_checks(integer):
    L = load("_lib")
    lib = L.lib()
    buf = 0x1000
    assert lib.marian_hip_int16_affine(buf, buf, None, buf, 1, 48, 8, 1.0, 0, None) == L.ERR_SHAPE     # K % 32
    assert lib.marian_hip_int16_affine(buf, buf, None, buf, 1, 64, 12, 1.0, 0, None) == L.ERR_SHAPE    # N % 8
    assert lib.marian_hip_int16_affine(None, buf, None, buf, 1, 64, 8, 1.0, 0, None) == L.ERR_NULL
    assert lib.marian_hip_int16_affine(buf + 2, buf, None, buf, 1, 64, 8, 1.0, 0, None) == L.ERR_ALIGN
    assert lib.marian_hip_int16_affine(buf, buf, None, buf, 0, 64, 8, 1.0, 0, None) == L.OK
    assert lib.marian_hip_int16_prepare_a(buf, buf, 2, 40, None) == L.ERR_SHAPE
    assert lib.marian_hip_int16_prepare_b(buf, None, 64, 8, None) == L.ERR_NULL
