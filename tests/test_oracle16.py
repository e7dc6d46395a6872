"""Pins the CPU checker of the 16-bit intgemm path (oracle/intgemm16_oracle.c) against what the
mathematics and the reference's own operator vectors fix.  No GPU."""
import numpy as np
import pytest

f32 = np.float32


@pytest.fixture(scope="module")
def o16():
    from oracle import oracle16
    oracle16.lib()
    return oracle16


def test_quantize_hand_vectors(o16):
    g = f32(1.0) / f32(1024.0)                      # one quantization step
    x = np.array([0.0, 0.5, -0.5, 1.0, g, -g,
                  0.5 * g, 1.5 * g, 2.5 * g, -0.5 * g, -1.5 * g,       # ties: to even
                  0.49 * g, 0.51 * g,
                  31.9990234375, 32.0, 40.0, -32.0, -32.0009765625, -40.0,   # saturation at both ends
                  1e30, -1e30, np.inf, -np.inf, np.nan], f32)
    want = [0, 512, -512, 1024, 1, -1,
            0, 2, 2, 0, -2,
            0, 1,
            32767, 32767, 32767, -32768, -32768, -32768,
            -32768, -32768, -32768, -32768, -32768]   # out of int32 / NaN: integer indefinite, packed
    assert o16.quantize(x).tolist() == want


def test_quantize_exact_on_the_grid_and_monotone(o16):
    k = np.arange(-32768, 32768, dtype=np.int64)
    assert np.array_equal(o16.quantize((k / 1024.0).astype(f32)), k.astype(np.int16))
    rng = np.random.default_rng(3)
    x = np.sort(rng.normal(0, 8, 20000).astype(f32))
    q = o16.quantize(x).astype(np.int32)
    assert np.all(np.diff(q) >= 0)
    # round-half-even of the fp32 product, restated in numpy
    assert np.array_equal(q, np.clip(np.rint((x * f32(1024.0)).astype(f32)), -32768, 32767).astype(np.int32))


def test_prepare_b_layout_by_hand(o16):
    W = np.array([[1.0, -2.0, 0.5], [0.25, 3.0, -1.0]], f32)     # K = 2, N = 3
    q = o16.prepare_b(W)
    assert q[:6].tolist() == [1024, 256, -2048, 3072, 512, -1024]   # payload[n * K + k] = W[k, n] * 1024
    assert o16.tail(q, 6) == 1024.0
    a = o16.prepare_a(W)
    assert a[:6].tolist() == [1024, -2048, 512, 256, 3072, -1024] and o16.tail(a, 6) == 1024.0


def test_multiply_wraps_like_pmaddwd_and_paddd(o16):
    rng = np.random.default_rng(5)
    M, K, N = 7, 96, 9
    A = rng.integers(-32768, 32768, (M, K), dtype=np.int16)
    Bt = rng.integers(-32768, 32768, (N, K), dtype=np.int16)
    A[0, :] = -32768
    Bt[0, :] = -32768                                 # 96 * 2^30 overflows int32 many times over
    want = (A.astype(np.int64) @ Bt.astype(np.int64).T) & 0xFFFFFFFF
    got = o16.multiply_i32(A, Bt, M, K, N).astype(np.int64) & 0xFFFFFFFF
    assert np.array_equal(got, want)
    small = rng.integers(-2000, 2000, (M, K), dtype=np.int16)
    smallB = rng.integers(-2000, 2000, (N, K), dtype=np.int16)
    assert np.array_equal(o16.multiply_i32(small, smallB, M, K, N), (small.astype(np.int64) @ smallB.astype(np.int64).T))


def test_marian_dot_and_affine_vectors(o16):
    """reference src/tests/units/operator_tests.cpp:508-534 and :618-659: small integers are exact
    at a multiplier of 1024 (products are multiples of 2^20, the unquantization factor is 2^-20), so
    the 16-bit pipeline has to reproduce the reference's expected outputs exactly."""
    vA = np.arange(1, 13, dtype=f32).reshape(4, 3)
    vB = np.array([[1, 2], [3, 4], [5, 6]], f32)
    vC = np.array([22, 28, 49, 64, 76, 100, 103, 136], f32).reshape(4, 2)
    out, acc = o16.affine(o16.prepare_a(vA), o16.prepare_b(vB), None, 4, 3, 2)
    assert np.array_equal(out, vC) and np.array_equal(acc, (vC * 1024 * 1024).astype(np.int64))
    vB2 = np.array([[1, -2], [3, 4], [-5, 6]], f32)
    vAff = np.array([-6, 26, -9, 50, -12, 74, -15, 98], f32).reshape(4, 2)
    vAffRelu = np.array([0, 26, 0, 50, 0, 74, 0, 98], f32).reshape(4, 2)
    bias = np.full(2, 2.0, f32)
    Aq, Bq = o16.prepare_a(vA), o16.prepare_b(vB2)
    assert np.array_equal(o16.affine(Aq, Bq, bias, 4, 3, 2)[0], vAff)
    assert np.array_equal(o16.affine(Aq, Bq, bias, 4, 3, 2, relu=True)[0], vAffRelu)
    assert np.array_equal(o16.affine(Aq, Bq, None, 4, 3, 2)[0] + bias, vAff)      # affine == dot + bias


def test_affine_closed_form(o16):
    rng = np.random.default_rng(9)
    M, K, N = 5, 64, 16
    A = rng.normal(0, 1, (M, K)).astype(f32)
    W = rng.normal(0, 0.02, (K, N)).astype(f32)
    bias = rng.normal(0, 0.01, N).astype(f32)
    Aq, Bq = o16.prepare_a(A), o16.prepare_b(W)
    out, acc = o16.affine(Aq, Bq, bias, M, K, N, 0.5, True)
    want_acc = Aq[:M * K].reshape(M, K).astype(np.int64) @ Bq[:K * N].reshape(N, K).astype(np.int64).T
    assert np.array_equal(acc, want_acc)
    unquant = f32(f32(f32(1.0) / f32(f32(1024.0) * f32(1024.0))) * f32(0.5))
    y = (acc.astype(f32) * unquant).astype(f32)
    y = (y + bias).astype(f32)
    assert np.array_equal(out, np.where(y > 0, y, f32(0)))
    # close to the float product: 16-bit quantization at 1/1024 is fine-grained
    ref = 0.5 * (A.astype(np.float64) @ W.astype(np.float64)) + bias
    assert np.allclose(out, np.maximum(ref, 0), atol=6e-3)   # (weights of 0.02 sit on a grid of 1/1024)
