"""GPU parity: the HIP path (through the C ABI) against the CPU checker on the same seeded inputs.

Bars: quantized operands, quantMult tails and int32 accumulators bit-exact; fp32 outputs within
1e-5 relative (plus an absolute floor of 1e-6 * unquant * K * 127 that absorbs cancellation
against the bias).  The kernels keep multiply and bias add as separate roundings, so the fp32
outputs are in fact expected to be bit-identical; that stricter check is asserted too.
"""
import os
import sys

import numpy as np
import pytest

from conftest import load

pytestmark = pytest.mark.gpu

f32 = np.float32
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "intgemm8_small.npz")
REL_TOL = 1e-5


def forced(kernel):
    """kernel == 0: the shipped library and its automatic selection.  Other ids pin a kernel
    family, which only the tuning build of the library can do."""
    import contextlib
    from conftest import load
    return load("_lib").forced_kernel(kernel) if kernel else contextlib.nullcontext()


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def dev(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def upload_q(integer, flat, shape):
    from conftest import load
    T = load("types")
    return integer.QTensor.from_numpy(flat, shape, T.Type.intgemm8, "cuda")


def upload_b(integer, flat, shape):
    """Weights as the CPU checker (and a model file) holds them, rows [N, K] + quantMult -> usable B."""
    return integer.prepareAndTransposeB(upload_q(integer, flat, shape))


def assert_close_fp32(got, want, unquant, K):
    floor = 1e-6 * abs(float(unquant)) * K * 127
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    bound = REL_TOL * np.abs(want.astype(np.float64)) + floor
    bad = err > bound
    assert not bad.any(), "max rel err %g at %s" % (float((err / (np.abs(want) + floor)).max()),
                                                     np.argwhere(bad)[:4].tolist())


def inputs(synth, seed, M, K, N):
    A = synth.normal(seed, synth.STREAM_A, (M, K), 1.0)
    W = synth.normal(seed, synth.STREAM_W, (K, N), 0.02)
    bias = synth.normal(seed, synth.STREAM_BIAS, (N,), 0.01)
    return A, W, bias


# ---------------------------------------------------------------- prepareA / prepareB

@pytest.mark.parametrize("M,K", [(1, 64), (1, 512), (3, 128), (16, 512), (64, 512), (100, 448),
                                 (128, 1024), (257, 320), (1000, 1024), (4096, 1024)])
def test_prepare_a_bit_exact(integer, orc, synth, M, K):
    say("prepare_a", M, K)
    A = synth.normal(100 + M, synth.STREAM_A, (M, K), 1.0)
    want = orc.prepare_a(A)
    got = integer.prepareA(dev(A)).numpy()
    assert np.array_equal(got[-4:].view(f32), want[-4:].view(f32)), "quantMult tail"
    assert np.array_equal(got, want)


def test_prepare_a_keeps_leading_dims_and_saturates(integer, orc):
    say("prepare_a 4-d")
    rng = np.random.default_rng(5)
    A = rng.standard_normal((2, 3, 5, 64)).astype(f32)
    A[1, 2, 4, 63] = -77.25   # arg-max is negative and sits in the last element
    q = integer.prepareA(dev(A))
    assert q.shape == (2, 3, 5, 64)
    got = q.numpy()
    assert np.array_equal(got, orc.prepare_a(A))
    assert got[30 * 64 - 1] == -127 and got[:-4].min() == -127


@pytest.mark.parametrize("kernel", [0, 700, 701, 702])
@pytest.mark.parametrize("M,K", [(2048, 1024), (4096, 1024), (4096, 4096), (3001, 1088), (128, 4096), (40, 1024),
                                 (4100, 4096), (1500, 2048)])
def test_prepare_a_one_pass_and_two_pass(integer, orc, synth, M, K, kernel):
    """prepareA at encoder sizes: two passes over the input (id 700), one pass with the abs-max
    exchanged between the workgroups (701; the automatic choice from 4 M values on), and one pass
    in which no workgroup waits for the others and each scans the whole input itself (702, the way
    out of a wait that ran out).  One, two and four 16-value sets per thread, ragged last
    workgroups, inputs beyond what the one-pass form holds (4100 x 4096: two passes whatever the id)."""
    if kernel == 702 and M * K > (4 << 20):
        pytest.skip("every workgroup scanning 16 M values: correct, and slow on purpose")
    say("prepare_a passes", M, K, kernel)
    A = synth.normal(150 + M, synth.STREAM_A, (M, K), 1.0)
    A.flat[(M * 31 + 7) % A.size] = np.float32(-9.5)      # the extreme sits in one workgroup's share
    want = orc.prepare_a(A)
    with forced(kernel):
        got = integer.prepareA(dev(A)).numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("K,N", [(64, 8), (128, 24), (512, 2048), (2048, 512), (1024, 1000)])
def test_prepare_b_bit_exact(integer, orc, synth, K, N):
    say("prepare_b", K, N)
    W = synth.normal(200 + N, synth.STREAM_W, (K, N), 0.02)
    want = orc.prepare_b(W)
    q = integer.prepareB(dev(W))
    assert q.shape == (K, N) and q.prepared
    assert np.array_equal(q.file_bytes(), want)
    # the device bytes are the prepared order of the same values, and the re-tiling of the file
    # order gives the same bytes
    L = load("layout")
    assert np.array_equal(q.numpy().view(np.uint8), L.to_prepared(want, K, N))
    assert np.array_equal(upload_b(integer, want, (K, N)).numpy(), q.numpy())


def _random_prepare_cases(n):
    rng = np.random.default_rng(20261131)
    return [(i, int(rng.choice([1, 2, 5, 31, 64, 100, 511, 512, 513, 1500, 4099])), 64 * int(rng.integers(1, 65)),
             8 * int(rng.integers(1, 600)), float(rng.choice([1e-3, 0.02, 1.0, 300.0])))
            for i in range(n)]


@pytest.mark.parametrize("i,M,K,N,sigma", _random_prepare_cases(20))
def test_prepare_a_and_b_random_shapes(integer, orc, synth, i, M, K, N, sigma):
    """Seeded random shapes and magnitudes through both quantizers; the extreme value sits at a
    random place with a random sign, and exact .5 multiples of the step make ties to round."""
    say("prepare random", i, M, K, N, sigma)
    rng = np.random.default_rng(8000 + i)
    A = synth.normal(8000 + i, synth.STREAM_A, (M, K), sigma)
    peak = np.float32(127.0 * 2.0 ** int(rng.integers(-9, 6)))       # quantMult is a power of two
    A = np.clip(A, -peak, peak)
    A.flat[int(rng.integers(A.size))] = peak if rng.integers(2) else -peak
    ties = rng.integers(A.size, size=min(64, A.size))
    A.flat[ties] = (rng.integers(-126, 126, size=ties.size) + 0.5).astype(f32) * (peak / np.float32(127.0))
    A.flat[int(rng.integers(A.size))] = peak
    got = integer.prepareA(dev(A)).numpy()
    assert np.array_equal(got, orc.prepare_a(A))
    W = synth.normal(8000 + i, synth.STREAM_W, (K, N), sigma)
    W.flat[int(rng.integers(W.size))] *= np.float32(-3.0)
    assert np.array_equal(integer.prepareB(dev(W)).file_bytes(), orc.prepare_b(W))


# ---------------------------------------------------------------- multiply: int32 and fp32

KERNELS = [0, 101, 102, 501, 511, 512, 514, 518, 521, 522, 524, 301, 302, 303, 304, 305, 306, 307, 308]


def run_case(integer, orc, synth, seed, M, K, N, kernel, bias_on=True, relu=False, scale=1.0):
    A, W, bias = inputs(synth, seed, M, K, N)
    Aq_h, Bq_h = orc.prepare_a(A), orc.prepare_b(W)
    want_out, want_acc = orc.affine(Aq_h, Bq_h, bias if bias_on else None, M, K, N, scale, relu)
    Aq, Bq = upload_q(integer, Aq_h, (M, K)), upload_b(integer, Bq_h, (K, N))
    with forced(kernel):
        acc = integer.multiply_i32(Aq, Bq).cpu().numpy()
        out = integer.multiply(Aq, Bq, dev(bias) if bias_on else None, scale=scale, relu=relu).cpu().numpy()
    assert np.array_equal(acc, want_acc), "int32 accumulators differ (kernel %d)" % kernel
    unquant = orc.unquant_mult(orc.tail(Aq_h, M * K), orc.tail(Bq_h, K * N), scale)
    assert_close_fp32(out, want_out, unquant, K)
    assert np.array_equal(out, want_out), "fp32 outputs not bit-identical (kernel %d)" % kernel


@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("M,K,N", [(1, 64, 8), (5, 128, 24), (16, 512, 512), (33, 192, 136),
                                   (64, 512, 2048), (128, 1024, 1024), (100, 2048, 512)])
def test_multiply_all_kernels_small_m(integer, orc, synth, M, K, N, kernel):
    say("multiply", M, K, N, "kernel", kernel)
    run_case(integer, orc, synth, 300 + M + N, M, K, N, kernel, bias_on=True, relu=(M % 2 == 0))


@pytest.mark.parametrize("kernel", [0, 501, 512, 521, 522, 524, 301, 302, 303, 304, 305, 306, 307, 308, 311, 312, 313, 330, 340,
                                    369, 371, 372, 373, 374, 375, 376, 377])
@pytest.mark.parametrize("M,K,N", [(129, 64, 8), (256, 1024, 504), (300, 320, 1000), (513, 128, 264)])
def test_multiply_tile_kernels_ragged(integer, orc, synth, M, K, N, kernel):
    say("multiply ragged", M, K, N, "kernel", kernel)
    run_case(integer, orc, synth, 400 + M + N, M, K, N, kernel, bias_on=(N % 16 == 8), relu=True,
             scale=0.5)


@pytest.mark.parametrize("M,K,N", [(384, 4096, 1024), (512, 2048, 1024), (640, 1024, 1024), (520, 2048, 1000),
                                   (300, 4096, 512), (512, 2048, 512), (384, 2112, 1024)])
def test_multiply_mid_size_dispatch(integer, orc, synth, M, K, N):
    """Between the decode and the encoder sizes: the shapes around the switch from the
    weight-streaming kernels to 128x64 tiles (few tiles, long K), both sides of it."""
    say("multiply mid size", M, K, N)
    run_case(integer, orc, synth, 470 + M + N, M, K, N, 0, bias_on=True, relu=(M % 128 == 0), scale=1.5)


@pytest.mark.parametrize("kernel", [0, 301, 302, 303, 307, 308, 309, 311, 312, 313, 330, 369])
@pytest.mark.parametrize("M,K,N", [(512, 192, 512), (1024, 1088, 1024), (640, 448, 264), (2048, 64, 2048),
                                   (1300, 2112, 776)])
def test_multiply_half_last_k_block(integer, orc, synth, M, K, N, kernel):
    """K a multiple of 64 but not of 128 at encoder sizes: the large-M kernels take a last block of
    64 columns (one, two and many blocks)."""
    say("multiply half last block", M, K, N, "kernel", kernel)
    run_case(integer, orc, synth, 480 + M + N, M, K, N, kernel, bias_on=True, relu=(K % 256 == 64), scale=0.75)


@pytest.mark.parametrize("kernel", [0, 369, 371, 372, 373, 374, 375, 376, 377, 378])
@pytest.mark.parametrize("M,K,N,bias_on,relu", [(128, 128, 128, True, False), (256, 256, 64, False, True), (640, 384, 1024, True, True),
                                                (1000, 512, 1032, True, False), (2048, 1024, 1024, False, False),
                                                (130, 2048, 136, True, True), (4096, 128, 1024, True, False)])
def test_multiply_split_form(integer, orc, synth, M, K, N, bias_on, relu, kernel):
    """The large-M form whose loads are issued by four waves of their own beside the four that
    multiply (three and four LDS stages, 128 x 128 and 128 x 64 tiles, plain and non-temporal
    stores): one K block (nothing to pipeline), fewer blocks than stages, many; tiles that hang over
    the edge of the output; 369 keeps the four-wave form everywhere, 378 takes the split form
    wherever K allows (the automatic choice: where CUs stay idle)."""
    say("multiply split form", M, K, N, "kernel", kernel)
    run_case(integer, orc, synth, 520 + M + N, M, K, N, kernel, bias_on=bias_on, relu=relu, scale=1.25)


@pytest.mark.parametrize("kernel", [330, 331])
@pytest.mark.parametrize("M,K,N,bias_on,relu", [(256, 1024, 256, True, True), (512, 1024, 512, False, False),
                                                (256, 1152, 256, True, False), (256, 1280, 512, False, True),
                                                (512, 2048, 256, True, True), (768, 1024, 1024, True, False)])
def test_multiply_tile_pair_kernel(integer, orc, synth, M, K, N, bias_on, relu, kernel):
    """The large-M kernel that writes one tile out while it multiplies the next: eight K blocks
    per tile (the write-out starts with the second tile) and more (it starts later), several
    workgroups, with and without bias and ReLU, plain and non-temporal stores."""
    say("multiply tile pair", M, K, N, "kernel", kernel)
    run_case(integer, orc, synth, 460 + M + N, M, K, N, kernel, bias_on=bias_on, relu=relu, scale=0.25)


@pytest.mark.parametrize("kernel", [0, 600, 611, 612, 614, 618, 620, 621, 622, 624, 628, 640, 641, 650, 651, 660, 661, 670, 690])
@pytest.mark.parametrize("M,K,N", [(1, 64, 8), (1, 512, 512), (4, 2048, 512), (16, 512, 1536),
                                   (33, 192, 136), (64, 512, 2048), (100, 256, 1000), (128, 256, 64),
                                   (16, 1024, 32000), (7, 4096, 64), (128, 1024, 1024),
                                   (100, 2048, 512), (200, 1024, 504), (128, 4096, 1024),
                                   (128, 1024, 4096), (96, 1024, 2048)])
def test_fused_affine_f32(integer, orc, synth, M, K, N, kernel):
    """prepareA + multiply in one call (one fused kernel where the activations are small):
    output, quantized activations and quantMult equal those of the two separate steps."""
    say("fused", M, K, N, "kernel", kernel)
    A, W, bias = inputs(synth, 500 + M + N, M, K, N)
    Aq_h, Bq_h = orc.prepare_a(A), orc.prepare_b(W)
    relu = (M % 2 == 1)
    want, _ = orc.affine(Aq_h, Bq_h, bias, M, K, N, 0.5, relu)
    Bq = upload_b(integer, Bq_h, (K, N))
    with forced(kernel):
        out, Aq = integer.affine_f32(dev(A), Bq, dev(bias), scale=0.5, relu=relu)
        out = out.cpu().numpy()
        got_aq = Aq.numpy()
    assert np.array_equal(got_aq, Aq_h), "quantized activations / quantMult of the fused call"
    assert np.array_equal(out, want)


def test_fused_shortlist(integer, orc, synth):
    import torch
    say("fused shortlist")
    M, K, N = 8, 512, 4096
    A, W, bias = inputs(synth, 606, M, K, N)
    Aq_h, Bq_h = orc.prepare_a(A), orc.prepare_b(W)
    idx = synth.shortlist(606, N, 100, 300)
    want, _ = orc.affine_shortlist(Aq_h, Bq_h, bias, idx, M, K, N)
    Bq = upload_b(integer, Bq_h, (K, N))
    didx = torch.from_numpy(idx.view(np.int32)).cuda()
    out, Aq = integer.affine_f32(dev(A), Bq, dev(bias), shortlist=didx)
    assert np.array_equal(Aq.numpy(), Aq_h) and np.array_equal(out.cpu().numpy(), want)


@pytest.mark.parametrize("kernel", [0, 101, 102, 301, 307, 312, 372, 376, 501, 511, 512, 514, 518, 521, 522, 524, 600, 611, 612, 614, 618, 620, 621, 624, 628, 641, 651, 661, 670, 690])
@pytest.mark.parametrize("M", [8, 100])
def test_shortlist_every_kernel_family(integer, orc, synth, M, kernel):
    """The row gather of W^T and of the bias inside each kernel family (ids >= 600: fused call)."""
    import torch
    say("shortlist", M, "kernel", kernel)
    K, N = 256, 2048
    A, W, bias = inputs(synth, 707 + M, M, K, N)
    Aq_h, Bq_h = orc.prepare_a(A), orc.prepare_b(W)
    idx = synth.shortlist(707 + M, N, 100, 300)
    want, want_acc = orc.affine_shortlist(Aq_h, Bq_h, bias, idx, M, K, N)
    Bq = upload_b(integer, Bq_h, (K, N))
    didx = torch.from_numpy(idx.view(np.int32)).cuda()
    with forced(kernel):
        if kernel >= 600:
            out, Aq = integer.affine_f32(dev(A), Bq, dev(bias), shortlist=didx)
            assert np.array_equal(Aq.numpy(), Aq_h)
        else:
            Aq = upload_q(integer, Aq_h, (M, K))
            acc = integer.multiply_i32(Aq, Bq, shortlist=didx).cpu().numpy()
            assert np.array_equal(acc, want_acc)
            out = integer.multiply(Aq, Bq, dev(bias), shortlist=didx)
        out = out.cpu().numpy()
    assert np.array_equal(out, want)


def test_config1_single_affine_end_to_end(integer, orc, synth):
    """Benchmark configuration 1: A[64x512] ~ N(0,1), W[512x2048] ~ N(0,0.02^2), bias ~ N(0,0.01^2), ReLU."""
    say("config1")
    M, K, N = 64, 512, 2048
    A, W, bias = inputs(synth, 1001, M, K, N)
    Bq_h = orc.prepare_b(W)
    Aq_h = orc.prepare_a(A)
    want, want_acc = orc.affine(Aq_h, Bq_h, bias, M, K, N, 1.0, True)
    Bq = integer.prepareB(dev(W))                       # offline quantizer on the GPU
    assert np.array_equal(Bq.file_bytes(), Bq_h)
    Aq = integer.prepareA(dev(A))
    assert np.array_equal(Aq.numpy(), Aq_h)
    assert np.array_equal(integer.multiply_i32(Aq, Bq).cpu().numpy(), want_acc)
    got = integer.affineWithReluDropout(dev(A), Bq, dev(bias)).cpu().numpy()
    unquant = orc.unquant_mult(orc.tail(Aq_h, M * K), orc.tail(Bq_h, K * N), 1.0)
    assert_close_fp32(got, want, unquant, K)
    assert np.array_equal(got, want)
    assert (got == 0).mean() > 0.2 and (got > 0).mean() > 0.2   # ReLU really clipped something


@pytest.mark.parametrize("K,N", [(512, 1536), (512, 512), (512, 2048), (2048, 512), (512, 32000)])
@pytest.mark.parametrize("M", [1, 4, 16, 64])
def test_config2_decode_sweep(integer, orc, synth, M, K, N):
    """Benchmark configuration 2: transformer-base decode shapes."""
    say("config2", M, K, N)
    A, W, bias = inputs(synth, 1002, M, K, N)
    Bq_h, Aq_h = orc.prepare_b(W), orc.prepare_a(A)
    want, want_acc = orc.affine(Aq_h, Bq_h, bias, M, K, N)
    Bq = upload_b(integer, Bq_h, (K, N))
    Aq = integer.prepareA(dev(A))
    assert np.array_equal(Aq.numpy(), Aq_h)
    assert np.array_equal(integer.multiply_i32(Aq, Bq).cpu().numpy(), want_acc)
    got = integer.affine(dev(A), Bq, dev(bias)).cpu().numpy()
    assert np.array_equal(got, want)


def test_config3_transformer_big_step_shapes(integer, orc, synth):
    """Benchmark configuration 3, GEMM shapes at M = 128 (beam 4 x batch 32), d = 1024, ffn = 4096."""
    M = 128
    for K, N, relu in [(1024, 1024, False), (1024, 4096, True), (4096, 1024, False)]:
        say("config3", M, K, N)
        A, W, bias = inputs(synth, 1003, M, K, N)
        Bq_h, Aq_h = orc.prepare_b(W), orc.prepare_a(A)
        want, want_acc = orc.affine(Aq_h, Bq_h, bias, M, K, N, 1.0, relu)
        Bq = upload_b(integer, Bq_h, (K, N))
        Aq = integer.prepareA(dev(A))
        assert np.array_equal(Aq.numpy(), Aq_h)
        assert np.array_equal(integer.multiply_i32(Aq, Bq).cpu().numpy(), want_acc)
        got = integer.multiply(Aq, Bq, dev(bias), relu=relu).cpu().numpy()
        assert np.array_equal(got, want)
        # and as the decoder calls it: one call from the fp32 activations
        got = integer.affine(dev(A), Bq, dev(bias)).cpu().numpy() if not relu else \
            integer.affineWithReluDropout(dev(A), Bq, dev(bias)).cpu().numpy()
        assert np.array_equal(got, want)


def test_config3_vocabulary_projection_from_fp32(integer, orc, synth):
    """The 32000-word output layer of configuration 3 at M = 128, through the operator (abs-max,
    quantize and GEMM behind one call)."""
    M, K, N = 128, 1024, 32000
    say("config3 vocabulary", M, K, N)
    A, W, bias = inputs(synth, 1013, M, K, N)
    Bq_h, Aq_h = orc.prepare_b(W), orc.prepare_a(A)
    want, _ = orc.affine(Aq_h, Bq_h, bias, M, K, N, 1.0, False)
    Bq = upload_b(integer, Bq_h, (K, N))
    got = integer.affine(dev(A), Bq, dev(bias)).cpu().numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("K,N", [(1024, 4096), (4096, 1024)])
def test_config4_large_m_full_size(integer, orc, synth, K, N):
    """Benchmark configuration 4 at full size (M = 4096).  The checker runs on 96 sampled rows (rows are
    independent once A is quantized); the rest is covered by a column-sum identity in int64:
    sum_m acc[m, n] == (sum_m Aq[m, :]) . Bt[n, :]."""
    M = 4096
    say("config4", M, K, N)
    A, W, bias = inputs(synth, 1004, M, K, N)
    Bq_h, Aq_h = orc.prepare_b(W), orc.prepare_a(A)
    Bq = upload_b(integer, Bq_h, (K, N))
    Aq = integer.prepareA(dev(A))
    assert np.array_equal(Aq.numpy(), Aq_h)
    acc = integer.multiply_i32(Aq, Bq).cpu().numpy()
    got = integer.affineWithReluDropout(dev(A), Bq, dev(bias)).cpu().numpy()
    rows = np.unique(np.concatenate([[0, 1, 15, 16, 127, 128, 255, 256, M - 1],
                                     np.random.default_rng(4).integers(0, M, 87)]))
    sub = np.concatenate([Aq_h[:M * K].reshape(M, K)[rows].ravel(), Aq_h[M * K:]])
    want, want_acc = orc.affine(sub, Bq_h, bias, len(rows), K, N, 1.0, True)
    assert np.array_equal(acc[rows], want_acc)
    assert np.array_equal(got[rows], want)
    colsum = Aq_h[:M * K].reshape(M, K).astype(np.int64).sum(0)
    Bt = Bq_h[:K * N].reshape(N, K).astype(np.int64)
    assert np.array_equal(acc.astype(np.int64).sum(0), Bt @ colsum)
    # the fp32 output is the deterministic image of acc: recompute it everywhere in numpy
    u = orc.unquant_mult(orc.tail(Aq_h, M * K), orc.tail(Bq_h, K * N), 1.0)
    y = ((acc.astype(f32) * u).astype(f32) + bias[None, :]).astype(f32)
    assert np.array_equal(got, np.where(y > 0, y, f32(0)))


# ---------------------------------------------------------------- shortlist

@pytest.mark.parametrize("M", [4, 64, 256])
def test_config5_shortlist(integer, orc, synth, M):
    """Benchmark configuration 5: W int8 [32000 x 1024], shortlist of 500-2000 sorted unique ids.
    gather-GEMM == column pick of the dense GEMM, bit-exactly, and matches the checker."""
    import torch
    K, N = 1024, 32000
    say("config5", M)
    A = synth.normal(1005, synth.STREAM_A, (M, K), 1.0)
    Wt = synth.normal(1005, synth.STREAM_W, (N, K), 0.02)   # tied embedding matrix [V x D]
    bias = synth.normal(1005, synth.STREAM_BIAS, (N,), 0.01)
    # its int8 form is the payload of logical B = Wt^T: identical bytes, quantMult over all of it
    bqm = orc.quant_mult(orc.max_abs(Wt))
    Bq_h = np.concatenate([orc.quantize(Wt, bqm).ravel(), np.array([bqm], f32).view(np.int8)])
    Aq_h = orc.prepare_a(A)
    Bq = upload_b(integer, Bq_h, (K, N))
    Aq = integer.prepareA(dev(A))
    dense = integer.multiply(Aq, Bq, dev(bias)).cpu().numpy()
    dense_acc = integer.multiply_i32(Aq, Bq).cpu().numpy()
    for j, seed in enumerate([1005, 2005, 3005]):
        idx = synth.shortlist(seed, N)
        if j == 2:
            idx = idx[:8]                                   # smallest legal shortlist
        say("  n_idx", idx.size)
        want, want_acc = orc.affine_shortlist(Aq_h, Bq_h, bias, idx, M, K, N)
        didx = torch.from_numpy(idx.view(np.int32)).cuda()
        acc = integer.multiply_i32(Aq, Bq, shortlist=didx).cpu().numpy()
        out = integer.multiply(Aq, Bq, dev(bias), shortlist=didx).cpu().numpy()
        assert np.array_equal(acc, want_acc) and np.array_equal(acc, dense_acc[:, idx])
        assert np.array_equal(out, want) and np.array_equal(out, dense[:, idx])
    # dense full-vocabulary case against the checker on a few rows
    rows = [0, M // 2, M - 1]
    sub = np.concatenate([Aq_h[:M * K].reshape(M, K)[rows].ravel(), Aq_h[M * K:]])
    want, want_acc = orc.affine(sub, Bq_h, bias, len(rows), K, N)
    assert np.array_equal(dense_acc[rows], want_acc) and np.array_equal(dense[rows], want)


def _ragged_cases():
    """M and N a whole number of main tiles plus or minus 1 / 8 / about 100, for every large-M
    family that has a ragged form (forced: the automatic choice takes it only where it saves a
    round of workgroups on the whole chip)."""
    cases = []
    for kernel, T in ((361, 256), (362, 256), (366, 256), (363, 128), (367, 128), (364, 128), (368, 128)):
        K = 1024 if kernel in (361, 362, 366) else 256
        for dm, dn in ((1, 8), (-1, -8), (100, 104), (8, 0), (0, 8), (-100, 96), (1, -104)):
            cases.append((kernel, 2 * T + dm, K, 2 * T + dn))
    return cases


@pytest.mark.parametrize("kernel,M,K,N", _ragged_cases())
def test_multiply_ragged_main_and_edge_tiles(integer, orc, synth, kernel, M, K, N):
    """Whole main tiles for the first workgroups, 64 x 128 tiles below and 128 x 64 tiles to the
    right of them: accumulators and outputs as the checker's, with and without bias and ReLU."""
    say("multiply main + edge tiles", M, K, N, "kernel", kernel)
    run_case(integer, orc, synth, 490 + M + N, M, K, N, kernel, bias_on=(M % 2 == 1), relu=(N % 16 == 8), scale=0.5)


@pytest.mark.parametrize("M,K,N", [(4100, 1024, 4096), (4100, 1024, 4104), (2050, 1024, 2056), (4100, 4096, 1024),
                                   (4352, 1024, 4096), (4097, 512, 4096)])
def test_multiply_ragged_at_full_size(integer, orc, synth, M, K, N):
    """The shapes where a few rows or columns past a whole number of main tiles used to cost a
    second round of workgroups: the automatic choice, against sampled rows of the checker and an
    int64 column-sum identity over everything."""
    import torch
    say("ragged at full size", M, K, N)
    A, W, bias = inputs(synth, 495 + M + N, M, K, N)
    Aq_h, Bq_h = orc.prepare_a(A), orc.prepare_b(W)
    Aq, Bq = upload_q(integer, Aq_h, (M, K)), upload_b(integer, Bq_h, (K, N))
    acc = integer.multiply_i32(Aq, Bq).cpu().numpy()
    out = integer.multiply(Aq, Bq, dev(bias), relu=True).cpu().numpy()
    # every column sum of the accumulators = (column sums of Aq) . Bq, in int64
    a8 = Aq_h[:M * K].view(np.int8).reshape(M, K).astype(np.int64)
    b8 = Bq_h[:K * N].view(np.int8).reshape(N, K).astype(np.int64)
    assert np.array_equal(acc.astype(np.int64).sum(axis=0), b8 @ a8.sum(axis=0))
    assert np.array_equal(acc.astype(np.int64).sum(axis=1), a8 @ b8.sum(axis=0))
    # sampled rows (the last rows and columns are where the small tiles sit) against the checker
    rows = sorted(set([0, 1, 255, 256, M // 2, M - 130, M - 65, M - 5, M - 4, M - 3, M - 2, M - 1]))
    sub = np.ascontiguousarray(np.concatenate([Aq_h[:M * K].reshape(M, K)[rows].reshape(-1), Aq_h[M * K:]]))
    want, want_acc = orc.affine(sub, Bq_h, bias, len(rows), K, N, 1.0, True)
    assert np.array_equal(acc[rows], want_acc)
    assert np.array_equal(out[rows], np.asarray(want, dtype=f32).reshape(len(rows), N))
    # the whole fp32 image follows from the accumulators
    unquant = orc.unquant_mult(orc.tail(Aq_h, M * K), orc.tail(Bq_h, K * N), 1.0)
    img = np.maximum((acc.astype(f32) * f32(unquant)) + bias[None, :].astype(f32), f32(0))
    assert np.array_equal(out, img)


# ---------------------------------------------------------------- abs-max handed between calls

@pytest.mark.parametrize("M,K,N,N2", [(128, 1024, 1024, 1024), (128, 1024, 4096, 1024), (128, 4096, 1024, 512),
                                      (16, 512, 512, 64), (64, 2048, 512, 2048), (200, 1024, 504, 1000),
                                      (300, 1024, 32000, 64), (600, 512, 2048, 512), (33, 192, 136, 24)])
def test_absmax_chaining_equals_recomputation(integer, orc, synth, M, K, N, N2):
    """A first affine call leaves the abs-max of its output; a second one, reading that output,
    takes it instead of scanning the tensor: outputs and quantized activations are bit-identical to
    the unchained calls, and the slots' maximum is max|out| exactly - whichever kernel ran."""
    say("chain", M, K, N, N2)
    A, W, bias = inputs(synth, 8000 + M + N, M, K, N)
    W2 = synth.normal(8001 + M, synth.STREAM_W, (N, N2), 0.02) if N % 64 == 0 else None
    Bq = upload_b(integer, orc.prepare_b(W), (K, N))
    relu = (N % 16 == 0)
    out, Aq, omax = integer.affine_f32(dev(A), Bq, dev(bias), relu=relu, want_absmax=True)
    ref, Aq_ref = integer.affine_f32(dev(A), Bq, dev(bias), relu=relu)
    assert np.array_equal(out.cpu().numpy(), ref.cpu().numpy()) and np.array_equal(Aq.numpy(), Aq_ref.numpy())
    slots = omax.data.cpu().numpy()
    assert slots.shape == (2048,) and float(slots.max()) == float(np.abs(ref.cpu().numpy()).max())
    if W2 is None:
        return
    Bq2 = upload_b(integer, orc.prepare_b(W2), (N, N2))
    got, Aq2 = integer.affine_f32(out, Bq2, None, absmax=omax)
    want, Aq2_ref = integer.affine_f32(ref, Bq2, None)
    assert np.array_equal(Aq2.numpy(), Aq2_ref.numpy()) and np.array_equal(got.cpu().numpy(), want.cpu().numpy())


@pytest.mark.parametrize("M", [4096, 4100, 2304])
def test_encoder_layer_chain_hands_absmax_through_large_m_kernels(integer, orc, synth, M):
    """Layer norm -> W1 + ReLU -> W2 at encoder size (d = 1024, ffn = 4096): every kernel leaves
    the abs-max of what it wrote (the layer norm with more rows than slots, the large-M GEMM
    epilogues one slot per workgroup), so the chained calls never scan a tensor for it.  The
    slots' maximum is max|tensor| exactly, quantized activations and outputs equal the unchained
    calls' and the checker's, bit for bit."""
    import torch
    ops = load("ops")
    d, ffn = 1024, 4096
    say("encoder chain", M)
    X = synth.normal(9100 + M, synth.STREAM_A, (M, d), 1.0)
    gamma = (1.0 + 0.1 * synth.normal(9101, synth.STREAM_BIAS, (d,), 1.0)).astype(f32)
    beta = synth.normal(9102, synth.STREAM_BIAS, (d,), 0.1)
    W1 = synth.normal(9103, synth.STREAM_W, (d, ffn), 0.02)
    W2 = synth.normal(9104, synth.STREAM_W, (ffn, d), 0.02)
    b1 = synth.normal(9105, synth.STREAM_BIAS, (ffn,), 0.01)
    b2 = synth.normal(9106, synth.STREAM_BIAS, (d,), 0.01)
    B1h, B2h = orc.prepare_b(W1), orc.prepare_b(W2)
    B1, B2 = upload_b(integer, B1h, (d, ffn)), upload_b(integer, B2h, (ffn, d))
    x, xmax = ops.layerNorm(dev(X), dev(gamma), dev(beta), eps=1e-6, want_absmax=True)
    x_plain = ops.layerNorm(dev(X), dev(gamma), dev(beta), eps=1e-6)
    xh = x.cpu().numpy()
    assert np.array_equal(xh, x_plain.cpu().numpy())
    assert float(xmax.data.max()) == float(np.abs(xh).max())
    h, Aq1, hmax = integer.affine_f32(x, B1, dev(b1), relu=True, absmax=xmax, want_absmax=True)
    h_ref, Aq1_ref = integer.affine_f32(x, B1, dev(b1), relu=True)
    hh = h.cpu().numpy()
    assert np.array_equal(Aq1.numpy(), Aq1_ref.numpy()) and np.array_equal(hh, h_ref.cpu().numpy())
    assert float(hmax.data.max()) == float(np.abs(hh).max())
    Aq1_h = orc.prepare_a(xh)
    assert np.array_equal(Aq1.numpy(), Aq1_h)
    rows = sorted(set([0, 1, 255, 256, 2047, 2048, M // 2, M - 129, M - 5, M - 4, M - 1]))
    sub = np.ascontiguousarray(np.concatenate([Aq1_h[:M * d].reshape(M, d)[rows].reshape(-1), Aq1_h[M * d:]]))
    want1, _ = orc.affine(sub, B1h, b1, len(rows), d, ffn, 1.0, True)
    assert np.array_equal(hh[rows], np.asarray(want1, dtype=f32).reshape(len(rows), ffn))
    y, Aq2, ymax = integer.affine_f32(h, B2, dev(b2), absmax=hmax, want_absmax=True)
    y_ref, Aq2_ref = integer.affine_f32(h, B2, dev(b2))
    yh = y.cpu().numpy()
    assert np.array_equal(Aq2.numpy(), Aq2_ref.numpy()) and np.array_equal(yh, y_ref.cpu().numpy())
    assert float(ymax.data.max()) == float(np.abs(yh).max())
    Aq2_h = orc.prepare_a(hh)
    assert np.array_equal(Aq2.numpy(), Aq2_h)
    sub2 = np.ascontiguousarray(np.concatenate([Aq2_h[:M * ffn].reshape(M, ffn)[rows].reshape(-1), Aq2_h[M * ffn:]]))
    want2, _ = orc.affine(sub2, B2h, b2, len(rows), ffn, d, 1.0, False)
    assert np.array_equal(yh[rows], np.asarray(want2, dtype=f32).reshape(len(rows), d))


# ---------------------------------------------------------------- random shapes

def _random_cases(n):
    """Seeded shapes over everything the dispatch distinguishes: M 1..600, K a multiple of 64 up
    to 2048, N a multiple of 8 up to 5000, with and without bias / ReLU / scale / shortlist."""
    rng = np.random.default_rng(20261125)
    cases = []
    for i in range(n):
        M = int(rng.choice([1, 2, 7, 16, 17, 31, 33, 64, 65, 100, 128, 129, 200, 257, 384, 600]))
        K = 64 * int(rng.integers(1, 33))
        N = 8 * int(rng.integers(1, 626))
        cases.append((i, M, K, N, bool(rng.integers(2)), bool(rng.integers(2)),
                      float(rng.choice([1.0, 0.5, 0.125, 3.0])), bool(rng.integers(3) == 0)))
    return cases


@pytest.mark.parametrize("i,M,K,N,bias_on,relu,scale,short", _random_cases(48))
def test_random_shapes_both_entry_points(integer, orc, synth, i, M, K, N, bias_on, relu, scale, short):
    """Automatic kernel choice on seeded random shapes: the two-call form (prepareA, multiply) and
    the single fused call give the checker's bits."""
    import torch
    say("random", i, M, K, N, bias_on, relu, scale, short)
    A, W, bias = inputs(synth, 5000 + i, M, K, N)
    Aq_h, Bq_h = orc.prepare_a(A), orc.prepare_b(W)
    b = bias if bias_on else None
    idx = didx = None
    if short and N >= 64:
        idx = synth.shortlist(5000 + i, N, 8, max(8, N // 2))
        didx = torch.from_numpy(idx.view(np.int32)).cuda()
        want, want_acc = orc.affine_shortlist(Aq_h, Bq_h, b, idx, M, K, N, scale, relu)
    else:
        want, want_acc = orc.affine(Aq_h, Bq_h, b, M, K, N, scale, relu)
    Bq = upload_b(integer, Bq_h, (K, N))
    db = dev(bias) if bias_on else None
    Aq = integer.prepareA(dev(A))
    assert np.array_equal(Aq.numpy(), Aq_h)
    assert np.array_equal(integer.multiply_i32(Aq, Bq, shortlist=didx).cpu().numpy(), want_acc)
    out2 = integer.multiply(Aq, Bq, db, scale=scale, relu=relu, shortlist=didx).cpu().numpy()
    out1, Aq1 = integer.affine_f32(dev(A), Bq, db, scale=scale, relu=relu, shortlist=didx)
    assert np.array_equal(Aq1.numpy(), Aq_h)
    assert np.array_equal(out2, want) and np.array_equal(out1.cpu().numpy(), want)


def _random_large_cases(n):
    """Seeded shapes above the decode sizes: M 601..4500, K a multiple of 64 up to 4096, N a
    multiple of 8 up to 4096 - whole and ragged tiles of every large-M kernel under the automatic
    choice.  Sizes are bounded so that the checker needs at most a few seconds per case."""
    rng = np.random.default_rng(20261126)
    cases = []
    while len(cases) < n:
        M = int(rng.choice([640, 768, 1000, 1024, 1280, 1536, 2048, 2050, 2560, 3000, 4096, 4500]))
        K = 64 * int(rng.integers(1, 65))
        N = 8 * int(rng.integers(1, 513))
        if len(cases) % 3 == 0:   # whole tiles: the shapes the 256-wide kernels take
            K = 128 * int(rng.integers(4, 33))
            N = 256 * int(rng.integers(1, 17))
            M = 256 * int(rng.integers(3, 17))
        if M * K * N > 2.5e10:
            continue
        cases.append((len(cases), M, K, N, bool(rng.integers(2)), bool(rng.integers(2)),
                      float(rng.choice([1.0, 0.5, 3.0])), bool(rng.integers(4) == 0)))
    return cases


@pytest.mark.parametrize("i,M,K,N,bias_on,relu,scale,short", _random_large_cases(24))
def test_random_large_shapes_both_entry_points(integer, orc, synth, i, M, K, N, bias_on, relu, scale, short):
    """Automatic kernel choice on seeded random shapes of encoder size, both call forms."""
    import torch
    say("random large", i, M, K, N, bias_on, relu, scale, short)
    A, W, bias = inputs(synth, 7000 + i, M, K, N)
    Aq_h, Bq_h = orc.prepare_a(A), orc.prepare_b(W)
    b = bias if bias_on else None
    didx = None
    if short and N >= 64:
        idx = synth.shortlist(7000 + i, N, 8, max(8, N // 2))
        didx = torch.from_numpy(idx.view(np.int32)).cuda()
        want, want_acc = orc.affine_shortlist(Aq_h, Bq_h, b, idx, M, K, N, scale, relu)
    else:
        want, want_acc = orc.affine(Aq_h, Bq_h, b, M, K, N, scale, relu)
    Bq = upload_b(integer, Bq_h, (K, N))
    db = dev(bias) if bias_on else None
    Aq = integer.prepareA(dev(A))
    assert np.array_equal(Aq.numpy(), Aq_h)
    assert np.array_equal(integer.multiply_i32(Aq, Bq, shortlist=didx).cpu().numpy(), want_acc)
    out2 = integer.multiply(Aq, Bq, db, scale=scale, relu=relu, shortlist=didx).cpu().numpy()
    out1, Aq1 = integer.affine_f32(dev(A), Bq, db, scale=scale, relu=relu, shortlist=didx)
    assert np.array_equal(Aq1.numpy(), Aq_h)
    assert np.array_equal(out2, want) and np.array_equal(out1.cpu().numpy(), want)


# ---------------------------------------------------------------- fixtures, contract, errors

def test_golden_fixtures_on_gpu(integer):
    g = np.load(GOLDEN)
    for i in range(int(g["n_cases"])):
        A, W = g["c%d_A" % i], g["c%d_W" % i]
        M, K = A.shape
        N = W.shape[1]
        say("golden", i, M, K, N)
        Bq = integer.prepareB(dev(W))
        Aq = integer.prepareA(dev(A))
        assert np.array_equal(Aq.numpy()[:M * K].reshape(M, K), g["c%d_Aq" % i])
        assert np.array_equal(Bq.file_bytes()[:K * N].reshape(N, K), g["c%d_Bt" % i])
        assert integer.getQuantMult(Aq) == g["c%d_aqm" % i] and integer.getQuantMult(Bq) == g["c%d_bqm" % i]
        assert np.array_equal(integer.multiply_i32(Aq, Bq).cpu().numpy(), g["c%d_acc" % i])
        bias = dev(g["c%d_bias" % i]) if int(g["c%d_with_bias" % i]) else None
        out = integer.affineOrDot(dev(A), Bq, bias, scale=float(g["c%d_scale" % i]),
                                  relu=bool(g["c%d_relu" % i])).cpu().numpy()
        assert np.array_equal(out, g["c%d_out" % i])


def test_marian_operator_vectors_on_gpu(integer):
    """reference src/tests/units/operator_tests.cpp:508-534 (dot) and :618-659 (affine,
    affineWithReluDropout, affine == dot + bias), embedded so that both quantMults are 1 and K is
    padded with zeros to 64."""
    say("marian operator vectors")
    vA = np.arange(1, 13, dtype=f32).reshape(4, 3)

    def embed(A, B, n_pad=8):
        A2 = np.zeros((A.shape[0] + 1, 64), f32)
        A2[:-1, :A.shape[1]] = A
        A2[-1, 0] = 127
        B2 = np.zeros((64, n_pad), f32)
        B2[:B.shape[0], :B.shape[1]] = B
        B2[0, n_pad - 1] = 127
        return dev(A2), integer.prepareB(dev(B2))

    a, b = embed(vA, np.array([[1, 2], [3, 4], [5, 6]], f32))
    C = integer.dot(a.reshape(5, 1, 64), b)
    assert tuple(C.shape) == (5, 1, 8)                      # shape = A's with last dim <- N
    assert C.cpu().numpy().reshape(5, 8)[:4, :2].ravel().tolist() == [22, 28, 49, 64, 76, 100, 103, 136]

    a, b = embed(vA, np.array([[1, -2], [3, 4], [-5, 6]], f32))
    bias = dev(np.full(8, 2.0, f32))
    aff = integer.affine(a, b, bias).cpu().numpy()
    assert aff[:4, :2].ravel().tolist() == [-6, 26, -9, 50, -12, 74, -15, 98]
    assert np.array_equal(aff, integer.dot(a, b).cpu().numpy() + 2.0)
    rel = integer.affineWithReluDropout(a, b, bias).cpu().numpy()
    assert rel[:4, :2].ravel().tolist() == [0, 26, 0, 50, 0, 74, 0, 98]
    assert np.array_equal(rel, np.maximum(aff, 0))


def test_scale_and_transA(integer, orc, synth):
    say("scale/transA")
    M, K, N = 24, 128, 64
    A, W, bias = inputs(synth, 77, M, K, N)
    Bq_h = orc.prepare_b(W)
    Bq = upload_b(integer, Bq_h, (K, N))
    At = dev(A.T.copy())                                    # [K, M]; transA gives back A
    got = integer.affine(At, Bq, dev(bias), transA=True, scale=0.25).cpu().numpy()
    want, _ = orc.affine(orc.prepare_a(A), Bq_h, bias, M, K, N, 0.25)
    assert np.array_equal(got, want)


def test_repeatable_and_input_untouched(integer, synth):
    say("repeatable")
    A, W, bias = inputs(synth, 78, 64, 512, 2048)
    a, b = dev(A), integer.prepareB(dev(W))
    r1 = integer.affine(a, b, dev(bias)).cpu().numpy()
    r2 = integer.affine(a, b, dev(bias)).cpu().numpy()
    assert np.array_equal(r1, r2) and np.array_equal(a.cpu().numpy(), A)


def test_float_weights_are_quantized_once_when_the_gemm_type_is_intgemm8(integer, orc, synth):
    """On-line quantization of a float32 model: with the backend's gemm type set, dot/affine take
    float32 weights, quantize them on first use (same bytes as the offline packer) and reuse the
    result; without it they refuse, as before."""
    import torch
    M, K, N = 9, 128, 72
    A, W, bias = inputs(synth, 911, M, K, N)
    be = integer.Backend.get("cuda:0")
    dW = dev(W)
    with pytest.raises(integer.MarianRuntimeError):
        integer.affine(dev(A), dW, dev(bias))
    be.setGemmType(integer.Type.intgemm8)
    try:
        out = integer.affine(dev(A), dW, dev(bias)).cpu().numpy()
        q1 = be.memoizedPrepareB(dW)
        assert np.array_equal(q1.file_bytes(), orc.prepare_b(W))
        assert be.memoizedPrepareB(dW) is q1                      # remembered
        want, _ = orc.affine(orc.prepare_a(A), orc.prepare_b(W), bias, M, K, N)
        assert np.array_equal(out, want)
        assert np.array_equal(integer.dot(dev(A), dW).cpu().numpy(),
                              orc.affine(orc.prepare_a(A), orc.prepare_b(W), None, M, K, N)[0])
        dW.mul_(2.0)                                               # a changed parameter is re-quantized
        assert be.memoizedPrepareB(dW) is not q1
    finally:
        be.setGemmType(None)


def test_type_errors_like_the_reference(integer):
    import torch
    from conftest import load
    T = load("types")
    say("type errors")
    b = integer.prepareB(torch.ones(64, 8, device="cuda"))
    with pytest.raises(integer.MarianRuntimeError, match="Intgemm expects type of A to be float32"):
        integer.affineOrDot(torch.ones(2, 64, device="cuda", dtype=torch.float16), b)
    with pytest.raises(integer.MarianRuntimeError, match="Intgemm expects type of B"):
        integer.affineOrDot(torch.ones(2, 64, device="cuda"), torch.ones(64, 8, device="cuda"))
    tiled = integer.QTensor(b.data, b.shape, T.Type.intgemm8avx512)  # CPU-tiled payload
    with pytest.raises(integer.MarianRuntimeError, match="Unsupported type"):
        integer.affineOrDot(torch.ones(2, 64, device="cuda"), tiled)
    with pytest.raises(integer.MarianRuntimeError, match="bad shape"):
        integer.prepareA(torch.ones(2, 100, device="cuda"))
    empty = integer.affine(torch.ones(0, 64, device="cuda"), b, None)
    assert tuple(empty.shape) == (0, 8)


def test_model_file_weights_run(integer, orc, synth, tmp_path):
    """A Type::intgemm8 item read from a .bin file is uploaded byte for byte, re-tiled on the device
    (prepareAndTransposeB, as the reference's loader does for its CPU) and multiplied."""
    from conftest import load
    B = load("binary")
    say("bin file -> gpu")
    M, K, N = 12, 128, 40
    A, W, bias = inputs(synth, 808, M, K, N)
    path = os.path.join(tmp_path, "m.bin")
    B.save_items(path, [B.intgemm8_item("decoder_l1_ffn_W1", orc.prepare_b(W), (K, N)),
                        B.float_item("decoder_l1_ffn_b1", bias.reshape(1, N))])
    w, b = B.load_items(path)
    Bq = integer.prepareAndTransposeB(integer.QTensor.from_numpy(w.bytes, w.shape, w.type, "cuda"))
    got = integer.affineWithReluDropout(dev(A), Bq, dev(b.bytes.view(f32)[:N].copy())).cpu().numpy()
    want, _ = orc.affine(orc.prepare_a(A), orc.prepare_b(W), bias, M, K, N, 1.0, True)
    assert np.array_equal(got, want)


GROUPED_CASES = [
    # M, K, [N of every matrix], bias on?, ReLU, abs-max handed over
    (128, 1024, [1024, 1024, 1024], True, False, True),     # self-attention projections of transformer-big
    (128, 1024, [1024, 1024, 1024], True, False, False),
    (128, 512, [512, 512, 512], True, False, False),        # transformer-base
    (1, 512, [512, 512, 512], False, False, False),
    (4, 512, [512], True, True, False),
    (33, 192, [136, 8, 72, 1000], True, True, False),       # ragged widths, four matrices
    (64, 1024, [2048, 1024], True, False, True),
    (200, 1024, [504, 520], True, True, False),
    (128, 4096, [1024, 1024], True, False, False),          # long rows: 16-row workgroups, K split eight ways
    (256, 2048, [4096, 4096], True, False, False),          # too wide for one launch: one quantization, two multiplies
    (300, 1024, [512, 512, 512], True, True, True),         # too many rows for the quantize-on-stage kernel
    (16, 64, [8, 8], False, False, False),
]


@pytest.mark.parametrize("M,K,Ns,bias_on,relu,handed", GROUPED_CASES)
def test_grouped_affine_equals_separate_calls_and_checker(integer, orc, synth, M, K, Ns, bias_on, relu, handed):
    """One activation tensor through several weight matrices in one call: every output equals the
    single-matrix call's and the CPU checker's bit for bit, and the quantized activations (written
    once) are the checker's."""
    from conftest import load
    ops = load("ops")
    say("grouped", M, K, Ns, bias_on, relu, handed)
    A = synth.normal(900 + M + K, synth.STREAM_A, (M, K), 1.0)
    Ws = [synth.normal(900 + g, synth.STREAM_W, (K, N), 0.02 * (g + 1)) for g, N in enumerate(Ns)]
    biases = [synth.normal(900 + g, synth.STREAM_BIAS, (N,), 0.01) if bias_on and g != 1 else None
              for g, N in enumerate(Ns)]          # (the second matrix never has a bias)
    Aq_h = orc.prepare_a(A)
    Bq_h = [orc.prepare_b(W) for W in Ws]
    Bq = [upload_b(integer, b, (K, N)) for b, N in zip(Bq_h, Ns)]
    dA = dev(A)
    absmax = None
    if handed:   # the abs-max as a producing kernel leaves it: a layer norm that reproduces A
        import torch
        ln, absmax = ops.layerNorm(dA, torch.ones(K, device="cuda"), None, 1e-9, want_absmax=True)
        dA = ln
        A = ln.cpu().numpy()
        Aq_h = orc.prepare_a(A)
    dbias = [None if b is None else dev(b) for b in biases]
    outs, Aq = integer.affine_f32_grouped(dA, list(zip(Bq, dbias)), scale=0.5, relu=relu, absmax=absmax)
    assert np.array_equal(Aq.numpy(), Aq_h), "quantized activations / quantMult"
    for g, N in enumerate(Ns):
        want, _ = orc.affine(Aq_h, Bq_h[g], biases[g], M, K, N, 0.5, relu)
        single, _ = integer.affine_f32(dA, Bq[g], dbias[g], scale=0.5, relu=relu)
        got = outs[g].cpu().numpy()
        assert np.array_equal(got.view(np.uint32), single.cpu().numpy().view(np.uint32)), "matrix %d vs single call" % g
        assert np.array_equal(got, want), "matrix %d vs checker" % g


def test_grouped_affine_argument_checks(integer):
    import ctypes
    from conftest import load
    L = load("_lib")
    lib = L.lib()
    buf = 0x1000
    one = (ctypes.c_void_p * 1)(buf)
    n8 = (ctypes.c_int64 * 1)(8)
    call = lambda n, Bq, bias, out, N, M, K: lib.marian_hip_int8_affine_f32_grouped(
        buf, buf, n, Bq, bias, out, N, M, K, 1.0, 0, None, buf, 4096, None)
    assert call(0, one, None, one, n8, 1, 64) == L.ERR_SHAPE
    assert call(5, one, None, one, n8, 1, 64) == L.ERR_SHAPE
    assert call(1, None, None, one, n8, 1, 64) == L.ERR_NULL
    assert call(1, one, None, one, (ctypes.c_int64 * 1)(12), 1, 64) == L.ERR_SHAPE
    assert call(1, one, None, one, n8, 1, 100) == L.ERR_SHAPE
    assert call(1, one, None, one, n8, 0, 64) == L.OK


def write_host_check_fixture(path, orc, synth):
    """Inputs and the CPU checker's expected values for marian-dev_amd/host/host_check.cpp (layout in
    that file's header)."""
    from oracle import decode_ops
    M, K, N, N2, R, C, nbestN = 24, 192, 128, 40, 6, 520, 4   # (N is the K of the chained second call)
    A = synth.normal(7, synth.STREAM_A, (M, K), 1.0)
    W = synth.normal(7, synth.STREAM_W, (K, N), 0.02)
    bias = synth.normal(7, synth.STREAM_BIAS, (N,), 0.01)
    W2 = synth.normal(8, synth.STREAM_W, (N, N2), 0.02)
    idx = np.sort(np.random.default_rng(7).choice(N, size=16, replace=False)).astype(np.uint32)
    Aq, Bq, Bq2 = orc.prepare_a(A), orc.prepare_b(W), orc.prepare_b(W2)
    L = load("layout")
    Bq_dev, Bq2_dev = L.to_prepared(Bq, K, N), L.to_prepared(Bq2, N, N2)   # as the device holds them
    out_relu, acc = orc.affine(Aq, Bq, bias, M, K, N, 1.0, True)
    out_sl, _ = orc.affine_shortlist(Aq, Bq, bias, idx, M, K, N, 0.5, False)
    out2, _ = orc.affine(orc.prepare_a(out_relu), Bq2, None, M, N, N2, 1.0, False)
    X = synth.normal(9, synth.STREAM_A, (R, C), 2.0)
    gamma = synth.normal(9, synth.STREAM_W, (C,), 0.2) + f32(1.0)
    beta = synth.normal(9, synth.STREAM_BIAS, (C,), 0.5)
    Xrev = np.ascontiguousarray(X.ravel()[::-1].reshape(R, C))
    ln = decode_ops.layer_norm(X, gamma, beta, 1e-6, add=Xrev)
    sm, lsm = decode_ops.softmax(X), decode_ops.logsoftmax(X)
    nb_val, nb_key = decode_ops.nbest(lsm, nbestN)
    from oracle import oracle16
    Aq16, Bq16 = oracle16.prepare_a(A), oracle16.prepare_b(W)
    out16, _ = oracle16.affine(Aq16, Bq16, bias, M, K, N, 1.0, True)
    with open(path, "wb") as f:
        f.write(b"MHC3")
        f.write(np.array([M, K, N, N2, idx.size, R, C, nbestN], np.int32).tobytes())
        for arr, ty in [(A, f32), (W, f32), (bias, f32), (W2, f32), (idx, np.uint32), (Aq, np.int8),
                        (Bq_dev.view(np.int8), np.int8), (Bq2_dev.view(np.int8), np.int8), (Bq, np.int8), (acc, np.int32), (out_relu, f32), (out_sl, f32), (out2, f32), (X, f32),
                        (gamma, f32), (beta, f32), (ln, f32), (sm, f32), (lsm, f32), (nb_val, f32),
                        (nb_key, np.uint32), (Aq16, np.int16), (Bq16, np.int16), (out16, f32)]:
            f.write(np.ascontiguousarray(arr, dtype=ty).tobytes())


def test_cpp_host_side(integer, orc, synth, tmp_path):
    """The C++ host side (host/hip_device.h: Device, Allocator, TensorAllocator, copy, fill;
    host/hip_int8_interface.h and host/hip_ops_interface.h: the operator wrappers) on the GPU, every
    buffer carved from the allocator, whose slab is forced to move between prepareA and multiply,
    between two affineOrDot calls and inside a chained pair; results against the CPU checker's
    values handed over in a fixture file.  Built by __graft_entry__.build()."""
    import subprocess
    from conftest import ROOT
    exe = os.path.join(ROOT, "marian-dev_amd", "host", "host_check")
    assert os.path.exists(exe), "host_check not built"
    say("host_check")
    fixture = os.path.join(tmp_path, "host_check.fixture")
    write_host_check_fixture(fixture, orc, synth)
    r = subprocess.run([exe, fixture], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    print(r.stdout)
    assert r.returncode == 0 and "-> OK" in r.stdout and "FAILED" not in r.stdout, r.stdout


@pytest.mark.parametrize("program,key", [("eager_sweep", "eager_ms_per_pass_cpp_host"), ("eager_step", "eager_ms_per_step_cpp_host")])
def test_cpp_host_programs_that_launch_call_by_call(program, key):
    """The two C++ programs bench.py takes its eager figures from (the decode sweep and the full
    transformer-big decoding step through the C++ wrappers, no recorded graph) run and report; the
    step's own check - finite log-probabilities, every n-best key inside its sentence - holds."""
    import json
    import subprocess
    from conftest import ROOT
    exe = os.path.join(ROOT, "marian-dev_amd", "host", program)
    assert os.path.exists(exe), program + " not built"
    say(program)
    r = subprocess.run([exe, "3", "1"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=150)
    assert r.returncode == 0, r.stderr[-1000:]
    line = json.loads(r.stdout.strip().splitlines()[-1])
    assert line[key] > 0
    if program == "eager_step":
        assert line["nbest_sane"] is True and line["launches_per_step"] == 58
