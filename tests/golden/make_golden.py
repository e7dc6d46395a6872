"""Writes tests/golden/intgemm8_small.npz: inputs and expected results of the int8 affine path
on small shapes, computed with plain numpy (float32 element ops, int64 matmul) - an
implementation independent of both the C checker in oracle/ and the HIP kernels.

Nothing from the reference is imported or executed: the reference's arithmetic for this path
lives in the intgemm submodule, which is not part of the reference tree, and the reference
holds no int8 test vectors.  The expected values follow the call sites
src/tensors/cpu/intgemm_interface.h:17-32,60-88 and
src/tensors/cpu/expression_graph_packable.h:160-201.

Run from the repo root:  python tests/golden/make_golden.py
"""
import importlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
synth = importlib.import_module("marian-dev_amd.synth")

f32 = np.float32


def quantize(x, qm):
    v = (x.astype(f32) * f32(qm)).astype(f32)
    return np.clip(np.rint(v), -127, 127).astype(np.int8)


def case(seed, M, K, N, scale, relu, with_bias):
    A = synth.normal(seed, synth.STREAM_A, (M, K), 1.0)
    W = synth.normal(seed, synth.STREAM_W, (K, N), 0.02)
    bias = synth.normal(seed, synth.STREAM_BIAS, (N,), 0.01) if with_bias else None
    aqm = f32(127.0) / np.max(np.abs(A)).astype(f32)
    bqm = f32(127.0) / np.max(np.abs(W)).astype(f32)
    Aq = quantize(A, aqm)
    Bt = quantize(W.T.copy(), bqm)  # payload: quantized transpose, [N, K]
    acc = (Aq.astype(np.int64) @ Bt.astype(np.int64).T)
    assert np.abs(acc).max() < 2 ** 31
    unquant = (f32(1.0) / (aqm * bqm).astype(f32)).astype(f32) * f32(scale)
    y = (acc.astype(f32) * f32(unquant)).astype(f32)
    if with_bias:
        y = (y + bias[None, :]).astype(f32)
    if relu:
        y = np.where(y > 0, y, f32(0)).astype(f32)
    return dict(A=A, W=W, bias=bias if with_bias else np.zeros(0, f32), aqm=aqm, bqm=bqm,
                Aq=Aq, Bt=Bt, acc=acc.astype(np.int32), out=y, scale=f32(scale),
                relu=np.int32(relu), with_bias=np.int32(with_bias))


def main():
    cases = [
        case(11, 8, 64, 16, 1.0, 0, 1),
        case(12, 5, 128, 8, 1.0, 1, 1),
        case(13, 19, 64, 24, 0.125, 0, 0),
        case(14, 1, 64, 8, 1.0, 1, 1),
    ]
    out = {}
    for i, c in enumerate(cases):
        for k, v in c.items():
            out["c{}_{}".format(i, k)] = v
    out["n_cases"] = np.int32(len(cases))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "intgemm8_small.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
