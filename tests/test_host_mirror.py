"""Host-side logic of the Python mirror that needs no GPU."""
import gc

import torch

from conftest import load


def _backend_without_device(integer):
    be = object.__new__(integer.Backend)   # (the constructor allocates a device workspace)
    be._memo = {}
    be.gemmType = None
    return be


def test_memoized_prepare_b_is_keyed_on_the_tensor_not_on_its_address(monkeypatch):
    """Two different tensors that present the same (address, shape, version) - what torch's
    caching allocator produces when a weight is freed and a new one of the same shape is created -
    must not share a quantized copy; entries go away with their tensors."""
    integer = load("integer")
    be = _backend_without_device(integer)
    made = []

    def fake_prepare_b(w):
        made.append(object())
        return made[-1]
    monkeypatch.setattr(integer, "prepareB", fake_prepare_b)
    monkeypatch.setattr(integer.Backend, "_memo_key", staticmethod(lambda w: (0x7000, tuple(w.shape), 0)))
    w1, w2 = torch.zeros(64, 8), torch.ones(64, 8)
    q1 = be.memoizedPrepareB(w1)
    assert be.memoizedPrepareB(w1) is q1 and len(made) == 1          # remembered
    q2 = be.memoizedPrepareB(w2)                                      # same key, other tensor
    assert q2 is not q1 and len(made) == 2
    assert be.memoizedPrepareB(w2) is q2 and len(made) == 2
    assert be.memoizedPrepareB(w1) is not q2 and len(made) == 3      # and back: never the other's copy
    del w1, w2
    gc.collect()
    assert be._memo == {}


def test_memoized_prepare_b_drops_old_versions_and_dead_owners(monkeypatch):
    integer = load("integer")
    be = _backend_without_device(integer)
    monkeypatch.setattr(integer, "prepareB", lambda w: object())
    w = torch.zeros(64, 8)
    q0 = be.memoizedPrepareB(w)
    w.add_(1.0)                                  # in-place update: new version
    q1 = be.memoizedPrepareB(w)
    assert q1 is not q0 and len(be._memo) == 1   # the stale version's entry is gone
    for _ in range(50):                          # a loop over freshly created weights does not grow the cache
        be.memoizedPrepareB(torch.zeros(64, 8))
        gc.collect()
    assert len(be._memo) <= 2


def _nbest_plan_shim(tmp_path):
    """nbest_plan() of the library's host code, compiled on its own with g++ (it is plain C++)."""
    import ctypes
    import os
    import subprocess
    from conftest import ROOT
    src = tmp_path / "plan_shim.cpp"
    src.write_text('#include "nbest_plan.h"\n'
                   'extern "C" void plan(long long beam, long long batch, long long vocab, long long n, long long* out) {\n'
                   '  const marian_hip::NbestPlan p = marian_hip::nbest_plan(beam, batch, vocab, n);\n'
                   '  out[0] = p.perSeg; out[1] = p.sliceLen; out[2] = p.parts;\n}\n')
    so = tmp_path / "plan_shim.so"
    subprocess.check_call(["g++", "-O1", "-shared", "-fPIC", "-I", os.path.join(ROOT, "marian-dev_amd", "csrc"),
                           "-o", str(so), str(src)])
    lib = ctypes.CDLL(str(so))
    lib.plan.argtypes = [ctypes.c_longlong] * 4 + [ctypes.POINTER(ctypes.c_longlong)]

    def plan(beam, batch, vocab, n):
        out = (ctypes.c_longlong * 3)()
        lib.plan(beam, batch, vocab, n, out)
        return int(out[0]), int(out[1]), int(out[2])
    return plan


def test_nbest_plan_tiles_every_row_and_merge_equals_global_nbest(tmp_path):
    """The split n-best: the slices of the plan tile every beam segment exactly (no gap, no
    overlap, no empty slice, 16-byte aligned starts), the merge never sees more than 1024
    candidates, and - with the order (score descending, position ascending) used at both levels -
    the N best of the slices' N best are the N best of the row, ties included."""
    import numpy as np
    plan = _nbest_plan_shim(tmp_path)
    rng = np.random.default_rng(11)
    for beam, batch, vocab, n in [(4, 32, 32000, 4), (1, 1, 32000, 1), (4, 1, 32000, 4), (8, 2, 50000, 8),
                                  (64, 1, 4096, 16), (4, 32, 100, 4), (2, 3, 4097, 2), (6, 64, 128000, 6),
                                  (1, 1, 7, 7), (12, 1, 65536, 16), (4, 4096, 8, 4), (3, 5, 12289, 3)]:
        per_seg, slice_len, parts = plan(beam, batch, vocab, n)
        assert per_seg >= 1 and parts == beam * per_seg
        assert slice_len % 4 == 0
        assert per_seg * slice_len >= vocab > (per_seg - 1) * slice_len      # tiles the segment, last slice not empty
        assert per_seg == 1 or parts * n <= 1024                            # the merge's capacity
        assert per_seg == 1 or slice_len >= 1024                            # slices stay long
        # the algorithm on this plan, in numpy, with many ties
        row = np.round(rng.standard_normal(beam * vocab), 1).astype(np.float32)
        order = np.lexsort((np.arange(row.size), -row))                      # score desc, position asc
        want = order[:n]
        cand = []
        for k in range(beam):
            for p in range(per_seg):
                lo, hi = k * vocab + p * slice_len, k * vocab + min((p + 1) * slice_len, vocab)
                seg = row[lo:hi]
                best = np.lexsort((np.arange(seg.size), -seg))[:n] + lo
                cand.extend(best.tolist())
        cand = np.array(cand)
        got = cand[np.lexsort((cand, -row[cand]))][:n]
        assert np.array_equal(got, want), (beam, batch, vocab, n)
