"""The .bin container keeps Type::intgemm8 items in their on-disk layout (reference
src/common/binary.cpp; container test src/tests/units/binary_tests.cpp:14-79 saves two items and
checks names, shapes and bytes after loading - repeated here, plus the intgemm8 specifics)."""
import os
import struct

import numpy as np
import pytest

from conftest import load

f32 = np.float32


def test_roundtrip_names_shapes_bytes_and_alignment(tmp_path, orc, synth):
    B = load("binary")
    T = load("types")
    W = synth.normal(5, synth.STREAM_W, (64, 24), 0.02)
    q = orc.prepare_b(W)
    items = [B.float_item("decoder_ff_logit_out_b", np.arange(24, dtype=f32).reshape(1, 24)),
             B.intgemm8_item("decoder_l1_ffn_W1", q, (64, 24)),
             B.float_item("Wemb", synth.normal(6, synth.STREAM_W, (10, 64), 0.02))]
    path = os.path.join(tmp_path, "model.bin")
    B.save_items(path, items)
    raw = open(path, "rb").read()
    version, n = struct.unpack_from("<QQ", raw, 0)
    assert version == 1 and n == 3
    # second header: type id of intgemm8 is 0x10000 + 1, shape length 2, data padded to 256
    name_len, type_id, shape_len, data_len = struct.unpack_from("<QQQQ", raw, 16 + 32)
    assert type_id == 0x10000 + 1 and shape_len == 2 and name_len == len("decoder_l1_ffn_W1") + 1
    assert data_len % 256 == 0 and data_len >= 64 * 24 + 4
    total_payload = sum(len(it.bytes) for it in items)
    assert (len(raw) - total_payload) % 256 == 0            # payload starts 256-byte aligned
    got = B.load_items(path)
    assert [g.name for g in got] == [i.name for i in items]
    assert [g.shape for g in got] == [i.shape for i in items]
    for g, i in zip(got, items):
        assert g.type == i.type and np.array_equal(g.bytes, i.bytes)
    w = got[1]
    assert w.shape == (64, 24)                               # logical [K, N], NOT transposed
    assert w.quant_mult() == f32(127.0) / np.max(np.abs(W))
    want = np.clip(np.rint((W.T * w.quant_mult()).astype(f32)), -127, 127).astype(np.int8)
    assert np.array_equal(w.payload(), want)                 # payload is W^T row-major [N, K]
    assert T.requiredBytes(w.shape, w.type) == 64 * 24 + 4


def test_cpu_tiled_items_are_refused(tmp_path, orc, synth):
    B = load("binary")
    T = load("types")
    q = orc.prepare_b(synth.normal(7, synth.STREAM_W, (64, 8), 0.02))
    it = B.intgemm8_item("encoder_l1_self_Wq", q, (64, 8))
    it.type = T.Type.intgemm8avx512vnni
    path = os.path.join(tmp_path, "tiled.bin")
    B.save_items(path, [it])
    with pytest.raises(ValueError, match="CPU-tiled"):
        B.load_items(path)


def test_unaligned_item_is_refused_on_save(tmp_path):
    B = load("binary")
    T = load("types")
    with pytest.raises(ValueError, match="not 256-byte aligned"):
        B.save_items(os.path.join(tmp_path, "x.bin"),
                     [B.Item("a", (3,), T.Type.float32, np.zeros(12, np.uint8))])
