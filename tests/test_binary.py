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


@pytest.mark.parametrize("name", ["intgemm16sse2", "intgemm16avx2", "intgemm16avx512"])
def test_cpu_tiled_sixteen_bit_items_are_refused(tmp_path, name):
    """The CPU-tiled 16-bit variants (what the reference turns an intgemm16 item into at load,
    src/common/binary.cpp:108-110) cannot be consumed by a GPU."""
    B = load("binary")
    T = load("types")
    raw = np.zeros(64 * 8 * 2 + 4, np.uint8)
    raw[-4:] = np.frombuffer(f32(1024.0).tobytes(), np.uint8)
    it = B.Item("decoder_l1_ffn_W1", (64, 8), T.Type[name], np.frombuffer(B._pad256(raw.tobytes()), np.uint8))
    path = os.path.join(tmp_path, "w16.bin")
    B.save_items(path, [it])
    with pytest.raises(ValueError, match="decoder_l1_ffn_W1 has the CPU-tiled type %s" % name):
        B.load_items(path)


def test_sixteen_bit_item_roundtrip_keeps_the_payload_verbatim(tmp_path, synth):
    """A hardware-agnostic Type::intgemm16 item: int16 W^T [N, K] then quantMult 1024 at byte 2*K*N
    (reference src/tensors/cpu/expression_graph_packable.h:203-235), kept as stored."""
    from oracle import oracle16
    B = load("binary")
    T = load("types")
    W = synth.normal(5, synth.STREAM_W, (64, 24), 0.02)
    q = oracle16.prepare_b(W)
    path = os.path.join(tmp_path, "m16.bin")
    B.save_items(path, [B.intgemm16_item("decoder_l1_ffn_W1", q, (64, 24))])
    (w,) = B.load_items(path)
    assert w.type == T.Type.intgemm16 and w.shape == (64, 24) and w.quant_mult() == 1024.0
    assert T.requiredBytes(w.shape, w.type) == 64 * 24 * 2 + 4
    want = np.clip(np.rint((W.T * f32(1024.0)).astype(f32)), -32768, 32767).astype(np.int16)
    assert np.array_equal(w.payload(), want)


def test_unknown_item_type_is_reported_with_the_item_name(tmp_path):
    B = load("binary")
    T = load("types")
    it = B.float_item("special:model.yml", np.zeros(64, f32))
    path = os.path.join(tmp_path, "u.bin")
    B.save_items(path, [it])
    raw = bytearray(open(path, "rb").read())
    struct.pack_into("<Q", raw, 16 + 8, 0x20000 + 1)         # no such id in Marian's enum
    open(path, "wb").write(raw)
    with pytest.raises(ValueError, match=r"special:model.yml has the unsupported item type 0x20001"):
        B.load_items(path)
    struct.pack_into("<Q", raw, 16 + 8, int(T.Type.packed8avx2))
    open(path, "wb").write(raw)
    with pytest.raises(ValueError, match=r"special:model.yml has the FBGEMM-packed type packed8avx2"):
        B.load_items(path)


def test_operator_refuses_cpu_tiled_weights_with_the_reference_text():
    """affineOrDot's type switch (reference src/tensors/cpu/intgemm_interface.h:104-127): on a GPU
    only the hardware-agnostic intgemm8 and intgemm16 weights can be multiplied; the CPU-tiled
    variants end in the default branch."""
    import torch
    integer = load("integer")
    T = load("types")
    a = torch.zeros(2, 64)
    for t in (T.Type.intgemm16avx2, T.Type.intgemm8avx2, T.Type.intgemm16sse2):
        w = integer.QTensor(torch.zeros(64 * 8 * 2 + 4, dtype=torch.int8), (64, 8), t)
        with pytest.raises(integer.MarianRuntimeError, match=r"Unsupported type .*%s.* for Intgemm type\?\?" % t.name):
            integer.affineOrDot(a, w)
    with pytest.raises(integer.MarianRuntimeError, match="Intgemm expects type of B to be a variant of intgemm"):
        integer.affineOrDot(a, integer.QTensor(torch.zeros(64 * 8 * 4, dtype=torch.int8), (64, 8), T.Type.float32))
    # 8-bit weights as a model file holds them (plain rows) are refused until they have been re-tiled
    from_file = integer.QTensor(torch.zeros(64 * 8 + 4, dtype=torch.int8), (64, 8), T.Type.intgemm8)
    assert not from_file.prepared
    for call in (lambda: integer.affineOrDot(a, from_file), lambda: integer.affine_f32(a, from_file),
                 lambda: integer.affine_f32_grouped(a, [(from_file, None)]),
                 lambda: integer.multiply(integer.QTensor(torch.zeros(2 * 64 + 4, dtype=torch.int8), (2, 64), T.Type.intgemm8), from_file)):
        with pytest.raises(integer.MarianRuntimeError, match="file order.*prepareAndTransposeB"):
            call()
