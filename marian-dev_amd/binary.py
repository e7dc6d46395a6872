"""Marian `.bin` model container (version 1) for a HIP backend.

Restates the reader and writer of reference src/common/binary.cpp:
  header  u64 version (=1), u64 n, n x Header{u64 nameLength (with NUL), u64 type, u64 shapeLength,
          u64 dataLength}, all names (NUL-terminated), all shapes (int32), u64 offset, `offset`
          zero bytes so that the payload starts on a 256-byte boundary  (:217-254, :158-215)
  payload items back to back, each padded to a multiple of 256 bytes                  (:242-250)

What differs from the reference loader (:88-114): a `Type::intgemm8` item is returned exactly as
stored - int8 W^T row-major [N, K] followed by the fp32 quantMult at byte K*N; the reference re-tiles
it on the spot for the CPU it runs on (prepareAndTransposeB, src/tensors/cpu/integer_common.h:189-216),
here that step happens on the device once the bytes are uploaded (integer.prepareAndTransposeB).  Items whose type is one of the CPU-tiled variants
(intgemm8ssse3/avx2/avx512/avx512vnni, intgemm16sse2/avx2/avx512) cannot be used on a GPU and are
refused, and so are FBGEMM-packed items.  A hardware-agnostic `Type::intgemm16` item (int16 W^T
[N, K] + quantMult 1024 at byte 2*K*N, src/tensors/cpu/expression_graph_packable.h:203-235) is kept
verbatim like an intgemm8 one.  A type id outside Marian's enum is reported with the item's name.
"""
import struct

import numpy as np

from .types import Type, elements, isHardwareSpecific, isIntgemm, isPacked, requiredBytes, sizeOf

BINARY_FILE_VERSION = 1
_HEADER = struct.Struct("<QQQQ")


class Item:
    """Counterpart of io::Item (reference src/common/io_item.h:11-27): name, shape, type, bytes."""

    def __init__(self, name, shape, type_, data):
        self.name = name
        self.shape = tuple(int(d) for d in shape)
        self.type = Type(type_)
        self.bytes = np.ascontiguousarray(data).view(np.uint8).ravel()

    def quant_mult(self):
        n = elements(self.shape) * sizeOf(self.type)
        return self.bytes[n:n + 4].view(np.float32)[0]

    def payload(self):
        """int8 (int16) W^T [N, K] for an intgemm8 (intgemm16) item of logical shape [K, N]."""
        K, N = self.shape
        width = sizeOf(self.type)
        return self.bytes[: K * N * width].view(np.int8 if width == 1 else np.int16).reshape(N, K)


def _pad256(b):
    pad = (-len(b)) % 256
    return b + b"\x00" * pad


def intgemm8_item(name, q_flat, shape):
    """Item for a quantized weight: q_flat = payload + quantMult tail (K*N + 4 bytes), padded to a
    multiple of 256 bytes like Marian's allocator pieces
    (reference src/tensors/cpu/expression_graph_packable.h:242-250)."""
    raw = np.ascontiguousarray(q_flat).view(np.uint8).tobytes()[: requiredBytes(shape, Type.intgemm8)]
    return Item(name, shape, Type.intgemm8, np.frombuffer(_pad256(raw), dtype=np.uint8))


def intgemm16_item(name, q_flat, shape):
    """Item for a 16-bit quantized weight: q_flat = int16 payload + quantMult tail (2*K*N + 4 bytes)."""
    raw = np.ascontiguousarray(q_flat).view(np.uint8).tobytes()[: requiredBytes(shape, Type.intgemm16)]
    return Item(name, shape, Type.intgemm16, np.frombuffer(_pad256(raw), dtype=np.uint8))


def float_item(name, array):
    a = np.ascontiguousarray(array, dtype=np.float32)
    return Item(name, a.shape, Type.float32, np.frombuffer(_pad256(a.tobytes()), dtype=np.uint8))


def save_items(path, items):
    """reference src/common/binary.cpp:158-254 (unencrypted form)."""
    buf = bytearray()
    buf += struct.pack("<Q", BINARY_FILE_VERSION)
    buf += struct.pack("<Q", len(items))
    for it in items:
        if len(it.bytes) % 256 != 0:
            raise ValueError("Binary item size ({}) is not 256-byte aligned for tensor {}".format(
                len(it.bytes), it.name))
        buf += _HEADER.pack(len(it.name.encode()) + 1, int(it.type), len(it.shape), len(it.bytes))
    for it in items:
        buf += it.name.encode() + b"\x00"
    for it in items:
        buf += struct.pack("<%di" % len(it.shape), *it.shape)
    pos = len(buf)
    nextpos = ((pos + 8) // 256 + 1) * 256
    offset = nextpos - pos - 8
    buf += struct.pack("<Q", offset) + b"\x00" * offset
    with open(path, "wb") as f:
        f.write(buf)
        for it in items:
            f.write(it.bytes.tobytes())


def load_items(path):
    """reference src/common/binary.cpp:35-116, keeping intgemm8 payloads verbatim."""
    data = np.fromfile(path, dtype=np.uint8)
    mv = memoryview(data)
    pos = 0
    (version,) = struct.unpack_from("<Q", mv, pos)
    pos += 8
    if version != BINARY_FILE_VERSION:
        raise ValueError("Unknown binary file version {}".format(version))
    (n,) = struct.unpack_from("<Q", mv, pos)
    pos += 8
    headers = []
    for _ in range(n):
        headers.append(_HEADER.unpack_from(mv, pos))
        pos += _HEADER.size
    names = []
    for h in headers:
        names.append(bytes(mv[pos:pos + h[0] - 1]).decode())
        pos += h[0]
    shapes = []
    for h in headers:
        shapes.append(struct.unpack_from("<%di" % h[2], mv, pos))
        pos += 4 * h[2]
    (offset,) = struct.unpack_from("<Q", mv, pos)
    pos += 8 + offset
    items = []
    for h, name, shape in zip(headers, names, shapes):
        try:
            type_ = Type(h[1])
        except ValueError:
            raise ValueError("Item {} has the unsupported item type 0x{:x} (this loader knows: {})".format(
                name, h[1], ", ".join(t.name for t in Type))) from None
        if isPacked(type_):
            raise ValueError("Item {} has the FBGEMM-packed type {}: a CPU cache layout that a GPU backend "
                             "cannot consume (reference src/tensors/cpu/fbgemm/packed_gemm.h)".format(name, type_.name))
        if isHardwareSpecific(type_):
            raise ValueError(
                "Item {} has the CPU-tiled type {}; a GPU backend needs the hardware-agnostic "
                "intgemm8 / intgemm16 payload (convert the model with marian-conv --gemm-type intgemm8)".format(
                    name, type_.name))
        if isIntgemm(type_) and h[3] < requiredBytes(shape, type_):
            raise ValueError("Item {} is shorter than payload + quantMult".format(name))
        items.append(Item(name, shape, type_, data[pos:pos + h[3]]))
        pos += h[3]
    return items
