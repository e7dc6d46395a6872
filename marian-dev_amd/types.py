"""Element types of the path, numerically identical to Marian's `enum class Type`
(reference src/common/types.h:270-328) so that .bin model files keep their meaning."""
import enum


class TypeClass(enum.IntEnum):
    signed_type = 0x00100
    unsigned_type = 0x00200
    float_type = 0x00400
    avx2_type = 0x01000
    avx512_type = 0x02000
    sse2_type = 0x04000
    ssse3_type = 0x08000
    packed_type = 0x00800
    intgemm_type = 0x10000
    size_mask = 0x000FF
    class_mask = 0xFFF00


class Type(enum.IntEnum):
    int8 = TypeClass.signed_type + 1
    int16 = TypeClass.signed_type + 2
    int32 = TypeClass.signed_type + 4
    int64 = TypeClass.signed_type + 8
    uint8 = TypeClass.unsigned_type + 1
    uint16 = TypeClass.unsigned_type + 2
    uint32 = TypeClass.unsigned_type + 4
    uint64 = TypeClass.unsigned_type + 8
    float16 = TypeClass.float_type + 2
    float32 = TypeClass.float_type + 4
    float64 = TypeClass.float_type + 8
    packed16 = TypeClass.packed_type + 2
    packed8avx2 = TypeClass.packed_type + 1 + TypeClass.avx2_type
    packed8avx512 = TypeClass.packed_type + 1 + TypeClass.avx512_type
    intgemm8 = TypeClass.intgemm_type + 1
    intgemm16 = TypeClass.intgemm_type + 2
    intgemm8ssse3 = TypeClass.intgemm_type + 1 + TypeClass.ssse3_type
    intgemm8avx2 = TypeClass.intgemm_type + 1 + TypeClass.avx2_type
    intgemm8avx512 = TypeClass.intgemm_type + 1 + TypeClass.avx512_type
    intgemm8avx512vnni = TypeClass.intgemm_type + 1 + TypeClass.avx512_type + 4096
    intgemm16sse2 = TypeClass.intgemm_type + 2 + TypeClass.sse2_type
    intgemm16avx2 = TypeClass.intgemm_type + 2 + TypeClass.avx2_type
    intgemm16avx512 = TypeClass.intgemm_type + 2 + TypeClass.avx512_type

    # messages print a type by name, like operator<< of reference src/common/types.h:419-456
    def __str__(self):
        return self.name

    def __format__(self, spec):
        return format(self.name, spec)


def sizeOf(t):
    """Bytes per element (reference src/common/types.h:346-348)."""
    return int(t) & TypeClass.size_mask


def isFloat(t):
    return (int(t) & TypeClass.float_type) != 0


def isIntgemm(t):
    """reference src/common/types.h:378-380"""
    return (int(t) & TypeClass.intgemm_type) != 0


def isPacked(t):
    """reference src/common/types.h:358-360"""
    return (int(t) & TypeClass.packed_type) != 0


def isHardwareSpecific(t):
    """True for the CPU-tiled intgemm variants whose payload a GPU cannot consume."""
    hw = (TypeClass.avx2_type | TypeClass.avx512_type | TypeClass.sse2_type
          | TypeClass.ssse3_type)
    return isIntgemm(t) and (int(t) & hw) != 0


def elements(shape):
    n = 1
    for d in shape:
        n *= int(d)
    return n


def requiredBytes(shape, t):
    """reference src/common/types.cpp:32-34: intgemm tensors carry one extra fp32 (quantMult)."""
    if isIntgemm(t):
        return elements(shape) * sizeOf(t) + 4
    return elements(shape) * sizeOf(t)


def typeFromString(s):
    """reference src/common/types.h:500-540 (subset relevant to this path)."""
    try:
        return Type[s]
    except KeyError:
        raise ValueError("Unknown type {}".format(s))
