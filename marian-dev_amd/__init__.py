"""MI355X (gfx950) backend for Marian's intgemm8 affine/dot path.

Layout:
  csrc/        hand-written HIP kernels and the C ABI (built into libmarian_hip_int8.so)
  _lib.py      ctypes binding of the C ABI; raises if the library is missing
  types.py     Marian's element types for this path (Type::intgemm8 ...) and requiredBytes
  integer.py   host mirror of src/tensors/cpu/intgemm_interface.h (prepareA, affineOrDot) and of
               the dot/affine/affineWithReluDropout dispatch of src/graph/expression_operators.cpp
  binary.py    Marian .bin model container with intgemm8 items kept in their on-disk layout
  output.py    tied int8 output layer: Shortlist id maps and padding, logits, best words
  synth.py     deterministic synthetic inputs for tests and the benchmark

Device memory and streams come from torch (ROCm build); all arithmetic runs in the HIP library.
"""
from . import types  # noqa: F401
