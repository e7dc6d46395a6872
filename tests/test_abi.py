"""The C-ABI library loads and exports every symbol include/marian_hip_int8.h declares; argument
validation (which runs before any HIP call) behaves as documented.  No compute without a GPU."""
import ctypes
import os
import re
import subprocess

import pytest

from conftest import ROOT, load

HEADERS = [os.path.join(ROOT, "include", h) for h in ("marian_hip_int8.h", "marian_hip_int16.h", "marian_hip_ops.h")]
TUNING_HEADER = os.path.join(ROOT, "include", "marian_hip_int8_tuning.h")


def exported_symbols(path):
    out = subprocess.run(["nm", "-D", "--defined-only", path], check=True, capture_output=True, text=True).stdout
    return sorted(line.split()[-1] for line in out.splitlines() if line.strip())


def declared_functions(headers=HEADERS):
    names = set()
    for header in headers:
        text = open(header).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(marian_hip_\w+)\s*\(", text))
    return sorted(names)


def test_header_declares_expected_entry_points():
    names = declared_functions()
    for must in ("marian_hip_int8_prepare_a", "marian_hip_int8_prepare_b",
                 "marian_hip_int8_prepare_b_quantized_transposed", "marian_hip_int8_affine",
                 "marian_hip_int8_affine_shortlist", "marian_hip_int8_multiply_i32",
                 "marian_hip_layer_norm", "marian_hip_softmax", "marian_hip_logsoftmax",
                 "marian_hip_transpose0213", "marian_hip_bdot_legacy", "marian_hip_attention",
                 "marian_hip_nbest"):
        assert must in names


def test_library_exports_every_declared_symbol():
    L = load("_lib")
    assert os.path.exists(L.LIB_PATH), "build the library first (__graft_entry__.build())"
    lib = ctypes.CDLL(L.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), name
    # and the Python binding covers the same set
    assert sorted(L.SIGNATURES) == declared_functions()


def test_shipped_library_exports_exactly_what_the_headers_declare():
    """No measurement switch, no undeclared hook and no C++ symbol leaves the shipped library; the
    tuning build adds exactly the functions of its own header."""
    L = load("_lib")
    assert exported_symbols(L.LIB_PATH) == declared_functions()
    assert os.path.exists(L.TUNING_LIB_PATH), "build the library first (__graft_entry__.build())"
    tuning = declared_functions([TUNING_HEADER])
    assert tuning == ["marian_hip_int8_debug_profile", "marian_hip_int8_set_kernel", "marian_hip_nbest_set_fenced",
                      "marian_hip_probe_mfma", "marian_hip_probe_mix", "marian_hip_probe_stream"]
    assert exported_symbols(L.TUNING_LIB_PATH) == sorted(declared_functions() + tuning)
    assert sorted(L.TUNING_SIGNATURES) == tuning


def test_status_strings_and_version():
    L = load("_lib")
    lib = L.lib()
    assert lib.marian_hip_int8_abi_version() == 3
    assert lib.marian_hip_int8_workspace_bytes() >= 4096
    seen = {lib.marian_hip_status_string(i) for i in range(8)}
    assert len(seen) == 8 and lib.marian_hip_status_string(0) == b"ok"


def test_argument_validation_returns_codes_not_aborts():
    L = load("_lib")
    lib = L.lib()
    buf = 0x1000  # never dereferenced: every call below is rejected or a no-op before launch
    assert lib.marian_hip_int8_affine(None, buf, None, buf, 1, 64, 8, 1.0, 0, None) == L.ERR_NULL
    assert lib.marian_hip_int8_affine(buf, buf, None, buf, 1, 63, 8, 1.0, 0, None) == L.ERR_SHAPE
    assert lib.marian_hip_int8_affine(buf, buf, None, buf, 1, 64, 12, 1.0, 0, None) == L.ERR_SHAPE
    assert lib.marian_hip_int8_affine(buf, buf, None, buf, -1, 64, 8, 1.0, 0, None) == L.ERR_SHAPE
    assert lib.marian_hip_int8_affine(buf + 4, buf, None, buf, 1, 64, 8, 1.0, 0, None) == L.ERR_ALIGN
    assert lib.marian_hip_int8_affine(buf, buf, buf + 2, buf, 1, 64, 8, 1.0, 0, None) == L.ERR_ALIGN
    assert lib.marian_hip_int8_affine(buf, buf, None, buf, 1 << 26, 64, 8, 1.0, 0, None) == L.ERR_RANGE
    assert lib.marian_hip_int8_affine(buf, buf, None, buf, 0, 64, 8, 1.0, 0, None) == L.OK  # empty batch
    assert lib.marian_hip_int8_affine_shortlist(buf, buf, None, None, 8, buf, 1, 64, 8, 1.0, 0, None) == L.ERR_NULL
    assert lib.marian_hip_int8_affine(None, None, None, None, 0, 64, 8, 1.0, 0, None) == L.OK
    # float operators of include/marian_hip_ops.h
    assert lib.marian_hip_layer_norm(buf, None, buf, 8, None, 0, buf, 2, 0, 1e-9, None, None) == L.ERR_SHAPE
    assert lib.marian_hip_layer_norm(buf, None, buf, 7, None, 0, buf, 2, 8, 1e-9, None, None) == L.ERR_SHAPE
    assert lib.marian_hip_layer_norm(None, None, buf, 8, None, 0, buf, 2, 8, 1e-9, None, None) == L.ERR_NULL
    assert lib.marian_hip_layer_norm(buf, None, buf, 8, None, 0, buf, 0, 8, 1e-9, None, None) == L.OK
    assert lib.marian_hip_softmax(buf, buf, 0, 1, buf, 2, 8, None) == L.ERR_SHAPE
    assert lib.marian_hip_softmax(buf + 2, None, 0, 0, buf, 2, 8, None) == L.ERR_ALIGN
    assert lib.marian_hip_logsoftmax(buf, None, 2, 8, None) == L.ERR_NULL
    assert lib.marian_hip_transpose0213(buf, buf, 1, 2, 3, 4, None) == L.ERR_SHAPE   # aliasing
    assert lib.marian_hip_transpose0213(buf, buf + 64, 0, 2, 3, 4, None) == L.OK
    assert lib.marian_hip_bdot_legacy(buf, buf, buf, 2, 2, 0, 4, 4, 0, 0, 1.0, None) == L.ERR_SHAPE
    assert lib.marian_hip_bdot_legacy(buf, None, buf, 2, 2, 1, 4, 4, 0, 0, 1.0, None) == L.ERR_NULL
    assert lib.marian_hip_attention(buf, buf, buf, None, 0, 0, buf, 2, 2, 1, 5000, 64, 0.125, None, None, None, None) == L.ERR_RANGE
    assert lib.marian_hip_nbest(buf, 2, 100, 17, buf, buf, None) == L.ERR_SHAPE
    assert lib.marian_hip_nbest(buf, 2, 100, 4, None, buf, None) == L.ERR_NULL
    assert lib.marian_hip_attention(buf, buf, None, None, 0, 0, buf, 2, 2, 1, 40, 64, 0.125, None, None, None, None) == L.ERR_NULL
    assert lib.marian_hip_attention(buf, buf, buf, None, 0, 0, buf, 4, 2, 1, 40, 64, 0.125, None, buf, buf, None) == L.ERR_SHAPE
    assert lib.marian_hip_attention_cached(buf, buf, buf, None, 0, 0, buf, 2, 2, 1, 40, 39, 64, 0.125, None, None, None, None) == L.ERR_SHAPE
    assert lib.marian_hip_attention_cached(buf, buf, buf, None, 0, 0, buf, 2, 2, 1, 5000, 6000, 64, 0.125, None, None, None, None) == L.ERR_RANGE
    assert lib.marian_hip_attention_cached(buf, None, buf, None, 0, 0, buf, 2, 2, 1, 40, 64, 64, 0.125, None, None, None, None) == L.ERR_NULL
    assert lib.marian_hip_attention_cached(buf, buf, buf, None, 0, 0, buf, 0, 2, 1, 40, 64, 64, 0.125, None, None, None, None) == L.OK
    assert lib.marian_hip_int8_affine_shortlist(buf, buf, None, buf, 12, buf, 1, 64, 8, 1.0, 0, None) == L.ERR_SHAPE
    assert lib.marian_hip_embed(buf, buf, 4, 0, 8, 1.0, None, 0, 0, buf, None, None) == L.ERR_SHAPE
    assert lib.marian_hip_embed(buf, buf, 4, 10, 8, 1.0, buf, 0, 1, buf, None, None) == L.ERR_SHAPE
    assert lib.marian_hip_embed(buf, None, 4, 10, 8, 1.0, None, 0, 0, buf, None, None) == L.ERR_NULL
    assert lib.marian_hip_embed(buf, buf, 4096, 10, 8, 1.0, None, 0, 0, buf, buf, None) == L.ERR_RANGE
    assert lib.marian_hip_embed(buf, buf + 2, 4, 10, 8, 1.0, None, 0, 0, buf, None, None) == L.ERR_ALIGN
    assert lib.marian_hip_embed(buf, buf, 0, 10, 8, 1.0, None, 0, 0, buf, None, None) == L.OK
    assert lib.marian_hip_attention_ancestors(buf, buf, buf, buf, 4, 2, 5, 8, 32, 0.125, None, buf, buf, buf, None) == L.ERR_SHAPE
    assert lib.marian_hip_attention_ancestors(buf, buf, buf, buf, 4, 2, 5, 8, 64, 0.125, None, buf, buf, None, None) == L.ERR_NULL
    assert lib.marian_hip_attention_ancestors(buf, buf, buf, buf, 4, 2, 5, 8, 64, 0.125, None, buf + 4, buf, buf, None) == L.ERR_ALIGN
    assert lib.marian_hip_attention_ancestors(buf, buf, buf, buf, 4, 2, 9, 8, 64, 0.125, None, buf, buf, buf, None) == L.ERR_SHAPE
    assert lib.marian_hip_attention_ancestors(buf, buf, buf, buf, 0, 2, 5, 8, 64, 0.125, None, buf, buf, buf, None) == L.OK
    assert lib.marian_hip_ancestors_advance(buf, buf, 4, 8, 8, buf + 4096, None) == L.ERR_SHAPE
    assert lib.marian_hip_ancestors_advance(buf, None, 4, 8, 3, buf + 4096, None) == L.ERR_NULL
    assert lib.marian_hip_select_state(buf, buf, 4, 8, 2, 64, 65, buf + 65536, None) == L.ERR_SHAPE
    assert lib.marian_hip_select_state(buf, None, 4, 8, 2, 64, 64, buf + 65536, None) == L.ERR_NULL
    assert lib.marian_hip_select_state(buf, buf, 4, 8, 2, 64, 64, buf + 1024, None) == L.ERR_ALIAS
    assert lib.marian_hip_select_state(buf, buf, 4, 8, 2, 64, 0, buf, None) == L.OK
    assert lib.marian_hip_sinusoidal_position_embeddings(None, 4, 8, 0) == L.ERR_NULL
    assert lib.marian_hip_sinusoidal_position_embeddings(None, 4, 3, 0) == L.ERR_SHAPE
    assert lib.marian_hip_sinusoidal_position_embeddings(None, 0, 8, 0) == L.OK
    assert lib.marian_hip_int8_prepare_a(buf, buf, 4, 100, buf, 4096, None) == L.ERR_SHAPE
    assert lib.marian_hip_int8_prepare_a(buf, buf, 4096, 1024, buf, 16, None) == L.ERR_WORKSPACE
    assert lib.marian_hip_int8_prepare_a(buf, buf, 0, 64, None, 0, None) == L.OK
    assert lib.marian_hip_int8_prepare_b(buf, buf, 64, 8, None, 4096, None) == L.ERR_NULL
    # the re-tiling of a model file's weights is a permutation: not in place, not on overlapping buffers
    assert lib.marian_hip_int8_prepare_b_quantized_transposed(buf, buf, 64, 8, None) == L.ERR_ALIAS
    assert lib.marian_hip_int8_prepare_b_quantized_transposed(buf, buf + 256, 64, 8, None) == L.ERR_ALIAS
    assert lib.marian_hip_int8_prepare_b_quantized_transposed(buf, buf + 1024, 100, 8, None) == L.ERR_SHAPE
    assert lib.marian_hip_int8_prepare_b_quantized_transposed(buf, None, 64, 8, None) == L.ERR_NULL
    assert lib.marian_hip_status_string(L.ERR_ALIAS).decode() == "input and output overlap"
    # the 16-bit counterpart (a copy): shapes as for the other 16-bit calls, in place is a no-op,
    # a partial overlap is refused
    assert lib.marian_hip_int16_prepare_b_quantized_transposed(buf, buf + 256, 64, 8, None) == L.ERR_ALIAS
    assert lib.marian_hip_int16_prepare_b_quantized_transposed(buf, buf, 64, 8, None) == L.OK
    assert lib.marian_hip_int16_prepare_b_quantized_transposed(buf, buf + 4096, 48, 8, None) == L.ERR_SHAPE
    assert lib.marian_hip_int16_prepare_b_quantized_transposed(buf, buf + 4096, 64, 12, None) == L.ERR_SHAPE
    assert lib.marian_hip_int16_prepare_b_quantized_transposed(None, buf, 64, 8, None) == L.ERR_NULL
    with pytest.raises(L.MarianHipError):
        L.check(L.ERR_SHAPE, "test")


def test_position_signal_made_on_the_host_equals_the_checker():
    """marian_hip_sinusoidal_position_embeddings makes no HIP call: it runs here, and its rows are
    the checker's bit for bit (the same float expressions through the same C library)."""
    import numpy as np
    from oracle import decode_ops as chk
    chk.lib()
    ops = load("ops")
    for words, d, start in ((1, 1024, 0), (1, 1024, 37), (50, 512, 0), (7, 6, 3), (3, 7, 1), (2, 4, 5)):
        got = ops.sinusoidalPositionEmbeddings(words, d, start)
        assert tuple(got.shape) == (words, 1, d)
        assert np.array_equal(got.numpy().reshape(words, d), chk.sinusoidal_position_embeddings(words, d, start)), (words, d, start)


def test_types_match_marian_enum():
    T = load("types")
    # reference src/common/types.h:282,317-323 and src/common/types.cpp:32-34
    assert int(T.Type.intgemm8) == 0x10000 + 1
    assert int(T.Type.intgemm8avx512vnni) == 0x10000 + 1 + 0x2000 + 4096
    assert int(T.Type.float32) == 0x400 + 4
    assert T.isIntgemm(T.Type.intgemm8) and not T.isIntgemm(T.Type.float32)
    assert T.isHardwareSpecific(T.Type.intgemm8avx2) and not T.isHardwareSpecific(T.Type.intgemm8)
    assert T.requiredBytes((512, 2048), T.Type.intgemm8) == 512 * 2048 + 4
    assert T.requiredBytes((512, 2048), T.Type.float32) == 512 * 2048 * 4
