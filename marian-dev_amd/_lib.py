"""ctypes binding of libmarian_hip_int8.so (the C ABI declared in include/marian_hip_int8.h and
include/marian_hip_ops.h).

There is no fallback: if the library has not been built, loading raises.

libmarian_hip_int8_tuning.so is the same code built with -DMARIAN_HIP_TUNING
(include/marian_hip_int8_tuning.h): it adds a process-wide kernel selection override, the kernel
families only measurements select, and in-kernel clocks.  Tests and measurement scripts reach it
through `forced_kernel(which)`; nothing else loads it."""
import contextlib
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmarian_hip_int8.so")
TUNING_LIB_PATH = os.path.join(_HERE, "libmarian_hip_int8_tuning.so")

OK, ERR_NULL, ERR_SHAPE, ERR_ALIGN, ERR_WORKSPACE, ERR_HIP, ERR_RANGE, ERR_STATIC_LIMIT, ERR_ALIAS = range(9)

# name -> (restype, argtypes); the single place the Python side states the ABI
_c = ctypes
_vp, _i64, _f, _i, _sz = _c.c_void_p, _c.c_int64, _c.c_float, _c.c_int, _c.c_size_t
SIGNATURES = {
    "marian_hip_status_string": (_c.c_char_p, [_i]),
    "marian_hip_last_hip_error": (_i, []),
    "marian_hip_int8_abi_version": (_i, []),
    "marian_hip_int8_workspace_bytes": (_sz, []),
    "marian_hip_int8_prepare_a": (_i, [_vp, _vp, _i64, _i64, _vp, _sz, _vp]),
    "marian_hip_int8_prepare_b": (_i, [_vp, _vp, _i64, _i64, _vp, _sz, _vp]),
    "marian_hip_int8_prepare_b_quantized_transposed": (_i, [_vp, _vp, _i64, _i64, _vp]),
    "marian_hip_int8_affine": (_i, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _f, _i, _vp]),
    "marian_hip_int8_affine_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _i64, _vp, _i64, _i64, _i64, _f, _i,
                                        _vp, _sz, _vp]),
    "marian_hip_int8_affine_f32_chained": (_i, [_vp, _vp, _vp, _vp, _vp, _i64, _vp, _i64, _i64, _i64, _f,
                                                _i, _vp, _vp, _vp, _sz, _vp]),
    "marian_hip_int8_affine_f32_grouped": (_i, [_vp, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _f, _i, _vp, _vp, _sz, _vp]),
    "marian_hip_int8_proj_attention": (_i, [_vp, _vp, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _i64, _i64, _vp,
                                            _i64, _f, _vp, _vp, _vp, _vp, _sz, _vp]),
    "marian_hip_int8_affine_f32_static": (_i, [_vp, _vp, _vp, _vp, _i64, _vp, _i64, _i64, _i64, _f, _i, _vp]),
    "marian_hip_int8_affine_shortlist": (_i, [_vp, _vp, _vp, _vp, _i64, _vp, _i64, _i64, _i64,
                                              _f, _i, _vp]),
    "marian_hip_int8_multiply_i32": (_i, [_vp, _vp, _vp, _i64, _vp, _i64, _i64, _i64, _vp]),
    # include/marian_hip_int16.h
    "marian_hip_int16_prepare_a": (_i, [_vp, _vp, _i64, _i64, _vp]),
    "marian_hip_int16_prepare_b": (_i, [_vp, _vp, _i64, _i64, _vp]),
    "marian_hip_int16_prepare_b_quantized_transposed": (_i, [_vp, _vp, _i64, _i64, _vp]),
    "marian_hip_int16_affine": (_i, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _f, _i, _vp]),
    "marian_hip_int16_multiply_i32": (_i, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    # include/marian_hip_ops.h
    "marian_hip_layer_norm": (_i, [_vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _i64, _f, _vp, _vp]),
    "marian_hip_softmax": (_i, [_vp, _vp, _i64, _i64, _vp, _i64, _i64, _vp]),
    "marian_hip_logsoftmax": (_i, [_vp, _vp, _i64, _i64, _vp]),
    "marian_hip_transpose0213": (_i, [_vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "marian_hip_bdot_legacy": (_i, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i, _i, _f, _vp]),
    "marian_hip_nbest": (_i, [_vp, _i64, _i64, _i64, _vp, _vp, _vp]),
    "marian_hip_nbest_beams_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64]),
    "marian_hip_nbest_beams_workspace_init": (_i, [_vp, _sz, _vp]),
    "marian_hip_nbest_beams": (_i, [_vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _sz, _vp]),
    "marian_hip_logsoftmax_nbest_beams": (_i, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _sz, _vp]),
    "marian_hip_embed": (_i, [_vp, _vp, _i64, _i64, _i64, _f, _vp, _i64, _i64, _vp, _vp, _vp]),
    "marian_hip_sinusoidal_position_embeddings": (_i, [_vp, _i64, _i64, _i64]),
    "marian_hip_attention_ancestors": (_i, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _f, _vp, _vp, _vp, _vp, _vp]),
    "marian_hip_ancestors_advance": (_i, [_vp, _vp, _i64, _i64, _i64, _vp, _vp]),
    "marian_hip_select_state": (_i, [_vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _vp]),
    "marian_hip_fill": (_i, [_vp, _i64, _i, _c.c_uint64, _vp]),
    "marian_hip_attention": (_i, [_vp, _vp, _vp, _vp, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _i64,
                                  _f, _vp, _vp, _vp, _vp]),
    "marian_hip_attention_cached": (_i, [_vp, _vp, _vp, _vp, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _i64, _i64,
                                         _f, _vp, _vp, _vp, _vp]),
}

# include/marian_hip_int8_tuning.h (tuning build only)
TUNING_SIGNATURES = {
    "marian_hip_int8_set_kernel": (_i, [_i]),
    "marian_hip_int8_debug_profile": (None, [_vp]),
    "marian_hip_probe_stream": (_i, [_vp, _sz, _vp, _sz, _i, _i, _i, _i, _vp]),
    "marian_hip_probe_mfma": (_i, [_vp, _i, _i, _vp, _vp, _vp]),
    "marian_hip_probe_mix": (_i, [_vp, _sz, _sz, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "marian_hip_nbest_set_fenced": (_i, [_i]),
}

ABSMAX_SLOTS = 2048   # MARIAN_HIP_ABSMAX_SLOTS
STATIC_MAX_ELEMS = 16 * 1024 * 1024   # MARIAN_HIP_STATIC_MAX_ELEMS

_lib = None
_tuning = None
_active = None   # the tuning build while a forced_kernel() block runs, else None


class MarianHipError(RuntimeError):
    """Raised where the C++ wrappers would ABORT (reference src/common/logging.h:100-116)."""

    def __init__(self, status, what):
        self.status = status
        super().__init__(what)


def build(verbose=False):
    """Compile the HIP libraries for gfx950 with hipcc (always recompiles)."""
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), "-B", "-j4"]
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or out.returncode != 0:
        print(out.stdout)
    if out.returncode != 0:
        raise RuntimeError("hipcc build of libmarian_hip_int8.so failed")
    return LIB_PATH


def _load(path, signatures):
    if not os.path.exists(path):
        raise MarianHipError(
            -1, "{} is not built ({}); run __graft_entry__.build() or "
            "`make -C marian-dev_amd/csrc`. There is no CPU fallback.".format(os.path.basename(path), path))
    # torch must load first: it ships its own libamdhip64.so.7 / HSA runtime, and a process
    # can hold only one of them - loading ours first would pull in the system copy and
    # leave torch's runtime without a device (hipErrorNoDevice on the first launch)
    import torch  # noqa: F401
    L = ctypes.CDLL(path)
    for name, (res, args) in signatures.items():
        f = getattr(L, name)  # AttributeError if a declared symbol is not exported
        f.restype = res
        f.argtypes = args
    return L


def lib():
    """The shipped library (inside a forced_kernel() block: the tuning build)."""
    global _lib
    if _active is not None:
        return _active
    if _lib is None:
        _lib = _load(LIB_PATH, SIGNATURES)
    return _lib


def tuning_lib():
    global _tuning
    if _tuning is None:
        _tuning = _load(TUNING_LIB_PATH, dict(SIGNATURES, **TUNING_SIGNATURES))
    return _tuning


@contextlib.contextmanager
def forced_kernel(which):
    """Runs the block on the tuning build with kernel family `which` pinned (0: the tuning build's
    automatic selection); lib() returns the tuning build inside the block."""
    global _active
    T = tuning_lib()
    outer = _active
    _active = T
    prev = T.marian_hip_int8_set_kernel(int(which))
    try:
        yield T
    finally:
        T.marian_hip_int8_set_kernel(prev)
        _active = outer


def check(status, where):
    if status != OK:
        L = lib()
        msg = L.marian_hip_status_string(status).decode()
        if status == ERR_HIP:
            msg += " (hipError_t {})".format(L.marian_hip_last_hip_error())
        raise MarianHipError(status, "{}: {}".format(where, msg))
