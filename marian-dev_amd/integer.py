"""Host mirror of Marian's intgemm operator glue, running on the HIP library.

Mirrors, name for name:
  reference src/tensors/cpu/intgemm_interface.h   prepareA, affineOrDotTyped, affineOrDot
  reference src/tensors/cpu/integer_common.h      cols, rows, getQuantMult, computeQuantMult
  reference src/graph/expression_operators.cpp    dot (:554-619), affine (:647-718),
                                                  affineWithReluDropout (:721-731)
  reference src/tensors/cpu/expression_graph_packable.h:153-253  (prepareB = offline packer)

Tensors are torch tensors on the GPU (device memory and streams only); every arithmetic step
is a call into the C ABI.  Quantized tensors are `QTensor`: a flat int8 buffer holding the
payload plus the fp32 quantMult tail, with Marian's logical shape and element type.
"""
import weakref

import numpy as np
import torch

from . import _lib, layout
from .types import Type, elements, isFloat, isHardwareSpecific, isIntgemm, requiredBytes, sizeOf

MarianRuntimeError = _lib.MarianHipError


def _abort_if(cond, msg, *args):
    if cond:
        raise MarianRuntimeError(-2, msg.format(*args))


def _align256(n):
    return (n + 255) // 256 * 256


class QTensor:
    """An intgemm-typed tensor: Marian allocates requiredBytes(shape, type) rounded up to 256
    bytes (reference src/tensors/allocator.h:86,178-181); `shape` is the logical shape
    ([.., K] for activations, [K, N] for weights whose payload is the transposed [N, K])."""

    def __init__(self, data, shape, type_, prepared=False):
        self.data = data
        self.shape = tuple(int(d) for d in shape)
        self.type = type_
        # 8-bit weights only: the payload is in the order the GEMM kernels read (written by prepareB
        # or prepareAndTransposeB), not in the file order [N, K].  The reference tells the two apart
        # by type (intgemm8 against intgemm8avx2 ...: src/common/types.h); its enum has no GPU
        # variant, so this mirror keeps a flag.
        self.prepared = prepared

    @staticmethod
    def empty(shape, type_, device, prepared=False):
        nbytes = _align256(requiredBytes(shape, type_))
        # (the bytes past elements + 4 are allocation padding and are never read)
        return QTensor(torch.empty(nbytes, dtype=torch.int8, device=device), shape, type_, prepared)

    @staticmethod
    def from_numpy(flat_int8, shape, type_, device):
        """Upload payload+tail bytes (e.g. a Type::intgemm8 item of a .bin file) verbatim: for
        8-bit weights that is the file order, which prepareAndTransposeB turns into a usable B."""
        q = QTensor.empty(shape, type_, device)
        src = torch.from_numpy(np.ascontiguousarray(flat_int8).view(np.int8))
        n = min(src.numel(), q.data.numel())
        q.data[:n].copy_(src[:n])
        return q

    def value_type(self):
        return self.type

    def elements(self):
        return elements(self.shape)

    def payload(self):
        return self.data[: self.elements()]

    def numpy(self):
        """payload + tail as host bytes (requiredBytes: elements * element size + 4)."""
        return self.data[: requiredBytes(self.shape, self.type)].cpu().numpy()

    def file_bytes(self):
        """payload + tail as a model file holds them: prepared 8-bit weights are put back into
        plain rows [N, K] (on the host); everything else is numpy()."""
        raw = self.numpy()
        if self.prepared and sizeOf(self.type) == 1:
            K, N = self.shape
            return layout.from_prepared(raw, K, N).view(np.int8)
        return raw

    def data_ptr(self):
        return self.data.data_ptr()


def cols(t):
    """reference src/tensors/cpu/integer_common.h:48"""
    return int(t.shape[-1])


def rows(t):
    """reference src/tensors/cpu/integer_common.h:49"""
    return elements(t.shape) // cols(t)


def getQuantMult(q):
    """reference src/tensors/cpu/integer_common.h:101-111 (device read; for tests and tools)."""
    _abort_if(not isIntgemm(q.type), "getQuantMult does not work for type {}", q.type)
    n = q.elements() * sizeOf(q.type)
    return float(q.data[n:n + 4].cpu().numpy().view(np.float32)[0])


class Backend:
    """Per-device state the path needs: a stream and the abs-max workspace, the counterpart of
    gpu::Backend (reference src/tensors/gpu/backend.h:23-110) reduced to this path.  The stream is
    torch's current stream of the calling thread, and every stream has a workspace of its own:
    worker threads that share a device (reference src/translator/translator.h:158-164) each run on
    their own stream and never meet in a workspace."""

    _instances = {}

    def __init__(self, device):
        self.device = torch.device(device)
        self.workspace_bytes = int(self.lib.marian_hip_int8_workspace_bytes())
        self._workspaces = {}   # stream handle -> workspace (kept for good: a graph may have recorded it)
        # float32 weights are quantized on first use and remembered when this is Type.intgemm8:
        # the counterpart of getGemmType() (reference src/tensors/backend.h:36-40) with the
        # memoized packing of src/graph/expression_operators.cpp:564-598 (its FBGEMM branch
        # packs a memoized float B the same way)
        self.gemmType = None
        self._memo = {}

    @property
    def lib(self):
        return _lib.lib()

    @property
    def workspace(self):
        """The workspace of the current stream (calls on one stream run one after the other and
        share it; calls on different streams may overlap and must not)."""
        key = self.stream()
        ws = self._workspaces.get(key)
        if ws is None:
            ws = self._workspaces.setdefault(key, torch.empty(self.workspace_bytes, dtype=torch.uint8, device=self.device))
        return ws

    def setGemmType(self, type_):
        _abort_if(type_ not in (None, Type.intgemm8), "Unsupported type {} for Intgemm type??", type_)
        self.gemmType = type_

    @staticmethod
    def _memo_key(w):
        return (w.data_ptr(), tuple(w.shape), w._version)

    def memoizedPrepareB(self, w):
        """prepareB of a float32 parameter, once per parameter and version.  The reference
        memoizes per parameter node (src/graph/expression_operators.cpp:564-598); here an entry
        belongs to one tensor object: it holds a weak reference to it, a hit requires that very
        object to be alive and to be the one asked for (an address can be handed to a new tensor of
        the same shape once the old one is freed), and the entry goes when the tensor does."""
        key = self._memo_key(w)
        hit = self._memo.get(key)
        if hit is not None and hit[0]() is w:
            return hit[1]
        q = prepareB(w)
        memo = self._memo
        for k in [k for k, (ref, _) in memo.items() if ref() is None or ref() is w]:
            del memo[k]   # dead owners, and earlier versions of this parameter

        def evict(_ref, key=key, memo=memo):
            ent = memo.get(key)
            if ent is not None and ent[0] is _ref:
                del memo[key]
        memo[key] = (weakref.ref(w, evict), q)
        return q

    @classmethod
    def get(cls, device):
        device = torch.device(device)
        key = (device.type, device.index if device.index is not None else torch.cuda.current_device())
        if key not in cls._instances:
            cls._instances[key] = Backend(device)
        return cls._instances[key]

    def stream(self):
        return torch.cuda.current_stream(self.device).cuda_stream

    def synchronize(self):
        torch.cuda.current_stream(self.device).synchronize()


def _backend_of(t):
    dev = t.device if isinstance(t, torch.Tensor) else t.data.device
    _abort_if(dev.type != "cuda", "the HIP int8 backend needs device tensors, got {}", dev)
    return Backend.get(dev)


def prepareA(a, type_=Type.intgemm8):
    """reference src/tensors/cpu/intgemm_interface.h:17-32 for vtype = intgemm8 (abs-max quantMult)
    or intgemm16 (quantMult 1024, src/tensors/cpu/integer_common.h:174-175)."""
    _abort_if(a.dtype != torch.float32, "Intgemm expects type of A to be float32 not {}", a.dtype)
    _abort_if(type_ not in (Type.intgemm8, Type.intgemm16), "Unsupported type {} for Intgemm type??", type_)
    a = a.contiguous()
    be = _backend_of(a)
    out = QTensor.empty(a.shape, type_, a.device)
    K = cols(a)
    M = rows(a) if a.numel() else 0
    if type_ == Type.intgemm16:
        _lib.check(be.lib.marian_hip_int16_prepare_a(a.data_ptr(), out.data_ptr(), M, K, be.stream()), "prepareA")
        return out
    st = be.lib.marian_hip_int8_prepare_a(a.data_ptr(), out.data_ptr(), M, K,
                                          be.workspace.data_ptr(), be.workspace_bytes, be.stream())
    _lib.check(st, "prepareA")
    return out


def prepareB(w, type_=Type.intgemm8):
    """Offline weight quantizer, reference src/tensors/cpu/expression_graph_packable.h:153-253
    (intgemm8 branch): fp32 W [K, N] -> Type::intgemm8 tensor of shape [K, N] whose payload is
    the quantized transpose."""
    _abort_if(type_ not in (Type.intgemm8, Type.intgemm16), "Type {} is not supported", type_)
    _abort_if(w.dtype != torch.float32 or w.dim() != 2, "prepareB expects a float32 matrix, got {}", w.dtype)
    w = w.contiguous()
    be = _backend_of(w)
    K, N = w.shape
    out = QTensor.empty((K, N), type_, w.device, prepared=True)
    if type_ == Type.intgemm16:   # the 16-bit branch of the packer (:203-235): quantMult 1024
        _lib.check(be.lib.marian_hip_int16_prepare_b(w.data_ptr(), out.data_ptr(), K, N, be.stream()), "prepareB")
        return out
    st = be.lib.marian_hip_int8_prepare_b(w.data_ptr(), out.data_ptr(), K, N,
                                          be.workspace.data_ptr(), be.workspace_bytes, be.stream())
    _lib.check(st, "prepareB")
    return out


def prepareAndTransposeB(q):
    """A quantized weight item as a model file holds it (plain rows [N, K] + quantMult) -> the
    order the kernels read; reference prepareAndTransposeB, src/tensors/cpu/integer_common.h:189-216
    (there: the tiling of the CPU the process runs on)."""
    _abort_if(not isinstance(q, QTensor) or not isIntgemm(q.type) or isHardwareSpecific(q.type) or len(q.shape) != 2,
              "prepareAndTransposeB expects a hardware-agnostic intgemm matrix, got {}", getattr(q, "type", type(q)))
    _abort_if(q.prepared, "the weights are prepared already (type {})", q.type)
    be = _backend_of(q)
    K, N = q.shape
    out = QTensor.empty((K, N), q.type, q.data.device, prepared=True)
    fn = be.lib.marian_hip_int16_prepare_b_quantized_transposed if sizeOf(q.type) == 2 else \
        be.lib.marian_hip_int8_prepare_b_quantized_transposed
    _lib.check(fn(q.data_ptr(), out.data_ptr(), K, N, be.stream()), "prepareAndTransposeB")
    return out


def _check_weights(bQuant):
    _abort_if(not isinstance(bQuant, QTensor) or not isIntgemm(bQuant.type),
              "Intgemm expects type of B to be a variant of intgemm not {}", getattr(bQuant, "type", type(bQuant)))
    _abort_if(isHardwareSpecific(bQuant.type) or sizeOf(bQuant.type) not in (1, 2),
              "Unsupported type {} for Intgemm type??", bQuant.type)
    _abort_if(sizeOf(bQuant.type) == 1 and not bQuant.prepared,
              "B of type {} is in file order: it has to go through prepareAndTransposeB first", bQuant.type)


def affineOrDot(a, bQuant, bias=None, transA=False, transB=False, scale=1.0, relu=False,
                shortlist=None):
    """reference src/tensors/cpu/intgemm_interface.h:46-99,102-128.

    a: float32 activations; bQuant: QTensor of type intgemm8 with logical shape [K, N].
    transB is ignored like in the reference (:47).  `relu` fuses the in-place ReLU node the
    reference appends (src/graph/expression_operators.cpp:721-731).  `shortlist`: optional
    uint32 device tensor of sorted unique output ids (multiple of 8 many)."""
    _abort_if(not isinstance(a, torch.Tensor) or not a.dtype.is_floating_point or a.dtype != torch.float32,
              "Intgemm expects type of A to be float32 not {}", getattr(a, "dtype", type(a)))
    _check_weights(bQuant)
    if transA:
        a = a.transpose(-1, -2)
    if sizeOf(bQuant.type) == 2:   # Type::intgemm16: the two nodes one after the other
        _abort_if(shortlist is not None, "the 16-bit path has no shortlist form (type {})", bQuant.type)
        return multiply(prepareA(a, Type.intgemm16), bQuant, bias, scale=scale, relu=relu)
    out, _ = affine_f32(a, bQuant, bias, scale=scale, relu=relu, shortlist=shortlist)
    return out


class AbsMax:
    """Values whose maximum is max|x| of the tensor they were produced with (2048 floats on the
    device): handed from the call that writes a tensor to the affine call that reads it, in place
    of the abs-max pass of prepareA (reference src/tensors/cpu/intgemm_interface.h:23)."""

    def __init__(self, device):
        self.data = torch.empty(_lib.ABSMAX_SLOTS, dtype=torch.float32, device=device)

    def data_ptr(self):
        return self.data.data_ptr()


def affine_f32(a, bQuant, bias=None, scale=1.0, relu=False, shortlist=None, absmax=None,
               want_absmax=False):
    """prepareA node + multiply node through the single C-ABI call marian_hip_int8_affine_f32
    (one fused kernel for small activations).  Returns (out, aQuant): aQuant is what the
    prepareA node would have produced.  absmax: the AbsMax left by the call that produced `a`;
    want_absmax: also return an AbsMax of `out` as a third value."""
    _check_weights(bQuant)
    a = a.contiguous()
    be = _backend_of(a)
    aQuant = QTensor.empty(a.shape, Type.intgemm8, a.device)
    K, N = cols(a), cols(bQuant)
    _abort_if(rows(bQuant) != K, "Matrix product requires inner dimensions to match: {} vs {}", K, rows(bQuant))
    M = rows(a) if a.numel() else 0
    n_out = N if shortlist is None else int(shortlist.numel())
    out = torch.empty(tuple(a.shape[:-1]) + (n_out,), dtype=torch.float32, device=a.device)
    bias_ptr = None
    if bias is not None:
        _abort_if(bias.dtype != torch.float32 or bias.numel() != N, "bias must be float32 [1, {}]", N)
        bias = bias.contiguous()
        bias_ptr = bias.data_ptr()
    if shortlist is not None:
        _abort_if(shortlist.dtype not in (torch.int32, torch.uint32), "shortlist ids must be uint32, got {}", shortlist.dtype)
    idx_ptr = None if shortlist is None else shortlist.data_ptr()
    n_idx = n_out if shortlist is not None else 0
    if absmax is None and not want_absmax:
        st = be.lib.marian_hip_int8_affine_f32(
            a.data_ptr(), aQuant.data_ptr(), bQuant.data_ptr(), bias_ptr, idx_ptr, n_idx,
            out.data_ptr(), M, K, N, scale, int(relu), be.workspace.data_ptr(), be.workspace_bytes,
            be.stream())
        _lib.check(st, "affineOrDot")
        return out, aQuant
    omax = AbsMax(a.device) if want_absmax else None
    st = be.lib.marian_hip_int8_affine_f32_chained(
        a.data_ptr(), aQuant.data_ptr(), bQuant.data_ptr(), bias_ptr, idx_ptr, n_idx,
        out.data_ptr(), M, K, N, scale, int(relu), None if absmax is None else absmax.data_ptr(),
        None if omax is None else omax.data_ptr(), be.workspace.data_ptr(), be.workspace_bytes,
        be.stream())
    _lib.check(st, "affineOrDot")
    return (out, aQuant, omax) if want_absmax else (out, aQuant)


def affine_f32_grouped(a, weights, scale=1.0, relu=False, absmax=None):
    """One activation tensor through several weight matrices in one call
    (marian_hip_int8_affine_f32_grouped): the self-attention projections Wq, Wk, Wv of reference
    src/models/transformer.h:290-325 read the same input.  weights: list of (bQuant, bias or None).
    Returns ([out, ...], aQuant); each out equals affine_f32(a, bQuant, bias)[0] bit for bit."""
    import ctypes
    for bQuant, _ in weights:
        _check_weights(bQuant)
    a = a.contiguous()
    be = _backend_of(a)
    K = cols(a)
    M = rows(a) if a.numel() else 0
    n = len(weights)
    _abort_if(n < 1 or n > 4, "between one and four weight matrices per call, got {}", n)
    aQuant = QTensor.empty(a.shape, Type.intgemm8, a.device)
    outs, keep = [], []
    Bq_arr, bias_arr, out_arr, N_arr = ((ctypes.c_void_p * n)(), (ctypes.c_void_p * n)(), (ctypes.c_void_p * n)(),
                                        (ctypes.c_int64 * n)())
    for g, (bQuant, bias) in enumerate(weights):
        _check_weights(bQuant)
        _abort_if(sizeOf(bQuant.type) != 1, "Unsupported type {} for Intgemm type??", bQuant.type)
        _abort_if(rows(bQuant) != K, "Matrix product requires inner dimensions to match: {} vs {}", K, rows(bQuant))
        N = cols(bQuant)
        if bias is not None:
            _abort_if(bias.dtype != torch.float32 or bias.numel() != N, "bias must be float32 [1, {}]", N)
            bias = bias.contiguous()
            keep.append(bias)
        out = torch.empty(tuple(a.shape[:-1]) + (N,), dtype=torch.float32, device=a.device)
        outs.append(out)
        Bq_arr[g], bias_arr[g], out_arr[g], N_arr[g] = (bQuant.data_ptr(), None if bias is None else bias.data_ptr(),
                                                        out.data_ptr(), N)
    st = be.lib.marian_hip_int8_affine_f32_grouped(
        a.data_ptr(), aQuant.data_ptr(), n, Bq_arr, bias_arr, out_arr, N_arr, M, K, scale, int(relu),
        None if absmax is None else absmax.data_ptr(), be.workspace.data_ptr(), be.workspace_bytes, be.stream())
    _lib.check(st, "affineOrDot")
    return outs, aQuant


def multiply(aQuant, bQuant, bias=None, scale=1.0, relu=False, shortlist=None):
    """The multiply node of reference src/tensors/cpu/intgemm_interface.h:60-94."""
    _check_weights(bQuant)
    be = _backend_of(aQuant)
    K, N = cols(aQuant), cols(bQuant)
    _abort_if(rows(bQuant) != K, "Matrix product requires inner dimensions to match: {} vs {}", K, rows(bQuant))
    M = rows(aQuant) if aQuant.elements() else 0
    n_out = N if shortlist is None else int(shortlist.numel())
    out = torch.empty(aQuant.shape[:-1] + (n_out,), dtype=torch.float32, device=aQuant.data.device)
    bias_ptr = None
    if bias is not None:
        _abort_if(bias.dtype != torch.float32 or bias.numel() != N, "bias must be float32 [1, {}]", N)
        bias = bias.contiguous()
        bias_ptr = bias.data_ptr()
    _abort_if(sizeOf(aQuant.type) != sizeOf(bQuant.type), "Intgemm operands of different widths: {} and {}",
              aQuant.type, bQuant.type)
    if sizeOf(bQuant.type) == 2:
        _abort_if(shortlist is not None, "the 16-bit path has no shortlist form (type {})", bQuant.type)
        st = be.lib.marian_hip_int16_affine(aQuant.data_ptr(), bQuant.data_ptr(), bias_ptr, out.data_ptr(), M, K, N,
                                            scale, int(relu), be.stream())
    elif shortlist is None:
        st = be.lib.marian_hip_int8_affine(aQuant.data_ptr(), bQuant.data_ptr(), bias_ptr,
                                           out.data_ptr(), M, K, N, scale, int(relu), be.stream())
    else:
        _abort_if(shortlist.dtype not in (torch.int32, torch.uint32), "shortlist ids must be uint32, got {}", shortlist.dtype)
        st = be.lib.marian_hip_int8_affine_shortlist(aQuant.data_ptr(), bQuant.data_ptr(), bias_ptr,
                                                     shortlist.data_ptr(), n_out, out.data_ptr(),
                                                     M, K, N, scale, int(relu), be.stream())
    _lib.check(st, "affineOrDot")
    return out


def multiply_i32(aQuant, bQuant, shortlist=None):
    """int32 accumulators of the multiply (what Kernels8::Multiply hands to its callback)."""
    _check_weights(bQuant)
    be = _backend_of(aQuant)
    K, N = cols(aQuant), cols(bQuant)
    M = rows(aQuant) if aQuant.elements() else 0
    n_out = N if shortlist is None else int(shortlist.numel())
    acc = torch.empty(aQuant.shape[:-1] + (n_out,), dtype=torch.int32, device=aQuant.data.device)
    if sizeOf(bQuant.type) == 2:
        _abort_if(shortlist is not None, "the 16-bit path has no shortlist form (type {})", bQuant.type)
        _lib.check(be.lib.marian_hip_int16_multiply_i32(aQuant.data_ptr(), bQuant.data_ptr(), acc.data_ptr(), M, K, N,
                                                        be.stream()), "multiply_i32")
        return acc
    st = be.lib.marian_hip_int8_multiply_i32(aQuant.data_ptr(), bQuant.data_ptr(),
                                             None if shortlist is None else shortlist.data_ptr(),
                                             n_out if shortlist is not None else 0, acc.data_ptr(),
                                             M, K, N, be.stream())
    _lib.check(st, "multiply_i32")
    return acc


# ---- graph-operator surface (reference src/graph/expression_operators.cpp) --------------------

def _maybe_quantize_b(a, b):
    """float32 B with the backend's gemm type set to intgemm8: quantize on first use, remembered"""
    if isinstance(b, torch.Tensor) and b.dtype == torch.float32 and b.dim() == 2:
        be = _backend_of(a)
        if be.gemmType == Type.intgemm8:
            return be.memoizedPrepareB(b)
    return b


def _float_b_unsupported(b):
    raise MarianRuntimeError(
        -2, "GPU-based GEMM only supports float types in the reference; this backend implements "
        "the intgemm8 weight path only, got B of type {}".format(getattr(b, "dtype", type(b))))


def dot(a, b, transA=False, transB=False, scale=1.0):
    """reference src/graph/expression_operators.cpp:554-619: isIntgemm(b) selects the int8 path."""
    b = _maybe_quantize_b(a, b)
    if isinstance(b, QTensor) and isIntgemm(b.type):
        return affineOrDot(a, b, None, transA, transB, scale)
    _float_b_unsupported(b)


def affine(a, b, bias, transA=False, transB=False, scale=1.0):
    """reference src/graph/expression_operators.cpp:647-718."""
    b = _maybe_quantize_b(a, b)
    if isinstance(b, QTensor) and isIntgemm(b.type):
        return affineOrDot(a, b, bias, transA, transB, scale)
    _float_b_unsupported(b)


def affineWithReluDropout(x, W, bias, dropProb=0.0):
    """reference src/graph/expression_operators.cpp:721-731 at inference (dropProb == 0): the
    reference runs affine() and then an in-place ReLU node; here the ReLU is the GEMM epilogue."""
    _abort_if(dropProb != 0.0, "dropout is a training feature; inference path expects dropProb == 0, got {}", dropProb)
    W = _maybe_quantize_b(x, W)
    if isinstance(W, QTensor) and isIntgemm(W.type):
        return affineOrDot(x, W, bias, False, False, 1.0, relu=True)
    _float_b_unsupported(W)
