"""Host mirror of the float operators between the int8 GEMMs of a transformer decode step,
running on the HIP library (include/marian_hip_ops.h).

Mirrors, name for name:
  reference src/graph/expression_operators.cpp:901-913   layerNorm(x, gamma, beta, eps = 1e-9)
  reference src/graph/expression_operators.cpp           softmax(a), logsoftmax(a),
                                                         transpose(a, {0, 2, 1, 3}),
                                                         bdot_legacy(a, b, transA, transB, scalar)
  reference src/models/transformer.h:145-170             SplitHeads, JoinHeads
  reference src/graph/expression_operators.cpp           rows(a, indices)
  reference src/graph/node_initializers.cpp:224-226      sinusoidalPositionEmbeddings(start)
  reference src/models/transformer.h:93,110-117          scaledEmbeddings: sqrt(dimEmb) * rows(E, ids) + signal

Tensors are torch float32 tensors on the GPU (device memory and streams only); every arithmetic
step is a call into the C ABI.  There is no CPU fallback.
"""
import torch

from . import _lib
from .integer import AbsMax, _abort_if, _backend_of


def _f32c(x, what):
    _abort_if(x.dtype != torch.float32, "{} expects float32, got {}", what, x.dtype)
    return x.contiguous()


def layerNorm(x, gamma, beta=None, eps=1e-9, add=None, want_absmax=False):
    """reference src/graph/expression_operators.cpp:901-913; `add` fuses the skip connection in
    front of it (out = layerNorm(x + add)).  want_absmax: also return the AbsMax of the output
    for the affine calls that read it."""
    x = _f32c(x, "layerNorm")
    be = _backend_of(x)
    cols = x.shape[-1]
    rows = x.numel() // cols if x.numel() else 0
    gamma = _f32c(gamma, "layerNorm").reshape(-1)
    _abort_if(gamma.numel() not in (1, cols), "layerNorm: gamma must have {} or 1 values", cols)
    if beta is not None:
        beta = _f32c(beta, "layerNorm").reshape(-1)
        _abort_if(beta.numel() not in (1, cols), "layerNorm: beta must have {} or 1 values", cols)
    if add is not None:
        add = _f32c(add, "layerNorm")
        _abort_if(tuple(add.shape) != tuple(x.shape), "layerNorm: skip input shape {} vs {}", tuple(add.shape), tuple(x.shape))
    out = torch.empty_like(x)
    omax = AbsMax(x.device) if want_absmax else None
    st = be.lib.marian_hip_layer_norm(
        x.data_ptr(), None if add is None else add.data_ptr(), gamma.data_ptr(), gamma.numel(),
        None if beta is None else beta.data_ptr(), 0 if beta is None else beta.numel(),
        out.data_ptr(), rows, cols, eps, None if omax is None else omax.data_ptr(), be.stream())
    _lib.check(st, "layerNorm")
    return (out, omax) if want_absmax else out


def scaledEmbeddings(E, ids, scale=1.0, signal=None, rowsPerSignal=1, want_absmax=False, out=None):
    """scale * E[ids] (+ signal): the embedding step in front of the first layer (reference
    src/layers/embedding.cpp:161-168 and src/models/transformer.h:93,117) as one launch.  E
    [vocab, dimEmb]; ids: integer tensor on the device, any shape; signal: None or [n, dimEmb],
    output row r taking signal row (r / rowsPerSignal) % n.  Returns [*ids.shape, dimEmb] (`out`
    when given: a contiguous float32 tensor of that many values that does not overlap E)."""
    E = _f32c(E, "scaledEmbeddings")
    be = _backend_of(E)
    _abort_if(E.dim() != 2, "scaledEmbeddings: the table has to be a matrix, got shape {}", tuple(E.shape))
    _abort_if(ids.dtype not in (torch.int32, torch.int64, torch.uint32) or ids.device != E.device,
              "scaledEmbeddings: indices have to be an integer tensor on the table's device")
    vocab, dimEmb = E.shape
    words = ids.contiguous()
    if words.dtype == torch.int64:   # the reference's IndexType has 32 bits
        words = words.to(torch.int32)
    n_signals = 0
    if signal is not None:
        signal = _f32c(signal, "scaledEmbeddings").reshape(-1, dimEmb)
        n_signals = signal.shape[0]
    if out is None:
        out = torch.empty(tuple(ids.shape) + (dimEmb,), dtype=torch.float32, device=E.device)
    else:
        _abort_if(out.dtype != torch.float32 or not out.is_contiguous() or out.device != E.device or
                  out.numel() != ids.numel() * dimEmb, "scaledEmbeddings: out has to be a contiguous float32 "
                  "tensor of {} x {} values on the table's device", ids.numel(), dimEmb)
        lo, hi = out.data_ptr(), out.data_ptr() + 4 * out.numel()
        _abort_if(lo < E.data_ptr() + 4 * E.numel() and E.data_ptr() < hi, "scaledEmbeddings: out overlaps the table")
    omax = AbsMax(E.device) if want_absmax else None
    st = be.lib.marian_hip_embed(E.data_ptr(), words.data_ptr(), words.numel(), vocab, dimEmb, float(scale),
                                 None if signal is None else signal.data_ptr(), rowsPerSignal, n_signals,
                                 out.data_ptr(), None if omax is None else omax.data_ptr(), be.stream())
    _lib.check(st, "scaledEmbeddings")
    return (out, omax) if want_absmax else out


def rows(a, indices, out=None):
    """reference rows(a, indices) (CopyRows, src/tensors/cpu/tensor_operators.cpp:577-603); also
    the selection of the surviving hypotheses' decoder states between two steps of the beam search
    (reference src/rnn/types.h:22-42)"""
    return scaledEmbeddings(a, indices.reshape(-1), out=out)


def selectState(state, indices, out, used=None):
    """The decoder state of the surviving hypotheses (reference src/models/states.h:87-107,
    src/rnn/types.h:22-42): out[r, s, :used] = state[indices[r], s, :used] for a state [entries,
    segments, capacity] whose segments (the cached positions of a head) are in use up to `used`
    values (None: entirely); out [len(indices), segments, capacity] is a tensor of its own."""
    _abort_if(state.dtype != torch.float32 or out.dtype != torch.float32 or state.dim() != 3 or out.dim() != 3 or
              not state.is_contiguous() or not out.is_contiguous(), "selectState expects contiguous float32 "
              "tensors [entries, segments, capacity], got {} and {}", tuple(state.shape), tuple(out.shape))
    be = _backend_of(state)
    entries, segments, cap = state.shape
    _abort_if(tuple(out.shape) != (indices.numel(), segments, cap), "selectState: out has shape {}, not {}",
              tuple(out.shape), (indices.numel(), segments, cap))
    _abort_if(indices.dtype not in (torch.int32, torch.int64, torch.uint32) or indices.device != state.device,
              "selectState: indices have to be an integer tensor on the state's device")
    ids = indices.contiguous()
    if ids.dtype == torch.int64:
        ids = ids.to(torch.int32)
    st = be.lib.marian_hip_select_state(state.data_ptr(), ids.data_ptr(), ids.numel(), entries, segments, cap,
                                        cap if used is None else int(used), out.data_ptr(), be.stream())
    _lib.check(st, "selectState")
    return out


def sinusoidalPositionEmbeddings(dimWords, dimEmb, start=0, device=None):
    """The constant [dimWords, 1, dimEmb] of reference src/models/transformer.h:110-111, made on the
    host by the library (reference src/tensors/cpu/tensor_operators.cpp:1733-1746) and copied to
    `device` when one is given."""
    out = torch.empty((dimWords, 1, dimEmb), dtype=torch.float32)
    _lib.check(_lib.lib().marian_hip_sinusoidal_position_embeddings(out.data_ptr(), dimWords, dimEmb, start),
               "sinusoidalPositionEmbeddings")
    return out if device is None else out.to(device)


def softmax(a, mask=None, rowsPerMask=1):
    """softmax over the last axis; `mask` [n, cols] fuses the `a + mask` in front of it, row r of
    `a` taking mask row (r / rowsPerMask) % n (reference src/models/transformer.h:264,772-774)."""
    a = _f32c(a, "softmax")
    be = _backend_of(a)
    cols = a.shape[-1]
    rows = a.numel() // cols if a.numel() else 0
    n_masks = 0
    if mask is not None:
        mask = _f32c(mask, "softmax").reshape(-1, cols)
        n_masks = mask.shape[0]
    out = torch.empty_like(a)
    st = be.lib.marian_hip_softmax(a.data_ptr(), None if mask is None else mask.data_ptr(), n_masks,
                                   rowsPerMask, out.data_ptr(), rows, cols, be.stream())
    _lib.check(st, "softmax")
    return out


def logsoftmax(a):
    a = _f32c(a, "logsoftmax")
    be = _backend_of(a)
    cols = a.shape[-1]
    rows = a.numel() // cols if a.numel() else 0
    out = torch.empty_like(a)
    _lib.check(be.lib.marian_hip_logsoftmax(a.data_ptr(), out.data_ptr(), rows, cols, be.stream()),
               "logsoftmax")
    return out


def transpose0213(a):
    """transpose(a, {0, 2, 1, 3}) of a 4-d tensor.  With a middle dimension of 1 (the single
    target position of a decoding step) the transposed tensor has the same memory image, so it
    is returned as a view and no kernel runs."""
    a = _f32c(a, "transpose")
    _abort_if(a.dim() != 4, "transpose0213 expects a 4-d tensor, got {} dimensions", a.dim())
    be = _backend_of(a)
    d0, d1, d2, d3 = a.shape
    if d1 == 1 or d2 == 1:
        return a.reshape(d0, d2, d1, d3)
    out = torch.empty((d0, d2, d1, d3), dtype=torch.float32, device=a.device)
    _lib.check(be.lib.marian_hip_transpose0213(a.data_ptr(), out.data_ptr(), d0, d1, d2, d3, be.stream()),
               "transpose")
    return out


def SplitHeads(input, dimHeads):
    """reference src/models/transformer.h:145-156: [beam, batch, steps, model] ->
    [batch * beam, heads, steps, depth]"""
    dimBeam, dimBatch, dimSteps, dimModel = input.shape
    return transpose0213(input.reshape(dimBatch * dimBeam, dimSteps, dimHeads, dimModel // dimHeads))


def JoinHeads(input, dimBeam=1):
    """reference src/models/transformer.h:158-170"""
    dimBatchBeam, dimHeads, dimSteps, dimDepth = input.shape
    out = transpose0213(input)
    return out.reshape(dimBeam, dimBatchBeam // dimBeam, dimSteps, dimHeads * dimDepth)


def bdot_legacy(a, b, transA=False, transB=False, scalar=1.0):
    """reference src/tensors/cpu/prod.cpp:233-330: batch entry i uses a[i % batchA], b[i % batchB]"""
    a, b = _f32c(a, "bdot"), _f32c(b, "bdot")
    be = _backend_of(a)
    batchA = a.numel() // (a.shape[-1] * a.shape[-2])
    batchB = b.numel() // (b.shape[-1] * b.shape[-2])
    m, k = a.shape[-2], a.shape[-1]
    if transA:
        m, k = k, m
    l, n = b.shape[-2], b.shape[-1]
    if transB:
        l, n = n, l
    _abort_if(l != k, "Matrix product requires inner dimensions to match: {} vs {}", k, l)
    lead = tuple(a.shape[:-2]) if batchA >= batchB else tuple(b.shape[:-2])
    out = torch.empty(lead + (m, n), dtype=torch.float32, device=a.device)
    st = be.lib.marian_hip_bdot_legacy(a.data_ptr(), b.data_ptr(), out.data_ptr(), batchA, batchB,
                                       m, n, k, int(transA), int(transB), scalar, be.stream())
    _lib.check(st, "bdot")
    return out


def Attention(q, k, v, mask=None, rowsPerMask=1, want_absmax=False, kNew=None, vNew=None, kvLen=None):
    """reference src/models/transformer.h:241-280 (inference: no dropout, weights not kept):
    softmax(bdot_legacy(q, k, false, true, 1/sqrt(dk)) + mask) then bdot_legacy(weights, v), in
    one launch.  q: [batch*beam, heads, tgt, dk]; k, v: [batch(*beam), heads, len, dk].
    kNew, vNew [batch*beam*heads, dk]: key and value of the newest position of a decoding step;
    they stand for position len - 1 and are also stored there in k and v (the concatenation onto
    the cached positions, src/models/transformer.h:683-700).
    kvLen: k and v have room for k.shape[-2] positions per entry, of which the first kvLen are in
    use (caches that stay in place from step to step); None: all of them."""
    q = _f32c(q, "Attention")
    _abort_if(k.dtype != torch.float32 or v.dtype != torch.float32, "Attention expects float32, got {}", k.dtype)
    if kNew is None:
        k, v = k.contiguous(), v.contiguous()
    else:
        _abort_if(not (k.is_contiguous() and v.is_contiguous()), "Attention: the key/value cache must be contiguous{}", "")
        kNew, vNew = _f32c(kNew, "Attention"), _f32c(vNew, "Attention")
    be = _backend_of(q)
    dk, m, cap = q.shape[-1], q.shape[-2], k.shape[-2]
    L = cap if kvLen is None else int(kvLen)
    _abort_if(not 0 < L <= cap, "Attention: {} positions in use of {} the cache has room for", L, cap)
    _abort_if(k.shape[-1] != dk or tuple(v.shape) != tuple(k.shape), "Attention: key/value shapes {} {} vs dk {}",
              tuple(k.shape), tuple(v.shape), dk)
    batchQ = q.numel() // (m * dk)
    batchKV = k.numel() // (cap * dk)
    if m >= 8 and kNew is None and not want_absmax and L == cap:
        # Many query positions per head (encoder layers, whole target sentences): the one-launch
        # form gives every query row a wave that walks the head's keys and values on its own; the
        # three operators share them through LDS tiles (1024 heads of 64 x 64 x 64: 57 us against 105).
        scores = bdot_legacy(q.reshape(batchQ, m, dk), k.reshape(batchKV, L, dk), False, True, 1.0 / float(dk) ** 0.5)
        weights = softmax(scores, mask, rowsPerMask)
        return bdot_legacy(weights, v.reshape(batchKV, L, dk)).reshape(q.shape)
    n_masks = 0
    if mask is not None:
        mask = _f32c(mask, "Attention").reshape(-1, L)
        n_masks = mask.shape[0]
    out = torch.empty_like(q)
    omax = AbsMax(q.device) if want_absmax else None
    st = be.lib.marian_hip_attention_cached(q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                            None if mask is None else mask.data_ptr(), n_masks, rowsPerMask,
                                            out.data_ptr(), batchQ, batchKV, m, L, cap, dk, 1.0 / float(dk) ** 0.5,
                                            None if omax is None else omax.data_ptr(),
                                            None if kNew is None else kNew.data_ptr(),
                                            None if vNew is None else vNew.data_ptr(), be.stream())
    _lib.check(st, "Attention")
    return (out, omax) if want_absmax else out


def ProjectedAttention(x, weights, k, v, heads, kvLen=None, mask=None, absmax=None, want_absmax=False,
                       want_projections=False):
    """The projections in front of an attention and the attention itself for one new target
    position, in one launch (reference src/models/transformer.h:279-348: MultiHead's affine nodes
    for q - and, in self-attention, k and v - then the head split and Attention()).
    x [M, K] float32; weights: [(Wq, bq)] - attention over caches that are complete (the encoder's
    keys and values) - or [(Wq, bq), (Wk, bk), (Wv, bv)] - self-attention: the new key and value
    are appended to the caches k, v at position kvLen - 1 (quantized weights, bias or None each).
    k, v [entries, capacity, 64] with kvLen positions in use; mask [n, len] or None, one row per
    sentence (query row r of [M * heads] uses row (r // heads) % n).  absmax: the AbsMax the producer
    of x left.  Returns (out [M, heads * 64], aQuant) and, when asked for, the AbsMax of out and
    the projections themselves - bit for bit what affine_f32_grouped / affine_f32 followed by
    Attention give (and faster than those up to 128 rows, level at 256, slower at 512)."""
    import ctypes
    from . import integer
    x = _f32c(x, "ProjectedAttention")
    be = _backend_of(x)
    n = len(weights)
    _abort_if(n not in (1, 3), "ProjectedAttention: one projection (q) or three (q, k, v), got {}", n)
    K = x.shape[-1]
    M = x.numel() // K if x.numel() else 0
    N = heads * 64
    _abort_if(not (k.is_contiguous() and v.is_contiguous()) or k.dtype != torch.float32 or v.dtype != torch.float32,
              "ProjectedAttention: the key/value caches must be contiguous float32{}", "")
    _abort_if(k.shape[-1] != 64 or tuple(k.shape) != tuple(v.shape), "ProjectedAttention: head size 64, got caches {} {}",
              tuple(k.shape), tuple(v.shape))
    cap = k.shape[-2]
    L = cap if kvLen is None else int(kvLen)
    batchKV = k.numel() // (cap * 64)
    aQuant = integer.QTensor.empty(x.shape, integer.Type.intgemm8, x.device)
    Bq_arr, bias_arr, proj_arr = (ctypes.c_void_p * n)(), (ctypes.c_void_p * n)(), (ctypes.c_void_p * n)()
    keep, projections = [], []
    for g, (bQuant, bias) in enumerate(weights):
        integer._check_weights(bQuant)
        _abort_if(integer.rows(bQuant) != K or integer.cols(bQuant) != N, "ProjectedAttention: weights {} vs [{}, {}]",
                  tuple(bQuant.shape), K, N)
        Bq_arr[g] = bQuant.data_ptr()
        if bias is not None:
            bias = _f32c(bias, "ProjectedAttention")
            keep.append(bias)
        bias_arr[g] = None if bias is None else bias.data_ptr()
        if want_projections:
            projections.append(torch.empty(tuple(x.shape[:-1]) + (N,), dtype=torch.float32, device=x.device))
        proj_arr[g] = projections[g].data_ptr() if want_projections else None
    n_masks = 0
    if mask is not None:
        mask = _f32c(mask, "ProjectedAttention").reshape(-1, L)
        n_masks = mask.shape[0]
    out = torch.empty(tuple(x.shape[:-1]) + (N,), dtype=torch.float32, device=x.device)
    omax = AbsMax(x.device) if want_absmax else None
    st = be.lib.marian_hip_int8_proj_attention(
        x.data_ptr(), aQuant.data_ptr(), n, Bq_arr, bias_arr, proj_arr, M, K, heads, k.data_ptr(), v.data_ptr(), batchKV,
        L, cap, None if mask is None else mask.data_ptr(), n_masks, 1.0 / 8.0, out.data_ptr(),
        None if absmax is None else absmax.data_ptr(), None if omax is None else omax.data_ptr(),
        be.workspace.data_ptr(), be.workspace_bytes, be.stream())
    _lib.check(st, "ProjectedAttention")
    res = (out, aQuant)
    if want_absmax:
        res += (omax,)
    if want_projections:
        res += (projections,)
    return res


def AttentionByAncestors(q, k, v, ancestors, kvLen, kNew, vNew, want_absmax=False):
    """Self-attention of a decoding step on caches that are never moved (no counterpart in the
    reference, which copies the surviving hypotheses' states, src/rnn/types.h:22-42): cached
    position p of hypothesis h is read from the cache entry of hypothesis ancestors[h, p].
    q [hyps * heads, 1, dk]; k, v [hyps * heads, capacity, dk]; ancestors int32 [hyps, capacity];
    kNew, vNew [hyps * heads, dk] become position kvLen - 1 of the hypotheses' own entries."""
    q, kNew, vNew = _f32c(q, "AttentionByAncestors"), _f32c(kNew, "AttentionByAncestors"), _f32c(vNew, "AttentionByAncestors")
    be = _backend_of(q)
    _abort_if(k.dtype != torch.float32 or v.dtype != torch.float32 or not (k.is_contiguous() and v.is_contiguous()) or
              k.dim() != 3 or tuple(k.shape) != tuple(v.shape), "AttentionByAncestors: the caches have to be contiguous "
              "float32 tensors [entries, capacity, dk], got {} and {}", tuple(k.shape), tuple(v.shape))
    entries, cap, dk = k.shape
    _abort_if(ancestors.dtype not in (torch.int32, torch.uint32) or ancestors.dim() != 2 or ancestors.shape[1] != cap or
              not ancestors.is_contiguous() or entries % ancestors.shape[0] != 0,
              "AttentionByAncestors: ancestors have to be a contiguous int32 tensor [hypotheses, {}]", cap)
    hyps = ancestors.shape[0]
    _abort_if(q.numel() != entries * dk or kNew.numel() != entries * dk or vNew.numel() != entries * dk,
              "AttentionByAncestors: one query, key and value row of {} values per cache entry", dk)
    out = torch.empty_like(q)
    omax = AbsMax(q.device) if want_absmax else None
    st = be.lib.marian_hip_attention_ancestors(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), hyps,
                                               entries // hyps, int(kvLen), cap, dk, 1.0 / float(dk) ** 0.5,
                                               None if omax is None else omax.data_ptr(), kNew.data_ptr(),
                                               vNew.data_ptr(), ancestors.data_ptr(), be.stream())
    _lib.check(st, "AttentionByAncestors")
    return (out, omax) if want_absmax else out


def advanceAncestors(prev, parents, lenPrev, out):
    """the table of ancestors of the next step: out[h, p] = prev[parents[h], p] for p < lenPrev,
    out[h, lenPrev] = h (prev, out: int32 [hypotheses, capacity], two tensors)"""
    _abort_if(prev.dtype != torch.int32 or out.dtype != torch.int32 or tuple(prev.shape) != tuple(out.shape) or
              prev.dim() != 2 or not (prev.is_contiguous() and out.is_contiguous()),
              "advanceAncestors expects two contiguous int32 tensors [hypotheses, capacity]{}", "")
    be = _backend_of(prev)
    par = parents.contiguous()
    if par.dtype == torch.int64:
        par = par.to(torch.int32)
    _abort_if(par.dtype not in (torch.int32, torch.uint32) or par.numel() != prev.shape[0],
              "advanceAncestors: one int32 back-pointer per hypothesis{}", "")
    st = be.lib.marian_hip_ancestors_advance(prev.data_ptr(), par.data_ptr(), prev.shape[0], prev.shape[1], int(lenPrev),
                                             out.data_ptr(), be.stream())
    _lib.check(st, "advanceAncestors")
    return out


def getNBestList(scores, N):
    """reference src/translator/nth_element.cpp:26-67: scores [dimBatch, 1, beam, vocab]; returns
    (pathScores, keys) of dimBatch * N entries, keys = position in the flattened tensor."""
    scores = _f32c(scores, "getNBestList")
    be = _backend_of(scores)
    dimBatch = scores.shape[0]
    rowLen = scores.numel() // dimBatch if dimBatch else 0
    vals = torch.empty(dimBatch * N, dtype=torch.float32, device=scores.device)
    keys = torch.empty(dimBatch * N, dtype=torch.int32, device=scores.device)
    st = be.lib.marian_hip_nbest(scores.data_ptr(), dimBatch, rowLen, N, vals.data_ptr(), keys.data_ptr(),
                                 be.stream())
    _lib.check(st, "getNBestList")
    return vals, keys


# (device, stream) -> list of uint8 tensors, the last one the largest.  The reference's NthElement
# owns its buffers too (src/translator/nth_element.cu).  A workspace holds arrival counters that
# every call leaves at zero, so calls on one stream share it; two streams never do.  A workspace
# that has been handed out is kept for good (a HIP graph may have recorded its address): a larger
# call gets an additional one.
_nbest_workspaces = {}


def getNBestListOfBeams(scores, N):
    """reference src/translator/beam_search.cpp:472 + :492: swapAxes(expandedPathScores, 0, 2)
    followed by getNBestList, without the transposed copy.  scores [beam, 1, dimBatch, vocab] (or
    [beam, dimBatch, vocab]); returns what getNBestList returns for the transposed tensor."""
    scores = _f32c(scores, "getNBestListOfBeams")
    be = _backend_of(scores)
    beam, vocab = scores.shape[0], scores.shape[-1]
    dimBatch = scores.numel() // (beam * vocab) if beam * vocab else 0
    vals = torch.empty(dimBatch * N, dtype=torch.float32, device=scores.device)
    keys = torch.empty(dimBatch * N, dtype=torch.int32, device=scores.device)
    need = be.lib.marian_hip_nbest_beams_workspace_bytes(beam, dimBatch, vocab, N)
    held = _nbest_workspaces.setdefault((scores.device, be.stream()), [])
    if not held or held[-1].numel() < need:
        ws = torch.empty(max(int(need), 4), dtype=torch.uint8, device=scores.device)
        _lib.check(be.lib.marian_hip_nbest_beams_workspace_init(ws.data_ptr(), ws.numel(), be.stream()),
                   "getNBestListOfBeams")
        held.append(ws)
    ws = held[-1]
    st = be.lib.marian_hip_nbest_beams(scores.data_ptr(), beam, dimBatch, vocab, N, vals.data_ptr(),
                                       keys.data_ptr(), ws.data_ptr(), ws.numel(), be.stream())
    _lib.check(st, "getNBestListOfBeams")
    return vals, keys


def logsoftmaxNBestOfBeams(logits, N, pathScores=None, want_logprobs=False):
    """The end of a beam-search step in one call: logsoftmax over the vocabulary (reference
    src/tensors/cpu/tensor_operators.cpp:474-526), + the hypotheses' path scores
    (src/translator/beam_search.cpp:433-436), then what getNBestListOfBeams does (:472, :492).
    logits [beam, 1, dimBatch, vocab] (or [beam, dimBatch, vocab]); pathScores: None or one value
    per row [beam, dimBatch]; returns (vals, keys), and the log-probabilities as a third value when
    asked for.  Bit for bit what the separate calls give."""
    logits = _f32c(logits, "logsoftmaxNBestOfBeams")
    be = _backend_of(logits)
    beam, vocab = logits.shape[0], logits.shape[-1]
    dimBatch = logits.numel() // (beam * vocab) if beam * vocab else 0
    if not (vocab % 4 == 0 and 4096 < vocab <= 32768 and logits.data_ptr() % 16 == 0):
        # sizes the one-launch form does not take: the separate calls
        lp = logsoftmax(logits)
        scored = lp if pathScores is None else lp + _f32c(pathScores, "logsoftmaxNBestOfBeams").reshape(
            (beam,) + (1,) * (logits.dim() - 3) + (dimBatch, 1))
        vals, keys = getNBestListOfBeams(scored, N)
        return (vals, keys, lp) if want_logprobs else (vals, keys)
    add = None
    if pathScores is not None:
        add = _f32c(pathScores, "logsoftmaxNBestOfBeams").reshape(-1)
        _abort_if(add.numel() != beam * dimBatch, "one path score per hypothesis, got {}", add.numel())
    vals = torch.empty(dimBatch * N, dtype=torch.float32, device=logits.device)
    keys = torch.empty(dimBatch * N, dtype=torch.int32, device=logits.device)
    lp = torch.empty_like(logits) if want_logprobs else None
    need = be.lib.marian_hip_nbest_beams_workspace_bytes(beam, dimBatch, vocab, N)
    held = _nbest_workspaces.setdefault((logits.device, be.stream()), [])
    if not held or held[-1].numel() < need:
        ws = torch.empty(max(int(need), 4), dtype=torch.uint8, device=logits.device)
        _lib.check(be.lib.marian_hip_nbest_beams_workspace_init(ws.data_ptr(), ws.numel(), be.stream()),
                   "logsoftmaxNBestOfBeams")
        held.append(ws)
    ws = held[-1]
    st = be.lib.marian_hip_logsoftmax_nbest_beams(
        logits.data_ptr(), None if add is None else add.data_ptr(), None if lp is None else lp.data_ptr(), beam,
        dimBatch, vocab, N, vals.data_ptr(), keys.data_ptr(), ws.data_ptr(), ws.numel(), be.stream())
    _lib.check(st, "logsoftmaxNBestOfBeams")
    return (vals, keys, lp) if want_logprobs else (vals, keys)
