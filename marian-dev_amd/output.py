"""Tied int8 output layer with shortlist plumbing, on top of integer.py.

Mirrors the parts of the reference that sit either side of the output-layer GEMM:
  reference src/data/shortlist.cpp:20-37       Shortlist (indices, reverseMap, tryForwardMap)
  reference src/data/shortlist.cpp:513-520,
            src/data/shortlist.h:320-327       padding of the id set to a multiple of eight
  reference src/layers/output.cpp:31-76        Output::lazyConstruct (tied Wt = the embedding
                                               matrix [V x D], optional bias [1 x V])
  reference src/layers/output.cpp:94-121,
            :335-354                           applyAsLogits, dense and shortlisted
  reference src/layers/embedding.cpp:160-170   Embedding::applyIndices = rows(E, ids)

The reference runs the shortlisted product in fp32 (index_select of rows of Wt, then dot with
transB).  Here the matrix Wt [V x D] row-major *is* the Type::intgemm8 file payload of the logical
B = Wt^T (K = D, N = V): quantizing Wt row by row with one per-tensor quantMult gives exactly
the bytes the weight packer would write for B; prepareAndTransposeB puts them into the order the
kernels read.  The tied matrix is quantized once, its fp32 rows stay available for the embedding
lookup, and the shortlist is a column gather inside the GEMM.
"""
import bisect

import numpy as np
import torch

from . import integer
from .types import Type

npos = -1   # reference src/data/shortlist.h: Shortlist::npos


class Shortlist:
    """reference src/data/shortlist.cpp:20-37.  `indices`: sorted unique vocabulary ids, one list
    per batch; its length must be a multiple of eight for the intgemm path."""

    def __init__(self, indices):
        idx = np.asarray(indices, dtype=np.uint32)
        integer._abort_if(idx.ndim != 1, "Shortlist expects a vector of word indices")
        integer._abort_if(idx.size > 1 and not np.all(idx[1:] > idx[:-1]),
                          "Shortlist indices must be sorted and unique")
        self.indices_ = idx
        self._device_ids = {}

    def indices(self):
        return self.indices_

    def reverseMap(self, beamIdx, batchIdx, idx):
        """shortlist coordinate -> vocabulary id (beam and batch are ignored, :26-28)"""
        return int(self.indices_[idx])

    def tryForwardMap(self, wIdx, batchIdx=0):
        """vocabulary id -> shortlist coordinate, or npos (:30-37, std::lower_bound)"""
        i = bisect.bisect_left(self.indices_, wIdx)
        if i < self.indices_.size and int(self.indices_[i]) == int(wIdx):
            return i
        return npos

    def getIndicesExpr(self, device):
        """the uint32 ids on the device (cached), as the GEMM's gather list"""
        key = str(device)
        if key not in self._device_ids:
            self._device_ids[key] = torch.from_numpy(self.indices_.view(np.int32)).to(device)
        return self._device_ids[key]

    @staticmethod
    def padToMultipleOfEight(ids, trgVocabSize, firstNum=0):
        """reference src/data/shortlist.cpp:513-520: while the number of selected ids is not a
        multiple of eight, add the lowest ids >= firstNum that are not selected yet."""
        table = np.zeros(trgVocabSize, dtype=bool)
        table[np.asarray(ids, dtype=np.int64)] = True
        ones = int(table.sum())
        i = firstNum
        while i < trgVocabSize and ones % 8 != 0:
            if not table[i]:
                table[i] = True
                ones += 1
            i += 1
        return Shortlist(np.nonzero(table)[0].astype(np.uint32))


class Output:
    """Output layer with tied embeddings (reference src/layers/output.cpp).  Wt: fp32 [V x D] on
    the GPU (the embedding matrix E when tied); b: fp32 [1 x V] or None."""

    def __init__(self, Wt, b=None):
        integer._abort_if(Wt.dtype != torch.float32 or Wt.dim() != 2,
                          "Output expects a float32 matrix [dimVoc x dimEmb], got {}", Wt.dtype)
        self.Wt_ = Wt.contiguous()
        self.b_ = None if b is None else b.contiguous().reshape(-1)
        V, D = self.Wt_.shape
        integer._abort_if(self.b_ is not None and self.b_.numel() != V, "bias must be [1 x {}]", V)
        # Quantized tied matrix: prepareA over Wt as a [V x D] tensor = per-tensor abs-max,
        # row-major int8 + quantMult tail = the intgemm8 file order of the logical [D x V], which
        # prepareAndTransposeB puts into the order the kernels read
        q = integer.prepareA(self.Wt_)
        self.WtQuant_ = integer.prepareAndTransposeB(integer.QTensor(q.data, (D, V), Type.intgemm8))
        self.shortlist_ = None

    def setShortlist(self, shortlist):
        self.shortlist_ = shortlist

    def clear(self):
        self.shortlist_ = None

    def embed(self, embIdx):
        """rows(E, ids), reference src/layers/embedding.cpp:160-170 (fp32 rows of the tied matrix)"""
        ids = torch.as_tensor(np.asarray(embIdx, dtype=np.int64), device=self.Wt_.device)
        return self.Wt_.index_select(0, ids)

    def applyAsLogits(self, input):
        """logits [.., V], or [.., k] in shortlist coordinates when a shortlist is set
        (reference src/layers/output.cpp:335-354)"""
        ids = None if self.shortlist_ is None else self.shortlist_.getIndicesExpr(input.device)
        out, _ = integer.affine_f32(input, self.WtQuant_, self.b_, shortlist=ids)
        return out

    def bestWords(self, input, k=1):
        """the k best words per row (k <= 16), returned as (scores, vocabulary ids): shortlist
        coordinates are mapped back like Shortlist::reverseMap does for the beam search
        (src/translator/beam_search.cpp); selection by the n-best kernel of the library"""
        from . import ops
        logits = self.applyAsLogits(input)
        rows, cols = logits.numel() // logits.shape[-1], logits.shape[-1]
        scores, keys = ops.getNBestList(logits.reshape(rows, 1, 1, cols), k)   # one "batch" entry per row
        scores = scores.reshape(rows, k)
        pos = keys.reshape(rows, k).to(torch.int64) - torch.arange(rows, device=logits.device)[:, None] * cols
        if self.shortlist_ is not None:
            pos = self.shortlist_.getIndicesExpr(input.device).to(torch.int64)[pos]
        return scores, pos
