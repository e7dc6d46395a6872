// C++ host side of the float operators between the int8 GEMMs (include/marian_hip_ops.h), with the
// names and argument meaning of the tensor-level functions a HIP backend of Marian has to provide.
//
// Mirrors (reference file:line):
//   src/tensors/tensor_operators.h (gpu:: declarations)                LayerNormalization, Softmax, LogSoftmax
//   src/tensors/cpu/tensor_operators.cpp:220-246,415-526,1087-1162     their CPU bodies
//   src/tensors/gpu/prod.cpp:471-574                                   ProdBatchedLegacy
//   src/models/transformer.h:241-280                                   Attention()
//   src/translator/nth_element.cpp:26-67, nth_element.cu               NthElement::getNBestList
//   src/tensors/cpu/tensor_operators.cpp:577-603                       CopyRows
//   src/tensors/cpu/tensor_operators.cpp:1733-1746                     SinusoidalPositionEmbeddings
//   src/models/transformer.h:92-117                                    ScaledEmbeddings (rows * sqrt(d) + signal)
//   src/rnn/types.h:22-42                                              SelectState (State::select); AdvanceAncestors +
//                                                                      AttentionByAncestors do without the copy
#pragma once

#include "../../include/marian_hip_ops.h"
#include "hip_int8_interface.h"

namespace marian {
namespace hip {

// out = gamma * ((x - mean) / sigma) (+ beta) over the last dimension, x = in (+ add).
// absmaxOut: optional tensor of MARIAN_HIP_ABSMAX_SLOTS floats for the affine call that reads `out`.
inline void LayerNormalization(Backend& be, Tensor& out, const Tensor& in, const Tensor& gamma,
                               const Tensor* beta, float eps, const Tensor* add = nullptr,
                               Tensor* absmaxOut = nullptr) {
  MARIAN_HIP_CHECK(marian_hip_layer_norm(
      in.data<float>(), add ? add->data<float>() : nullptr, gamma.data<float>(), (int64_t)gamma.elements(),
      beta ? beta->data<float>() : nullptr, beta ? (int64_t)beta->elements() : 0, out.data<float>(), rows(in),
      cols(in), eps, absmaxOut ? absmaxOut->data<float>() : nullptr, be.stream()));
}

// out[r, :] = scale * in[indices[r], :] (+ signal[(r / rowsPerSignal) % rows(signal), :]): the embedding
// step in front of the first layer as one launch.  indices: uint32 tensor on the device.
inline void ScaledEmbeddings(Backend& be, Tensor& out, const Tensor& in, const Tensor& indices, float scale,
                             const Tensor* signal = nullptr, int64_t rowsPerSignal = 1, Tensor* absmaxOut = nullptr) {
  if(indices.type != Type::uint32) abortWith("ScaledEmbeddings expects indices of type uint32");
  if(in.shape.size() != 2) abortWith("ScaledEmbeddings expects a [rows, cols] table");
  if(cols(out) != cols(in) || out.elements() != indices.elements() * (size_t)cols(in))
    abortWith("ScaledEmbeddings: the output has to hold one row of the table per index");
  if(signal && cols(*signal) != cols(in)) abortWith("ScaledEmbeddings: signal rows and table rows differ in length");
  MARIAN_HIP_CHECK(marian_hip_embed(in.data<float>(), indices.data<uint32_t>(), (int64_t)indices.elements(),
                                    rows(in), cols(in), scale, signal ? signal->data<float>() : nullptr,
                                    rowsPerSignal, signal ? (int64_t)rows(*signal) : 0, out.data<float>(),
                                    absmaxOut ? absmaxOut->data<float>() : nullptr, be.stream()));
}

// out[j, :] = in[indices[j], :]
inline void CopyRows(Backend& be, Tensor& out, const Tensor& in, const Tensor& indices) {
  ScaledEmbeddings(be, out, in, indices, 1.0f);
}

// The decoder state of the surviving hypotheses (State::select, src/rnn/types.h:22-42) for states
// [entries, segments, capacity] that stay in place: out[r, s, 0 .. used) = state[indices[r], s, 0 .. used).
inline void SelectState(Backend& be, Tensor& out, const Tensor& state, const Tensor& indices, int64_t used) {
  if(indices.type != Type::uint32) abortWith("SelectState expects indices of type uint32");
  if(state.shape.size() != 3 || out.shape.size() != 3 || out.shape[1] != state.shape[1] || out.shape[2] != state.shape[2] ||
     (size_t)out.shape[0] != indices.elements())
    abortWith("SelectState expects [entries, segments, capacity] tensors and one index per output entry");
  MARIAN_HIP_CHECK(marian_hip_select_state(state.data<float>(), indices.data<uint32_t>(), (int64_t)indices.elements(),
                                           state.shape[0], state.shape[1], state.shape[2], used, out.data<float>(),
                                           be.stream()));
}

// The constant [dimWords, 1, dimEmb] of the position signal, made on the host: `host` receives
// dimWords * dimEmb floats for positions start, start + 1, ...
inline void SinusoidalPositionEmbeddings(std::vector<float>& host, int64_t dimWords, int64_t dimEmb, int start) {
  host.resize((size_t)(dimWords * dimEmb));
  MARIAN_HIP_CHECK(marian_hip_sinusoidal_position_embeddings(host.data(), dimWords, dimEmb, start));
}

// mask: optional [nMasks, cols] log-mask; row r of `in` uses mask row (r / rowsPerMask) % nMasks.
inline void Softmax(Backend& be, Tensor& out, const Tensor& in, const Tensor* mask = nullptr,
                    int64_t rowsPerMask = 1) {
  MARIAN_HIP_CHECK(marian_hip_softmax(in.data<float>(), mask ? mask->data<float>() : nullptr,
                                      mask ? (int64_t)rows(*mask) : 0, rowsPerMask, out.data<float>(), rows(in),
                                      cols(in), be.stream()));
}

inline void LogSoftmax(Backend& be, Tensor& out, const Tensor& in) {
  MARIAN_HIP_CHECK(marian_hip_logsoftmax(in.data<float>(), out.data<float>(), rows(in), cols(in), be.stream()));
}

// in [d0, d1, d2, d3] -> out [d0, d2, d1, d3] (head split and join)
inline void Transpose0213(Backend& be, Tensor& out, const Tensor& in) {
  if(in.shape.size() != 4) abortWith("Transpose0213 expects a 4-d tensor");
  MARIAN_HIP_CHECK(marian_hip_transpose0213(in.data<float>(), out.data<float>(), in.shape[0], in.shape[1],
                                            in.shape[2], in.shape[3], be.stream()));
}

// C[i] = scalar * op(A[i % batchA]) * op(B[i % batchB]); the last two dimensions are the matrices.
inline void ProdBatchedLegacy(Backend& be, Tensor& C, const Tensor& A, const Tensor& B, bool transA, bool transB,
                              float scalar) {
  const int64_t ra = A.shape[A.shape.size() - 2], ca = A.shape.back();
  const int64_t rb = B.shape[B.shape.size() - 2], cb = B.shape.back();
  const int64_t m = transA ? ca : ra, k = transA ? ra : ca, l = transB ? cb : rb, n = transB ? rb : cb;
  if(l != k) abortWith("Matrix product requires inner dimensions to match");
  MARIAN_HIP_CHECK(marian_hip_bdot_legacy(A.data<float>(), B.data<float>(), C.data<float>(),
                                          (int64_t)(A.elements() / (size_t)(ra * ca)),
                                          (int64_t)(B.elements() / (size_t)(rb * cb)), m, n, k, transA ? 1 : 0,
                                          transB ? 1 : 0, scalar, be.stream()));
}

// q [batchQ, m, dk]; k, v [batchKV, positions, dk]; out [batchQ, m, dk].  kNew / vNew [batchQ, dk]:
// the newest position of a decoding step, appended to k and v by the call.  kvLen: the first kvLen
// of the cache's positions are in use (caches that stay in place from step to step); 0: all.
inline void Attention(Backend& be, Tensor& out, const Tensor& q, Tensor& k, Tensor& v, float scale,
                      const Tensor* mask = nullptr, int64_t rowsPerMask = 1, Tensor* absmaxOut = nullptr,
                      const Tensor* kNew = nullptr, const Tensor* vNew = nullptr, int64_t kvLen = 0) {
  if(q.shape.size() != 3 || k.shape.size() != 3) abortWith("Attention expects [batch, positions, dk] tensors");
  MARIAN_HIP_CHECK(marian_hip_attention_cached(
      q.data<float>(), k.data<float>(), v.data<float>(), mask ? mask->data<float>() : nullptr,
      mask ? (int64_t)rows(*mask) : 0, rowsPerMask, out.data<float>(), q.shape[0], k.shape[0], q.shape[1],
      kvLen ? kvLen : k.shape[1], k.shape[1], q.shape[2], scale, absmaxOut ? absmaxOut->data<float>() : nullptr,
      kNew ? kNew->data<float>() : nullptr, vNew ? vNew->data<float>() : nullptr, be.stream()));
}

// The projections in front of an attention and the attention itself for one new target position
// per row of a, in one launch (reference src/models/transformer.h:279-348).  weights: {Wq} - caches
// complete, e.g. the encoder's - or {Wq, Wk, Wv} - self-attention, the new key and value go into
// the caches at position kvLen - 1; biases: one entry per matrix (null entries allowed) or empty.
// a [M, K] float32; aQuant: the prepareA node's tensor; k, v [entries, capacity, 64]; out [M, heads * 64].
// Measured ahead of the two separate calls (affineOrDot for the projections, then Attention) up to
// 128 rows, level with them at 256, behind at 512: a caller with larger batches issues those.
inline void ProjectedAttention(TensorAllocator& ta, Tensor& out, const Tensor& a, Tensor& aQuant,
                               const std::vector<const Tensor*>& weights, const std::vector<const Tensor*>& biases,
                               Tensor& k, Tensor& v, int64_t heads, int64_t kvLen = 0, const Tensor* mask = nullptr,
                               const Tensor* absmaxIn = nullptr, Tensor* absmaxOut = nullptr) {
  if((weights.size() != 1 && weights.size() != 3) || (!biases.empty() && biases.size() != weights.size()))
    abortWith("ProjectedAttention: one projection (q) or three (q, k, v), one bias entry each");
  if(k.shape.size() != 3 || k.shape[2] != 64 || v.shape != k.shape) abortWith("ProjectedAttention expects caches [entries, capacity, 64]");
  void* ws = ta.workspace();   // (may allocate and move the slab: before any pointer is read)
  const int8_t* bq[3] = {nullptr, nullptr, nullptr};
  const float* bi[3] = {nullptr, nullptr, nullptr};
  for(size_t g = 0; g < weights.size(); ++g) {
    integer::checkB(*weights[g]);
    bq[g] = weights[g]->data<int8_t>();
    if(!biases.empty() && biases[g]) bi[g] = biases[g]->data<float>();
  }
  MARIAN_HIP_CHECK(marian_hip_int8_proj_attention(
      a.data<float>(), aQuant.data<int8_t>(), (int64_t)weights.size(), bq, bi, nullptr, rows(a), cols(a), heads,
      k.data<float>(), v.data<float>(), k.shape[0], kvLen ? kvLen : k.shape[1], k.shape[1],
      mask ? mask->data<float>() : nullptr, mask ? (int64_t)rows(*mask) : 0, 0.125f, out.data<float>(),
      absmaxIn ? absmaxIn->data<float>() : nullptr, absmaxOut ? absmaxOut->data<float>() : nullptr, ws,
      ta.workspaceBytes(), ta.backend().stream()));
}

// Self-attention of a decoding step on caches that are never moved: cached position p of hypothesis
// h is read from the entry of hypothesis ancestors[h, p] (uint32 [hypotheses, capacity]); kNew / vNew
// become position kvLen - 1 of the hypotheses' own entries.  q, kNew, vNew, out [hyps * heads, 1 or -, 64].
inline void AttentionByAncestors(Backend& be, Tensor& out, const Tensor& q, Tensor& k, Tensor& v, float scale,
                                 const Tensor& ancestors, int64_t kvLen, const Tensor& kNew, const Tensor& vNew,
                                 Tensor* absmaxOut = nullptr) {
  if(k.shape.size() != 3 || ancestors.shape.size() != 2 || ancestors.type != Type::uint32 ||
     ancestors.shape[1] != k.shape[1] || k.shape[0] % ancestors.shape[0] != 0)
    abortWith("AttentionByAncestors expects caches [entries, capacity, dk] and uint32 ancestors [hypotheses, capacity]");
  MARIAN_HIP_CHECK(marian_hip_attention_ancestors(
      q.data<float>(), k.data<float>(), v.data<float>(), out.data<float>(), ancestors.shape[0],
      k.shape[0] / ancestors.shape[0], kvLen, k.shape[1], k.shape[2], scale,
      absmaxOut ? absmaxOut->data<float>() : nullptr, kNew.data<float>(), vNew.data<float>(),
      ancestors.data<uint32_t>(), be.stream()));
}

// The table of the next step: next[h, p] = prev[parents[h], p] for p < lenPrev, next[h, lenPrev] = h.
inline void AdvanceAncestors(Backend& be, Tensor& next, const Tensor& prev, const Tensor& parents, int64_t lenPrev) {
  if(prev.shape.size() != 2 || next.shape != prev.shape || prev.type != Type::uint32 || next.type != Type::uint32 ||
     parents.type != Type::uint32 || parents.elements() != (size_t)prev.shape[0])
    abortWith("AdvanceAncestors expects uint32 tables [hypotheses, capacity] and one back-pointer per hypothesis");
  MARIAN_HIP_CHECK(marian_hip_ancestors_advance(prev.data<uint32_t>(), parents.data<uint32_t>(), prev.shape[0],
                                                prev.shape[1], lenPrev, next.data<uint32_t>(), be.stream()));
}

// The beam search's n-best selection; it owns its device buffers like the reference's NthElement.
class NthElement {
public:
  explicit NthElement(TensorAllocator& ta) : ta_(ta) {}

  // scores [dimBatch, beam * vocab] -> the N best scores and keys of every row (device tensors)
  void getNBestList(const Tensor& scores, int64_t N, Tensor& outScores, Tensor& outKeys) {
    const int64_t dimBatch = scores.shape[0], rowLen = (int64_t)scores.elements() / dimBatch;
    ta_.allocate(outScores, {(int)(dimBatch * N)}, Type::float32);
    ta_.allocate(outKeys, {(int)(dimBatch * N)}, Type::uint32);
    MARIAN_HIP_CHECK(marian_hip_nbest(scores.data<float>(), dimBatch, rowLen, N, outScores.data<float>(),
                                      outKeys.data<uint32_t>(), ta_.backend().stream()));
  }

  // scores [beam, dimBatch, vocab] as they leave the decoder: transposition + n-best in one call
  void getNBestListOfBeams(const Tensor& scores, int64_t N, Tensor& outScores, Tensor& outKeys) {
    if(scores.shape.size() != 3) abortWith("getNBestListOfBeams expects [beam, batch, vocab]");
    const int64_t beam = scores.shape[0], dimBatch = scores.shape[1], vocab = scores.shape[2];
    ta_.allocate(outScores, {(int)(dimBatch * N)}, Type::float32);
    ta_.allocate(outKeys, {(int)(dimBatch * N)}, Type::uint32);
    const size_t need = marian_hip_nbest_beams_workspace_bytes(beam, dimBatch, vocab, N);
    if(!workspace_ || workspace_.elements() < need) {
      // (a larger one replaces the old one; its counters are cleared once, by a kernel)
      if(workspace_) ta_.free(workspace_);
      ta_.allocate(workspace_, {(int)need}, Type::int8);
      MARIAN_HIP_CHECK(marian_hip_nbest_beams_workspace_init(workspace_.data<void>(), need, ta_.backend().stream()));
    }
    MARIAN_HIP_CHECK(marian_hip_nbest_beams(scores.data<float>(), beam, dimBatch, vocab, N, outScores.data<float>(),
                                            outKeys.data<uint32_t>(), workspace_.data<void>(), workspace_.elements(),
                                            ta_.backend().stream()));
  }

  // The end of a beam-search step in one call: LogSoftmax of the logits [beam, dimBatch, vocab], + the
  // path score of each hypothesis (pathScores: null or [beam, dimBatch]), transposition + n-best;
  // logProbs: null, or a tensor that also receives the log-probabilities.
  void logSoftmaxNBestOfBeams(const Tensor& logits, const Tensor* pathScores, int64_t N, Tensor& outScores,
                              Tensor& outKeys, Tensor* logProbs = nullptr) {
    if(logits.shape.size() != 3) abortWith("logSoftmaxNBestOfBeams expects [beam, batch, vocab]");
    const int64_t beam = logits.shape[0], dimBatch = logits.shape[1], vocab = logits.shape[2];
    if(vocab % 4 != 0 || vocab <= 4096 || vocab > 32768) {   // sizes the one-launch form does not take
      if(pathScores) abortWith("logSoftmaxNBestOfBeams: path scores need the one-launch form (4096 < vocab <= 32768)");
      Tensor lp;
      Tensor& target = logProbs ? *logProbs : lp;
      ta_.allocate(target, logits.shape, Type::float32);
      Tensor rows = logits, out = target;
      rows.shape = {(int)(beam * dimBatch), (int)vocab};
      out.shape = rows.shape;
      LogSoftmax(ta_.backend(), out, rows);
      getNBestListOfBeams(target, N, outScores, outKeys);
      if(!logProbs) ta_.free(lp);
      return;
    }
    ta_.allocate(outScores, {(int)(dimBatch * N)}, Type::float32);
    ta_.allocate(outKeys, {(int)(dimBatch * N)}, Type::uint32);
    if(logProbs) ta_.allocate(*logProbs, logits.shape, Type::float32);
    reserveWorkspace(beam, dimBatch, vocab, N);
    MARIAN_HIP_CHECK(marian_hip_logsoftmax_nbest_beams(
        logits.data<float>(), pathScores ? pathScores->data<float>() : nullptr, logProbs ? logProbs->data<float>() : nullptr,
        beam, dimBatch, vocab, N, outScores.data<float>(), outKeys.data<uint32_t>(), workspace_.data<void>(),
        workspace_.elements(), ta_.backend().stream()));
  }

private:
  void reserveWorkspace(int64_t beam, int64_t dimBatch, int64_t vocab, int64_t N) {
    const size_t need = marian_hip_nbest_beams_workspace_bytes(beam, dimBatch, vocab, N);
    if(!workspace_ || workspace_.elements() < need) {
      if(workspace_) ta_.free(workspace_);
      ta_.allocate(workspace_, {(int)need}, Type::int8);
      MARIAN_HIP_CHECK(marian_hip_nbest_beams_workspace_init(workspace_.data<void>(), need, ta_.backend().stream()));
    }
  }
  TensorAllocator& ta_;
  Tensor workspace_;
};

}  // namespace hip
}  // namespace marian
