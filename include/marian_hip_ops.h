/*
 * marian_hip_ops.h - C ABI of the float32 operators that sit between the int8 GEMMs of a
 * transformer decode step (same library and conventions as marian_hip_int8.h: device pointers,
 * caller-owned buffers, nothing retained, work enqueued on `stream`, status codes, no
 * synchronisation).  All tensors are dense row-major fp32; pointers need 4-byte alignment only
 * (16-byte aligned rows take a vector path).  In-place operation (out == in) is allowed for
 * layer_norm, softmax and logsoftmax.
 */
#ifndef MARIAN_HIP_OPS_H
#define MARIAN_HIP_OPS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Replaces LayerNormalization, reference src/tensors/gpu/tensor_operators.cu (gLNormalization)
 * and src/tensors/cpu/tensor_operators.cpp:1087-1162, node LayerNormalizationOp
 * (src/graph/expression_operators.cpp:901-913):
 *   mean = sum(x) / cols; sigma = sqrt(sum((x - mean)^2) / cols + eps);
 *   out = gamma * ((x - mean) / sigma) (+ beta)
 * over the last dimension.  gamma_cols / beta_cols: `cols`, or 1 for a single broadcast value;
 * beta may be NULL.  add != NULL fuses the skip connection that precedes the normalization in
 * the transformer's post-processing (`output + prevInput`, src/models/transformer.h:192-193,207):
 * x = in + add, else x = in.
 * absmax_out: NULL, or MARIAN_HIP_ABSMAX_SLOTS (2048) floats that receive values whose maximum is
 * max|out|, for marian_hip_int8_affine_f32_chained.  Up to 2048 rows own a slot each; more rows
 * (an encoder's sentence batch) share the slots, which a second small kernel of the same call
 * clears first.
 */
int marian_hip_layer_norm(const float* in, const float* add, const float* gamma,
                          int64_t gamma_cols, const float* beta, int64_t beta_cols, float* out,
                          int64_t rows, int64_t cols, float eps, float* absmax_out, void* stream);

/*
 * Replaces Softmax, reference src/tensors/gpu/tensor_operators.cu (gSoftmax) and
 * src/tensors/cpu/tensor_operators.cpp:415-470, over the last dimension.  mask != NULL fuses the
 * `z + mask` node in front of it (src/models/transformer.h:264): mask holds n_masks rows of
 * `cols` values and row r of `in` uses mask row (r / rows_per_mask) % n_masks - a
 * [batch, 1, 1, len] log-mask, repeated over the beam (src/models/transformer.h:772-774),
 * against scores of shape [beam * batch, heads, tgt, len] has rows_per_mask = heads * tgt,
 * n_masks = batch.
 */
int marian_hip_softmax(const float* in, const float* mask, int64_t n_masks, int64_t rows_per_mask,
                       float* out, int64_t rows, int64_t cols, void* stream);

/* Replaces LogSoftmax, reference src/tensors/gpu/tensor_operators.cu (gLogSoftmax) and
 * src/tensors/cpu/tensor_operators.cpp:474-526. */
int marian_hip_logsoftmax(const float* in, float* out, int64_t rows, int64_t cols, void* stream);

/*
 * Replaces TransposeND for the axes {0, 2, 1, 3} (Transpose0213, reference
 * src/tensors/cpu/tensor_operators.cpp:220-246, gTranspose0213 on the GPU), the head split and
 * join of src/models/transformer.h:145-170: in [d0, d1, d2, d3] -> out [d0, d2, d1, d3].
 * out must not alias in.
 */
int marian_hip_transpose0213(const float* in, float* out, int64_t d0, int64_t d1, int64_t d2,
                             int64_t d3, void* stream);

/*
 * Replaces ProdBatchedLegacy with beta = 0, reference src/tensors/cpu/prod.cpp:233-330 and
 * src/tensors/gpu/prod.cpp:471-574 (node bdot_legacy, the attention products of
 * src/models/transformer.h:261,277):
 *   C[i] = scalar * op(A[i % batchA]) * op(B[i % batchB]),  i < max(batchA, batchB)
 * A: [batchA, m, k] ([batchA, k, m] when transA), B: [batchB, k, n] ([batchB, n, k] when
 * transB), C: [max(batchA, batchB), m, n].
 */
int marian_hip_bdot_legacy(const float* A, const float* B, float* C, int64_t batchA,
                           int64_t batchB, int64_t m, int64_t n, int64_t k, int transA,
                           int transB, float scalar, void* stream);

/*
 * The attention of one decoding step in one launch: the nodes bdot_legacy(q, k, false, true,
 * scale), `+ mask`, softmax and bdot_legacy(weights, v) of Attention(), reference
 * src/models/transformer.h:241-280.  The arithmetic is that of the three separate entry points
 * above; for head sizes other than 64 operation for operation (the result equals theirs bit for
 * bit), for dk == 64 with the dot products summed sixteen lanes wide and the weighted values four
 * positions wide (equal within the 1e-5 relative bar of the float operators).
 *   q: [batchQ, m, dk], k and v: [batchKV, len, dk] (entry i uses k, v of i % batchKV: encoder
 *   keys shared by the beam), out: [batchQ, m, dk]; mask as in marian_hip_softmax for score rows
 *   [batchQ * m, len], or NULL.  len <= 4096.
 *   Built for decoding steps (m = 1 or a few query positions per head): every query row gets a
 *   wave that walks the head's keys and values itself.  With eight or more positions per head
 *   (encoder layers) the three separate entry points, which share a head's keys and values
 *   through LDS tiles, are about twice as fast; the host mirror switches over by itself.
 *   Where several query rows share a cache entry (batchKV < batchQ, m == 1, dk == 64, len <= 96,
 *   16-byte aligned tensors, no k_new) the rows of an entry are taken by one workgroup, which
 *   reads the entry's keys and values once: same bits, 28 instead of 50 us for 512 rows x 16 heads
 *   over 60 source positions with four hypotheses a sentence.
 *   absmax_out: as for marian_hip_layer_norm (needs batchQ * m <= 2048).
 *   k_new, v_new: NULL, or [batchQ, dk] keys and values of the newest position (self-attention of
 *   a decoding step: m == 1, batchKV == batchQ).  They take the place of position len - 1 of k and
 *   v, and the call also stores them there, which is the concatenation of the new position onto
 *   the cached ones (decoder state of src/models/transformer.h:683-700) without a copy launch; k
 *   and v are written in that case.
 */
int marian_hip_attention(const float* q, float* k, float* v, const float* mask, int64_t n_masks,
                         int64_t rows_per_mask, float* out, int64_t batchQ, int64_t batchKV,
                         int64_t m, int64_t len, int64_t dk, float scale, float* absmax_out,
                         const float* k_new, const float* v_new, void* stream);

/*
 * marian_hip_attention on caches that have room to grow: k and v are [batchKV, kv_capacity, dk]
 * with the first len positions of every entry in use (kv_capacity >= len; the mask still has len
 * values per row).  The decoder state of a translation then stays where it is from step to step:
 * the reference concatenates the new position onto the cached ones into a fresh tensor every
 * step (src/models/transformer.h:409-416), here a step passes len = positions so far + 1 with k_new,
 * v_new, which the call stores at position len - 1, and the selection of the surviving
 * hypotheses between two steps (src/rnn/types.h:22-42) is rows() over entries of kv_capacity * dk
 * values.  marian_hip_attention is this call with kv_capacity = len.
 */
int marian_hip_attention_cached(const float* q, float* k, float* v, const float* mask, int64_t n_masks,
                                int64_t rows_per_mask, float* out, int64_t batchQ, int64_t batchKV,
                                int64_t m, int64_t len, int64_t kv_capacity, int64_t dk, float scale,
                                float* absmax_out, const float* k_new, const float* v_new, void* stream);

/*
 * The embedding step in front of the first layer, reference src/layers/embedding.cpp:161-168
 * (rows(E, ids): CopyRows, src/tensors/cpu/tensor_operators.cpp:577-603), followed by
 * src/models/transformer.h:93 (sqrt(dimEmb) * embeddings) and :117 (embeddings + signal, the
 * sinusoidal position signal of src/tensors/cpu/tensor_operators.cpp:1733-1746) as one launch:
 *   out[r, :] = scale * E[ids[r], :] + signal[(r / rows_per_signal) % n_signals, :]
 * with the product and the sum rounded one after the other like the reference's two nodes, so
 * the result equals theirs bit for bit.
 *   E: [vocab, dimEmb] float32; ids: rows word indices (uint32, the reference's IndexType), on the
 *   device.  The reference reads past the table for an id >= vocab; this call reads the table's
 *   last row instead.
 *   signal: NULL (no sum: a pure gather when scale == 1), or [n_signals, dimEmb].  A decoding step
 *   passes the one row of its position (n_signals == 1); a whole sentence batch [dimWords,
 *   dimBatch] passes rows_per_signal = dimBatch, n_signals = dimWords.
 *   absmax_out: as for marian_hip_layer_norm (needs rows * ceil(dimEmb / 4096) <= 2048): the int8
 *   products of the first layer then need no abs-max launch of their own.
 * With scale 1 and no signal the call is rows(E, ids) itself, which is also the selection of the
 * surviving hypotheses' decoder states between two steps of the beam search (reference
 * src/rnn/types.h:22-42: rows(reshape(state, [beam * batch, positions * depth]), selIdx)); rows
 * longer than 4096 values are split over several workgroups.
 */
int marian_hip_embed(const float* E, const uint32_t* ids, int64_t rows, int64_t vocab, int64_t dimEmb,
                     float scale, const float* signal, int64_t rows_per_signal, int64_t n_signals,
                     float* out, float* absmax_out, void* stream);

/*
 * Self-attention of a decoding step on caches that are never moved: where the reference selects
 * the surviving hypotheses' states between two steps by copying them (src/rnn/types.h:22-42), a
 * table of ancestors says in whose cache entry a position of a hypothesis's history lies, and the
 * call follows it.  No counterpart in the reference; the result is that of
 * marian_hip_attention_cached on caches gathered position by position, bit for bit.
 *   q, k_new, v_new, out: [n_hyp * heads, dk]; k, v: [n_hyp * heads, kv_capacity, dk], entry =
 *   hypothesis * heads + head; ancestors: uint32 [n_hyp, kv_capacity] on the device: cached position
 *   p < len - 1 of hypothesis h is read from the entry of hypothesis ancestors[h * kv_capacity + p]
 *   (values at or past n_hyp read the last hypothesis); position len - 1 is k_new / v_new, which the
 *   call stores into hypothesis h's own entry.  dk == 64, all tensors 16-byte aligned.
 * marian_hip_ancestors_advance makes the table of the next step: next[h, p] = prev[parents[h], p]
 * for the len_prev positions cached so far and next[h, len_prev] = h (prev and next must not
 * overlap); parents: uint32 [n_hyp], the back-pointers of the beam search.
 */
int marian_hip_attention_ancestors(const float* q, float* k, float* v, float* out, int64_t n_hyp, int64_t heads,
                                   int64_t len, int64_t kv_capacity, int64_t dk, float scale, float* absmax_out,
                                   const float* k_new, const float* v_new, const uint32_t* ancestors,
                                   void* stream);
int marian_hip_ancestors_advance(const uint32_t* prev, const uint32_t* parents, int64_t n_hyp, int64_t kv_capacity,
                                 int64_t len_prev, uint32_t* next, void* stream);

/*
 * The selection of the surviving hypotheses' decoder states between two steps of the beam search
 * (reference src/models/states.h:87-107, src/rnn/types.h:22-42: rows(reshape(state, [beam * batch,
 * positions * depth]), selIdx)) for states that stay in place and have room to grow:
 *   state: [entries, segments, seg_capacity] float32 (the caches of marian_hip_attention_cached:
 *   segments = heads, seg_capacity = kv_capacity * dk), out: [rows, segments, seg_capacity];
 *   out[r, s, 0 .. seg_len) = state[ids[r], s, 0 .. seg_len), seg_len = positions in use * dk.
 * What lies behind seg_len is neither read nor written.  state and out must not overlap
 * (MARIAN_HIP_ERR_ALIAS); an id at or past `entries` reads the last entry.
 * With seg_len == seg_capacity and one segment this is marian_hip_embed with scale 1.
 */
int marian_hip_select_state(const float* state, const uint32_t* ids, int64_t rows, int64_t entries,
                            int64_t segments, int64_t seg_capacity, int64_t seg_len, float* out, void* stream);

/*
 * Replaces SinusoidalPositionEmbeddings, reference src/tensors/cpu/tensor_operators.cpp:1733-1746,
 * the initializer of the constant that src/models/transformer.h:110-111 adds to the embeddings:
 *   host_out[j, i] = sin or cos of (j + start) * exp((i % (dimEmb / 2)) * -log(10000) / (dimEmb / 2 - 1)),
 * sine for the first half of a row, cosine for the rest, in float arithmetic with the C library's
 * functions like the reference's loop.  host_out: dimWords * dimEmb floats in HOST memory (the
 * constant is made once per position on the host and copied to the device by the caller);
 * dimEmb >= 4 (with fewer the reference's increment divides by zero).  No HIP call is made.
 */
int marian_hip_sinusoidal_position_embeddings(float* host_out, int64_t dimWords, int64_t dimEmb, int64_t start);

/*
 * Replaces NthElement::getNBestList, reference src/translator/nth_element.cpp:26-67 (CPU) and
 * src/translator/nth_element.cu (GPU): for each of dimBatch rows of rowLen = beam * vocabulary
 * scores, the N best scores in descending order and their keys = absolute positions
 * row * rowLen + index (uint32).  Equal scores come out lowest index first (the reference's
 * partial_sort leaves that order unspecified).  1 <= N <= 16, N <= rowLen.
 * outScores, outKeys: dimBatch * N values each, on the device.
 */
int marian_hip_nbest(const float* scores, int64_t dimBatch, int64_t rowLen, int64_t N,
                     float* outScores, uint32_t* outKeys, void* stream);

/*
 * The transposition and the n-best selection of a beam-search step in one call: reference
 * src/translator/beam_search.cpp:472 (swapAxes(expandedPathScores, 0, 2)) followed by :492
 * (getNBestList).  scores: [beam, dimBatch, vocab], the layout in which the step's scores leave the
 * decoder.  The result is that of marian_hip_nbest on the transposed tensor [dimBatch, beam * vocab]
 * - the same scores, the same keys b * beam * vocab + k * vocab + v, the same order - without
 * writing that tensor, and with the row of a batch entry split over several workgroups (the N best
 * of every part, then the N best of those, in one launch).  1 <= N <= 16, beam * N <= 1024, dimBatch <= 4096.
 *   workspace: device memory of at least marian_hip_nbest_beams_workspace_bytes(...) bytes (the
 *   reference's NthElement holds such buffers itself, src/translator/nth_element.cu): the
 *   candidates of the parts, and one counter per batch entry by which the workgroup that finishes an
 *   entry last knows that it is to draw the final list.  The counters are zero between calls:
 *   marian_hip_nbest_beams_workspace_init clears a freshly allocated workspace once (a kernel, so it
 *   may be captured in a graph).  One workspace serves one stream: calls that share a workspace must
 *   not overlap (two streams, or two threads, need a workspace each), and a workspace whose address a
 *   recorded graph holds must stay allocated as long as that graph is replayed.
 */
size_t marian_hip_nbest_beams_workspace_bytes(int64_t beam, int64_t dimBatch, int64_t vocab, int64_t N);
int marian_hip_nbest_beams_workspace_init(void* workspace, size_t workspace_bytes, void* stream);
int marian_hip_nbest_beams(const float* scores, int64_t beam, int64_t dimBatch, int64_t vocab, int64_t N,
                           float* outScores, uint32_t* outKeys, void* workspace, size_t workspace_bytes,
                           void* stream);

/*
 * The end of a beam-search step in one call: the log-softmax of the decoder's logits (LogSoftmax,
 * src/tensors/cpu/tensor_operators.cpp:474-526, as marian_hip_logsoftmax computes it), the addition of
 * the hypotheses' path scores (expandedPathScores = prevPathScores + logProbs,
 * src/translator/beam_search.cpp:433-436) and the transposition + n-best selection of
 * marian_hip_nbest_beams (:472, :492), without writing the log-probabilities and reading them back.
 *   logits: [beam, dimBatch, vocab]; vocab % 4 == 0, 4096 < vocab <= 32768 (a row is held in the
 *   registers of one 1024-thread workgroup, as marian_hip_logsoftmax does for these sizes; other
 *   sizes: MARIAN_HIP_ERR_SHAPE - use the separate calls), 16-byte aligned.
 *   rowAdd: NULL, or one value per row [beam * dimBatch] that is added to every log-probability of
 *   the row before the selection (the path score; what is written to logProbs is without it).
 *   logProbs: NULL, or [beam, dimBatch, vocab] that receives the log-probabilities as well.
 * outScores, outKeys, N, workspace: as for marian_hip_nbest_beams (a workspace sized and initialised
 * for it with the same beam, dimBatch, vocab and N serves this call too); the results are those of
 * marian_hip_logsoftmax (+ rowAdd) followed by marian_hip_nbest_beams, bit for bit.
 */
int marian_hip_logsoftmax_nbest_beams(const float* logits, const float* rowAdd, float* logProbs, int64_t beam,
                                      int64_t dimBatch, int64_t vocab, int64_t N, float* outScores,
                                      uint32_t* outKeys, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Replaces gpu::fill, reference src/tensors/gpu/algorithm.cu:37-60 (gFill): `count` elements of
 * elem_bytes (1, 2, 4 or 8) bytes each, starting at `begin` (aligned to elem_bytes), receive the
 * low elem_bytes bytes of `pattern` - the bit pattern of the value, so one entry point serves
 * every element type.  A kernel, not a memset: it may be recorded into a HIP graph.  Like every
 * function here it does not synchronise; the C++ wrapper adds the reference's stream synchronisation.
 */
int marian_hip_fill(void* begin, int64_t count, int elem_bytes, uint64_t pattern, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MARIAN_HIP_OPS_H */
