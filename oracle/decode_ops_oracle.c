/*
 * CPU restatement of the float32 operators that sit between the int8 GEMMs of a transformer
 * decode step in Marian.  TEST INFRASTRUCTURE ONLY: only tests, the smoke check and the
 * cpu_baseline leg of the benchmark may link or call it; the shipped library never does.
 *
 * Each function follows the reference's own CPU implementation, loop for loop, in plain float
 * arithmetic (the reference compiles these loops with fast-math and SIMD widths of 4 or 8, so its
 * summation order is not fixed; the checks therefore carry a tolerance):
 *   oracle_layer_norm      reference src/tensors/cpu/tensor_operators.cpp:1087-1125
 *                          (LayerNormalizationImpl), optionally preceded by the skip connection
 *                          `output + prevInput` of src/models/transformer.h:192-193
 *   oracle_softmax         reference src/tensors/cpu/tensor_operators.cpp:415-452, optionally
 *                          preceded by `z + mask` of src/models/transformer.h:264
 *   oracle_logsoftmax      reference src/tensors/cpu/tensor_operators.cpp:474-509
 *   oracle_transpose0213   reference src/tensors/cpu/tensor_operators.cpp:220-246
 *   oracle_bdot_legacy     reference src/tensors/cpu/prod.cpp:233-330 (ProdBatchedLegacy, beta = 0)
 *   oracle_nbest           reference src/translator/nth_element.cpp:26-67 (getNBestList)
 *   oracle_embed           reference src/layers/embedding.cpp:161-168 (rows(E, ids), i.e. CopyRows,
 *                          src/tensors/cpu/tensor_operators.cpp:577-603) followed by the two nodes of
 *                          src/models/transformer.h:93 (sqrt(dimEmb) * embeddings) and :117
 *                          (embeddings + signal, the signal row shared by the words of a position)
 *   oracle_sinusoidal_position_embeddings
 *                          reference src/tensors/cpu/tensor_operators.cpp:1733-1746
 *
 * Pinning status (tests/test_decode_ops.py): every function is checked against float64 closed
 * forms in numpy and against invariants that a dropped term or a wrong index would break
 * (softmax rows sum to one and are shift invariant; layer-norm output has mean beta and
 * variance gamma^2 for constant gamma/beta; transposing twice is the identity; the batched
 * product against numpy matmul including the batch broadcast i % batchA, i % batchB; the n-best
 * list against a full numpy sort; the embedding step against numpy indexing with scale 1 and no
 * signal - a pure row copy - and against float64 with both; the position signal against float64
 * sin/cos of position / 10000^(i / (d/2 - 1)) and its values at position 0: zeros and ones): pinned.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

/* out = gamma * ((x - mean) / sigma) + beta per row, x = in (+ add);
 * gamma_stride / beta_stride: 1 = one value per column, 0 = a single broadcast value;
 * beta may be NULL. */
void oracle_layer_norm(float* out, const float* in, const float* add, const float* gamma,
                       int gamma_stride, const float* beta, int beta_stride, float eps,
                       int64_t rows, int64_t cols) {
  for(int64_t j = 0; j < rows; ++j) {
    float* so = out + j * cols;
    const float* sp = in + j * cols;
    const float* sa = add ? add + j * cols : NULL;
    float sum = 0.f;
    for(int64_t i = 0; i < cols; ++i) {
      float x = sa ? sp[i] + sa[i] : sp[i];
      so[i] = x; /* the summed input is what the normalization reads */
      sum += x;
    }
    float mean = sum / (float)cols;
    float sqSum = 0.f;
    for(int64_t i = 0; i < cols; ++i) {
      float ex = so[i] - mean;
      sqSum += ex * ex;
    }
    float sigma = sqrtf(sqSum / (float)cols + eps);
    for(int64_t i = 0; i < cols; ++i) {
      float t = gamma[gamma_stride * i] * ((so[i] - mean) / sigma);
      if(beta)
        t += beta[beta_stride * i];
      so[i] = t;
    }
  }
}

/* out = softmax(in + mask) over the last dimension.  mask (may be NULL): n_masks rows of cols
 * values; row r of `in` uses mask row (r / rows_per_mask) % n_masks, which is how a
 * [batch, 1, 1, len] mask repeated over the beam (src/models/transformer.h:774) meets scores of
 * shape [beam * batch, heads, 1, len]. */
void oracle_softmax(float* out, const float* in, const float* mask, int64_t rows, int64_t cols,
                    int64_t rows_per_mask, int64_t n_masks) {
  for(int64_t j = 0; j < rows; ++j) {
    float* so = out + j * cols;
    const float* sp = in + j * cols;
    const float* sm = mask ? mask + ((j / rows_per_mask) % n_masks) * cols : NULL;
    for(int64_t i = 0; i < cols; ++i) so[i] = sm ? sp[i] + sm[i] : sp[i];
    float max = so[0];
    for(int64_t i = 1; i < cols; ++i) max = so[i] > max ? so[i] : max;
    float sum = 0.f;
    for(int64_t i = 0; i < cols; ++i) {
      float ex = expf(so[i] - max);
      sum += ex;
      so[i] = ex;
    }
    for(int64_t i = 0; i < cols; ++i) so[i] = so[i] / sum;
  }
}

void oracle_logsoftmax(float* out, const float* in, int64_t rows, int64_t cols) {
  for(int64_t j = 0; j < rows; ++j) {
    float* so = out + j * cols;
    const float* sp = in + j * cols;
    float max = sp[0];
    for(int64_t i = 1; i < cols; ++i) max = sp[i] > max ? sp[i] : max;
    float sum = 0.f;
    for(int64_t i = 0; i < cols; ++i) {
      float sm = sp[i] - max;
      sum += expf(sm);
      so[i] = sm;
    }
    float logSum = logf(sum);
    for(int64_t i = 0; i < cols; ++i) so[i] = so[i] - logSum;
  }
}

/* in [d0, d1, d2, d3] -> out [d0, d2, d1, d3]; with r2 = d1, r1 = d2 this is the reference loop:
 * source row j (of r1 * r2 per outer index) goes to row j / r1 + (j % r1) * r2. */
void oracle_transpose0213(float* out, const float* in, int64_t d0, int64_t d1, int64_t d2,
                          int64_t d3) {
  const int64_t r1 = d2, r2 = d1;
  for(int64_t k = 0; k < d0; ++k) {
    const int64_t shift = k * r1 * r2;
    for(int64_t j = 0; j < r1 * r2; ++j) {
      const int64_t src = j + shift;
      const int64_t dst = j / r1 + (j % r1) * r2 + shift;
      for(int64_t i = 0; i < d3; ++i) out[dst * d3 + i] = in[src * d3 + i];
    }
  }
}

/* C[i] = scalar * op(A[i % batchA]) * op(B[i % batchB]) for i < max(batchA, batchB);
 * A is [batchA, m, k] (or [batchA, k, m] when transA), B is [batchB, k, n] (or [batchB, n, k]),
 * C is [batchC, m, n], all row-major. */
void oracle_bdot_legacy(float* C, const float* A, const float* B, int64_t batchA, int64_t batchB,
                        int64_t m, int64_t n, int64_t k, int transA, int transB, float scalar) {
  const int64_t batchC = batchA > batchB ? batchA : batchB;
  const int64_t lda = transA ? m : k, ldb = transB ? k : n;
  for(int64_t i = 0; i < batchC; ++i) {
    const float* a = A + (i % batchA) * m * k;
    const float* b = B + (i % batchB) * n * k;
    float* c = C + i * m * n;
    for(int64_t r = 0; r < m; ++r)
      for(int64_t q = 0; q < n; ++q) {
        float s = 0.f;
        for(int64_t p = 0; p < k; ++p) {
          float av = transA ? a[p * lda + r] : a[r * lda + p];
          float bv = transB ? b[q * ldb + p] : b[p * ldb + q];
          s += av * bv;
        }
        c[r * n + q] = scalar * s;
      }
  }
}

/* For each of dimBatch rows of rowLen scores: the N best in descending order (selection by
 * repeated maximum; equal scores lowest index first, an order the reference's partial_sort leaves
 * open) and their keys = row * rowLen + index. */
void oracle_nbest(const float* scores, int64_t dimBatch, int64_t rowLen, int64_t N,
                  float* outScores, uint32_t* outKeys) {
  for(int64_t b = 0; b < dimBatch; ++b) {
    const float* x = scores + b * rowLen;
    for(int64_t n = 0; n < N; ++n) {
      int64_t best = -1;
      for(int64_t i = 0; i < rowLen; ++i) {
        int taken = 0;
        for(int64_t p = 0; p < n; ++p)
          if(outKeys[b * N + p] == (uint32_t)(b * rowLen + i)) taken = 1;
        if(taken) continue;
        if(best < 0 || x[i] > x[best]) best = i;
      }
      outScores[b * N + n] = x[best];
      outKeys[b * N + n] = (uint32_t)(b * rowLen + best);
    }
  }
}

/* out[r, :] = scale * E[ids[r], :] (+ signal[(r / rows_per_signal) % n_signals, :]); the product and
 * the sum round separately (two graph nodes in the reference). */
void oracle_embed(float* out, const float* E, const uint32_t* ids, int64_t rows, int64_t dimEmb,
                  float scale, const float* signal, int64_t rows_per_signal, int64_t n_signals) {
  for(int64_t r = 0; r < rows; ++r) {
    const float* src = E + (size_t)ids[r] * dimEmb;
    const float* sg = signal ? signal + ((r / rows_per_signal) % n_signals) * dimEmb : NULL;
    for(int64_t i = 0; i < dimEmb; ++i) {
      volatile float scaled = scale * src[i];   /* (kept apart from the addition: no fused multiply-add) */
      out[r * dimEmb + i] = sg ? scaled + sg[i] : scaled;
    }
  }
}

/* t[j, i] = sin or cos of (j + start) * exp((i % (d/2)) * -log(10000) / (d/2 - 1)), sine for the
 * first half of the row, cosine for the second; float arithmetic and the C library's expf / sinf /
 * cosf, as the reference's loop has them. */
void oracle_sinusoidal_position_embeddings(float* t, int64_t dimWords, int64_t dimEmb, int start) {
  const float numTimescales = (float)dimEmb / 2;
  const float logTimescaleIncrement = logf(10000.f) / (numTimescales - 1.f);
  for(int64_t j = 0; j < dimWords; ++j)
    for(int64_t i = 0; i < dimEmb; ++i) {
      const float v = (float)(j + start) * expf((float)(i % (int)numTimescales) * -logTimescaleIncrement);
      t[j * dimEmb + i] = i < (int)numTimescales ? sinf(v) : cosf(v);
    }
}
