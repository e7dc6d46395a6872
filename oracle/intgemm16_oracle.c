/*
 * CPU restatement of Marian's 16-bit intgemm affine/dot path (Type::intgemm16).  TEST
 * INFRASTRUCTURE ONLY: the checker for the HIP path's 16-bit entry points; only tests may link or
 * call it, the shipped library never falls back to it.
 *
 * As for the 8-bit path the arithmetic lives in the absent third-party library marian-nmt/intgemm
 * (reference .gitmodules:17-19), so each function follows the Marian call site named in its comment
 * and the published behaviour of the intgemm routine that call site invokes (Kernels16 of the
 * SSE2 / AVX2 / AVX512BW back ends: cvtps2dq + packssdw to quantize, pmaddwd + paddd to multiply).
 *
 * Pinning status (tests/test_oracle16.py):
 *   oracle16_quantize      hand vectors (ties to even at the 1/1024 grid, saturation at both ends of
 *                          int16), exactness for multiples of 1/1024, monotonicity            pinned
 *   oracle16_prepare_b     hand-written 2 x 3 matrix (layout n*K + k, tail 1024), numpy        pinned
 *   oracle16_multiply_i32  numpy int64 matmul reduced mod 2^32 (pmaddwd and paddd wrap), extremes
 *                          that overflow int32, Marian's own dot/affine vectors
 *                          (operator_tests.cpp:508-534,618-659): small integers are exact at a
 *                          multiplier of 1024, so the whole 16-bit pipeline must reproduce them    pinned
 *   NaN / Inf inputs (cvtps2dq gives INT_MIN, packssdw then -32768)                     PARITY UNPINNED
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

/* quantMult of every 16-bit intgemm tensor, activations and weights alike:
 * src/tensors/cpu/integer_common.h:174-175. */
float oracle16_quant_mult(void) { return 1024.0f; }

/* intgemm::Int16::PrepareA == Quantize (src/tensors/cpu/intgemm_interface.h:23-27 for a 16-bit
 * vtype): the fp32 product is converted with round-to-nearest-even and packed with signed
 * saturation, so the range is the whole of int16 (the 8-bit kernels alone ban the most negative
 * value).  A product that is NaN or outside int32 converts to INT_MIN and packs to -32768. */
static inline int16_t quantize16_one(float x, float qm) {
  volatile float p = x * qm;
  float v = p;
  if(!(fabsf(v) < 2147483648.0f)) return (int16_t)-32768;
  float r = nearbyintf(v);
  if(r > 32767.0f) r = 32767.0f;
  if(r < -32768.0f) r = -32768.0f;
  return (int16_t)(int)r;
}

void oracle16_quantize(const float* in, int16_t* out, float qm, size_t n) {
  for(size_t i = 0; i < n; ++i) out[i] = quantize16_one(in[i], qm);
}

/* prepareA node for a 16-bit type: Aq holds M*K int16 and the fp32 quantMult behind them
 * (byte offset 2*M*K; src/tensors/cpu/integer_common.h:101-106 with Integer = int16_t). */
void oracle16_prepare_a(const float* A, int16_t* Aq, int64_t M, int64_t K) {
  size_t n = (size_t)M * (size_t)K;
  float qm = oracle16_quant_mult();
  oracle16_quantize(A, Aq, qm, n);
  memcpy(Aq + n, &qm, sizeof(float));
}

/* 16-bit branch of the offline packer, src/tensors/cpu/expression_graph_packable.h:203-235:
 * quantMult 1024, Transpose10, Int16::PrepareA on the transpose, tail behind K*N int16. */
void oracle16_prepare_b(const float* W, int16_t* Bq, int64_t K, int64_t N) {
  size_t n = (size_t)K * (size_t)N;
  float qm = oracle16_quant_mult();
  for(int64_t c = 0; c < N; ++c)
    for(int64_t k = 0; k < K; ++k) Bq[(size_t)c * K + k] = quantize16_one(W[(size_t)k * N + c], qm);
  memcpy(Bq + n, &qm, sizeof(float));
}

/* Kernels16::Multiply: pmaddwd adds two int16 products into an int32 lane, paddd accumulates the
 * lanes; both wrap around, so the result is the exact sum reduced mod 2^32 in whatever order the
 * lanes are added. */
void oracle16_multiply_i32(const int16_t* Aq, const int16_t* Bt, int32_t* acc, int64_t M, int64_t K,
                           int64_t N) {
  for(int64_t m = 0; m < M; ++m)
    for(int64_t n = 0; n < N; ++n) {
      const int16_t* a = Aq + (size_t)m * K;
      const int16_t* b = Bt + (size_t)n * K;
      uint32_t s = 0;
      for(int64_t k = 0; k < K; ++k) s += (uint32_t)((int32_t)a[k] * (int32_t)b[k]);
      acc[(size_t)m * N + n] = (int32_t)s;
    }
}

/* Multiply node, src/tensors/cpu/intgemm_interface.h:60-88 (the callbacks do not depend on the
 * integer width): unquant = fl32(fl32(1 / fl32(aqm * bqm)) * scale);
 * y = fl32(float(acc) * unquant) (+ bias[n]); relu: y > 0 ? y : 0.  acc receives the accumulators. */
void oracle16_affine(const int16_t* Aq, const int16_t* Bq, const float* bias, float* out, int32_t* acc,
                     int64_t M, int64_t K, int64_t N, float scale, int relu) {
  float aqm, bqm;
  memcpy(&aqm, Aq + (size_t)M * K, sizeof(float));
  memcpy(&bqm, Bq + (size_t)K * N, sizeof(float));
  volatile float prod = aqm * bqm;
  volatile float u = 1.0f / prod;
  volatile float unquant = u * scale;
  oracle16_multiply_i32(Aq, Bq, acc, M, K, N);
  for(int64_t m = 0; m < M; ++m)
    for(int64_t n = 0; n < N; ++n) {
      volatile float y = (float)acc[(size_t)m * N + n] * unquant;
      if(bias) y = y + bias[n];
      float r = y;
      if(relu) r = r > 0.0f ? r : 0.0f;
      out[(size_t)m * N + n] = r;
    }
}
