/*
 * CPU restatement of Marian's intgemm8 affine/dot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker for the HIP path: only tests, the smoke check and the
 * cpu_baseline leg of the benchmark may link or call it.  It is never part of the
 * shipped library and the shipped library never falls back to it.
 *
 * Why a restatement: Marian delegates all arithmetic of this path to the third-party
 * library marian-nmt/intgemm (reference .gitmodules:17-19, pinned commit not recoverable,
 * directory src/3rd_party/intgemm is empty), so the reference implementation cannot be
 * compiled.  Each function below follows the Marian call site named in its comment and the
 * published behaviour of the intgemm routine that call site invokes.
 *
 * Pinning status (what independent evidence each function is checked against in tests/):
 *   oracle_max_abs            brute force + order independence                         pinned
 *   oracle_quant_mult         single IEEE fp32 division, compared with a double divide   pinned
 *   oracle_quantize           hand vectors (ties-to-even, saturation), symmetry,
 *                             monotonicity, never -128                                  pinned
 *   oracle_multiply_i32       numpy int64 matmul, triple loop, Marian's own dot/affine
 *                             vectors (operator_tests.cpp:508-534,618-659) with qm == 1  pinned
 *   oracle_unquantize         closed form in numpy float32, Marian affine vectors        pinned
 *   oracle_prepare_b          numpy restatement of transpose+quantize, layout by hand    pinned
 *   oracle_affine_shortlist   equals column pick of the dense result                     pinned
 *   behaviour for NaN / Inf / maxabs == 0 inputs                                 PARITY UNPINNED
 *     (would need the real intgemm binary; unreachable with finite non-zero inputs)
 *   int16-saturating accumulation of intgemm's SSSE3/AVX2/AVX512BW kernels is deliberately
 *     not reproduced: the target is the exact int32 sum of the AVX512-VNNI kernel, which is
 *     what Marian selects on VNNI hardware (src/tensors/cpu/integer_common.h:113-126).
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off, no fast-math).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#if defined(__x86_64__)
#include <immintrin.h>
#endif

/* ---- A1: src/tensors/cpu/integer_common.h:169-173 (intgemm::MaxAbsolute) ------------- */
float oracle_max_abs(const float* x, size_t n) {
  float m = 0.0f;
  for(size_t i = 0; i < n; ++i) {
    float a = fabsf(x[i]);
    if(a > m) m = a;
  }
  return m;
}

/* quantMult = 127.0f / maxabs, one fp32 division (integer_common.h:173). */
float oracle_quant_mult(float maxabs) {
  volatile float q = 127.0f / maxabs;
  return q;
}

/* ---- A2: src/tensors/cpu/intgemm_interface.h:23-27 (Kernels8::PrepareA == Quantize) ----
 * q = clamp(rne(fl32(x * qm)), -127, 127).  The product is rounded to fp32 before the
 * round-to-nearest-even conversion.  Out-of-int32-range and NaN products follow the x86
 * cvtps2dq "integer indefinite" result (INT_MIN) which the saturating packs and the final
 * max(-127) turn into -127 (unpinned edge case, see header). */
static inline int8_t quantize_one(float x, float qm) {
  volatile float p = x * qm;
  float v = p;
  if(!(fabsf(v) < 2147483648.0f)) return (int8_t)-127;
  float r = nearbyintf(v); /* default rounding mode: ties to even */
  if(r > 127.0f) r = 127.0f;
  if(r < -127.0f) r = -127.0f;
  return (int8_t)(int)r;
}

void oracle_quantize(const float* in, int8_t* out, float qm, size_t n) {
  for(size_t i = 0; i < n; ++i) out[i] = quantize_one(in[i], qm);
}

/* Whole prepareA node: intgemm_interface.h:17-32.  Aq has M*K + 4 bytes; the fp32
 * quantMult is stored at byte offset M*K (integer_common.h:101-106). */
void oracle_prepare_a(const float* A, int8_t* Aq, int64_t M, int64_t K) {
  size_t n = (size_t)M * (size_t)K;
  float qm = oracle_quant_mult(oracle_max_abs(A, n));
  oracle_quantize(A, Aq, qm, n);
  memcpy(Aq + n, &qm, sizeof(float));
}

/* ---- A6: src/tensors/cpu/expression_graph_packable.h:160-201 ---------------------------
 * Offline weight quantizer for Type::intgemm8.  W is fp32 row-major [K x N]; quantMult is
 * taken over the untransposed W (:170); the payload is the quantized transpose, row-major
 * [N x K] (Transpose10 :165-167, Int8::PrepareA on the transpose :192-199), followed by the
 * fp32 quantMult at byte K*N (:201). */
void oracle_prepare_b(const float* W, int8_t* Bq, int64_t K, int64_t N) {
  size_t n = (size_t)K * (size_t)N;
  float qm = oracle_quant_mult(oracle_max_abs(W, n));
  for(int64_t c = 0; c < N; ++c)
    for(int64_t k = 0; k < K; ++k)
      Bq[(size_t)c * K + k] = quantize_one(W[(size_t)k * N + c], qm);
  memcpy(Bq + n, &qm, sizeof(float));
}

/* ---- A4 integer part: intgemm_interface.h:73-87 (Kernels8::Multiply) -------------------
 * acc[m,n] = sum_k Aq[m,k] * Bt[n,k] in exact int32.  Bt is the [N x K] payload. */
void oracle_multiply_i32_scalar(const int8_t* Aq, const int8_t* Bt, int32_t* acc,
                                int64_t M, int64_t K, int64_t N) {
  for(int64_t m = 0; m < M; ++m)
    for(int64_t n = 0; n < N; ++n) {
      int32_t s = 0;
      const int8_t* a = Aq + (size_t)m * K;
      const int8_t* b = Bt + (size_t)n * K;
      for(int64_t k = 0; k < K; ++k) s += (int32_t)a[k] * (int32_t)b[k];
      acc[(size_t)m * N + n] = s;
    }
}

#if defined(__x86_64__)
/* AVX512-VNNI version, same arithmetic as intgemm's VNNI kernel: vpdpbusd on |a| and
 * sign(a)*b, both within [-127,127] so every partial sum is exact in int32. */
__attribute__((target("avx512f,avx512bw,avx512vnni")))
static void multiply_i32_vnni(const int8_t* Aq, const int8_t* Bt, int32_t* acc,
                              int64_t M, int64_t K, int64_t N) {
  const int64_t K64 = K & ~(int64_t)63;
  const __m512i zero = _mm512_setzero_si512();
  for(int64_t m = 0; m < M; ++m) {
    const int8_t* a = Aq + (size_t)m * K;
    int64_t n = 0;
    for(; n + 4 <= N; n += 4) {
      const int8_t* b0 = Bt + (size_t)(n + 0) * K;
      const int8_t* b1 = Bt + (size_t)(n + 1) * K;
      const int8_t* b2 = Bt + (size_t)(n + 2) * K;
      const int8_t* b3 = Bt + (size_t)(n + 3) * K;
      __m512i s0 = zero, s1 = zero, s2 = zero, s3 = zero;
      for(int64_t k = 0; k < K64; k += 64) {
        __m512i av = _mm512_loadu_si512((const void*)(a + k));
        __mmask64 neg = _mm512_movepi8_mask(av);
        __m512i aa = _mm512_abs_epi8(av);
        __m512i v0 = _mm512_loadu_si512((const void*)(b0 + k));
        __m512i v1 = _mm512_loadu_si512((const void*)(b1 + k));
        __m512i v2 = _mm512_loadu_si512((const void*)(b2 + k));
        __m512i v3 = _mm512_loadu_si512((const void*)(b3 + k));
        v0 = _mm512_mask_sub_epi8(v0, neg, zero, v0);
        v1 = _mm512_mask_sub_epi8(v1, neg, zero, v1);
        v2 = _mm512_mask_sub_epi8(v2, neg, zero, v2);
        v3 = _mm512_mask_sub_epi8(v3, neg, zero, v3);
        s0 = _mm512_dpbusd_epi32(s0, aa, v0);
        s1 = _mm512_dpbusd_epi32(s1, aa, v1);
        s2 = _mm512_dpbusd_epi32(s2, aa, v2);
        s3 = _mm512_dpbusd_epi32(s3, aa, v3);
      }
      int32_t r0 = _mm512_reduce_add_epi32(s0), r1 = _mm512_reduce_add_epi32(s1);
      int32_t r2 = _mm512_reduce_add_epi32(s2), r3 = _mm512_reduce_add_epi32(s3);
      for(int64_t k = K64; k < K; ++k) {
        r0 += (int32_t)a[k] * b0[k]; r1 += (int32_t)a[k] * b1[k];
        r2 += (int32_t)a[k] * b2[k]; r3 += (int32_t)a[k] * b3[k];
      }
      int32_t* o = acc + (size_t)m * N + n;
      o[0] = r0; o[1] = r1; o[2] = r2; o[3] = r3;
    }
    for(; n < N; ++n) {
      const int8_t* b = Bt + (size_t)n * K;
      int32_t s = 0;
      for(int64_t k = 0; k < K; ++k) s += (int32_t)a[k] * b[k];
      acc[(size_t)m * N + n] = s;
    }
  }
}
#endif

/* 1 when the VNNI kernel is used by oracle_multiply_i32 on this host. */
int oracle_has_vnni(void) {
#if defined(__x86_64__)
  return __builtin_cpu_supports("avx512vnni") && __builtin_cpu_supports("avx512bw");
#else
  return 0;
#endif
}

void oracle_multiply_i32(const int8_t* Aq, const int8_t* Bt, int32_t* acc,
                         int64_t M, int64_t K, int64_t N) {
#if defined(__x86_64__)
  if(oracle_has_vnni()) {
    multiply_i32_vnni(Aq, Bt, acc, M, K, N);
    return;
  }
#endif
  oracle_multiply_i32_scalar(Aq, Bt, acc, M, K, N);
}

/* unquant_mult exactly as intgemm_interface.h:69-70: two fp32 operations in this order. */
float oracle_unquant_mult(float aqm, float bqm, float scale) {
  volatile float prod = aqm * bqm;
  volatile float u = 1.0f / prod;
  volatile float us = u * scale;
  return us;
}

/* ---- A4 float part + A7: callbacks UnquantizeAndWrite / UnquantizeAndAddBiasAndWrite
 * (intgemm_interface.h:79,86) then the separate in-place ReLU of the CPU graph
 * (src/graph/expression_operators.cpp:721-731, src/functional/operators.h:128).
 * y = fl32(fl32(float(acc)) * unquant) (+ bias[n]); relu: y > 0 ? y : 0. */
void oracle_unquantize(const int32_t* acc, float unquant, const float* bias, int relu,
                       float* out, int64_t M, int64_t N) {
  for(int64_t m = 0; m < M; ++m)
    for(int64_t n = 0; n < N; ++n) {
      volatile float y = (float)acc[(size_t)m * N + n] * unquant;
      if(bias) y = y + bias[n];
      float r = y;
      if(relu) r = r > 0.0f ? r : 0.0f;
      out[(size_t)m * N + n] = r;
    }
}

/* Whole multiply node: intgemm_interface.h:60-88.  Aq and Bq carry their quantMult tails.
 * acc_out may be NULL; when given it receives the int32 accumulators [M x N]. */
void oracle_affine(const int8_t* Aq, const int8_t* Bq, const float* bias, float* out,
                   int32_t* acc_out, int32_t* acc_tmp, int64_t M, int64_t K, int64_t N,
                   float scale, int relu) {
  float aqm, bqm;
  memcpy(&aqm, Aq + (size_t)M * K, sizeof(float));
  memcpy(&bqm, Bq + (size_t)K * N, sizeof(float));
  int32_t* acc = acc_out ? acc_out : acc_tmp;
  oracle_multiply_i32(Aq, Bq, acc, M, K, N);
  oracle_unquantize(acc, oracle_unquant_mult(aqm, bqm, scale), bias, relu, out, M, N);
}

/* ---- A8 (derived): shortlisted output layer.  Reference semantics in fp32:
 * index_select(Wt, 0, idx) and index_select(b, -1, idx) then dot/affine with transB
 * (src/data/shortlist.cpp:62-79, src/layers/output.cpp:335-350).  The int8 form gathers
 * rows idx[j] of the [N x K] payload and bias[idx[j]]; bqm is the full matrix's quantMult.
 * out and acc are [M x n_idx]. */
void oracle_affine_shortlist(const int8_t* Aq, const int8_t* Bq, const float* bias,
                             const uint32_t* idx, int64_t n_idx, float* out, int32_t* acc,
                             int64_t M, int64_t K, int64_t N, float scale, int relu) {
  float aqm, bqm;
  memcpy(&aqm, Aq + (size_t)M * K, sizeof(float));
  memcpy(&bqm, Bq + (size_t)K * N, sizeof(float));
  float unquant = oracle_unquant_mult(aqm, bqm, scale);
  for(int64_t m = 0; m < M; ++m)
    for(int64_t j = 0; j < n_idx; ++j) {
      const int8_t* a = Aq + (size_t)m * K;
      const int8_t* b = Bq + (size_t)idx[j] * K;
      int32_t s = 0;
      for(int64_t k = 0; k < K; ++k) s += (int32_t)a[k] * (int32_t)b[k];
      acc[(size_t)m * n_idx + j] = s;
      volatile float y = (float)s * unquant;
      if(bias) y = y + bias[idx[j]];
      float r = y;
      if(relu) r = r > 0.0f ? r : 0.0f;
      out[(size_t)m * n_idx + j] = r;
    }
}

/* The reference CPU sequence for one affine call, as timed for the CPU baseline:
 * prepareA node (max-abs pass + quantize pass), multiply node with the unquantize(+bias)
 * callback, then the separate ReLU pass.  Aq (M*K+4 bytes) and acc (M*N int32) are caller
 * scratch. */
void oracle_affine_f32(const float* A, const int8_t* Bq, const float* bias, float* out,
                       int8_t* Aq, int32_t* acc, int64_t M, int64_t K, int64_t N,
                       float scale, int relu) {
  oracle_prepare_a(A, Aq, M, K);
  oracle_affine(Aq, Bq, bias, out, acc, NULL, M, K, N, scale, 0);
  if(relu) {
    size_t n = (size_t)M * (size_t)N;
    for(size_t i = 0; i < n; ++i) out[i] = out[i] > 0.0f ? out[i] : 0.0f;
  }
}
