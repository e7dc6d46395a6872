// Host-side check of the C++ wrappers: quantizes a small weight matrix on the GPU, runs
// affineOrDot with bias and ReLU, and compares with a plain CPU restatement written out here
// (max-abs, round-half-even quantize, exact integer dot product, two-step unquantize).
#include <cmath>
#include <cstring>
#include <random>

#include "hip_int8_interface.h"

using namespace marian::hip;

static int8_t q1(float x, float qm) {
  float v = x * qm;
  float r = std::nearbyint(v);
  r = std::fmin(std::fmax(r, -127.f), 127.f);
  return (int8_t)r;
}

int main() {
  const int M = 24, K = 192, N = 72;
  std::mt19937 gen(7);
  std::normal_distribution<float> da(0.f, 1.f), dw(0.f, 0.02f), db(0.f, 0.01f);
  std::vector<float> A(M * K), W(K * N), bias(N), out(M * N), want(M * N);
  for(auto& v : A) v = da(gen);
  for(auto& v : W) v = dw(gen);
  for(auto& v : bias) v = db(gen);

  Backend be(0);
  Tensor a{nullptr, {M, K}, Type::float32}, w{nullptr, {K, N}, Type::float32};
  Tensor aq{nullptr, {M, K}, Type::intgemm8}, bq{nullptr, {K, N}, Type::intgemm8};
  Tensor b{nullptr, {1, N}, Type::float32}, o{nullptr, {M, N}, Type::float32};
  HIP_CHECK(hipMalloc(&a.data, A.size() * 4));
  HIP_CHECK(hipMalloc(&w.data, W.size() * 4));
  HIP_CHECK(hipMalloc(&b.data, bias.size() * 4));
  HIP_CHECK(hipMalloc(&o.data, out.size() * 4));
  HIP_CHECK(hipMalloc(&aq.data, (requiredBytes(aq.shape, aq.type) + 255) / 256 * 256));
  HIP_CHECK(hipMalloc(&bq.data, (requiredBytes(bq.shape, bq.type) + 255) / 256 * 256));
  HIP_CHECK(hipMemcpy(a.data, A.data(), A.size() * 4, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(w.data, W.data(), W.size() * 4, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(b.data, bias.data(), bias.size() * 4, hipMemcpyHostToDevice));

  integer::prepareB(be, w, bq);
  integer::affineOrDot(be, a, aq, bq, &b, o, 1.0f, /*relu=*/true);
  be.synchronize();
  HIP_CHECK(hipMemcpy(out.data(), o.data, out.size() * 4, hipMemcpyDeviceToHost));
  float aqm = integer::getQuantMult(be, aq), bqm = integer::getQuantMult(be, bq);

  float ma = 0.f, mw = 0.f;
  for(float v : A) ma = std::fmax(ma, std::fabs(v));
  for(float v : W) mw = std::fmax(mw, std::fabs(v));
  const float qa = 127.0f / ma, qb = 127.0f / mw;
  volatile float prod = qa * qb;
  volatile float unq = 1.0f / prod;
  int bad = 0;
  for(int m = 0; m < M; ++m)
    for(int n = 0; n < N; ++n) {
      int32_t acc = 0;
      for(int k = 0; k < K; ++k) acc += (int32_t)q1(A[m * K + k], qa) * (int32_t)q1(W[k * N + n], qb);
      volatile float y = (float)acc * unq;
      y = y + bias[n];
      float r = y > 0.f ? y : 0.f;
      if(r != out[m * N + n]) ++bad;
    }
  bool ok = bad == 0 && aqm == qa && bqm == qb;

  // error path: a CPU-tiled weight type must be refused with the reference's message
  bool refused = false;
  try {
    Tensor tiled = bq;
    tiled.type = Type::intgemm8avx512;
    integer::affineOrDot(be, a, aq, tiled, &b, o);
  } catch(const std::runtime_error& e) {
    refused = std::strstr(e.what(), "Unsupported type") != nullptr;
  }
  std::printf("host_check: mismatches %d, quantMult A %s B %s, tiled type refused %s -> %s\n", bad,
              aqm == qa ? "ok" : "BAD", bqm == qb ? "ok" : "BAD", refused ? "yes" : "NO",
              (ok && refused) ? "OK" : "FAILED");
  return (ok && refused) ? 0 : 1;
}
