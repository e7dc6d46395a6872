// The transformer-base decode GEMM sweep launched the way Marian's forward tape launches it: one
// call after the other from a C++ host thread, no recorded graph (reference
// src/graph/expression_graph.cpp:141-175: forward() runs the nodes of the tape in order, each
// node's functor enqueues its kernels).  Twenty affineOrDot calls per pass - M in {1, 4, 16, 64}
// times {512x1536, 512x512, 512x2048, 2048x512, 512x32000}, float32 in, float32 out, bias - through
// host/hip_int8_interface.h on tensors carved from one allocator; eight rotating sets of weights
// so that they come from HBM.  Prints one line of JSON with the time per pass.
//
//   eager_sweep [passes] [warm-up passes]
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "hip_int8_interface.h"

using namespace marian::hip;

int main(int argc, char** argv) {
  const int passes = argc > 1 ? std::atoi(argv[1]) : 200;
  const int warmup = argc > 2 ? std::atoi(argv[2]) : 20;
  const int kSets = 8;
  try {
    Backend backend(0);
    TensorAllocator ta(backend, 256ull << 20);
    const int Ms[] = {1, 4, 16, 64};
    const int KN[][2] = {{512, 1536}, {512, 512}, {512, 2048}, {2048, 512}, {512, 32000}};
    struct Call {
      Tensor a, aQuant, bias, out;
      std::vector<Tensor> bQuant;
    };
    std::vector<Call> calls;
    std::mt19937 rng(1234);
    std::normal_distribution<float> unit(0.f, 1.f);
    auto upload = [&](Tensor& t, const Shape& shape, float sigma) {
      ta.allocate(t, shape, Type::float32);
      std::vector<float> h(t.elements());
      for(auto& x : h) x = unit(rng) * sigma;
      HIP_CHECK(hipMemcpy(t.data<float>(), h.data(), h.size() * sizeof(float), hipMemcpyHostToDevice));
    };
    // (every tensor is allocated before the first pointer is used: the slab may move while it grows)
    double ops = 0;
    for(auto& kn : KN)
      for(int M : Ms) {
        Call c;
        const int K = kn[0], N = kn[1];
        upload(c.a, {M, K}, 1.0f);
        upload(c.bias, {1, N}, 0.01f);
        ta.allocate(c.aQuant, {M, K}, Type::intgemm8);
        ta.allocate(c.out, {M, N}, Type::float32);
        Tensor w;
        upload(w, {K, N}, 0.02f);
        c.bQuant.resize(kSets);
        for(int s = 0; s < kSets; ++s) {
          ta.allocate(c.bQuant[s], {K, N}, Type::intgemm8);
          integer::prepareB(ta, w, c.bQuant[s]);
        }
        backend.synchronize();
        ta.free(w);
        ops += 2.0 * M * K * N;
        calls.push_back(std::move(c));
      }
    (void)ta.workspace();
    auto pass = [&](int p) {
      for(auto& c : calls) integer::affineOrDot(ta, c.a, c.aQuant, c.bQuant[p % kSets], &c.bias, c.out);
    };
    for(int p = 0; p < warmup; ++p) pass(p);
    backend.synchronize();
    const auto t0 = std::chrono::steady_clock::now();
    for(int p = 0; p < passes; ++p) pass(p);
    backend.synchronize();
    const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / passes;
    std::printf("{\"eager_ms_per_pass_cpp_host\": %.5f, \"tops\": %.3f, \"passes\": %d, \"calls_per_pass\": %d}\n", ms,
                ops / (ms * 1e-3) / 1e12, passes, (int)calls.size());
  } catch(const std::exception& e) {
    std::fprintf(stderr, "eager_sweep: %s\n", e.what());
    return 1;
  }
  return 0;
}
