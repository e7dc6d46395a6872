// One decoding step of a transformer-big decoder launched the way Marian's forward tape launches
// it: call after call from a C++ host thread through the wrappers of this directory, no recorded
// graph (reference src/graph/expression_graph.cpp:141-175; layer structure src/models/transformer.h:
// 603-760 at inference, post-processing "dan"; the end of the step src/translator/beam_search.cpp:
// 433-492).  6 layers, d = 1024, ffn = 4096, 16 heads, tied 32000-word output layer, beam 4 x batch
// 32 (128 rows), 20 cached target positions + the new one, 60 source positions with source lengths
// 20 .. 60 behind a mask; random weights (six sets in rotation so that they come from HBM), random
// caches.  Per step: the embedding launch, per layer Wq/Wk/Wv + self-attention with the cache
// append (one launch), Wo, skip + layer norm, the context attention's Wq + context attention (one
// launch), its Wo, skip + layer norm, W1 + ReLU, W2, skip + layer norm, then the output layer and
// log-softmax + beam/batch transposition + n-best (one launch): 58 launches, every affine input's
// abs-max handed over by the kernel that produced it.  Prints one line of JSON with the time per step.
//
//   eager_step [steps] [warm-up steps]
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "hip_int8_interface.h"
#include "hip_ops_interface.h"

using namespace marian::hip;

namespace {

struct Rng {   // xorshift: fast enough for a few hundred MB of test data
  uint64_t s = 0x9E3779B97F4A7C15ull;
  float uniform() {   // [-1, 1)
    s ^= s << 13; s ^= s >> 7; s ^= s << 17;
    return (float)((s >> 40) * (1.0 / 8388608.0) - 1.0);
  }
};

struct Layer {
  Tensor Wq, Wk, Wv, Wo, cWq, cWo, W1, W2;
  Tensor bq, bk, bv, bo, bcq, bco, b1, b2;
  Tensor g1, s1, g2, s2, g3, s3;
};

}  // namespace

int main(int argc, char** argv) {
  const int steps = argc > 1 ? std::atoi(argv[1]) : 200;
  const int warmup = argc > 2 ? std::atoi(argv[2]) : 20;
  const int kSets = 6, L = 6, d = 1024, ffn = 4096, H = 16, V = 32000, beam = 4, batch = 32, M = beam * batch;
  const int T = 21, S = 60, dk = d / H;
  try {
    Backend backend(0);
    TensorAllocator ta(backend, 3ull << 30);   // one slab: nothing moves once the tensors exist
    Rng rng;
    std::vector<float> host;
    auto upload = [&](Tensor& t, const Shape& shape, float scale, float shift = 0.f) {
      ta.allocate(t, shape, Type::float32);
      host.resize(t.elements());
      for(auto& x : host) x = rng.uniform() * scale + shift;
      HIP_CHECK(hipMemcpy(t.data<float>(), host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice));
    };
    auto copyOf = [&](Tensor& dst, const Tensor& src) {
      ta.allocate(dst, src.shape, src.type);
      dst.prepared = src.prepared;
      HIP_CHECK(hipMemcpy(dst.data<int8_t>(), src.data<int8_t>(), requiredBytes(src.shape, src.type), hipMemcpyDeviceToDevice));
    };
    (void)ta.workspace();
    // one quantized matrix per shape, copied for every use: distinct memory is what matters here
    auto quantized = [&](int K, int N) {
      Tensor w, q;
      upload(w, {K, N}, 0.035f);
      ta.allocate(q, {K, N}, Type::intgemm8);
      integer::prepareB(ta, w, q);
      backend.synchronize();
      ta.free(w);
      return q;
    };
    Tensor qdd = quantized(d, d), qdf = quantized(d, ffn), qfd = quantized(ffn, d), qdv = quantized(d, V);
    std::vector<std::vector<Layer>> sets(kSets, std::vector<Layer>(L));
    std::vector<Tensor> Wout(kSets);
    Tensor bd, bf, bv_out, gamma, beta;
    upload(bd, {1, d}, 0.01f);
    upload(bf, {1, ffn}, 0.01f);
    upload(bv_out, {1, V}, 0.01f);
    upload(gamma, {1, d}, 0.1f, 1.0f);
    upload(beta, {1, d}, 0.1f);
    for(int s = 0; s < kSets; ++s) {
      for(auto& ly : sets[s]) {
        for(Tensor* w : {&ly.Wq, &ly.Wk, &ly.Wv, &ly.Wo, &ly.cWq, &ly.cWo}) copyOf(*w, qdd);
        copyOf(ly.W1, qdf);
        copyOf(ly.W2, qfd);
        ly.bq = ly.bk = ly.bv = ly.bo = ly.bcq = ly.bco = ly.b2 = bd;   // (small vectors are shared)
        ly.b1 = bf;
        ly.g1 = ly.g2 = ly.g3 = gamma;
        ly.s1 = ly.s2 = ly.s3 = beta;
      }
      copyOf(Wout[s], qdv);
    }
    // state: embedding table, previous words, position signal, caches, source mask
    Tensor E, words, signal, mask;
    upload(E, {V, d}, 0.02f);
    ta.allocate(words, {M}, Type::uint32);
    {
      std::vector<uint32_t> w(M);
      for(auto& x : w) x = (uint32_t)((rng.uniform() * 0.5f + 0.5f) * (V - 1));
      HIP_CHECK(hipMemcpy(words.data<uint32_t>(), w.data(), w.size() * 4, hipMemcpyHostToDevice));
      std::vector<float> sig;
      SinusoidalPositionEmbeddings(sig, 1, d, T - 1);
      ta.allocate(signal, {1, d}, Type::float32);
      HIP_CHECK(hipMemcpy(signal.data<float>(), sig.data(), sig.size() * 4, hipMemcpyHostToDevice));
      std::vector<float> m((size_t)batch * S);
      for(int b = 0; b < batch; ++b) {
        const int len = 20 + (int)((rng.uniform() * 0.5f + 0.5f) * 40.99f);
        for(int p = 0; p < S; ++p) m[(size_t)b * S + p] = p >= len ? -99999999.0f : 0.0f;
      }
      ta.allocate(mask, {batch, S}, Type::float32);
      HIP_CHECK(hipMemcpy(mask.data<float>(), m.data(), m.size() * 4, hipMemcpyHostToDevice));
    }
    std::vector<Tensor> Kself(L), Vself(L), Kenc(L), Venc(L);
    for(int l = 0; l < L; ++l) {
      upload(Kself[l], {M * H, T, dk}, 1.0f);
      upload(Vself[l], {M * H, T, dk}, 1.0f);
      upload(Kenc[l], {batch * H, S, dk}, 1.0f);
      upload(Venc[l], {batch * H, S, dk}, 1.0f);
    }
    // activations, their quantized forms (the prepareA nodes' tensors) and abs-max slots
    Tensor x[2], o, a, x1, co, ca, x2, f1, f2, logits, scores, keys;
    Tensor xq, oq, x1q, coq, x2q, f1q;
    Tensor xmax, omax, x1max, comax, x2max, f1max;
    for(Tensor* t : {&x[0], &x[1], &o, &a, &x1, &co, &ca, &x2, &f2}) ta.allocate(*t, {M, d}, Type::float32);
    ta.allocate(f1, {M, ffn}, Type::float32);
    ta.allocate(logits, {beam, batch, V}, Type::float32);
    for(Tensor* t : {&xq, &oq, &x1q, &coq, &x2q}) ta.allocate(*t, {M, d}, Type::intgemm8);
    ta.allocate(f1q, {M, ffn}, Type::intgemm8);
    for(Tensor* t : {&xmax, &omax, &x1max, &comax, &x2max, &f1max}) ta.allocate(*t, {MARIAN_HIP_ABSMAX_SLOTS}, Type::float32);
    NthElement nth(ta);
    Backend& be = backend;
    const float embScale = std::sqrt((float)d);

    auto step = [&](int s) {
      auto& W = sets[s % kSets];
      int cur = 0;
      ScaledEmbeddings(be, x[cur], E, words, embScale, &signal, M, &xmax);
      for(auto& ly : W) {
        ProjectedAttention(ta, o, x[cur], xq, {&ly.Wq, &ly.Wk, &ly.Wv}, {&ly.bq, &ly.bk, &ly.bv}, Kself[&ly - &W[0]],
                           Vself[&ly - &W[0]], H, T, nullptr, &xmax, &omax);
        integer::affineOrDot(ta, o, oq, ly.Wo, &ly.bo, a, 1.f, false, nullptr, &omax, nullptr);
        LayerNormalization(be, x1, a, ly.g1, &ly.s1, 1e-6f, &x[cur], &x1max);
        ProjectedAttention(ta, co, x1, x1q, {&ly.cWq}, {&ly.bcq}, Kenc[&ly - &W[0]], Venc[&ly - &W[0]], H, 0, &mask,
                           &x1max, &comax);
        integer::affineOrDot(ta, co, coq, ly.cWo, &ly.bco, ca, 1.f, false, nullptr, &comax, nullptr);
        LayerNormalization(be, x2, ca, ly.g2, &ly.s2, 1e-6f, &x1, &x2max);
        integer::affineOrDot(ta, x2, x2q, ly.W1, &ly.b1, f1, 1.f, true, nullptr, &x2max, &f1max);
        integer::affineOrDot(ta, f1, f1q, ly.W2, &ly.b2, f2, 1.f, false, nullptr, &f1max, nullptr);
        LayerNormalization(be, x[1 - cur], f2, ly.g3, &ly.s3, 1e-6f, &x2, &xmax);
        cur = 1 - cur;
      }
      Tensor flat = logits;
      flat.shape = {M, V};
      integer::affineOrDot(ta, x[cur], xq, Wout[s % kSets], &bv_out, flat, 1.f, false, nullptr, &xmax, nullptr);
      nth.logSoftmaxNBestOfBeams(logits, nullptr, beam, scores, keys);
    };
    for(int i = 0; i < warmup; ++i) step(i);
    backend.synchronize();
    const auto t0 = std::chrono::steady_clock::now();
    for(int i = 0; i < steps; ++i) step(i);
    backend.synchronize();
    const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / steps;
    // a check that the step computed something: finite scores, keys inside beam * vocab per sentence
    std::vector<float> sc(scores.elements());
    std::vector<uint32_t> ky(keys.elements());
    HIP_CHECK(hipMemcpy(sc.data(), scores.data<float>(), sc.size() * 4, hipMemcpyDeviceToHost));
    HIP_CHECK(hipMemcpy(ky.data(), keys.data<uint32_t>(), ky.size() * 4, hipMemcpyDeviceToHost));
    bool sane = true;
    for(size_t i = 0; i < sc.size(); ++i) {
      const size_t sentence = i / beam;
      sane = sane && std::isfinite(sc[i]) && sc[i] <= 0.f && ky[i] / ((uint32_t)beam * V) == sentence;
    }
    std::printf("{\"eager_ms_per_step_cpp_host\": %.5f, \"steps\": %d, \"launches_per_step\": %d, \"nbest_sane\": %s}\n", ms,
                steps, 4 + 9 * L, sane ? "true" : "false");
    return sane ? 0 : 2;
  } catch(const std::exception& e) {
    std::fprintf(stderr, "eager_step: %s\n", e.what());
    return 1;
  }
}
