// Check program for the C++ host side: Device / Allocator / TensorAllocator and the operator
// wrappers, on the GPU, against expected values computed elsewhere.
//
//   host_check <fixture file>
//
// The fixture (written by the test that runs this program) holds the inputs and, for every step,
// the values the CPU checker of the test suite computed from them; nothing is recomputed here.
// Every buffer - inputs, quantized operands, outputs, the abs-max workspace - is carved from one
// allocator whose slab is forced to grow, i.e. to MOVE, between prepareA and multiply, between two
// affineOrDot calls and in the middle of a chained pair, so the "nothing is retained between
// calls" contract of the library is exercised, not assumed.
//
// Fixture layout (little endian): "MHC3", int32 M, K, N, N2, nIdx, R, C, nbestN; then
//   float A[M*K], W[K*N], bias[N], W2[N*N2]; uint32 idx[nIdx];
//   int8 Aq[M*K+4], Bq[K*N+4], Bq2[N*N2+4] (weights in the order the kernels read), fileBq[K*N+4] (the same
//   values as a model file holds them, rows [N, K]); int32 acc[M*N];
//   float outRelu[M*N]      affine(A, W, bias), ReLU, scale 1
//   float outSl[M*nIdx]     affine over the shortlist idx, no ReLU, scale 0.5
//   float out2[M*N2]        affine(outRelu, W2), no bias
//   float X[R*C], gamma[C], beta[C], ln[R*C] (eps 1e-6, skip input = X reversed), sm[R*C], lsm[R*C];
//   float nbVal[R*nbestN]; uint32 nbKey[R*nbestN]     n-best of lsm
//   int16 Aq16[M*K+2], Bq16[K*N+2]; float out16[M*N]  the 16-bit path: affine(A, W, bias), ReLU, scale 1
#include <cmath>
#include <cstring>
#include <fstream>

#include "hip_int8_interface.h"
#include "hip_ops_interface.h"

using namespace marian::hip;

namespace {

struct Reader {
  std::ifstream in;
  explicit Reader(const char* path) : in(path, std::ios::binary) {
    if(!in) abortWith(std::string("cannot open fixture ") + path);
  }
  template <typename T>
  std::vector<T> take(size_t n) {
    std::vector<T> v(n);
    in.read(reinterpret_cast<char*>(v.data()), (std::streamsize)(n * sizeof(T)));
    if(!in) abortWith("fixture is too short");
    return v;
  }
};

int failures = 0;
void expect(bool ok, const char* what) {
  std::printf("  %-74s %s\n", what, ok ? "ok" : "FAILED");
  std::fflush(stdout);
  if(!ok) ++failures;
}

template <typename T>
Tensor upload(TensorAllocator& ta, const std::vector<T>& host, const Shape& shape, Type type) {
  Tensor t;
  ta.allocate(t, shape, type);
  copy(ta.backend().stream(), reinterpret_cast<const uint8_t*>(host.data()),
       reinterpret_cast<const uint8_t*>(host.data()) + host.size() * sizeof(T), t.data<uint8_t>());
  return t;
}

template <typename T>
std::vector<T> download(Backend& be, const Tensor& t, size_t n) {
  std::vector<T> host(n);
  be.synchronize();
  copy(be.stream(), t.data<T>(), t.data<T>() + n, host.data());
  return host;
}

template <typename T>
bool sameBits(const std::vector<T>& a, const std::vector<T>& b) {
  return a.size() == b.size() && std::memcmp(a.data(), b.data(), a.size() * sizeof(T)) == 0;
}

bool closeTo(const std::vector<float>& got, const std::vector<float>& want, double rel, double floor) {
  if(got.size() != want.size()) return false;
  for(size_t i = 0; i < got.size(); ++i)
    if(!(std::fabs((double)got[i] - (double)want[i]) <= rel * std::fabs((double)want[i]) + floor)) return false;
  return true;
}

// Allocates `bytes` more than the slab has free, so that the allocator must grow; returns whether
// the slab moved.
bool forceMove(TensorAllocator& ta, std::vector<Tensor>& ballast) {
  const size_t before = ta.allocator()->device()->moves();
  const uint8_t* base = ta.allocator()->device()->data();
  Tensor t;
  ta.allocate(t, {(int)(ta.allocator()->available() + 4096)}, Type::int8);
  ballast.push_back(t);
  return ta.allocator()->device()->moves() > before && ta.allocator()->device()->data() != base;
}

}  // namespace

int main(int argc, char** argv) {
  if(argc < 2) {
    std::fprintf(stderr, "usage: host_check <fixture file>\n");
    return 2;
  }
  try {
    Reader rd(argv[1]);
    auto magic = rd.take<char>(4);
    if(std::memcmp(magic.data(), "MHC3", 4) != 0) abortWith("not a host_check fixture");
    auto dims = rd.take<int32_t>(8);
    const int M = dims[0], K = dims[1], N = dims[2], N2 = dims[3], nIdx = dims[4], R = dims[5], C = dims[6],
              nbestN = dims[7];
    auto A = rd.take<float>((size_t)M * K), W = rd.take<float>((size_t)K * N), bias = rd.take<float>(N),
         W2 = rd.take<float>((size_t)N * N2);
    auto idx = rd.take<uint32_t>(nIdx);
    auto wantAq = rd.take<int8_t>((size_t)M * K + 4), wantBq = rd.take<int8_t>((size_t)K * N + 4),
         wantBq2 = rd.take<int8_t>((size_t)N * N2 + 4);
    auto fileBq = rd.take<int8_t>((size_t)K * N + 4);
    auto wantAcc = rd.take<int32_t>((size_t)M * N);
    auto wantRelu = rd.take<float>((size_t)M * N), wantSl = rd.take<float>((size_t)M * nIdx),
         want2 = rd.take<float>((size_t)M * N2);
    auto X = rd.take<float>((size_t)R * C), gamma = rd.take<float>(C), beta = rd.take<float>(C),
         wantLn = rd.take<float>((size_t)R * C), wantSm = rd.take<float>((size_t)R * C),
         wantLsm = rd.take<float>((size_t)R * C);
    auto wantNbVal = rd.take<float>((size_t)R * nbestN);
    auto wantNbKey = rd.take<uint32_t>((size_t)R * nbestN);
    auto wantAq16 = rd.take<int16_t>((size_t)M * K + 2), wantBq16 = rd.take<int16_t>((size_t)K * N + 2);
    auto wantOut16 = rd.take<float>((size_t)M * N);

    Backend be(0);
    // a small step and a limit: growth happens often, and exhaustion can be provoked
    const size_t kStep = 1u << 20, kLimit = 256u << 20;
    TensorAllocator ta(be, kStep, kLimit);
    std::vector<Tensor> ballast;
    std::printf("host_check: M=%d K=%d N=%d N2=%d shortlist=%d, operators on %dx%d\n", M, K, N, N2, nIdx, R, C);

    // ---- allocator on its own ----
    {
      Allocator& al = *ta.allocator();
      expect(al.size() == 0 && al.available() == 0, "empty allocator: no slab yet");
      auto p1 = al.alloc(100), p2 = al.alloc(256), p3 = al.alloc(257);
      expect(al.size() == kStep && p1->size() == 256 && p2->size() == 256 && p3->size() == 512,
             "first allocation grows the slab by one step; sizes round up to 256");
      expect(((uintptr_t)p1->data() % 256) == 0 && p2->data() == p1->data() + 256 && p3->data() == p2->data() + 256,
             "pieces are 256-byte aligned and packed");
      expect(al.available() == kStep - 1024 && al.gaps() == 1, "one gap behind the pieces");
      al.free(p2);
      expect(al.gaps() == 2 && !p2->data(), "free leaves a gap and empties the handle");
      auto p4 = al.alloc(200);
      expect(p4->data() == p1->data() + 256 && al.gaps() == 1, "best fit: the freed 256 bytes are taken again");
      al.free(p1);
      al.free(p4);
      expect(al.gaps() == 2, "neighbouring gaps merge (front)");
      al.free(p3);
      expect(al.gaps() == 1 && al.available() == al.size(), "all free: one gap, the whole slab");
      auto q1 = al.alloc(1000);
      const uint8_t* before = q1->data();
      fill(be.stream(), q1->data<uint8_t>(), q1->data<uint8_t>() + 1000, (uint8_t)0x5A);
      auto q2 = al.alloc(kStep);   // does not fit: grow = new slab + copy + free
      std::vector<uint8_t> back(1000);
      copy(be.stream(), (const uint8_t*)q1->data(), (const uint8_t*)q1->data() + 1000, back.data());
      bool kept = true;
      for(uint8_t b : back) kept = kept && b == 0x5A;
      expect(al.device()->moves() == 1 && q1->data() != before && kept,
             "grow moves the slab, re-points the pieces, keeps their bytes");
      expect(al.size() == 2 * kStep && q2->size() == kStep, "grow adds max(step, request)");
      al.throwAtReallocation(true);
      bool threw = false;
      try {
        al.alloc(64u << 20);
      } catch(const AllocationException&) {
        threw = true;
      }
      al.throwAtReallocation(false);
      expect(threw, "throwAtReallocation: AllocationException instead of growing");
      bool refused = false;
      try {
        al.alloc(kLimit + 1);
      } catch(const std::runtime_error& e) {
        refused = std::strstr(e.what(), "Out of memory") != nullptr;
      }
      copy(be.stream(), (const uint8_t*)q1->data(), (const uint8_t*)q1->data() + 1000, back.data());
      expect(refused && back[999] == 0x5A && al.size() == 2 * kStep,
             "exhaustion is an error; slab and pieces survive it");
      ta.clear();
      expect(al.available() == al.size() && al.pieces() == 0 && !q1->data(), "clear forgets every piece");
    }

    // ---- fill and copy ----
    {
      Tensor f;
      ta.allocate(f, {1031}, Type::float32);
      fill(be.stream(), f.data<float>(), f.data<float>() + 1031, -1.0f);
      fill(be.stream(), f.data<float>() + 3, f.data<float>() + 1030, 1.5f);   // unaligned start, ragged end
      auto got = download<float>(be, f, 1031);
      bool ok = got[0] == -1.0f && got[2] == -1.0f && got[1030] == -1.0f;
      for(int i = 3; i < 1030; ++i) ok = ok && got[i] == 1.5f;
      fill(be.stream(), f.data<int8_t>() + 1, f.data<int8_t>() + 38, (int8_t)-7);
      fill(be.stream(), reinterpret_cast<uint16_t*>(f.data<int8_t>() + 40), reinterpret_cast<uint16_t*>(f.data<int8_t>() + 40) + 9, (uint16_t)0xBEEF);
      fill(be.stream(), reinterpret_cast<uint64_t*>(f.data<int8_t>() + 64), reinterpret_cast<uint64_t*>(f.data<int8_t>() + 64) + 5, (uint64_t)0x0123456789ABCDEFull);
      auto raw = download<uint8_t>(be, f, 128);
      for(int i = 1; i < 38; ++i) ok = ok && raw[i] == (uint8_t)-7;
      ok = ok && raw[0] == 0x00 && raw[38] == 0xC0;   // the bytes on either side (of -1.0f, of 1.5f) are untouched
      for(int i = 0; i < 9; ++i) ok = ok && raw[40 + 2 * i] == 0xEF && raw[41 + 2 * i] == 0xBE;
      for(int i = 0; i < 5; ++i) ok = ok && raw[64 + 8 * i] == 0xEF && raw[71 + 8 * i] == 0x01;
      expect(ok, "fill: 1-, 2-, 4- and 8-byte elements, unaligned starts, ragged ends");
      ta.free(f);
    }

    // ---- the int8 path, with the slab moving between the calls ----
    Tensor a = upload(ta, A, {M, K}, Type::float32), w = upload(ta, W, {K, N}, Type::float32);
    Tensor b = upload(ta, bias, {1, N}, Type::float32), w2 = upload(ta, W2, {N, N2}, Type::float32);
    Tensor sl = upload(ta, idx, {nIdx}, Type::uint32);
    Tensor aq, bq, bq2, acc, o, oSl, o2, aq2, omax;
    ta.allocate(aq, {M, K}, Type::intgemm8);
    ta.allocate(bq, {K, N}, Type::intgemm8);
    ta.allocate(bq2, {N, N2}, Type::intgemm8);
    ta.allocate(acc, {M, N}, Type::int32);
    ta.allocate(o, {M, N}, Type::float32);
    ta.allocate(oSl, {M, nIdx}, Type::float32);
    ta.allocate(o2, {M, N2}, Type::float32);
    ta.allocate(aq2, {M, N}, Type::intgemm8);
    ta.allocate(omax, {MARIAN_HIP_ABSMAX_SLOTS}, Type::float32);

    integer::prepareB(ta, w, bq);
    integer::prepareB(ta, w2, bq2);
    expect(sameBits(download<int8_t>(be, bq, wantBq.size()), wantBq) &&
               sameBits(download<int8_t>(be, bq2, wantBq2.size()), wantBq2),
           "prepareB: the checker's values and quantMult, in the order the kernels read");
    {
      Tensor fromFile = upload(ta, fileBq, {K, N}, Type::intgemm8), retiled;
      ta.allocate(retiled, {K, N}, Type::intgemm8);
      integer::prepareAndTransposeB(be, fromFile, retiled);
      expect(sameBits(download<int8_t>(be, retiled, wantBq.size()), wantBq),
             "prepareAndTransposeB: a model file's rows [N, K] re-tiled to the same bytes as prepareB");
      ta.free(retiled);
      ta.free(fromFile);
    }
    integer::prepareA(ta, a, aq);
    const void* aqBefore = aq.data<void>();
    expect(forceMove(ta, ballast) && aq.data<void>() != aqBefore, "slab moved between prepareA and multiply");
    expect(sameBits(download<int8_t>(be, aq, wantAq.size()), wantAq), "prepareA: payload and quantMult, after the move");
    integer::multiplyInt32(be, aq, bq, acc);
    integer::multiply(be, aq, bq, &b, o, 1.0f, /*relu=*/true);
    expect(sameBits(download<int32_t>(be, acc, wantAcc.size()), wantAcc), "multiply: int32 accumulators");
    expect(sameBits(download<float>(be, o, wantRelu.size()), wantRelu), "multiply: bias + ReLU output, bit for bit");
    float aqm = integer::getQuantMult(be, aq), wantAqm;
    std::memcpy(&wantAqm, wantAq.data() + (size_t)M * K, 4);
    expect(aqm == wantAqm, "getQuantMult reads the tail on the device");

    fill(be.stream(), o.data<float>(), o.data<float>() + (size_t)M * N, 0.0f);
    integer::affineOrDot(ta, a, aq, bq, &b, o, 1.0f, /*relu=*/true);
    expect(sameBits(download<float>(be, o, wantRelu.size()), wantRelu), "affineOrDot: bias + ReLU output");
    expect(forceMove(ta, ballast), "slab moved between two affineOrDot calls");
    integer::affineOrDot(ta, a, aq, bq, &b, oSl, 0.5f, /*relu=*/false, &sl);
    expect(sameBits(download<float>(be, oSl, wantSl.size()), wantSl), "affineOrDot over a shortlist, scale 0.5");
    integer::multiply(be, aq, bq, &b, oSl, 0.5f, false, &sl);
    expect(sameBits(download<float>(be, oSl, wantSl.size()), wantSl), "multiply over a shortlist");

    // chained pair: the first call leaves the abs-max of its output, the second one takes it
    integer::affineOrDot(ta, a, aq, bq, &b, o, 1.0f, true, nullptr, nullptr, &omax);
    expect(forceMove(ta, ballast), "slab moved inside a chained pair");
    integer::affineOrDot(ta, o, aq2, bq2, nullptr, o2, 1.0f, false, nullptr, &omax, nullptr);
    expect(sameBits(download<float>(be, o2, want2.size()), want2), "chained affineOrDot (abs-max handed over)");
    {   // two matrices behind one input in one call: the outputs of the separate calls
      Tensor g1, g2;
      ta.allocate(g1, {M, N}, Type::float32);
      ta.allocate(g2, {M, N}, Type::float32);
      integer::affineOrDotGrouped(ta, a, aq, {&bq, &bq}, {&b, nullptr}, {&g1, &g2}, 1.0f, true);
      integer::multiply(be, aq, bq, nullptr, o, 1.0f, true);
      expect(sameBits(download<float>(be, g1, wantRelu.size()), wantRelu) &&
                 sameBits(download<float>(be, g2, wantRelu.size()), download<float>(be, o, wantRelu.size())),
             "affineOrDotGrouped: both outputs as the separate calls'");
    }

    // ---- the binding on a forward tape in inference mode (graph::affineOrDot) ----
    {
      const size_t nA = (size_t)M * K;
      auto copyFwd = [&be, nA](graph::Expr out, const std::vector<graph::Expr>& in) {
        copy(be.stream(), in[0]->val.data<float>(), in[0]->val.data<float>() + nA, out->val.data<float>());
      };
      // after every node, whatever the tape has given back is overwritten (0xFF bytes: NaN as floats)
      auto spoil = [&](const graph::Node&) {
        be.synchronize();
        uint8_t* base = ta.allocator()->device()->data();
        ta.allocator()->forEachGap([&](size_t offset, size_t size) {
          fill(be.stream(), base + offset, base + offset + size, (uint8_t)0xFF);
        });
      };
      for(int form = 0; form < 2; ++form) {
        graph::ExpressionGraph g(ta, /*inferenceOnly=*/true);
        graph::Expr x = g.param(a), wq = g.param(bq), bb = g.param(b);
        // the activations are a node of the tape (a copy of the input): the tape owns and frees them
        graph::Expr act = g.lambda({x}, a.shape, Type::float32, copyFwd);
        std::weak_ptr<graph::Node> actAlive = act;
        graph::Expr y = form == 0 ? graph::affineOrDot(g, act, wq, bb, false, false, 1.0f, /*relu=*/true)
                                  : graph::affineOrDotTwoNodes(g, act, wq, bb, 1.0f, /*relu=*/true);
        act.reset();   // from here on only nodes hold the input, as in a model's forward pass
        g.forward(spoil);
        expect(sameBits(download<float>(be, y->val, wantRelu.size()), wantRelu),
               form == 0 ? "tape, inference mode: one-call binding (input a direct child of node 2), freed memory overwritten"
                         : "tape, inference mode: two real nodes as in the reference, freed memory overwritten");
        expect(actAlive.expired(), "the input is given back once the last node that reads it has run");
      }
      {   // why the one-call form needs the input as a direct child of node 2
        graph::ExpressionGraph g(ta, true);
        graph::Expr x = g.param(a), wq = g.param(bq), bb = g.param(b);
        graph::Expr act = g.lambda({x}, a.shape, Type::float32, copyFwd);
        std::weak_ptr<graph::Node> actAlive = act;
        graph::Expr n1 = g.lambda({act}, a.shape, Type::intgemm8, [](graph::Expr, const std::vector<graph::Expr>&) {});
        bool goneBeforeNode2 = false;
        graph::Expr n2 = g.lambda({n1, wq, bb}, Shape{M, N}, Type::float32,
                                  [&](graph::Expr, const std::vector<graph::Expr>&) { goneBeforeNode2 = actAlive.expired(); });
        act.reset();
        g.forward();
        expect(goneBeforeNode2, "an input held only through node 1 is freed before node 2 runs");
      }
    }
    Tensor oStatic;
    ta.allocate(oStatic, {M, N}, Type::float32);
    integer::affineOrDotStatic(be, a, bq, &b, oStatic, 1.0f, true);
    expect(sameBits(download<float>(be, oStatic, wantRelu.size()), wantRelu), "affineOrDotStatic (no Aq, no workspace)");

    {   // the 16-bit path (Type::intgemm16) through the same wrappers, selected by the tensor types
      Tensor aq16, bq16, o16;
      ta.allocate(aq16, {M, K}, Type::intgemm16);
      ta.allocate(bq16, {K, N}, Type::intgemm16);
      ta.allocate(o16, {M, N}, Type::float32);
      integer::prepareB(ta, w, bq16);
      integer::affineOrDot(ta, a, aq16, bq16, &b, o16, 1.0f, /*relu=*/true);
      expect(sameBits(download<int16_t>(be, bq16, wantBq16.size()), wantBq16) &&
                 sameBits(download<int16_t>(be, aq16, wantAq16.size()), wantAq16),
             "intgemm16: prepareB and prepareA, payload and quantMult 1024");
      expect(sameBits(download<float>(be, o16, wantOut16.size()), wantOut16), "intgemm16: affineOrDot, bit for bit");
      expect(integer::getQuantMult(be, aq16) == 1024.0f && integer::getQuantMult(be, bq16) == 1024.0f,
             "intgemm16: getQuantMult reads the tail behind 2 * elements bytes");
    }

    // error paths: the reference's messages, as exceptions
    {
      bool tiled = false, sixteen = false, notq = false;
      Tensor t = bq;
      t.type = Type::intgemm8avx512;
      try { integer::affineOrDot(ta, a, aq, t, &b, o); } catch(const std::runtime_error& e) { tiled = std::strstr(e.what(), "Unsupported type") != nullptr; }
      t.type = Type::intgemm16avx2;
      try { integer::affineOrDot(ta, a, aq, t, &b, o); } catch(const std::runtime_error& e) { sixteen = std::strstr(e.what(), "Unsupported type") != nullptr; }
      t.type = Type::float32;
      try { integer::affineOrDot(ta, a, aq, t, &b, o); } catch(const std::runtime_error& e) { notq = std::strstr(e.what(), "variant of intgemm") != nullptr; }
      expect(tiled && sixteen && notq, "CPU-tiled 8- and 16-bit and float weights are refused with the reference's texts");
      bool fileOrder = false;
      t = bq;
      t.prepared = false;   // as uploaded from a model file
      try { integer::affineOrDot(ta, a, aq, t, &b, o); } catch(const std::runtime_error& e) { fileOrder = std::strstr(e.what(), "prepareAndTransposeB") != nullptr; }
      expect(fileOrder, "8-bit weights in file order are refused until they have been re-tiled");
    }

    // ---- float operators through their wrappers ----
    {
      std::vector<float> Xrev(X.rbegin(), X.rend());
      Tensor x = upload(ta, X, {R, C}, Type::float32), xr = upload(ta, Xrev, {R, C}, Type::float32);
      Tensor g = upload(ta, gamma, {C}, Type::float32), bt = upload(ta, beta, {C}, Type::float32);
      Tensor ln, sm, lsm, nbV, nbK, nbV2, nbK2;
      ta.allocate(ln, {R, C}, Type::float32);
      ta.allocate(sm, {R, C}, Type::float32);
      ta.allocate(lsm, {R, C}, Type::float32);
      LayerNormalization(be, ln, x, g, &bt, 1e-6f, &xr);
      Softmax(be, sm, x);
      LogSoftmax(be, lsm, x);
      expect(closeTo(download<float>(be, ln, wantLn.size()), wantLn, 2e-5, 4e-6), "LayerNormalization with skip input");
      expect(closeTo(download<float>(be, sm, wantSm.size()), wantSm, 2e-5, 1e-7), "Softmax");
      expect(closeTo(download<float>(be, lsm, wantLsm.size()), wantLsm, 2e-5, 4e-6), "LogSoftmax");
      // n-best of the checker's log-probabilities (so that equal inputs decide, not rounding)
      Tensor lsmRef = upload(ta, wantLsm, {R, C}, Type::float32);
      NthElement nth(ta);
      nth.getNBestList(lsmRef, nbestN, nbV, nbK);
      expect(sameBits(download<float>(be, nbV, wantNbVal.size()), wantNbVal) &&
                 sameBits(download<uint32_t>(be, nbK, wantNbKey.size()), wantNbKey),
             "NthElement::getNBestList: scores and keys");
      Tensor asBeams = lsmRef;   // the same rows seen as [beam 1, batch R, vocab C]
      asBeams.shape = {1, R, C};
      nth.getNBestListOfBeams(asBeams, nbestN, nbV2, nbK2);
      expect(sameBits(download<float>(be, nbV2, wantNbVal.size()), wantNbVal) &&
                 sameBits(download<uint32_t>(be, nbK2, wantNbKey.size()), wantNbKey),
             "NthElement::getNBestListOfBeams: the same list");
      // the fused end of a step against the separate calls on the same logits
      Tensor xb = x, lsmGpu = lsm, fusedV, fusedK, sepV, sepK, fusedLp;
      xb.shape = {1, R, C};
      lsmGpu.shape = {1, R, C};
      nth.getNBestListOfBeams(lsmGpu, nbestN, sepV, sepK);
      nth.logSoftmaxNBestOfBeams(xb, nullptr, nbestN, fusedV, fusedK, &fusedLp);
      expect(sameBits(download<float>(be, fusedV, (size_t)R * nbestN), download<float>(be, sepV, (size_t)R * nbestN)) &&
                 sameBits(download<uint32_t>(be, fusedK, (size_t)R * nbestN), download<uint32_t>(be, sepK, (size_t)R * nbestN)) &&
                 sameBits(download<float>(be, fusedLp, (size_t)R * C), download<float>(be, lsm, (size_t)R * C)),
             "NthElement::logSoftmaxNBestOfBeams (short rows: the separate calls inside), bit for bit");
      // rows long enough for the one-launch form: 2 beam entries x 3 sentences x 4100 words
      const int kBeam = 2, kBatch = 3, kVocab = 4100;
      std::vector<float> logits((size_t)kBeam * kBatch * kVocab), path((size_t)kBeam * kBatch);
      uint32_t rng = 12345u;
      for(auto& v : logits) { rng = rng * 1664525u + 1013904223u; v = (float)(rng >> 8) * (1.0f / 1048576.0f) - 8.0f; }
      for(size_t i = 0; i < path.size(); ++i) path[i] = -0.75f * (float)i;
      logits[5] = logits[kVocab + 77] = logits[3 * kVocab + 9] = 9.5f;   // equal scores across rows
      Tensor lg = upload(ta, logits, {kBeam, kBatch, kVocab}, Type::float32), ps = upload(ta, path, {kBeam, kBatch}, Type::float32);
      Tensor oneV, oneK, oneLp, twoLp, twoV, twoK;
      nth.logSoftmaxNBestOfBeams(lg, &ps, nbestN, oneV, oneK, &oneLp);
      ta.allocate(twoLp, {kBeam * kBatch, kVocab}, Type::float32);
      Tensor rowsIn = lg;
      rowsIn.shape = {kBeam * kBatch, kVocab};
      LogSoftmax(be, twoLp, rowsIn);
      std::vector<float> lpHost = download<float>(be, twoLp, logits.size());
      expect(sameBits(download<float>(be, oneLp, logits.size()), lpHost), "one-launch form: the log-probabilities of LogSoftmax");
      for(size_t r = 0; r < path.size(); ++r)
        for(int c = 0; c < kVocab; ++c) lpHost[r * kVocab + c] = lpHost[r * kVocab + c] + path[r];
      Tensor scored = upload(ta, lpHost, {kBeam, kBatch, kVocab}, Type::float32);
      nth.getNBestListOfBeams(scored, nbestN, twoV, twoK);
      expect(sameBits(download<float>(be, oneV, (size_t)kBatch * nbestN), download<float>(be, twoV, (size_t)kBatch * nbestN)) &&
                 sameBits(download<uint32_t>(be, oneK, (size_t)kBatch * nbestN), download<uint32_t>(be, twoK, (size_t)kBatch * nbestN)),
             "one-launch form with path scores: the n-best of LogSoftmax + path score, bit for bit");
    }
    // ---- the embedding step: rows of a table (the reference's own vectors for rows(),
    // src/tests/units/operator_tests.cpp:773-826), then scale and position signal ----
    {
      const std::vector<float> table{1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12};
      const std::vector<uint32_t> picks{2, 1, 1, 0, 3};
      const std::vector<float> wantRows{7, 8, 9, 4, 5, 6, 4, 5, 6, 1, 2, 3, 10, 11, 12};
      Tensor tb = upload(ta, table, {4, 3}, Type::float32), ix = upload(ta, picks, {(int)picks.size()}, Type::uint32);
      Tensor got;
      ta.allocate(got, {(int)picks.size(), 3}, Type::float32);
      CopyRows(be, got, tb, ix);
      expect(sameBits(download<float>(be, got, wantRows.size()), wantRows), "CopyRows: the reference's rows() vectors");
      const int dE = 8, nWords = 6, perSignal = 3;
      std::vector<float> emb((size_t)5 * dE), signal;
      for(size_t i = 0; i < emb.size(); ++i) emb[i] = 0.013f * (float)((int)(i * 7 % 23) - 11);
      SinusoidalPositionEmbeddings(signal, 2, dE, 4);
      expect(signal.size() == (size_t)2 * dE && std::fabs(signal[0] - std::sin(4.0f)) < 1e-6f &&
                 std::fabs(signal[dE / 2] - std::cos(4.0f)) < 1e-6f && std::fabs(signal[dE + dE / 2 - 1] - std::sin(5.0e-4f)) < 1e-9f,
             "SinusoidalPositionEmbeddings: sine half, cosine half, slowest timescale");
      const std::vector<uint32_t> words{4, 0, 3, 3, 1, 2};
      const float scale = std::sqrt((float)dE);
      std::vector<float> wantEmb((size_t)nWords * dE);
      for(int r = 0; r < nWords; ++r)
        for(int i = 0; i < dE; ++i) {
          volatile float scaled = scale * emb[(size_t)words[r] * dE + i];   // two roundings, like two graph nodes
          wantEmb[(size_t)r * dE + i] = scaled + signal[(size_t)(r / perSignal) * dE + i];
        }
      Tensor et = upload(ta, emb, {5, dE}, Type::float32), wt = upload(ta, words, {nWords}, Type::uint32);
      Tensor sg = upload(ta, signal, {2, dE}, Type::float32), eo, emax;
      ta.allocate(eo, {nWords, dE}, Type::float32);
      ta.allocate(emax, {MARIAN_HIP_ABSMAX_SLOTS}, Type::float32);
      ScaledEmbeddings(be, eo, et, wt, scale, &sg, perSignal, &emax);
      expect(sameBits(download<float>(be, eo, wantEmb.size()), wantEmb), "ScaledEmbeddings: sqrt(d) * rows + position signal, bit for bit");
      std::vector<float> slots = download<float>(be, emax, MARIAN_HIP_ABSMAX_SLOTS);
      bool slotsOk = true;
      for(int r = 0; r < MARIAN_HIP_ABSMAX_SLOTS; ++r) {
        float m = 0.0f;
        for(int i = 0; r < nWords && i < dE; ++i) m = std::max(m, std::fabs(wantEmb[(size_t)r * dE + i]));
        slotsOk = slotsOk && slots[r] == m;
      }
      expect(slotsOk, "ScaledEmbeddings: abs-max slot per row, zero past the last row");
      // state selection: 3 entries x 2 segments x capacity 6, four values of every segment in use
      std::vector<float> stateHost(3 * 2 * 6), before(4 * 2 * 6, -1.0f);
      for(size_t i = 0; i < stateHost.size(); ++i) stateHost[i] = (float)i;
      const std::vector<uint32_t> back{2, 0, 2, 1};
      Tensor stT = upload(ta, stateHost, {3, 2, 6}, Type::float32), bk = upload(ta, back, {4}, Type::uint32);
      Tensor sel = upload(ta, before, {4, 2, 6}, Type::float32);
      SelectState(be, sel, stT, bk, 4);
      std::vector<float> wantSel = before;
      for(int r = 0; r < 4; ++r)
        for(int sg = 0; sg < 2; ++sg)
          for(int i = 0; i < 4; ++i) wantSel[(size_t)(r * 2 + sg) * 6 + i] = stateHost[(size_t)(back[r] * 2 + sg) * 6 + i];
      expect(sameBits(download<float>(be, sel, wantSel.size()), wantSel), "SelectState: the values in use of the chosen entries, the rest untouched");
      // the same beam-search step without the copy: 3 hypotheses x 2 heads, two cached positions + the new one
      const int nh = 3, hd = 2, cp = 4, ln = 3, dkk = 64;
      std::vector<float> kc((size_t)nh * hd * cp * dkk), vc(kc.size()), qv((size_t)nh * hd * dkk), knv(qv.size()), vnv(qv.size());
      uint32_t r2 = 777u;
      auto nextf = [&]() { r2 = r2 * 1664525u + 1013904223u; return (float)(r2 >> 8) * (1.0f / 8388608.0f) - 1.0f; };
      for(auto& x : kc) x = nextf();
      for(auto& x : vc) x = nextf();
      for(auto& x : qv) x = nextf();
      for(auto& x : knv) x = nextf();
      for(auto& x : vnv) x = nextf();
      const std::vector<uint32_t> prevAnc{0, 0, 0, 0, 1, 1, 1, 1, 2, 2, 2, 2}, parents{2, 2, 0};
      Tensor pa = upload(ta, prevAnc, {nh, cp}, Type::uint32), pr = upload(ta, parents, {nh}, Type::uint32), na;
      ta.allocate(na, {nh, cp}, Type::uint32);
      AdvanceAncestors(be, na, pa, pr, ln - 1);
      const std::vector<uint32_t> gotAnc = download<uint32_t>(be, na, (size_t)nh * cp);
      expect(gotAnc[0] == 2 && gotAnc[1] == 2 && gotAnc[2] == 0 && gotAnc[4] == 2 && gotAnc[6] == 1 && gotAnc[8] == 0 &&
                 gotAnc[9] == 0 && gotAnc[10] == 2,
             "AdvanceAncestors: the parents' rows, then the hypothesis itself");
      // reference: the caches of the parents copied (SelectState), then the attention on them
      std::vector<uint32_t> rowsOfParents;
      for(int h = 0; h < nh; ++h) rowsOfParents.push_back(parents[h]);
      Tensor kT = upload(ta, kc, {nh, hd, cp * dkk}, Type::float32), vT = upload(ta, vc, {nh, hd, cp * dkk}, Type::float32);
      Tensor kG = upload(ta, kc, {nh, hd, cp * dkk}, Type::float32), vG = upload(ta, vc, {nh, hd, cp * dkk}, Type::float32);
      Tensor rp = upload(ta, rowsOfParents, {nh}, Type::uint32);
      SelectState(be, kG, kT, rp, (ln - 1) * dkk);
      SelectState(be, vG, vT, rp, (ln - 1) * dkk);
      Tensor qT = upload(ta, qv, {nh * hd, 1, dkk}, Type::float32), knT = upload(ta, knv, {nh * hd, dkk}, Type::float32);
      Tensor vnT = upload(ta, vnv, {nh * hd, dkk}, Type::float32), o1, o2;
      ta.allocate(o1, {nh * hd, 1, dkk}, Type::float32);
      ta.allocate(o2, {nh * hd, 1, dkk}, Type::float32);
      kG.shape = {nh * hd, cp, dkk}; vG.shape = kG.shape;
      Attention(be, o1, qT, kG, vG, 0.125f, nullptr, 1, nullptr, &knT, &vnT, ln);
      kT.shape = {nh * hd, cp, dkk}; vT.shape = kT.shape;
      AttentionByAncestors(be, o2, qT, kT, vT, 0.125f, na, ln, knT, vnT);
      expect(sameBits(download<float>(be, o2, qv.size()), download<float>(be, o1, qv.size())),
             "AttentionByAncestors: the attention on the copied caches, bit for bit");
    }

    {   // projections + attention in one launch against the separate wrappers: 5 rows of 128 values, 2 heads (N = 128)
      const int hd = 2, NN = hd * 64, Mr = 5, cap = 6, len = 4, K5 = 128;
      if((size_t)Mr * K5 <= A.size()) {
        std::vector<float> wq((size_t)K5 * NN), wk(wq.size()), wv(wq.size()), kc((size_t)Mr * hd * cap * 64), vc(kc.size());
        uint32_t r3 = 4242u;
        auto nx = [&]() { r3 = r3 * 1664525u + 1013904223u; return (float)(r3 >> 8) * (1.0f / 8388608.0f) - 1.0f; };
        for(auto& x : wq) x = 0.02f * nx();
        for(auto& x : wk) x = 0.02f * nx();
        for(auto& x : wv) x = 0.02f * nx();
        for(auto& x : kc) x = nx();
        for(auto& x : vc) x = nx();
        std::vector<float> a5(A.begin(), A.begin() + (size_t)Mr * K5);
        Tensor a5t = upload(ta, a5, {Mr, K5}, Type::float32);
        Tensor wqf = upload(ta, wq, {K5, NN}, Type::float32), wkf = upload(ta, wk, {K5, NN}, Type::float32),
               wvf = upload(ta, wv, {K5, NN}, Type::float32);
        Tensor wqq, wkq, wvq, aqa, aqb, q5, k5, v5, o1, o2;
        for(Tensor* t : {&wqq, &wkq, &wvq}) ta.allocate(*t, {K5, NN}, Type::intgemm8);
        integer::prepareB(ta, wqf, wqq);
        integer::prepareB(ta, wkf, wkq);
        integer::prepareB(ta, wvf, wvq);
        ta.allocate(aqa, {Mr, K5}, Type::intgemm8);
        ta.allocate(aqb, {Mr, K5}, Type::intgemm8);
        for(Tensor* t : {&q5, &k5, &v5, &o1, &o2}) ta.allocate(*t, {Mr, NN}, Type::float32);
        Tensor kA = upload(ta, kc, {Mr * hd, cap, 64}, Type::float32), vA = upload(ta, vc, {Mr * hd, cap, 64}, Type::float32);
        Tensor kB = upload(ta, kc, {Mr * hd, cap, 64}, Type::float32), vB = upload(ta, vc, {Mr * hd, cap, 64}, Type::float32);
        integer::affineOrDotGrouped(ta, a5t, aqa, {&wqq, &wkq, &wvq}, {}, {&q5, &k5, &v5});
        Tensor q3 = q5, kn = k5, vn = v5, o13 = o1;
        q3.shape = {Mr * hd, 1, 64}; o13.shape = q3.shape; kn.shape = {Mr * hd, 64}; vn.shape = kn.shape;
        Attention(be, o13, q3, kA, vA, 0.125f, nullptr, 1, nullptr, &kn, &vn, len);
        ProjectedAttention(ta, o2, a5t, aqb, {&wqq, &wkq, &wvq}, {}, kB, vB, hd, len);
        expect(sameBits(download<float>(be, o2, (size_t)Mr * NN), download<float>(be, o1, (size_t)Mr * NN)) &&
                   sameBits(download<float>(be, kB, kc.size()), download<float>(be, kA, kc.size())) &&
                   sameBits(download<int8_t>(be, aqb, (size_t)Mr * K5 + 4), download<int8_t>(be, aqa, (size_t)Mr * K5 + 4)),
               "ProjectedAttention: the grouped affine + Attention, output, caches and quantized input bit for bit");
      }
    }
    be.synchronize();
    std::printf("host_check: %d failure(s), slab moved %zu times -> %s\n", failures,
                ta.allocator()->device()->moves(), failures == 0 ? "OK" : "FAILED");
    return failures == 0 ? 0 : 1;
  } catch(const std::exception& e) {
    std::printf("host_check: exception: %s -> FAILED\n", e.what());
    return 1;
  }
}
