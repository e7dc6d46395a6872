// C++ host side of the HIP int8 path, shaped like Marian's intgemm glue so that it can be dropped
// into src/tensors/hip/ with Marian's own Tensor/Expr types substituted for the minimal ones here.
//
// Mirrors (reference file:line):
//   src/tensors/cpu/integer_common.h:48-49     cols(), rows()
//   src/tensors/cpu/integer_common.h:101-111   getQuantMult()  (device read here)
//   src/tensors/cpu/intgemm_interface.h:17-32  prepareA()
//   src/tensors/cpu/intgemm_interface.h:46-99  affineOrDotTyped()  -> affineOrDot()
//   src/tensors/gpu/backend.h:23-110           Backend (stream, synchronize), reduced to this path
//   src/tensors/tensor_allocator.h:12-93       TensorAllocator (tensors carved from hip_device.h's Allocator)
//   src/tensors/gpu/cuda_helpers.h:15-19       CUDA_CHECK -> MARIAN_HIP_CHECK (status code -> abort)
//   src/graph/expression_graph.cpp:120-185     forward tape (inference mode clears a node's children)  -> graph::
//
// Tensors hold a MemoryPiece handle, not a pointer: the allocator may move its slab whenever
// something is allocated, and every wrapper below reads the pointers at the moment of the call.
// The library retains nothing between calls, so a move between two calls is harmless.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <functional>
#include <list>
#include <string>
#include <vector>

#include "../../include/marian_hip_int16.h"
#include "../../include/marian_hip_int8.h"
#include "hip_device.h"

namespace marian {
namespace hip {

#define MARIAN_HIP_CHECK(expr)                                                              \
  do {                                                                                      \
    int st_ = (expr);                                                                       \
    if(st_ != MARIAN_HIP_OK)                                                                \
      ::marian::hip::abortWith(std::string(#expr) + ": " + marian_hip_status_string(st_) +  \
                               (st_ == MARIAN_HIP_ERR_HIP                                   \
                                    ? " (hipError " + std::to_string(marian_hip_last_hip_error()) + ")" \
                                    : std::string()));                                      \
  } while(0)

// Element types with Marian's numeric values (src/common/types.h:270-328).
enum class Type : size_t {
  int8 = 0x100 + 1,
  int32 = 0x100 + 4,
  uint32 = 0x200 + 4,
  float32 = 0x400 + 4,
  intgemm8 = 0x10000 + 1,
  intgemm16 = 0x10000 + 2,
  intgemm8ssse3 = 0x10000 + 1 + 0x8000,
  intgemm8avx2 = 0x10000 + 1 + 0x1000,
  intgemm8avx512 = 0x10000 + 1 + 0x2000,
  intgemm8avx512vnni = 0x10000 + 1 + 0x2000 + 4096,
  intgemm16sse2 = 0x10000 + 2 + 0x4000,
  intgemm16avx2 = 0x10000 + 2 + 0x1000,
  intgemm16avx512 = 0x10000 + 2 + 0x2000,
};
inline size_t sizeOf(Type t) { return (size_t)t & 0xFF; }
inline bool isIntgemm(Type t) { return ((size_t)t & 0x10000) != 0; }
inline bool isFloat(Type t) { return ((size_t)t & 0x400) != 0; }
inline bool isHardwareSpecific(Type t) { return isIntgemm(t) && ((size_t)t & 0xF000) != 0; }

typedef std::vector<int> Shape;
inline size_t elements(const Shape& shape) {
  size_t n = 1;
  for(int d : shape) n *= (size_t)d;
  return n;
}
// src/common/types.cpp:32-34: intgemm tensors carry one extra fp32, the quantMult
inline size_t requiredBytes(const Shape& shape, Type type) {
  return elements(shape) * sizeOf(type) + (isIntgemm(type) ? sizeof(float) : 0);
}

// A device tensor: a piece of the allocator's slab with a shape and an element type.
struct Tensor {
  MemoryPiece::PtrType memory;
  Shape shape;
  Type type = Type::float32;
  // 8-bit weights only: the payload is in the order the GEMM kernels read (written by prepareB or
  // prepareAndTransposeB), not in the file order [N, K].  The reference tells such tensors apart by
  // type (intgemm8avx2 ... next to the hardware-agnostic intgemm8, src/common/types.h); a Marian
  // build with this backend would add an enum value of that kind, this stand-in keeps a flag.
  bool prepared = false;
  size_t elements() const { return ::marian::hip::elements(shape); }
  template <typename T>
  T* data() const { return memory ? memory->data<T>() : nullptr; }
  explicit operator bool() const { return memory && memory->data(); }
};
inline int cols(const Tensor& t) { return t.shape.back(); }
inline int rows(const Tensor& t) { return (int)(t.elements() / (size_t)cols(t)); }

// Per-device state of the path: the device number and one stream.
class Backend {
public:
  explicit Backend(int device) : device_(device) {
    HIP_CHECK(hipSetDevice(device_));
    HIP_CHECK(hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking));
  }
  ~Backend() { (void)hipStreamDestroy(stream_); }
  Backend(const Backend&) = delete;
  Backend& operator=(const Backend&) = delete;
  void setDevice() { HIP_CHECK(hipSetDevice(device_)); }
  void synchronize() { HIP_CHECK(hipStreamSynchronize(stream_)); }
  hipStream_t stream() const { return stream_; }
  int deviceNo() const { return device_; }

private:
  int device_;
  hipStream_t stream_ = nullptr;
};

// Tensors out of an Allocator (reference src/tensors/tensor_allocator.h:12-93).  It also owns the
// abs-max workspace of the int8 calls, a piece like any other (it moves with the slab).
class TensorAllocator {
public:
  static constexpr size_t kGrow = 128ull << 20, kAlign = 256;
  explicit TensorAllocator(Backend& backend, size_t step = kGrow, size_t limit = 0)
      : backend_(backend),
        device_(std::make_shared<Device>(backend.deviceNo(), kAlign)),
        allocator_(std::make_shared<Allocator>(device_, 0, step, kAlign, limit, backend.stream())) {}

  void throwAtReallocation(bool flag) { allocator_->throwAtReallocation(flag); }
  void reserveExact(size_t bytes) {
    allocator_->reserve(bytes);
    workspace_.reset();
  }
  void clear() {
    allocator_->clear();
    workspace_.reset();
  }
  size_t capacity(const Shape& shape, Type type = Type::float32) const {
    return allocator_->alignedSize(requiredBytes(shape, type));
  }
  void allocate(Tensor& t, const Shape& shape, Type type = Type::float32) {
    if(!t || t.shape != shape || t.type != type) {
      t.memory = allocator_->alloc(requiredBytes(shape, type));
      t.shape = shape;
      t.type = type;
    }
  }
  void free(Tensor& t) {
    if(t.memory) allocator_->free(t.memory);
    t.memory.reset();
  }
  // the abs-max workspace of marian_hip_int8_prepare_a / _prepare_b / _affine_f32
  void* workspace() {
    if(!workspace_ || !workspace_->data()) workspace_ = allocator_->alloc(workspaceBytes());
    return workspace_->data();
  }
  size_t workspaceBytes() const { return marian_hip_int8_workspace_bytes(); }
  const std::shared_ptr<Allocator>& allocator() const { return allocator_; }
  Backend& backend() const { return backend_; }

private:
  Backend& backend_;
  std::shared_ptr<Device> device_;
  std::shared_ptr<Allocator> allocator_;
  MemoryPiece::PtrType workspace_;
};

namespace integer {

// Device read of the trailing quantMult (host code must not dereference device memory).
inline float getQuantMult(Backend& be, const Tensor& t) {
  if(!isIntgemm(t.type)) abortWith("getQuantMult does not work for this type");
  float qm = 0.f;
  // the tail sits behind the payload: elements * 1 byte for intgemm8, * 2 bytes for intgemm16
  const float* tail = reinterpret_cast<const float*>(t.data<int8_t>() + t.elements() * sizeOf(t.type));
  copy(be.stream(), tail, tail + 1, &qm);
  return qm;
}

// Forward body of the prepareA node: out has the shape of a and the type of the weights it will
// meet - intgemm8 (abs-max quantMult) or intgemm16 (quantMult 1024) - and requiredBytes(shape) bytes.
inline void prepareA(TensorAllocator& ta, const Tensor& a, Tensor& out) {
  if(!isFloat(a.type)) abortWith("Intgemm expects type of A to be float32");
  if(out.type == Type::intgemm16) {
    MARIAN_HIP_CHECK(marian_hip_int16_prepare_a(a.data<float>(), out.data<int16_t>(), rows(a), cols(a),
                                                ta.backend().stream()));
    return;
  }
  void* ws = ta.workspace();   // (may allocate: before any pointer is read)
  MARIAN_HIP_CHECK(marian_hip_int8_prepare_a(a.data<float>(), out.data<int8_t>(), rows(a), cols(a), ws,
                                             ta.workspaceBytes(), ta.backend().stream()));
}

// Offline quantizer body (marian-conv): w float32 [K, N] -> out intgemm8 [K, N] (payload: the quantized W^T
// in the order the kernels read).
inline void prepareB(TensorAllocator& ta, const Tensor& w, Tensor& out) {
  if(out.type == Type::intgemm16) {
    MARIAN_HIP_CHECK(marian_hip_int16_prepare_b(w.data<float>(), out.data<int16_t>(), w.shape[0], w.shape[1],
                                                ta.backend().stream()));
    return;
  }
  void* ws = ta.workspace();
  MARIAN_HIP_CHECK(marian_hip_int8_prepare_b(w.data<float>(), out.data<int8_t>(), w.shape[0], w.shape[1],
                                             ws, ta.workspaceBytes(), ta.backend().stream()));
  out.prepared = true;
}

// A quantized weight item as a model file holds it (plain rows [N, K] + quantMult) -> the order the
// kernels read; reference prepareAndTransposeB, src/tensors/cpu/integer_common.h:189-216 (there: the
// tiling of the CPU the process runs on).  in and out are different tensors of the same shape and type.
inline void prepareAndTransposeB(Backend& be, const Tensor& in, Tensor& out) {
  if(!isIntgemm(in.type) || isHardwareSpecific(in.type) || in.type != out.type)
    abortWith("prepareAndTransposeB expects a hardware-agnostic intgemm matrix");
  if(in.type == Type::intgemm16) {
    MARIAN_HIP_CHECK(marian_hip_int16_prepare_b_quantized_transposed(in.data<int16_t>(), out.data<int16_t>(),
                                                                     in.shape[0], in.shape[1], be.stream()));
    return;
  }
  if(in.prepared) abortWith("the weights are prepared already");
  MARIAN_HIP_CHECK(marian_hip_int8_prepare_b_quantized_transposed(in.data<int8_t>(), out.data<int8_t>(), in.shape[0],
                                                                  in.shape[1], be.stream()));
  out.prepared = true;
}

inline void checkB(const Tensor& bQuant) {
  if(!isIntgemm(bQuant.type)) abortWith("Intgemm expects type of B to be a variant of intgemm");
  if(isHardwareSpecific(bQuant.type) || (sizeOf(bQuant.type) != 1 && sizeOf(bQuant.type) != 2))
    abortWith("Unsupported type for Intgemm type??");
  if(sizeOf(bQuant.type) == 1 && !bQuant.prepared)
    abortWith("B is in file order: it has to go through prepareAndTransposeB first");
}

// Forward body of the multiply node; bias may be null (dot).  relu fuses the in-place ReLU node.
// shortlist: device ids (sorted, unique, a multiple of eight many) or null.
inline void multiply(Backend& be, const Tensor& aQuant, const Tensor& bQuant, const Tensor* bias, Tensor& out,
                     float scale, bool relu, const Tensor* shortlist = nullptr) {
  checkB(bQuant);
  if(sizeOf(bQuant.type) == 2) {   // Type::intgemm16
    if(shortlist) abortWith("the 16-bit path has no shortlist form");
    MARIAN_HIP_CHECK(marian_hip_int16_affine(aQuant.data<int16_t>(), bQuant.data<int16_t>(),
                                             bias ? bias->data<float>() : nullptr, out.data<float>(), rows(aQuant),
                                             cols(aQuant), cols(bQuant), scale, relu ? 1 : 0, be.stream()));
    return;
  }
  if(shortlist)
    MARIAN_HIP_CHECK(marian_hip_int8_affine_shortlist(
        aQuant.data<int8_t>(), bQuant.data<int8_t>(), bias ? bias->data<float>() : nullptr,
        shortlist->data<uint32_t>(), (int64_t)shortlist->elements(), out.data<float>(), rows(aQuant),
        cols(aQuant), cols(bQuant), scale, relu ? 1 : 0, be.stream()));
  else
    MARIAN_HIP_CHECK(marian_hip_int8_affine(aQuant.data<int8_t>(), bQuant.data<int8_t>(),
                                            bias ? bias->data<float>() : nullptr, out.data<float>(),
                                            rows(aQuant), cols(aQuant), cols(bQuant), scale, relu ? 1 : 0,
                                            be.stream()));
}

// The int32 accumulators Kernels8::Multiply hands to its callback (parity hook).
inline void multiplyInt32(Backend& be, const Tensor& aQuant, const Tensor& bQuant, Tensor& acc,
                          const Tensor* shortlist = nullptr) {
  checkB(bQuant);
  MARIAN_HIP_CHECK(marian_hip_int8_multiply_i32(
      aQuant.data<int8_t>(), bQuant.data<int8_t>(), shortlist ? shortlist->data<uint32_t>() : nullptr,
      shortlist ? (int64_t)shortlist->elements() : 0, acc.data<int32_t>(), rows(aQuant), cols(aQuant),
      cols(bQuant), be.stream()));
}

// affineOrDot: type guards as in the reference, then both node bodies in one call.  aQuant is the
// prepareA node's output tensor (it is filled exactly as prepareA would fill it).
// absmaxIn / absmaxOut: optional tensors of MARIAN_HIP_ABSMAX_SLOTS floats; absmaxIn is what the
// call that produced `a` left (then the abs-max pass over `a` is skipped), absmaxOut receives the
// same for `out`.
inline void affineOrDot(TensorAllocator& ta, const Tensor& a, Tensor& aQuant, const Tensor& bQuant,
                        const Tensor* bias, Tensor& out, float scale = 1.f, bool relu = false,
                        const Tensor* shortlist = nullptr, const Tensor* absmaxIn = nullptr,
                        Tensor* absmaxOut = nullptr) {
  if(!isFloat(a.type)) abortWith("Intgemm expects type of A to be float32");
  checkB(bQuant);
  if(sizeOf(bQuant.type) == 2) {   // Type::intgemm16: the two node bodies one after the other
    if(aQuant.type != Type::intgemm16) abortWith("the prepareA node of a 16-bit weight must be typed intgemm16");
    prepareA(ta, a, aQuant);
    multiply(ta.backend(), aQuant, bQuant, bias, out, scale, relu, shortlist);
    return;
  }
  void* ws = ta.workspace();   // (may allocate and move the slab: before any pointer is read)
  const uint32_t* idx = shortlist ? shortlist->data<uint32_t>() : nullptr;
  const int64_t nIdx = shortlist ? (int64_t)shortlist->elements() : 0;
  if(absmaxIn || absmaxOut)
    MARIAN_HIP_CHECK(marian_hip_int8_affine_f32_chained(
        a.data<float>(), aQuant.data<int8_t>(), bQuant.data<int8_t>(), bias ? bias->data<float>() : nullptr,
        idx, nIdx, out.data<float>(), rows(a), cols(a), cols(bQuant), scale, relu ? 1 : 0,
        absmaxIn ? absmaxIn->data<float>() : nullptr, absmaxOut ? absmaxOut->data<float>() : nullptr, ws,
        ta.workspaceBytes(), ta.backend().stream()));
  else
    MARIAN_HIP_CHECK(marian_hip_int8_affine_f32(
        a.data<float>(), aQuant.data<int8_t>(), bQuant.data<int8_t>(), bias ? bias->data<float>() : nullptr,
        idx, nIdx, out.data<float>(), rows(a), cols(a), cols(bQuant), scale, relu ? 1 : 0, ws,
        ta.workspaceBytes(), ta.backend().stream()));
}

// One activation tensor through several weight matrices (the self-attention projections Wq, Wk, Wv
// of src/models/transformer.h:290-325): one abs-max, one quantization, for decode sizes one launch.
// outs[g] is what affineOrDot(a, aQuant, *bQuants[g], biases[g], *outs[g], scale, relu) writes.
inline void affineOrDotGrouped(TensorAllocator& ta, const Tensor& a, Tensor& aQuant,
                               const std::vector<const Tensor*>& bQuants, const std::vector<const Tensor*>& biases,
                               const std::vector<Tensor*>& outs, float scale = 1.f, bool relu = false,
                               const Tensor* absmaxIn = nullptr) {
  if(!isFloat(a.type)) abortWith("Intgemm expects type of A to be float32");
  if(bQuants.empty() || bQuants.size() > 4 || outs.size() != bQuants.size() ||
     (!biases.empty() && biases.size() != bQuants.size()))
    abortWith("affineOrDotGrouped: between one and four weight matrices, one output (and bias entry) each");
  void* ws = ta.workspace();   // (may allocate and move the slab: before any pointer is read)
  std::vector<const int8_t*> bq(bQuants.size());
  std::vector<const float*> bi(bQuants.size(), nullptr);
  std::vector<float*> o(bQuants.size());
  std::vector<int64_t> n(bQuants.size());
  for(size_t g = 0; g < bQuants.size(); ++g) {
    checkB(*bQuants[g]);
    bq[g] = bQuants[g]->data<int8_t>();
    if(!biases.empty() && biases[g]) bi[g] = biases[g]->data<float>();
    o[g] = outs[g]->data<float>();
    n[g] = cols(*bQuants[g]);
  }
  MARIAN_HIP_CHECK(marian_hip_int8_affine_f32_grouped(
      a.data<float>(), aQuant.data<int8_t>(), (int64_t)bq.size(), bq.data(), bi.data(), o.data(), n.data(), rows(a),
      cols(a), scale, relu ? 1 : 0, absmaxIn ? absmaxIn->data<float>() : nullptr, ws, ta.workspaceBytes(),
      ta.backend().stream()));
}

// The same for callers that cannot allocate: no aQuant tensor, no workspace (the library's static
// scratch holds both; rows(a) * cols(a) <= MARIAN_HIP_STATIC_MAX_ELEMS).
inline void affineOrDotStatic(Backend& be, const Tensor& a, const Tensor& bQuant, const Tensor* bias,
                              Tensor& out, float scale = 1.f, bool relu = false,
                              const Tensor* shortlist = nullptr) {
  if(!isFloat(a.type)) abortWith("Intgemm expects type of A to be float32");
  checkB(bQuant);
  MARIAN_HIP_CHECK(marian_hip_int8_affine_f32_static(
      a.data<float>(), bQuant.data<int8_t>(), bias ? bias->data<float>() : nullptr,
      shortlist ? shortlist->data<uint32_t>() : nullptr, shortlist ? (int64_t)shortlist->elements() : 0,
      out.data<float>(), rows(a), cols(a), cols(bQuant), scale, relu ? 1 : 0, be.stream()));
}

}  // namespace integer

// ---- the graph side: lambda nodes on a forward tape, reduced to what this path needs -------
// Mirrors (reference file:line):
//   src/graph/node_operators_binary.h:16-80, src/graph/expression_operators.h:29-34   LambdaNodeOp, lambda()
//   src/graph/expression_graph.cpp:120-185   ExpressionGraph::forward: for every node of the tape in
//       order - allocate its value, run its forward functor, and in inference mode clear its
//       children (:168-169) so that a tensor is given back as soon as no later node holds it
//   src/graph/node.cpp (Node::free)          a node that nobody holds any more gives its value back
// The affine binding below is what a src/tensors/hip/int8_interface.h of a Marian build would hold;
// here it runs on these minimal types so that it is compiled and exercised (host_check.cpp).
namespace graph {

struct Node;
typedef std::shared_ptr<Node> Expr;
typedef std::function<void(Expr out, const std::vector<Expr>& in)> LambdaNodeFunctor;

struct Node {
  TensorAllocator& ta;
  std::vector<Expr> children;
  Shape shape;
  Type type;
  LambdaNodeFunctor forward;
  Tensor val;
  bool parameter = false;   // parameters own their memory elsewhere; the tape never frees it
  Node(TensorAllocator& ta_, std::vector<Expr> children_, Shape shape_, Type type_, LambdaNodeFunctor forward_)
      : ta(ta_), children(std::move(children_)), shape(std::move(shape_)), type(type_), forward(std::move(forward_)) {}
  Node(const Node&) = delete;
  Node& operator=(const Node&) = delete;
  ~Node() {
    if(!parameter && val.memory && val.memory->data()) ta.free(val);
  }
  Type value_type() const { return type; }
};

class ExpressionGraph {
public:
  ExpressionGraph(TensorAllocator& ta, bool inferenceOnly) : ta_(ta), inferenceOnly_(inferenceOnly) {}
  TensorAllocator& allocator() const { return ta_; }

  // A parameter or constant input: wraps a tensor that lives outside the tape.
  Expr param(const Tensor& t) {
    auto n = std::make_shared<Node>(ta_, std::vector<Expr>(), t.shape, t.type, LambdaNodeFunctor());
    n->val = t;
    n->parameter = true;
    return n;
  }
  // lambda(nodes, shape, type, forward): a node whose forward step is the given functor.
  Expr lambda(std::vector<Expr> nodes, Shape shape, Type type, LambdaNodeFunctor forward) {
    auto n = std::make_shared<Node>(ta_, std::move(nodes), std::move(shape), type, std::move(forward));
    tape_.push_back(n);
    return n;
  }
  // Runs the tape front to back.  afterNode (optional) is called after every node with the tape's
  // own reference already dropped, i.e. at the point where the node's inputs may have been freed.
  void forward(const std::function<void(const Node&)>& afterNode = nullptr) {
    while(!tape_.empty()) {
      Expr v = tape_.front();
      tape_.pop_front();
      ta_.allocate(v->val, v->shape, v->type);
      if(v->forward) v->forward(v, v->children);
      if(inferenceOnly_) v->children.clear();
      if(afterNode) afterNode(*v);
    }
  }

private:
  TensorAllocator& ta_;
  bool inferenceOnly_;
  std::list<Expr> tape_;
};

// affineOrDot of the HIP backend: the reference's node structure (src/tensors/cpu/intgemm_interface.h:
// 46-99) - node 1 holds the quantized activations (typed like the weights, M * K + 4 bytes), node 2
// the float32 product - with BOTH node bodies run by node 2 in one library call
// (marian_hip_int8_affine_f32: one kernel at decode sizes).  Node 2 therefore reads the float32
// input itself and must hold it as a DIRECT child: in inference mode the tape clears node 1's
// children as soon as node 1 has run (src/graph/expression_graph.cpp:168-169), and an input held only
// through node 1 would be freed - and its memory handed to node 2's own output - before node 2 runs.
// Children of node 2: {aQuant, bQuant, [bias,] a}; `a` is last, so a bias is present iff there are four.
inline Expr affineOrDot(ExpressionGraph& g, Expr a, Expr bQuant, Expr bias, bool transA, bool /*transB*/,
                        float scale, bool relu = false) {
  if(!isFloat(a->value_type())) abortWith("Intgemm expects type of A to be float32");
  integer::checkB(bQuant->val);
  if(transA) abortWith("transA: put a transpose node in front (the reference does, intgemm_interface.h:52)");
  // node 1: the output tensor of prepareA.  Its functor is empty - node 2's call fills it, exactly
  // as prepareA would - but it is a real node: the tape allocates its value and frees it after use.
  Expr aQuant = g.lambda({a}, a->shape, bQuant->value_type(), [](Expr, const std::vector<Expr>&) {});
  Shape outShape = a->shape;
  outShape.back() = bQuant->shape.back();
  auto fwd = [scale, relu](Expr out, const std::vector<Expr>& in) {
    Expr aQ = in[0], bQ = in[1], a_ = in.back();
    Expr bias_ = in.size() > 3 ? in[2] : nullptr;
    integer::affineOrDot(out->ta, a_->val, aQ->val, bQ->val, bias_ ? &bias_->val : nullptr, out->val, scale, relu);
  };
  std::vector<Expr> children = {aQuant, bQuant};
  if(bias) children.push_back(bias);
  children.push_back(a);
  return g.lambda(children, outShape, Type::float32, fwd);   // inference-only node
}

// The same as two real nodes, the reference's structure one to one: node 1 runs prepareA, node 2
// reads nothing but the values of its children {aQuant, bQuant, [bias]}.
inline Expr affineOrDotTwoNodes(ExpressionGraph& g, Expr a, Expr bQuant, Expr bias, float scale, bool relu = false) {
  if(!isFloat(a->value_type())) abortWith("Intgemm expects type of A to be float32");
  integer::checkB(bQuant->val);
  Expr aQuant = g.lambda({a}, a->shape, bQuant->value_type(), [](Expr out, const std::vector<Expr>& in) {
    integer::prepareA(out->ta, in[0]->val, out->val);
  });
  Shape outShape = a->shape;
  outShape.back() = bQuant->shape.back();
  auto fwd = [scale, relu](Expr out, const std::vector<Expr>& in) {
    Expr bias_ = in.size() > 2 ? in[2] : nullptr;
    integer::multiply(out->ta.backend(), in[0]->val, in[1]->val, bias_ ? &bias_->val : nullptr, out->val, scale, relu);
  };
  std::vector<Expr> children = {aQuant, bQuant};
  if(bias) children.push_back(bias);
  return g.lambda(children, outShape, Type::float32, fwd);
}

}  // namespace graph
}  // namespace hip
}  // namespace marian
