// C++ host side of the HIP int8 path, shaped like Marian's intgemm glue so that it can be dropped
// into src/tensors/hip/ with Marian's own Tensor/Expr types substituted for the minimal ones here.
//
// Mirrors (reference file:line):
//   src/tensors/cpu/integer_common.h:48-49     cols(), rows()
//   src/tensors/cpu/integer_common.h:101-111   getQuantMult()  (device read here)
//   src/tensors/cpu/intgemm_interface.h:17-32  prepareA()
//   src/tensors/cpu/intgemm_interface.h:46-99  affineOrDotTyped()  -> affineOrDot()
//   src/tensors/gpu/backend.h:23-110           Backend (stream, synchronize), reduced to this path
//   src/tensors/gpu/cuda_helpers.h:15-19       CUDA_CHECK -> MARIAN_HIP_CHECK (status code -> abort)
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/marian_hip_int8.h"

namespace marian {
namespace hip {

// ABORT of src/common/logging.h:100-116: throws when asked to (setThrowExceptionOnAbort), else aborts.
inline bool& throwOnAbort() {
  static bool flag = true;
  return flag;
}
[[noreturn]] inline void abortWith(const std::string& msg) {
  if(throwOnAbort()) throw std::runtime_error(msg);
  std::fprintf(stderr, "Error: %s\n", msg.c_str());
  std::abort();
}
#define MARIAN_HIP_CHECK(expr)                                                              \
  do {                                                                                      \
    int st_ = (expr);                                                                       \
    if(st_ != MARIAN_HIP_OK)                                                                \
      ::marian::hip::abortWith(std::string(#expr) + ": " + marian_hip_status_string(st_) +  \
                               (st_ == MARIAN_HIP_ERR_HIP                                   \
                                    ? " (hipError " + std::to_string(marian_hip_last_hip_error()) + ")" \
                                    : std::string()));                                      \
  } while(0)
#define HIP_CHECK(expr)                                                                     \
  do {                                                                                      \
    hipError_t e_ = (expr);                                                                 \
    if(e_ != hipSuccess) ::marian::hip::abortWith(std::string(#expr) + ": " + hipGetErrorString(e_)); \
  } while(0)

// Element types with Marian's numeric values (src/common/types.h:270-328).
enum class Type : size_t {
  float32 = 0x400 + 4,
  intgemm8 = 0x10000 + 1,
  intgemm8ssse3 = 0x10000 + 1 + 0x8000,
  intgemm8avx2 = 0x10000 + 1 + 0x1000,
  intgemm8avx512 = 0x10000 + 1 + 0x2000,
  intgemm8avx512vnni = 0x10000 + 1 + 0x2000 + 4096,
};
inline bool isIntgemm(Type t) { return ((size_t)t & 0x10000) != 0; }
inline bool isFloat(Type t) { return ((size_t)t & 0x400) != 0; }
inline bool isHardwareSpecific(Type t) { return isIntgemm(t) && ((size_t)t & 0xF000) != 0; }

// A device tensor view: the caller (Marian's allocator) owns the memory.
struct Tensor {
  void* data = nullptr;
  std::vector<int> shape;
  Type type = Type::float32;
  size_t elements() const {
    size_t n = 1;
    for(int d : shape) n *= (size_t)d;
    return n;
  }
};
inline int cols(const Tensor& t) { return t.shape.back(); }
inline int rows(const Tensor& t) { return (int)(t.elements() / (size_t)cols(t)); }
// src/common/types.cpp:32-34
inline size_t requiredBytes(const std::vector<int>& shape, Type type) {
  size_t n = 1;
  for(int d : shape) n *= (size_t)d;
  return isIntgemm(type) ? n + sizeof(float) : n * sizeof(float);
}

// Per-device state of the path: one stream and the abs-max workspace.
class Backend {
public:
  explicit Backend(int device) : device_(device) {
    HIP_CHECK(hipSetDevice(device_));
    HIP_CHECK(hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking));
    workspaceBytes_ = marian_hip_int8_workspace_bytes();
    HIP_CHECK(hipMalloc(&workspace_, workspaceBytes_));
  }
  ~Backend() {
    (void)hipFree(workspace_);
    (void)hipStreamDestroy(stream_);
  }
  Backend(const Backend&) = delete;
  Backend& operator=(const Backend&) = delete;
  void setDevice() { HIP_CHECK(hipSetDevice(device_)); }
  void synchronize() { HIP_CHECK(hipStreamSynchronize(stream_)); }
  hipStream_t stream() const { return stream_; }
  void* workspace() const { return workspace_; }
  size_t workspaceBytes() const { return workspaceBytes_; }

private:
  int device_;
  hipStream_t stream_ = nullptr;
  void* workspace_ = nullptr;
  size_t workspaceBytes_ = 0;
};

namespace integer {

// Device read of the trailing quantMult (host code must not dereference device memory).
inline float getQuantMult(Backend& be, const Tensor& t) {
  if(!isIntgemm(t.type)) abortWith("getQuantMult does not work for this type");
  float qm = 0.f;
  HIP_CHECK(hipMemcpyAsync(&qm, (const int8_t*)t.data + t.elements(), sizeof(float),
                           hipMemcpyDeviceToHost, be.stream()));
  be.synchronize();
  return qm;
}

// Forward body of the prepareA node: out has shape of a, type intgemm8, requiredBytes(shape) bytes.
inline void prepareA(Backend& be, const Tensor& a, Tensor& out) {
  if(!isFloat(a.type)) abortWith("Intgemm expects type of A to be float32");
  MARIAN_HIP_CHECK(marian_hip_int8_prepare_a((const float*)a.data, (int8_t*)out.data, rows(a), cols(a),
                                             be.workspace(), be.workspaceBytes(), be.stream()));
}

// Offline quantizer body (marian-conv): w float32 [K, N] -> out intgemm8 [K, N] (payload W^T).
inline void prepareB(Backend& be, const Tensor& w, Tensor& out) {
  MARIAN_HIP_CHECK(marian_hip_int8_prepare_b((const float*)w.data, (int8_t*)out.data, w.shape[0],
                                             w.shape[1], be.workspace(), be.workspaceBytes(),
                                             be.stream()));
}

// Forward body of the multiply node; bias may be null (dot).  relu fuses the in-place ReLU node.
inline void multiply(Backend& be, const Tensor& aQuant, const Tensor& bQuant, const Tensor* bias,
                     Tensor& out, float scale, bool relu) {
  MARIAN_HIP_CHECK(marian_hip_int8_affine((const int8_t*)aQuant.data, (const int8_t*)bQuant.data,
                                          bias ? (const float*)bias->data : nullptr,
                                          (float*)out.data, rows(aQuant), cols(aQuant), cols(bQuant),
                                          scale, relu ? 1 : 0, be.stream()));
}

// affineOrDot: type guards as in the reference, then both node bodies in one call.  aQuant is the
// prepareA node's output tensor (it is filled exactly as prepareA would fill it).
inline void affineOrDot(Backend& be, const Tensor& a, Tensor& aQuant, const Tensor& bQuant,
                        const Tensor* bias, Tensor& out, float scale = 1.f, bool relu = false,
                        const uint32_t* shortlist = nullptr, int nShortlist = 0) {
  if(!isFloat(a.type)) abortWith("Intgemm expects type of A to be float32");
  if(!isIntgemm(bQuant.type)) abortWith("Intgemm expects type of B to be a variant of intgemm");
  if(isHardwareSpecific(bQuant.type)) abortWith("Unsupported type for Intgemm type??");
  MARIAN_HIP_CHECK(marian_hip_int8_affine_f32(
      (const float*)a.data, (int8_t*)aQuant.data, (const int8_t*)bQuant.data,
      bias ? (const float*)bias->data : nullptr, shortlist, nShortlist, (float*)out.data, rows(a),
      cols(a), cols(bQuant), scale, relu ? 1 : 0, be.workspace(), be.workspaceBytes(), be.stream()));
}

}  // namespace integer
}  // namespace hip
}  // namespace marian
