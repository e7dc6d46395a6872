// Device memory for a HIP backend of Marian: one slab per device, an allocator that carves
// 256-byte aligned pieces out of it, and copy/fill on the backend's stream.
//
// Counterparts (reference file:line):
//   src/tensors/device.h:10-36, src/tensors/gpu/device.cu:19-41   Device / gpu::Device::reserve
//   src/tensors/memory_piece.h:9-59, src/tensors/allocator.h:81-257   MemoryPiece, Allocator: host/allocator.h
//   src/tensors/tensor_allocator.h:12-93                          TensorAllocator
//   src/tensors/gpu/algorithm.cu:11-60                            gpu::copy, gpu::fill
//
// What is kept: the contract.  reserve() may only grow, growing MOVES the slab (every piece's
// pointer changes, MemoryPiece handles are re-pointed), sizes are rounded up to 256 bytes, an
// allocation that does not fit grows the slab by `step` bytes or, after throwAtReallocation(true),
// throws AllocationException; free() merges neighbouring gaps.
// What is different, because the device is an MI355X with 288 GB of HBM and not a 16 GB card:
//   * a grow copies old slab -> new slab on the device (both exist for a moment); only if the
//     new slab cannot be allocated next to the old one is the content parked in host memory, which
//     is what the reference always does;
//   * the allocator (host/allocator.h) keeps gaps and pieces as offsets into the slab and has an
//     optional byte limit; a grow that fails leaves the pieces pointing into whatever slab the
//     device still has, or empties them if it has none.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iterator>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/marian_hip_int8.h"
#include "../../include/marian_hip_ops.h"
#include "allocator.h"

namespace marian {
namespace hip {

#define HIP_CHECK(expr)                                                                     \
  do {                                                                                      \
    hipError_t e_ = (expr);                                                                 \
    if(e_ != hipSuccess) ::marian::hip::abortWith(std::string(#expr) + ": " + hipGetErrorString(e_)); \
  } while(0)

// The slab of one device.
class Device {
public:
  typedef hipStream_t Stream;
  explicit Device(int deviceNo, size_t alignment = 256) : deviceNo_(deviceNo), alignment_(alignment) {}
  ~Device() {
    // (no error checks: nothing can be done about them in a destructor)
    (void)hipSetDevice(deviceNo_);
    if(data_) (void)hipFree(data_);
  }
  Device(const Device&) = delete;
  Device& operator=(const Device&) = delete;

  // Grows the slab to `size` bytes (rounded up).  The content moves to a new address; pending work
  // on `stream` that uses the old one is waited for first.
  void reserve(size_t size, hipStream_t stream = nullptr) {
    size = alignUp(size, alignment_);
    HIP_CHECK(hipSetDevice(deviceNo_));
    if(size < size_ || size == 0) abortWith("New size must be larger than old size and larger than 0");
    if(size == size_) return;
    uint8_t* fresh = nullptr;
    if(!data_) {
      if(hipMalloc(reinterpret_cast<void**>(&fresh), size) != hipSuccess) {
        (void)hipGetLastError();
        abortWith("Out of device memory: cannot reserve " + std::to_string(size) + " bytes on device " + std::to_string(deviceNo_));
      }
    } else {
      HIP_CHECK(hipStreamSynchronize(stream));
      if(hipMalloc(reinterpret_cast<void**>(&fresh), size) == hipSuccess) {
        // (a failure from here on leaves the old slab in place and gives the new one back)
        hipError_t e = hipMemcpyAsync(fresh, data_, size_, hipMemcpyDeviceToDevice, stream);
        if(e == hipSuccess) e = hipStreamSynchronize(stream);
        if(e != hipSuccess) {
          (void)hipFree(fresh);
          abortWith(std::string("cannot copy the slab to its new place: ") + hipGetErrorString(e));
        }
        HIP_CHECK(hipFree(data_));
      } else {
        // not enough room for both: park the content in host memory while the slab is replaced
        (void)hipGetLastError();
        std::vector<uint8_t> parked(size_);
        HIP_CHECK(hipMemcpy(parked.data(), data_, size_, hipMemcpyDeviceToHost));
        HIP_CHECK(hipFree(data_));
        data_ = nullptr;
        if(hipMalloc(reinterpret_cast<void**>(&fresh), size) != hipSuccess) {
          (void)hipGetLastError();
          // put the old slab back so that the caller's tensors survive the failure; its address may
          // have changed (the allocator re-points its pieces when it sees the exception).  If even
          // that fails the device is left without a slab (size 0) and the allocator empties every piece.
          const size_t oldSize = size_;
          size_ = 0;
          if(hipMalloc(reinterpret_cast<void**>(&data_), oldSize) != hipSuccess) {
            (void)hipGetLastError();
            data_ = nullptr;
            abortWith("Out of device memory: the slab of " + std::to_string(oldSize) + " bytes could neither grow nor be put back");
          }
          size_ = oldSize;
          ++moves_;
          HIP_CHECK(hipMemcpy(data_, parked.data(), size_, hipMemcpyHostToDevice));
          abortWith("Out of device memory: cannot grow the slab from " + std::to_string(size_) + " to " + std::to_string(size) + " bytes");
        }
        hipError_t e = hipMemcpy(fresh, parked.data(), size_, hipMemcpyHostToDevice);
        if(e != hipSuccess) {
          (void)hipFree(fresh);
          size_ = 0;
          abortWith(std::string("cannot copy the parked slab back: ") + hipGetErrorString(e));
        }
      }
      ++moves_;
    }
    data_ = fresh;
    size_ = size;
  }

  uint8_t* data() const { return data_; }
  size_t size() const { return size_; }
  int deviceNo() const { return deviceNo_; }
  size_t moves() const { return moves_; }   // how often the slab has changed its address

private:
  int deviceNo_;
  size_t alignment_;
  uint8_t* data_ = nullptr;
  size_t size_ = 0;
  size_t moves_ = 0;
};

// The allocator on the device's slab (host/allocator.h holds the logic, which needs no GPU).
typedef BasicAllocator<Device> Allocator;

// gpu::copy (reference src/tensors/gpu/algorithm.cu:11-17): any direction, on the stream, then
// the stream is synchronised like in the reference.
template <typename T>
inline void copy(hipStream_t stream, const T* begin, const T* end, T* dest) {
  if(end == begin) return;
  HIP_CHECK(hipMemcpyAsync(dest, begin, (size_t)(end - begin) * sizeof(T), hipMemcpyDefault, stream));
  HIP_CHECK(hipStreamSynchronize(stream));
}

// gpu::fill (reference src/tensors/gpu/algorithm.cu:37-60), through the library's fill kernel.
template <typename T>
inline void fill(hipStream_t stream, T* begin, T* end, T value) {
  static_assert(sizeof(T) == 1 || sizeof(T) == 2 || sizeof(T) == 4 || sizeof(T) == 8, "element size");
  if(end == begin) return;
  uint64_t pattern = 0;
  std::memcpy(&pattern, &value, sizeof(T));
  int st = marian_hip_fill(begin, (int64_t)(end - begin), (int)sizeof(T), pattern, stream);
  if(st != MARIAN_HIP_OK) abortWith("marian_hip_fill failed with status " + std::to_string(st));
  HIP_CHECK(hipStreamSynchronize(stream));
}

}  // namespace hip
}  // namespace marian
