// Device memory for a HIP backend of Marian: one slab per device, an allocator that carves
// 256-byte aligned pieces out of it, and copy/fill on the backend's stream.
//
// Counterparts (reference file:line):
//   src/tensors/device.h:10-36, src/tensors/gpu/device.cu:19-41   Device / gpu::Device::reserve
//   src/tensors/memory_piece.h:9-59                               MemoryPiece
//   src/tensors/allocator.h:81-257                                Allocator (gaps, grow, free, clear)
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
//   * gaps and pieces are kept as OFFSETS into the slab, in a map by offset (neighbours for merging
//     are found by lookup, not by a scan over all gaps) and a multimap by size (best fit by
//     lower_bound), so a move re-points the handed-out pieces and nothing else;
//   * an optional byte limit per allocator, so that exhaustion is an error a caller (and a test)
//     can provoke and handle without asking the driver for all of the device's memory.
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
#define HIP_CHECK(expr)                                                                     \
  do {                                                                                      \
    hipError_t e_ = (expr);                                                                 \
    if(e_ != hipSuccess) ::marian::hip::abortWith(std::string(#expr) + ": " + hipGetErrorString(e_)); \
  } while(0)

// What Allocator throws instead of growing after throwAtReallocation(true)
// (reference src/tensors/allocator.h:18-33).
class AllocationException : public std::runtime_error {
public:
  AllocationException(size_t available, size_t asked)
      : std::runtime_error("Attempted allocation of " + std::to_string(asked) + ", but only " +
                           std::to_string(available) + " free") {}
};

inline size_t alignUp(size_t size, size_t alignment) { return (size + alignment - 1) / alignment * alignment; }

// The slab of one device.
class Device {
public:
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
        HIP_CHECK(hipMemcpyAsync(fresh, data_, size_, hipMemcpyDeviceToDevice, stream));
        HIP_CHECK(hipStreamSynchronize(stream));
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
          // put the old slab back so that the caller's tensors survive the failure
          HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&data_), size_));
          HIP_CHECK(hipMemcpy(data_, parked.data(), size_, hipMemcpyHostToDevice));
          ++moves_;   // (the address may have changed all the same)
          abortWith("Out of device memory: cannot grow the slab from " + std::to_string(size_) + " to " + std::to_string(size) + " bytes");
        }
        HIP_CHECK(hipMemcpy(fresh, parked.data(), size_, hipMemcpyHostToDevice));
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

// A piece of the slab.  Holders keep the handle, never the raw pointer: data() is valid until the
// next call that may grow the slab.
class MemoryPiece {
public:
  typedef std::shared_ptr<MemoryPiece> PtrType;
  static PtrType New(uint8_t* data, size_t size) { return PtrType(new MemoryPiece(data, size)); }
  uint8_t* data() const { return data_; }
  template <typename T>
  T* data() const { return reinterpret_cast<T*>(data_); }
  size_t size() const { return size_; }
  void set(uint8_t* data, size_t size) { data_ = data; size_ = size; }
  void setPtr(uint8_t* data) { data_ = data; }

private:
  MemoryPiece(uint8_t* data, size_t size) : data_(data), size_(size) {}
  uint8_t* data_;
  size_t size_;
};

class Allocator {
public:
  // bytes: initial slab; step: growth per exhaustion; limit: the slab never exceeds it (0 = none)
  Allocator(std::shared_ptr<Device> device, size_t bytes, size_t step, size_t alignment = 256,
            size_t limit = 0, hipStream_t stream = nullptr)
      : device_(std::move(device)), step_(step), alignment_(alignment), limit_(limit), stream_(stream) {
    reserve(bytes);
  }

  size_t alignedSize(size_t size) const { return alignUp(size, alignment_); }
  void throwAtReallocation(bool flag) { throw_ = flag; }

  // Makes the slab at least `bytes` large and forgets every allocation (reference :172-177).
  void reserve(size_t bytes) {
    bytes = alignedSize(bytes);
    if(bytes > device_->size()) growDevice(bytes);
    clear();
  }

  MemoryPiece::PtrType alloc(size_t bytes) {
    bytes = alignedSize(bytes == 0 ? 1 : bytes);
    auto fit = bySize_.lower_bound(bytes);   // best fit: the smallest gap that is large enough
    if(fit == bySize_.end() && throw_) throw AllocationException(available_, bytes);
    while(fit == bySize_.end()) {
      grow(step_ > bytes ? step_ : bytes);
      fit = bySize_.lower_bound(bytes);
    }
    const size_t offset = fit->second, gapSize = fit->first;
    eraseGap(offset);
    if(gapSize > bytes) insertGap(offset + bytes, gapSize - bytes, /*merge=*/false);
    auto piece = MemoryPiece::New(device_->data() + offset, bytes);
    pieces_[offset] = piece;
    return piece;
  }
  template <typename T>
  MemoryPiece::PtrType alloc(size_t num) { return alloc(num * sizeof(T)); }

  bool free(const MemoryPiece::PtrType& piece) {
    if(!piece || !piece->data()) abortWith("Double free?");
    const size_t offset = (size_t)(piece->data() - device_->data());
    auto it = pieces_.find(offset);
    if(it == pieces_.end() || it->second != piece) return false;
    pieces_.erase(it);
    insertGap(offset, piece->size(), /*merge=*/true);
    piece->set(nullptr, 0);
    return true;
  }

  void clear() {
    for(auto& p : pieces_) p.second->set(nullptr, 0);
    pieces_.clear();
    byOffset_.clear();
    bySize_.clear();
    available_ = 0;
    if(device_->size() > 0) insertGap(0, device_->size(), false);
  }

  MemoryPiece::PtrType memory() const { return MemoryPiece::New(device_->data(), device_->size()); }
  size_t size() const { return device_->size(); }
  size_t available() const { return available_; }
  size_t gaps() const { return byOffset_.size(); }
  size_t pieces() const { return pieces_.size(); }
  const std::shared_ptr<Device>& device() const { return device_; }

  // Grows the slab by `add` bytes: the new room becomes a gap (merged with a gap that ends where
  // the old slab ended) and every handed-out piece is re-pointed into the moved slab.
  void grow(size_t add) {
    add = alignedSize(add);
    const size_t oldSize = device_->size();
    growDevice(oldSize + add);
    insertGap(oldSize, device_->size() - oldSize, /*merge=*/true);
    uint8_t* base = device_->data();
    for(auto& p : pieces_) p.second->setPtr(base + p.first);
  }

private:
  void growDevice(size_t size) {
    if(limit_ && size > limit_)
      abortWith("Out of memory: the allocator's limit of " + std::to_string(limit_) + " bytes does not allow a slab of " + std::to_string(size));
    device_->reserve(size, stream_);
  }
  void eraseGap(size_t offset) {
    auto it = byOffset_.find(offset);
    auto range = bySize_.equal_range(it->second);
    for(auto s = range.first; s != range.second; ++s)
      if(s->second == offset) {
        bySize_.erase(s);
        break;
      }
    available_ -= it->second;
    byOffset_.erase(it);
  }
  void insertGap(size_t offset, size_t size, bool merge) {
    if(merge) {
      auto next = byOffset_.find(offset + size);          // a gap that starts where this one ends
      if(next != byOffset_.end()) {
        size += next->second;
        eraseGap(next->first);
      }
      auto after = byOffset_.lower_bound(offset);          // the gap in front, if it ends here
      if(after != byOffset_.begin()) {
        auto prev = std::prev(after);
        if(prev->first + prev->second == offset) {
          offset = prev->first;
          size += prev->second;
          eraseGap(offset);
        }
      }
    }
    byOffset_[offset] = size;
    bySize_.emplace(size, offset);
    available_ += size;
  }

  std::shared_ptr<Device> device_;
  size_t step_, alignment_, limit_;
  hipStream_t stream_;
  bool throw_ = false;
  size_t available_ = 0;
  std::map<size_t, size_t> byOffset_;                       // gap offset -> size
  std::multimap<size_t, size_t> bySize_;                    // gap size -> offset
  std::unordered_map<size_t, MemoryPiece::PtrType> pieces_; // piece offset -> handle
};

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
