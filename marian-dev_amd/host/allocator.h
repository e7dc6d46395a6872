// The allocator of a HIP backend of Marian, independent of where the slab lives: it carves
// 256-byte aligned pieces out of ONE contiguous slab that a Device object owns and grows.
//
// Counterparts (reference file:line):
//   src/tensors/memory_piece.h:9-59      MemoryPiece
//   src/tensors/allocator.h:18-33        AllocationException
//   src/tensors/allocator.h:81-257       Allocator (gaps, best fit, grow, free, clear)
//
// What is kept: the contract.  Sizes are rounded up to the alignment; an allocation takes the
// smallest gap that is large enough (the lowest one among equals, `std::set<Gap>` order of the
// reference); one that fits no gap grows the slab or, after throwAtReallocation(true), throws
// AllocationException; growing MOVES the slab and re-points every handed-out MemoryPiece; free()
// merges the gap with its neighbours; clear() forgets every piece.
// What is different: gaps and pieces are kept as OFFSETS into the slab - a map by offset
// (neighbours for merging are found by lookup, not by a scan over all gaps) and a set by
// (size, offset) - so a move re-points the handed-out pieces and nothing else; an optional byte
// limit makes exhaustion an error a caller (and a test) can provoke and handle.
//
// DeviceT provides: typedef Stream; void reserve(size_t bytes, Stream) (grow only; may move the
// slab; throws when it cannot, leaving a slab of the old size - possibly at a new address - or no
// slab at all); uint8_t* data(); size_t size().  The class is a template so that the same code
// runs on a malloc-backed slab under the host sanitizers (host/allocator_check.cpp).
#pragma once

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <memory>
#include <set>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <utility>

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

// What Allocator throws instead of growing after throwAtReallocation(true)
// (reference src/tensors/allocator.h:18-33).
class AllocationException : public std::runtime_error {
public:
  AllocationException(size_t available, size_t asked)
      : std::runtime_error("Attempted allocation of " + std::to_string(asked) + ", but only " +
                           std::to_string(available) + " free") {}
};

inline size_t alignUp(size_t size, size_t alignment) { return (size + alignment - 1) / alignment * alignment; }

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

template <class DeviceT>
class BasicAllocator {
public:
  typedef typename DeviceT::Stream Stream;

  // bytes: initial slab; step: growth per exhaustion; limit: the slab never exceeds it (0 = none)
  BasicAllocator(std::shared_ptr<DeviceT> device, size_t bytes, size_t step, size_t alignment = 256,
                 size_t limit = 0, Stream stream = Stream())
      : device_(std::move(device)), step_(step), alignment_(alignment), limit_(limit), stream_(stream) {
    reserve(bytes);
  }

  size_t alignedSize(size_t size) const { return alignUp(size, alignment_); }
  void throwAtReallocation(bool flag) { throw_ = flag; }

  // Makes the slab at least `bytes` large and forgets every allocation (reference :172-177).
  void reserve(size_t bytes) {
    bytes = alignedSize(bytes);
    if(bytes > device_->size()) {
      try {
        growDevice(bytes);
      } catch(...) {
        clear();   // whatever slab is left holds no piece any more
        throw;
      }
    }
    clear();
  }

  MemoryPiece::PtrType alloc(size_t bytes) {
    bytes = alignedSize(bytes == 0 ? 1 : bytes);
    auto fit = bySize_.lower_bound(std::make_pair(bytes, (size_t)0));   // best fit, lowest offset among equals
    if(fit == bySize_.end() && throw_) throw AllocationException(available_, bytes);
    while(fit == bySize_.end()) {
      grow(step_ > bytes ? step_ : bytes);
      fit = bySize_.lower_bound(std::make_pair(bytes, (size_t)0));
    }
    const size_t gapSize = fit->first, offset = fit->second;
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
  const std::shared_ptr<DeviceT>& device() const { return device_; }
  // Calls fn(offset, size) for every gap, lowest offset first.
  template <class Fn>
  void forEachGap(Fn fn) const {
    for(const auto& g : byOffset_) fn(g.first, g.second);
  }

  // Grows the slab by `add` bytes: the new room becomes a gap (merged with a gap that ends where
  // the old slab ended) and every handed-out piece is re-pointed into the moved slab.  If the
  // device cannot grow, the exception passes through with the allocator still consistent: the
  // pieces point into the slab the device is left with (it may have moved all the same), or, if
  // the device lost its slab altogether, every piece is emptied like after clear().
  void grow(size_t add) {
    add = alignedSize(add);
    const size_t oldSize = device_->size();
    try {
      growDevice(oldSize + add);
    } catch(...) {
      if(device_->size() == oldSize) repoint();
      else clear();
      throw;
    }
    insertGap(oldSize, device_->size() - oldSize, /*merge=*/true);
    repoint();
  }

private:
  void repoint() {
    uint8_t* base = device_->data();
    for(auto& p : pieces_) p.second->setPtr(base + p.first);
  }
  void growDevice(size_t size) {
    if(limit_ && size > limit_)
      abortWith("Out of memory: the allocator's limit of " + std::to_string(limit_) + " bytes does not allow a slab of " + std::to_string(size));
    device_->reserve(size, stream_);
  }
  void eraseGap(size_t offset) {
    auto it = byOffset_.find(offset);
    bySize_.erase(std::make_pair(it->second, offset));
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

  std::shared_ptr<DeviceT> device_;
  size_t step_, alignment_, limit_;
  Stream stream_;
  bool throw_ = false;
  size_t available_ = 0;
  std::map<size_t, size_t> byOffset_;                       // gap offset -> size
  std::set<std::pair<size_t, size_t>> bySize_;              // (gap size, offset)
  std::unordered_map<size_t, MemoryPiece::PtrType> pieces_; // piece offset -> handle
};

}  // namespace hip
}  // namespace marian
