// Check program for host/allocator.h on the CPU: the allocator on a malloc-backed slab, driven
// by a seeded random sequence of alloc / free / grow / clear / exhaustion / failing-device steps
// and compared after every step with a plain model (the list of handed-out intervals).  Needs no
// GPU and no HIP; meant to be built with -fsanitize=address,undefined, so that a piece that
// points into a freed slab, an iterator used after erase or an overflow in the offset arithmetic
// stops the run.
//
//   allocator_check [seed] [steps]
//
// Behaviours checked against the reference (src/tensors/allocator.h): sizes rounded up to the
// alignment (:167-170), best fit with the lowest address among equal gaps (std::set<Gap>, :43-46,
// :113-116), grow moves the slab and re-points every piece (:93-115), AllocationException instead
// of growing after throwAtReallocation (:121-124), free merges neighbouring gaps (:139-155),
// "Double free?" (:205), clear (:236-241).
#include <cstring>
#include <random>
#include <vector>

#include "allocator.h"

using namespace marian::hip;

namespace {

// A slab in host memory.  reserve() always moves it (the new block is taken before the old one is
// given back).  failNext: 1 = the next reserve fails and the slab stays; 2 = fails, and the slab of
// the old size has moved; 3 = fails and the slab is lost.
class HostDevice {
public:
  typedef int Stream;
  explicit HostDevice(size_t alignment) : alignment_(alignment) {}
  ~HostDevice() { std::free(data_); }
  HostDevice(const HostDevice&) = delete;
  HostDevice& operator=(const HostDevice&) = delete;

  void reserve(size_t size, Stream) {
    size = alignUp(size, alignment_);
    if(size < size_ || size == 0) abortWith("New size must be larger than old size and larger than 0");
    if(size == size_) return;
    const int fail = failNext;
    failNext = 0;
    if(fail == 1) abortWith("Out of device memory (slab untouched)");
    if(fail == 2) {
      move(size_);
      abortWith("Out of device memory (slab put back at a new address)");
    }
    if(fail == 3) {
      std::free(data_);
      data_ = nullptr;
      size_ = 0;
      abortWith("Out of device memory (slab lost)");
    }
    move(size);
  }
  uint8_t* data() const { return data_; }
  size_t size() const { return size_; }
  size_t moves() const { return moves_; }
  int failNext = 0;

private:
  void move(size_t size) {
    uint8_t* fresh = static_cast<uint8_t*>(std::aligned_alloc(alignment_, size));
    if(!fresh) abortWith("host memory exhausted");
    std::memset(fresh, 0xEE, size);
    if(data_) std::memcpy(fresh, data_, size_ < size ? size_ : size);
    std::free(data_);
    data_ = fresh;
    size_ = size;
    ++moves_;
  }
  size_t alignment_;
  uint8_t* data_ = nullptr;
  size_t size_ = 0;
  size_t moves_ = 0;
};

typedef BasicAllocator<HostDevice> Allocator;

struct Held {
  MemoryPiece::PtrType piece;
  size_t offset, size;
  uint8_t pattern;
};

long failures = 0;
void expect(bool ok, const char* what, long step) {
  if(ok) return;
  std::printf("  step %ld: %s FAILED\n", step, what);
  ++failures;
}

// The maximal free intervals of [0, slab) given the handed-out ones.
std::vector<std::pair<size_t, size_t>> freeIntervals(const std::vector<Held>& held, size_t slab) {
  std::map<size_t, size_t> used;
  for(const Held& h : held) used[h.offset] = h.size;
  std::vector<std::pair<size_t, size_t>> out;
  size_t at = 0;
  for(const auto& u : used) {
    if(u.first > at) out.emplace_back(at, u.first - at);
    at = u.first + u.second;
  }
  if(slab > at) out.emplace_back(at, slab - at);
  return out;
}

void checkState(const Allocator& al, const std::vector<Held>& held, long step) {
  const auto gaps = freeIntervals(held, al.size());
  size_t avail = 0;
  for(const auto& g : gaps) avail += g.second;
  expect(al.gaps() == gaps.size(), "number of gaps = maximal free intervals of the model", step);
  expect(al.available() == avail, "available() = free bytes of the model", step);
  expect(al.pieces() == held.size(), "pieces() = handed-out pieces of the model", step);
  std::map<size_t, size_t> seen;
  for(const Held& h : held) {
    expect(h.piece->data() == al.device()->data() + h.offset, "piece points at its offset of the current slab", step);
    expect(h.piece->size() == h.size, "piece keeps its size", step);
    expect(h.offset % 256 == 0 && h.offset + h.size <= al.size(), "piece is aligned and inside the slab", step);
    bool same = true;
    for(size_t i = 0; i < h.size; i += 97) same = same && h.piece->data()[i] == h.pattern;
    same = same && h.piece->data()[h.size - 1] == h.pattern;
    expect(same, "piece keeps its bytes", step);
    seen[h.offset] = h.size;
  }
  size_t at = 0;
  for(const auto& s : seen) {
    expect(s.first >= at, "pieces do not overlap", step);
    at = s.first + s.second;
  }
}

}  // namespace

int main(int argc, char** argv) {
  const unsigned seed = argc > 1 ? (unsigned)std::strtoul(argv[1], nullptr, 10) : 1u;
  const long steps = argc > 2 ? std::strtol(argv[2], nullptr, 10) : 20000;
  const size_t kStep = 64u << 10, kLimit = 3u << 20;
  std::mt19937 rng(seed);
  auto device = std::make_shared<HostDevice>(256);
  Allocator al(device, 0, kStep, 256, kLimit);
  std::vector<Held> held;
  uint8_t nextPattern = 1;
  long grows = 0, refusals = 0, failedGrows = 0;
  expect(al.size() == 0 && al.available() == 0 && al.gaps() == 0, "empty allocator: no slab yet", 0);

  for(long step = 1; step <= steps; ++step) {
    const unsigned op = rng() % 1000;
    if(op < 560 || held.empty()) {
      // ---- alloc: mostly small, now and then larger than a growth step ----
      size_t bytes = 1 + rng() % 5000;
      if(rng() % 16 == 0) bytes = 1 + rng() % (192u << 10);
      const size_t rounded = alignUp(bytes, 256);
      // the model's choice: smallest maximal free interval that fits, lowest offset among equals
      const auto gaps = freeIntervals(held, al.size());
      bool fits = false;
      size_t best = 0, bestSize = 0;
      for(const auto& g : gaps)
        if(g.second >= rounded && (!fits || g.second < bestSize)) {
          fits = true;
          best = g.first;
          bestSize = g.second;
        }
      const size_t before = al.size(), movesBefore = device->moves();
      const size_t grownTo = before + (kStep > rounded ? kStep : rounded);
      size_t expectAt = best;
      if(!fits) {
        // grows by max(step, request); the new room merges with a free tail of the old slab
        size_t tail = before;
        if(!gaps.empty() && gaps.back().first + gaps.back().second == before) tail = gaps.back().first;
        expectAt = tail;
      }
      if(!fits && grownTo > kLimit) {
        bool refused = false;
        try {
          al.alloc(bytes);
        } catch(const std::runtime_error& e) {
          refused = std::strstr(e.what(), "Out of memory") != nullptr;
        }
        expect(refused && al.size() == before && device->moves() == movesBefore, "beyond the limit: an error, nothing changes", step);
        ++refusals;
      } else if(!fits && rng() % 3 == 0) {
        // ---- the same request with throwAtReallocation, then with a device that cannot grow ----
        al.throwAtReallocation(true);
        bool threw = false;
        try {
          al.alloc(bytes);
        } catch(const AllocationException&) {
          threw = true;
        }
        al.throwAtReallocation(false);
        expect(threw && al.size() == before, "throwAtReallocation: AllocationException instead of growing", step);
        const int mode = 1 + (int)(rng() % 3);
        if(mode == 3 && rng() % 4 != 0) continue;   // (losing the slab empties everything: keep it rare)
        device->failNext = mode;
        bool failed = false;
        try {
          al.alloc(bytes);
        } catch(const std::runtime_error&) {
          failed = true;
        }
        ++failedGrows;
        expect(failed, "a device that cannot grow: the error reaches the caller", step);
        if(mode == 3) {
          bool emptied = al.size() == 0 && al.pieces() == 0 && al.available() == 0;
          for(const Held& h : held) emptied = emptied && !h.piece->data() && h.piece->size() == 0;
          expect(emptied, "slab lost: every piece is emptied, the allocator starts over", step);
          held.clear();
        } else {
          expect(al.size() == before && (mode == 1 || device->moves() == movesBefore + 1),
                 "failed grow: the slab keeps its size (and may have moved)", step);
        }
      } else {
        auto piece = al.alloc(bytes);
        if(!fits) {
          ++grows;
          expect(al.size() == grownTo && device->moves() == movesBefore + 1, "grow adds max(step, request) and moves the slab", step);
        } else {
          expect(al.size() == before && device->moves() == movesBefore, "a request that fits does not grow", step);
        }
        expect(piece->size() == rounded, "size rounded up to 256", step);
        expect((size_t)(piece->data() - device->data()) == expectAt, "best fit: the model's gap", step);
        Held h{piece, (size_t)(piece->data() - device->data()), rounded, nextPattern};
        nextPattern = (uint8_t)(nextPattern == 255 ? 1 : nextPattern + 1);
        std::memset(piece->data(), h.pattern, rounded);
        held.push_back(h);
      }
    } else if(op < 950) {
      // ---- free a random piece ----
      const size_t i = rng() % held.size();
      Held h = held[i];
      held[i] = held.back();
      held.pop_back();
      expect(al.free(h.piece), "free of a handed-out piece", step);
      expect(!h.piece->data() && h.piece->size() == 0, "free empties the handle", step);
      bool doubleFree = false;
      try {
        al.free(h.piece);
      } catch(const std::runtime_error& e) {
        doubleFree = std::strstr(e.what(), "Double free?") != nullptr;
      }
      expect(doubleFree, "freeing it again: Double free?", step);
    } else if(op < 960) {
      // ---- a piece that is not this allocator's ----
      std::vector<uint8_t> elsewhere(512);
      auto foreign = MemoryPiece::New(elsewhere.data(), 256);
      expect(!al.free(foreign) && foreign->data() == elsewhere.data(), "free of a foreign piece is refused", step);
    } else if(op < 998) {
      // ---- an explicit grow ----
      if(al.size() + kStep <= kLimit) {
        const size_t before = al.size();
        al.grow(1);
        expect(al.size() == before + 256, "grow(1) adds one aligned unit", step);
      }
    } else if(op < 999) {
      al.clear();
      bool emptied = al.pieces() == 0 && al.available() == al.size() && al.gaps() == (al.size() ? 1u : 0u);
      for(const Held& h : held) emptied = emptied && !h.piece->data();
      expect(emptied, "clear forgets every piece: one gap, the whole slab", step);
      held.clear();
    } else {
      // ---- reserve: at least that large, and forgets everything ----
      const size_t want = al.size() + (rng() % 2) * 1024;
      if(want > 0 && want <= kLimit) {
        al.reserve(want);
        expect(al.size() >= want && al.pieces() == 0 && al.available() == al.size(), "reserve: large enough, empty", step);
        for(const Held& h : held) expect(!h.piece->data(), "reserve empties the handles", step);
        held.clear();
      }
    }
    checkState(al, held, step);
    if(failures > 20) break;
  }
  std::printf("allocator_check: seed %u, %ld steps, slab %zu bytes after %zu moves (%ld grows, %ld refusals at the limit, "
              "%ld failed grows), %zu pieces held, %ld failure(s) -> %s\n",
              seed, steps, al.size(), device->moves(), grows, refusals, failedGrows, held.size(), failures,
              failures == 0 ? "OK" : "FAILED");
  return failures == 0 ? 0 : 1;
}
