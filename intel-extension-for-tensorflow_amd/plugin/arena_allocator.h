// Device memory sub-allocator of the StreamExecutor plugin: best fit with coalescing over a few large
// regions obtained from the raw device allocator.  It plays the part of the reference's BFCAllocator
// (itex/core/devices/bfc_allocator.{h,cc}: 256-byte granularity :48-49, split :195-230, merge on free
// :375-377, region growth :274-330, ITEX_LIMIT_MEMORY_SIZE_IN_MB :253-267), laid out for a 288 GB device:
// regions start at 1 GiB and double up to 16 GiB, so a serving process ends up with a handful of
// hipMalloc calls; chunks are kept in two ordered maps (by address for neighbours, by size for best
// fit) instead of bins, which is exact best fit at O(log n).
// Host-only logic: the raw allocator is injected, so the unit tests run it over plain malloc.
#ifndef ITEX_AMD_ARENA_ALLOCATOR_H_
#define ITEX_AMD_ARENA_ALLOCATOR_H_

#include <cstddef>
#include <cstdint>
#include <functional>
#include <map>
#include <mutex>
#include <set>
#include <utility>
#include <vector>

namespace itex_amd {

struct ArenaStats {
  int64_t num_allocs = 0;          // successful Allocate calls so far
  int64_t bytes_in_use = 0;        // rounded bytes handed out and not yet returned
  int64_t peak_bytes_in_use = 0;
  int64_t largest_alloc_size = 0;
  int64_t bytes_reserved = 0;      // bytes held from the raw allocator
  int64_t peak_bytes_reserved = 0;
  int64_t bytes_limit = 0;         // 0: unlimited
  int64_t largest_free_block_bytes = 0;
  int64_t num_regions = 0;
};

class ArenaAllocator {
 public:
  using RawAlloc = std::function<void*(size_t)>;  // nullptr on failure
  using RawFree = std::function<void(void*)>;
  static constexpr size_t kAlign = 256;
  static constexpr size_t kFirstRegion = size_t{1} << 30;
  static constexpr size_t kMaxRegion = size_t{16} << 30;

  ArenaAllocator(RawAlloc raw_alloc, RawFree raw_free, size_t bytes_limit = 0, size_t first_region = kFirstRegion)
      : raw_alloc_(std::move(raw_alloc)), raw_free_(std::move(raw_free)), next_region_(RoundUp(first_region)) {
    stats_.bytes_limit = static_cast<int64_t>(bytes_limit);
  }
  ~ArenaAllocator() {
    for (const Region& r : regions_) raw_free_(r.base);
  }
  ArenaAllocator(const ArenaAllocator&) = delete;
  ArenaAllocator& operator=(const ArenaAllocator&) = delete;

  static size_t RoundUp(size_t n) { return n == 0 ? kAlign : (n + kAlign - 1) / kAlign * kAlign; }

  // nullptr when the request cannot be met (limit reached or the raw allocator is out of memory)
  void* Allocate(size_t bytes) {
    const size_t need = RoundUp(bytes);
    std::lock_guard<std::mutex> lock(mu_);
    auto it = free_by_size_.lower_bound({need, 0});
    if (it == free_by_size_.end()) {
      if (!Grow(need)) return nullptr;
      it = free_by_size_.lower_bound({need, 0});
      if (it == free_by_size_.end()) return nullptr;
    }
    const uintptr_t addr = it->second;
    const size_t have = it->first;
    free_by_size_.erase(it);
    Chunk& c = chunks_[addr];
    c.in_use = true;
    if (have - need >= kAlign) {  // split: the tail stays free
      c.size = need;
      Chunk tail{have - need, false, c.region};
      chunks_[addr + need] = tail;
      free_by_size_.insert({tail.size, addr + need});
    }
    stats_.num_allocs++;
    stats_.bytes_in_use += static_cast<int64_t>(c.size);
    if (stats_.bytes_in_use > stats_.peak_bytes_in_use) stats_.peak_bytes_in_use = stats_.bytes_in_use;
    if (static_cast<int64_t>(c.size) > stats_.largest_alloc_size) stats_.largest_alloc_size = static_cast<int64_t>(c.size);
    return reinterpret_cast<void*>(addr);
  }

  // false when `ptr` is not the start of a live allocation of this arena
  bool Deallocate(void* ptr) {
    if (ptr == nullptr) return true;
    std::lock_guard<std::mutex> lock(mu_);
    uintptr_t addr = reinterpret_cast<uintptr_t>(ptr);
    auto it = chunks_.find(addr);
    if (it == chunks_.end() || !it->second.in_use) return false;
    it->second.in_use = false;
    stats_.bytes_in_use -= static_cast<int64_t>(it->second.size);
    // merge with the free neighbours of the same region
    auto next = std::next(it);
    if (next != chunks_.end() && !next->second.in_use && next->second.region == it->second.region &&
        it->first + it->second.size == next->first) {
      free_by_size_.erase({next->second.size, next->first});
      it->second.size += next->second.size;
      chunks_.erase(next);
    }
    if (it != chunks_.begin()) {
      auto prev = std::prev(it);
      if (!prev->second.in_use && prev->second.region == it->second.region && prev->first + prev->second.size == it->first) {
        free_by_size_.erase({prev->second.size, prev->first});
        prev->second.size += it->second.size;
        chunks_.erase(it);
        it = prev;
      }
    }
    free_by_size_.insert({it->second.size, it->first});
    return true;
  }

  // size the arena reserved for the allocation that starts at `ptr`, 0 if unknown
  size_t AllocatedSize(const void* ptr) {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = chunks_.find(reinterpret_cast<uintptr_t>(ptr));
    return (it == chunks_.end() || !it->second.in_use) ? 0 : it->second.size;
  }

  ArenaStats stats() {
    std::lock_guard<std::mutex> lock(mu_);
    ArenaStats s = stats_;
    s.largest_free_block_bytes = free_by_size_.empty() ? 0 : static_cast<int64_t>(free_by_size_.rbegin()->first);
    s.num_regions = static_cast<int64_t>(regions_.size());
    return s;
  }

 private:
  struct Chunk {
    size_t size;
    bool in_use;
    int region;
  };
  struct Region {
    void* base;
    size_t size;
  };

  bool Grow(size_t need) {
    size_t want = next_region_ > need ? next_region_ : need;
    const size_t limit = static_cast<size_t>(stats_.bytes_limit);
    const size_t reserved = static_cast<size_t>(stats_.bytes_reserved);
    if (limit != 0) {
      if (reserved + need > limit) return false;
      if (reserved + want > limit) want = (limit - reserved) / kAlign * kAlign;  // still >= need
    }
    void* base = nullptr;
    // back off towards the request itself when the device cannot give a whole region any more
    for (;;) {
      base = raw_alloc_(want);
      if (base != nullptr || want == need) break;
      want = want / 2 > need ? RoundUp(want / 2) : need;
    }
    if (base == nullptr) return false;
    const int id = static_cast<int>(regions_.size());
    regions_.push_back({base, want});
    const uintptr_t addr = reinterpret_cast<uintptr_t>(base);
    chunks_[addr] = Chunk{want, false, id};
    free_by_size_.insert({want, addr});
    stats_.bytes_reserved += static_cast<int64_t>(want);
    if (stats_.bytes_reserved > stats_.peak_bytes_reserved) stats_.peak_bytes_reserved = stats_.bytes_reserved;
    if (next_region_ < kMaxRegion) next_region_ *= 2;
    return true;
  }

  RawAlloc raw_alloc_;
  RawFree raw_free_;
  std::mutex mu_;
  std::map<uintptr_t, Chunk> chunks_;                      // every chunk, by address
  std::set<std::pair<size_t, uintptr_t>> free_by_size_;    // free chunks, by (size, address)
  std::vector<Region> regions_;
  size_t next_region_;
  ArenaStats stats_;
};

}  // namespace itex_amd
#endif  // ITEX_AMD_ARENA_ALLOCATOR_H_
