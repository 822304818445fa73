// C entry points around the plugin's ArenaAllocator for the CPU unit tests: the raw allocator is plain
// aligned host memory and can be told to fail above a total, like a device that runs out of memory.
#include <cstdlib>

#include <memory>

#include "arena_allocator.h"

using itex_amd::ArenaAllocator;
using itex_amd::ArenaStats;

namespace {
struct Harness {
  size_t raw_total = 0, raw_capacity = 0;
  int raw_allocs = 0, raw_frees = 0;
  std::map<void*, size_t> raw_live;
  std::unique_ptr<ArenaAllocator> arena;
};
}  // namespace

extern "C" {
void* arena_new(uint64_t limit, uint64_t first_region, uint64_t raw_capacity) {
  auto* h = new Harness;
  h->raw_capacity = raw_capacity;
  h->arena.reset(new ArenaAllocator(
      [h](size_t n) -> void* {
        if (h->raw_capacity && h->raw_total + n > h->raw_capacity) return nullptr;
        void* p = std::aligned_alloc(4096, (n + 4095) / 4096 * 4096);
        if (!p) return nullptr;
        h->raw_total += n;
        h->raw_allocs++;
        h->raw_live[p] = n;
        return p;
      },
      [h](void* p) {
        h->raw_total -= h->raw_live[p];
        h->raw_live.erase(p);
        h->raw_frees++;
        std::free(p);
      },
      limit, first_region));
  return h;
}
void* arena_alloc(void* h, uint64_t n) { return static_cast<Harness*>(h)->arena->Allocate(n); }
int arena_free(void* h, void* p) { return static_cast<Harness*>(h)->arena->Deallocate(p) ? 0 : 1; }
uint64_t arena_allocated_size(void* h, void* p) { return static_cast<Harness*>(h)->arena->AllocatedSize(p); }
void arena_stats(void* h, int64_t* out /* 9 values */) {
  const ArenaStats s = static_cast<Harness*>(h)->arena->stats();
  out[0] = s.num_allocs; out[1] = s.bytes_in_use; out[2] = s.peak_bytes_in_use; out[3] = s.largest_alloc_size;
  out[4] = s.bytes_reserved; out[5] = s.peak_bytes_reserved; out[6] = s.bytes_limit; out[7] = s.largest_free_block_bytes;
  out[8] = s.num_regions;
}
void arena_raw_counts(void* h, int64_t* out /* allocs, frees, live bytes */) {
  auto* hh = static_cast<Harness*>(h);
  out[0] = hh->raw_allocs; out[1] = hh->raw_frees; out[2] = static_cast<int64_t>(hh->raw_total);
}
// destroys the arena (which must return every region) and reports raw allocations still alive
int arena_delete(void* h) {
  auto* hh = static_cast<Harness*>(h);
  hh->arena.reset();
  const int leaked = static_cast<int>(hh->raw_live.size());
  delete hh;
  return leaked;
}
}
