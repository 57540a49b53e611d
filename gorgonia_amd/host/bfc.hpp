// Best-Fit-with-Coalescing arena bookkeeping over one device reservation.
// Re-implements the observable behaviour of cuda/bfc.go (bfc, freelist,
// memblock) on top of an address-ordered std::map instead of a hand-linked
// list: the same offsets come back for the same alloc/free sequence, the free
// list has the same blocks, and the same coalescing rules apply.
//
//   alloc(size):  first block in address order whose size >= align(size)
//                 (cuda/bfc.go:413-420 - "best fit" is first fit); the block is
//                 cut to the aligned size and then to the requested size, both
//                 remnants go back on the free list (cuda/bfc.go:246-256)
//   free(addr):   unknown addresses are ignored (cuda/bfc.go:394-401); the
//                 freed block re-enters the list; when frees/allocs >= 0.75 the
//                 list is coalesced (cuda/bfc.go:408-410)
//   coalesce():   starting only from blocks whose offset is a multiple of the
//                 alignment, merge every directly adjacent successor
//                 (cuda/bfc.go:425-458)
//   out of memory: coalesce once and retry, then report reserved/allocated
//                 (cuda/bfc.go:363-372, cuda/errors.go:6-13)
#pragma once
#include <cstdint>
#include <map>
#include <string>
#include <unordered_map>
#include <vector>

namespace gorgonia {

struct OomError {
  int64_t reserved = 0;
  int64_t allocated = 0;
};

class BFC {
 public:
  explicit BFC(int64_t alignment = 32) : block_size_(alignment) {}

  // cuda/bfc.go:335-343
  void reserve(uint64_t start, int64_t size);
  // cuda/bfc.go:345-352; returns the start address that was reserved
  uint64_t release();
  // cuda/bfc.go:354-385. Returns 0 on success, 1 for size <= 0, 2 for out of
  // memory (oom filled in).  *addr is start + offset.
  int alloc(int64_t size, uint64_t* addr, OomError* oom = nullptr);
  // cuda/bfc.go:387-411
  void free(uint64_t address);
  void coalesce();
  // cuda/bfc.go:327-333: statistics only
  void reset_stats() { allocated_ = 0; allocs_ = 0; frees_ = 0; }
  // Engine.ResetAllocator (cuda/arena.go:25-36): free everything in use,
  // coalesce, reset statistics.
  void reset_allocator();

  int64_t align(int64_t size) const;  // cuda/bfc.go:460-467
  int freelist_len() const { return (int)free_.size(); }
  std::vector<std::pair<uint64_t, int64_t>> freelist() const;  // (offset, size) in address order
  std::string freelist_string() const;
  int64_t allocated() const { return allocated_; }
  int64_t size() const { return size_; }
  int64_t reserved_size() const { return reserved_size_; }
  uint64_t start() const { return start_; }
  int used_count() const { return (int)used_.size(); }
  int allocs() const { return allocs_; }
  int frees() const { return frees_; }

 private:
  void insert(uint64_t off, int64_t size);
  uint64_t start_ = 0;
  int64_t size_ = 0;
  int64_t block_size_;
  int64_t reserved_size_ = 0;
  std::map<uint64_t, int64_t> free_;            // offset -> size
  std::unordered_map<uint64_t, int64_t> used_;  // offset -> requested size
  int64_t allocated_ = 0;
  int allocs_ = 0;
  int frees_ = 0;
};

}  // namespace gorgonia
