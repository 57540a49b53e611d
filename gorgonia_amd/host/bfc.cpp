#include "bfc.hpp"

#include <sstream>

namespace gorgonia {

void BFC::reserve(uint64_t start, int64_t size) {
  start_ = start;
  size_ = size - (size % block_size_);
  reserved_size_ = size;
  insert(0, size);
}

uint64_t BFC::release() {
  uint64_t r = start_;
  start_ = 0;
  size_ = 0;
  free_.clear();
  used_.clear();
  return r;
}

int64_t BFC::align(int64_t size) const {
  const int64_t rem = size % block_size_;
  return rem == 0 ? size : size - rem + block_size_;
}

// Ordered insert.  In correct use a freed block never overlaps a free one
// (the used map rejects double frees), so the reference's overlap-merging
// branches (cuda/bfc.go:125-218) reduce to a plain insert; a block that does
// overlap an existing free block is merged into it rather than duplicated.
void BFC::insert(uint64_t off, int64_t size) {
  if (size <= 0) return;
  auto next = free_.lower_bound(off);
  if (next != free_.begin()) {
    auto prev = std::prev(next);
    if (prev->first + (uint64_t)prev->second > off) {  // overlaps predecessor
      const uint64_t cap = off + (uint64_t)size, pcap = prev->first + (uint64_t)prev->second;
      if (cap > pcap) prev->second += (int64_t)(cap - pcap);
      return;
    }
  }
  if (next != free_.end() && (next->first == off || off + (uint64_t)size > next->first)) {
    const uint64_t cap = off + (uint64_t)size, ncap = next->first + (uint64_t)next->second;
    const int64_t merged = (int64_t)((cap > ncap ? cap : ncap) - off);
    free_.erase(next);
    free_[off] = merged;
    return;
  }
  free_[off] = size;
}

int BFC::alloc(int64_t size, uint64_t* addr, OomError* oom) {
  if (size <= 0) return 1;  // "Cannot allocate memory with size 0 or less"
  const int64_t aligned = align(size);
  auto fit = [&]() {
    for (auto it = free_.begin(); it != free_.end(); ++it)
      if (it->second >= aligned) return it;
    return free_.end();
  };
  auto it = fit();
  if (it == free_.end()) {
    coalesce();
    it = fit();
    if (it == free_.end()) {
      if (oom) { oom->reserved = size_; oom->allocated = allocated_; }
      return 2;
    }
  }
  const uint64_t off = it->first;
  const int64_t bsize = it->second;
  free_.erase(it);
  if (bsize > aligned) insert(off + (uint64_t)aligned, bsize - aligned);
  if (aligned > size) insert(off + (uint64_t)size, aligned - size);
  used_[off] = size;
  allocated_ += size;
  allocs_++;
  if (addr) *addr = off + start_;
  return 0;
}

void BFC::free(uint64_t address) {
  const uint64_t off = address - start_;
  auto it = used_.find(off);
  if (it == used_.end()) return;  // unknown address: silently ignored
  const int64_t size = it->second;
  used_.erase(it);
  insert(off, size);
  allocated_ -= size;
  frees_++;
  if (allocs_ > 0 && (double)frees_ / (double)allocs_ >= 0.75) coalesce();
}

void BFC::coalesce() {
  for (auto it = free_.begin(); it != free_.end(); ++it) {
    if (it->first % (uint64_t)block_size_ != 0) continue;
    for (auto next = std::next(it); next != free_.end(); next = std::next(it)) {
      if (it->first + (uint64_t)it->second != next->first) break;
      it->second += next->second;
      free_.erase(next);
    }
  }
}

void BFC::reset_allocator() {
  std::vector<uint64_t> offs;
  offs.reserve(used_.size());
  for (auto& kv : used_) offs.push_back(kv.first);
  for (uint64_t o : offs) free(o + start_);
  coalesce();
  reset_stats();
}

std::vector<std::pair<uint64_t, int64_t>> BFC::freelist() const {
  return std::vector<std::pair<uint64_t, int64_t>>(free_.begin(), free_.end());
}

std::string BFC::freelist_string() const {
  std::ostringstream os;
  os << "[";
  for (auto& kv : free_) os << "{0x" << std::hex << kv.first << std::dec << " " << kv.second << "}, ";
  os << "]";
  return os.str();
}

}  // namespace gorgonia
