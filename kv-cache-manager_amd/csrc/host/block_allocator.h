// Physical page ids of one cache group: a LIFO free list plus a reference count per page.
// The page freed last is handed out first, so under pressure pages are reused at once.
// Behaviour follows the reference allocator (src/core/block_allocator.h:8-33,
// src/core/block_allocator.cpp:7-46); misuse throws std::logic_error.
#pragma once
#include <cstdint>
#include <stdexcept>
#include <vector>

namespace kvcm {

class BlockAllocator {
 public:
  explicit BlockAllocator(int num_blocks) : refs_(num_blocks, 0), parked_(num_blocks, 1) {
    free_.resize(num_blocks);
    // ids come out as 0, 1, 2, ... from a fresh pool
    for (int i = 0; i < num_blocks; ++i) free_[i] = num_blocks - 1 - i;
  }

  // A free page with refcount 1, or -1 when none is left.
  int allocate() {
    if (free_.empty()) return -1;
    const int id = free_.back();
    free_.pop_back();
    parked_[id] = 0;
    refs_[id] = 1;
    return id;
  }
  // Drops one reference; the page goes back to the free list at zero.
  void free(int id) {
    if (decref(id)) push_free(id);
  }
  void incref(int id) {
    check(id);
    if (parked_[id]) throw std::logic_error("incref: page is on the free list");
    ++refs_[id];
  }
  // Drops one reference without touching the free list; true when it reached zero.
  bool decref(int id) {
    check(id);
    if (refs_[id] <= 0) throw std::logic_error("decref: page has no reference");
    return --refs_[id] == 0;
  }
  // Puts a page with no reference back on the free list.
  void push_free(int id) {
    check(id);
    if (refs_[id] != 0 || parked_[id]) throw std::logic_error("push_free: page is live or already free");
    parked_[id] = 1;
    free_.push_back(id);
  }
  // Takes one particular page that has no reference and is not on the free list.
  void revive(int id) {
    check(id);
    if (refs_[id] != 0 || parked_[id]) throw std::logic_error("revive: page is live or on the free list");
    refs_[id] = 1;
  }

  int refcount(int id) const { return refs_[id]; }
  int num_free() const { return static_cast<int>(free_.size()); }
  int num_blocks() const { return static_cast<int>(refs_.size()); }

 private:
  void check(int id) const {
    if (id < 0 || id >= num_blocks()) throw std::logic_error("page id out of range");
  }
  std::vector<int32_t> free_;
  std::vector<int32_t> refs_;
  std::vector<uint8_t> parked_;  // 1 while the id sits on the free list
};

}  // namespace kvcm
