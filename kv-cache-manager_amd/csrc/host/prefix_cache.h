// Hash-chained cache over the full pages of one cache group.
//
// A page whose tokens are all computed may be registered under its chain hash.  When its last
// reference goes it is parked at the tail of an LRU list instead of the free list: it can still
// be found, and is only evicted (from the LRU head) when the free list is empty.  A hit checks
// the stored parent hash and the token ids, so a 64-bit collision cannot alias two prefixes.
// Behaviour follows src/core/prefix_cache.h:25-72 and src/core/prefix_cache.cpp:10-119 of the
// reference.
#pragma once
#include <cstdint>
#include <list>
#include <unordered_map>
#include <vector>

#include "block_allocator.h"
#include "xxhash64.h"

namespace kvcm {

struct PrefixCacheStats {
  int64_t queried_blocks = 0;     // full prompt pages that were looked up
  int64_t hit_blocks = 0;
  int64_t inserted_blocks = 0;
  int64_t evictions = 0;
  int64_t duplicate_inserts = 0;  // same content computed twice at the same time
};

class PrefixCache {
 public:
  PrefixCache(BlockAllocator& alloc, int block_size, bool enabled)
      : alloc_(alloc), bs_(block_size), on_(enabled) {
    const size_t n = static_cast<size_t>(alloc.num_blocks());
    meta_.resize(n);
    if (on_) tokens_.assign(n * bs_, 0);
  }

  bool enabled() const { return on_; }

  // A writable page: the free list first, else the least recently used parked page.
  int allocate() {
    if (alloc_.num_free() == 0 && !lru_.empty()) evict_oldest();
    return alloc_.allocate();
  }

  // Drops one reference.  At zero a registered page is parked on the LRU tail, any other page
  // returns to the free list.
  void release(int id) {
    if (!alloc_.decref(id)) return;
    Meta& m = meta_[id];
    if (m.registered) {
      m.lru_it = lru_.insert(lru_.end(), id);
      m.parked = true;
    } else {
      alloc_.push_free(id);
    }
  }

  // Length of the leading run of pages of `tokens` that are cached, at most `limit` pages,
  // without changing anything.  *parked_hits counts the hits that sit on the LRU list (taking
  // them shrinks the set of pages that allocate() could still hand out).
  int count_match(const int32_t* tokens, int limit, int* parked_hits) const {
    int hits = 0, parked = 0;
    if (on_) {
      uint64_t parent = 0;
      for (; hits < limit; ++hits) {
        const int32_t* t = tokens + static_cast<size_t>(hits) * bs_;
        const uint64_t h = chain_hash(parent, t, bs_);
        const int id = find(parent, h, t);
        if (id < 0) break;
        parked += meta_[id].parked ? 1 : 0;
        parent = h;
      }
    }
    if (parked_hits) *parked_hits = parked;
    return hits;
  }

  // Same walk, taking a reference on every hit (reviving parked pages).  Page ids and hashes are
  // appended to the outputs.  `eligible` is what the statistics count as looked up.
  int match_and_acquire(const int32_t* tokens, int limit, int eligible, std::vector<int32_t>& pages,
                        std::vector<uint64_t>& hashes) {
    if (!on_) return 0;
    stats_.queried_blocks += eligible;
    uint64_t parent = 0;
    int hits = 0;
    for (; hits < limit; ++hits) {
      const int32_t* t = tokens + static_cast<size_t>(hits) * bs_;
      const uint64_t h = chain_hash(parent, t, bs_);
      const int id = find(parent, h, t);
      if (id < 0) break;
      Meta& m = meta_[id];
      if (m.parked) {
        lru_.erase(m.lru_it);
        m.parked = false;
        alloc_.revive(id);
      } else {
        alloc_.incref(id);
      }
      pages.push_back(id);
      hashes.push_back(h);
      parent = h;
    }
    stats_.hit_blocks += hits;
    return hits;
  }

  // Registers a full, computed page.  false when the page already has a hash or the hash is
  // taken by another page (the page then stays private and is freed the ordinary way).
  bool insert(int page, uint64_t parent_hash, uint64_t hash, const int32_t* tokens) {
    if (!on_ || meta_[page].registered) return false;
    if (by_hash_.count(hash)) {
      ++stats_.duplicate_inserts;
      return false;
    }
    by_hash_.emplace(hash, page);
    Meta& m = meta_[page];
    m.hash = hash;
    m.parent = parent_hash;
    m.registered = true;
    std::memcpy(&tokens_[static_cast<size_t>(page) * bs_], tokens, sizeof(int32_t) * bs_);
    ++stats_.inserted_blocks;
    return true;
  }

  int num_available() const { return alloc_.num_free() + static_cast<int>(lru_.size()); }
  int num_cached_free() const { return static_cast<int>(lru_.size()); }
  int num_hashed() const { return static_cast<int>(by_hash_.size()); }
  bool is_hashed(int id) const { return meta_[id].registered; }
  const PrefixCacheStats& stats() const { return stats_; }
  std::vector<int> lru_order() const { return {lru_.begin(), lru_.end()}; }  // oldest first

 private:
  struct Meta {
    uint64_t hash = 0, parent = 0;
    bool registered = false, parked = false;
    std::list<int32_t>::iterator lru_it;
  };

  int find(uint64_t parent, uint64_t h, const int32_t* tokens) const {
    auto it = by_hash_.find(h);
    if (it == by_hash_.end()) return -1;
    const int id = it->second;
    if (meta_[id].parent != parent) return -1;
    if (std::memcmp(&tokens_[static_cast<size_t>(id) * bs_], tokens, sizeof(int32_t) * bs_) != 0) return -1;
    return id;
  }

  void evict_oldest() {
    const int id = lru_.front();
    lru_.pop_front();
    Meta& m = meta_[id];
    by_hash_.erase(m.hash);
    m.registered = m.parked = false;
    ++stats_.evictions;
    alloc_.push_free(id);
  }

  BlockAllocator& alloc_;
  int bs_;
  bool on_;
  std::unordered_map<uint64_t, int32_t> by_hash_;
  std::vector<Meta> meta_;
  std::vector<int32_t> tokens_;  // [num_blocks][block_size] for verification
  std::list<int32_t> lru_;
  PrefixCacheStats stats_;
};

}  // namespace kvcm
