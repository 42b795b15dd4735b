// Hash-chained cache over the full pages of one cache group.
//
// A page whose tokens are all computed may be registered under its chain hash.  When its last
// reference goes it is parked at the young end of a recency list instead of the free list: it can
// still be found, and is only evicted (oldest first) when the free list is empty.  A hit checks
// the stored parent hash and the token ids, so a 64-bit collision cannot alias two prefixes.
// Behaviour follows src/core/prefix_cache.h:25-72 and src/core/prefix_cache.cpp:10-119 of the
// reference.  The recency list is threaded through two arrays indexed by page id (no node is
// allocated when a page is parked or revived); entry `num_pages` is the list's head and tail.
#pragma once
#include <cstdint>
#include <cstring>
#include <unordered_map>
#include <vector>

#include "block_allocator.h"
#include "xxhash64.h"

namespace kvcm {

struct PrefixCacheStats {
  int64_t queried_blocks = 0, hit_blocks = 0;   // full prompt pages that were looked up; found
  int64_t inserted_blocks = 0, evictions = 0;
  int64_t duplicate_inserts = 0;                // same content computed twice at the same time
};

class PrefixCache {
 public:
  PrefixCache(BlockAllocator& pages, int page_tokens, bool enabled)
      : pages_(pages), width_(page_tokens), enabled_(enabled), ring_(pages.num_blocks()) {
    const size_t n = static_cast<size_t>(pages.num_blocks());
    entry_.resize(n);
    older_.assign(n + 1, ring_);
    younger_.assign(n + 1, ring_);
    if (enabled_) content_.assign(n * width_, 0);
  }

  bool enabled() const { return enabled_; }

  // A writable page: the free list first, else the parked page that was used longest ago.
  int allocate() {
    if (pages_.num_free() == 0 && parked_ > 0) evict(younger_[ring_]);
    return pages_.allocate();
  }

  // Drops one reference.  At zero a registered page is parked (youngest), any other page
  // returns to the free list.
  void release(int page) {
    if (!pages_.decref(page)) return;
    if (entry_[page].registered) park(page);
    else pages_.push_free(page);
  }

  // Length of the leading run of pages of `tokens` that are cached, at most `limit` pages,
  // without changing anything.  *parked_hits counts the hits that are parked (taking them shrinks
  // the set of pages that allocate() could still hand out).
  int count_match(const int32_t* tokens, int limit, int* parked_hits) const {
    int parked = 0;
    const int found = walk(tokens, limit, [&](int page, uint64_t) { parked += entry_[page].parked; });
    if (parked_hits) *parked_hits = parked;
    return found;
  }

  // Same walk, taking a reference on every hit (reviving parked pages).  Page ids and hashes are
  // appended to the outputs.  `eligible` is what the statistics count as looked up.
  int match_and_acquire(const int32_t* tokens, int limit, int eligible, std::vector<int32_t>& table,
                        std::vector<uint64_t>& chain) {
    if (!enabled_) return 0;
    const int found = walk(tokens, limit, [&](int page, uint64_t hash) {
      if (entry_[page].parked) {
        unlink(page);
        pages_.revive(page);
      } else {
        pages_.incref(page);
      }
      table.push_back(page);
      chain.push_back(hash);
    });
    stats_.queried_blocks += eligible;
    stats_.hit_blocks += found;
    return found;
  }

  // Registers a full, computed page.  false when the page already has a hash or the hash is
  // taken by another page (the page then stays private and is freed the ordinary way).
  bool insert(int page, uint64_t parent_hash, uint64_t hash, const int32_t* tokens) {
    if (!enabled_ || entry_[page].registered) return false;
    if (!index_.emplace(hash, page).second) {
      stats_.duplicate_inserts += 1;
      return false;
    }
    Entry& e = entry_[page];
    e.hash = hash;
    e.parent = parent_hash;
    e.registered = true;
    std::memcpy(content_of(page), tokens, sizeof(int32_t) * width_);
    stats_.inserted_blocks += 1;
    return true;
  }

  int num_available() const { return pages_.num_free() + parked_; }
  int num_cached_free() const { return parked_; }
  int num_hashed() const { return static_cast<int>(index_.size()); }
  bool is_hashed(int page) const { return entry_[page].registered; }
  const PrefixCacheStats& stats() const { return stats_; }
  // Parked pages, the one that would be evicted first in front.
  std::vector<int> lru_order() const {
    std::vector<int> order;
    order.reserve(parked_);
    for (int p = younger_[ring_]; p != ring_; p = younger_[p]) order.push_back(p);
    return order;
  }

 private:
  struct Entry {
    uint64_t hash = 0, parent = 0;
    bool registered = false, parked = false;
  };

  int32_t* content_of(int page) { return &content_[static_cast<size_t>(page) * width_]; }
  const int32_t* content_of(int page) const { return &content_[static_cast<size_t>(page) * width_]; }

  // Follows the chain of hashes over the leading pages of `tokens` while each is registered with
  // the right parent and the same token ids; calls hit(page, hash) for each.
  template <class Hit>
  int walk(const int32_t* tokens, int limit, Hit&& hit) const {
    if (!enabled_) return 0;
    uint64_t parent = 0;
    int n = 0;
    while (n < limit) {
      const int32_t* ids = tokens + static_cast<size_t>(n) * width_;
      const uint64_t hash = chain_hash(parent, ids, width_);
      const auto at = index_.find(hash);
      if (at == index_.end()) break;
      const int page = at->second;
      if (entry_[page].parent != parent || std::memcmp(content_of(page), ids, sizeof(int32_t) * width_) != 0) break;
      hit(page, hash);
      parent = hash;
      ++n;
    }
    return n;
  }

  void park(int page) {   // youngest: just before the ring entry
    const int last = older_[ring_];
    younger_[last] = page;
    older_[page] = last;
    younger_[page] = ring_;
    older_[ring_] = page;
    entry_[page].parked = true;
    ++parked_;
  }
  void unlink(int page) {
    younger_[older_[page]] = younger_[page];
    older_[younger_[page]] = older_[page];
    entry_[page].parked = false;
    --parked_;
  }
  void evict(int page) {
    unlink(page);
    index_.erase(entry_[page].hash);
    entry_[page].registered = false;
    stats_.evictions += 1;
    pages_.push_free(page);
  }

  BlockAllocator& pages_;
  int width_;       // tokens per page
  bool enabled_;
  int ring_;        // index of the list's own entry in older_ / younger_
  int parked_ = 0;
  std::unordered_map<uint64_t, int32_t> index_;   // chain hash -> page
  std::vector<Entry> entry_;
  std::vector<int32_t> older_, younger_;
  std::vector<int32_t> content_;   // [pages][width_]: the token ids of registered pages, compared at a hit
  PrefixCacheStats stats_;
};

}  // namespace kvcm
