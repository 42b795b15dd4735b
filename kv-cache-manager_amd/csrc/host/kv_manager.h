// Cache managers: who owns which page.
//
// The layers of a model are partitioned into cache groups.  A group is either paged keys and
// values (every key kept, or only a window of the most recent ones) or a fixed-size state per
// request.  Every paged group has a pool of pages of its own and every request one page table per
// group.  Two allocation policies sit behind one interface, as in the reference
// (src/core/kv_manager.h:32-74): PagedManager takes pages on demand
// (src/core/paged_manager.cpp:9-66), ContiguousManager reserves max_seq_len worth of consecutive
// pages at admission (src/core/contiguous_manager.cpp:7-66).  Groups, windows and state slots are
// additions; with one full group the behaviour is the reference's.
#pragma once
#include <algorithm>
#include <cstdint>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "block_allocator.h"
#include "prefix_cache.h"
#include "sequence.h"

namespace kvcm {

enum class GroupKind : int { FullKV = 0, WindowKV = 1, State = 2 };

struct GroupSpec {
  GroupKind kind = GroupKind::FullKV;
  int window = 0;      // WindowKV: a query at position p sees keys t with p - t < window
  int num_blocks = 0;  // pages in this group's pool (ignored for State)
};

struct KVStats {
  int num_blocks = 0, block_size = 0;
  int blocks_in_use = 0;              // referenced (a reserved page counts)
  int blocks_cached_free = 0;         // unreferenced but kept for prefix hits
  int64_t allocated_slots = 0;        // blocks_in_use * block_size
  int64_t used_slots = 0;             // physical slots that hold a token
  int64_t tail_waste_slots = 0;       // empty slots in partly filled pages
  int64_t reserved_unused_slots = 0;  // slots of reserved pages that hold nothing
  int64_t block_table_entries = 0;
  int num_seqs = 0;
  PrefixCacheStats prefix;
  double fragmentation() const {
    return allocated_slots ? double(allocated_slots - used_slots) / double(allocated_slots) : 0.0;
  }
};

// Fixed-size per-request state: a pool of slot ids, one taken at admission, returned at release.
class StateSlotPool {
 public:
  explicit StateSlotPool(int n) : taken_(n, 0) {
    for (int i = n - 1; i >= 0; --i) free_.push_back(i);
  }
  int take() {
    if (free_.empty()) return -1;
    const int s = free_.back();
    free_.pop_back();
    taken_[s] = 1;
    return s;
  }
  void give_back(int s) {
    if (s < 0 || s >= static_cast<int>(taken_.size()) || !taken_[s])
      throw std::logic_error("state slot returned twice or never taken");
    taken_[s] = 0;
    free_.push_back(s);
  }
  int num_free() const { return static_cast<int>(free_.size()); }
  int capacity() const { return static_cast<int>(taken_.size()); }

 private:
  std::vector<int32_t> free_;
  std::vector<uint8_t> taken_;
};

class KVManager {
 public:
  virtual ~KVManager() = default;
  virtual std::string name() const = 0;
  int block_size() const { return bs_; }
  int max_seq_len() const { return max_seq_len_; }
  int num_groups() const { return static_cast<int>(groups_.size()); }
  const GroupSpec& group(int g) const { return groups_[g]; }
  int num_blocks(int g = 0) const { return groups_[g].num_blocks; }
  const StateSlotPool& slots() const { return slots_; }

  // Can every token now in seq.tokens be given room?
  virtual bool can_admit(const Sequence& seq) const = 0;
  // Builds the tables for all of seq.tokens (prefix hits first), takes a state slot and sets
  // num_computed to the number of tokens whose keys are already cached.
  virtual void admit(Sequence& seq) = 0;
  // Room for every token in seq.tokens; false = out of pages (nothing is rolled back: pages
  // taken so far stay in the table, as in the reference).
  virtual bool append_slot(Sequence& seq) = 0;
  // After a step: newly full pages become findable, pages a window has passed are given back.
  virtual void commit(Sequence& seq) = 0;
  virtual void release(Sequence& seq) = 0;

  virtual int blocks_in_use(int g = 0) const = 0;
  virtual int blocks_cached_free(int /*g*/ = 0) const { return 0; }
  virtual PrefixCacheStats prefix_stats(int /*g*/ = 0) const { return {}; }

  // Occupancy of one group over the live sequences; the fill of a shared page is the largest
  // fill among its holders (src/core/kv_manager.cpp:11-39).
  KVStats stats(const std::vector<const Sequence*>& live, int g = 0) const {
    KVStats s;
    s.num_blocks = groups_[g].num_blocks;
    s.block_size = bs_;
    s.blocks_in_use = blocks_in_use(g);
    s.blocks_cached_free = blocks_cached_free(g);
    s.allocated_slots = int64_t(s.blocks_in_use) * bs_;
    s.num_seqs = static_cast<int>(live.size());
    s.prefix = prefix_stats(g);
    std::vector<int> fill(static_cast<size_t>(s.num_blocks), -1);
    for (const Sequence* q : live) {
      if (g >= static_cast<int>(q->tables.size())) continue;
      const auto& tab = q->tables[g];
      s.block_table_entries += static_cast<int64_t>(tab.size());
      for (size_t b = 0; b < tab.size(); ++b) {
        if (tab[b] < 0) continue;
        const int f = std::clamp(q->num_computed - static_cast<int>(b) * bs_, 0, bs_);
        fill[tab[b]] = std::max(fill[tab[b]], f);
      }
    }
    for (int f : fill) {
      if (f < 0) continue;
      s.used_slots += f;
      if (f == 0) s.reserved_unused_slots += bs_;
      else s.tail_waste_slots += bs_ - f;
    }
    return s;
  }

 protected:
  KVManager(std::vector<GroupSpec> groups, int block_size, int max_seq_len, int max_slots)
      : groups_(std::move(groups)), bs_(block_size), max_seq_len_(max_seq_len), slots_(max_slots) {
    if (block_size <= 0) throw std::invalid_argument("block_size must be positive");
    if (groups_.empty()) throw std::invalid_argument("a cache manager needs at least one group");
    for (const auto& g : groups_)
      if (g.kind == GroupKind::WindowKV && g.window <= 0)
        throw std::invalid_argument("a windowed group needs window > 0");
  }
  int blocks_for(int ntok) const { return (ntok + bs_ - 1) / bs_; }
  bool paged(int g) const { return groups_[g].kind != GroupKind::State; }
  void prepare(Sequence& seq) const {
    seq.tables.assign(groups_.size(), {});
    seq.released_below.assign(groups_.size(), 0);
  }

  std::vector<GroupSpec> groups_;
  int bs_, max_seq_len_;
  StateSlotPool slots_;
};

// ------------------------------------------------------------------------------------- paged
class PagedManager : public KVManager {
 public:
  PagedManager(std::vector<GroupSpec> groups, int block_size, int max_seq_len, bool prefix_caching,
               int watermark_blocks, int max_slots)
      : KVManager(std::move(groups), block_size, max_seq_len, max_slots), watermark_(watermark_blocks) {
    for (const auto& g : groups_) {
      if (prefix_caching && g.kind != GroupKind::FullKV)
        throw std::invalid_argument(
            "prefix caching needs every cache group to keep all keys (no window, no state)");
      pools_.emplace_back(new Pool(g.kind == GroupKind::State ? 0 : g.num_blocks, block_size,
                                   prefix_caching));
    }
    prefix_ = prefix_caching;
  }
  std::string name() const override { return prefix_ ? "paged+prefix" : "paged"; }

  bool can_admit(const Sequence& seq) const override {
    const int n = seq.size();
    if (n > max_seq_len_ || slots_.num_free() == 0) return false;
    const int hits = common_hits(seq, nullptr);
    for (int g = 0; g < num_groups(); ++g) {
      if (!paged(g)) continue;
      int parked = 0;
      if (prefix_) pools_[g]->cache.count_match(seq.tokens.data(), hits, &parked);
      const int need = blocks_for(n) - hits;
      const int available = pools_[g]->cache.num_available() - parked;
      if (need > available - watermark_) return false;
    }
    return true;
  }

  void admit(Sequence& seq) override {
    for (const auto& t : seq.tables)
      if (!t.empty()) throw std::logic_error("admit: the sequence already holds pages");
    if (seq.state_slot >= 0) throw std::logic_error("admit: the sequence already holds a state slot");
    prepare(seq);
    seq.page_hashes.clear();
    int hits = 0;
    if (prefix_) {
      hits = common_hits(seq, nullptr);
      for (int g = 0; g < num_groups(); ++g) {
        std::vector<uint64_t> hashes;
        pools_[g]->cache.match_and_acquire(seq.tokens.data(), hits, matchable(seq), seq.tables[g], hashes);
        if (g == 0) seq.page_hashes = hashes;
      }
    }
    seq.cached_tokens = hits * bs_;
    seq.num_computed = seq.cached_tokens;
    seq.prefill_tokens_saved += seq.cached_tokens;
    seq.state_slot = slots_.take();
    if (seq.state_slot < 0) throw std::runtime_error("admit: no state slot left (call can_admit first)");
    if (!append_slot(seq)) throw std::runtime_error("admit: out of pages (call can_admit first)");
  }

  bool append_slot(Sequence& seq) override {
    if (seq.tables.size() != groups_.size()) throw std::logic_error("append_slot: sequence was not admitted");
    const int need = blocks_for(seq.size());
    for (int g = 0; g < num_groups(); ++g) {
      if (!paged(g)) continue;
      auto& tab = seq.tables[g];
      while (static_cast<int>(tab.size()) < need) {
        const int id = pools_[g]->cache.allocate();
        if (id < 0) return false;
        tab.push_back(id);
      }
    }
    return true;
  }

  void commit(Sequence& seq) override {
    if (prefix_) {
      const int full = seq.num_computed / bs_;
      for (int b = static_cast<int>(seq.page_hashes.size()); b < full; ++b) {
        const uint64_t parent = b ? seq.page_hashes[b - 1] : 0;
        const int32_t* t = seq.tokens.data() + static_cast<size_t>(b) * bs_;
        const uint64_t h = chain_hash(parent, t, bs_);
        for (int g = 0; g < num_groups(); ++g) pools_[g]->cache.insert(seq.tables[g][b], parent, h, t);
        seq.page_hashes.push_back(h);
      }
    }
    // The next query sits at position >= num_computed and sees keys t > position - window.
    for (int g = 0; g < num_groups(); ++g) {
      if (groups_[g].kind != GroupKind::WindowKV) continue;
      const int first_needed_token = std::max(0, seq.num_computed - groups_[g].window + 1);
      const int first_needed_page = std::min<int>(first_needed_token / bs_, static_cast<int>(seq.tables[g].size()));
      for (int b = seq.released_below[g]; b < first_needed_page; ++b) {
        pools_[g]->cache.release(seq.tables[g][b]);
        seq.tables[g][b] = -1;
      }
      seq.released_below[g] = std::max(seq.released_below[g], first_needed_page);
    }
  }

  void release(Sequence& seq) override {
    // Tail first, so that the end of a cached prefix is evicted before its head.
    for (int g = 0; g < static_cast<int>(seq.tables.size()); ++g) {
      auto& tab = seq.tables[g];
      for (auto it = tab.rbegin(); it != tab.rend(); ++it)
        if (*it >= 0) pools_[g]->cache.release(*it);
      tab.clear();
    }
    std::fill(seq.released_below.begin(), seq.released_below.end(), 0);
    if (seq.state_slot >= 0) {
      slots_.give_back(seq.state_slot);
      seq.state_slot = -1;
    }
    seq.page_hashes.clear();
    seq.num_computed = 0;
  }

  int blocks_in_use(int g = 0) const override { return pools_[g]->alloc.num_blocks() - pools_[g]->cache.num_available(); }
  int blocks_cached_free(int g = 0) const override { return pools_[g]->cache.num_cached_free(); }
  PrefixCacheStats prefix_stats(int g = 0) const override { return pools_[g]->cache.stats(); }
  const BlockAllocator& allocator(int g = 0) const { return pools_[g]->alloc; }
  const PrefixCache& cache(int g = 0) const { return pools_[g]->cache; }

 private:
  struct Pool {
    Pool(int n, int bs, bool prefix) : alloc(n), cache(alloc, bs, prefix) {}
    BlockAllocator alloc;
    PrefixCache cache;
  };
  // Leading full pages that may be shared: the page of the last token never is, because that
  // token is run again for its logits (src/core/paged_manager.h:33-35).
  int matchable(const Sequence& s) const { return (s.size() - 1) / bs_; }
  // Hits that every group can serve.
  int common_hits(const Sequence& seq, int* /*unused*/) const {
    if (!prefix_) return 0;
    int hits = matchable(seq);
    for (int g = 0; g < num_groups(); ++g)
      hits = std::min(hits, pools_[g]->cache.count_match(seq.tokens.data(), hits, nullptr));
    return hits;
  }

  std::vector<std::unique_ptr<Pool>> pools_;
  bool prefix_ = false;
  int watermark_;
};

// -------------------------------------------------------------------------------- contiguous
class ContiguousManager : public KVManager {
 public:
  ContiguousManager(std::vector<GroupSpec> groups, int block_size, int max_seq_len, int max_slots)
      : KVManager(std::move(groups), block_size, max_seq_len, max_slots),
        reserve_(blocks_for(max_seq_len)) {
    for (const auto& g : groups_) {
      Extents e;
      e.free_blocks = g.kind == GroupKind::State ? 0 : g.num_blocks;
      if (e.free_blocks > 0) e.spans[0] = e.free_blocks;
      ext_.push_back(std::move(e));
    }
  }
  std::string name() const override { return "contiguous"; }

  bool can_admit(const Sequence& seq) const override {
    if (seq.size() > max_seq_len_ || slots_.num_free() == 0) return false;
    for (int g = 0; g < num_groups(); ++g)
      if (paged(g) && first_fit(g) < 0) return false;
    return true;
  }

  void admit(Sequence& seq) override {
    for (const auto& t : seq.tables)
      if (!t.empty()) throw std::logic_error("admit: the sequence already holds pages");
    if (!can_admit(seq)) throw std::runtime_error("admit: no run of consecutive pages (call can_admit first)");
    prepare(seq);
    for (int g = 0; g < num_groups(); ++g) {
      if (!paged(g)) continue;
      const int start = first_fit(g);
      auto it = ext_[g].spans.find(start);
      const int len = it->second;
      ext_[g].spans.erase(it);
      if (len > reserve_) ext_[g].spans[start + reserve_] = len - reserve_;
      ext_[g].free_blocks -= reserve_;
      seq.tables[g].resize(reserve_);
      for (int i = 0; i < reserve_; ++i) seq.tables[g][i] = start + i;
    }
    seq.state_slot = slots_.take();
    seq.cached_tokens = 0;
    seq.num_computed = 0;
  }

  bool append_slot(Sequence& seq) override { return seq.size() <= reserve_ * bs_; }
  void commit(Sequence&) override {}

  void release(Sequence& seq) override {
    for (int g = 0; g < static_cast<int>(seq.tables.size()); ++g) {
      auto& tab = seq.tables[g];
      if (tab.empty()) continue;
      int start = tab.front();
      int len = static_cast<int>(tab.size());
      auto& spans = ext_[g].spans;
      ext_[g].free_blocks += len;
      auto right = spans.lower_bound(start);
      if (right != spans.end() && right->first == start + len) {
        len += right->second;
        right = spans.erase(right);
      }
      if (right != spans.begin()) {
        auto left = std::prev(right);
        if (left->first + left->second == start) {
          start = left->first;
          len += left->second;
          spans.erase(left);
        }
      }
      spans[start] = len;
      tab.clear();
    }
    if (seq.state_slot >= 0) {
      slots_.give_back(seq.state_slot);
      seq.state_slot = -1;
    }
    seq.num_computed = 0;
  }

  int blocks_in_use(int g = 0) const override { return groups_[g].num_blocks - ext_[g].free_blocks; }
  int num_free_extents(int g = 0) const { return static_cast<int>(ext_[g].spans.size()); }

 private:
  struct Extents {
    std::map<int, int> spans;  // start -> length of a free run
    int free_blocks = 0;
  };
  int first_fit(int g) const {
    for (const auto& [start, len] : ext_[g].spans)
      if (len >= reserve_) return start;
    return -1;
  }
  int reserve_;
  std::vector<Extents> ext_;
};

struct KVManagerConfig {
  std::string policy = "paged";  // "paged" | "contiguous"
  std::vector<GroupSpec> groups; // empty => one full group of num_blocks pages
  int num_blocks = 1024;
  int block_size = 16;
  int max_seq_len = 2048;
  bool prefix_caching = false;
  int watermark_blocks = -1;     // paged: pages kept spare at admission (-1 => watermark_frac)
  double watermark_frac = 0.01;
  int max_slots = 256;           // state slots = most requests admitted at once
};

inline std::unique_ptr<KVManager> make_kv_manager(const KVManagerConfig& c) {
  std::vector<GroupSpec> groups = c.groups;
  if (groups.empty()) groups.push_back({GroupKind::FullKV, 0, c.num_blocks});
  int pool = 0;
  for (const auto& g : groups)
    if (g.kind != GroupKind::State) pool = pool ? std::min(pool, g.num_blocks) : g.num_blocks;
  if (c.policy == "paged") {
    const int wm = c.watermark_blocks >= 0 ? c.watermark_blocks : static_cast<int>(c.watermark_frac * pool);
    return std::make_unique<PagedManager>(groups, c.block_size, c.max_seq_len, c.prefix_caching, wm, c.max_slots);
  }
  if (c.policy == "contiguous")
    return std::make_unique<ContiguousManager>(groups, c.block_size, c.max_seq_len, c.max_slots);
  throw std::invalid_argument("unknown KV policy: " + c.policy);
}

}  // namespace kvcm
