// Page bookkeeping of the cache: which physical pages hold which request's positions.
// Pure host logic, no GPU (as crates/kvcache/src/lib.rs:1-5 of the reference).
//
// The reference has one pool whose block ids address every layer (lib.rs:3-5).  Here layers
// are collected in *groups* with pages of their own: a group keeps either every position of a
// request or only a window of the latest ones.  Every group has its own pool, and every
// request one block table per group.  A page of a windowed group is given back as soon as all
// its positions have left the window; all pages go back when the request is freed.  Beside
// the pages, a request holds one *state slot* (a fixed-size area for mixers whose memory of
// the past does not grow) from its first reservation until it is freed.
//
// Kept from the reference: reference counts with a LIFO free list that hands out page 0 first
// (lib.rs:57-82, 123-165), all-or-nothing reservation that grows whole pages (lib.rs:282-336),
// copy-on-write of a shared, partly filled last page (lib.rs:293-297, 319-328), fork
// (lib.rs:338-354) and the invariant checker (lib.rs:372-437).  Left out: the hash registry and
// the evictable set of its prefix cache.
#pragma once
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

namespace rlis {

using SeqId = int64_t;

struct PageCopy {
  int group;
  int src;
  int dst;
};

class PageAllocator {
 public:
  explicit PageAllocator(int num_pages);
  int num_pages() const { return (int)refcounts_.size(); }
  int num_free() const { return (int)free_.size(); }
  int refcount(int p) const { return refcounts_[p]; }
  int allocate();            // -1 when none is free
  void incref(int p);
  void decref(int p);        // throws on a page that is already free
  const std::vector<int>& free_list() const { return free_; }

 private:
  std::vector<int> refcounts_;
  std::vector<int> free_;    // LIFO
};

struct GroupSpec {
  int window;      // 0: every position is kept; w > 0: only the last w positions
  int num_pages;
};

struct SeqEntry {
  // Per group: physical page of logical page i, or -1 once the window has passed it.
  std::vector<std::vector<int>> pages;
  int num_tokens = 0;     // positions with a slot reserved
  int num_computed = 0;   // positions whose keys and values are written
  int state_slot = -1;
};

enum ReserveResult { kReserved = 0, kOutOfPages = 1, kOutOfSlots = 2 };

class CacheManager {
 public:
  CacheManager(int page_size, std::vector<GroupSpec> groups, int num_state_slots);

  int page_size() const { return page_size_; }
  int num_groups() const { return (int)groups_.size(); }
  int num_pages(int g) const { return alloc_[g].num_pages(); }
  int num_free(int g) const { return alloc_[g].num_free(); }
  int refcount(int g, int p) const { return alloc_[g].refcount(p); }
  int window(int g) const { return groups_[g].window; }
  int num_state_slots() const { return num_state_slots_; }
  int num_free_slots() const { return (int)free_slots_.size(); }
  int pages_for(int tokens) const { return (tokens + page_size_ - 1) / page_size_; }

  bool contains(SeqId s) const { return seqs_.count(s) != 0; }
  const SeqEntry* entry(SeqId s) const;

  // Pages `reserve(s, total)` would take from group g, a copy-on-write included.
  int pages_needed(SeqId s, int total_tokens, int g) const;
  // Makes positions up to total_tokens addressable in every group; creates the request on
  // first use (and takes a state slot).  All or nothing: on failure nothing changes.
  ReserveResult reserve(SeqId s, int total_tokens, std::vector<PageCopy>* copies);
  // Positions [0, computed) are written; windowed groups give back pages no later query
  // can see.
  void advance(SeqId s, int computed);
  void fork(SeqId parent, SeqId child);
  void free_seq(SeqId s);

  // Empty when every invariant holds, else a description of the first violation.
  std::string check_invariants() const;

 private:
  bool needs_cow(const SeqEntry& e, int g) const;
  int first_live_page(int computed, int g) const;

  int page_size_;
  std::vector<GroupSpec> groups_;
  std::vector<PageAllocator> alloc_;
  int num_state_slots_;
  std::vector<int> free_slots_;   // LIFO
  std::unordered_map<SeqId, SeqEntry> seqs_;
};

}  // namespace rlis
