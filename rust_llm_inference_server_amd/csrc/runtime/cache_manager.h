// Page bookkeeping of the cache: which physical pages hold which request's positions, and
// which seat (slot of fixed-size state) a request sits in.  Pure host logic, no GPU.
//
// Layers are collected in *groups* with pools of their own: a group keeps every position of a
// request or only a window of the latest ones.  A request holds one *lease*: per group the
// run of pages that back its positions (pages that a window has passed are given back while
// the request lives), the number of positions reserved and of positions computed, and its
// seat.  Three rules carry everything else:
//
//  * A reservation is quoted before it is made.  `quote` says what making positions
//    [0, total) of a request addressable *and writable from its computed length on* would take
//    from every pool, and whether it takes a seat; `reserve` commits a quote only if every pool
//    can pay it, so a reservation that fails changes nothing.  The scheduler admits with the
//    same quote plus its watermark.
//  * Pages are shared by reference count.  A fork shares the pages of the positions that are
//    computed and nothing beyond; whoever then reserves a range that touches a shared page
//    gets a copy of it first (the copy is returned for the device to perform) and lets go of
//    the original.
//  * Pools hand out the page that was returned last (page 0 first in a fresh pool), so pages
//    are used again at once and stale contents are what the next request finds.
//
// What this must do is the reference's BlockManager contract (crates/kvcache/src/lib.rs:
// 177-438: all-or-nothing reserve, copy-on-write, fork, free, invariants); groups, windows,
// seats, the quote and the computed length are this engine's.
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

// One group's pages: a reference count per page and the free pages as a stack threaded
// through `below_`.
class PagePool {
 public:
  explicit PagePool(int num_pages);
  int size() const { return (int)refs_.size(); }
  int free_count() const { return free_count_; }
  int refs(int p) const { return refs_[p]; }
  int take();                  // the page on top of the stack, now held once; -1 when empty
  void share(int p);           // one more holder
  void drop(int p);            // one holder fewer; the page goes back on the stack at zero
  // Pages on the free stack from the top down (for the audit).
  std::vector<int> free_pages() const;

 private:
  std::vector<int> refs_;
  std::vector<int> below_;     // for a free page: the free page under it, -1 at the bottom
  int top_ = -1;
  int free_count_ = 0;
};

struct GroupSpec {
  int window;      // 0: every position is kept; w > 0: only the last w positions
  int num_pages;
};

// The pages of one group that back a request: logical page i is gone (returned, a window has
// passed it) for i < gone, else live[i - gone].
struct PageRun {
  int gone = 0;
  std::vector<int> live;
  int count() const { return gone + (int)live.size(); }
  int at(int i) const { return i < gone ? -1 : live[i - gone]; }
};

struct Lease {
  std::vector<PageRun> runs;   // one per group
  int reserved = 0;            // positions with a place in the pages
  int computed = 0;            // positions whose contents are written
  int seat = -1;               // state slot, -1 when the model keeps no state
};

// What a reservation would take.
struct Quote {
  std::vector<int> pages;      // per group: pages to grow by plus shared pages to copy
  bool seat = false;           // a seat too (the request is new and seats exist)
};

enum ReserveResult { kReserved = 0, kOutOfPages = 1, kOutOfSlots = 2 };

class CacheManager {
 public:
  CacheManager(int page_size, std::vector<GroupSpec> groups, int num_state_slots);

  int page_size() const { return page_size_; }
  int num_groups() const { return (int)groups_.size(); }
  int num_pages(int g) const { return pools_[g].size(); }
  int num_free(int g) const { return pools_[g].free_count(); }
  int refcount(int g, int p) const { return pools_[g].refs(p); }
  int window(int g) const { return groups_[g].window; }
  int num_state_slots() const { return num_seats_; }
  int num_free_slots() const { return (int)free_seats_.size(); }
  int pages_for(int tokens) const { return (tokens + page_size_ - 1) / page_size_; }

  bool contains(SeqId s) const { return leases_.count(s) != 0; }
  const Lease* lease(SeqId s) const;

  Quote quote(SeqId s, int total_tokens) const;
  // Whether every pool can pay the quote and still keep `spare` pages free, and a seat is
  // there if the quote takes one.  `short_of_seats` (may be null) says which of the two failed.
  bool affordable(const Quote& q, int spare, bool* short_of_seats = nullptr) const;
  // Makes positions [0, total_tokens) of s addressable in every group and the pages from its
  // computed length on its own; creates the request on first use (and seats it).  All or
  // nothing.  Copies to perform on the device are appended to `copies`.
  ReserveResult reserve(SeqId s, int total_tokens, std::vector<PageCopy>* copies);
  // Positions [0, computed) are written; windowed groups give back pages no later query sees.
  void advance(SeqId s, int computed);
  // child shares parent's computed positions.  Returns the seats (parent's, child's) whose
  // state the device must copy, both -1 when there are no seats.
  std::pair<int, int> fork(SeqId parent, SeqId child);
  void free_seq(SeqId s);

  // Empty when the books balance, else the first thing that does not.
  std::string audit() const;

 private:
  int first_visible_page(int computed, int g) const;

  int page_size_;
  std::vector<GroupSpec> groups_;
  std::vector<PagePool> pools_;
  int num_seats_;
  std::vector<int> free_seats_;   // a stack: the seat returned last is taken next
  std::unordered_map<SeqId, Lease> leases_;
};

}  // namespace rlis
