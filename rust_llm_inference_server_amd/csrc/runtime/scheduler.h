// What each step computes: continuous batching with chunked prefill under a token budget, and
// preemption by recompute when pages run out.  The decisions are the reference's
// (crates/engine/src/scheduler.rs:1-8, 193-306); the book-keeping is this engine's.
//
// Every request sits in one *roster*, ordered by arrival, with a standing: queued (never ran),
// parked (preempted: it holds nothing and will recompute), or running (it holds a lease).  A
// request is `tokens` (prompt plus generated) and `computed` (positions in the cache); a step
// computes the next portion of the gap between the two, which is prefill, chunked prefill,
// decode or recompute depending only on how large the gap is.
//
// A step is planned in two passes over the roster:
//  1. Running requests, oldest first, each take min(gap, budget left) tokens.  When the cache
//     cannot give a request its pages, the *youngest* running request is parked (it returns its
//     lease and starts over later); that may be the request that asked, which then waits.
//  2. Admission, unless the first pass parked someone (static policy: only when nothing runs):
//     the oldest parked request, or else the oldest queued one, is admitted while a seat among
//     max_num_seqs is free, budget is left (the static policy ignores the budget) and the cache
//     can pay for the whole known length with `watermark` pages to spare in every group.  The
//     head of the line is never skipped; an admitted request reserves its whole known length
//     at once, so that later admissions cannot overcommit the pools.
#pragma once
#include <map>
#include <unordered_map>
#include <vector>

#include "cache_manager.h"

namespace rlis {

enum Policy { kContinuous = 0, kStatic = 1 };

struct SchedulerConfig {
  int max_num_seqs;
  int max_batched_tokens;
  int watermark_pages;
  Policy policy;
};

struct ScheduledSeq {
  SeqId id;
  int start;
  int end;
};

struct Schedule {
  std::vector<ScheduledSeq> seqs;
  std::vector<PageCopy> copies;
  std::vector<SeqId> preempted;
};

class Scheduler {
 public:
  Scheduler(SchedulerConfig cfg, CacheManager* cache);

  // Longest request (prompt plus output) that can ever be admitted: what the smallest pool
  // holds beyond the watermark.
  int max_seq_tokens() const;
  void add(SeqId id, int prompt_len);
  Schedule schedule();
  void advance(SeqId id, int end);
  void append_token(SeqId id);
  bool is_caught_up(SeqId id) const;
  void remove(SeqId id);
  bool has_work() const { return !roster_.empty(); }
  int num_running() const { return standing_count_[kRunning]; }
  int num_waiting() const { return standing_count_[kQueued] + standing_count_[kParked]; }
  long long num_preemptions() const { return num_preemptions_; }
  int num_tokens(SeqId id) const;
  int num_computed(SeqId id) const;
  std::string check() const;

 private:
  enum Standing { kQueued = 0, kParked = 1, kRunning = 2 };
  struct Member {
    SeqId id;
    int tokens;
    int computed;
    Standing standing;
  };
  using Roster = std::map<long long, Member>;   // by arrival

  Member* find(SeqId id);
  const Member* find(SeqId id) const;
  void stand(Member& m, Standing s);
  void take_portion(Member& m, int* budget, Schedule* plan);
  Roster::iterator youngest_running();
  Roster::iterator next_in_line();

  SchedulerConfig cfg_;
  CacheManager* cache_;
  Roster roster_;
  std::unordered_map<SeqId, long long> arrival_of_;
  int standing_count_[3] = {0, 0, 0};
  long long next_arrival_ = 0;
  long long num_preemptions_ = 0;
};

}  // namespace rlis
