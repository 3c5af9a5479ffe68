// Iteration-level scheduling over the paged cache: continuous batching with chunked prefill
// and preemption by recompute, as crates/engine/src/scheduler.rs of the reference decides it.
//
// A request is `num_tokens` (prompt plus generated) and `num_computed` (positions whose keys
// and values are cached); every step computes the next portion of the gap.  That one rule is
// prefill (gap = prompt), chunked prefill (gap above the token budget), decode (gap = 1) and
// recompute after preemption (gap = everything) (scheduler.rs:1-8).
//
//  * Running requests go first, oldest first, within max_batched_tokens (scheduler.rs:207-226).
//  * When a running request needs a page and none is free, the newest running request is
//    preempted: its pages and state slot are freed, it recomputes later (scheduler.rs:227-246).
//  * Admission is first come, first served: preempted requests (oldest first) before new ones,
//    only while the whole known length fits with `watermark` pages to spare in every group;
//    the head of the line is never skipped; no admission in a step that preempted
//    (scheduler.rs:193-205, 253-306).
//  * The static policy admits only when nothing is running, and ignores the token budget
//    then (scheduler.rs:197-200, 254-255).
// Left out: forked requests and the prefix cache.
#pragma once
#include <deque>
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

  // Longest request (prompt plus output) that can ever be admitted (scheduler.rs:48-53).
  int max_seq_tokens() const;
  void add(SeqId id, int prompt_len);
  Schedule schedule();
  void advance(SeqId id, int end);
  void append_token(SeqId id);
  bool is_caught_up(SeqId id) const;
  void remove(SeqId id);
  bool has_work() const { return !(running_.empty() && waiting_.empty() && preempted_.empty()); }
  int num_running() const { return (int)running_.size(); }
  int num_waiting() const { return (int)(waiting_.size() + preempted_.size()); }
  long long num_preemptions() const { return num_preemptions_; }
  int num_tokens(SeqId id) const;
  int num_computed(SeqId id) const;
  std::string check() const;

 private:
  struct SeqState {
    SeqId id;
    long long arrival;
    int num_tokens;
    int num_computed;
  };
  void schedule_running(Schedule* out, int* budget);
  void admit(Schedule* out, int* budget);
  void preempt(SeqState s, Schedule* out);
  const SeqState* find(SeqId id) const;

  SchedulerConfig cfg_;
  CacheManager* cache_;
  std::deque<SeqState> waiting_;
  std::deque<SeqState> preempted_;   // sorted by arrival
  std::vector<SeqState> running_;    // sorted by arrival; the last one is the victim
  long long next_arrival_ = 0;
  long long num_preemptions_ = 0;
};

}  // namespace rlis
