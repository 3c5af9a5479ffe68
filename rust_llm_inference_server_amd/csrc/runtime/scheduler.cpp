#include "scheduler.h"

#include <algorithm>
#include <stdexcept>

namespace rlis {

Scheduler::Scheduler(SchedulerConfig cfg, CacheManager* cache) : cfg_(cfg), cache_(cache) {
  if (cfg_.max_num_seqs <= 0) throw std::invalid_argument("max_num_seqs must be positive");
  if (cfg_.max_batched_tokens < cfg_.max_num_seqs)
    throw std::invalid_argument("max_batched_tokens must cover one decode token per sequence");
}

int Scheduler::max_seq_tokens() const {
  int smallest = cache_->num_pages(0);
  for (int g = 1; g < cache_->num_groups(); ++g) smallest = std::min(smallest, cache_->num_pages(g));
  return std::max(0, smallest - cfg_.watermark_pages) * cache_->page_size();
}

Scheduler::Member* Scheduler::find(SeqId id) {
  auto it = arrival_of_.find(id);
  return it == arrival_of_.end() ? nullptr : &roster_.at(it->second);
}

const Scheduler::Member* Scheduler::find(SeqId id) const {
  auto it = arrival_of_.find(id);
  return it == arrival_of_.end() ? nullptr : &roster_.at(it->second);
}

void Scheduler::stand(Member& m, Standing s) {
  --standing_count_[m.standing];
  m.standing = s;
  ++standing_count_[s];
}

void Scheduler::add(SeqId id, int prompt_len) {
  if (prompt_len <= 0) throw std::invalid_argument("empty sequence");
  if (arrival_of_.count(id)) throw std::invalid_argument("request " + std::to_string(id) + " is known already");
  const long long arrival = next_arrival_++;
  roster_.emplace(arrival, Member{id, prompt_len, 0, kQueued});
  arrival_of_[id] = arrival;
  ++standing_count_[kQueued];
}

// The next portion of m's gap goes into the plan (m holds the pages for it already).
void Scheduler::take_portion(Member& m, int* budget, Schedule* plan) {
  const int portion = std::min(m.tokens - m.computed, std::max(*budget, 0));
  if (portion <= 0) return;
  plan->seqs.push_back(ScheduledSeq{m.id, m.computed, m.computed + portion});
  *budget -= portion;
}

Scheduler::Roster::iterator Scheduler::youngest_running() {
  for (auto it = roster_.end(); it != roster_.begin();) {
    --it;
    if (it->second.standing == kRunning) return it;
  }
  return roster_.end();
}

// Who is admitted next: the oldest parked request, else the oldest queued one.
Scheduler::Roster::iterator Scheduler::next_in_line() {
  auto queued = roster_.end();
  for (auto it = roster_.begin(); it != roster_.end(); ++it) {
    if (it->second.standing == kParked) return it;
    if (it->second.standing == kQueued && queued == roster_.end()) {
      if (standing_count_[kParked] == 0) return it;
      queued = it;
    }
  }
  return queued;
}

Schedule Scheduler::schedule() {
  Schedule plan;
  int budget = cfg_.max_batched_tokens;

  // Pass 1: the running requests, oldest first.
  for (auto it = roster_.begin(); it != roster_.end() && budget > 0;) {
    Member& m = it->second;
    const int gap = m.tokens - m.computed;
    if (m.standing != kRunning || gap == 0) {
      ++it;
      continue;
    }
    const int portion = std::min(gap, budget);
    if (cache_->reserve(m.id, m.computed + portion, &plan.copies) == kReserved) {
      take_portion(m, &budget, &plan);
      ++it;
      continue;
    }
    // No room: the youngest running request gives way.  It stands at or behind `it` in the
    // roster, so it has no portion in this plan; if it is m itself, m simply waits.
    auto victim = youngest_running();
    cache_->free_seq(victim->second.id);
    victim->second.computed = 0;
    stand(victim->second, kParked);
    plan.preempted.push_back(victim->second.id);
    ++num_preemptions_;
    // `it` stays: m asks again, unless m was the victim and is skipped as not running.
  }

  // Pass 2: admission.
  const bool may_admit = cfg_.policy == kContinuous ? plan.preempted.empty()
                                                    : standing_count_[kRunning] == 0;
  const bool budget_counts = cfg_.policy != kStatic;
  while (may_admit && standing_count_[kRunning] < cfg_.max_num_seqs && (!budget_counts || budget > 0)) {
    auto it = next_in_line();
    if (it == roster_.end()) break;
    Member& m = it->second;
    if (!cache_->affordable(cache_->quote(m.id, m.tokens), cfg_.watermark_pages)) break;
    if (cache_->reserve(m.id, m.tokens, &plan.copies) != kReserved)
      throw std::logic_error("admission could not reserve what the cache had quoted");
    stand(m, kRunning);
    take_portion(m, &budget, &plan);
  }
  return plan;
}

void Scheduler::advance(SeqId id, int end) {
  Member* m = find(id);
  if (!m || m->standing != kRunning) return;
  if (end > m->tokens) throw std::invalid_argument("advance past the known tokens");
  m->computed = end;
  cache_->advance(id, end);
}

void Scheduler::append_token(SeqId id) {
  Member* m = find(id);
  if (m && m->standing == kRunning) ++m->tokens;
}

bool Scheduler::is_caught_up(SeqId id) const {
  const Member* m = find(id);
  return m && m->standing == kRunning && m->computed == m->tokens;
}

void Scheduler::remove(SeqId id) {
  auto it = arrival_of_.find(id);
  if (it != arrival_of_.end()) {
    --standing_count_[roster_.at(it->second).standing];
    roster_.erase(it->second);
    arrival_of_.erase(it);
  }
  cache_->free_seq(id);
}

int Scheduler::num_tokens(SeqId id) const {
  const Member* m = find(id);
  return m ? m->tokens : -1;
}

int Scheduler::num_computed(SeqId id) const {
  const Member* m = find(id);
  return m ? m->computed : -1;
}

std::string Scheduler::check() const {
  const std::string books = cache_->audit();
  if (!books.empty()) return books;
  int count[3] = {0, 0, 0};
  for (const auto& entry : roster_) {
    const Member& m = entry.second;
    ++count[m.standing];
    const Lease* lease = cache_->lease(m.id);
    if (m.standing == kRunning) {
      if (!lease || lease->reserved < m.computed)
        return "running request " + std::to_string(m.id) + " computed " + std::to_string(m.computed) +
               " positions but holds " + std::to_string(lease ? lease->reserved : 0);
    } else if (lease) {
      return "request " + std::to_string(m.id) + " waits and still holds pages";
    }
    if (m.computed > m.tokens)
      return "request " + std::to_string(m.id) + " computed more than it has tokens";
    auto known = arrival_of_.find(m.id);
    if (known == arrival_of_.end() || known->second != entry.first)
      return "request " + std::to_string(m.id) + " is missing from the index";
  }
  for (int s = 0; s < 3; ++s)
    if (count[s] != standing_count_[s]) return "the standing counts are off";
  if (arrival_of_.size() != roster_.size()) return "the index names requests that are gone";
  if (count[kRunning] > cfg_.max_num_seqs) return "more running requests than max_num_seqs";
  return std::string();
}

}  // namespace rlis
