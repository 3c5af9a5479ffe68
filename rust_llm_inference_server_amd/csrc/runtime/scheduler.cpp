#include "scheduler.h"

#include <algorithm>
#include <sstream>
#include <stdexcept>

namespace rlis {

Scheduler::Scheduler(SchedulerConfig cfg, CacheManager* cache) : cfg_(cfg), cache_(cache) {
  if (cfg_.max_batched_tokens < cfg_.max_num_seqs)
    throw std::invalid_argument("max_batched_tokens must cover one decode token per sequence");
  if (cfg_.max_num_seqs <= 0) throw std::invalid_argument("max_num_seqs must be positive");
}

int Scheduler::max_seq_tokens() const {
  int pages = cache_->num_pages(0);
  for (int g = 1; g < cache_->num_groups(); ++g) pages = std::min(pages, cache_->num_pages(g));
  return std::max(0, pages - cfg_.watermark_pages) * cache_->page_size();
}

void Scheduler::add(SeqId id, int prompt_len) {
  if (prompt_len <= 0) throw std::invalid_argument("empty sequence");
  waiting_.push_back(SeqState{id, next_arrival_++, prompt_len, 0});
}

Schedule Scheduler::schedule() {
  Schedule out;
  int budget = cfg_.max_batched_tokens;
  schedule_running(&out, &budget);
  const bool may_admit =
      cfg_.policy == kContinuous ? out.preempted.empty() : running_.empty();
  if (may_admit) admit(&out, &budget);
  return out;
}

void Scheduler::schedule_running(Schedule* out, int* budget) {
  size_t i = 0;
  while (i < running_.size() && *budget > 0) {
    const SeqState& s = running_[i];
    const int want = std::min(s.num_tokens - s.num_computed, *budget);
    if (want == 0) {
      ++i;
      continue;
    }
    if (cache_->reserve(s.id, s.num_computed + want, &out->copies) == kReserved) {
      out->seqs.push_back(ScheduledSeq{s.id, s.num_computed, s.num_computed + want});
      *budget -= want;
      ++i;
    } else {
      // Free the newest request; if that is this one, it waits its turn.
      SeqState victim = running_.back();
      running_.pop_back();
      // The victim is never ahead of index i, so it holds no portion of this step yet.
      preempt(victim, out);
    }
  }
}

void Scheduler::preempt(SeqState s, Schedule* out) {
  cache_->free_seq(s.id);
  s.num_computed = 0;
  out->preempted.push_back(s.id);
  ++num_preemptions_;
  auto at = std::partition_point(preempted_.begin(), preempted_.end(),
                                 [&](const SeqState& p) { return p.arrival < s.arrival; });
  preempted_.insert(at, s);
}

void Scheduler::admit(Schedule* out, int* budget) {
  const bool ignore_budget = cfg_.policy == kStatic;
  while ((int)running_.size() < cfg_.max_num_seqs && (ignore_budget || *budget > 0)) {
    auto& queue = preempted_.empty() ? waiting_ : preempted_;
    if (queue.empty()) break;
    const SeqState& head = queue.front();
    bool fits = cache_->num_state_slots() == 0 || cache_->num_free_slots() > 0;
    for (int g = 0; fits && g < cache_->num_groups(); ++g)
      fits = cache_->pages_for(head.num_tokens) + cfg_.watermark_pages <= cache_->num_free(g);
    if (!fits) break;
    SeqState s = head;
    queue.pop_front();
    // Reserve the whole known length now, so later admissions cannot overcommit.
    if (cache_->reserve(s.id, s.num_tokens, &out->copies) != kReserved)
      throw std::logic_error("admission reserved less than it had checked");
    const int want = std::min(s.num_tokens - s.num_computed, std::max(*budget, 0));
    if (want > 0) {
      out->seqs.push_back(ScheduledSeq{s.id, s.num_computed, s.num_computed + want});
      *budget -= want;
    }
    auto at = std::partition_point(running_.begin(), running_.end(),
                                   [&](const SeqState& r) { return r.arrival < s.arrival; });
    running_.insert(at, s);
  }
}

const Scheduler::SeqState* Scheduler::find(SeqId id) const {
  for (const auto& s : running_)
    if (s.id == id) return &s;
  for (const auto& s : preempted_)
    if (s.id == id) return &s;
  for (const auto& s : waiting_)
    if (s.id == id) return &s;
  return nullptr;
}

void Scheduler::advance(SeqId id, int end) {
  for (auto& s : running_)
    if (s.id == id) {
      if (end > s.num_tokens) throw std::invalid_argument("advance past the known tokens");
      s.num_computed = end;
      cache_->advance(id, end);
      return;
    }
}

void Scheduler::append_token(SeqId id) {
  for (auto& s : running_)
    if (s.id == id) {
      ++s.num_tokens;
      return;
    }
}

bool Scheduler::is_caught_up(SeqId id) const {
  for (const auto& s : running_)
    if (s.id == id) return s.num_computed == s.num_tokens;
  return false;
}

void Scheduler::remove(SeqId id) {
  auto gone = [&](const SeqState& s) { return s.id == id; };
  running_.erase(std::remove_if(running_.begin(), running_.end(), gone), running_.end());
  waiting_.erase(std::remove_if(waiting_.begin(), waiting_.end(), gone), waiting_.end());
  preempted_.erase(std::remove_if(preempted_.begin(), preempted_.end(), gone), preempted_.end());
  cache_->free_seq(id);
}

int Scheduler::num_tokens(SeqId id) const {
  const SeqState* s = find(id);
  return s ? s->num_tokens : -1;
}

int Scheduler::num_computed(SeqId id) const {
  const SeqState* s = find(id);
  return s ? s->num_computed : -1;
}

std::string Scheduler::check() const {
  std::string e = cache_->check_invariants();
  if (!e.empty()) return e;
  std::ostringstream err;
  for (const auto& s : running_) {
    const SeqEntry* entry = cache_->entry(s.id);
    const int held = entry ? entry->num_tokens : 0;
    if (held < s.num_computed) {
      err << "request " << s.id << " computed " << s.num_computed << " but holds " << held << " slots";
      return err.str();
    }
  }
  for (const auto* q : {&waiting_, &preempted_})
    for (const auto& s : *q)
      if (cache_->contains(s.id)) {
        err << "queued request " << s.id << " holds pages";
        return err.str();
      }
  for (size_t i = 1; i < running_.size(); ++i)
    if (!(running_[i - 1].arrival < running_[i].arrival)) return "running is not sorted by arrival";
  if ((int)running_.size() > cfg_.max_num_seqs) return "more running requests than max_num_seqs";
  return std::string();
}

}  // namespace rlis
