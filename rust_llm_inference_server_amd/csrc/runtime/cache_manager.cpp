#include "cache_manager.h"

#include <algorithm>
#include <sstream>
#include <stdexcept>

namespace rlis {

// ------------------------------------------------------------------ PageAllocator
PageAllocator::PageAllocator(int num_pages) : refcounts_(num_pages, 0) {
  free_.reserve(num_pages);
  for (int p = num_pages - 1; p >= 0; --p) free_.push_back(p);  // page 0 is handed out first
}

int PageAllocator::allocate() {
  if (free_.empty()) return -1;
  const int p = free_.back();
  free_.pop_back();
  if (refcounts_[p] != 0) throw std::logic_error("free page " + std::to_string(p) + " had references");
  refcounts_[p] = 1;
  return p;
}

void PageAllocator::incref(int p) {
  if (refcounts_.at(p) <= 0) throw std::logic_error("incref on free page " + std::to_string(p));
  ++refcounts_[p];
}

void PageAllocator::decref(int p) {
  if (refcounts_.at(p) <= 0) throw std::logic_error("double free of page " + std::to_string(p));
  if (--refcounts_[p] == 0) free_.push_back(p);
}

// ------------------------------------------------------------------- CacheManager
CacheManager::CacheManager(int page_size, std::vector<GroupSpec> groups, int num_state_slots)
    : page_size_(page_size), groups_(std::move(groups)), num_state_slots_(num_state_slots) {
  if (page_size_ <= 0) throw std::invalid_argument("page_size must be positive");
  if (groups_.empty()) throw std::invalid_argument("at least one page group is needed");
  for (const auto& g : groups_) {
    if (g.num_pages < 0 || g.window < 0) throw std::invalid_argument("bad page group");
    alloc_.emplace_back(g.num_pages);
  }
  for (int s = num_state_slots_ - 1; s >= 0; --s) free_slots_.push_back(s);
}

const SeqEntry* CacheManager::entry(SeqId s) const {
  auto it = seqs_.find(s);
  return it == seqs_.end() ? nullptr : &it->second;
}

// First logical page that a query at position >= computed can still see in group g.
int CacheManager::first_live_page(int computed, int g) const {
  const int w = groups_[g].window;
  if (w <= 0) return 0;
  const int first_pos = computed - w + 1;   // a query at `computed` sees keys > computed - w
  return first_pos <= 0 ? 0 : first_pos / page_size_;
}

bool CacheManager::needs_cow(const SeqEntry& e, int g) const {
  if (e.num_tokens % page_size_ == 0) return false;
  const auto& pages = e.pages[g];
  if (pages.empty() || pages.back() < 0) return false;
  return alloc_[g].refcount(pages.back()) > 1;
}

int CacheManager::pages_needed(SeqId s, int total_tokens, int g) const {
  const SeqEntry* e = entry(s);
  const int have = e ? (int)e->pages[g].size() : 0;
  const int held_tokens = e ? e->num_tokens : 0;
  if (total_tokens <= held_tokens) return 0;
  const int grow = std::max(0, pages_for(total_tokens) - have);
  return grow + ((e && needs_cow(*e, g)) ? 1 : 0);
}

ReserveResult CacheManager::reserve(SeqId s, int total_tokens, std::vector<PageCopy>* copies) {
  const bool is_new = !contains(s);
  for (int g = 0; g < num_groups(); ++g)
    if (pages_needed(s, total_tokens, g) > alloc_[g].num_free()) return kOutOfPages;
  if (is_new && num_state_slots_ > 0 && free_slots_.empty()) return kOutOfSlots;

  SeqEntry& e = seqs_[s];
  if (is_new) {
    e.pages.assign(num_groups(), {});
    if (num_state_slots_ > 0) {
      e.state_slot = free_slots_.back();
      free_slots_.pop_back();
    }
  }
  if (total_tokens <= e.num_tokens) return kReserved;   // shrinking is a no-op
  const int target = pages_for(total_tokens);
  for (int g = 0; g < num_groups(); ++g) {
    auto& pages = e.pages[g];
    if (needs_cow(e, g)) {
      const int fresh = alloc_[g].allocate();
      if (copies) copies->push_back(PageCopy{g, pages.back(), fresh});
      alloc_[g].decref(pages.back());
      pages.back() = fresh;
    }
    while ((int)pages.size() < target) pages.push_back(alloc_[g].allocate());
  }
  e.num_tokens = total_tokens;
  return kReserved;
}

void CacheManager::advance(SeqId s, int computed) {
  auto it = seqs_.find(s);
  if (it == seqs_.end()) throw std::invalid_argument("advance of unknown request " + std::to_string(s));
  SeqEntry& e = it->second;
  if (computed > e.num_tokens)
    throw std::invalid_argument("advance past the reserved positions of request " + std::to_string(s));
  if (computed < e.num_computed) return;
  e.num_computed = computed;
  for (int g = 0; g < num_groups(); ++g) {
    const int live = std::min(first_live_page(computed, g), (int)e.pages[g].size());
    for (int i = 0; i < live; ++i) {
      if (e.pages[g][i] >= 0) {
        alloc_[g].decref(e.pages[g][i]);
        e.pages[g][i] = -1;
      }
    }
  }
}

void CacheManager::fork(SeqId parent, SeqId child) {
  auto it = seqs_.find(parent);
  if (it == seqs_.end()) throw std::invalid_argument("fork of unknown request");
  if (contains(child)) throw std::invalid_argument("fork into an existing request");
  if (num_state_slots_ > 0 && free_slots_.empty()) throw std::runtime_error("no state slot for a fork");
  SeqEntry c = it->second;
  for (int g = 0; g < num_groups(); ++g)
    for (int p : c.pages[g])
      if (p >= 0) alloc_[g].incref(p);
  if (num_state_slots_ > 0) {
    c.state_slot = free_slots_.back();
    free_slots_.pop_back();
  }
  seqs_[child] = std::move(c);
}

void CacheManager::free_seq(SeqId s) {
  auto it = seqs_.find(s);
  if (it == seqs_.end()) return;   // unknown requests are ignored (lib.rs:356-364)
  for (int g = 0; g < num_groups(); ++g)
    for (int p : it->second.pages[g])
      if (p >= 0) alloc_[g].decref(p);
  if (it->second.state_slot >= 0) free_slots_.push_back(it->second.state_slot);
  seqs_.erase(it);
}

std::string CacheManager::check_invariants() const {
  std::ostringstream err;
  for (int g = 0; g < num_groups(); ++g) {
    const int n = alloc_[g].num_pages();
    std::vector<int> holders(n, 0);
    for (const auto& kv : seqs_) {
      const SeqEntry& e = kv.second;
      if ((int)e.pages[g].size() != pages_for(e.num_tokens)) {
        err << "request " << kv.first << " group " << g << ": " << e.pages[g].size()
            << " pages for " << e.num_tokens << " tokens";
        return err.str();
      }
      const int live = first_live_page(e.num_computed, g);
      for (int i = 0; i < (int)e.pages[g].size(); ++i) {
        const int p = e.pages[g][i];
        if (p < 0) {
          if (i >= live) {
            err << "request " << kv.first << " group " << g << ": live page " << i << " is missing";
            return err.str();
          }
          continue;
        }
        if (p >= n) {
          err << "request " << kv.first << " group " << g << ": page id " << p << " out of range";
          return err.str();
        }
        if (i < live) {
          err << "request " << kv.first << " group " << g << ": page " << i
              << " is behind the window and still held";
          return err.str();
        }
        ++holders[p];
      }
    }
    std::vector<char> in_free(n, 0);
    for (int p : alloc_[g].free_list()) {
      if (p < 0 || p >= n) {
        err << "group " << g << ": free list holds page id " << p;
        return err.str();
      }
      if (in_free[p]) {
        err << "group " << g << ": page " << p << " is on the free list twice";
        return err.str();
      }
      in_free[p] = 1;
    }
    for (int p = 0; p < n; ++p) {
      const int rc = alloc_[g].refcount(p);
      if (rc != holders[p]) {
        err << "group " << g << " page " << p << ": refcount " << rc << " but " << holders[p]
            << " tables hold it";
        return err.str();
      }
      if ((rc == 0) != (in_free[p] != 0)) {
        err << "group " << g << " page " << p << ": refcount " << rc << ", on the free list: "
            << (int)in_free[p];
        return err.str();
      }
    }
  }
  if (num_state_slots_ > 0) {
    std::vector<int> used(num_state_slots_, 0);
    for (const auto& kv : seqs_) {
      const int s = kv.second.state_slot;
      if (s < 0 || s >= num_state_slots_) {
        err << "request " << kv.first << " holds no valid state slot";
        return err.str();
      }
      if (used[s]++) {
        err << "state slot " << s << " is held twice";
        return err.str();
      }
    }
    for (int s : free_slots_) {
      if (s < 0 || s >= num_state_slots_ || used[s]++) {
        err << "state slot " << s << " is both free and held, or free twice";
        return err.str();
      }
    }
    for (int s = 0; s < num_state_slots_; ++s)
      if (!used[s]) {
        err << "state slot " << s << " is lost";
        return err.str();
      }
  }
  return std::string();
}

}  // namespace rlis
