#include "cache_manager.h"

#include <algorithm>
#include <stdexcept>

namespace rlis {

// ------------------------------------------------------------------------- PagePool
PagePool::PagePool(int num_pages) : refs_(num_pages, 0), below_(num_pages, -1) {
  // Stack the pages so that page 0 lies on top of a fresh pool.
  for (int p = num_pages - 1; p >= 0; --p) {
    below_[p] = top_;
    top_ = p;
  }
  free_count_ = num_pages;
}

int PagePool::take() {
  if (top_ < 0) return -1;
  const int p = top_;
  if (refs_[p] != 0) throw std::logic_error("page " + std::to_string(p) + " lay free while held");
  top_ = below_[p];
  below_[p] = -1;
  refs_[p] = 1;
  --free_count_;
  return p;
}

void PagePool::share(int p) {
  if (refs_.at(p) < 1) throw std::logic_error("page " + std::to_string(p) + " is shared but not held");
  ++refs_[p];
}

void PagePool::drop(int p) {
  if (refs_.at(p) < 1) throw std::logic_error("page " + std::to_string(p) + " is returned twice");
  if (--refs_[p] == 0) {
    below_[p] = top_;
    top_ = p;
    ++free_count_;
  }
}

std::vector<int> PagePool::free_pages() const {
  std::vector<int> out;
  // A broken chain must not run forever: it can hold at most size() pages.
  for (int p = top_; p >= 0 && (int)out.size() <= size(); p = below_[p]) out.push_back(p);
  return out;
}

// --------------------------------------------------------------------- CacheManager
CacheManager::CacheManager(int page_size, std::vector<GroupSpec> groups, int num_state_slots)
    : page_size_(page_size), groups_(std::move(groups)), num_seats_(num_state_slots) {
  if (page_size_ <= 0) throw std::invalid_argument("page_size must be positive");
  if (groups_.empty()) throw std::invalid_argument("at least one page group is needed");
  for (const GroupSpec& g : groups_) {
    if (g.num_pages < 0 || g.window < 0) throw std::invalid_argument("bad page group");
    pools_.emplace_back(g.num_pages);
  }
  for (int seat = num_seats_ - 1; seat >= 0; --seat) free_seats_.push_back(seat);   // seat 0 on top
}

const Lease* CacheManager::lease(SeqId s) const {
  auto it = leases_.find(s);
  return it == leases_.end() ? nullptr : &it->second;
}

// The first logical page that a query at position `computed` or later can still see in group g:
// with a window w such a query sees keys after computed - w.
int CacheManager::first_visible_page(int computed, int g) const {
  const int w = groups_[g].window;
  const int oldest = w > 0 ? computed - w + 1 : 0;
  return oldest > 0 ? oldest / page_size_ : 0;
}

Quote CacheManager::quote(SeqId s, int total_tokens) const {
  const Lease* l = lease(s);
  Quote q;
  q.pages.assign(num_groups(), 0);
  q.seat = !l && num_seats_ > 0;
  const int reserved = l ? l->reserved : 0;
  const int upto = std::max(total_tokens, reserved);
  for (int g = 0; g < num_groups(); ++g) {
    const int have = l ? l->runs[g].count() : 0;
    int need = std::max(0, pages_for(upto) - have);
    if (l && total_tokens > l->computed) {
      // pages that the range [computed, total) lands in and that someone else holds too
      const PageRun& run = l->runs[g];
      const int last = std::min(have, pages_for(total_tokens));
      for (int i = std::max(l->computed / page_size_, run.gone); i < last; ++i)
        if (pools_[g].refs(run.at(i)) > 1) ++need;
    }
    q.pages[g] = need;
  }
  return q;
}

bool CacheManager::affordable(const Quote& q, int spare, bool* short_of_seats) const {
  if (short_of_seats) *short_of_seats = false;
  for (int g = 0; g < num_groups(); ++g)
    if (q.pages[g] + spare > pools_[g].free_count()) return false;
  if (q.seat && free_seats_.empty()) {
    if (short_of_seats) *short_of_seats = true;
    return false;
  }
  return true;
}

ReserveResult CacheManager::reserve(SeqId s, int total_tokens, std::vector<PageCopy>* copies) {
  const Quote q = quote(s, total_tokens);
  bool seats = false;
  if (!affordable(q, 0, &seats)) return seats ? kOutOfSlots : kOutOfPages;

  Lease& l = leases_[s];
  if (l.runs.empty()) {
    l.runs.resize(num_groups());
    if (q.seat) {
      l.seat = free_seats_.back();
      free_seats_.pop_back();
    }
  }
  const int upto = std::max(total_tokens, l.reserved);
  for (int g = 0; g < num_groups(); ++g) {
    PageRun& run = l.runs[g];
    PagePool& pool = pools_[g];
    if (total_tokens > l.computed) {
      const int last = std::min(run.count(), pages_for(total_tokens));
      for (int i = std::max(l.computed / page_size_, run.gone); i < last; ++i) {
        int& page = run.live[i - run.gone];
        if (pool.refs(page) > 1) {
          const int own = pool.take();
          if (copies) copies->push_back(PageCopy{g, page, own});
          pool.drop(page);
          page = own;
        }
      }
    }
    while (run.count() < pages_for(upto)) run.live.push_back(pool.take());
  }
  l.reserved = upto;
  return kReserved;
}

void CacheManager::advance(SeqId s, int computed) {
  auto it = leases_.find(s);
  if (it == leases_.end())
    throw std::invalid_argument("advance of unknown request " + std::to_string(s));
  Lease& l = it->second;
  if (computed > l.reserved)
    throw std::invalid_argument("advance past the reserved positions of request " + std::to_string(s));
  if (computed <= l.computed) return;
  l.computed = computed;
  for (int g = 0; g < num_groups(); ++g) {
    PageRun& run = l.runs[g];
    const int keep_from = std::min(first_visible_page(computed, g), run.count());
    const int passed = keep_from - run.gone;
    if (passed <= 0) continue;
    for (int i = 0; i < passed; ++i) pools_[g].drop(run.live[i]);
    run.live.erase(run.live.begin(), run.live.begin() + passed);
    run.gone = keep_from;
  }
}

std::pair<int, int> CacheManager::fork(SeqId parent, SeqId child) {
  auto it = leases_.find(parent);
  if (it == leases_.end()) throw std::invalid_argument("fork of unknown request");
  if (contains(child)) throw std::invalid_argument("fork into an existing request");
  if (num_seats_ > 0 && free_seats_.empty()) throw std::runtime_error("no state slot for a fork");
  const Lease& from = it->second;
  Lease to;
  to.reserved = to.computed = from.computed;
  to.runs.resize(num_groups());
  const int pages = pages_for(from.computed);
  for (int g = 0; g < num_groups(); ++g) {
    const PageRun& src = from.runs[g];
    PageRun& dst = to.runs[g];
    dst.gone = std::min(src.gone, pages);
    for (int i = dst.gone; i < pages; ++i) {
      pools_[g].share(src.at(i));
      dst.live.push_back(src.at(i));
    }
  }
  if (num_seats_ > 0) {
    to.seat = free_seats_.back();
    free_seats_.pop_back();
  }
  const std::pair<int, int> seats(from.seat, to.seat);
  leases_[child] = std::move(to);
  return seats;
}

void CacheManager::free_seq(SeqId s) {
  auto it = leases_.find(s);
  if (it == leases_.end()) return;   // a request that holds nothing has nothing to return
  for (int g = 0; g < num_groups(); ++g)
    for (int p : it->second.runs[g].live) pools_[g].drop(p);
  if (it->second.seat >= 0) free_seats_.push_back(it->second.seat);
  leases_.erase(it);
}

// The audit counts every page from both sides: who holds it according to the leases, and what
// the pool believes.  A page is either free (on the stack once, held by no one) or held by
// exactly as many leases as its count says.
std::string CacheManager::audit() const {
  auto who = [](SeqId s, int g) { return "request " + std::to_string(s) + ", group " + std::to_string(g); };
  for (int g = 0; g < num_groups(); ++g) {
    const PagePool& pool = pools_[g];
    std::vector<int> holders(pool.size(), 0);
    for (const auto& entry : leases_) {
      const Lease& l = entry.second;
      const PageRun& run = l.runs[g];
      if (l.computed > l.reserved)
        return who(entry.first, g) + ": " + std::to_string(l.computed) + " positions computed of " +
               std::to_string(l.reserved) + " reserved";
      if (run.count() != pages_for(l.reserved))
        return who(entry.first, g) + ": " + std::to_string(run.count()) + " pages back " +
               std::to_string(l.reserved) + " positions";
      const int visible = std::min(first_visible_page(l.computed, g), run.count());
      if (run.gone != visible)
        return who(entry.first, g) + ": pages up to " + std::to_string(run.gone) +
               " are gone, the window has passed " + std::to_string(visible);
      for (int p : run.live) {
        if (p < 0 || p >= pool.size())
          return who(entry.first, g) + ": holds page " + std::to_string(p) + ", which does not exist";
        ++holders[p];
      }
    }
    std::vector<char> stacked(pool.size(), 0);
    const std::vector<int> free_pages = pool.free_pages();
    if ((int)free_pages.size() != pool.free_count())
      return "group " + std::to_string(g) + ": " + std::to_string(free_pages.size()) +
             " pages on the free stack, the pool counts " + std::to_string(pool.free_count());
    for (int p : free_pages) {
      if (stacked[p]) return "group " + std::to_string(g) + ": page " + std::to_string(p) + " lies free twice";
      stacked[p] = 1;
    }
    for (int p = 0; p < pool.size(); ++p) {
      if (pool.refs(p) != holders[p])
        return "group " + std::to_string(g) + ": page " + std::to_string(p) + " counts " +
               std::to_string(pool.refs(p)) + " holders, the leases name " + std::to_string(holders[p]);
      if ((holders[p] == 0) != (stacked[p] != 0))
        return "group " + std::to_string(g) + ": page " + std::to_string(p) +
               (stacked[p] ? " is held and lies free" : " is neither held nor free (lost)");
    }
  }
  if (num_seats_ > 0) {
    std::vector<int> taken(num_seats_, 0);
    for (const auto& entry : leases_) {
      const int seat = entry.second.seat;
      if (seat < 0 || seat >= num_seats_)
        return "request " + std::to_string(entry.first) + " has no seat";
      if (taken[seat]++) return "seat " + std::to_string(seat) + " is taken twice";
    }
    for (int seat : free_seats_) {
      if (seat < 0 || seat >= num_seats_ || taken[seat]++)
        return "seat " + std::to_string(seat) + " is free and taken, or free twice";
    }
    for (int seat = 0; seat < num_seats_; ++seat)
      if (!taken[seat]) return "seat " + std::to_string(seat) + " is lost";
  }
  return std::string();
}

}  // namespace rlis
