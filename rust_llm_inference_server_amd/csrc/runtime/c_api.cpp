// C entry points of the host runtime (page manager and scheduler) for the Python binding.
// Handles are opaque pointers; functions return a negative value and keep a message for
// rlis_rt_last_error() when an argument is wrong or an internal check fails.
#include <cstring>
#include <exception>
#include <string>

#include "cache_manager.h"
#include "scheduler.h"
#include "step_builder.h"

#define RT_API extern "C" __attribute__((visibility("default")))

using rlis::CacheManager;
using rlis::Scheduler;

static thread_local std::string g_error;

RT_API const char* rlis_rt_last_error() { return g_error.c_str(); }

#define GUARD(expr)                     \
  try {                                 \
    expr;                               \
  } catch (const std::exception& e) {   \
    g_error = e.what();                 \
    return -1;                          \
  }

static int copy_message(const std::string& msg, char* buf, int cap) {
  if (buf && cap > 0) {
    std::strncpy(buf, msg.c_str(), cap - 1);
    buf[cap - 1] = 0;
  }
  return msg.empty() ? 0 : 1;
}

// ------------------------------------------------------------------------ cache
RT_API void* rlis_cache_create(int page_size, int num_groups, const int* windows,
                               const int* num_pages, int num_state_slots) {
  try {
    std::vector<rlis::GroupSpec> groups;
    for (int g = 0; g < num_groups; ++g) groups.push_back({windows[g], num_pages[g]});
    return new CacheManager(page_size, groups, num_state_slots);
  } catch (const std::exception& e) {
    g_error = e.what();
    return nullptr;
  }
}

RT_API void rlis_cache_destroy(void* h) { delete static_cast<CacheManager*>(h); }

// Returns 0 reserved, 1 out of pages, 2 out of state slots.  Copies come back as triples
// (group, src, dst); more than `cap` of them is an error.
RT_API int rlis_cache_reserve(void* h, long long seq, int total, int* copies, int cap, int* n_copies) {
  auto* m = static_cast<CacheManager*>(h);
  std::vector<rlis::PageCopy> out;
  int rc = 0;
  GUARD(rc = m->reserve(seq, total, &out));
  if ((int)out.size() > cap) {
    g_error = "copy list does not fit";
    return -1;
  }
  for (size_t i = 0; i < out.size(); ++i) {
    copies[3 * i] = out[i].group;
    copies[3 * i + 1] = out[i].src;
    copies[3 * i + 2] = out[i].dst;
  }
  if (n_copies) *n_copies = (int)out.size();
  return rc;
}

RT_API int rlis_cache_advance(void* h, long long seq, int computed) {
  GUARD(static_cast<CacheManager*>(h)->advance(seq, computed));
  return 0;
}

// seats[0..1] = the parent's and the child's state slot (-1, -1 without state slots): the
// device copies the first onto the second.
RT_API int rlis_cache_fork(void* h, long long parent, long long child, int* seats) {
  std::pair<int, int> moved(-1, -1);
  GUARD(moved = static_cast<CacheManager*>(h)->fork(parent, child));
  if (seats) {
    seats[0] = moved.first;
    seats[1] = moved.second;
  }
  return 0;
}

RT_API int rlis_cache_free(void* h, long long seq) {
  GUARD(static_cast<CacheManager*>(h)->free_seq(seq));
  return 0;
}

RT_API int rlis_cache_num_free(void* h, int g) { return static_cast<CacheManager*>(h)->num_free(g); }
RT_API int rlis_cache_num_pages(void* h, int g) { return static_cast<CacheManager*>(h)->num_pages(g); }
RT_API int rlis_cache_refcount(void* h, int g, int p) { return static_cast<CacheManager*>(h)->refcount(g, p); }
RT_API int rlis_cache_num_free_slots(void* h) { return static_cast<CacheManager*>(h)->num_free_slots(); }
RT_API int rlis_cache_contains(void* h, long long seq) { return static_cast<CacheManager*>(h)->contains(seq); }

// Pages that reserve(seq, total) would take from group g (growth plus copies of shared pages).
RT_API int rlis_cache_pages_needed(void* h, long long seq, int total, int g) {
  return static_cast<CacheManager*>(h)->quote(seq, total).pages[g];
}

// Writes the block table of (seq, group) into out (up to cap entries) and returns its
// length, or -1 for an unknown request.
RT_API int rlis_cache_table(void* h, long long seq, int g, int* out, int cap) {
  const rlis::Lease* l = static_cast<CacheManager*>(h)->lease(seq);
  if (!l) return -1;
  const rlis::PageRun& run = l->runs[g];
  const int n = run.count() < cap ? run.count() : cap;
  for (int i = 0; i < n; ++i) out[i] = run.at(i);
  return run.count();
}

// info[0..2] = reserved tokens, computed tokens, state slot; returns -1 for an unknown request.
RT_API int rlis_cache_info(void* h, long long seq, int* info) {
  const rlis::Lease* l = static_cast<CacheManager*>(h)->lease(seq);
  if (!l) return -1;
  info[0] = l->reserved;
  info[1] = l->computed;
  info[2] = l->seat;
  return 0;
}

// One decode token per request, for n requests at once: for request i writes the cached
// length (the new token's position) to positions[i], its state slot to state_slots[i], and for
// every group g its block table into tables[g][i * width ...] (missing pages as 0, the rest
// of the row untouched) and the new token's write slot into slots[g][i].  tables and slots
// are arrays of one pointer per group.  Returns 0, or -1 with a message when a request is
// unknown, has no position reserved for the token, or a table is wider than `width`.
RT_API int rlis_cache_decode_batch(void* h, const long long* seqs, int n, int width,
                                   int* positions, int* state_slots, int** tables, int** slots) {
  auto* m = static_cast<CacheManager*>(h);
  const int ps = m->page_size();
  for (int i = 0; i < n; ++i) {
    const rlis::Lease* l = m->lease(seqs[i]);
    if (!l || l->computed + 1 > l->reserved) {
      g_error = "request " + std::to_string(seqs[i]) + ": position " +
                std::to_string(l ? l->reserved : 0) + " has no page reserved";
      return -1;
    }
    const int pos = l->computed;
    positions[i] = pos;
    state_slots[i] = l->seat < 0 ? 0 : l->seat;
    for (int g = 0; g < m->num_groups(); ++g) {
      const rlis::PageRun& run = l->runs[g];
      if (run.count() > width) {
        g_error = "block table of request " + std::to_string(seqs[i]) + " is wider than the buffer";
        return -1;
      }
      int* row = tables[g] + (long long)i * width;
      for (int p = 0; p < run.gone; ++p) row[p] = 0;
      for (size_t p = 0; p < run.live.size(); ++p) row[run.gone + p] = run.live[p];
      const int page = run.at(pos / ps);
      if (page < 0) {
        g_error = "request " + std::to_string(seqs[i]) + ": position " + std::to_string(pos) +
                  " has no page reserved";
        return -1;
      }
      slots[g][i] = page * ps + pos % ps;
    }
  }
  return 0;
}

// A step's common metadata (step_builder.h).  The entries come as parallel arrays: request
// ids, token counts, all tokens in one array, counts of wanted indices and all of those in one
// array.  rlis_cache_step_layout writes info = {tokens, sequences, wanted rows, single-token
// sequences, longest context, most new tokens, then the table width of every group}, the
// offsets of the arrays (8 + 2 per group), the entry index of every sequence of the step, and
// returns the buffer's size in ints; rlis_cache_step_fill fills a buffer of that size.  Both
// return a negative value with a message for a step that cannot run.
static std::vector<rlis::StepEntryView> entry_views(int n, const long long* seqs, const int* counts,
                                                    const long long* tokens, const int* want_counts,
                                                    const int* wants) {
  std::vector<rlis::StepEntryView> v(n > 0 ? n : 0);
  long long t = 0, w = 0;
  for (int i = 0; i < n; ++i) {
    v[i] = {seqs[i], tokens + t, counts[i], wants + w, want_counts[i]};
    t += counts[i] > 0 ? counts[i] : 0;
    w += want_counts[i] > 0 ? want_counts[i] : 0;
  }
  return v;
}

RT_API long long rlis_cache_step_layout(void* h, int n, const long long* seqs, const int* counts,
                                        const long long* tokens, const int* want_counts,
                                        const int* wants, int* info, long long* offsets,
                                        int* order) {
  auto* m = static_cast<CacheManager*>(h);
  rlis::StepLayout lay;
  GUARD(lay = rlis::plan_step(*m, entry_views(n, seqs, counts, tokens, want_counts, wants)));
  const int head[6] = {lay.tokens, lay.seqs, lay.wanted, lay.num_single, lay.max_context, lay.max_new};
  std::copy(head, head + 6, info);
  std::copy(lay.widths.begin(), lay.widths.end(), info + 6);
  std::copy(lay.offsets.begin(), lay.offsets.end(), offsets);
  std::copy(lay.order.begin(), lay.order.end(), order);
  return lay.total;
}

RT_API int rlis_cache_step_fill(void* h, int n, const long long* seqs, const int* counts,
                                const long long* tokens, const int* want_counts, const int* wants,
                                int vocab_size, int* buf, long long cap) {
  auto* m = static_cast<CacheManager*>(h);
  try {
    const auto entries = entry_views(n, seqs, counts, tokens, want_counts, wants);
    const rlis::StepLayout lay = rlis::plan_step(*m, entries);
    if (lay.total > cap) {
      g_error = "the step's metadata does not fit the buffer";
      return -1;
    }
    rlis::fill_step(*m, entries, lay, vocab_size, buf);
  } catch (const std::exception& e) {
    g_error = e.what();
    return -1;
  }
  return 0;
}

RT_API int rlis_cache_check(void* h, char* buf, int cap) {
  return copy_message(static_cast<CacheManager*>(h)->audit(), buf, cap);
}

// -------------------------------------------------------------------- scheduler
RT_API void* rlis_sched_create(void* cache, int max_num_seqs, int max_batched_tokens,
                               int watermark_pages, int policy) {
  try {
    rlis::SchedulerConfig cfg{max_num_seqs, max_batched_tokens, watermark_pages,
                              policy == 1 ? rlis::kStatic : rlis::kContinuous};
    return new Scheduler(cfg, static_cast<CacheManager*>(cache));
  } catch (const std::exception& e) {
    g_error = e.what();
    return nullptr;
  }
}

RT_API void rlis_sched_destroy(void* h) { delete static_cast<Scheduler*>(h); }

RT_API int rlis_sched_add(void* h, long long id, int prompt_len) {
  GUARD(static_cast<Scheduler*>(h)->add(id, prompt_len));
  return 0;
}

// seqs: triples (id, start, end) as long long; copies: triples (group, src, dst).
RT_API int rlis_sched_schedule(void* h, long long* seqs, int seq_cap, int* n_seqs,
                               long long* preempted, int pre_cap, int* n_pre, int* copies,
                               int copy_cap, int* n_copies) {
  rlis::Schedule s;
  GUARD(s = static_cast<Scheduler*>(h)->schedule());
  if ((int)s.seqs.size() > seq_cap || (int)s.preempted.size() > pre_cap ||
      (int)s.copies.size() > copy_cap) {
    g_error = "schedule does not fit the buffers";
    return -1;
  }
  for (size_t i = 0; i < s.seqs.size(); ++i) {
    seqs[3 * i] = s.seqs[i].id;
    seqs[3 * i + 1] = s.seqs[i].start;
    seqs[3 * i + 2] = s.seqs[i].end;
  }
  for (size_t i = 0; i < s.preempted.size(); ++i) preempted[i] = s.preempted[i];
  for (size_t i = 0; i < s.copies.size(); ++i) {
    copies[3 * i] = s.copies[i].group;
    copies[3 * i + 1] = s.copies[i].src;
    copies[3 * i + 2] = s.copies[i].dst;
  }
  *n_seqs = (int)s.seqs.size();
  *n_pre = (int)s.preempted.size();
  *n_copies = (int)s.copies.size();
  return 0;
}

RT_API int rlis_sched_advance(void* h, long long id, int end) {
  GUARD(static_cast<Scheduler*>(h)->advance(id, end));
  return 0;
}
RT_API int rlis_sched_append_token(void* h, long long id) {
  GUARD(static_cast<Scheduler*>(h)->append_token(id));
  return 0;
}
// One more token each for the n requests of ids (what rlis_sched_append_token does one by one).
RT_API int rlis_sched_append_tokens(void* h, const long long* ids, int n) {
  auto* s = static_cast<Scheduler*>(h);
  for (int i = 0; i < n; ++i) GUARD(s->append_token(ids[i]));
  return 0;
}
RT_API int rlis_sched_is_caught_up(void* h, long long id) { return static_cast<Scheduler*>(h)->is_caught_up(id); }
RT_API int rlis_sched_remove(void* h, long long id) {
  GUARD(static_cast<Scheduler*>(h)->remove(id));
  return 0;
}
RT_API int rlis_sched_has_work(void* h) { return static_cast<Scheduler*>(h)->has_work(); }
RT_API int rlis_sched_num_running(void* h) { return static_cast<Scheduler*>(h)->num_running(); }
RT_API int rlis_sched_num_waiting(void* h) { return static_cast<Scheduler*>(h)->num_waiting(); }
RT_API long long rlis_sched_num_preemptions(void* h) { return static_cast<Scheduler*>(h)->num_preemptions(); }
RT_API int rlis_sched_max_seq_tokens(void* h) { return static_cast<Scheduler*>(h)->max_seq_tokens(); }
RT_API int rlis_sched_num_tokens(void* h, long long id) { return static_cast<Scheduler*>(h)->num_tokens(id); }
RT_API int rlis_sched_num_computed(void* h, long long id) { return static_cast<Scheduler*>(h)->num_computed(id); }
RT_API int rlis_sched_check(void* h, char* buf, int cap) {
  return copy_message(static_cast<Scheduler*>(h)->check(), buf, cap);
}
