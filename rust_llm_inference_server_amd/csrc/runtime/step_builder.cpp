#include "step_builder.h"

#include <algorithm>
#include <set>
#include <stdexcept>

namespace rlis {

namespace {
long long round4(long long n) { return (n + 3) / 4 * 4; }
std::string request(long long id) { return "request " + std::to_string(id); }
}  // namespace

StepLayout plan_step(const CacheManager& cache, const std::vector<StepEntryView>& entries) {
  if (entries.empty()) throw std::invalid_argument("a step needs at least one request");
  StepLayout lay;
  const int n = (int)entries.size(), groups = cache.num_groups();
  // single tokens first, otherwise in the caller's order
  for (int pass = 0; pass < 2; ++pass)
    for (int i = 0; i < n; ++i)
      if ((entries[i].count == 1) == (pass == 0)) lay.order.push_back(i);
  std::set<long long> seen;
  lay.widths.assign(groups, 8);
  for (int i : lay.order) {
    const StepEntryView& e = entries[i];
    if (e.count <= 0) throw std::invalid_argument("empty sequence in batch");
    if (!seen.insert(e.seq).second)
      throw std::invalid_argument(request(e.seq) + " appears twice in one step");
    const Lease* l = cache.lease(e.seq);
    if (!l) throw std::invalid_argument(request(e.seq) + ": position 0 has no page reserved");
    if (l->computed + e.count > l->reserved)
      throw std::invalid_argument(request(e.seq) + ": position " + std::to_string(l->reserved) +
                                  " has no page reserved");
    lay.tokens += e.count;
    lay.wanted += e.num_want;
    lay.num_single += e.count == 1;
    lay.max_context = std::max(lay.max_context, l->computed + e.count);
    lay.max_new = std::max(lay.max_new, e.count);
    for (int g = 0; g < groups; ++g)
      lay.widths[g] = std::max(lay.widths[g], (l->runs[g].count() + 7) / 8 * 8);
  }
  lay.seqs = n;
  const long long T = lay.tokens, S = n;
  const long long sizes[kFixedArrays] = {T, T, T, S + 1, S, S, lay.wanted, S};
  long long at = 0;
  for (long long size : sizes) {
    lay.offsets.push_back(at);
    at += round4(size);
  }
  for (int g = 0; g < groups; ++g) {
    lay.offsets.push_back(at);
    at += round4(T);
    lay.offsets.push_back(at);
    at += round4(S * lay.widths[g]);
  }
  lay.total = at;
  return lay;
}

void fill_step(const CacheManager& cache, const std::vector<StepEntryView>& entries,
               const StepLayout& lay, int vocab_size, int* buf) {
  const int groups = cache.num_groups(), ps = cache.page_size(), S = lay.seqs;
  std::fill(buf, buf + lay.total, 0);
  int* ids = buf + lay.offsets[kIds];
  int* positions = buf + lay.offsets[kPositions];
  int* seq_of_token = buf + lay.offsets[kSeqOfToken];
  int* cu = buf + lay.offsets[kCu];
  int* start_pos = buf + lay.offsets[kStartPos];
  int* ctx_lens = buf + lay.offsets[kCtxLens];
  int* logit_rows = buf + lay.offsets[kLogitRows];
  int* state_slots = buf + lay.offsets[kStateSlots];
  std::vector<int> base_of(S, 0);
  int row = 0;
  cu[0] = 0;
  for (int s = 0; s < S; ++s) {
    const int i = lay.order[s];
    const StepEntryView& e = entries[i];
    const Lease* l = cache.lease(e.seq);
    base_of[i] = row;
    start_pos[s] = l->computed;
    ctx_lens[s] = l->computed + e.count;
    state_slots[s] = l->seat < 0 ? 0 : l->seat;
    for (int w = 0; w < e.num_want; ++w)
      if (e.want[w] < 0 || e.want[w] >= e.count)
        throw std::invalid_argument(request(e.seq) + ": wanted index " + std::to_string(e.want[w]) +
                                    " is outside its " + std::to_string(e.count) + " tokens");
    for (int t = 0; t < e.count; ++t) {
      const long long id = e.tokens[t];
      if (id < 0 || id >= vocab_size)
        throw std::invalid_argument(request(e.seq) + ": token id " + std::to_string(id) +
                                    " is outside the vocabulary of " + std::to_string(vocab_size));
      ids[row + t] = (int)id;
      positions[row + t] = l->computed + t;
      seq_of_token[row + t] = s;
    }
    for (int g = 0; g < groups; ++g) {
      const PageRun& run = l->runs[g];
      int* slots = buf + lay.offsets[kFixedArrays + 2 * g];
      int* table = buf + lay.offsets[kFixedArrays + 2 * g + 1] + (long long)s * lay.widths[g];
      for (size_t p = 0; p < run.live.size(); ++p) table[run.gone + p] = std::max(run.live[p], 0);
      for (int t = 0; t < e.count; ++t) {
        const int pos = l->computed + t, index = pos / ps;
        const int page = index < run.count() ? run.at(index) : -1;
        if (page < 0)
          throw std::invalid_argument(request(e.seq) + ": position " + std::to_string(pos) +
                                      " has no page reserved");
        slots[row + t] = page * ps + pos % ps;
      }
    }
    row += e.count;
    cu[s + 1] = row;
  }
  int r = 0;
  for (size_t i = 0; i < entries.size(); ++i)
    for (int w = 0; w < entries[i].num_want; ++w) logit_rows[r++] = base_of[i] + entries[i].want[w];
}

}  // namespace rlis
