// The part of a step's metadata that every mixer needs, laid out in one int32 buffer for one
// copy to the device.  The reference builds the same per step in PagedBatch::new
// (crates/model/src/paged.rs:256-296): the positions P_i .. P_i + n_i of every sequence in
// batch order, the write slot table[pos / page] * page + pos % page of every new token
// (paged.rs:258-263), zero-padded block tables and context lengths (paged.rs:199-213).
//
// Inside a step the sequences that bring a single token come first (the decode kernels take
// them beside the portions); `order` maps the step's sequences back to the caller's entries,
// and the wanted rows keep the order of the entries and of their `want`.
#pragma once
#include <string>
#include <vector>

#include "cache_manager.h"

namespace rlis {

struct StepEntryView {
  long long seq;
  const long long* tokens;   // the request's next tokens, continuing at its computed length
  int count;
  const int* want;           // indices among them whose logits are asked for
  int num_want;
};

// Arrays of the layout, each starting on a multiple of 4 ints (16 bytes).
enum StepArray {
  kIds = 0,        // T
  kPositions,      // T, absolute
  kSeqOfToken,     // T, index into the step's sequences
  kCu,             // S + 1
  kStartPos,       // S: positions cached before the step
  kCtxLens,        // S: positions cached after it
  kLogitRows,      // R: token rows whose logits are wanted
  kStateSlots,     // S
  kFixedArrays
};
// ... followed, for every page group g, by slots (T) and tables (S x width[g]).

struct StepLayout {
  int tokens = 0, seqs = 0, wanted = 0, num_single = 0, max_context = 0, max_new = 0;
  std::vector<int> widths;               // per group, a multiple of 8 and at least 8
  std::vector<long long> offsets;        // kFixedArrays + 2 * groups entries
  std::vector<int> order;                // entry index of every sequence of the step
  long long total = 0;                   // ints
};

// Sizes and offsets of the step's buffer.  Throws std::invalid_argument with the message the
// step builder's caller sees: an empty step, an empty sequence, a request twice, an unknown
// request or one without a reserved position for its tokens.
StepLayout plan_step(const CacheManager& cache, const std::vector<StepEntryView>& entries);

// Fills `buf` (layout.total ints).  Throws std::invalid_argument for a token outside the
// vocabulary, a wanted index outside a request's tokens or a position without a page.
void fill_step(const CacheManager& cache, const std::vector<StepEntryView>& entries,
               const StepLayout& layout, int vocab_size, int* buf);

}  // namespace rlis
