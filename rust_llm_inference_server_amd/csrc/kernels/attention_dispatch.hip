// Checks the arguments of the matrix-core attention kernels and hands them to the unit built
// for the head size at hand.  Each unit (attention_mfma.hip compiled with RLIS_HEAD_DIM = 32,
// 64, ... 256) serves head sizes up to its own, padding the rest with zeros.
#include "common.h"

typedef int (*PrefillUnit)(const void* q, long long q_stride, void* out, long long out_stride,
                           const void* k_pages, const void* v_pages, const int* block_tables,
                           int max_pages, const int* cu_seqlens, const int* start_pos,
                           const int* tile_map, int num_tiles, int nh, int nkv, int d,
                           int page_shift, int window, float scale, int tile_queries, int splits,
                           int row0, float* part_ml, float* part_acc, const float* cos,
                           const float* sin, int rot, const float* slopes, hipStream_t stream);
typedef int (*DecodeUnit)(const void* q, long long q_stride, void* out, long long out_stride,
                          float* part_ml, float* part_acc, const void* k_pages,
                          const void* v_pages, const int* block_tables, int max_pages,
                          const int* ctx_lens, int S, int nh, int nkv, int d, int page_shift,
                          int window, float scale, int splits, int part_keys, int max_parts,
                          int merge_inside, int groups, int cap, const DecodeRope* rope,
                          const DecodeMerge* merge, const float* slopes, hipStream_t stream);

// The units (attention_mfma.hip compiled for a padded head size of 32, 64, ... 256) are
// libraries of their own, built and loaded when a model needs them and registered here.
constexpr int kUnits = 8;
static PrefillUnit prefill_units[kUnits];
static DecodeUnit decode_units[kUnits];

static int unit_index(int d) { return (d + 31) / 32 - 1; }

RLIS_API int rlis_attn_register_unit(int padded_head_dim, void* prefill, void* decode) {
  RLIS_REQUIRE(padded_head_dim % 32 == 0 && padded_head_dim >= 32 && padded_head_dim <= 32 * kUnits &&
                   prefill && decode,
               "attn_register_unit: bad unit for head size %d", padded_head_dim);
  prefill_units[unit_index(padded_head_dim)] = (PrefillUnit)prefill;
  decode_units[unit_index(padded_head_dim)] = (DecodeUnit)decode;
  return 0;
}

// What a unit's return code says.
static int unit_result(const char* name, int rc, int d) {
  if (rc == 0) return 0;
  if (rc == 1) rlis_set_error("%s: too many tiles", name);
  else if (rc == 2)
    rlis_set_error("%s: rotation inside the kernel needs head_dim = rotated width = 64, 128 or "
                   "256 (got %d)", name, d);
  else if (rc == 3)
    rlis_set_error("%s: partitions must be a multiple of 256 keys", name);
  else if (rc == 4)
    rlis_set_error("%s: too many sequences and KV heads to merge inside the kernel", name);
  else if (rc == 5)
    rlis_set_error("%s: a workgroup walks several partitions only when it merges inside, with "
                   "partitions of a multiple of 512 keys whose parked sums fit the LDS (64 KB up "
                   "to head size 64, 159 KB beyond)", name);
  else if (rc >= 1000)
    rlis_set_error("%s: launch failed: %s", name, hipGetErrorString((hipError_t)(rc - 1000)));
  else rlis_set_error("%s: unit error %d", name, rc);
  return 1;
}

int rlis_launch_attn_reduce_bf16(void* out, long long out_stride, const float* part_ml,
                                 const float* part_acc, int S, int nh, int d, int splits,
                                 hipStream_t stream);

// unit_map lists num_units quadruples (sequence, first new-token index of a tile, run, runs of
// the sequence): the keys of a tile of a sequence with more than one run are cut into that
// many runs, one workgroup each, whose partial results go to part_ml (rows, nh, part_stride, 2)
// and part_acc (rows, nh, part_stride, d) float32, indexed by the row relative to row0, and are
// merged afterwards by rlis_attn_reduce_rows.  part_stride is at least the largest run count
// (1: no sequence has runs, nothing is stored there).
//
// cos == null: q is rotated already.  Otherwise cos/sin are float32 (max positions, rot / 2)
// with rot = d = 64, 128 or 256, and the kernel turns each query by its position (start_pos of
// its sequence plus its index among the new tokens) as it loads it; q itself stays as it is.
//
// slopes != null: nh float32 values, one per query head; slopes[head] * (key position - query
// position) is added to every score in float32 before the softmax.
RLIS_API int rlis_attn_prefill_mfma(const void* q, long long q_stride, void* out,
                                    long long out_stride, const void* k_pages,
                                    const void* v_pages, const int* block_tables, int max_pages,
                                    const int* cu_seqlens, const int* start_pos,
                                    const int* unit_map, int num_tiles, int nh, int nkv, int d,
                                    int page_size, int window, float scale, int tile_queries,
                                    int splits, int row0, float* part_ml,
                                    float* part_acc, const float* cos, const float* sin,
                                    int rot, const float* slopes, hipStream_t stream) {
  // unit_map lists tiles of tile_queries new tokens: 64 (0 means that too) or 128.
  if (tile_queries == 0) tile_queries = 64;
  RLIS_REQUIRE(tile_queries == 64 || tile_queries == 128,
               "attn_prefill_mfma: tiles of %d queries, 64 or 128 only", tile_queries);
  RLIS_REQUIRE(num_tiles >= 0 && nh > 0 && nkv > 0 && d > 0 && page_size > 0,
               "attn_prefill_mfma: bad sizes");
  RLIS_REQUIRE(splits >= 1 && splits <= 64, "attn_prefill_mfma: %d key runs, 1 to 64", splits);
  RLIS_REQUIRE(splits == 1 || (part_ml && part_acc && row0 >= 0 && d % 4 == 0),
               "attn_prefill_mfma: key runs need a workspace and the first row they cover");
  RLIS_REQUIRE(scale > 0.f, "attn_prefill_mfma: the score scale must be positive, got %g", scale);
  RLIS_REQUIRE(nh % nkv == 0, "attn_prefill_mfma: %d query heads are not a multiple of %d KV heads",
               nh, nkv);
  RLIS_REQUIRE(d % 16 == 0 && d <= 256,
               "attn_prefill_mfma: head_dim %d must be a multiple of 16 and at most 256", d);
  RLIS_REQUIRE(page_size >= 8 && (page_size & (page_size - 1)) == 0,
               "attn_prefill_mfma: page size %d must be a power of two, at least 8", page_size);
  int page_shift = 0;
  while ((1 << page_shift) < page_size) ++page_shift;
  RLIS_REQUIRE(q_stride % 8 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)k_pages % 16) == 0 &&
                   ((uintptr_t)v_pages % 16) == 0,
               "attn_prefill_mfma: operands must be 16-byte aligned with row strides in steps of 8");
  RLIS_REQUIRE(!cos || (sin && ((uintptr_t)cos % 16) == 0 && ((uintptr_t)sin % 16) == 0),
               "attn_prefill_mfma: a rotation needs cos and sin, 16-byte aligned");
  const PrefillUnit unit = prefill_units[unit_index(d)];
  RLIS_REQUIRE(unit != nullptr, "attn_prefill_mfma: the unit for head size %d is not loaded", d);
  return unit_result(
      "attn_prefill_mfma",
      unit(q, q_stride, out, out_stride, k_pages, v_pages, block_tables, max_pages, cu_seqlens,
           start_pos, unit_map, num_tiles, nh, nkv, d, page_shift, window, scale, tile_queries,
           splits, row0, part_ml, part_acc, cos, sin, rot, slopes, stream),
      d);
}

// One query token per sequence (bfloat16): q rows are the sequences themselves.  Needs at most
// 16 query heads per KV head.  A sequence's visible keys are cut into partitions of
// decode_part_len(keys, part_keys, max_parts); `splits` must be at least the live partitions of
// the longest context (at most max_parts); part_ml (S, nh, splits, 2) and part_acc
// (S, nh, splits, d) float32 when splits > 1.
//
// positions == null: q is rotated and the pages hold the step's keys and values already.
// Otherwise the kernel does that itself: q rows hold the k heads at column k_off and the v
// heads at v_off; with cos/sin (float32 (max positions, rot / 2), rot = d = 64, 128 or 256) q
// and the new k are rotated by positions[s], without them nothing is; with slots the new k and
// v go to the pages at slots[s] (page * page_size + offset).
//
// arrivals != null: the partitions of a sequence are merged by the last of their workgroups to
// finish instead of by a second kernel (which still runs for more than arrival_slots sequences
// times KV heads).  The workgroups count themselves in at arrivals[sequence * nkv + KV head]:
// arrival_slots counters of the caller's, all zero before the launch and all zero again after
// it.  Same sums in the same order either way.  Launches that overlap in time (several streams)
// must not share counters: each stream, or each owner of a stream, brings its own.
//
// groups, cap: when merging inside, a sequence's partitions are dealt out evenly to `groups`
// workgroups (to more where a share would pass `cap` partitions, which is what the LDS holds
// of parked sums; cap = 1: a workgroup per partition).  The partitions, their sums and the
// order in which they are merged stay what part_keys makes them, so the floats are the same
// whoever computes them; fewer workgroups pay fewer start-ups and hand-overs, which a batch
// that fills the chip anyway does not need.
//
// slopes as in rlis_attn_prefill_mfma (the query's position is the last of its context).
RLIS_API int rlis_attn_decode_mfma(const void* q, long long q_stride, void* out,
                                   long long out_stride, float* part_ml, float* part_acc,
                                   void* k_pages, void* v_pages,
                                   const int* block_tables, int max_pages, const int* ctx_lens,
                                   int S, int nh, int nkv, int d, int page_size, int window,
                                   float scale, int splits, int part_keys, int max_parts,
                                   unsigned* arrivals, int arrival_slots, int groups, int cap,
                                   const float* cos, const float* sin,
                                   int rot, const int* positions, const int* slots,
                                   long long k_off, long long v_off, const float* slopes,
                                   hipStream_t stream) {
  DecodeRope rope;
  rope.cos = positions ? cos : nullptr;
  rope.sin = positions ? sin : nullptr;
  rope.positions = positions;
  rope.slots = positions ? slots : nullptr;
  rope.k_off = k_off;
  rope.v_off = v_off;
  rope.rot = rot;
  RLIS_REQUIRE(!rope.cos || (sin && rot % 2 == 0 && ((uintptr_t)cos % 16) == 0 &&
                             ((uintptr_t)sin % 16) == 0),
               "attn_decode_mfma: rotation needs cos and sin tables, 16-byte aligned");
  RLIS_REQUIRE(!rope.slots || (k_off >= (long long)nh * d && v_off >= 0 &&
                               k_off + (long long)nkv * d <= q_stride &&
                               v_off + (long long)nkv * d <= q_stride),
               "attn_decode_mfma: k and v columns %lld, %lld do not fit rows of %lld", k_off,
               v_off, q_stride);
  RLIS_REQUIRE(S >= 0 && nh > 0 && nkv > 0 && d > 0 && page_size > 0, "attn_decode_mfma: bad sizes");
  RLIS_REQUIRE(scale > 0.f, "attn_decode_mfma: the score scale must be positive, got %g", scale);
  RLIS_REQUIRE(nh % nkv == 0 && nh / nkv <= 16,
               "attn_decode_mfma: %d query heads per KV head, at most 16", nkv ? nh / nkv : 0);
  RLIS_REQUIRE(d % 16 == 0 && d <= 256,
               "attn_decode_mfma: head_dim %d must be a multiple of 16 and at most 256", d);
  RLIS_REQUIRE((long long)(nh / nkv) * (d + 2) * 32 <= 64 * 1024,
               "attn_decode_mfma: group of %d heads of size %d does not fit the merge buffer",
               nh / nkv, d);
  RLIS_REQUIRE(page_size >= 8 && (page_size & (page_size - 1)) == 0,
               "attn_decode_mfma: page size %d must be a power of two, at least 8", page_size);
  RLIS_REQUIRE(q_stride % 8 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)k_pages % 16) == 0 &&
                   ((uintptr_t)v_pages % 16) == 0,
               "attn_decode_mfma: operands must be 16-byte aligned with row strides in steps of 8");
  RLIS_REQUIRE(splits >= 1 && splits <= 8192 && S <= 65535, "attn_decode_mfma: bad grid");
  RLIS_REQUIRE(splits == 1 || (part_ml && part_acc), "attn_decode_mfma: partitions need a workspace");
  RLIS_REQUIRE(max_parts >= 1 && splits <= max_parts && part_keys > 0,
               "attn_decode_mfma: %d partitions deep, at most %d", splits, max_parts);
  int page_shift = 0;
  while ((1 << page_shift) < page_size) ++page_shift;
  const DecodeUnit unit = decode_units[unit_index(d)];
  RLIS_REQUIRE(unit != nullptr, "attn_decode_mfma: the unit for head size %d is not loaded", d);
  RLIS_REQUIRE(!arrivals || (arrival_slots > 0 && ((uintptr_t)arrivals % 4) == 0),
               "attn_decode_mfma: %d arrival counters", arrival_slots);
  const int inside = arrivals && splits > 1 && (long long)S * nkv <= arrival_slots;
  DecodeMerge merge;
  merge.arrivals = inside ? arrivals : nullptr;
  merge.slots = inside ? arrival_slots : 0;
  RLIS_REQUIRE(groups >= 1 && cap >= 1, "attn_decode_mfma: %d workgroups of up to %d partitions",
               groups, cap);
  if (!inside) cap = 1;           // same floats either way
  if (cap > splits) cap = splits;
  const int rc = unit_result(
      "attn_decode_mfma",
      unit(q, q_stride, out, out_stride, part_ml, part_acc, k_pages, v_pages, block_tables,
           max_pages, ctx_lens, S, nh, nkv, d, page_shift, window, scale, splits, part_keys,
           max_parts, inside, groups, cap, &rope, &merge, slopes, stream),
      d);
  if (rc) return rc;
  if (splits > 1 && S > 0 && !inside)
    return rlis_launch_attn_reduce_bf16(out, out_stride, part_ml, part_acc, S, nh, d, splits, stream);
  return 0;
}
