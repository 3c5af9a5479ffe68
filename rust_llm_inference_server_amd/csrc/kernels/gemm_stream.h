// What the streaming products (gemm.hip: up to 16 rows; gemm_wide.hip: 17 to 32 rows) share.
#pragma once
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

union Frag8 {
  uint4 u;
  bf16x8 v;
};

// ---- streaming skinny products
constexpr int kStreamItem = 256;                        // k per item
constexpr int kStreamTileBytes = 16 * kStreamItem * 2;  // one wave's tile in LDS

__device__ __forceinline__ void wave_lds_fence() {
  // LDS operations of one wave execute in order; this only stops the compiler from moving
  // reads of other lanes' data above the writes.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}


struct StreamShape {
  int T, N, K;
  long long ldx, ldw, ldy, part_stride;   // part_stride: elements between partial results
  int num_tiles, num_slices;
};


// NORM: x is not given but made on the fly as (resid + delta) * norm_weight, and the products
// are scaled by rsqrt(mean((resid + delta)^2) + eps) of their row at the end, which is the
// RMSNorm of crates/model/src/layers.rs:103-122 in front of the projection (the scale is one
// number per row and commutes with the product).  Needs all of K in one slice, so that the
// workgroup sees whole rows.  Workgroup 0 also stores resid + delta to resid_out.
struct StreamNorm {
  const float* resid;        // (rows, K) float32
  const void* delta;         // null, or `parts` arrays (rows, K), part_stride elements apart
  int delta_f32, parts;
  int round_parts;           // round the sum of the parts to bfloat16 before it is added
  long long part_stride;
  const void* weight;        // (K)
  int weight_f32;
  float eps;
  const int* rows;           // null, or the row of resid/delta that token t reads
  float* resid_out;          // null, or where resid + delta goes (not resid itself)
  // Without NORM, the two halves of a norm that sits between two products, neither of which
  // needs a prologue over whole rows.  The product in front of the norm (ss_out given; one k
  // slice, no gate) adds its result to resid (N wide, in place when resid_out is resid: every
  // element is read and written by one thread), and stores the sum, the sum times the norm's
  // weight in bfloat16, and per token and tile of output columns the sum of the squares.  The
  // product behind the norm (scale_parts given) takes those rows as its x and scales its
  // results by rsqrt(sum of the scale_count partial sums / K + eps) of their row.
  bf16_t* xw_out;            // (T, N) bfloat16
  float* ss_out;             // (rows up to a multiple of 16, ss_stride) float32: token-major,
                             // one entry per tile
  const float* scale_parts;  // the same layout, scale_count entries a token
  int scale_count;
  int ss_stride;             // a multiple of 4
};


// What a kernel does beside the product: nothing, the fused norm (x made from the residual in
// the prologue), the scale from partial sums of squares, or joining the residual at the end.
enum { kStreamPlain = 0, kStreamNorm = 1, kStreamScaled = 2, kStreamJoin = 3 };


// The compute units of the current device (0: unknown).
int rlis_stream_compute_units();

// Weight rows per tile (16, 12 or 8) for N outputs over `slices` k slices: a compute unit draws
// only its share of the memory bandwidth, however much it has in flight, so what counts is the
// most weight rows that any unit streams: rounds of tiles over the units times the rows of a
// tile.  Ties go to the larger tile (fewer workgroups, fewer prologues).
int rlis_stream_balanced_rows(int N, int slices, bool gated, int num_cus);

// The most rows of x that the streaming products take for rows of K: 16, or 32 where the kernel
// for 17 to 32 rows holds them (gemm_wide.hip).
int rlis_stream_wide_rows(int K);

// 17 to 32 rows (gemm_wide.hip).  mode: kStreamPlain, kStreamScaled or kStreamJoin; the
// arguments as the entry points of gemm.hip take them.
int rlis_launch_stream_wide(const char* name, int mode, const void* X, const void* W, void* Y,
                            int y_dtype, int T, int N, int K, long long ldx, long long ldw,
                            long long ldy, int gated, const StreamNorm& nm, hipStream_t stream);
