// Token selection on the device from rows of float32 logits: greedy argmax, or
// temperature sampling by the Gumbel-max trick with noise from a counter-based hash of
// (row key, token id), so a draw does not depend on what else is in the batch.
//
// Exactly the reference's formulas (crates/model/src/sampling.rs:11-23, 53-63, 84-100 and
// sampling.metal:26-74): h = lowbias32(key ^ (v * 0x9e3779b9)); u = ((h >> 9) + 0.5) / 2^23;
// score = logit * (1/T) - ln(-ln(u)); the largest score wins, ties go to the lowest index;
// 1/T == 0 marks a greedy row.  The product and the sum are rounded separately (no fused
// multiply-add), as the host reference computes them.
#include "common.h"
#include "no_alloc.h"

#include <math.h>

#include <mutex>

__device__ __forceinline__ uint32_t lowbias32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}

__device__ __forceinline__ bool better(float s, int v, float bs, int bv) {
  return s > bs || (s == bs && v < bv);
}

__device__ __forceinline__ float sample_score(float logit, int v, uint32_t key, float inv_t) {
  if (!(inv_t > 0.f)) return logit;
  const uint32_t h = lowbias32(key ^ ((uint32_t)v * 0x9e3779b9u));
  const float u = __fmul_rn((float)(h >> 9) + 0.5f, 1.0f / 8388608.0f);
  const float g = -logf(-logf(u));
  return __fadd_rn(__fmul_rn(logit, inv_t), g);
}

// Best (score, index) over the block; valid in thread 0.  `better` is a total order, so the
// result does not depend on how the candidates were spread over threads or chunks.
template <int NT>
__device__ __forceinline__ void block_best(float& best, int& best_v) {
  __shared__ float s_best[NT / kWave];
  __shared__ int s_idx[NT / kWave];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float os = __shfl_xor(best, o, kWave);
    const int ov = __shfl_xor(best_v, o, kWave);
    if (better(os, ov, best, best_v)) {
      best = os;
      best_v = ov;
    }
  }
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (lane == 0) {
    s_best[wave] = best;
    s_idx[wave] = best_v;
  }
  __syncthreads();
  if (threadIdx.x == 0)
    for (int w = 1; w < NT / kWave; ++w)
      if (better(s_best[w], s_idx[w], best, best_v)) {
        best = s_best[w];
        best_v = s_idx[w];
      }
}

// One workgroup per (chunk of the vocabulary, row).  With one chunk the token goes straight to
// out; with more, the chunk's best goes to part_best / part_idx (rows x chunks) and
// sample_final_kernel picks among them: a single row then keeps many compute units busy.
template <int NT>
__global__ __launch_bounds__(NT) void sample_rows_kernel(const float* __restrict__ logits,
                                                         long long row_stride, int vocab,
                                                         const uint32_t* __restrict__ keys,
                                                         const float* __restrict__ inv_temps,
                                                         int* __restrict__ out, int chunk_len,
                                                         float* __restrict__ part_best,
                                                         int* __restrict__ part_idx) {
  const int r = blockIdx.y, c = blockIdx.x;
  const float* row = logits + (long long)r * row_stride;
  const uint32_t key = keys[r];
  const float inv_t = inv_temps[r];
  float best = -INFINITY;
  int best_v = 0x7fffffff;
  const int end = min(vocab, (c + 1) * chunk_len);
  for (int v = c * chunk_len + threadIdx.x; v < end; v += NT) {
    const float s = sample_score(row[v], v, key, inv_t);
    if (better(s, v, best, best_v)) {
      best = s;
      best_v = v;
    }
  }
  block_best<NT>(best, best_v);
  if (threadIdx.x == 0) {
    if (gridDim.x == 1) {
      // A row of NaNs or of -inf only never beats the start value: fall back to index 0,
      // as the host reference's scan does for -inf and an argmax would.
      out[r] = best_v == 0x7fffffff ? 0 : best_v;
    } else {
      part_best[(long long)r * gridDim.x + c] = best;
      part_idx[(long long)r * gridDim.x + c] = best_v;
    }
  }
}

__global__ __launch_bounds__(64) void sample_final_kernel(const float* __restrict__ part_best,
                                                          const int* __restrict__ part_idx,
                                                          int chunks, int* __restrict__ out) {
  const int r = blockIdx.x;
  float best = -INFINITY;
  int best_v = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += 64) {
    const float s = part_best[(long long)r * chunks + c];
    const int v = part_idx[(long long)r * chunks + c];
    if (better(s, v, best, best_v)) {
      best = s;
      best_v = v;
    }
  }
  block_best<64>(best, best_v);
  if (threadIdx.x == 0) out[r] = best_v == 0x7fffffff ? 0 : best_v;
}

// chunks > 1 needs part_best and part_idx with rows * chunks entries each.
RLIS_API int rlis_sample_rows(const float* logits, long long row_stride, int rows, int vocab,
                              const uint32_t* keys, const float* inv_temps, int* out, int chunks,
                              float* part_best, int* part_idx, hipStream_t stream) {
  RLIS_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "sample_rows: bad sizes");
  RLIS_REQUIRE(chunks >= 1 && chunks <= 65535 && (chunks == 1 || (part_best && part_idx)),
               "sample_rows: %d chunks need scratch for the partial results", chunks);
  RLIS_REQUIRE(rows <= 65535, "sample_rows: %d rows, at most 65535", rows);
  if (rows == 0) return 0;
  const int chunk_len = ceil_div(vocab, chunks);
  if (chunks == 1) {
    sample_rows_kernel<1024><<<dim3(1, rows), 1024, 0, stream>>>(
        logits, row_stride, vocab, keys, inv_temps, out, chunk_len, nullptr, nullptr);
  } else {
    sample_rows_kernel<256><<<dim3(chunks, rows), 256, 0, stream>>>(
        logits, row_stride, vocab, keys, inv_temps, out, chunk_len, part_best, part_idx);
    sample_final_kernel<<<rows, 64, 0, stream>>>(part_best, part_idx, chunks, out);
  }
  RLIS_LAUNCH_CHECK("sample_rows");
  return 0;
}

// ------------------------------------------------------------ the variant that allocates nothing
// The per-chunk winners of rlis_sample_rows_static live here: kStaticMaxParts scores followed
// by as many indices.  In host code this name is only a stand-in for the device array (each GPU
// has a copy of its own at an address of its own); what kernels and copies get is the address
// that hipGetSymbolAddress returns for the current device, kept in g_scratch_ptr.
constexpr int kStaticMaxParts = 16384;
constexpr int kStaticMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticMaxParts * (sizeof(float) +
                                                                            sizeof(int))];
static void* g_scratch_ptr[kStaticMaxDevices];
static std::mutex g_scratch_mutex;

// The current device's copy of `scratch`; looked up once per device.
static int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  RLIS_REQUIRE(e == hipSuccess, "sample_rows_static: hipGetDevice failed: %s",
               hipGetErrorString(e));
  RLIS_REQUIRE(dev >= 0 && dev < kStaticMaxDevices,
               "sample_rows_static: device %d is beyond the %d devices it keeps scratch for", dev,
               kStaticMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    RLIS_REQUIRE(e == hipSuccess && p,
                 "sample_rows_static: hipGetSymbolAddress failed on device %d: %s", dev,
                 hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

RLIS_API int rlis_sample_rows_static_max_parts(void) { return kStaticMaxParts; }

RLIS_API int rlis_sample_rows_static(const float* logits, long long row_stride, int rows, int vocab,
                                     const uint32_t* keys, const float* inv_temps, int* out,
                                     int chunks, hipStream_t stream) {
  RLIS_REQUIRE(rows >= 0 && chunks >= 1, "sample_rows_static: bad sizes");
  RLIS_REQUIRE((long long)rows * chunks <= kStaticMaxParts,
               "sample_rows_static: %d rows x %d chunks exceed the %d partial results its static "
               "scratch holds", rows, chunks, kStaticMaxParts);
  if (chunks == 1 || rows == 0)
    return rlis_sample_rows(logits, row_stride, rows, vocab, keys, inv_temps, out, 1, nullptr,
                            nullptr, stream);
  void* base = nullptr;
  if (int rc = static_scratch(&base)) return rc;
  float* part_best = static_cast<float*>(base);
  int* part_idx = reinterpret_cast<int*>(part_best + kStaticMaxParts);
  return rlis_sample_rows(logits, row_stride, rows, vocab, keys, inv_temps, out, chunks, part_best,
                          part_idx, stream);
}
