// Token selection on the device, one workgroup per row of float32 logits: greedy argmax, or
// temperature sampling by the Gumbel-max trick with noise from a counter-based hash of
// (row key, token id), so a draw does not depend on what else is in the batch.
//
// Exactly the reference's formulas (crates/model/src/sampling.rs:11-23, 53-63, 84-100 and
// sampling.metal:26-74): h = lowbias32(key ^ (v * 0x9e3779b9)); u = ((h >> 9) + 0.5) / 2^23;
// score = logit * (1/T) - ln(-ln(u)); the largest score wins, ties go to the lowest index;
// 1/T == 0 marks a greedy row.  The product and the sum are rounded separately (no fused
// multiply-add), as the host reference computes them.
#include "common.h"

#include <math.h>

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

template <int NT>
__global__ __launch_bounds__(NT) void sample_rows_kernel(const float* __restrict__ logits,
                                                         long long row_stride, int vocab,
                                                         const uint32_t* __restrict__ keys,
                                                         const float* __restrict__ inv_temps,
                                                         int* __restrict__ out) {
  __shared__ float s_best[NT / kWave];
  __shared__ int s_idx[NT / kWave];
  const int r = blockIdx.x;
  const float* row = logits + (long long)r * row_stride;
  const uint32_t key = keys[r];
  const float inv_t = inv_temps[r];
  float best = -INFINITY;
  int best_v = 0x7fffffff;
  for (int v = threadIdx.x; v < vocab; v += NT) {
    float s = row[v];
    if (inv_t > 0.f) {
      const uint32_t h = lowbias32(key ^ ((uint32_t)v * 0x9e3779b9u));
      const float u = __fmul_rn((float)(h >> 9) + 0.5f, 1.0f / 8388608.0f);
      const float g = -logf(-logf(u));
      s = __fadd_rn(__fmul_rn(s, inv_t), g);
    }
    if (better(s, v, best, best_v)) {
      best = s;
      best_v = v;
    }
  }
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
  if (threadIdx.x == 0) {
    for (int w = 1; w < NT / kWave; ++w)
      if (better(s_best[w], s_idx[w], best, best_v)) {
        best = s_best[w];
        best_v = s_idx[w];
      }
    // A row of NaNs or of -inf only never beats the start value: fall back to index 0,
    // as the host reference's scan does for -inf and an argmax would.
    out[r] = best_v == 0x7fffffff ? 0 : best_v;
  }
}

RLIS_API int rlis_sample_rows(const float* logits, long long row_stride, int rows, int vocab,
                              const uint32_t* keys, const float* inv_temps, int* out,
                              hipStream_t stream) {
  RLIS_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "sample_rows: bad sizes");
  if (rows == 0) return 0;
  sample_rows_kernel<1024><<<rows, 1024, 0, stream>>>(logits, row_stride, vocab, keys, inv_temps,
                                                      out);
  RLIS_LAUNCH_CHECK("sample_rows");
  return 0;
}
