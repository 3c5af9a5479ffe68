// Shared helpers for the gfx950 kernels: bf16 <-> f32 conversion, wave64 reductions and the
// error channel of the C entry points.  Every entry point returns 0 on success and nonzero
// after storing a message that rlis_last_error() returns; launches go to the stream the
// caller passes, nothing is allocated and nothing synchronises.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#define RLIS_API extern "C" __attribute__((visibility("default")))

typedef uint16_t bf16_t;

enum { RLIS_F32 = 0, RLIS_BF16 = 1 };

constexpr int kWave = 64;

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}

// Round to nearest, ties to even; NaN stays NaN.
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (bf16_t)(u >> 16);
}

__device__ __forceinline__ float ld(const float* p) { return *p; }
__device__ __forceinline__ float ld(const bf16_t* p) { return bf16_to_f32(*p); }
__device__ __forceinline__ float widen(float v) { return v; }
__device__ __forceinline__ float widen(bf16_t v) { return bf16_to_f32(v); }
__device__ __forceinline__ void st(float* p, float v) { *p = v; }
__device__ __forceinline__ void st(bf16_t* p, float v) { *p = f32_to_bf16(v); }

// A delta for the residual stream that arrives as `parts` float32 partial sums, part_stride
// elements apart: they are added in order and, with round16, the sum is rounded to bfloat16 as
// a delta that arrives whole in bfloat16 was, so that a block's output is rounded once to the
// activation dtype whichever kernel produced it.
template <typename TD>
__device__ __forceinline__ float delta_sum(const TD* d, int parts, long long part_stride,
                                           int round16) {
  float s = ld(d);
  for (int p = 1; p < parts; ++p) s += ld(d + p * part_stride);
  return round16 ? bf16_to_f32(f32_to_bf16(s)) : s;
}

// Sum and maximum of a value with its partner 16 or 32 lanes away (lane ^ 16, lane ^ 32): every
// lane gets the result.  gfx950 swaps 16- and 32-lane halves of two registers in the vector
// unit (v_permlane16_swap: odd rows of the first with even rows of the second;
// v_permlane32_swap: upper half of the first with lower half of the second), which spares the
// trip through LDS that a general shuffle takes.  Swapping a value with itself leaves one
// register holding rows [0, 0, 2, 2] (halves [lo, lo]) and the other [1, 1, 3, 3] ([hi, hi]).
__device__ __forceinline__ float xor16_sum(float v) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float xor32_sum(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float xor16_max(float v) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xor32_max(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

__device__ __forceinline__ float wave_sum(float v) {
  v = xor32_sum(v);
  v = xor16_sum(v);
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
  v = xor32_max(v);
  v = xor16_max(v);
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

// Sum over a block of NT threads (NT a multiple of 64); every thread gets the result.  The
// order of the additions is fixed by NT alone.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* smem /* NT/64 floats */) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  __syncthreads();
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NT / kWave; ++i) t += smem[i];
  return t;
}

// ------------------------------------------------------------------ error channel
void rlis_set_error(const char* fmt, ...);

#define RLIS_REQUIRE(cond, ...)            \
  do {                                     \
    if (!(cond)) {                         \
      rlis_set_error(__VA_ARGS__);         \
      return 1;                            \
    }                                      \
  } while (0)

// A kernel's limit of dynamic LDS is raised once on every device it runs on (function
// attributes are the device's): `LdsGrant` remembers where, `grant_lds` raises it for the
// current device when it has not been yet.
struct LdsGrant {
  static constexpr int kDevices = 64;
  bool done[kDevices] = {};
};
inline hipError_t grant_lds(LdsGrant& grant, const void* kernel, int bytes) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const bool known = dev >= 0 && dev < LdsGrant::kDevices;
  if (known && grant.done[dev]) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && known) grant.done[dev] = true;
  return e;
}

#define RLIS_LAUNCH_CHECK(name)                                              \
  do {                                                                       \
    hipError_t e_ = hipGetLastError();                                       \
    if (e_ != hipSuccess) {                                                  \
      rlis_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));  \
      return 1;                                                              \
    }                                                                        \
  } while (0)

// Rotation and cache write of a decode step's own tokens, when the decode attention kernel
// does them itself: q rows are (q heads | ... k heads at k_off | ... v heads at v_off).
struct DecodeRope {
  const float* cos;       // (max positions, rot / 2) float32; null: nothing is rotated
  const float* sin;
  const int* positions;   // (S) position of each sequence's token; null: q comes rotated and
                          // K, V are in the pages already
  const int* slots;       // (S) page * page_size + offset of the new key; null: no cache write
  long long k_off, v_off;
  int rot;                // rotated width of a head
};

// Where the workgroups of one decode attention launch count themselves in when they merge a
// sequence's partitions inside the kernel: `slots` counters in device memory, one per (sequence,
// KV head), that the caller owns.  They are zero before the launch and the workgroup that
// merges sets its counter back to zero, so they are zero again after it.  Launches that share
// the counters must not overlap in time: a caller with several streams brings one set each.
struct DecodeMerge {
  unsigned* arrivals;     // null: the partitions are merged by a second kernel
  int slots;
};

// Keys per partition of a decode context of n visible keys: part_keys up to max_parts
// partitions, then the multiple of part_keys that keeps them at max_parts.  It depends on the
// sequence's own length and on constants only, so a sequence is cut (and its partitions are
// merged) the same way whatever else is in the batch; ceil(n / length) partitions are live.
__host__ __device__ inline int decode_part_len(int n, int part_keys, int max_parts) {
  const int span = part_keys * max_parts;
  const int mult = (n + span - 1) / span;
  return part_keys * (mult < 1 ? 1 : mult);
}

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
static inline long long ceil_div_ll(long long a, long long b) { return (a + b - 1) / b; }
