// Row-wise and element-wise kernels of the decoder step: embedding gather, residual add fused
// with RMSNorm, SwiGLU, rotary position encoding fused with the write of K and V into cache
// pages, and page copies.  All arithmetic is float32; storage is float32 or bfloat16.
//
// Formulas follow the reference: RMSNorm y = x * rsqrt(mean(x^2) + eps) * w
// (crates/model/src/layers.rs:141-146), SwiGLU silu(gate) * up (layers.rs:179-186), rotate-half
// rotation with per-position cos/sin rows (crates/model/src/rope.rs:111-117), K and V written
// at slot = table[pos / page] * page + pos % page before attention reads them
// (crates/model/src/paged.rs:258-263, 324-337).
#include "common.h"

static thread_local char g_err[512] = "";

void rlis_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

RLIS_API const char* rlis_last_error() { return g_err; }

// ------------------------------------------------------------------------ embedding
template <typename TW>
__global__ void embed_kernel(float* __restrict__ out, const TW* __restrict__ table,
                             const int* __restrict__ ids, int H) {
  const int t = blockIdx.x;
  const long long row = ids[t];
  const TW* src = table + row * H;
  float* dst = out + (long long)t * H;
  for (int j = threadIdx.x; j < H; j += blockDim.x) dst[j] = ld(src + j);
}

// out (T,H) f32 <- table[ids] ; ids are checked against V on the host before the call.
RLIS_API int rlis_embed(float* out, const void* table, int table_dtype, const int* ids, int T,
                        int H, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && H > 0, "embed: bad sizes T=%d H=%d", T, H);
  if (T == 0) return 0;
  if (table_dtype == RLIS_F32)
    embed_kernel<float><<<T, 256, 0, stream>>>(out, (const float*)table, ids, H);
  else if (table_dtype == RLIS_BF16)
    embed_kernel<bf16_t><<<T, 256, 0, stream>>>(out, (const bf16_t*)table, ids, H);
  else
    RLIS_REQUIRE(false, "embed: unknown table dtype %d", table_dtype);
  RLIS_LAUNCH_CHECK("embed");
  return 0;
}

// ------------------------------------------------------------------- residual add
// delta may come as `parts` partial sums of n elements each, one after the other; they are
// added in order (and their sum rounded to bfloat16 first when round_parts is set).
template <typename TD>
__global__ void add_residual_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                                    long long n, int parts, int round_parts) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    resid[i] += delta_sum(delta + i, parts, n, round_parts);
  }
}

RLIS_API int rlis_add_residual(float* resid, const void* delta, int delta_dtype, long long n,
                               int parts, int round_parts, hipStream_t stream) {
  RLIS_REQUIRE(parts >= 1, "add_residual: parts=%d", parts);
  if (n <= 0) return 0;
  const int blocks = (int)(ceil_div_ll(n, 256) < 4096 ? ceil_div_ll(n, 256) : 4096);
  if (delta_dtype == RLIS_F32)
    add_residual_kernel<float><<<blocks, 256, 0, stream>>>(resid, (const float*)delta, n, parts,
                                                           round_parts);
  else if (delta_dtype == RLIS_BF16)
    add_residual_kernel<bf16_t><<<blocks, 256, 0, stream>>>(resid, (const bf16_t*)delta, n, parts,
                                                            round_parts);
  else
    RLIS_REQUIRE(false, "add_residual: unknown dtype %d", delta_dtype);
  RLIS_LAUNCH_CHECK("add_residual");
  return 0;
}

// ------------------------------------------------------- residual add + RMSNorm
// One block per output row r; the source row is rows[r] when rows is given.  The residual is
// float32; delta (may be null) is added first and, when write_resid is set, the sum is stored
// back.  delta may come as `parts` partial sums, part_stride elements apart, added in order
// (their sum rounded to bfloat16 first when round_parts is set).
// Sum of squares, rsqrt and both multiplies are float32; one rounding at the store.
template <typename TD, typename TW, typename TO, int NT>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                                   const TW* __restrict__ weight, TO* __restrict__ out,
                                   const int* __restrict__ rows, int H, float eps,
                                   int write_resid, int parts, long long part_stride,
                                   int round_parts) {
  __shared__ float red[NT / kWave];
  const int r = blockIdx.x;
  const long long src = rows ? (long long)rows[r] : (long long)r;
  float* x = resid + src * H;
  const TD* d = delta ? delta + src * H : nullptr;
  float ss = 0.f;
  for (int j = threadIdx.x; j < H; j += NT) {
    float v = x[j];
    if (d) {
      v += delta_sum(d + j, parts, part_stride, round_parts);
      if (write_resid) x[j] = v;
    }
    ss += v * v;
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  TO* o = out + (long long)r * H;
  const bool reread_sum = d && !write_resid;
  for (int j = threadIdx.x; j < H; j += NT) {
    float v = x[j];
    if (reread_sum) v += delta_sum(d + j, parts, part_stride, round_parts);
    st(o + j, v * inv * ld(weight + j));
  }
}

// The same for rows of at most NT * VPT elements, which stay in registers between the sum
// of squares and the store: one read of every input, no second pass.
template <typename TD, typename TW, typename TO, int NT, int VPT>
__global__ __launch_bounds__(NT) void add_rmsnorm_small_kernel(
    float* __restrict__ resid, const TD* __restrict__ delta, const TW* __restrict__ weight,
    TO* __restrict__ out, const int* __restrict__ rows, int H, float eps, int write_resid,
    int parts, long long part_stride, int round_parts) {
  __shared__ float red[NT / kWave];
  const int r = blockIdx.x;
  const long long src = rows ? (long long)rows[r] : (long long)r;
  float* x = resid + src * H;
  const TD* d = delta ? delta + src * H : nullptr;
  float v[VPT], w[VPT];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int j = threadIdx.x + i * NT;
    v[i] = 0.f;
    w[i] = 0.f;
    if (j < H) {
      v[i] = x[j];
      if (d) v[i] += delta_sum(d + j, parts, part_stride, round_parts);
      w[i] = ld(weight + j);
    }
    ss += v[i] * v[i];
  }
  if (d && write_resid) {
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int j = threadIdx.x + i * NT;
      if (j < H) x[j] = v[i];
    }
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  TO* o = out + (long long)r * H;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int j = threadIdx.x + i * NT;
    if (j < H) st(o + j, v[i] * inv * w[i]);
  }
}

// The all-bfloat16 case with rows of a multiple of 8 and at most 256 * 8 * CH elements: eight
// elements per thread and chunk, 16- and 32-byte accesses.
template <int CH>
__global__ __launch_bounds__(256) void add_rmsnorm_bf16x8_kernel(
    float* __restrict__ resid, const bf16_t* __restrict__ delta, const bf16_t* __restrict__ weight,
    bf16_t* __restrict__ out, const int* __restrict__ rows, int H, float eps, int write_resid) {
  __shared__ float red[256 / kWave];
  const int r = blockIdx.x;
  const long long src = rows ? (long long)rows[r] : (long long)r;
  float* x = resid + src * H;
  const bf16_t* d = delta ? delta + src * H : nullptr;
  float v[CH][8];
  float ss = 0.f;
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    const int j = (threadIdx.x + ch * 256) * 8;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[ch][e] = 0.f;
    if (j < H) {
      const float4 a = *(const float4*)(x + j), b = *(const float4*)(x + j + 4);
      v[ch][0] = a.x; v[ch][1] = a.y; v[ch][2] = a.z; v[ch][3] = a.w;
      v[ch][4] = b.x; v[ch][5] = b.y; v[ch][6] = b.z; v[ch][7] = b.w;
      if (d) {
        const uint4 dv = *(const uint4*)(d + j);
        const uint32_t dw[4] = {dv.x, dv.y, dv.z, dv.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[ch][2 * e] += __uint_as_float(dw[e] << 16);
          v[ch][2 * e + 1] += __uint_as_float(dw[e] & 0xffff0000u);
        }
        if (write_resid) {
          *(float4*)(x + j) = make_float4(v[ch][0], v[ch][1], v[ch][2], v[ch][3]);
          *(float4*)(x + j + 4) = make_float4(v[ch][4], v[ch][5], v[ch][6], v[ch][7]);
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += v[ch][e] * v[ch][e];
    }
  }
  ss = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  bf16_t* o = out + (long long)r * H;
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    const int j = (threadIdx.x + ch * 256) * 8;
    if (j < H) {
      const uint4 wv = *(const uint4*)(weight + j);
      const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
      uint32_t ow[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float r0 = v[ch][2 * e] * inv * __uint_as_float(ww[e] << 16);
        const float r1 = v[ch][2 * e + 1] * inv * __uint_as_float(ww[e] & 0xffff0000u);
        ow[e] = (uint32_t)f32_to_bf16(r0) | ((uint32_t)f32_to_bf16(r1) << 16);
      }
      *(uint4*)(o + j) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
    }
  }
}

// True when the vectorised kernel took the call.
static bool launch_add_rmsnorm_bf16x8(float* resid, const void* delta, const void* weight, void* out,
                                      const int* rows, int R, int H, float eps, int write_resid,
                                      int parts, hipStream_t stream) {
  if (H % 8 != 0 || H > 256 * 8 * 4 || parts != 1) return false;
  if (((uintptr_t)resid | (uintptr_t)delta | (uintptr_t)weight | (uintptr_t)out) % 16) return false;
#define LAUNCH(CH)                                                                               \
  add_rmsnorm_bf16x8_kernel<CH><<<R, 256, 0, stream>>>(resid, (const bf16_t*)delta,              \
                                                       (const bf16_t*)weight, (bf16_t*)out, rows, \
                                                       H, eps, write_resid)
  if (H <= 256 * 8) LAUNCH(1);
  else if (H <= 256 * 16) LAUNCH(2);
  else LAUNCH(4);
#undef LAUNCH
  return true;
}

// The delta as a stack of float32 partial sums (what the split-k and the streaming products
// leave for their consumer), rows of a multiple of 4 and at most NT * 4 * CH elements: four
// elements per thread and chunk, 16-byte accesses.  Such stacks come with few rows (64 at most)
// and up to dozens of parts, so a row gets a wide workgroup (NT threads, as many as the row has
// groups of four, up to 1024) and every thread keeps eight parts of its chunk in flight (four
// of each where it has several chunks); the parts are added in order and their sum rounded to
// bfloat16 when round_parts is set.
template <typename TW, typename TO, int CH, int NT>
__global__ __launch_bounds__(NT) void add_rmsnorm_stack_kernel(
    float* __restrict__ resid, const float* __restrict__ delta, const TW* __restrict__ weight,
    TO* __restrict__ out, const int* __restrict__ rows, int H, float eps, int write_resid,
    int parts, long long part_stride, int round_parts) {
  __shared__ float red[NT / kWave];
  const int r = blockIdx.x;
  const long long src = rows ? (long long)rows[r] : (long long)r;
  float* x = resid + src * H;
  const float* d = delta + src * H;
  // A chunk past the row reads the row's first elements instead (and stores nothing).
  int col[CH];
  bool live[CH];
  float4 xr[CH], s[CH];
  // The norm's weight is asked for with the first loads, long before it is needed.
  TW wt[CH][4];
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    const int j = (threadIdx.x + ch * NT) * 4;
    live[ch] = j < H;
    col[ch] = live[ch] ? j : 0;
    xr[ch] = *(const float4*)(x + col[ch]);
#pragma unroll
    for (int e = 0; e < 4; ++e) wt[ch][e] = weight[col[ch] + e];
  }
  // The parts in batches of AHEAD, every batch's loads issued together and none under a
  // condition (a part past the last reads the last again and adds nothing): a stack of eight
  // parts is one trip to memory, and no part waits for the one before it.  They are added in
  // order, the first one as it is.
  constexpr int AHEAD = CH == 1 ? 8 : 4;
  for (int p = 0; p < parts; p += AHEAD) {
    float4 a[CH][AHEAD];
#pragma unroll
    for (int ch = 0; ch < CH; ++ch)
#pragma unroll
      for (int q = 0; q < AHEAD; ++q)
        a[ch][q] = *(const float4*)(d + (long long)min(p + q, parts - 1) * part_stride + col[ch]);
#pragma unroll
    for (int ch = 0; ch < CH; ++ch)
#pragma unroll
      for (int q = 0; q < AHEAD; ++q) {
        if (p == 0 && q == 0) {
          s[ch] = a[ch][0];
        } else if (p + q < parts) {
          s[ch].x += a[ch][q].x; s[ch].y += a[ch][q].y; s[ch].z += a[ch][q].z; s[ch].w += a[ch][q].w;
        }
      }
  }
  float v[CH][4];
  float ss = 0.f;
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    if (round_parts) {
      s[ch].x = bf16_to_f32(f32_to_bf16(s[ch].x)); s[ch].y = bf16_to_f32(f32_to_bf16(s[ch].y));
      s[ch].z = bf16_to_f32(f32_to_bf16(s[ch].z)); s[ch].w = bf16_to_f32(f32_to_bf16(s[ch].w));
    }
    v[ch][0] = xr[ch].x + s[ch].x; v[ch][1] = xr[ch].y + s[ch].y;
    v[ch][2] = xr[ch].z + s[ch].z; v[ch][3] = xr[ch].w + s[ch].w;
    if (live[ch]) {
      if (write_resid)
        *(float4*)(x + col[ch]) = make_float4(v[ch][0], v[ch][1], v[ch][2], v[ch][3]);
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += v[ch][e] * v[ch][e];
    }
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  TO* o = out + (long long)r * H;
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    if (live[ch]) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        st(o + col[ch] + e, v[ch][e] * inv * widen(wt[ch][e]));
    }
  }
}

// True when the kernel for stacks of float32 partial sums took the call.
template <typename TW, typename TO>
static bool launch_add_rmsnorm_stack(float* resid, const void* delta, const void* weight,
                                     void* out, const int* rows, int R, int H, float eps,
                                     int write_resid, int parts, long long part_stride,
                                     int round_parts, hipStream_t stream) {
  if (H % 4 != 0 || H > 1024 * 4 * 4 || part_stride % 4 != 0) return false;
  if (((uintptr_t)resid | (uintptr_t)delta) % 16) return false;
#define LAUNCH(CH, NT)                                                                        \
  add_rmsnorm_stack_kernel<TW, TO, CH, NT><<<R, NT, 0, stream>>>(                             \
      resid, (const float*)delta, (const TW*)weight, (TO*)out, rows, H, eps, write_resid,     \
      parts, part_stride, round_parts)
  if (H <= 256 * 4) LAUNCH(1, 256);
  else if (H <= 512 * 4) LAUNCH(1, 512);
  else if (H <= 1024 * 4) LAUNCH(1, 1024);
  else if (H <= 1024 * 8) LAUNCH(2, 1024);
  else LAUNCH(4, 1024);
#undef LAUNCH
  return true;
}

template <typename TD, typename TW, typename TO>
static void launch_add_rmsnorm(float* resid, const void* delta, const void* weight, void* out,
                               const int* rows, int R, int H, float eps, int write_resid,
                               int parts, long long part_stride, int round_parts,
                               hipStream_t stream) {
  if (H <= 256 * 4)
    add_rmsnorm_small_kernel<TD, TW, TO, 256, 4><<<R, 256, 0, stream>>>(
        resid, (const TD*)delta, (const TW*)weight, (TO*)out, rows, H, eps, write_resid, parts,
        part_stride, round_parts);
  else if (H <= 256 * 16)
    add_rmsnorm_small_kernel<TD, TW, TO, 256, 16><<<R, 256, 0, stream>>>(
        resid, (const TD*)delta, (const TW*)weight, (TO*)out, rows, H, eps, write_resid, parts,
        part_stride, round_parts);
  else
    add_rmsnorm_kernel<TD, TW, TO, 256><<<R, 256, 0, stream>>>(
        resid, (const TD*)delta, (const TW*)weight, (TO*)out, rows, H, eps, write_resid, parts,
        part_stride, round_parts);
}

RLIS_API int rlis_add_rmsnorm(float* resid, const void* delta, int delta_dtype,
                              const void* weight, int weight_dtype, void* out, int out_dtype,
                              const int* rows, int R, int H, float eps, int write_resid,
                              int parts, long long part_stride, int round_parts,
                              hipStream_t stream) {
  RLIS_REQUIRE(R >= 0 && H > 0, "add_rmsnorm: bad sizes R=%d H=%d", R, H);
  RLIS_REQUIRE(parts >= 1, "add_rmsnorm: parts=%d", parts);
  RLIS_REQUIRE(!(rows && write_resid && delta),
               "add_rmsnorm: writing the residual back needs all rows, not a selection");
  if (R == 0) return 0;
  if ((!delta || delta_dtype == RLIS_BF16) && weight_dtype == RLIS_BF16 && out_dtype == RLIS_BF16 &&
      launch_add_rmsnorm_bf16x8(resid, delta, weight, out, rows, R, H, eps, write_resid, parts,
                                stream)) {
    RLIS_LAUNCH_CHECK("add_rmsnorm");
    return 0;
  }
  if (delta && delta_dtype == RLIS_F32 && parts > 1) {
    bool took = false;
    if (weight_dtype == RLIS_BF16 && out_dtype == RLIS_BF16)
      took = launch_add_rmsnorm_stack<bf16_t, bf16_t>(resid, delta, weight, out, rows, R, H, eps,
                                                      write_resid, parts, part_stride, round_parts,
                                                      stream);
    else if (weight_dtype == RLIS_F32 && out_dtype == RLIS_BF16)
      took = launch_add_rmsnorm_stack<float, bf16_t>(resid, delta, weight, out, rows, R, H, eps,
                                                     write_resid, parts, part_stride, round_parts,
                                                     stream);
    else if (weight_dtype == RLIS_F32 && out_dtype == RLIS_F32)
      took = launch_add_rmsnorm_stack<float, float>(resid, delta, weight, out, rows, R, H, eps,
                                                    write_resid, parts, part_stride, round_parts,
                                                    stream);
    if (took) {
      RLIS_LAUNCH_CHECK("add_rmsnorm");
      return 0;
    }
  }
  const int key = (delta ? delta_dtype : out_dtype) * 4 + weight_dtype * 2 + out_dtype;
#define CASE(k, TD, TW, TO)                                                                  \
  case k:                                                                                    \
    launch_add_rmsnorm<TD, TW, TO>(resid, delta, weight, out, rows, R, H, eps, write_resid,  \
                                   parts, part_stride, round_parts, stream);                 \
    break;
  switch (key) {
    CASE(0, float, float, float)
    CASE(1, float, float, bf16_t)
    CASE(2, float, bf16_t, float)
    CASE(3, float, bf16_t, bf16_t)
    CASE(4, bf16_t, float, float)
    CASE(5, bf16_t, float, bf16_t)
    CASE(6, bf16_t, bf16_t, float)
    CASE(7, bf16_t, bf16_t, bf16_t)
    default:
      RLIS_REQUIRE(false, "add_rmsnorm: unknown dtypes %d %d %d", delta_dtype, weight_dtype,
                   out_dtype);
  }
#undef CASE
  RLIS_LAUNCH_CHECK("add_rmsnorm");
  return 0;
}

// -------------------------------------------------------------------------- SwiGLU
// gu (T, 2I): columns [0, I) are the gate projection, [I, 2I) the up projection.
template <typename TX>
__global__ void swiglu_kernel(TX* __restrict__ out, const TX* __restrict__ gu, int I,
                              long long total) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < total; i += stride) {
    const long long t = i / I;
    const int c = (int)(i - t * I);
    const float g = ld(gu + t * 2 * I + c);
    const float u = ld(gu + t * 2 * I + I + c);
    const float s = g / (1.0f + expf(-g));
    st(out + i, s * u);
  }
}

// bfloat16 rows whose width is a multiple of 8: eight columns per thread, 16-byte accesses.
__global__ void swiglu_bf16x8_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ gu,
                                     int I8 /* I / 8 */, long long total8) {
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < total8; i += stride) {
    const long long t = i / I8;
    const int c = (int)(i - t * I8);
    const uint4 gv = *(const uint4*)(gu + (t * 2 * I8 + c) * 8);
    const uint4 uv = *(const uint4*)(gu + (t * 2 * I8 + I8 + c) * 8);
    const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
    uint32_t ow[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
      const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xffff0000u);
      // silu(g) * u with the hardware's exponential and reciprocal (an ulp each, far inside
      // what the rounding to bfloat16 leaves): the library functions made this kernel spend as
      // long on arithmetic as on its bytes.
      const float e0 = __builtin_amdgcn_exp2f(g0 * -1.4426950408889634f);
      const float e1 = __builtin_amdgcn_exp2f(g1 * -1.4426950408889634f);
      const float r0 = g0 * __builtin_amdgcn_rcpf(1.0f + e0) * u0;
      const float r1 = g1 * __builtin_amdgcn_rcpf(1.0f + e1) * u1;
      ow[j] = (uint32_t)f32_to_bf16(r0) | ((uint32_t)f32_to_bf16(r1) << 16);
    }
    *(uint4*)(out + i * 8) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
  }
}

RLIS_API int rlis_swiglu(void* out, const void* gu, int dtype, int T, int I, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && I > 0, "swiglu: bad sizes T=%d I=%d", T, I);
  const long long total = (long long)T * I;
  if (total == 0) return 0;
  if (dtype == RLIS_BF16 && I % 8 == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)gu % 16) == 0) {
    const long long total8 = total / 8;
    const int blocks8 = (int)(ceil_div_ll(total8, 256) < 16384 ? ceil_div_ll(total8, 256) : 16384);
    swiglu_bf16x8_kernel<<<blocks8, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, I / 8, total8);
    RLIS_LAUNCH_CHECK("swiglu");
    return 0;
  }
  const int blocks = (int)(ceil_div_ll(total, 256) < 8192 ? ceil_div_ll(total, 256) : 8192);
  if (dtype == RLIS_F32)
    swiglu_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)gu, I, total);
  else if (dtype == RLIS_BF16)
    swiglu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, I, total);
  else
    RLIS_REQUIRE(false, "swiglu: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("swiglu");
  return 0;
}

// ------------------------------------------------ rotary encoding + K/V page write
// qkv (T, row_stride): q heads at columns [0, nh*d), k heads at [k_off, k_off + nkv*d), v heads
// at [v_off, v_off + nkv*d).  The first rot_dim dims of every q and k head are rotated
// (rotate-half: dim j pairs with j + rot_dim/2; or, `interleaved`, dim 2j pairs with 2j + 1;
// either way with the j-th angle of the position's row), the rest pass through.  q is rotated in
// place (not at all without rotate_q: the consumer turns it as it loads it).  When write_kv is
// set, rotated k goes to k_pages[page][kv head][offset][d] and v to
// v_pages[page][kv head][d][offset] (v is stored transposed inside a page), with
// page = slot / page_size, offset = slot % page_size; rotated k is not stored back to qkv.
template <typename TX>
__global__ void rope_kv_write_kernel(TX* __restrict__ qkv, long long row_stride, int k_off,
                                     int v_off, int nh, int nkv, int d, int rot_dim,
                                     const float* __restrict__ cos_t,
                                     const float* __restrict__ sin_t,
                                     const int* __restrict__ positions,
                                     const int* __restrict__ slots, TX* __restrict__ k_pages,
                                     TX* __restrict__ v_pages, int page_size, int write_kv,
                                     int interleaved, int rotate_q) {
  const int t = blockIdx.x;
  TX* row = qkv + (long long)t * row_stride;
  const int pos = positions[t];
  const int half = rot_dim / 2;
  const float* c = cos_t + (long long)pos * half;
  const float* s = sin_t + (long long)pos * half;
  // q heads: rotate in place.
  for (int i = threadIdx.x; i < (rotate_q ? nh * half : 0); i += blockDim.x) {
    const int h = i / half, j = i - h * half;
    TX* p = row + h * d;
    const int a = interleaved ? 2 * j : j, b = interleaved ? 2 * j + 1 : j + half;
    const float x1 = ld(p + a), x2 = ld(p + b);
    const float cc = c[j], sn = s[j];
    st(p + a, x1 * cc - x2 * sn);
    st(p + b, x2 * cc + x1 * sn);
  }
  if (!write_kv) return;
  const int slot = slots[t];
  if (slot < 0) return;
  const long long page = slot / page_size;
  const int off = slot - (int)page * page_size;
  // k heads: rotate and store to the page.
  for (int i = threadIdx.x; i < nkv * half; i += blockDim.x) {
    const int h = i / half, j = i - h * half;
    const TX* p = row + k_off + h * d;
    const int a = interleaved ? 2 * j : j, b = interleaved ? 2 * j + 1 : j + half;
    const float x1 = ld(p + a), x2 = ld(p + b);
    const float cc = c[j], sn = s[j];
    TX* dst = k_pages + ((page * nkv + h) * page_size + off) * d;
    st(dst + a, x1 * cc - x2 * sn);
    st(dst + b, x2 * cc + x1 * sn);
  }
  const int tail = d - rot_dim;
  for (int i = threadIdx.x; i < nkv * tail; i += blockDim.x) {
    const int h = i / tail, j = rot_dim + (i - h * tail);
    TX* dst = k_pages + ((page * nkv + h) * page_size + off) * d;
    dst[j] = row[k_off + h * d + j];
  }
  // v heads: store transposed.
  for (int i = threadIdx.x; i < nkv * d; i += blockDim.x) {
    const int h = i / d, j = i - h * d;
    v_pages[((page * nkv + h) * d + j) * page_size + off] = row[v_off + h * d + j];
  }
}

// bfloat16 with every head segment a multiple of 8 wide: 16-byte accesses.  The first
// `qk_blocks` workgroups rotate q in place and k into its page, tok_qk tokens each (heads from
// first_head on: nh when q is left alone); the others take kRopeTokV tokens times kRopeVCols value columns each and turn them through LDS, so
// that lanes which are neighbours in a page's (d, offset) layout store neighbouring offsets
// (tokens with adjacent slots fill whole 32-byte runs, whatever their alignment).
constexpr int kRopeTokV = 16;
constexpr int kRopeVCols = 256;                // v columns per workgroup
constexpr int kRopeVRow = kRopeVCols + 8;      // padded: rows stay 16-byte aligned, banks spread

__device__ __forceinline__ void unpack8(const uint4 u, float (&v)[8]) {
  const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ uint4 pack8(const float (&v)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = (uint32_t)f32_to_bf16(v[2 * i]) | ((uint32_t)f32_to_bf16(v[2 * i + 1]) << 16);
  return make_uint4(w[0], w[1], w[2], w[3]);
}

__global__ __launch_bounds__(256) void rope_kv_write_bf16x8_kernel(
    bf16_t* __restrict__ qkv, long long row_stride, int k_off, int v_off, int T, int nh, int nkv,
    int d, int rot_dim, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ slots,
    bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages, int page_size, int write_kv,
    int qk_blocks, int tok_qk, int first_head) {
  const int tid = threadIdx.x;
  const int half = rot_dim / 2;
  if ((int)blockIdx.x < qk_blocks) {
    const int t0 = blockIdx.x * tok_qk;
    const int hc = half / 8;                             // chunks of 8 pairs per head
    const int heads = nh + (write_kv ? nkv : 0) - first_head;
    const int per_tok = heads * hc;
    for (int i = tid; i < tok_qk * per_tok; i += blockDim.x) {
      const int tt = i / per_tok, r = i - tt * per_tok, t = t0 + tt;
      if (t >= T) break;
      const int h = first_head + r / hc, j = (r - (h - first_head) * hc) * 8;
      const bool is_k = h >= nh;
      const int slot = is_k ? slots[t] : 0;
      if (slot < 0) continue;
      bf16_t* src = qkv + (long long)t * row_stride + (is_k ? k_off + (h - nh) * d : h * d);
      bf16_t* dst = src;
      if (is_k) {
        const long long page = slot / page_size;
        const int off = slot - (int)page * page_size;
        dst = k_pages + ((page * nkv + (h - nh)) * page_size + off) * d;
      }
      const long long cs = (long long)positions[t] * half + j;
      float x1[8], x2[8], c[8], s[8], o1[8], o2[8];
      unpack8(*(const uint4*)(src + j), x1);
      unpack8(*(const uint4*)(src + j + half), x2);
      *(float4*)&c[0] = *(const float4*)(cos_t + cs);
      *(float4*)&c[4] = *(const float4*)(cos_t + cs + 4);
      *(float4*)&s[0] = *(const float4*)(sin_t + cs);
      *(float4*)&s[4] = *(const float4*)(sin_t + cs + 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        o1[e] = x1[e] * c[e] - x2[e] * s[e];
        o2[e] = x2[e] * c[e] + x1[e] * s[e];
      }
      *(uint4*)(dst + j) = pack8(o1);
      *(uint4*)(dst + j + half) = pack8(o2);
    }
    if (write_kv && d > rot_dim) {                       // the dims of k that are not rotated
      const int tc = (d - rot_dim) / 8, per = nkv * tc;
      for (int i = tid; i < tok_qk * per; i += blockDim.x) {
        const int tt = i / per, r = i - tt * per, t = t0 + tt;
        if (t >= T) break;
        const int h = r / tc, j = rot_dim + (r - h * tc) * 8;
        const int slot = slots[t];
        if (slot < 0) continue;
        const long long page = slot / page_size;
        const int off = slot - (int)page * page_size;
        *(uint4*)(k_pages + ((page * nkv + h) * page_size + off) * d + j) =
            *(const uint4*)(qkv + (long long)t * row_stride + k_off + h * d + j);
      }
    }
    return;
  }
  // Values: a tile of kRopeTokV tokens times kRopeVCols columns per workgroup.
  __shared__ __attribute__((aligned(16))) bf16_t v_s[kRopeTokV * kRopeVRow];
  __shared__ long long page_s[kRopeTokV];                // -1: the token is not stored
  __shared__ int off_s[kRopeTokV];
  const int cols = nkv * d;
  const int chunks = (cols + kRopeVCols - 1) / kRopeVCols;
  const int vb = (int)blockIdx.x - qk_blocks;
  const int t0 = (vb / chunks) * kRopeTokV, c0 = (vb % chunks) * kRopeVCols;
  if (tid < kRopeTokV) {
    const int slot = t0 + tid < T ? slots[t0 + tid] : -1;
    const int page = slot < 0 ? -1 : slot / page_size;
    page_s[tid] = page;
    off_s[tid] = slot < 0 ? 0 : slot - page * page_size;
  }
  const int nc = min(kRopeVCols, cols - c0), nc8 = nc / 8;
  for (int i = tid; i < kRopeTokV * nc8; i += blockDim.x) {
    const int tt = i / nc8, c = (i - tt * nc8) * 8;
    if (t0 + tt < T)
      *(uint4*)(v_s + tt * kRopeVRow + c) =
          *(const uint4*)(qkv + (long long)(t0 + tt) * row_stride + v_off + c0 + c);
  }
  __syncthreads();
  for (int i = tid; i < kRopeTokV * nc; i += blockDim.x) {
    const int tt = i % kRopeTokV, c = i / kRopeTokV;
    const long long page = page_s[tt];
    if (page < 0) continue;
    const int col = c0 + c, h = col / d, j = col - h * d;
    v_pages[((page * nkv + h) * d + j) * page_size + off_s[tt]] = v_s[tt * kRopeVRow + c];
  }
}

RLIS_API int rlis_rope_kv_write(void* qkv, int dtype, long long row_stride, int k_off, int v_off,
                                int T, int nh, int nkv, int d, int rot_dim, const float* cos_t,
                                const float* sin_t, const int* positions, const int* slots,
                                void* k_pages, void* v_pages, int page_size, int write_kv,
                                int interleaved, int rotate_q, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && nh > 0 && nkv > 0 && d > 0, "rope_kv_write: bad sizes");
  RLIS_REQUIRE(rot_dim >= 0 && rot_dim <= d && rot_dim % 2 == 0,
               "rope_kv_write: rot_dim %d must be even and at most head_dim %d", rot_dim, d);
  RLIS_REQUIRE(!write_kv || (page_size > 0 && k_pages && v_pages && slots),
               "rope_kv_write: cache write asked for without pages");
  if (T == 0 || (!rotate_q && !write_kv)) return 0;
  const bool by8 = !interleaved && dtype == RLIS_BF16 && d % 8 == 0 && rot_dim % 16 == 0 && row_stride % 8 == 0 &&
                   k_off % 8 == 0 && v_off % 8 == 0 && ((uintptr_t)qkv % 16) == 0 &&
                   ((uintptr_t)cos_t % 16) == 0 && ((uintptr_t)sin_t % 16) == 0 &&
                   (!write_kv || (((uintptr_t)k_pages % 16) == 0 && T <= (1 << 30)));
  if (by8) {
    // about 64 chunks of 8 pairs or more to a workgroup of the first kind
    const int first_head = rotate_q ? 0 : nh;
    const int per_tok = (nh + (write_kv ? nkv : 0) - first_head) * (rot_dim / 16);
    int tok_qk = 2;
    while (tok_qk < 16 && tok_qk * per_tok < 256) tok_qk *= 2;
    const int qk_blocks = (per_tok > 0 || (write_kv && d > rot_dim)) ? ceil_div(T, tok_qk) : 0;
    const int v_blocks = write_kv ? ceil_div(T, kRopeTokV) * ceil_div(nkv * d, kRopeVCols) : 0;
    if (qk_blocks + v_blocks == 0) return 0;             // nothing is rotated, nothing stored
    rope_kv_write_bf16x8_kernel<<<qk_blocks + v_blocks, 256, 0, stream>>>(
        (bf16_t*)qkv, row_stride, k_off, v_off, T, nh, nkv, d, rot_dim, cos_t, sin_t, positions,
        slots, (bf16_t*)k_pages, (bf16_t*)v_pages, page_size, write_kv, qk_blocks, tok_qk,
        first_head);
    RLIS_LAUNCH_CHECK("rope_kv_write");
    return 0;
  }
  if (dtype == RLIS_F32)
    rope_kv_write_kernel<float><<<T, 256, 0, stream>>>(
        (float*)qkv, row_stride, k_off, v_off, nh, nkv, d, rot_dim, cos_t, sin_t, positions,
        slots, (float*)k_pages, (float*)v_pages, page_size, write_kv, interleaved, rotate_q);
  else if (dtype == RLIS_BF16)
    rope_kv_write_kernel<bf16_t><<<T, 256, 0, stream>>>(
        (bf16_t*)qkv, row_stride, k_off, v_off, nh, nkv, d, rot_dim, cos_t, sin_t, positions,
        slots, (bf16_t*)k_pages, (bf16_t*)v_pages, page_size, write_kv, interleaved, rotate_q);
  else
    RLIS_REQUIRE(false, "rope_kv_write: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("rope_kv_write");
  return 0;
}

// ---------------------------------------------------------------------- page copies
// pages (num_layers, num_pages, page_elems): copy page src[i] to dst[i] in every layer.
template <typename TX>
__global__ void copy_pages_kernel(TX* __restrict__ pages, long long layer_stride,
                                  long long page_elems, const int* __restrict__ src,
                                  const int* __restrict__ dst) {
  const int pair = blockIdx.x, layer = blockIdx.y;
  const TX* s = pages + layer * layer_stride + (long long)src[pair] * page_elems;
  TX* d = pages + layer * layer_stride + (long long)dst[pair] * page_elems;
  for (long long i = threadIdx.x; i < page_elems; i += blockDim.x) d[i] = s[i];
}

RLIS_API int rlis_copy_pages(void* pages, int dtype, int num_layers, long long num_pages,
                             long long page_elems, const int* src, const int* dst, int num_pairs,
                             hipStream_t stream) {
  RLIS_REQUIRE(num_layers > 0 && num_pages > 0 && page_elems > 0, "copy_pages: bad sizes");
  if (num_pairs <= 0) return 0;
  dim3 grid(num_pairs, num_layers);
  if (dtype == RLIS_F32)
    copy_pages_kernel<float><<<grid, 256, 0, stream>>>((float*)pages, num_pages * page_elems,
                                                       page_elems, src, dst);
  else if (dtype == RLIS_BF16)
    copy_pages_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)pages, num_pages * page_elems,
                                                        page_elems, src, dst);
  else
    RLIS_REQUIRE(false, "copy_pages: unknown dtype %d", dtype);
  RLIS_LAUNCH_CHECK("copy_pages");
  return 0;
}

// ------------------------------------------------------------- seeded random weights
// The generator of runtime/random_fill.cpp on the device: value i of a tensor is a function of
// (seed, tensor index, i) alone: two splitmix64 hashes of the pair index give two uniforms,
// Box-Muller in double precision turns them into the pair's two normals, rounded once to
// float32 (and, for a bfloat16 destination, once more).  The host's and the device's log, cos
// and sin may differ in the last digit of a double, which the rounding to float32 hides but for
// a value in a few hundred million.
__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

template <typename TO>
__global__ void fill_normal_kernel(TO* __restrict__ out, long long n, uint64_t key, double mean,
                                   double std_dev) {
  const long long pairs = (n + 1) / 2;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long j = (long long)blockIdx.x * blockDim.x + threadIdx.x; j < pairs; j += stride) {
    const uint64_t a = splitmix64(key + 2 * (uint64_t)j), b = splitmix64(key + 2 * (uint64_t)j + 1);
    const double u1 = ((double)(a >> 11) + 0.5) * (1.0 / 9007199254740992.0);
    const double u2 = ((double)(b >> 11) + 0.5) * (1.0 / 9007199254740992.0);
    const double r = sqrt(-2.0 * log(u1));
    const double angle = 6.283185307179586476925286766559 * u2;
    st(out + 2 * j, (float)(mean + std_dev * (r * cos(angle))));
    if (2 * j + 1 < n) st(out + 2 * j + 1, (float)(mean + std_dev * (r * sin(angle))));
  }
}

// out[0 .. n) = mean + std * N(0, 1) keyed by (seed, tensor); out is float32 or bfloat16.
RLIS_API int rlis_fill_normal_device(void* out, int out_dtype, long long n, unsigned long long seed,
                                     unsigned long long tensor, double mean, double std_dev,
                                     hipStream_t stream) {
  RLIS_REQUIRE(n >= 0 && out, "fill_normal: bad arguments");
  if (n == 0) return 0;
  // host side of the same hash
  auto mix = [](uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
  };
  const uint64_t key = mix((uint64_t)seed ^ mix((uint64_t)tensor));
  const long long pairs = (n + 1) / 2;
  const int blocks = (int)(ceil_div_ll(pairs, 256) < 8192 ? ceil_div_ll(pairs, 256) : 8192);
  if (out_dtype == RLIS_F32)
    fill_normal_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, n, key, mean, std_dev);
  else if (out_dtype == RLIS_BF16)
    fill_normal_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, n, key, mean, std_dev);
  else
    RLIS_REQUIRE(false, "fill_normal: unknown dtype %d", out_dtype);
  RLIS_LAUNCH_CHECK("fill_normal");
  return 0;
}
