// Attention over the paged cache, float32 arithmetic on ordinary vector units.
//
// Cache layout per layer: k_pages[page][kv head][offset][d], v_pages[page][kv head][d][offset]
// (values transposed inside a page).  The key of position p of a sequence lives in page
// table[p / page_size] at offset p % page_size (crates/kvcache/src/lib.rs:168-175); K and V
// of the step's own tokens are already there when attention runs (crates/model/src/paged.rs:
// 324-337).
//
// Math as in the reference's attention_block (crates/model/src/attention.rs:204-223) and its
// decode kernel (crates/model/src/paged_attention.metal:56-198): query head h uses KV head
// h / group; score = (q . k) * scale; a query at position p sees keys at positions <= p
// (attention.rs:225-233) and, when a window w is given, > p - w; a position encoding that works
// on the scores gives `slopes` (one float per query head; the reference has none): the score of
// key position u for a query at position p then gets slope * (u - p) added, in float32, before
// the softmax; softmax statistics (running
// maximum m, denominator l, unnormalised accumulator) are float32; partitions of a long
// context are merged with weights e^(m_i - max m) over the non-empty ones (metal:276-304).
//
//  * attn_generic: one wave per (token, query head); any way of cutting the batch.
//  * attn_decode: one query token per sequence; a workgroup serves up to 8 query heads of one
//    KV head, so K and V are read once per group; contexts are split into partitions.
//  * attn_reduce: merges the partitions.
#include "common.h"

#include <math.h>

// ================================================================== generic kernel
template <typename TX, int DPL>
__global__ __launch_bounds__(64) void attn_generic_kernel(
    const TX* __restrict__ q, long long q_stride, TX* __restrict__ out, long long out_stride,
    const TX* __restrict__ k_pages, const TX* __restrict__ v_pages,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ seq_of_token,
    const int* __restrict__ positions, int nh, int nkv, int d, int page_size, float scale,
    int window, const float* __restrict__ slopes) {
  extern __shared__ float smem[];
  float* q_s = smem;                          // d
  float* p_s = smem + d;                      // 64
  long long* vbase_s = (long long*)(p_s + 64);  // 64
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int seq = seq_of_token[t];
  const int pos = positions[t];
  const int kvh = h / (nh / nkv);
  const float slope = slopes ? slopes[h] : 0.f;
  const int* table = block_tables + (long long)seq * max_pages;
  for (int j = lane; j < d; j += 64) q_s[j] = ld(q + (long long)t * q_stride + h * d + j) * scale;
  __syncthreads();
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  float m = -INFINITY, l = 0.f;
  float acc[DPL];
#pragma unroll
  for (int i = 0; i < DPL; ++i) acc[i] = 0.f;
  for (int k0 = lo; k0 <= pos; k0 += 64) {
    const int kpos = k0 + lane;
    const bool valid = kpos <= pos;
    float s = -INFINITY;
    long long vbase = 0;
    if (valid) {
      const long long page = table[kpos / page_size];
      const int off = kpos % page_size;
      const TX* kp = k_pages + ((page * nkv + kvh) * page_size + off) * d;
      float dot = 0.f;
      for (int j = 0; j < d; ++j) dot = fmaf(q_s[j], ld(kp + j), dot);
      s = dot + slope * (float)(kpos - pos);
      vbase = (page * nkv + kvh) * (long long)d * page_size + off;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
    l = l * corr + wave_sum(p);
    p_s[lane] = p;
    vbase_s[lane] = vbase;
    __syncthreads();
    const int n = min(64, pos - k0 + 1);
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const int j = lane + 64 * i;
      if (j < d) {
        float a = acc[i] * corr;
        for (int kk = 0; kk < n; ++kk)
          a = fmaf(p_s[kk], ld(v_pages + vbase_s[kk] + (long long)j * page_size), a);
        acc[i] = a;
      }
    }
    __syncthreads();
    m = m_new;
  }
  const float inv_l = 1.0f / l;
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int j = lane + 64 * i;
    if (j < d) st(out + (long long)t * out_stride + h * d + j, acc[i] * inv_l);
  }
}

RLIS_API int rlis_attn_generic(const void* q, int dtype, long long q_stride, void* out,
                               long long out_stride, const void* k_pages, const void* v_pages,
                               const int* block_tables, int max_pages, const int* seq_of_token,
                               const int* positions, int T, int nh, int nkv, int d, int page_size,
                               float scale, int window, const float* slopes,
                               hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && nh > 0 && nkv > 0 && d > 0 && page_size > 0, "attn_generic: bad sizes");
  RLIS_REQUIRE(nh % nkv == 0, "attn_generic: %d query heads are not a multiple of %d KV heads",
               nh, nkv);
  RLIS_REQUIRE(d <= 512 && d % 2 == 0, "attn_generic: head_dim %d must be even and at most 512", d);
  RLIS_REQUIRE(nh <= 65535, "attn_generic: too many heads");
  if (T == 0) return 0;
  dim3 grid(T, nh);
  const size_t smem = (size_t)d * 4 + 64 * 4 + 64 * 8 + 8;
  const int dpl = ceil_div(d, 64);
#define LAUNCH(TX, DPL)                                                                        \
  attn_generic_kernel<TX, DPL><<<grid, 64, smem, stream>>>(                                    \
      (const TX*)q, q_stride, (TX*)out, out_stride, (const TX*)k_pages, (const TX*)v_pages,    \
      block_tables, max_pages, seq_of_token, positions, nh, nkv, d, page_size, scale, window,  \
      slopes)
#define BY_DPL(TX)                         \
  do {                                     \
    if (dpl <= 1) LAUNCH(TX, 1);           \
    else if (dpl <= 2) LAUNCH(TX, 2);      \
    else if (dpl <= 4) LAUNCH(TX, 4);      \
    else LAUNCH(TX, 8);                    \
  } while (0)
  if (dtype == RLIS_F32) BY_DPL(float);
  else if (dtype == RLIS_BF16) BY_DPL(bf16_t);
  else RLIS_REQUIRE(false, "attn_generic: unknown dtype %d", dtype);
#undef BY_DPL
#undef LAUNCH
  RLIS_LAUNCH_CHECK("attn_generic");
  return 0;
}

// =================================================================== decode kernel
template <typename TX> struct Vec16;
template <> struct Vec16<float> {
  static constexpr int N = 4;
  __device__ static void load(const float* p, float* o) {
    const float4 v = *(const float4*)p;
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
};
template <> struct Vec16<bf16_t> {
  static constexpr int N = 8;
  __device__ static void load(const bf16_t* p, float* o) {
    const uint4 v = *(const uint4*)p;
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __uint_as_float(w[i] << 16);
      o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

// Grid (kv head * head chunks, sequence, split); 256 threads.  Head chunk c serves query
// heads kvh * g + c * G + [0, G) (those beyond the group are computed on a clamped head and
// dropped).  Partition `split` of a sequence with n visible keys covers
// [lo + split * part, lo + (split + 1) * part) with part = decode_part_len(n, part_keys,
// max_parts): a function of the sequence's own length.  `splits` is the grid's depth and the
// stride of the partial results, at least the live partitions of the longest sequence;
// partitions beyond a sequence's own store an empty result (l = 0), which the merge skips.
// Output per (sequence, head, split): m, l and the unnormalised accumulator (d floats); with
// splits == 1 the normalised result goes straight to `out`.
template <typename TX, int G, int DPL>
__global__ __launch_bounds__(256) void attn_decode_kernel(
    const TX* __restrict__ q, long long q_stride, TX* __restrict__ out, long long out_stride,
    float* __restrict__ part_ml, float* __restrict__ part_acc, const TX* __restrict__ k_pages,
    const TX* __restrict__ v_pages, const int* __restrict__ block_tables, int max_pages,
    const int* __restrict__ ctx_lens, const int* __restrict__ token_rows, int nh, int nkv, int d,
    int page_size, float scale, int window, int splits, int chunks_per_kv, int part_keys,
    int max_parts, const float* __restrict__ slopes) {
  extern __shared__ float smem[];
  float* q_s = smem;                     // G * d
  float* p_s = q_s + G * d;              // 4 waves * G * 64
  float* ml_s = p_s + 4 * G * 64;        // 4 waves * G * 2
  float* acc_s = ml_s + 4 * G * 2;       // 4 waves * G * d
  long long* vbase_s = (long long*)(acc_s + 4 * G * d);  // 4 waves * 64
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int kvh = blockIdx.x / chunks_per_kv, chunk = blockIdx.x % chunks_per_kv;
  const int seq = blockIdx.y, split = blockIdx.z;
  const int g = nh / nkv;
  const int h0 = kvh * g + chunk * G;
  const int gn = min(G, g - chunk * G);
  const int ctx = ctx_lens[seq];
  const int row = token_rows ? token_rows[seq] : seq;
  const int* table = block_tables + (long long)seq * max_pages;
  const int lo = (window > 0 && ctx - window > 0) ? ctx - window : 0;
  const int nkeys = ctx - lo;
  const int part = decode_part_len(nkeys, part_keys, max_parts);
  const int kbeg = lo + split * part;
  const int kend = min(ctx, kbeg + part);

  for (int i = tid; i < G * d; i += 256) {
    const int hh = min(i / d, gn - 1), j = i % d;
    q_s[i] = ld(q + (long long)row * q_stride + (h0 + hh) * d + j) * scale;
  }
  __syncthreads();

  float m[G], l[G], acc[G][DPL];
#pragma unroll
  for (int hh = 0; hh < G; ++hh) {
    m[hh] = -INFINITY;
    l[hh] = 0.f;
#pragma unroll
    for (int i = 0; i < DPL; ++i) acc[hh][i] = 0.f;
  }
  float slope[G];
#pragma unroll
  for (int hh = 0; hh < G; ++hh) slope[hh] = slopes ? slopes[h0 + min(hh, gn - 1)] : 0.f;
  float* my_p = p_s + wave * G * 64;
  long long* my_vbase = vbase_s + wave * 64;
  constexpr int VN = Vec16<TX>::N;
  // Values of VN consecutive keys are contiguous inside a page when the partition starts on
  // a multiple of VN and the page size is one.
  const bool vec_ok = (kbeg % VN == 0) && (page_size % VN == 0);

  // Every wave runs the same number of rounds so that the block-wide barriers match.
  const int rounds = kend > kbeg ? (kend - kbeg + 255) / 256 : 0;
  for (int it = 0; it < rounds; ++it) {
    const int k0 = kbeg + it * 256 + wave * 64;
    const int kpos = k0 + lane;
    const bool valid = kpos < kend;
    float s[G];
#pragma unroll
    for (int hh = 0; hh < G; ++hh) s[hh] = 0.f;
    long long vbase = 0;
    if (valid) {
      const long long page = table[kpos / page_size];
      const int off = kpos % page_size;
      const TX* kp = k_pages + ((page * nkv + kvh) * page_size + off) * d;
      vbase = (page * nkv + kvh) * (long long)d * page_size + off;
      for (int j = 0; j < d; j += VN) {
        float kv[VN];
        Vec16<TX>::load(kp + j, kv);
#pragma unroll
        for (int hh = 0; hh < G; ++hh) {
          float a = s[hh];
#pragma unroll
          for (int e = 0; e < VN; ++e) a = fmaf(q_s[hh * d + j + e], kv[e], a);
          s[hh] = a;
        }
      }
    }
    float corr[G];
#pragma unroll
    for (int hh = 0; hh < G; ++hh) {
      const float sv = valid ? s[hh] + slope[hh] * (float)(kpos - (ctx - 1)) : -INFINITY;
      const float m_new = fmaxf(m[hh], wave_max(sv));
      const float p = valid ? expf(sv - m_new) : 0.f;
      corr[hh] = (m[hh] == -INFINITY) ? 0.f : expf(m[hh] - m_new);
      l[hh] = l[hh] * corr[hh] + wave_sum(p);
      m[hh] = m_new;
      my_p[hh * 64 + lane] = p;
    }
    my_vbase[lane] = vbase;
    __syncthreads();
    const int n = max(0, min(64, kend - k0));
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const int j = lane + 64 * i;
      float a[G];
#pragma unroll
      for (int hh = 0; hh < G; ++hh) a[hh] = acc[hh][i] * corr[hh];
      if (j < d) {
        int kk = 0;
        if (vec_ok) {
          for (; kk + VN <= n; kk += VN) {
            float v[VN];
            Vec16<TX>::load(v_pages + my_vbase[kk] + (long long)j * page_size, v);
#pragma unroll
            for (int e = 0; e < VN; ++e)
#pragma unroll
              for (int hh = 0; hh < G; ++hh) a[hh] = fmaf(my_p[hh * 64 + kk + e], v[e], a[hh]);
          }
        }
        for (; kk < n; ++kk) {
          const float v = ld(v_pages + my_vbase[kk] + (long long)j * page_size);
#pragma unroll
          for (int hh = 0; hh < G; ++hh) a[hh] = fmaf(my_p[hh * 64 + kk], v, a[hh]);
        }
      }
#pragma unroll
      for (int hh = 0; hh < G; ++hh) acc[hh][i] = a[hh];
    }
    __syncthreads();
  }

  // Merge the four waves in order.
#pragma unroll
  for (int hh = 0; hh < G; ++hh) {
    if (lane == 0) {
      ml_s[(wave * G + hh) * 2] = m[hh];
      ml_s[(wave * G + hh) * 2 + 1] = l[hh];
    }
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const int j = lane + 64 * i;
      if (j < d) acc_s[(wave * G + hh) * d + j] = acc[hh][i];
    }
  }
  __syncthreads();
  for (int i = tid; i < gn * d; i += 256) {
    const int hh = i / d, j = i % d;
    float big = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) big = fmaxf(big, ml_s[(w * G + hh) * 2]);
    float lsum = 0.f, a = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = ml_s[(w * G + hh) * 2];
      if (mw == -INFINITY) continue;
      const float e = expf(mw - big);
      lsum += ml_s[(w * G + hh) * 2 + 1] * e;
      a += acc_s[(w * G + hh) * d + j] * e;
    }
    const int h = h0 + hh;
    if (splits == 1) {
      st(out + (long long)row * out_stride + h * d + j, a / lsum);
    } else {
      const long long idx = ((long long)seq * nh + h) * splits + split;
      part_acc[idx * d + j] = a;
      if (j == 0) {
        part_ml[idx * 2] = big;
        part_ml[idx * 2 + 1] = lsum;
      }
    }
  }
}

// Grid (query head, row); merges the partitions of one head of one output row.  The row's
// sequence is seq_of_row[row0 + row] (the row itself without that table) and the number of its
// live partitions seq_parts[sequence] (`splits`, the stride of the partial results, without
// that table); a row with one partition or none was stored by its kernel already and is left
// alone.  A thread owns output dims
// j, j + blockDim, ...; the first kReduceAhead partitions' sums for its first dim are loaded
// together with the maxima, before the weights exp(m_s - max m) are known, so that the whole
// merge waits for memory once.  The weights go through LDS (`splits` floats); sums run over s
// in order.
constexpr int kReduceAhead = 16;

template <typename TX>
__global__ void attn_reduce_kernel(TX* __restrict__ out, long long out_stride,
                                   const float* __restrict__ part_ml,
                                   const float* __restrict__ part_acc,
                                   const int* __restrict__ token_rows, int nh, int d, int stride,
                                   const int* __restrict__ seq_of_row,
                                   const int* __restrict__ seq_parts, int row0) {
  extern __shared__ float reduce_w[];            // stride weights, then 8 floats of scratch
  float* scratch = reduce_w + stride;
  const int h = blockIdx.x, seq = blockIdx.y;
  const int row = token_rows ? token_rows[seq] : seq + row0;
  int splits = stride;
  if (seq_parts) {
    splits = min(stride, seq_parts[seq_of_row ? seq_of_row[row] : row]);
    if (splits <= 1) return;
  }
  const long long base = ((long long)seq * nh + h) * stride;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, nwaves = blockDim.x / kWave;
  const int j0 = (int)threadIdx.x < d ? (int)threadIdx.x : 0;
  const float* acc0 = part_acc + base * d + j0;
  float ahead[kReduceAhead];
#pragma unroll
  for (int s = 0; s < kReduceAhead; ++s) ahead[s] = acc0[(long long)min(s, splits - 1) * d];
  float big = -INFINITY;
  for (int s = threadIdx.x; s < splits; s += blockDim.x)
    if (part_ml[(base + s) * 2 + 1] > 0.f) big = fmaxf(big, part_ml[(base + s) * 2]);
  big = wave_max(big);
  if (lane == 0) scratch[wave] = big;
  __syncthreads();
  for (int w = 0; w < nwaves; ++w) big = fmaxf(big, scratch[w]);
  for (int s = threadIdx.x; s < splits; s += blockDim.x) {
    const float ls = part_ml[(base + s) * 2 + 1];
    reduce_w[s] = ls > 0.f ? expf(part_ml[(base + s) * 2] - big) : 0.f;
  }
  __syncthreads();
  float lsum = 0.f;
  for (int s = 0; s < splits; ++s) {
    const float e = reduce_w[s];
    if (e > 0.f) lsum += part_ml[(base + s) * 2 + 1] * e;
  }
  for (int j = threadIdx.x; j < d; j += blockDim.x) {
    float a = 0.f;
    const float* acc = part_acc + base * d + j;
    int s = 0;
    if (j == j0) {
#pragma unroll
      for (; s < kReduceAhead; ++s) {
        if (s >= splits) break;
        const float e = reduce_w[s];
        if (e > 0.f) a += ahead[s] * e;
      }
    }
#pragma unroll 8
    for (; s < splits; ++s) {
      const float e = reduce_w[s];
      const float v = acc[(long long)s * d];
      if (e > 0.f) a += v * e;
    }
    st(out + (long long)row * out_stride + h * d + j, a / lsum);
  }
}

// Launches the merge of `splits` partitions for S sequences of bfloat16 output (used by the
// matrix-core decode kernel, which lives in another unit).
int rlis_launch_attn_reduce_bf16(void* out, long long out_stride, const float* part_ml,
                                 const float* part_acc, int S, int nh, int d, int splits,
                                 hipStream_t stream) {
  dim3 grid(nh, S);
  const int threads = d <= 64 ? 64 : (d <= 128 ? 128 : 256);
  attn_reduce_kernel<bf16_t><<<grid, threads, (splits + 8) * sizeof(float), stream>>>(
      (bf16_t*)out, out_stride, part_ml, part_acc, nullptr, nh, d, splits, nullptr, nullptr, 0);
  RLIS_LAUNCH_CHECK("attn_reduce");
  return 0;
}

// The same merge for the key runs of a prefill step, where the rows are many (every new token
// of a portion, times the heads) and the runs few: one wave per (row, head), four of them to a
// workgroup, no LDS and no barrier.  Every lane reads the runs' maxima and denominators for
// itself (the same addresses across the wave) and owns dims lane, lane + 64, ...; the first
// kRowRuns runs are loaded at once.  Same sums in the same order as attn_reduce_kernel.
constexpr int kRowRuns = 8;

__global__ __launch_bounds__(256) void attn_reduce_rows_kernel(
    bf16_t* __restrict__ out, long long out_stride, const float* __restrict__ part_ml,
    const float* __restrict__ part_acc, int nh, int d, int stride,
    const int* __restrict__ seq_of_row, const int* __restrict__ seq_parts, int row0,
    long long pairs) {
  const long long pair = (long long)blockIdx.x * 4 + threadIdx.x / kWave;
  if (pair >= pairs) return;
  const int lane = threadIdx.x % kWave;
  const int r = (int)(pair / nh), h = (int)(pair % nh);
  const int row = row0 + r;
  const int splits = min(stride, seq_parts[seq_of_row[row]]);
  if (splits <= 1) return;
  const long long base = (pair)*stride;
  float mv[kRowRuns], lv[kRowRuns];
#pragma unroll
  for (int s = 0; s < kRowRuns; ++s) {
    const long long idx = base + min(s, splits - 1);
    mv[s] = part_ml[idx * 2];
    lv[s] = s < splits ? part_ml[idx * 2 + 1] : 0.f;
  }
  float big = -INFINITY;
#pragma unroll
  for (int s = 0; s < kRowRuns; ++s)
    if (lv[s] > 0.f) big = fmaxf(big, mv[s]);
  for (int s = kRowRuns; s < splits; ++s)
    if (part_ml[(base + s) * 2 + 1] > 0.f) big = fmaxf(big, part_ml[(base + s) * 2]);
  float ev[kRowRuns];
  float lsum = 0.f;
#pragma unroll
  for (int s = 0; s < kRowRuns; ++s) {
    ev[s] = lv[s] > 0.f ? expf(mv[s] - big) : 0.f;
    if (ev[s] > 0.f) lsum += lv[s] * ev[s];
  }
  for (int s = kRowRuns; s < splits; ++s) {
    const float l = part_ml[(base + s) * 2 + 1];
    const float e = l > 0.f ? expf(part_ml[(base + s) * 2] - big) : 0.f;
    if (e > 0.f) lsum += l * e;
  }
  for (int j = lane; j < d; j += kWave) {
    const float* acc = part_acc + base * d + j;
    float av[kRowRuns];
#pragma unroll
    for (int s = 0; s < kRowRuns; ++s) av[s] = acc[(long long)min(s, splits - 1) * d];
    float a = 0.f;
#pragma unroll
    for (int s = 0; s < kRowRuns; ++s)
      if (ev[s] > 0.f) a += av[s] * ev[s];
    for (int s = kRowRuns; s < splits; ++s) {
      const float l = part_ml[(base + s) * 2 + 1];
      const float e = l > 0.f ? expf(part_ml[(base + s) * 2] - big) : 0.f;
      if (e > 0.f) a += acc[(long long)s * d] * e;
    }
    out[(long long)row * out_stride + h * d + j] = f32_to_bf16(a / lsum);
  }
}

// Merges the key runs of the matrix-core prefill kernel: `rows` output rows from row0 on, whose
// partial results lie at part_ml (rows, nh, stride, 2) and part_acc (rows, nh, stride, d);
// row r belongs to sequence seq_of_token[row0 + r], which has seq_runs[sequence] runs (rows
// of sequences with a single run are already stored and stay untouched).
RLIS_API int rlis_attn_reduce_rows(void* out, long long out_stride, const float* part_ml,
                                   const float* part_acc, const int* seq_of_token,
                                   const int* seq_runs, int row0, int rows, int nh, int d,
                                   int stride, hipStream_t stream) {
  RLIS_REQUIRE(rows >= 0 && row0 >= 0 && nh > 0 && d > 0 && stride >= 1 && stride <= 64,
               "attn_reduce_rows: bad sizes");
  RLIS_REQUIRE(part_ml && part_acc && seq_of_token && seq_runs,
               "attn_reduce_rows: partial results and the run counts are needed");
  RLIS_REQUIRE(rows <= 65535 * 32, "attn_reduce_rows: %d rows are too many", rows);
  const long long pairs = (long long)rows * nh;
  RLIS_REQUIRE((pairs + 3) / 4 <= 0x7fffffffLL, "attn_reduce_rows: %d rows are too many", rows);
  if (pairs > 0)
    attn_reduce_rows_kernel<<<(unsigned)((pairs + 3) / 4), 256, 0, stream>>>(
        (bf16_t*)out, out_stride, part_ml, part_acc, nh, d, stride, seq_of_token, seq_runs, row0,
        pairs);
  RLIS_LAUNCH_CHECK("attn_reduce_rows");
  return 0;
}

template <typename TX, int G>
static int launch_decode(const void* q, long long q_stride, void* out, long long out_stride,
                         float* part_ml, float* part_acc, const void* k_pages,
                         const void* v_pages, const int* block_tables, int max_pages,
                         const int* ctx_lens, const int* token_rows, int S, int nh, int nkv, int d,
                         int page_size, float scale, int window, int splits, int part_keys,
                         int max_parts, const float* slopes, hipStream_t stream) {
  const int g = nh / nkv;
  const int chunks = ceil_div(g, G);
  dim3 grid(nkv * chunks, S, splits);
  const size_t smem =
      ((size_t)G * d + 4 * G * 64 + 4 * G * 2 + 4 * (size_t)G * d) * sizeof(float) + 4 * 64 * 8;
  RLIS_REQUIRE(smem <= 64 * 1024, "attn_decode: head_dim %d needs %zu bytes of LDS", d, smem);
  const int dpl = ceil_div(d, 64);
#define LAUNCH(DPL)                                                                            \
  attn_decode_kernel<TX, G, DPL><<<grid, 256, smem, stream>>>(                                 \
      (const TX*)q, q_stride, (TX*)out, out_stride, part_ml, part_acc, (const TX*)k_pages,     \
      (const TX*)v_pages, block_tables, max_pages, ctx_lens, token_rows, nh, nkv, d, page_size, \
      scale, window, splits, chunks, part_keys, max_parts, slopes)
  if (dpl <= 1) LAUNCH(1);
  else if (dpl <= 2) LAUNCH(2);
  else LAUNCH(4);
#undef LAUNCH
  return 0;
}

// q rows are token_rows[seq] (or seq when null) of a (T, q_stride) matrix, out likewise.
// A sequence's visible keys are cut into partitions of decode_part_len(keys, part_keys,
// max_parts); `splits` must be at least the live partitions of the longest context (at most
// max_parts).  part_ml (S, nh, splits, 2) and part_acc (S, nh, splits, d) float32 are needed
// when splits > 1.
RLIS_API int rlis_attn_decode(const void* q, int dtype, long long q_stride, void* out,
                              long long out_stride, float* part_ml, float* part_acc,
                              const void* k_pages, const void* v_pages, const int* block_tables,
                              int max_pages, const int* ctx_lens, const int* token_rows, int S,
                              int nh, int nkv, int d, int page_size, float scale, int window,
                              int splits, int part_keys, int max_parts, const float* slopes,
                              hipStream_t stream) {
  RLIS_REQUIRE(S >= 0 && nh > 0 && nkv > 0 && d > 0 && page_size > 0, "attn_decode: bad sizes");
  RLIS_REQUIRE(part_keys >= 64 && part_keys % 64 == 0 && max_parts >= 1 && splits <= max_parts,
               "attn_decode: partitions of %d keys (a multiple of 64), %d deep of at most %d",
               part_keys, splits, max_parts);
  RLIS_REQUIRE(nh % nkv == 0, "attn_decode: %d query heads are not a multiple of %d KV heads",
               nh, nkv);
  RLIS_REQUIRE(d <= 256, "attn_decode: head_dim %d is above the limit of 256", d);
  RLIS_REQUIRE(d % 8 == 0, "attn_decode: head_dim %d must be a multiple of 8", d);
  RLIS_REQUIRE(splits >= 1 && splits <= 8192 && S <= 65535, "attn_decode: bad grid");
  RLIS_REQUIRE(splits == 1 || (part_ml && part_acc), "attn_decode: partitions need a workspace");
  if (S == 0) return 0;
  const int g = nh / nkv;
  int rc = 0;
#define BY_G(TX)                                                                                 \
  do {                                                                                           \
    if (g == 1)                                                                                  \
      rc = launch_decode<TX, 1>(q, q_stride, out, out_stride, part_ml, part_acc, k_pages,        \
                                v_pages, block_tables, max_pages, ctx_lens, token_rows, S, nh,   \
                                nkv, d, page_size, scale, window, splits, part_keys, max_parts,       \
                                slopes, stream);               \
    else if (g == 2)                                                                             \
      rc = launch_decode<TX, 2>(q, q_stride, out, out_stride, part_ml, part_acc, k_pages,        \
                                v_pages, block_tables, max_pages, ctx_lens, token_rows, S, nh,   \
                                nkv, d, page_size, scale, window, splits, part_keys, max_parts,       \
                                slopes, stream);               \
    else if (g <= 4)                                                                             \
      rc = launch_decode<TX, 4>(q, q_stride, out, out_stride, part_ml, part_acc, k_pages,        \
                                v_pages, block_tables, max_pages, ctx_lens, token_rows, S, nh,   \
                                nkv, d, page_size, scale, window, splits, part_keys, max_parts,       \
                                slopes, stream);               \
    else                                                                                         \
      rc = launch_decode<TX, 8>(q, q_stride, out, out_stride, part_ml, part_acc, k_pages,        \
                                v_pages, block_tables, max_pages, ctx_lens, token_rows, S, nh,   \
                                nkv, d, page_size, scale, window, splits, part_keys, max_parts,       \
                                slopes, stream);               \
  } while (0)
  if (dtype == RLIS_F32) BY_G(float);
  else if (dtype == RLIS_BF16) BY_G(bf16_t);
  else RLIS_REQUIRE(false, "attn_decode: unknown dtype %d", dtype);
#undef BY_G
  if (rc) return rc;
  RLIS_LAUNCH_CHECK("attn_decode");
  if (splits > 1) {
    dim3 grid(nh, S);
    const int threads = d <= 64 ? 64 : (d <= 128 ? 128 : 256);
    if (dtype == RLIS_F32)
      attn_reduce_kernel<float><<<grid, threads, (splits + 8) * sizeof(float), stream>>>(
          (float*)out, out_stride, part_ml, part_acc, token_rows, nh, d, splits, nullptr, nullptr,
          0);
    else
      attn_reduce_kernel<bf16_t><<<grid, threads, (splits + 8) * sizeof(float), stream>>>(
          (bf16_t*)out, out_stride, part_ml, part_acc, token_rows, nh, d, splits, nullptr, nullptr,
          0);
    RLIS_LAUNCH_CHECK("attn_reduce");
  }
  return 0;
}
