// The streaming product for 17 to 32 rows of x: y (T, N) = x W^T at the speed of the weight
// stream, with the same forms as the kernel for up to 16 rows (gemm.hip): plain, gated (the
// SwiGLU before the store), scaled (rows that come normed but for a scale, taken from partial
// sums of squares) and joining (the product adds itself to the residual and leaves the rows
// times the next norm's weight and their sums of squares).
//
// The cut is the same: tiles of 16, 12 or 8 weight rows, a wave per k item of 256, persistent
// workgroups that walk over tiles with their rows of x in registers, weights loaded row by row
// (512 contiguous bytes per half wave) one tile ahead and turned into operand layout through an
// LDS tile private to the wave.  What differs is that a wave holds TG = 2 groups of 16 tokens:
// TG accumulators and 32 TG registers of x, which every weight fragment read from LDS then
// serves.  That fits up to 12 waves (K = 3072); K is a whole number of items, and one slice.
// Rows of x past T take row T - 1 (their results are not stored), so nothing is zeroed after a
// load.  (The kernel is written for any TG; four groups are not offered, see launch_groups.)
#include "gemm_stream.h"

namespace {

typedef const __attribute__((address_space(1))) bf16_t* GlobalBf16;
typedef uint32_t Bits4 __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(1))) Bits4* GlobalU4;

template <typename TC, bool GATED, int TR, int MODE, int TG, int AHEAD>
__global__ __launch_bounds__(AHEAD == 2 ? 512 : (TG == 2 ? 768 : 512)) void gemm_bf16_stream_wide_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, TC* __restrict__ Y,
    const StreamShape sh, const StreamNorm nm) {
  extern __shared__ __attribute__((aligned(16))) unsigned char wide_smem[];
  constexpr bool SCALED = MODE == kStreamScaled, JOIN = MODE == kStreamJoin;
  static_assert(MODE != kStreamNorm, "the norm's prologue over whole rows is for 16 rows at most");
  static_assert(!(JOIN && GATED), "a product that joins the residual has no gate");
  constexpr int kTileBytes = TR * kStreamItem * 2;
  constexpr int kRed = TG * 256;                           // floats a wave hands over per tile
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64, nwaves = blockDim.x / 64;
  unsigned char* tile_s = wide_smem + wave * kTileBytes;
  float* red = (float*)(wide_smem + nwaves * kTileBytes);  // [2][nwaves][TG][16 tokens][16 rows]
  float* inv_s = red + 2 * nwaves * kRed;                  // [TG * 16]: the rows' scales
  const int half = lane / 32, l32 = lane % 32;             // loading: row parity, 16-byte chunk
  const int oi = lane % 16, og = lane / 16;                // operand: row (or token), k group
  const int T = sh.T, N = sh.N;
  const int nitems = sh.K / kStreamItem;
  const bool has_item = wave < nitems;                     // a wave without one adds nothing
  const int kb = (has_item ? wave : 0) * kStreamItem;
  // The order of the first loads matters (loads are served in order, and the weights must
  // not leave behind 32 TG loads of x): the two pointers pass through an empty statement, after
  // which the compiler knows nothing about what they point to and keeps their loads on their
  // side of the memory barrier below.
  GlobalBf16 w_base = (GlobalBf16)W;
  GlobalBf16 x_base = (GlobalBf16)X;
  asm volatile("" : "+s"(w_base), "+s"(x_base));
  GlobalBf16 w_lane = w_base + kb + l32 * 8;

  // Tile row r = 2 p + half of tile `tile` is weight row tile * rows + r; gated, the first
  // half of a tile's rows are the gate rows of consecutive columns and the second half their
  // up rows, N further down.  A row past the end, and every row of a tile past the last one,
  // reads row 0 instead and is not stored: no load stands under a condition, so that the
  // compiler can count the loads in flight and wait for the oldest tile alone.
  constexpr int cols_per_tile = GATED ? TR / 2 : TR;
#define RLIS_WIDE_LOAD_TILE(a, tile_)                                                           \
  {                                                                                             \
    const int tl_ = (tile_);                                                                    \
    const int col0 = tl_ < sh.num_tiles ? tl_ * cols_per_tile + half : N;                       \
    GlobalBf16 w_tile = w_lane + (long long)col0 * sh.ldw;                                      \
    _Pragma("unroll") for (int p = 0; p < TR / 2; ++p) {                                        \
      const int c = GATED ? (2 * p) % cols_per_tile : 2 * p;   /* column within the tile */     \
      const long long up = (GATED && 2 * p >= cols_per_tile) ? (long long)N * sh.ldw : 0;       \
      GlobalBf16 ptr = col0 + c < N ? w_tile + (long long)c * sh.ldw + up : w_lane;             \
      const Bits4 v_ = *(GlobalU4)ptr;                                                          \
      a[p].x = v_.x;            /* member by member: a struct copy would go through scratch */  \
      a[p].y = v_.y;                                                                            \
      a[p].z = v_.z;                                                                            \
      a[p].w = v_.w;                                                                            \
    }                                                                                           \
  }

  // One tile ahead of the arithmetic, or two (two sets of registers taking turns) where the
  // registers allow: with one workgroup per compute unit it takes both to keep as many bytes
  // on their way as two workgroups of the kernel for up to 16 rows do.
  uint4 a0[TR / 2], a1[AHEAD == 2 ? TR / 2 : 1];
  int tile = blockIdx.x;
  RLIS_WIDE_LOAD_TILE(a0, tile);         // the first tile is on its way during the prologue
  asm volatile("" ::: "memory");

  // The rows of x in operand layout: token 16 g + oi, k = kb + (4 j + og) * 8 .. + 8 for step
  // j; the eight loads of a group share one address.
  Frag8 b[TG][8];
#pragma unroll
  for (int g = 0; g < TG; ++g) {
    GlobalBf16 xb = x_base + (long long)min(16 * g + oi, T - 1) * sh.ldx + kb + og * 8;
#pragma unroll
    for (int j = 0; j < 8; ++j) b[g][j].v = __builtin_bit_cast(bf16x8, *(GlobalU4)(xb + j * 32));
  }
  // The second tile follows the rows of x: the first products wait for the first tile and x,
  // not for the second tile as well.
  if constexpr (AHEAD == 2) {
    asm volatile("" ::: "memory");
    RLIS_WIDE_LOAD_TILE(a1, tile + (int)gridDim.x);
  }

  // SCALED: the rows' scales come as partial sums of squares, scale_count a token.  A wave
  // takes the tokens wave, wave + nwaves, ... (at most kScaleTokens of them: a workgroup has
  // four waves or more, nine or more with one tile ahead), a lane the parts lane, lane + 64,
  // ...  They are asked for here, all at once and without a condition, and added up only when
  // the first tile is stored; the order of a sum depends on scale_count alone (at most 64
  // kScaleParts: the launch sees to that).
  constexpr int kScaleTokens = SCALED ? (AHEAD == 1 ? 2 : 4) * TG : 1, kScaleParts = SCALED ? 4 : 1;
  float scale_ahead[kScaleTokens][kScaleParts];
  if constexpr (SCALED) {
#pragma unroll
    for (int i = 0; i < kScaleTokens; ++i) {
      const int tok = min(wave + i * nwaves, T - 1);
#pragma unroll
      for (int q = 0; q < kScaleParts; ++q)
        scale_ahead[i][q] = nm.scale_parts[(long long)tok * nm.ss_stride +
                                           min(lane + 64 * q, nm.scale_count - 1)];
    }
  }

  int par = 0;
  bool scale_due = SCALED;
  auto one_tile = [&](uint4 (&A_)[TR / 2]) __attribute__((always_inline)) {
    f32x4 acc[TG];
#pragma unroll
    for (int g = 0; g < TG; ++g) acc[g] = (f32x4){0.f, 0.f, 0.f, 0.f};
    if (has_item) {
#pragma unroll
      for (int p = 0; p < TR / 2; ++p) {
        const int r = 2 * p + half;
        *(uint4*)(tile_s + r * (kStreamItem * 2) + ((l32 ^ r) * 16)) = A_[p];
      }
    }
    RLIS_WIDE_LOAD_TILE(A_, tile + AHEAD * (int)gridDim.x);   /* on its way during the arithmetic */
    if (has_item) {
      wave_lds_fence();
#pragma unroll
      for (int j0 = 0; j0 < 8; j0 += 4) {
        // Four reads from LDS are asked for before the first of their products (two or three
        // waves share a SIMD: nobody else fills the time a read takes); the statement, which
        // every read feeds and every product depends on, keeps the compiler from pairing each
        // read with its products again.
        Bits4 af[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          // tile rows beyond TR repeat the first ones: their products are not stored
          af[j] = *(const Bits4*)(tile_s + (oi % TR) * (kStreamItem * 2) +
                                  (((4 * (j0 + j) + og) ^ (oi % TR)) * 16));
        }
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[0]), "+v"(af[1]), "+v"(af[2]), "+v"(af[3]));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
          for (int g = 0; g < TG; ++g)
            acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[j]),
                                                             b[g][j0 + j].v, acc[g], 0, 0, 0);
        }
      }
      wave_lds_fence();
    }
    // acc[g]: token 16 g + oi, tile rows og * 4 + r.  red[par][wave][g][token][row]; the buffer
    // of the tile before is still being read by slower waves, the one before that is free
    // again after this tile's barrier.
    float* red_p = red + par * nwaves * kRed;
#pragma unroll
    for (int g = 0; g < TG; ++g)
      *(float4*)(red_p + wave * kRed + g * 256 + oi * 16 + og * 4) =
          make_float4(acc[g][0], acc[g][1], acc[g][2], acc[g][3]);
    if (SCALED && scale_due) {
      // The rows' scales, once per workgroup: a wave per token in turn adds the token's partial
      // sums of squares (lane l takes parts l, l + 64, ...; the order depends on their number
      // alone).
#pragma unroll
      for (int i = 0; i < kScaleTokens; ++i) {
        const int tok = wave + i * nwaves;
        float tot = 0.f;
#pragma unroll
        for (int q = 0; q < kScaleParts; ++q)
          tot += lane + 64 * q < nm.scale_count ? scale_ahead[i][q] : 0.f;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) tot += __shfl_xor(tot, o, kWave);
        if (lane == 0 && tok < 16 * TG) inv_s[tok] = 1.0f / sqrtf(tot / (float)sh.K + nm.eps);
      }
      scale_due = false;
    }
    __syncthreads();
    // 256 threads store a group of 16 tokens: thread (token t, row i); the groups are dealt
    // out to the workgroup's sets of 256 threads.
    const int sets = blockDim.x / 256;
    for (int g = tid < sets * 256 ? tid / 256 : TG; g < TG; g += sets) {
      const int t = (tid % 256) / 16, i = tid % 16;
      const int tok = 16 * g + t;
      const float* mine = red_p + g * 256 + t * 16;
      const float inv_rms = SCALED ? inv_s[tok] : 1.f;
      if constexpr (GATED) {
        constexpr int h = TR / 2;
        const long long c = (long long)tile * h + i;
        if (i < h && tok < T && c < N) {
          float gate = 0.f, up = 0.f;
          for (int w = 0; w < nwaves; ++w) {
            gate += mine[w * kRed + i];
            up += mine[w * kRed + h + i];
          }
          gate *= inv_rms;
          up *= inv_rms;
          st(Y + (long long)tok * sh.ldy + c, gate / (1.0f + expf(-gate)) * up);
        }
      } else if constexpr (JOIN) {
        const long long n = (long long)tile * TR + i;
        float sq = 0.f;
        if (i < TR && tok < T && n < N) {
          float sum = 0.f;
          for (int w = 0; w < nwaves; ++w) sum += mine[w * kRed + i];
          if (nm.round_parts) sum = bf16_to_f32(f32_to_bf16(sum));
          const float wn = nm.weight_f32 ? ((const float*)nm.weight)[n]
                                         : bf16_to_f32(((const bf16_t*)nm.weight)[n]);
          const float total = nm.resid[(long long)tok * N + n] + sum;
          nm.resid_out[(long long)tok * N + n] = total;
          nm.xw_out[(long long)tok * N + n] = f32_to_bf16(total * wn);
          sq = total * total;
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) sq += __shfl_xor(sq, o, kWave);
        if (i == 0 && tok < T) nm.ss_out[(long long)tok * nm.ss_stride + tile] = sq;
      } else {
        const long long n = (long long)tile * TR + i;
        if (i < TR && tok < T && n < N) {
          float sum = 0.f;
          for (int w = 0; w < nwaves; ++w) sum += mine[w * kRed + i];
          st(Y + (long long)tok * sh.ldy + n, sum * inv_rms);
        }
      }
    }
    par ^= 1;
  };
  for (;;) {
    if (tile >= sh.num_tiles) break;
    one_tile(a0);
    tile += gridDim.x;
    if constexpr (AHEAD == 2) {
      if (tile >= sh.num_tiles) break;
      one_tile(a1);
      tile += gridDim.x;
    }
  }
#undef RLIS_WIDE_LOAD_TILE
}

// Waves a workgroup may have with TG groups of tokens in registers, and with two tiles ahead.
constexpr int wide_max_waves(int tg) { return tg == 2 ? 12 : 8; }
constexpr int kWideDeepWaves = 8;
// The partial sums of squares a row that the scaled form takes (64 lanes, four each).
constexpr int kWideScaleParts = 256;

template <typename TC, bool GATED, int TR, int MODE, int TG, int AHEAD>
int launch_tiles(const void* X, const void* W, void* Y, StreamShape sh, const StreamNorm& nm,
                 int nwaves, int num_cus, hipStream_t stream) {
  constexpr size_t kPerWave = TR * kStreamItem * 2 + 2 * TG * 256 * sizeof(float);
  constexpr size_t kScales = TG * 16 * sizeof(float);
  static LdsGrant lds_raised;
  {
    hipError_t e = grant_lds(
        lds_raised, (const void*)gemm_bf16_stream_wide_kernel<TC, GATED, TR, MODE, TG, AHEAD>,
        (int)(wide_max_waves(TG) * kPerWave + kScales));
    RLIS_REQUIRE(e == hipSuccess, "gemm_bf16_stream (17 to 32 rows): cannot raise the LDS limit: %s",
                 hipGetErrorString(e));
  }
  const size_t smem = nwaves * kPerWave + kScales;
  const int per_cu = max(1, (int)((160 * 1024) / smem));
  const long long tiles = ceil_div_ll(sh.N, GATED ? TR / 2 : TR);
  RLIS_REQUIRE(tiles <= 0x3fffffffll, "gemm_bf16_stream: N=%d is too large", sh.N);
  sh.num_tiles = (int)tiles;
  const long long cap = (long long)num_cus * per_cu;
  const long long groups = tiles < cap ? tiles : cap;
  gemm_bf16_stream_wide_kernel<TC, GATED, TR, MODE, TG, AHEAD>
      <<<(int)groups, nwaves * 64, smem, stream>>>((const bf16_t*)X, (const bf16_t*)W, (TC*)Y, sh,
                                                   nm);
  return 0;
}

template <typename TC, bool GATED, int MODE, int TG>
int launch_rows(const void* X, const void* W, void* Y, const StreamShape& sh, const StreamNorm& nm,
                int nwaves, int num_cus, hipStream_t stream) {
  const int tr = rlis_stream_balanced_rows(sh.N, 1, GATED, num_cus);
#define RLIS_WIDE_GO(TR_)                                                                       \
  return nwaves <= kWideDeepWaves                                                               \
             ? launch_tiles<TC, GATED, TR_, MODE, TG, 2>(X, W, Y, sh, nm, nwaves, num_cus, stream) \
             : launch_tiles<TC, GATED, TR_, MODE, TG, 1>(X, W, Y, sh, nm, nwaves, num_cus, stream)
  if (tr == 8) RLIS_WIDE_GO(8);
  if (tr == 12) RLIS_WIDE_GO(12);
  RLIS_WIDE_GO(16);
#undef RLIS_WIDE_GO
}

template <typename TC, bool GATED, int MODE>
int launch_groups(const void* X, const void* W, void* Y, const StreamShape& sh,
                  const StreamNorm& nm, int nwaves, int num_cus, hipStream_t stream) {
  // (Four groups, 33 to 64 rows, fit eight waves' registers with one tile ahead only: with one
  // workgroup per compute unit that keeps half the bytes on their way that it takes, and the
  // library's products with the norm and SwiGLU kernels are faster.  Not offered.)
  return launch_rows<TC, GATED, MODE, 2>(X, W, Y, sh, nm, nwaves, num_cus, stream);
}

}  // namespace

int rlis_stream_wide_rows(int K) {
  if (K <= 0 || K % kStreamItem != 0) return 16;
  return K / kStreamItem <= wide_max_waves(2) ? 32 : 16;
}

int rlis_launch_stream_wide(const char* name, int mode, const void* X, const void* W, void* Y,
                            int y_dtype, int T, int N, int K, long long ldx, long long ldw,
                            long long ldy, int gated, const StreamNorm& nm, hipStream_t stream) {
  RLIS_REQUIRE(T > 16 && T <= rlis_stream_wide_rows(K),
               "%s: %d rows of K=%d, at most %d", name, T, K, rlis_stream_wide_rows(K));
  RLIS_REQUIRE(!gated || y_dtype == RLIS_BF16, "%s: the gated form stores bfloat16", name);
  RLIS_REQUIRE(mode != kStreamScaled || nm.scale_count <= kWideScaleParts,
               "%s: %d partial sums of squares a row, at most %d with 17 to 32 rows", name,
               nm.scale_count, kWideScaleParts);
  const int num_cus = rlis_stream_compute_units();
  RLIS_REQUIRE(num_cus > 0, "%s: cannot read the device properties", name);
  StreamShape sh;
  sh.T = T; sh.N = N; sh.K = K; sh.ldx = ldx; sh.ldw = ldw; sh.ldy = ldy;
  sh.part_stride = 0;
  sh.num_slices = 1;
  sh.num_tiles = 0;
  const int nwaves = max(4, K / kStreamItem);
  int rc = 1;
  if (mode == kStreamJoin) {
    RLIS_REQUIRE(!gated, "%s: a product that joins the residual has no gate", name);
    rc = launch_groups<bf16_t, false, kStreamJoin>(X, W, Y, sh, nm, nwaves, num_cus, stream);
  } else if (mode == kStreamScaled) {
    if (gated) rc = launch_groups<bf16_t, true, kStreamScaled>(X, W, Y, sh, nm, nwaves, num_cus, stream);
    else if (y_dtype == RLIS_F32)
      rc = launch_groups<float, false, kStreamScaled>(X, W, Y, sh, nm, nwaves, num_cus, stream);
    else if (y_dtype == RLIS_BF16)
      rc = launch_groups<bf16_t, false, kStreamScaled>(X, W, Y, sh, nm, nwaves, num_cus, stream);
    else RLIS_REQUIRE(false, "%s: unknown output dtype %d", name, y_dtype);
  } else if (mode == kStreamPlain) {
    if (gated) rc = launch_groups<bf16_t, true, kStreamPlain>(X, W, Y, sh, nm, nwaves, num_cus, stream);
    else if (y_dtype == RLIS_F32)
      rc = launch_groups<float, false, kStreamPlain>(X, W, Y, sh, nm, nwaves, num_cus, stream);
    else if (y_dtype == RLIS_BF16)
      rc = launch_groups<bf16_t, false, kStreamPlain>(X, W, Y, sh, nm, nwaves, num_cus, stream);
    else RLIS_REQUIRE(false, "%s: unknown output dtype %d", name, y_dtype);
  } else {
    RLIS_REQUIRE(false, "%s: no such form for 17 to 32 rows", name);
  }
  if (rc) return rc;
  RLIS_LAUNCH_CHECK(name);
  return 0;
}
