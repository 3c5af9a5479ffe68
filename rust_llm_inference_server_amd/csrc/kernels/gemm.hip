// Matrix products y = x * W^T for the projections (weights are (out, in) row-major, as the
// reference's Linear holds them: crates/model/src/layers.rs:17-19, 65-69, 82).
//
//  * gemm_plain: any sizes, float32 accumulation with ordinary FMAs (no matrix-core
//    shortcut), operands float32 or bfloat16.  This is the product of the true 32-bit path.
//  * gemm_bf16_mfma: bfloat16 operands on the matrix cores (v_mfma_f32_32x32x16_bf16),
//    float32 accumulation, output bfloat16 or float32.  K must be a multiple of 8.
//  * gemm_bf16_skinny: the decode shape, up to 64 rows of x.  Each weight row is read once
//    for all rows of x; a wave owns 16 (or 32) weight rows and a slice of K, the eight waves of
//    a workgroup are summed in a fixed order.  K must be a multiple of 8.  A gated variant
//    fuses the SwiGLU of the feed-forward into the gate/up product.
//  * gemm_bf16_stream: up to 16 rows of x at the streaming rate of the memory: weights are
//    loaded row-contiguously and turned into operand layout in LDS.  Plain and gated.
//
// In every kernel an output element is a sum over k in an order that depends only on the
// kernel and K, never on which other rows are in the batch.
#include "common.h"
#include "gemm_stream.h"

// ============================================================== plain FMA product
template <typename TA, typename TB, typename TC>
__global__ __launch_bounds__(256) void gemm_plain_kernel(const TA* __restrict__ A,
                                                         const TB* __restrict__ B,
                                                         TC* __restrict__ C, int M, int N, int K,
                                                         long long lda, long long ldb,
                                                         long long ldc) {
  constexpr int BM = 64, BN = 64, BK = 16;
  __shared__ float As[BK][BM + 4];
  __shared__ float Bs[BK][BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + i * 256;
      const int r = idx / BK, kk = idx % BK;
      const int gm = m0 + r, gn = n0 + r, gk = k0 + kk;
      As[kk][r] = (gm < M && gk < K) ? ld(A + (long long)gm * lda + gk) : 0.f;
      Bs[kk][r] = (gn < N && gk < K) ? ld(B + (long long)gn * ldb + gk) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + ty * 4 + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn < N) st(C + (long long)gm * ldc + gn, acc[i][j]);
    }
  }
}

template <typename TA, typename TB, typename TC>
static void launch_plain(const void* A, const void* B, void* C, int M, int N, int K,
                         long long lda, long long ldb, long long ldc, hipStream_t stream) {
  dim3 grid(ceil_div(N, 64), ceil_div(M, 64));
  gemm_plain_kernel<TA, TB, TC><<<grid, 256, 0, stream>>>((const TA*)A, (const TB*)B, (TC*)C, M,
                                                          N, K, lda, ldb, ldc);
}

// C (M,N) = A (M,K) * B (N,K)^T with row strides lda/ldb/ldc in elements.
RLIS_API int rlis_gemm_plain(const void* A, int a_dtype, const void* B, int b_dtype, void* C,
                             int c_dtype, int M, int N, int K, long long lda, long long ldb,
                             long long ldc, hipStream_t stream) {
  RLIS_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_plain: bad sizes M=%d N=%d K=%d", M, N, K);
  RLIS_REQUIRE(lda >= K && ldb >= K && ldc >= N, "gemm_plain: row strides shorter than rows");
  RLIS_REQUIRE(ceil_div(M, 64) <= 65535, "gemm_plain: M=%d is too large", M);
  if (M == 0) return 0;
  const int key = a_dtype * 4 + b_dtype * 2 + c_dtype;
#define CASE(k, TA, TB, TC)                                                    \
  case k:                                                                      \
    launch_plain<TA, TB, TC>(A, B, C, M, N, K, lda, ldb, ldc, stream);         \
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
      RLIS_REQUIRE(false, "gemm_plain: unknown dtypes %d %d %d", a_dtype, b_dtype, c_dtype);
  }
#undef CASE
  RLIS_LAUNCH_CHECK("gemm_plain");
  return 0;
}

// ================================================================ MFMA bf16 product
// Tile 128 x 128 x 64, four waves in a 2 x 2 arrangement, each wave 64 x 64 as 2 x 2 blocks of
// v_mfma_f32_32x32x16_bf16.  Operand fragments: lane l holds row (or column) l % 32 and the 8
// consecutive k at (l / 32) * 8; the accumulator holds column l % 32 and rows
// (r / 4) * 8 + (l / 32) * 4 + r % 4 for register r.
template <typename TC>
__global__ __launch_bounds__(256) void gemm_bf16_mfma_kernel(const bf16_t* __restrict__ A,
                                                             const bf16_t* __restrict__ B,
                                                             TC* __restrict__ C, int M, int N,
                                                             int K, long long lda, long long ldb,
                                                             long long ldc, int tiles_n) {
  constexpr int BM = 128, BN = 128, BK = 64, LDS_STRIDE = BK + 8;  // in bf16 elements
  __shared__ __attribute__((aligned(16))) bf16_t As[BM * LDS_STRIDE];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[BN * LDS_STRIDE];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int wm = wave / 2, wn = wave % 2;
  const int tile_m = blockIdx.x / tiles_n, tile_n = blockIdx.x % tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Each thread moves 4 chunks of 8 bf16 per operand per tile: chunk c covers row c / 8,
  // k offset (c % 8) * 8.
  uint4 ra[4], rb[4];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + i * 256;
      const int r = c / 8, kc = (c % 8) * 8;
      const int gk = k0 + kc;
      const int gm = m0 + r, gn = n0 + r;
      ra[i] = (gm < M && gk < K) ? *(const uint4*)(A + (long long)gm * lda + gk)
                                 : make_uint4(0, 0, 0, 0);
      rb[i] = (gn < N && gk < K) ? *(const uint4*)(B + (long long)gn * ldb + gk)
                                 : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_lds = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + i * 256;
      const int r = c / 8, kc = (c % 8) * 8;
      *(uint4*)(As + r * LDS_STRIDE + kc) = ra[i];
      *(uint4*)(Bs + r * LDS_STRIDE + kc) = rb[i];
    }
  };

  const int num_k = (K + BK - 1) / BK;
  load_global(0);
  store_lds();
  __syncthreads();
  for (int kt = 0; kt < num_k; ++kt) {
    if (kt + 1 < num_k) load_global((kt + 1) * BK);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      Frag8 a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int row = wm * 64 + i * 32 + (lane % 32);
        a[i].u = *(const uint4*)(As + row * LDS_STRIDE + ks * 16 + (lane / 32) * 8);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int row = wn * 64 + j * 32 + (lane % 32);
        b[j].u = *(const uint4*)(Bs + row * LDS_STRIDE + ks * 16 + (lane / 32) * 8);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i].v, b[j].v, acc[i][j], 0, 0, 0);
    }
    __syncthreads();
    if (kt + 1 < num_k) {
      store_lds();
      __syncthreads();
    }
  }

#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int gn = n0 + wn * 64 + j * 32 + (lane % 32);
      if (gn >= N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int gm = m0 + wm * 64 + i * 32 + (r / 4) * 8 + (lane / 32) * 4 + (r % 4);
        if (gm < M) st(C + (long long)gm * ldc + gn, acc[i][j][r]);
      }
    }
}

RLIS_API int rlis_gemm_bf16_mfma(const void* A, const void* B, void* C, int c_dtype, int M, int N,
                                 int K, long long lda, long long ldb, long long ldc,
                                 hipStream_t stream) {
  RLIS_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_bf16_mfma: bad sizes M=%d N=%d K=%d", M, N, K);
  RLIS_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0,
               "gemm_bf16_mfma: K=%d and the row strides must be multiples of 8", K);
  RLIS_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)B % 16) == 0,
               "gemm_bf16_mfma: operands must be 16-byte aligned");
  RLIS_REQUIRE(lda >= K && ldb >= K && ldc >= N, "gemm_bf16_mfma: row strides shorter than rows");
  if (M == 0) return 0;
  const int tiles_m = ceil_div(M, 128), tiles_n = ceil_div(N, 128);
  const long long blocks = (long long)tiles_m * tiles_n;
  RLIS_REQUIRE(blocks < (1ll << 31), "gemm_bf16_mfma: too many tiles");
  if (c_dtype == RLIS_F32)
    gemm_bf16_mfma_kernel<float><<<(int)blocks, 256, 0, stream>>>(
        (const bf16_t*)A, (const bf16_t*)B, (float*)C, M, N, K, lda, ldb, ldc, tiles_n);
  else if (c_dtype == RLIS_BF16)
    gemm_bf16_mfma_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>(
        (const bf16_t*)A, (const bf16_t*)B, (bf16_t*)C, M, N, K, lda, ldb, ldc, tiles_n);
  else
    RLIS_REQUIRE(false, "gemm_bf16_mfma: unknown output dtype %d", c_dtype);
  RLIS_LAUNCH_CHECK("gemm_bf16_mfma");
  return 0;
}

// ============================================================ skinny (decode) product
// y (T, N) = x (T, K) * W (N, K)^T for T <= 64 (NT = ceil(T / 16) token tiles).  A workgroup of
// eight waves owns 16 * RB weight rows; wave w owns the k range [w * kslice, (w + 1) * kslice)
// and walks it in chunks of 32 * U, issuing all loads of a chunk before its products so that
// U * RB 16-byte weight loads per lane are in flight.  v_mfma_f32_16x16x32_bf16 with the weight
// rows as the M side and the tokens as the N side: lane l holds weight row l % 16 (A) or token
// l % 16 (B) and the 8 consecutive k at (l / 16) * 8; the accumulator holds token l % 16 and
// weight rows (l / 16) * 4 + r.  The eight waves are summed through LDS in wave order.
//
// GATED: W holds gate rows [0, N) and up rows [N, 2N); the workgroup computes both for its
// columns and stores silu(gate) * up (the SwiGLU of crates/model/src/layers.rs:179-186), so
// the (T, 2N) intermediate never exists.
constexpr int kSkinnyWaves = 8;

template <typename TC, int NT, int RB, bool GATED>
__global__ __launch_bounds__(512) void gemm_bf16_skinny_kernel(const bf16_t* __restrict__ X,
                                                               const bf16_t* __restrict__ W,
                                                               TC* __restrict__ Y, int T, int N,
                                                               int K, long long ldx,
                                                               long long ldw, long long ldy,
                                                               int kslice) {
  constexpr int RBT = GATED ? 2 * RB : RB;                 // row blocks of 16 weight rows
  constexpr int U = (NT * RBT <= 1) ? 8 : ((NT * RBT <= 4) ? 4 : 2);
  __shared__ float red[kSkinnyWaves][NT][256];
  __shared__ float fin[RBT][NT][256];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int m = lane % 16, kq = (lane / 16) * 8;
  const int n0 = blockIdx.x * 16 * RB;

  const bf16_t* wp[RBT];
  bool wvalid[RBT];
#pragma unroll
  for (int rb = 0; rb < RBT; ++rb) {
    const int col = n0 + (rb % RB) * 16 + m;               // output column
    wvalid[rb] = col < N;
    const long long row = (GATED && rb >= RB) ? (long long)N + col : col;
    wp[rb] = W + (wvalid[rb] ? row : 0) * ldw;
  }
  const bf16_t* xp[NT];
  bool xvalid[NT];
#pragma unroll
  for (int tt = 0; tt < NT; ++tt) {
    const int tok = tt * 16 + m;
    xvalid[tt] = tok < T;
    xp[tt] = X + (long long)(xvalid[tt] ? tok : 0) * ldx;
  }
  f32x4 acc[RBT][NT];
#pragma unroll
  for (int rb = 0; rb < RBT; ++rb)
#pragma unroll
    for (int tt = 0; tt < NT; ++tt) acc[rb][tt] = (f32x4){0.f, 0.f, 0.f, 0.f};

  const int kbeg = wave * kslice;
  const int kend = min(K, kbeg + kslice);
  for (int k = kbeg; k < kend; k += 32 * U) {
    Frag8 a[RBT][U], b[NT][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int gk = k + u * 32 + kq;
      const bool kin = gk < kend;     // kslice is a multiple of 32 and K of 8: whole chunks only
      // Loads are never predicated off (the compiler would turn that into flat loads of a
      // zero kept in scratch): out-of-range lanes read a safe address and are zeroed after.
      const int sk = kin ? gk : k;
#pragma unroll
      for (int rb = 0; rb < RBT; ++rb) {
        const uint4 v = *(const uint4*)(wp[rb] + sk);
        const bool ok = wvalid[rb] && kin;
        a[rb][u].u = make_uint4(ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u);
      }
#pragma unroll
      for (int tt = 0; tt < NT; ++tt) {
        const uint4 v = *(const uint4*)(xp[tt] + sk);
        const bool ok = xvalid[tt] && kin;
        b[tt][u].u = make_uint4(ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int rb = 0; rb < RBT; ++rb)
#pragma unroll
        for (int tt = 0; tt < NT; ++tt)
          acc[rb][tt] =
              __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rb][u].v, b[tt][u].v, acc[rb][tt], 0, 0, 0);
  }

  // Sum the eight waves, one row block at a time: fin[rb][tt][r * 64 + l] is the product for
  // token tt * 16 + l % 16 and weight row (l / 16) * 4 + r of block rb.
#pragma unroll
  for (int rb = 0; rb < RBT; ++rb) {
    if (rb > 0) __syncthreads();
#pragma unroll
    for (int tt = 0; tt < NT; ++tt)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][tt][r * 64 + lane] = acc[rb][tt][r];
    __syncthreads();
    for (int i = tid; i < NT * 256; i += 512) {
      const int tt = i / 256, e = i % 256;
      float s = red[0][tt][e];
#pragma unroll
      for (int w = 1; w < kSkinnyWaves; ++w) s += red[w][tt][e];
      fin[rb][tt][e] = s;
    }
  }
  __syncthreads();
  for (int i = tid; i < RB * NT * 256; i += 512) {
    const int rb = i / (NT * 256), tt = (i / 256) % NT, e = i % 256;
    const int r = e / 64, l = e % 64;
    const int tok = tt * 16 + (l % 16);
    const int col = n0 + rb * 16 + (l / 16) * 4 + r;
    if (tok >= T || col >= N) continue;
    float v = fin[rb][tt][e];
    if (GATED) {
      const float up = fin[RB + rb][tt][e];
      v = v / (1.0f + expf(-v)) * up;
    }
    st(Y + (long long)tok * ldy + col, v);
  }
}

template <typename TC, int NT, int RB, bool GATED>
static void launch_skinny(const void* X, const void* W, void* Y, int T, int N, int K,
                          long long ldx, long long ldw, long long ldy, hipStream_t stream) {
  const int kslice = ceil_div(ceil_div(K, kSkinnyWaves), 32) * 32;
  const int blocks = ceil_div(N, 16 * RB);
  gemm_bf16_skinny_kernel<TC, NT, RB, GATED><<<blocks, 512, 0, stream>>>(
      (const bf16_t*)X, (const bf16_t*)W, (TC*)Y, T, N, K, ldx, ldw, ldy, kslice);
}

template <typename TC, bool GATED>
static void dispatch_skinny(const void* X, const void* W, void* Y, int T, int N, int K,
                            long long ldx, long long ldw, long long ldy, hipStream_t stream) {
  const int nt = ceil_div(T, 16);
  // Two row blocks per workgroup when that still leaves every compute unit a workgroup or two.
  const bool wide = !GATED && N >= 8192;
#define GO(NT)                                                                         \
  do {                                                                                 \
    if (wide) launch_skinny<TC, NT, 2, GATED>(X, W, Y, T, N, K, ldx, ldw, ldy, stream); \
    else launch_skinny<TC, NT, 1, GATED>(X, W, Y, T, N, K, ldx, ldw, ldy, stream);     \
  } while (0)
  switch (nt) {
    case 1: GO(1); break;
    case 2: GO(2); break;
    case 3: GO(3); break;
    default: GO(4); break;
  }
#undef GO
}

static int check_skinny(const char* name, const void* X, const void* W, int T, int N, int K,
                        long long ldx, long long ldw, long long ldy) {
  RLIS_REQUIRE(T >= 0 && T <= 64, "%s: T=%d rows, at most 64", name, T);
  RLIS_REQUIRE(N > 0 && K > 0, "%s: bad sizes N=%d K=%d", name, N, K);
  RLIS_REQUIRE(K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0,
               "%s: K=%d and the row strides must be multiples of 8", name, K);
  RLIS_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0,
               "%s: operands must be 16-byte aligned", name);
  RLIS_REQUIRE(ldx >= K && ldw >= K && ldy >= N, "%s: row strides shorter than rows", name);
  return 0;
}

RLIS_API int rlis_gemm_bf16_skinny(const void* X, const void* W, void* Y, int y_dtype, int T,
                                   int N, int K, long long ldx, long long ldw, long long ldy,
                                   hipStream_t stream) {
  if (check_skinny("gemm_bf16_skinny", X, W, T, N, K, ldx, ldw, ldy)) return 1;
  if (T == 0) return 0;
  if (y_dtype == RLIS_F32)
    dispatch_skinny<float, false>(X, W, Y, T, N, K, ldx, ldw, ldy, stream);
  else if (y_dtype == RLIS_BF16)
    dispatch_skinny<bf16_t, false>(X, W, Y, T, N, K, ldx, ldw, ldy, stream);
  else
    RLIS_REQUIRE(false, "gemm_bf16_skinny: unknown output dtype %d", y_dtype);
  RLIS_LAUNCH_CHECK("gemm_bf16_skinny");
  return 0;
}

// y (T, N) = silu(x Wg^T) * (x Wu^T) with W = [Wg; Wu] of shape (2N, K), bfloat16 throughout.
RLIS_API int rlis_gemm_bf16_skinny_swiglu(const void* X, const void* W, void* Y, int T, int N,
                                          int K, long long ldx, long long ldw, long long ldy,
                                          hipStream_t stream) {
  if (check_skinny("gemm_bf16_skinny_swiglu", X, W, T, N, K, ldx, ldw, ldy)) return 1;
  if (T == 0) return 0;
  dispatch_skinny<bf16_t, true>(X, W, Y, T, N, K, ldx, ldw, ldy, stream);
  RLIS_LAUNCH_CHECK("gemm_bf16_skinny_swiglu");
  return 0;
}

// ==================================================== split-k product for 17 to 64 rows
// y (T <= 64, N) = x W^T as float32 partial sums, one (T, N) array per k slice, for the
// projections whose result joins the residual stream (its next consumer adds the slices in
// order).  A workgroup of four waves owns 64 weight rows and one k slice of KS (256 or 512): the
// rows of x of that slice lie in LDS for all four waves (tokens beyond T and k beyond K as
// zeros), each wave loads its 16 weight rows of the slice straight into operand layout, all of
// them at once (16 rows x 64 bytes per instruction, KS / 32 instructions in flight per lane),
// and multiplies them with the four token groups from LDS (v_mfma_f32_16x16x32_bf16, weight
// rows as the M side).  Every weight is read once, x once per 64 weight rows through the L2.
// Which k a slice covers depends on K and N alone, so a row's sums do not depend on T.
constexpr int kSplitRows = 64;          // weight rows per workgroup
constexpr int kSplitPad = 16;           // bf16 elements between rows of x in LDS: 32 bytes mod 64

template <int KS, int NT, bool WALK>
__global__ __launch_bounds__(256, 2) void gemm_bf16_splitk_kernel(const bf16_t* __restrict__ X,
                                                               const bf16_t* __restrict__ W,
                                                               float* __restrict__ Y, int T, int N,
                                                               int K, long long ldx, long long ldw,
                                                               long long part_stride, int subs) {
  extern __shared__ __attribute__((aligned(16))) bf16_t splitk_x[];   // [NT * 16][KS + pad]
  constexpr int XS = KS + kSplitPad;
  constexpr int STEPS = KS / 32;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int l16 = lane % 16, lq = lane / 16;
  const int slice = blockIdx.y;
  const int n0 = blockIdx.x * kSplitRows + wave * 16;

  // This wave's weight rows, in operand layout: lane l holds row l % 16 and the 8 k at
  // (l / 16) * 8 of every step.  Loads are never predicated off: a row past N reads row N - 1
  // (its products are not stored), a k past K reads k = 0 (it meets a zero of x).
  const int row = min(n0 + l16, N - 1);
  const bf16_t* wrow = W + (long long)row * ldw;
  // The slice of x goes into LDS in 16-byte pieces, rows of tokens (zeros past T and past K).
  // All of a thread's pieces are loaded before the first is stored, so that they travel
  // together (and with the weights); the loads are unconditional from a safe address, the value
  // is selected.
  constexpr int PIECES = KS / 8;
  constexpr int XIT = NT * 16 * PIECES / 256;
  Frag8 a[STEPS], ahead[WALK ? STEPS : 1];
  uint4 xv[XIT];
  // (x first: loads come back in order, and the rows of x, which the L2 holds, are on their way
  // to LDS while the weights still arrive)
  auto load = [&](int k0, Frag8 (&w)[STEPS]) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < XIT; ++j) {
      const int i = tid + j * 256;
      const int tok = i / PIECES, k = k0 + (i % PIECES) * 8;
      const bool ok = tok < T && k < K;
      const uint4 v = *(const uint4*)(X + (ok ? (long long)tok * ldx + k : 0));
      xv[j] = make_uint4(ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u);
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int k = k0 + s * 32 + lq * 8;
      w[s].u = *(const uint4*)(wrow + (k < K ? k : 0));
    }
  };

  f32x4 acc[NT];
#pragma unroll
  for (int tg = 0; tg < NT; ++tg) acc[tg] = (f32x4){0.f, 0.f, 0.f, 0.f};
  // A workgroup walks over `subs` pieces of KS of its slice (WALK; one piece otherwise), the
  // next piece's weights and x on their way while the current one is multiplied.
  if (!WALK) subs = 1;
  int k0 = slice * subs * KS;
  load(k0, a);
  for (int sub = 0; sub < subs; ++sub) {
    if (sub) __syncthreads();             // the last piece's x has been read by every wave
#pragma unroll
    for (int j = 0; j < XIT; ++j) {
      const int i = tid + j * 256;
      *(uint4*)(splitk_x + (i / PIECES) * XS + (i % PIECES) * 8) = xv[j];
    }
    __syncthreads();
    k0 += KS;
    bool more = false;
    if constexpr (WALK) {
      more = sub + 1 < subs && k0 < K;
      if (more) load(k0, ahead);
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
#pragma unroll
      for (int tg = 0; tg < NT; ++tg) {
        Frag8 b;
        b.u = *(const uint4*)(splitk_x + (tg * 16 + l16) * XS + s * 32 + lq * 8);
        acc[tg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s].v, b.v, acc[tg], 0, 0, 0);
      }
    }
    if (!more) break;
    if constexpr (WALK) {
#pragma unroll
      for (int s = 0; s < STEPS; ++s) a[s] = ahead[s];
    }
  }
  // The accumulator holds token l % 16 of its group and weight rows (l / 16) * 4 + r.
  float* y = Y + (long long)slice * part_stride;
  const int col = n0 + lq * 4;
#pragma unroll
  for (int tg = 0; tg < NT; ++tg) {
    const int tok = tg * 16 + l16;
    if (tok >= T) continue;
    float* dst = y + (long long)tok * N + col;
    if (col + 3 < N && (N % 4) == 0 && (part_stride % 4) == 0) {
      *(float4*)dst = make_float4(acc[tg][0], acc[tg][1], acc[tg][2], acc[tg][3]);
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (col + r < N) dst[r] = acc[tg][r];
    }
  }
}

// How rlis_gemm_bf16_splitk cuts a product with N weight rows over K: pieces of 512 k, or of
// 256 where that is needed to give every compute unit a workgroup, and two pieces per workgroup
// where one would make more than two workgroups per compute unit (measured on 4096 x 14336 with
// 32 rows: one piece 29 us and 28 partial results for the consumer to add, two 30 us and 14,
// four 34 us and 7; the consumer gains more from 14 than the product loses).  Functions of N and
// K alone; the number of slices (and of partial results) is ceil(K / (piece * pieces per
// workgroup)).
struct SplitkCut {
  int piece, subs, slices;
};
static SplitkCut splitk_cut(int N, int K) {
  const long long groups = ceil_div(N, kSplitRows);
  const long long pieces512 = ceil_div(K, 512);
  SplitkCut c;
  c.piece = groups * pieces512 >= 256 ? 512 : 256;
  c.subs = 1;
  if (c.piece == 512) {
    const long long per = ceil_div_ll(groups * pieces512, 512);
    c.subs = per > 1 ? 2 : 1;
  }
  c.slices = ceil_div(K, c.piece * c.subs);
  return c;
}
RLIS_API int rlis_gemm_bf16_splitk_slices(int N, int K) { return splitk_cut(N, K).slices; }

// Y receives rlis_gemm_bf16_splitk_slices(N, K) partial results (T, N) float32 contiguous,
// part_stride elements apart, to be added in order.  17 <= T <= 64 is what it is for; fewer
// rows work too.  bfloat16 operands, K a multiple of 8.
RLIS_API int rlis_gemm_bf16_splitk(const void* X, const void* W, void* Y, int T, int N, int K,
                                   long long ldx, long long ldw, long long part_stride,
                                   hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && T <= 64, "gemm_bf16_splitk: T=%d rows, at most 64", T);
  RLIS_REQUIRE(N > 0 && K > 0 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && ldx >= K && ldw >= K,
               "gemm_bf16_splitk: bad sizes N=%d K=%d ldx=%lld ldw=%lld", N, K, ldx, ldw);
  RLIS_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0 && ((uintptr_t)Y % 16) == 0,
               "gemm_bf16_splitk: operands must be 16-byte aligned");
  RLIS_REQUIRE(part_stride >= (long long)T * N,
               "gemm_bf16_splitk: partial results %lld elements apart do not hold (T, N)",
               part_stride);
  if (T == 0) return 0;
  const SplitkCut cut = splitk_cut(N, K);
  // A workgroup that walks takes its slice in pieces of 256 (the registers of a piece are held
  // twice then): the same k in the same order as pieces of 512 would give.
  const int walk = cut.subs > 1;
  const int ks = walk ? 256 : cut.piece, slices = cut.slices;
  const int subs = cut.piece * cut.subs / ks;
  const int nt = ceil_div(T, 16);
  dim3 grid(ceil_div(N, kSplitRows), slices);
  RLIS_REQUIRE(slices <= 65535, "gemm_bf16_splitk: K=%d is too long", K);
  const size_t smem = (size_t)nt * 16 * (ks + kSplitPad) * sizeof(bf16_t);
#define GO(KS, NT, WALK)                                                                    \
  {                                                                                         \
    static LdsGrant raised;                                                                 \
    if (smem > 48 * 1024) {                                                                 \
      hipError_t e = grant_lds(raised, (const void*)gemm_bf16_splitk_kernel<KS, NT, WALK>,  \
                               (int)smem);                                                  \
      RLIS_REQUIRE(e == hipSuccess, "gemm_bf16_splitk: cannot raise the LDS limit: %s",     \
                   hipGetErrorString(e));                                                   \
    }                                                                                       \
    gemm_bf16_splitk_kernel<KS, NT, WALK><<<grid, 256, smem, stream>>>(                     \
        (const bf16_t*)X, (const bf16_t*)W, (float*)Y, T, N, K, ldx, ldw, part_stride,      \
        subs);                                                                              \
  }
#define BY_NT(KS, WALK)                        \
  switch (nt) {                                \
    case 1: GO(KS, 1, WALK) break;             \
    case 2: GO(KS, 2, WALK) break;             \
    case 3: GO(KS, 3, WALK) break;             \
    default: GO(KS, 4, WALK) break;            \
  }
  if (walk) BY_NT(256, true)
  else if (ks == 512) BY_NT(512, false)
  else BY_NT(256, false)
#undef BY_NT
#undef GO
  RLIS_LAUNCH_CHECK("gemm_bf16_splitk");
  return 0;
}

// ============================================================ streaming skinny product
// y (T <= 16, N) = x W^T at the speed of the weight stream.
//
// Work is cut into tiles of 16 (or 12, or 8) weight rows times a k slice of up to 16 items of 256; a
// workgroup has one wave per item and walks over tiles (persistent, its slice fixed), so the
// rows of x that a wave needs are loaded once, straight into operand layout, and stay in
// registers.  An item's weights are loaded row by row, 512 contiguous bytes per half wave,
// which keeps the memory system at its streaming rate, one tile ahead of the arithmetic.  The
// matrix-core operand wants lane l to hold row l % 16 instead, so the item goes through an
// LDS tile private to the wave (chunks XOR-swizzled by row, so both directions are free of
// bank conflicts).  One v_mfma_f32_16x16x32_bf16 accumulator per wave; the waves of a
// workgroup are summed in LDS in wave order.  Rows of 4096 < K <= 8192 in whole fours of items
// stay in one slice (plain and joining products only, tiles of 8 weight rows): a wave then
// takes four neighbouring items (IPW = 4; at most eight waves, which leaves each the registers
// for four items of x), each through an LDS tile of its own into the same accumulator, so that
// a projection over a feed-forward's width can still add itself to the residual.  With more than
// one slice (K > 8192) every slice stores its own float32 partial result, which the consumer
// adds in slice order: the order of a sum depends on K alone.  The gated form pairs gate rows with their up rows in one
// tile and applies the SwiGLU before the store.
constexpr int kStreamMaxWaves = 16;

__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
  const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* p, float (&v)[8]) {
  const uint4 u = *(const uint4*)p;
  const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

template <typename TC, bool GATED, int TR /* weight rows per tile: 16, 12 or 8 */, int MODE,
          int IPW /* k items per wave: 1 or 4 */, bool PACK = false /* see below */>
__global__ __launch_bounds__(IPW == 1 ? 1024 : 512) void gemm_bf16_stream_kernel(const bf16_t* __restrict__ X,
                                                                const bf16_t* __restrict__ W,
                                                                TC* __restrict__ Y,
                                                                const StreamShape sh,
                                                                const StreamNorm nm) {
  extern __shared__ __attribute__((aligned(16))) unsigned char stream_smem[];
  constexpr bool NORM = MODE == kStreamNorm, SCALED = MODE == kStreamScaled;
  constexpr bool JOIN = MODE == kStreamJoin;
  static_assert(!(JOIN && GATED), "a product that joins the residual has no gate");
  static_assert(IPW == 1 || (IPW == 4 && TR == 8 && !GATED && (MODE == kStreamPlain || JOIN)),
                "four items per wave: tiles of 8 rows of a plain or joining product");
  // PACK (up to 8 tokens): a tile of 8 weight rows and 8 tokens fill half
  // of a 16 x 16 product each, so two halves of k share one: lanes oi >= 8 hold, for weight row
  // and token oi - 8, the k chunks four further on.  Rows and columns 0..7 of the result then
  // carry one half of k and rows and columns 8..15 the other (the rest is not looked at), a
  // product covers 64 k, and x takes half the loads and registers.
  // (The launch sees to it that every wave then has whole items: nothing is zeroed.)
  static_assert(!PACK || (TR == 8 && !GATED && (MODE == kStreamPlain || JOIN)),
                "packing two halves of k: tiles of 8 rows of a plain or joining product");
  constexpr int NJ = PACK ? 4 : 8;                      // products per item
  constexpr int kTileBytes = NORM ? kStreamTileBytes : TR * kStreamItem * 2;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64, nwaves = blockDim.x / 64;
  unsigned char* tile_s = stream_smem + wave * (IPW * kTileBytes);     // a tile per item
  float* red = (float*)(stream_smem + nwaves * (IPW * kTileBytes));    // [2][nwaves][256]
  const int half = lane / 32, l32 = lane % 32;          // loading: row parity, 16-byte chunk
  const int oi = lane % 16, og = lane / 16;             // operand: row (or token), k group
  const int T = sh.T, N = sh.N, K = sh.K;
  const int slice = blockIdx.x % sh.num_slices;
  const int tile_step = gridDim.x / sh.num_slices;
  const int nitems = (K + kStreamItem - 1) / kStreamItem;
  const int item = (slice * nwaves + wave) * IPW;       // this wave's (first) k item
  const bool has_item = item < nitems;
  const int kb = item * kStreamItem;
  // Loads are never predicated off (that would cost registers for the zeros): a row past the
  // end reads row 0 instead and is not stored; a k past the end reads k = 0 instead and meets
  // a zero in the rows of x (weights are finite).
  // With several items per wave the order of the first loads matters (below): the two
  // pointers then pass through an empty statement, after which the compiler knows nothing
  // about what they point to and keeps their loads on their side of a memory barrier.
  // (They are declared as pointers to global memory, which the compiler could no longer tell
  // by itself.)
  typedef const __attribute__((address_space(1))) bf16_t* GlobalBf16;
  typedef uint32_t Bits4 __attribute__((ext_vector_type(4)));
  typedef const __attribute__((address_space(1))) Bits4* GlobalU4;
  GlobalBf16 w_base = (GlobalBf16)W;
  GlobalBf16 x_base = (GlobalBf16)X;
  if constexpr (IPW > 1) asm volatile("" : "+s"(w_base), "+s"(x_base));
  GlobalBf16 w_lane[IPW];
#pragma unroll
  for (int it = 0; it < IPW; ++it) {
    const int ka = kb + it * kStreamItem + l32 * 8;     // this lane's k when loading weights
    w_lane[it] = w_base + ((item + it < nitems && ka < K) ? ka : 0);
  }

  // Tile row r = 2 p + half of tile `tile` is weight row tile * rows + r; gated, the first
  // half of a tile's rows are the gate rows of consecutive columns and the second half their
  // up rows, N further down.  Everything but `half` and the lane's k is uniform over the wave.
  constexpr int cols_per_tile = GATED ? TR / 2 : TR;
#define RLIS_STREAM_LOAD_TILE(a, tile_)                                                         \
  {                                                                                             \
    const int tl_ = (tile_);                                                                    \
    if (tl_ < sh.num_tiles) {                                                                   \
      const int col0 = tl_ * cols_per_tile + half;                                              \
      _Pragma("unroll") for (int it_ = 0; it_ < IPW; ++it_) {                                   \
        GlobalBf16 w_tile = w_lane[it_] + (long long)col0 * sh.ldw;                             \
        _Pragma("unroll") for (int p = 0; p < TR / 2; ++p) {                                    \
          const int c = GATED ? (2 * p) % cols_per_tile : 2 * p; /* column within the tile */   \
          const long long up = (GATED && 2 * p >= cols_per_tile) ? (long long)N * sh.ldw : 0;   \
          GlobalBf16 ptr = col0 + c < N ? w_tile + (long long)c * sh.ldw + up : w_lane[it_];    \
          const Bits4 v_ = *(GlobalU4)ptr;       /* a k past the end meets a zero of x */       \
          a[it_][p].x = v_.x;   /* member by member: a struct copy would go through scratch */  \
          a[it_][p].y = v_.y;                                                                   \
          a[it_][p].z = v_.z;                                                                   \
          a[it_][p].w = v_.w;                                                                   \
        }                                                                                       \
      }                                                                                         \
    }                                                                                           \
  }

  uint4 a[IPW][TR / 2];
  int tile = blockIdx.x / sh.num_slices;
  RLIS_STREAM_LOAD_TILE(a, tile);        // the first tile is on its way during the prologue
  // The weights are asked for first: loads are served in order, and behind four items of x
  // (one address for eight loads: the compiler would gladly issue them first) the first weight
  // would leave two microseconds late.
  if constexpr (IPW > 1) asm volatile("" ::: "memory");

  // The rows of x in operand layout: token oi, k = kb + (4 j + og) * 8 .. + 8 for step j (of
  // item `it`, kStreamItem further on).
  Frag8 b[IPW][NJ];
  float inv_rms = 1.f;                   // NORM: of token tid / 16, in the threads that store
  // SCALED: the scale comes as partial sums of squares, scale_count a token.  Thread (token
  // tid / 16, i = tid % 16) of the 256 storing threads takes parts 4 i .. 4 i + 3, + 64, ...
  // The first 64 * kScaleAhead of them are asked for here, without a condition (so that the
  // loads in flight can be counted and nobody waits for these before the weights; the other
  // waves ask for one address), and added up only when the first tile is stored.  The order of
  // the sum depends on scale_count alone.
  constexpr int kScaleAhead = 4;
  float4 scale_ahead[SCALED ? kScaleAhead : 1];
  bool scale_due = SCALED;
  if (!NORM) {
#pragma unroll
    for (int it = 0; it < IPW; ++it) {
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int k = kb + it * kStreamItem + (4 * j + og) * 8;
        const bool ok = item + it < nitems && oi < T && k < K;
        if constexpr (PACK) {
          // token oi % 8, chunks 8 j + 4 (oi / 8) + og: one address for the four loads
          GlobalBf16 xb = x_base + (long long)min(oi % 8, T - 1) * sh.ldx + kb + it * kStreamItem +
                          (oi / 8) * 32 + og * 8;
          b[it][j].v = __builtin_bit_cast(bf16x8, *(GlobalU4)(xb + j * 64));
        } else if constexpr (IPW == 1) {
          const uint4 v = *(const uint4*)(X + (ok ? (long long)oi * sh.ldx + k : 0));
          b[it][j].u = make_uint4(ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u);
        } else {
          // Every wave has whole items (the launch sees to that), and a token past the end
          // takes the last one's row: its products are not stored.  So nothing is zeroed, no
          // load is waited for here, and the eight loads of an item share one address.
          GlobalBf16 xb = x_base + (long long)min(oi, T - 1) * sh.ldx + kb + it * kStreamItem + og * 8;
          b[it][j].v = __builtin_bit_cast(bf16x8, *(GlobalU4)(xb + j * 32));
        }
      }
    }
    if constexpr (SCALED) {
#pragma unroll
      for (int j = 0; j < kScaleAhead; ++j) {
        const int part = 4 * (tid % 16) + 64 * j;
        const bool mine = tid < 256 && part < nm.scale_count;
        const float4 v = *(const float4*)(nm.scale_parts +
                                          (mine ? (long long)(tid / 16) * nm.ss_stride + part : 0));
        scale_ahead[j] = make_float4(mine ? v.x : 0.f, mine && part + 1 < nm.scale_count ? v.y : 0.f,
                                     mine && part + 2 < nm.scale_count ? v.z : 0.f,
                                     mine && part + 3 < nm.scale_count ? v.w : 0.f);
      }
    }
  } else {
    // Each wave makes its own 16 x 256 item of x: (resid + delta) * norm_weight, rounded to
    // bfloat16, written to its LDS tile (which the weights use only afterwards) in units of
    // one token and 8 k, a half wave per token so that the reads are contiguous; then every
    // lane picks its operand chunks from there.  Sums of squares go per (wave, token) to the
    // second half of `red`, which the tiles use only after their first barrier.
    const bool store_sum = nm.resid_out != nullptr && blockIdx.x == 0;
    float* ss_s = red + nwaves * 256;
    if (!has_item) {
      if (lane < 16) ss_s[wave * 16 + lane] = 0.f;
    } else {
      // A lane keeps its chunk of 8 k and walks over tokens lane / 32, + 2, + 4, ...; the
      // loads of kU tokens are issued together.
      constexpr int kU = 2;
      const int c = l32, k = kb + c * 8;
      const bool ok = k < K;
      const int ks = ok ? k : 0;
      float w[8];
      if (nm.weight_f32)
        load8((const float*)nm.weight + ks, w);
      else
        load8((const bf16_t*)nm.weight + ks, w);
      for (int t0 = half; t0 < T; t0 += 2 * kU) {
        float v[kU][8];
        long long at[kU];
#pragma unroll
        for (int i = 0; i < kU; ++i) {
          const int t = min(t0 + 2 * i, T - 1);               // repeats the last token: not used
          at[i] = (nm.rows ? (long long)nm.rows[t] : (long long)t) * K + ks;
          load8(nm.resid + at[i], v[i]);
        }
        if (nm.delta) {
          // The first two parts are loaded together, so that their loads travel with the
          // residual's; the parts are summed in order on their own and then join the residual.
          const bool two = nm.parts > 1;
          float acc[kU][8], nxt[kU][8];
#pragma unroll
          for (int i = 0; i < kU; ++i) {
            if (nm.delta_f32) {
              const float* dp = (const float*)nm.delta + at[i];
              load8(dp, acc[i]);
              load8(two ? dp + nm.part_stride : dp, nxt[i]);
            } else {
              const bf16_t* dp = (const bf16_t*)nm.delta + at[i];
              load8(dp, acc[i]);
              load8(two ? dp + nm.part_stride : dp, nxt[i]);
            }
          }
          if (two) {
#pragma unroll
            for (int i = 0; i < kU; ++i)
#pragma unroll
              for (int e = 0; e < 8; ++e) acc[i][e] += nxt[i][e];
          }
          for (int s = 2; s < nm.parts; ++s) {
#pragma unroll
            for (int i = 0; i < kU; ++i) {
              if (nm.delta_f32)
                load8((const float*)nm.delta + s * nm.part_stride + at[i], nxt[i]);
              else
                load8((const bf16_t*)nm.delta + s * nm.part_stride + at[i], nxt[i]);
            }
#pragma unroll
            for (int i = 0; i < kU; ++i)
#pragma unroll
              for (int e = 0; e < 8; ++e) acc[i][e] += nxt[i][e];
          }
#pragma unroll
          for (int i = 0; i < kU; ++i)
#pragma unroll
            for (int e = 0; e < 8; ++e)
              v[i][e] += nm.round_parts ? bf16_to_f32(f32_to_bf16(acc[i][e])) : acc[i][e];
        }
#pragma unroll
        for (int i = 0; i < kU; ++i) {
          const int t = t0 + 2 * i;
          if (t < T) {
            if (nm.delta && store_sum && ok) {
              *(float4*)(nm.resid_out + at[i]) = make_float4(v[i][0], v[i][1], v[i][2], v[i][3]);
              *(float4*)(nm.resid_out + at[i] + 4) = make_float4(v[i][4], v[i][5], v[i][6], v[i][7]);
            }
            float ss = 0.f;
            Frag8 xw;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float x = ok ? v[i][e] : 0.f;
              ss += x * x;
              xw.v[e] = (__bf16)(x * w[e]);
            }
            *(uint4*)(tile_s + t * (kStreamItem * 2) + ((c ^ t) * 16)) = xw.u;
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) ss += __shfl_xor(ss, o, kWave);
            if (l32 == 0) ss_s[wave * 16 + t] = ss;
          }
        }
      }
      wave_lds_fence();
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint4 v = *(const uint4*)(tile_s + oi * (kStreamItem * 2) + (((4 * j + og) ^ oi) * 16));
        const bool tok = oi < T;
        b[0][j].u = make_uint4(tok ? v.x : 0u, tok ? v.y : 0u, tok ? v.z : 0u, tok ? v.w : 0u);
      }
      wave_lds_fence();
    }
    __syncthreads();
    if (tid < 256) {
      float tot = 0.f;
      for (int w = 0; w < nwaves; ++w) tot += ss_s[w * 16 + tid / 16];
      inv_rms = 1.0f / sqrtf(tot / (float)K + nm.eps);
    }
  }

  int par = 0;
  for (; tile < sh.num_tiles; tile += tile_step) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    if (has_item) {
#pragma unroll
      for (int it = 0; it < IPW; ++it) {
#pragma unroll
        for (int p = 0; p < TR / 2; ++p) {
          const int r = 2 * p + half;
          *(uint4*)(tile_s + it * kTileBytes + r * (kStreamItem * 2) + ((l32 ^ r) * 16)) = a[it][p];
        }
      }
    }
    // JOIN: this thread's element of the residual and of the norm's weight, asked for ahead of
    // the next tile's weights (loads come back in order: who waits for these must not wait
    // for those).
    // Both are kept as loaded and looked at only after the products (a conversion or a select
    // here would wait for them, and with them for every load issued before).
    float join_resid = 0.f;
    uint32_t join_weight_bits = 0;
    if constexpr (JOIN) {
      const int t = (tid / 16) % 16, i = tid % 16;
      const long long n = (long long)tile * TR + i;
      const bool ok = tid < 256 && i < TR && t < T && n < N;
      join_resid = nm.resid[ok ? (long long)t * N + n : 0];
      if (nm.weight_f32)
        join_weight_bits = ((const uint32_t*)nm.weight)[ok ? n : 0];
      else
        join_weight_bits = ((const bf16_t*)nm.weight)[ok ? n : 0];
    }
    // The next tile is on its way during the arithmetic; with several items per wave only
    // after it, so that the weights' registers are free for the reads from LDS to run ahead
    // of the products (such workgroups seldom have a second tile).
    if constexpr (IPW == 1) RLIS_STREAM_LOAD_TILE(a, tile + tile_step);
    if (has_item) {
      wave_lds_fence();
#pragma unroll
      for (int it = 0; it < IPW; ++it) {
#pragma unroll
        for (int j0 = 0; j0 < NJ; j0 += 4) {
          Bits4 af[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            // tile rows beyond TR repeat the first ones: their products are not stored (PACK:
            // they carry the chunks of the other half of k)
            const int chunk = PACK ? 8 * (j0 + j) + 4 * (oi / 8) + og : 4 * (j0 + j) + og;
            af[j] = *(const Bits4*)(tile_s + it * kTileBytes + (oi % TR) * (kStreamItem * 2) +
                                    ((chunk ^ (oi % TR)) * 16));
          }
          // With two waves per SIMD nobody else fills the time a read from LDS takes: four are
          // asked for before the first of their products (the statement, which every read
          // feeds and every product depends on, keeps the compiler from pairing each read
          // with its product again).
          if constexpr (IPW > 1)
            asm volatile("s_waitcnt lgkmcnt(0)"
                         : "+v"(af[0]), "+v"(af[1]), "+v"(af[2]), "+v"(af[3]));
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[j]),
                                                          b[it][j0 + j].v, acc, 0, 0, 0);
        }
      }
      wave_lds_fence();
    }
    if constexpr (IPW > 1) RLIS_STREAM_LOAD_TILE(a, tile + tile_step);
    // acc: token oi, tile rows og * 4 + r.  red[par][wave][token][row]; the buffer of the
    // tile before is still being read by slower waves, the one before that is free again
    // after this tile's barrier.
    float* red_p = red + par * nwaves * 256;
    *(float4*)(red_p + wave * 256 + oi * 16 + og * 4) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    __syncthreads();
    if (tid < 256) {
      const int t = tid / 16, i = tid % 16;
      if (SCALED && scale_due) {
        float tot = 0.f;
#pragma unroll
        for (int j = 0; j < kScaleAhead; ++j)
          tot += ((scale_ahead[j].x + scale_ahead[j].y) + scale_ahead[j].z) + scale_ahead[j].w;
        for (int part = 4 * i + 64 * kScaleAhead; part < nm.scale_count; part += 64)
          for (int e = 0; e < 4 && part + e < nm.scale_count; ++e)
            tot += nm.scale_parts[(long long)t * nm.ss_stride + part + e];
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) tot += __shfl_xor(tot, o, kWave);
        inv_rms = 1.0f / sqrtf(tot / (float)K + nm.eps);
        scale_due = false;
      }
      TC* y = Y + (long long)slice * sh.part_stride + (long long)t * sh.ldy;
      if (GATED) {
        constexpr int h = TR / 2;
        const long long c = (long long)tile * h + i;
        if (i < h && t < T && c < N) {
          float gate = 0.f, up = 0.f;
          for (int w = 0; w < nwaves; ++w) {
            gate += red_p[w * 256 + t * 16 + i];
            up += red_p[w * 256 + t * 16 + h + i];
          }
          gate *= inv_rms;
          up *= inv_rms;
          st(y + c, gate / (1.0f + expf(-gate)) * up);
        }
      } else if (JOIN) {
        const long long n = (long long)tile * TR + i;
        float sq = 0.f;
        if (i < TR && t < T && n < N) {
          float sum = 0.f;
          for (int w = 0; w < nwaves; ++w) {
            sum += red_p[w * 256 + t * 16 + i];
            if constexpr (PACK) sum += red_p[w * 256 + (t + 8) * 16 + i + 8];
          }
          sum *= inv_rms;
          if (nm.round_parts) sum = bf16_to_f32(f32_to_bf16(sum));
          const float total = join_resid + sum;
          const float join_weight = __uint_as_float(nm.weight_f32 ? join_weight_bits
                                                                  : join_weight_bits << 16);
          nm.resid_out[(long long)t * N + n] = total;
          nm.xw_out[(long long)t * N + n] = f32_to_bf16(total * join_weight);
          sq = total * total;
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) sq += __shfl_xor(sq, o, kWave);
        if (i == 0) nm.ss_out[(long long)t * nm.ss_stride + tile] = sq;
      } else {
        const long long n = (long long)tile * TR + i;
        if (i < TR && t < T && n < N) {
          float sum = 0.f;
          for (int w = 0; w < nwaves; ++w) {
            sum += red_p[w * 256 + t * 16 + i];
            if constexpr (PACK) sum += red_p[w * 256 + (t + 8) * 16 + i + 8];
          }
          st(y + n, sum * inv_rms);
        }
      }
    }
    par ^= 1;
  }
#undef RLIS_STREAM_LOAD_TILE
}

// A workgroup takes up to 16 k items, one per wave, or up to 32 in whole fours, four per wave
// (plain and joining products); other rows are cut into slices of up to 16 items.  All of it
// follows from K alone.
constexpr int kStreamFour = 4;
static int stream_items_per_wave(int K) {
  const int nitems = ceil_div(K, kStreamItem);
  return K % (kStreamFour * kStreamItem) == 0 && nitems > kStreamMaxWaves &&
                 nitems <= 2 * kStreamMaxWaves
             ? kStreamFour : 1;
}
static int stream_slices(int K) {
  return stream_items_per_wave(K) > 1 ? 1 : ceil_div(ceil_div(K, kStreamItem), kStreamMaxWaves);
}
// The fused norm needs whole rows in one workgroup, one item per wave; so do the gated and the
// scaled form.
constexpr int kStreamNormMaxK = kStreamMaxWaves * kStreamItem;

template <typename TC, bool GATED, int TR, int MODE, int IPW = 1, bool PACK = false>
static int launch_stream_tiles(const void* X, const void* W, void* Y, StreamShape sh,
                               const StreamNorm& nm, int nwaves, int num_cus,
                               hipStream_t stream) {
  constexpr int kTileBytes = IPW * (MODE == kStreamNorm ? kStreamTileBytes : TR * kStreamItem * 2);
  static LdsGrant lds_raised;
  {
    hipError_t e = grant_lds(
        lds_raised, (const void*)gemm_bf16_stream_kernel<TC, GATED, TR, MODE, IPW, PACK>,
        (IPW == 1 ? kStreamMaxWaves : 2 * kStreamMaxWaves / IPW) * (kTileBytes + 2048));
    RLIS_REQUIRE(e == hipSuccess, "gemm_bf16_stream: cannot raise the LDS limit: %s",
                 hipGetErrorString(e));
  }
  const size_t smem = (size_t)nwaves * (kTileBytes + 2048);
  const int per_cu = max(1, (int)((160 * 1024) / smem));
  const long long tiles = ceil_div_ll(sh.N, GATED ? TR / 2 : TR);
  RLIS_REQUIRE(tiles <= 0x3fffffffll, "gemm_bf16_stream: N=%d is too large", sh.N);
  sh.num_tiles = (int)tiles;
  long long groups = tiles;                                // workgroups per slice
  const long long cap = max(1, num_cus * per_cu / sh.num_slices);
  if (groups > cap) groups = cap;
  gemm_bf16_stream_kernel<TC, GATED, TR, MODE, IPW, PACK>
      <<<(int)(groups * sh.num_slices), nwaves * 64, smem, stream>>>(
          (const bf16_t*)X, (const bf16_t*)W, (TC*)Y, sh, nm);
  return 0;
}

int rlis_stream_compute_units() {
  constexpr int kDevices = 64;
  static int num_cus[kDevices];                    // of every device asked about so far
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  const bool known = dev >= 0 && dev < kDevices;
  if (known && num_cus[dev] > 0) return num_cus[dev];
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  if (known) num_cus[dev] = n;
  return n;
}

int rlis_stream_balanced_rows(int N, int slices, bool gated, int num_cus) {
  int best = 16;
  long long best_cost = 0;
  for (int tr : {16, 12, 8}) {
    const long long tiles = (long long)ceil_div(N, gated ? tr / 2 : tr) * slices;
    const long long cost = ceil_div_ll(tiles, num_cus) * tr;
    if (tr == 16 || cost < best_cost) {
      best = tr;
      best_cost = cost;
    }
  }
  return best;
}

// Weight rows per tile of the kernel for up to 16 rows of x.
static int stream_tile_rows(int N, int K, bool gated, bool norm, int num_cus) {
  (void)norm;
  if (stream_items_per_wave(K) > 1) return 8;            // what the registers hold
  return rlis_stream_balanced_rows(N, stream_slices(K), gated, num_cus);
}

template <typename TC, bool GATED, int MODE>
static int launch_stream(const void* X, const void* W, void* Y, int T, int N, int K, long long ldx,
                         long long ldw, long long ldy, long long part_stride,
                         const StreamNorm& nm, hipStream_t stream) {
  const int nitems = ceil_div(K, kStreamItem);
  const int slices = stream_slices(K), ipw = stream_items_per_wave(K);
  const int nwaves = max(4, ceil_div(nitems, slices * ipw));
  const int num_cus = rlis_stream_compute_units();
  RLIS_REQUIRE(num_cus > 0, "gemm_bf16_stream: cannot read the device properties");
  StreamShape sh;
  sh.T = T; sh.N = N; sh.K = K; sh.ldx = ldx; sh.ldw = ldw; sh.ldy = ldy;
  sh.part_stride = part_stride;
  sh.num_slices = slices;
  sh.num_tiles = 0;
  if (ipw > 1) {
    if constexpr (!GATED && (MODE == kStreamPlain || MODE == kStreamJoin)) {
      if (T <= 8)
        return launch_stream_tiles<TC, false, 8, MODE, kStreamFour, true>(X, W, Y, sh, nm, nwaves,
                                                                          num_cus, stream);
      return launch_stream_tiles<TC, false, 8, MODE, kStreamFour>(X, W, Y, sh, nm, nwaves, num_cus,
                                                                  stream);
    }
    RLIS_REQUIRE(false, "gemm_bf16_stream: K=%d is too long for this form (at most %d)", K,
                 kStreamNormMaxK);
  }
  switch (stream_tile_rows(N, K, GATED, MODE == kStreamNorm, num_cus)) {
    case 8:
      // up to 8 tokens over whole items, one for every wave: two halves of k share a product
      if constexpr (!GATED && (MODE == kStreamPlain || MODE == kStreamJoin)) {
        if (T <= 8 && K % kStreamItem == 0 && slices * nwaves == nitems)
          return launch_stream_tiles<TC, false, 8, MODE, 1, true>(X, W, Y, sh, nm, nwaves, num_cus,
                                                                  stream);
      }
      return launch_stream_tiles<TC, GATED, 8, MODE>(X, W, Y, sh, nm, nwaves, num_cus, stream);
    case 12:
      return launch_stream_tiles<TC, GATED, 12, MODE>(X, W, Y, sh, nm, nwaves, num_cus, stream);
    default:
      return launch_stream_tiles<TC, GATED, 16, MODE>(X, W, Y, sh, nm, nwaves, num_cus, stream);
  }
}

template <int MODE>
static int dispatch_stream(const char* name, const void* X, const void* W, void* Y, int y_dtype,
                           int T, int N, int K, long long ldx, long long ldw, long long ldy,
                           long long part_stride, int gated, const StreamNorm& nm,
                           hipStream_t stream) {
  RLIS_REQUIRE(!gated || y_dtype == RLIS_BF16, "%s: the gated form stores bfloat16", name);
  int rc;
  if constexpr (MODE == kStreamJoin) {
    RLIS_REQUIRE(!gated, "%s: a product that joins the residual has no gate", name);
    rc = launch_stream<bf16_t, false, MODE>(X, W, Y, T, N, K, ldx, ldw, ldy, part_stride, nm, stream);
  } else {
    if (gated)
      rc = launch_stream<bf16_t, true, MODE>(X, W, Y, T, N, K, ldx, ldw, ldy, part_stride, nm, stream);
    else if (y_dtype == RLIS_F32)
      rc = launch_stream<float, false, MODE>(X, W, Y, T, N, K, ldx, ldw, ldy, part_stride, nm, stream);
    else if (y_dtype == RLIS_BF16)
      rc = launch_stream<bf16_t, false, MODE>(X, W, Y, T, N, K, ldx, ldw, ldy, part_stride, nm, stream);
    else
      RLIS_REQUIRE(false, "%s: unknown output dtype %d", name, y_dtype);
  }
  if (rc) return rc;
  RLIS_LAUNCH_CHECK(name);
  return 0;
}

// Slices that rlis_gemm_bf16_stream cuts K into; with more than one, Y receives that many
// float32 partial results, part_stride elements apart, to be added in order.
RLIS_API int rlis_gemm_bf16_stream_slices(int K) { return stream_slices(K); }

// The most rows of x that rlis_gemm_bf16_stream and its joining and scaled forms take for rows
// of K: 16, or 32 where K is a whole number of items and short enough for the kernel that keeps
// 32 rows in registers.
RLIS_API int rlis_gemm_bf16_stream_max_rows(int K) { return rlis_stream_wide_rows(K); }

// The longest row that rlis_norm_linear_bf16 takes.
RLIS_API int rlis_norm_linear_max_k() { return kStreamNormMaxK; }

// gated == 0: y (T, N) = x W^T (one result up to K = 8192, float32 partial results per slice
// beyond).  gated != 0: W is (2N, K) = [Wg; Wu] and
// y (T, N) = silu(x Wg^T) * (x Wu^T), K <= 4096.  bfloat16 operands, K a multiple of 8, up to
// rlis_gemm_bf16_stream_max_rows(K) rows (more than 16 go to the kernel of gemm_wide.hip).
RLIS_API int rlis_gemm_bf16_stream(const void* X, const void* W, void* Y, int y_dtype, int T,
                                   int N, int K, long long ldx, long long ldw, long long ldy,
                                   long long part_stride, int gated, hipStream_t stream) {
  if (check_skinny("gemm_bf16_stream", X, W, T, N, K, ldx, ldw, ldy)) return 1;
  if (T > 16) {
    StreamNorm none = {};
    return rlis_launch_stream_wide("gemm_bf16_stream", kStreamPlain, X, W, Y, y_dtype, T, N, K, ldx,
                                   ldw, ldy, gated, none, stream);
  }
  const int slices = stream_slices(K);
  RLIS_REQUIRE(slices == 1 || (!gated && y_dtype == RLIS_F32 && part_stride >= (long long)T * ldy),
               "gemm_bf16_stream: K=%d takes %d slices, which need float32 partial results and "
               "no gate", K, slices);
  RLIS_REQUIRE(!gated || K <= kStreamNormMaxK, "gemm_bf16_stream: the gated form takes K up to "
               "%d, not %d", kStreamNormMaxK, K);
  if (T == 0) return 0;
  StreamNorm nm = {};
  return dispatch_stream<kStreamPlain>("gemm_bf16_stream", X, W, Y, y_dtype, T, N, K, ldx, ldw, ldy,
                                part_stride, gated, nm, stream);
}

// A norm between two products without a pass over whole rows, in two calls (rows as above, bfloat16
// operands, one k slice each).  rlis_gemm_bf16_stream_join: s = resid + x W^T (the product
// rounded to bfloat16 first with round_sum), stored to resid_out (resid itself is fine);
// xw_out (T, N) bfloat16 = s * norm_weight; ss_out (T up to a multiple of 16, ss_stride) float32 = per token the sums
// of s^2 over each of the rlis_gemm_bf16_stream_join_tiles(N, K) tiles of columns (ss_stride a
// multiple of 4, at least that many; what lies behind them in a row is not written).  resid and
// resid_out are (T, N) float32 contiguous.  rlis_gemm_bf16_stream_scaled: y = (x W^T) *
// rsqrt(sum of the row's scale_count partial sums / K + eps), gated as rlis_gemm_bf16_stream:
// with x = xw_out and the partial sums of the first call, the RMSNorm of s in front of this
// product.
RLIS_API int rlis_gemm_bf16_stream_join_tiles(int N, int K) {
  const int cus = rlis_stream_compute_units();
  return cus > 0 ? ceil_div(N, stream_tile_rows(N, K, false, false, cus)) : 0;
}

RLIS_API int rlis_gemm_bf16_stream_join(const void* X, const void* W, int T, int N, int K,
                                        long long ldx, long long ldw, const float* resid,
                                        float* resid_out, const void* norm_weight,
                                        int norm_weight_dtype, int round_sum, void* xw_out,
                                        float* ss_out, int ss_stride, hipStream_t stream) {
  if (check_skinny("gemm_bf16_stream_join", X, W, T, N, K, ldx, ldw, N)) return 1;
  RLIS_REQUIRE(stream_slices(K) == 1, "gemm_bf16_stream_join: K=%d takes more than one slice", K);
  RLIS_REQUIRE(resid && resid_out && norm_weight && xw_out && ss_out,
               "gemm_bf16_stream_join: an operand is missing");
  RLIS_REQUIRE(norm_weight_dtype == RLIS_F32 || norm_weight_dtype == RLIS_BF16,
               "gemm_bf16_stream_join: unknown norm weight dtype %d", norm_weight_dtype);
  RLIS_REQUIRE(ss_stride % 4 == 0 && ss_stride >= rlis_gemm_bf16_stream_join_tiles(N, K) &&
                   ((uintptr_t)ss_out % 16) == 0,
               "gemm_bf16_stream_join: the sums of squares need rows of %d entries or more, a "
               "multiple of 4, 16-byte aligned", rlis_gemm_bf16_stream_join_tiles(N, K));
  if (T == 0) return 0;
  StreamNorm nm = {};
  nm.resid = resid;
  nm.resid_out = resid_out;
  nm.weight = norm_weight;
  nm.weight_f32 = norm_weight_dtype == RLIS_F32;
  nm.round_parts = round_sum;
  nm.xw_out = (bf16_t*)xw_out;
  nm.ss_out = ss_out;
  nm.ss_stride = ss_stride;
  if (T > 16)
    return rlis_launch_stream_wide("gemm_bf16_stream_join", kStreamJoin, X, W, xw_out, RLIS_BF16, T,
                                   N, K, ldx, ldw, N, 0, nm, stream);
  return dispatch_stream<kStreamJoin>("gemm_bf16_stream_join", X, W, xw_out, RLIS_BF16, T, N, K, ldx,
                                ldw, N, 0, 0, nm, stream);
}

RLIS_API int rlis_gemm_bf16_stream_scaled(const void* X, const void* W, void* Y, int y_dtype,
                                          int T, int N, int K, long long ldx, long long ldw,
                                          long long ldy, int gated, const float* scale_parts,
                                          int scale_count, int ss_stride, float eps,
                                          hipStream_t stream) {
  if (check_skinny("gemm_bf16_stream_scaled", X, W, T, N, K, ldx, ldw, ldy)) return 1;
  RLIS_REQUIRE(K <= kStreamNormMaxK, "gemm_bf16_stream_scaled: K=%d, at most %d", K,
               kStreamNormMaxK);
  RLIS_REQUIRE(scale_parts && scale_count > 0 && ss_stride % 4 == 0 && ss_stride >= scale_count &&
                   ((uintptr_t)scale_parts % 16) == 0,
               "gemm_bf16_stream_scaled: %d partial sums in rows of %d", scale_count, ss_stride);
  if (T == 0) return 0;
  StreamNorm nm = {};
  nm.scale_parts = scale_parts;
  nm.scale_count = scale_count;
  nm.ss_stride = ss_stride;
  nm.eps = eps;
  if (T > 16)
    return rlis_launch_stream_wide("gemm_bf16_stream_scaled", kStreamScaled, X, W, Y, y_dtype, T, N, K,
                                   ldx, ldw, ldy, gated, nm, stream);
  return dispatch_stream<kStreamScaled>("gemm_bf16_stream_scaled", X, W, Y, y_dtype, T, N, K, ldx, ldw,
                                ldy, 0, gated, nm, stream);
}

// RMSNorm and projection in one pass, for T <= 16 tokens and K <= 4096:
//   s = resid[row(t)] + sum of the `parts` deltas (delta may be null; with round_parts the
//       sum of the parts is rounded to bfloat16 before it joins the residual),
//   y[t] = (s * rsqrt(mean(s^2) + eps) * norm_weight) W^T   (gated as above),
// where row(t) = rows[t], or t when rows is null.  resid is (R, K) float32 contiguous; each
// delta part is shaped like it (bfloat16, or float32 for partial sums), part_stride elements
// apart.  When resid_out is given (only without rows, and never resid itself: other
// workgroups still read that), it receives s.  The normalised row is rounded to bfloat16
// before the scale by rsqrt is applied rather than after; the scale is exact in float32.
RLIS_API int rlis_norm_linear_bf16(const float* resid, const void* delta, int delta_dtype,
                                   int parts, long long part_stride, int round_parts,
                                   const void* norm_weight,
                                   int norm_weight_dtype, float eps, const int* rows,
                                   float* resid_out, const void* W, void* Y, int y_dtype, int T,
                                   int N, int K, long long ldw, long long ldy, int gated,
                                   hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && T <= 16, "norm_linear: T=%d rows, at most 16", T);
  RLIS_REQUIRE(N > 0 && K > 0 && K % 8 == 0 && ldw % 8 == 0 && ldw >= K && ldy >= N,
               "norm_linear: bad sizes N=%d K=%d ldw=%lld ldy=%lld", N, K, ldw, ldy);
  RLIS_REQUIRE(K <= kStreamNormMaxK, "norm_linear: K=%d, at most %d", K, kStreamNormMaxK);
  RLIS_REQUIRE(((uintptr_t)W % 16) == 0 && ((uintptr_t)resid % 16) == 0 &&
                   ((uintptr_t)delta % 16) == 0 && ((uintptr_t)norm_weight % 16) == 0 &&
                   ((uintptr_t)resid_out % 16) == 0,
               "norm_linear: operands must be 16-byte aligned");
  RLIS_REQUIRE(!delta || (parts >= 1 && (parts == 1 || delta_dtype == RLIS_F32)),
               "norm_linear: %d delta parts of dtype %d", parts, delta_dtype);
  RLIS_REQUIRE(!resid_out || (resid_out != resid && !rows),
               "norm_linear: resid_out must be another buffer and excludes a row selection");
  RLIS_REQUIRE((delta_dtype == RLIS_F32 || delta_dtype == RLIS_BF16) &&
                   (norm_weight_dtype == RLIS_F32 || norm_weight_dtype == RLIS_BF16),
               "norm_linear: unknown dtypes %d %d", delta_dtype, norm_weight_dtype);
  if (T == 0) return 0;
  StreamNorm nm = {};
  nm.resid = resid;
  nm.delta = delta;
  nm.delta_f32 = delta_dtype == RLIS_F32;
  nm.parts = delta ? parts : 0;
  nm.part_stride = part_stride;
  nm.round_parts = round_parts;
  nm.weight = norm_weight;
  nm.weight_f32 = norm_weight_dtype == RLIS_F32;
  nm.eps = eps;
  nm.rows = rows;
  nm.resid_out = delta ? resid_out : nullptr;
  return dispatch_stream<kStreamNorm>("norm_linear", nullptr, W, Y, y_dtype, T, N, K, K, ldw, ldy, 0,
                               gated, nm, stream);
}
