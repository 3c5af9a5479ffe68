// Prefill attention over the paged cache on the matrix cores (bfloat16 operands, float32
// accumulation and softmax), one compile unit per padded head size RLIS_HEAD_DIM.
//
// A workgroup of four waves serves 64 (or, QB = 2, 128) consecutive new tokens of one sequence
// for one query head; each wave owns 16 (32, as two blocks of 16) of them.  With two query blocks
// every K and V fragment that a wave reads from LDS serves two products, which halves the LDS
// traffic per flop: long prompts, whose tiles are plenty, take that form.  Keys are walked in
// tiles of BN positions aligned to BN,
// read through the block table: the K tile [key][dim] and the V tile [dim][key] (the cache
// keeps V transposed inside a page, so both are copied as they lie) go to LDS once per
// workgroup, the next tile travelling global -> registers while the current one is computed.
//
// Both products are computed transposed with v_mfma_f32_16x16x32_bf16, whose 16 x 16 result
// holds, in lane l and register r, row (l / 16) * 4 + r and column l % 16:
//   S^T = K Q^T   (rows: keys, columns: queries)
//   O^T = V^T P^T (rows: dims, columns: queries)
// so a lane only ever holds values of ONE query, column l % 16: its running maximum,
// denominator and rescaling factor are plain per-lane scalars, the row reductions need two
// lane exchanges, and the probabilities a lane holds after the softmax are exactly the
// B-operand fragment of the second product (the k slots of a step of 32 keys are mapped to
// keys {16 * 2s + 4 q + j} and {16 * (2s + 1) + 4 q + j}), so P never leaves the registers.
//
// The mask is the reference's causal mask offset by the cached length (crates/model/src/
// attention.rs:225-233): the new token at index i of a sequence with P cached positions sees
// keys at positions <= P + i, and > P + i - window when a window is given.  Scores are scaled
// in float32 after the product (kept in the base-2 domain so that e^x is one v_exp_f32);
// probabilities are rounded to bfloat16 only as the operand of the second product (the row
// sums use the float32 values).
#include "common.h"

#include <math.h>

#ifndef RLIS_HEAD_DIM
#error "RLIS_HEAD_DIM must be defined (padded head size, a multiple of 32)"
#endif

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // 16 bytes in flight, a plain vector

union Frag8 {
  uint4 u;
  uint2 h[2];
  bf16x8 v;
  bf16_t e[8];
};


// A unit is a library of its own, loaded when a model needs its head size: it reports through
// return codes (kUnit...), which the dispatcher turns into messages.
constexpr int kUnitTooManyTiles = 1;
constexpr int kUnitBadRotation = 2;
constexpr int kUnitBadPartition = 3;
constexpr int kUnitTooManyArrivals = 4;
constexpr int kUnitBadWalk = 5;
constexpr int kUnitLaunchFailed = 1000;       // + the hipError_t
#define RLIS_UNIT_LAUNCH_CHECK()                                 \
  do {                                                           \
    hipError_t e_ = hipGetLastError();                           \
    if (e_ != hipSuccess) return kUnitLaunchFailed + (int)e_;    \
  } while (0)

#define RLIS_CAT2(a, b) a##b
#define RLIS_CAT(a, b) RLIS_CAT2(a, b)
#define KERNEL_NAME RLIS_CAT(rlis_attn_prefill_mfma_kernel_d, RLIS_HEAD_DIM)

namespace {

constexpr int D = RLIS_HEAD_DIM;
// Keys per tile: 64 up to head size 128, 32 beyond; with two query blocks per wave the
// accumulators take twice the registers, and 32 keys per tile keep the staging and score
// registers within what three (head size up to 64) or two waves per SIMD can have.
__host__ __device__ constexpr int tile_keys(int QB) {
  return (D > 128 || QB == 2) ? 32 : 64;
}
// LDS row strides.  A 16-byte read of a wave is served in four cycles, sixteen lanes each
// (lanes 0-3, 12-15, 20-27 in the first, 4-11, 16-19, 28-31 in the second, and the same
// plus 32), and a cycle is free of bank conflicts when its sixteen 16-byte pieces fall on
// sixteen different quarters of the 64 banks.  For 16 rows read at every second row (the K
// tile, see below) that holds with a row stride of 16 bytes mod 32; for 16 consecutive rows
// (the V^T tile) with a stride of 32 bytes mod 64.
constexpr int KS = D + 8;     // K tile row stride (bf16 elements)
constexpr int BM = 64;       // queries per workgroup and query block
// Two LDS tiles taking turns (one barrier per tile instead of two) where that does not cost a
// resident workgroup.
__host__ __device__ constexpr int tile_bufs(int QB) {
  return (D <= 64 || (QB == 2 && D <= 128)) ? 2 : 1;
}

}  // namespace

// Up to three waves per SIMD (two with two query blocks): the staging registers must not be
// traded for another.
// BIAS: a bias on the scores, slopes[head] * (key position - query position) added in float32
// before the softmax (the reference has none; a position encoding of another kind has).  A form
// of its own, so that the usual one pays nothing for it.
template <int QB, bool BIAS = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu((QB == 1 && D <= 64) ? 4 : 1, QB == 1 ? (D <= 64 ? 4 : 3) : (D <= 64 ? 3 : 2)))) void KERNEL_NAME(
    const bf16_t* __restrict__ q, long long q_stride, bf16_t* __restrict__ out,
    long long out_stride, const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ cu_seqlens,
    const int* __restrict__ start_pos, const int* __restrict__ unit_map, int nh, int nkv, int d,
    int page_shift, float scale, int window, int num_tiles, int tiles_per_round, int part_stride,
    int row0, float* __restrict__ part_ml, float* __restrict__ part_acc,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const float* __restrict__ slopes) {
  constexpr int BN = tile_keys(QB);
  // V^T tile rows: 64 keys padded to a stride of 32 bytes mod 64; 32 keys unpadded, with the
  // 16-byte piece index XORed with (-(row / 4)) & 3, which frees reads and stores of conflicts.
  constexpr int VS = BN == 32 ? 32 : BN + 16;
  constexpr int kTileBufs = tile_bufs(QB);
  __shared__ __attribute__((aligned(16))) bf16_t Ks_all[kTileBufs * BN * KS];
  __shared__ __attribute__((aligned(16))) bf16_t Vs_all[kTileBufs * D * VS];

  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int l16 = lane % 16, lq = lane / 16;
  // Blocks are numbered heads-fastest over the units of work, which arrive sorted by falling
  // work.  One round of blocks (tiles_per_round units x all heads) fills the compute units once;
  // every other round walks its units backwards, so that a compute unit that drew a long one in
  // one round draws a short one in the next.
  // A unit is (sequence, first new-token index of the tile, run, runs of this sequence): with
  // more than one run the keys of a tile are cut into that many runs of whole key tiles, one
  // workgroup each, so that few tiles with long walks over cached keys still fill the chip.
  // Such workgroups store unnormalised sums with their maximum and denominator, which
  // attn_reduce (attention.hip) merges.  How many runs a sequence has is decided from its own
  // lengths, never from what else is in the batch.
  const int h = blockIdx.x % nh;
  int tile = blockIdx.x / nh;
  if (tiles_per_round > 0) {
    const int round = tile / tiles_per_round, within = tile % tiles_per_round;
    const bool whole = (round + 1) * tiles_per_round <= num_tiles;
    if ((round & 1) && whole) tile = round * tiles_per_round + (tiles_per_round - 1 - within);
  }
  const int seq = unit_map[4 * tile], qb = unit_map[4 * tile + 1];
  const int split = unit_map[4 * tile + 2], splits = unit_map[4 * tile + 3];
  const int tok_begin = cu_seqlens[seq];
  const int n_new = cu_seqlens[seq + 1] - tok_begin;
  const int P = start_pos[seq];
  const int kvh = h / (nh / nkv);
  const int* table = block_tables + (long long)seq * max_pages;
  const int page_mask = (1 << page_shift) - 1;

  // This lane's queries: new-token indices qb + wave * 16 QB + b * 16 + l16, one per block b.
  // Their fragments serve as the B operand (column l16) of S^T = K Q^T.
  const int wave_q_first = qb + wave * 16 * QB;
  int my_qi[QB], my_qpos[QB];
  Frag8 qf[QB][D / 32];
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    my_qi[b] = wave_q_first + b * 16 + l16;
    my_qpos[b] = P + my_qi[b];
#pragma unroll
    for (int ks = 0; ks < D / 32; ++ks) {
      const int dim = ks * 32 + lq * 8;
      if (my_qi[b] < n_new && dim < d)
        qf[b][ks].u = *(const uint4*)(q + (long long)(tok_begin + my_qi[b]) * q_stride + h * d + dim);
      else
        qf[b][ks].u = make_uint4(0, 0, 0, 0);
    }
  }
  // With cos_t the queries arrive unrotated, and the kernel turns them by their positions as
  // rope_kv_write would have turned them in place (the dispatcher: rot == d == D, a multiple
  // of 64).  The angles are asked for here, with the queries (a query past the end takes the
  // last one's: it is zero anyway), and used once the first tiles' loads are on their way.
  constexpr int QHS = D % 64 == 0 ? D / 64 : 1;
  float q_cos[QB][QHS][8], q_sin[QB][QHS][8];
  if constexpr (D % 64 == 0) {
    if (cos_t != nullptr) {
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        const long long row = (long long)(P + min(my_qi[b], n_new - 1)) * (D / 2);
#pragma unroll
        for (int ks = 0; ks < QHS; ++ks) {
          const float* cs = cos_t + row + ks * 32 + lq * 8;
          const float* sn = sin_t + row + ks * 32 + lq * 8;
          *(float4*)&q_cos[b][ks][0] = *(const float4*)cs;
          *(float4*)&q_cos[b][ks][4] = *(const float4*)(cs + 4);
          *(float4*)&q_sin[b][ks][0] = *(const float4*)sn;
          *(float4*)&q_sin[b][ks][4] = *(const float4*)(sn + 4);
        }
      }
    }
  }

  float m_run[QB], l_run[QB];
  f32x4 o_acc[QB][D / 16];  // O^T: rows are dims db * 16 + lq * 4 + r, the column is this query
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    m_run[b] = -INFINITY;
    l_run[b] = 0.f;
#pragma unroll
    for (int db = 0; db < D / 16; ++db) o_acc[b][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  const int q_last = min(n_new, qb + BM * QB) - 1;      // last new-token index of the tile
  const int khi_all = P + q_last + 1;                    // keys [klo, khi_all) matter to the tile
  int klo = 0;
  if (window > 0) klo = max(0, P + qb - window + 1);
  const int kt0_all = (klo / BN) * BN;
  int kt0 = kt0_all, khi = khi_all;                      // this workgroup's run of them
  if (splits > 1) {
    const int per = ((khi_all - kt0_all + BN - 1) / BN + splits - 1) / splits;
    kt0 = kt0_all + split * per * BN;
    khi = min(khi_all, kt0 + per * BN);
  }
  const int wave_q_last = min(n_new - 1, wave_q_first + 16 * QB - 1);

  // Staging for the tiles to come.  A tile's page ids are fetched four tiles ahead of its use,
  // its keys and values two tiles ahead (two register sets taking turns), so that neither the
  // table lookup nor the loads themselves are waited for.  The loads are unconditional, so
  // that the compiler can count them: a key past the end of the range reads its place in the
  // last page of the range (its score is masked), a dim past d reads dim d - 8 (it meets a
  // zero of q, or a row of O^T that is not stored).  Keys and values past the end are whatever
  // the page holds: the pages start as zeros and only ever hold what a model wrote, and their
  // probabilities are exactly zero.
  constexpr int K_CHUNKS = BN * (D / 8);
  constexpr int KCH = (K_CHUNKS + 255) / 256;
  constexpr int V_CHUNKS = D * (BN / 8);     // rows past d receive copies of the last chunk
  constexpr int VCH = (V_CHUNKS + 255) / 256;
  const int v_chunks = d * (BN / 8);
  int k_key[KCH], k_dim[KCH], v_key[VCH], v_dim[VCH];   // this thread's chunks within a tile
#pragma unroll
  for (int i = 0; i < KCH; ++i) {
    const int c = min(tid + i * 256, K_CHUNKS - 1);
    k_key[i] = c / (D / 8);
    k_dim[i] = min((c % (D / 8)) * 8, d - 8);
  }
#pragma unroll
  for (int i = 0; i < VCH; ++i) {
    const int c = min(tid + i * 256, v_chunks - 1);
    v_dim[i] = c / (BN / 8);
    v_key[i] = (c % (BN / 8)) * 8;
  }
  // Addresses.  Tiles start at multiples of their size and pages are powers of two, so the
  // page of a chunk is (k0 >> page_shift) + a constant of the thread, and its place inside the
  // page is a constant of the thread plus (k0 & page_mask), which is zero unless pages are
  // larger than tiles: what changes from tile to tile is uniform over the workgroup.  The page
  // index is clamped to the last page of the range; 64 bits are needed only for page id times
  // the elements of a page.
  const int last_page = (khi - 1) >> page_shift;
  const unsigned page_elems = ((unsigned)nkv << page_shift) * (unsigned)d;
  int k_pg[KCH], v_pg[VCH];
  unsigned k_in[KCH], v_in[VCH];
#pragma unroll
  for (int i = 0; i < KCH; ++i) {
    k_pg[i] = k_key[i] >> page_shift;
    k_in[i] = (((unsigned)kvh << page_shift) + (unsigned)(k_key[i] & page_mask)) * (unsigned)d + k_dim[i];
  }
#pragma unroll
  for (int i = 0; i < VCH; ++i) {
    v_pg[i] = v_key[i] >> page_shift;
    v_in[i] = (((unsigned)(kvh * d + v_dim[i])) << page_shift) + (unsigned)(v_key[i] & page_mask);
  }
  // Two sets of staging registers (A, B) and of page ids; plain arrays and macros, so that they
  // stay in registers.
  u32x4 tile_ka[KCH], tile_va[VCH], tile_kb[KCH], tile_vb[VCH];
  int page_ka[KCH], page_va[VCH], page_kb[KCH], page_vb[VCH];
#define RLIS_LOAD_PAGES(k0_, PK, PV)                                                           \
  {                                                                                            \
    const int pg0_ = (k0_) >> page_shift;                                                      \
    _Pragma("unroll") for (int i = 0; i < KCH; ++i) PK[i] = table[(unsigned)min(pg0_ + k_pg[i], last_page)]; \
    _Pragma("unroll") for (int i = 0; i < VCH; ++i) PV[i] = table[(unsigned)min(pg0_ + v_pg[i], last_page)]; \
  }
#define RLIS_LOAD_TILE(k0_, PK, PV, TK, TV)                                                    \
  {                                                                                            \
    const unsigned off0_ = (unsigned)((k0_) & page_mask);                                      \
    const unsigned koff0_ = off0_ * (unsigned)d;                                               \
    _Pragma("unroll") for (int i = 0; i < KCH; ++i)                                            \
        TK[i] = *(const u32x4*)(k_pages + ((unsigned long long)(unsigned)PK[i] * page_elems +  \
                                           (k_in[i] + koff0_)));                               \
    _Pragma("unroll") for (int i = 0; i < VCH; ++i)                                            \
        TV[i] = *(const u32x4*)(v_pages + ((unsigned long long)(unsigned)PV[i] * page_elems +  \
                                           (v_in[i] + off0_)));                                \
  }
#define RLIS_STORE_TILE(TK, TV, buf_)                                                          \
  {                                                                                            \
    bf16_t* Ks = Ks_all + (buf_) * (BN * KS);                                                  \
    bf16_t* Vs = Vs_all + (buf_) * (D * VS);                                                   \
    _Pragma("unroll") for (int i = 0; i < KCH; ++i) {                                          \
      const int c_ = tid + i * 256;                                                            \
      if (K_CHUNKS % 256 == 0 || c_ < K_CHUNKS)                                                \
        *(u32x4*)(Ks + (c_ / (D / 8)) * KS + (c_ % (D / 8)) * 8) = TK[i];                      \
    }                                                                                          \
    _Pragma("unroll") for (int i = 0; i < VCH; ++i) {                                          \
      const int c_ = tid + i * 256;                                                            \
      if (V_CHUNKS % 256 == 0 || c_ < V_CHUNKS)                                                \
        *(u32x4*)(Vs + (c_ / (BN / 8)) * VS +                                                  \
                  ((c_ % (BN / 8)) ^ (BN == 32 ? ((0 - ((c_ / (BN / 8)) >> 2)) & 3) : 0)) * 8) = TV[i]; \
    }                                                                                          \
  }

  const float scale2 = scale * 1.4426950408889634f;      // scores in the base-2 domain
  // With a bias the scores are brought to the base-2 domain as soon as they are formed
  // (score * scale2 + slope2 * distance), and maximum and exponent take them as they are.
  const float slope2 = BIAS ? slopes[h] * 1.4426950408889634f : 0.f;
  const float in_exp = BIAS ? 1.f : scale2;
  if (kt0 < khi) {           // else this run has no keys (only with splits)
  RLIS_LOAD_PAGES(kt0, page_ka, page_va);
  RLIS_LOAD_PAGES(kt0 + BN, page_kb, page_vb);
  RLIS_LOAD_TILE(kt0, page_ka, page_va, tile_ka, tile_va);
  RLIS_LOAD_TILE(kt0 + BN, page_kb, page_vb, tile_kb, tile_vb);
  RLIS_LOAD_PAGES(kt0 + 2 * BN, page_ka, page_va);
  RLIS_LOAD_PAGES(kt0 + 3 * BN, page_kb, page_vb);
  RLIS_STORE_TILE(tile_ka, tile_va, 0);
  RLIS_LOAD_TILE(kt0 + 2 * BN, page_ka, page_va, tile_ka, tile_va);
  RLIS_LOAD_PAGES(kt0 + 4 * BN, page_ka, page_va);
  // The unrotated queries are turned by the angles asked for above (rotate-half over the
  // whole head): dim j of a lane's fragment ks meets dim j + D / 2 in its fragment ks + D / 64.
  // Here, behind the first tiles' loads, nothing is waited for that has not arrived anyway.
  if constexpr (D % 64 == 0) {
    if (cos_t != nullptr) {
#pragma unroll
      for (int b = 0; b < QB; ++b) {
#pragma unroll
        for (int ks = 0; ks < QHS; ++ks) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float x1 = (float)qf[b][ks].v[e], x2 = (float)qf[b][ks + QHS].v[e];
            qf[b][ks].v[e] = (__bf16)(x1 * q_cos[b][ks][e] - x2 * q_sin[b][ks][e]);
            qf[b][ks + QHS].v[e] = (__bf16)(x2 * q_cos[b][ks][e] + x1 * q_sin[b][ks][e]);
          }
        }
      }
    }
  }
  __syncthreads();
  // The arithmetic of one tile, which LDS holds.
  auto compute = [&](int k0, int buf) __attribute__((always_inline)) {
    const bf16_t* Ks = Ks_all + buf * (BN * KS);
    const bf16_t* Vs = Vs_all + buf * (D * VS);

    // Tiles wholly after this wave's last query contribute nothing to it.
    const bool wave_active = (wave_q_first < n_new) && (k0 <= P + wave_q_last);
    if (wave_active) {
      // ---- S^T = K Q^T for query l16.  Blocks 2 st and 2 st + 1 share the 32 keys from
      // k0 + 32 st on: row i of the even block is key 2 i of them, row i of the odd block
      // key 2 i + 1, so that the eight scores a lane holds of the pair (rows lq * 4 + r) are
      // the eight consecutive keys lq * 8 ... + 7, which is what one 16-byte read of a V^T
      // row delivers for the second product.
      f32x4 s[QB][BN / 16];
#pragma unroll
      for (int nb = 0; nb < BN / 16; ++nb) {
#pragma unroll
        for (int b = 0; b < QB; ++b) s[b][nb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < D / 32; ++ks) {
          Frag8 kf;
          kf.u = *(const uint4*)(Ks + ((nb / 2) * 32 + 2 * l16 + (nb % 2)) * KS + ks * 32 + lq * 8);
#pragma unroll
          for (int b = 0; b < QB; ++b)
            s[b][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qf[b][ks].v, s[b][nb], 0, 0, 0);
        }
      }
      if constexpr (BIAS) {
#pragma unroll
        for (int b = 0; b < QB; ++b)
#pragma unroll
          for (int nb = 0; nb < BN / 16; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int kpos = k0 + (nb / 2) * 32 + lq * 8 + 2 * r + (nb % 2);
              s[b][nb][r] = fmaf(s[b][nb][r], scale2, slope2 * (float)(kpos - my_qpos[b]));
            }
      }
      // ---- scale, mask (only where a tile meets the diagonal, the window or the end) -----
      const bool plain_tile = (k0 + BN - 1 <= P + wave_q_first) &&
                              (window <= 0 || k0 > P + wave_q_first + 16 * QB - 1 - window);
      // The scale (positive) is applied inside the exponent, with one fused multiply-add per
      // score; the maximum is taken over the raw scores and scaled once.
      bool moved = false;
      float corr[QB];
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        float mx = -INFINITY;
        if (plain_tile) {
#pragma unroll
          for (int nb = 0; nb < BN / 16; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[b][nb][r]);
        } else {
#pragma unroll
          for (int nb = 0; nb < BN / 16; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int kpos = k0 + (nb / 2) * 32 + lq * 8 + 2 * r + (nb % 2);
              const bool ok = (kpos <= my_qpos[b]) && (window <= 0 || kpos > my_qpos[b] - window);
              const float sv = ok ? s[b][nb][r] : -INFINITY;
              s[b][nb][r] = sv;
              mx = fmaxf(mx, sv);
            }
        }
        mx = xor32_max(xor16_max(mx));
        const float m_new = fmaxf(m_run[b], mx * in_exp);          // -inf stays -inf
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;   // a query with no key yet
        corr[b] = __builtin_amdgcn_exp2f(m_run[b] - m_safe);       // 0 when m_run is -inf
        float sum = 0.f;
#pragma unroll
        for (int nb = 0; nb < BN / 16; ++nb)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float p = __builtin_amdgcn_exp2f(fmaf(s[b][nb][r], in_exp, -m_safe));  // exp2(-inf) = 0
            s[b][nb][r] = p;
            sum += p;
          }
        // The denominator stays a partial sum per lane (the four lanes of a query share its
        // maximum, hence corr); the lanes are added once, after the last tile.
        l_run[b] = l_run[b] * corr[b] + sum;
        m_run[b] = m_new;
        moved = moved || corr[b] != 1.0f;
      }
      // The accumulators need rescaling only when some query's maximum moved.
      if (__any(moved)) {
#pragma unroll
        for (int b = 0; b < QB; ++b)
#pragma unroll
          for (int db = 0; db < D / 16; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) o_acc[b][db][r] *= corr[b];
      }
      // ---- O^T += V^T P^T: P^T fragments come straight from the registers ----------------
#pragma unroll
      for (int st = 0; st < BN / 32; ++st) {
        bf16x8 pf[QB];
#pragma unroll
        for (int b = 0; b < QB; ++b)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            pf[b][2 * j] = (__bf16)s[b][2 * st][j];
            pf[b][2 * j + 1] = (__bf16)s[b][2 * st + 1][j];
          }
#pragma unroll
        for (int db = 0; db < D / 16; ++db) {
          // Unconditional, so that reads and products of all blocks can overlap: rows of V^T
          // past d hold whatever LDS held and feed rows of O^T that are never stored.
          Frag8 vf;
          vf.u = *(const uint4*)(Vs + (db * 16 + l16) * VS + st * 32 +
                                 (lq ^ (BN == 32 ? ((0 - (l16 >> 2)) & 3) : 0)) * 8);
#pragma unroll
          for (int b = 0; b < QB; ++b)
            o_acc[b][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf[b], o_acc[b][db], 0, 0, 0);
        }
      }
    }
  };
  // On entry of the step for tile k0: LDS holds tile k0; the `next` registers hold tile k0 + BN
  // and the other set tile k0 + 2 BN (in flight); the `next` page ids are those of tile
  // k0 + 3 BN, the other set's those of tile k0 + 4 BN.  The next tile goes to LDS (after the
  // arithmetic and a barrier with one LDS tile; before the arithmetic, into the other tile,
  // with two) and its registers take tile k0 + 3 BN, whose page ids arrived long since.
#define RLIS_STEP(k0_, PK, PV, TK, TV, cur_)          \
  {                                                   \
    if (kTileBufs == 2) {                             \
      if ((k0_) + BN < khi) RLIS_STORE_TILE(TK, TV, 1 - (cur_)); \
      RLIS_LOAD_TILE((k0_) + 3 * BN, PK, PV, TK, TV); \
      RLIS_LOAD_PAGES((k0_) + 5 * BN, PK, PV);        \
      compute(k0_, cur_);                             \
      __syncthreads();                                \
    } else {                                          \
      compute(k0_, 0);                                \
      __syncthreads();                                \
      if ((k0_) + BN < khi) {                         \
        RLIS_STORE_TILE(TK, TV, 0);                   \
        __syncthreads();                              \
      }                                               \
      RLIS_LOAD_TILE((k0_) + 3 * BN, PK, PV, TK, TV); \
      RLIS_LOAD_PAGES((k0_) + 5 * BN, PK, PV);        \
    }                                                 \
  }
  for (int k0 = kt0; k0 < khi; k0 += 2 * BN) {
    RLIS_STEP(k0, page_kb, page_vb, tile_kb, tile_vb, 0);
    if (k0 + BN < khi) RLIS_STEP(k0 + BN, page_ka, page_va, tile_ka, tile_va, 1);
  }
#undef RLIS_STEP
#undef RLIS_STORE_TILE
#undef RLIS_LOAD_TILE
#undef RLIS_LOAD_PAGES
  }

  // ---- normalise and store: this lane holds dims db * 16 + lq * 4 + [0, 4) of its queries --
#pragma unroll
  for (int b = 0; b < QB; ++b) l_run[b] = xor32_sum(xor16_sum(l_run[b]));
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    if (my_qi[b] < n_new) {
      const long long row = tok_begin + my_qi[b];
      if (splits == 1) {
        const float inv_l = 1.0f / l_run[b];
        bf16_t* orow = out + row * out_stride + h * d;
#pragma unroll
        for (int db = 0; db < D / 16; ++db) {
          const int dim = db * 16 + lq * 4;
          if (dim < d) {
            union { uint2 u; bf16_t e[4]; } o;
#pragma unroll
            for (int r = 0; r < 4; ++r) o.e[r] = f32_to_bf16(o_acc[b][db][r] * inv_l);
            *(uint2*)(orow + dim) = o.u;
          }
        }
      } else {
        const long long idx = ((row - row0) * nh + h) * part_stride + split;
        float* arow = part_acc + idx * d;
#pragma unroll
        for (int db = 0; db < D / 16; ++db) {
          const int dim = db * 16 + lq * 4;
          if (dim < d)
            *(float4*)(arow + dim) = make_float4(o_acc[b][db][0], o_acc[b][db][1],
                                                 o_acc[b][db][2], o_acc[b][db][3]);
        }
        if (lq == 0) {
          // attn_reduce works with natural-log maxima: m * ln 2 (-inf, with a denominator of
          // zero, where the query sees no key of this run)
          part_ml[idx * 2] = m_run[b] * 0.6931471805599453f;
          part_ml[idx * 2 + 1] = l_run[b];
        }
      }
    }
  }
}

// unit_map holds num_units quadruples (sequence, first new-token index of a tile of
// tile_queries = 64 or 128 tokens, run, runs of the sequence), sorted by falling number of keys
// the unit walks.  Units of sequences with more than one run store partial results, part_stride
// of them per (row, head), from row0 on.
RLIS_API int RLIS_CAT(rlis_attn_prefill_mfma_d, RLIS_HEAD_DIM)(
    const void* q, long long q_stride, void* out, long long out_stride, const void* k_pages,
    const void* v_pages, const int* block_tables, int max_pages, const int* cu_seqlens,
    const int* start_pos, const int* tile_map, int num_tiles, int nh, int nkv, int d,
    int page_shift, int window, float scale, int tile_queries, int splits, int row0,
    float* part_ml, float* part_acc, const float* cos, const float* sin, int rot,
    const float* slopes, hipStream_t stream) {
  if (num_tiles == 0) return 0;
  // rotation inside the kernel needs head_dim = rotated width = 64, 128 or 256
  if (cos && !(sin && D % 64 == 0 && rot == D && d == D)) return kUnitBadRotation;
  const long long blocks = (long long)num_tiles * nh;
  if (blocks >= (1ll << 31)) return kUnitTooManyTiles;
  // 256 compute units: a round is the units whose blocks fill them once.
  const int tiles_per_round = (nh <= 256 && 256 % nh == 0) ? 256 / nh : 0;
#define RLIS_PREFILL_LAUNCH(QB, BIAS)                                                            \
  KERNEL_NAME<QB, BIAS><<<(int)blocks, 256, 0, stream>>>(                                        \
      (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pages,              \
      (const bf16_t*)v_pages, block_tables, max_pages, cu_seqlens, start_pos, tile_map, nh, nkv, \
      d, page_shift, scale, window, num_tiles, tiles_per_round, splits, row0, part_ml, part_acc, \
      cos, sin, slopes)
  if (tile_queries == 2 * BM) {
    if (slopes) RLIS_PREFILL_LAUNCH(2, true);
    else RLIS_PREFILL_LAUNCH(2, false);
  } else {
    if (slopes) RLIS_PREFILL_LAUNCH(1, true);
    else RLIS_PREFILL_LAUNCH(1, false);
  }
#undef RLIS_PREFILL_LAUNCH
  RLIS_UNIT_LAUNCH_CHECK();
  return 0;
}

// ===================================================================== decode kernel
// One query token per sequence.  A workgroup serves one (KV head, sequence, partition): its
// eight waves walk the partition in chunks of 32 keys (wave w takes chunks w, w + 8, ...) and
// are merged at the end; partitions are merged by attn_reduce (attention.hip).  The g query
// heads of the KV head take the place of the 16 queries of the prefill kernel: column l % 16
// of S^T = K Q^T and O^T = V^T P^T is head l % 16 of the group (columns beyond g are zero
// queries, never stored).  Nothing goes through LDS on the way in: lanes load K rows and V^T
// rows from the pages directly in operand layout, 16 keys x 64 bytes and 16 dims x 32 bytes per
// instruction, the next chunk while the current one is computed.
//
// Partitions are laid over key positions aligned to 32: with lo the first visible key and
// lo32 = lo rounded down to 32, partition s covers [lo32 + s * part, lo32 + (s + 1) * part)
// cut to [lo, ctx), part = decode_part_len(ctx - lo32, part_keys, max_parts): a function of the
// sequence's own length and of constants, so that a sequence is cut the same way whatever else
// is in the batch.  `splits` is the grid's depth and the stride of the partial results, at
// least the live partitions of the longest sequence; partitions beyond a sequence's own store an
// empty result.  Page ids of a chunk are fetched one chunk ahead of its keys and values, which
// are fetched one chunk ahead of use.
//
// How the keys are cut into partitions fixes the arithmetic (which sums are formed and in which
// order they meet); how many workgroups share them does not.  With cap > 1 (merging inside
// only) a sequence's partitions are dealt out evenly to `groups` workgroups, or to as many more
// as it takes for none to get more than `cap`, each taking its share in a row: at the end of a
// partition its waves park their sums in LDS, each by itself, and start the next from nothing;
// after the last key the workgroup merges the waves of every partition as a workgroup of its
// own would have, and treats the results as it would treat those of other workgroups.
// Every float is the one that a workgroup per partition gives; the caller picks `groups` by how
// many workgroups fill the chip (a full batch needs no help from partitions, and every
// workgroup costs three round trips to memory before its first key and a hand-over after its
// last) and `cap` by what the LDS holds.
//
// With rope.positions the kernel also does what rope_kv_write does for the step's own tokens
// (crates/model/src/llama.rs:205-222): every workgroup rotates its queries in registers
// (rotate-half over the whole head, which must be as wide as this unit: the partner of a dim
// is then in the same lane), and the workgroup whose partition holds the new key rotates it
// and stores it and the new value to the pages before it reads them back.
#define DECODE_KERNEL_NAME RLIS_CAT(rlis_attn_decode_mfma_kernel_d, RLIS_HEAD_DIM)

namespace {
__device__ __forceinline__ void load8f(const float* p, float (&v)[8]) {
  const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
}  // namespace

constexpr int kDecodeWaves = 8;

// Arrival counts of the partitions of one (sequence, KV head), for merging inside the kernel,
// live in the caller's memory (DecodeMerge): zero before a launch, and set back to zero by the
// workgroup that merges, so the next launch finds zeros.
constexpr int kMergeAhead = 8;           // partitions whose results the merge loads at once

// Partial results pass between workgroups of one launch, which may run on different compute
// dies, each with a cache of its own between it and memory.  They are therefore stored and
// loaded as device-scope atomics (relaxed): such a store goes through to where every die sees
// it, and has arrived there once the wave's store counter has drained (which is what the
// barrier in front of the arrival count waits for); such a load does not take a stale line.
// That keeps the whole-cache write-backs and invalidations of device-scope fences out of the
// kernel: 256 workgroups fencing cost more than the second kernel they were to save.
// a * b rounded to float32 by itself: the empty statement hides the product from the compiler,
// which would otherwise fuse it with an addition behind it.
__device__ __forceinline__ float rounded_product(float a, float b) {
  float p = a * b;
  asm volatile("" : "+v"(p));
  return p;
}
__device__ __forceinline__ void store_shared_result(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_shared_result(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Up to head size 64 two workgroups share a compute unit (four waves per SIMD, 128 registers
// each): the bound keeps the compiler from taking the few registers more that would halve that.
// WALKS: the form in which a workgroup may take several partitions (cap > 1); the other form
// is spared what that costs in registers.  EXACT: the head is as wide as the unit, a page holds
// 16 positions and there is no window, the usual case: with that known to the compiler the
// offsets of a lane's loads within a key's row and a value's page become constants of the
// instructions (30 fewer registers at head size 128, a tenth fewer instructions in the chunk
// loop), and no key is masked for lying in front of a window.
constexpr int kExactPageShift = 4;
// BIAS: slopes[head] * (key position - the token's position) is added to every score, as in
// the prefill kernel (a form of its own, in the general shape of the kernel only).
template <bool WALKS, bool EXACT, bool BIAS = false>
__global__ __launch_bounds__(512, RLIS_HEAD_DIM <= 64 ? 4 : 2) void DECODE_KERNEL_NAME(
    const bf16_t* __restrict__ q, long long q_stride, bf16_t* __restrict__ out,
    long long out_stride, float* __restrict__ part_ml, float* __restrict__ part_acc,
    const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ ctx_lens,
    int nh, int nkv, int d, int page_shift, float scale, int window, int splits, int part_keys,
    int max_parts, int merge_inside, int groups, int cap, const DecodeRope rope,
    const DecodeMerge merge, const float* __restrict__ slopes) {
  if constexpr (EXACT) {
    d = D;
    page_shift = kExactPageShift;
    window = 0;
  }
  // per partition that the workgroup walks: ml waves * g * 2, then acc waves * g * d
  extern __shared__ float dsm[];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int l16 = lane % 16, lq = lane / 16;
  const int kvh = blockIdx.x, seq = blockIdx.y, split = blockIdx.z;
  const int g = nh / nkv;
  // ---- first round trip to memory: what depends on the workgroup's place alone ---------
  // The context length, the token's position and slot, the raw q rows, and this KV head's new
  // key and value (element tid of each, with the key's rotation partner; d is at most 256, the
  // workgroup has 512 threads) are all asked for before anything is waited for.
  const bool rotates = rope.positions != nullptr;
  const bool stores_kv = rotates && rope.slots != nullptr;
  // None of these loads sits under a condition: a load in a branch makes the compiler wait,
  // where the branches meet, for everything asked for so far.  What is not wanted is read from
  // a place that is there anyway and dropped.
  const int ctx = ctx_lens[seq];
  const int pos_read = (rotates ? rope.positions : ctx_lens)[seq];
  const int slot_read = (stores_kv ? rope.slots : ctx_lens)[seq];
  const int pos = rotates ? pos_read : 0;
  const int slot = stores_kv ? slot_read : -1;
  Frag8 qf[D / 32];
#pragma unroll
  for (int ks = 0; ks < D / 32; ++ks) {
    const int dim = ks * 32 + lq * 8;
    const bool ok = l16 < g && dim < d;
    const uint4 v = *(const uint4*)(q + (long long)seq * q_stride + (ok ? (kvh * g + l16) * d + dim : 0));
    qf[ks].u = make_uint4(ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u);
  }
  const int half = rope.rot / 2;
  const bool kv_thread = stores_kv && tid < d;
  const bool k_turns = kv_thread && rope.cos && tid < rope.rot;
  // (without a cache write the same elements of the q row stand in)
  const int kv_i = min(tid, d - 1);
  const int partner_i = kv_i < half ? kv_i + half : max(kv_i - half, 0);
  const bf16_t* krow = q + (long long)seq * q_stride + (stores_kv ? rope.k_off : 0) + kvh * d;
  const bf16_t* vrow = q + (long long)seq * q_stride + (stores_kv ? rope.v_off : 0) + kvh * d;
  const bf16_t new_k = krow[kv_i], new_v = vrow[kv_i], new_partner = krow[min(partner_i, d - 1)];

  // ---- what follows from the context length ---------------------------------------------
  const int* table = block_tables + (long long)seq * max_pages;
  const int page_mask = (1 << page_shift) - 1;
  const int lo = (window > 0 && ctx - window > 0) ? ctx - window : 0;
  const int lo32 = lo & ~31;
  constexpr int kStride = 32 * kDecodeWaves;       // keys between two chunks of one wave
  const int part = decode_part_len(ctx - lo32, part_keys, max_parts);   // a multiple of kStride
  // Merging inside: only the partitions that hold keys of this sequence run, and the last of
  // them to finish merges them all; a sequence with one such partition stores its result itself.
  const int own = merge_inside ? max(1, min(splits, (ctx - lo32 + part - 1) / part)) : splits;
  // This workgroup's partitions: first .. first + mine, one of `sharers` even shares.
  int sharers = own, first = split, mine = 1;
  if constexpr (WALKS) {
    sharers = min(own, max(groups, (own + cap - 1) / cap));
    first = split * own / sharers;
    mine = (split + 1) * own / sharers - first;
  }
  if (split >= sharers) return;
  const int kbeg = lo32 + first * part;
  const int kend = min(ctx, kbeg + mine * part);

  // A wave takes its chunks two at a time: the page ids of both, then all their keys and
  // values, are on their way before the first product, and the page ids of the next two follow
  // at once.  The loads are unconditional, so that the compiler can count them: a key past the
  // end of the partition reads the last key in it instead (its score is masked, its
  // probability exactly zero; values past the end inside a group of 4 keys are whatever the
  // page holds, and the pages only ever hold zeros or values that a model wrote); a dim past d
  // reads one below d (it meets a zero of q, or a row of O^T that is not stored).
  const int last_key = max(kend - 1, 0), last_quad = last_key & ~3;
  int k_dim[D / 32], v_dim[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 32; ++ks) k_dim[ks] = min(ks * 32 + lq * 8, d - 8);
#pragma unroll
  for (int db = 0; db < D / 16; ++db) v_dim[db] = min(db * 16 + l16, d - 1);
  Frag8 k_a[2][D / 32], v_a[D / 16], k_b[2][D / 32], v_b[D / 16];
  int pk_a[2], pv_a[2], pk_b[2], pv_b[2];
  // Addresses: 64 bits only for page id times the elements of a page (keys are never negative,
  // so the clamp is a minimum alone).
  const unsigned page_elems = ((unsigned)nkv << page_shift) * (unsigned)d;
  const unsigned k_head = ((unsigned)kvh << page_shift) * (unsigned)d;
  const unsigned v_head = ((unsigned)(kvh * d)) << page_shift;
#define RLIS_DEC_PAGES(c0_, PK, PV)                                                             \
  {                                                                                             \
    _Pragma("unroll") for (int i = 0; i < 2; ++i) {                                             \
      PK[i] = table[min((c0_) + i * 16 + l16, last_key) >> page_shift];                         \
      PV[i] = table[min((c0_) + i * 16 + lq * 4, last_quad) >> page_shift];                     \
    }                                                                                           \
  }
#define RLIS_DEC_CHUNK(c0_, PK, PV, KF, VF)                                                     \
  {                                                                                             \
    _Pragma("unroll") for (int nb = 0; nb < 2; ++nb) {                                          \
      const unsigned off_ = (unsigned)(min((c0_) + nb * 16 + l16, last_key) & page_mask);       \
      const bf16_t* kp_ = k_pages + ((unsigned long long)(unsigned)PK[nb] * page_elems +        \
                                     (k_head + off_ * (unsigned)d));                            \
      _Pragma("unroll") for (int ks = 0; ks < D / 32; ++ks)                                     \
          KF[nb][ks].u = *(const uint4*)(kp_ + k_dim[ks]);                                      \
    }                                                                                           \
    _Pragma("unroll") for (int hf = 0; hf < 2; ++hf) {                                          \
      const unsigned off_ = (unsigned)(min((c0_) + hf * 16 + lq * 4, last_quad) & page_mask);   \
      const bf16_t* vp_ = v_pages + ((unsigned long long)(unsigned)PV[hf] * page_elems +        \
                                     (v_head + off_));                                          \
      _Pragma("unroll") for (int db = 0; db < D / 16; ++db)                                     \
          VF[db].h[hf] = *(const uint2*)(vp_ + ((unsigned)v_dim[db] << page_shift));            \
    }                                                                                           \
  }

  // ---- second round trip: the page ids of this wave's first chunks and the rotation's
  // angles, which need the context length and the position ------------------------------
  int c0 = kbeg + wave * 32;
  constexpr bool kPairs = D <= 128;      // wider heads have no registers for two chunks
  const bool one_by_one = part <= kStride || !kPairs;
  RLIS_DEC_PAGES(c0, pk_a, pv_a);
  if constexpr (kPairs) {
    // (clamped loads: harmless where a wave has one chunk only, and no branch around loads)
    RLIS_DEC_PAGES(c0 + kStride, pk_b, pv_b);
  }
  // The angles, again without a branch: where nothing is rotated the q row itself (D / 2
  // floats are D bf16 elements of it) is read instead and dropped.
  constexpr int HS = D % 64 == 0 ? D / 64 : 1;     // fragments between a dim and its partner
  const bool q_turns = D % 64 == 0 && rotates && rope.cos;   // the dispatcher: rot == d == D
  const float* no_angles = (const float*)(q + (long long)seq * q_stride);
  float q_cos[HS][8], q_sin[HS][8];
  if constexpr (D % 64 == 0) {
    const float* cs = q_turns ? rope.cos + (long long)pos * (D / 2) : no_angles;
    const float* sn = q_turns ? rope.sin + (long long)pos * (D / 2) : no_angles;
#pragma unroll
    for (int ks = 0; ks < HS; ++ks) {
      load8f(cs + ks * 32 + lq * 8, q_cos[ks]);
      load8f(sn + ks * 32 + lq * 8, q_sin[ks]);
    }
  }
  const bool k_angles = stores_kv && rope.cos && half > 0;
  const int k_j = min(kv_i < half ? kv_i : kv_i - half, max(half - 1, 0));
  const float k_cos_read = (k_angles ? rope.cos + (long long)pos * half + k_j : no_angles)[0];
  const float k_sin_read = (k_angles ? rope.sin + (long long)pos * half + k_j : no_angles)[0];
  const float k_cos = k_turns ? k_cos_read : 1.f, k_sin = k_turns ? k_sin_read : 0.f;

  // ---- the step's own key and value go to the pages before anyone reads them back --------
  if (stores_kv && kbeg < ctx && kend == ctx) {
    // This workgroup's partition ends with the step's own key.
    if (slot >= 0 && kv_thread) {
      const long long page = slot >> page_shift;
      const int off = slot & page_mask;
      bf16_t* kdst = const_cast<bf16_t*>(k_pages) + (((page * nkv + kvh) << page_shift) + off) * d;
      bf16_t* vdst = const_cast<bf16_t*>(v_pages) + (((page * nkv + kvh) * d) << page_shift) + off;
      bf16_t kv = new_k;
      if (k_turns) {
        const float x = bf16_to_f32(new_k), y = bf16_to_f32(new_partner);
        kv = f32_to_bf16(tid < half ? x * k_cos - y * k_sin : x * k_cos + y * k_sin);
      }
      kdst[tid] = kv;
      vdst[(long long)tid << page_shift] = new_v;
    }
    __syncthreads();       // the stores are visible to the whole workgroup from here on
  }

  if constexpr (D % 64 == 0) {
    if (q_turns) {
#pragma unroll
      for (int ks = 0; ks < HS; ++ks) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float x1 = (float)qf[ks].v[e], x2 = (float)qf[ks + HS].v[e];
          qf[ks].v[e] = (__bf16)(x1 * q_cos[ks][e] - x2 * q_sin[ks][e]);
          qf[ks + HS].v[e] = (__bf16)(x2 * q_cos[ks][e] + x1 * q_sin[ks][e]);
        }
      }
    }
  }
  float m_run = -INFINITY, l_run = 0.f;
  f32x4 o_acc[D / 16];
#pragma unroll
  for (int db = 0; db < D / 16; ++db) o_acc[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const float scale2 = scale * 1.4426950408889634f;
  // (with a bias the scores go to the base-2 domain as they are formed, see the prefill kernel)
  const float slope2 = BIAS ? slopes[kvh * g + min(l16, g - 1)] * 1.4426950408889634f : 0.f;
  const float in_exp = BIAS ? 1.f : scale2;

  auto compute = [&](int c0, const Frag8 (&kf)[2][D / 32], const Frag8 (&vf)[D / 16])
                     __attribute__((always_inline)) {
    f32x4 s[2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      s[nb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < D / 32; ++ks)
        s[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[nb][ks].v, qf[ks].v, s[nb], 0, 0, 0);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int key = c0 + nb * 16 + lq * 4 + r;
        if constexpr (BIAS) s[nb][r] = fmaf(s[nb][r], scale2, slope2 * (float)(key - (ctx - 1)));
        const float sv = (key >= lo && key < kend) ? s[nb][r] : -INFINITY;
        s[nb][r] = sv;
        mx = fmaxf(mx, sv);
      }
    mx = xor32_max(xor16_max(mx));
    const float m_new = fmaxf(m_run, mx * in_exp);    // in_exp > 0; -inf stays -inf
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float corr = __builtin_amdgcn_exp2f(m_run - m_safe);
    float sum = 0.f;
    bf16x8 pf;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s[nb][r], in_exp, -m_safe));
        sum += p;
        pf[nb * 4 + r] = (__bf16)p;
      }
    l_run = l_run * corr + sum;        // per lane; the four lanes of a head are added at the end
    m_run = m_new;
#pragma unroll
    for (int db = 0; db < D / 16; ++db) {   // blocks past d: rows of O^T that are never stored
#pragma unroll
      for (int r = 0; r < 4; ++r) o_acc[db][r] *= corr;
      o_acc[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[db].v, pf, o_acc[db], 0, 0, 0);
    }
  };

  // ---- the end of a partition: every wave parks its sums in LDS ----------------------
  // One region per partition that the workgroup walks: [wave][head][2] maxima and
  // denominators, then [wave][head][d] sums.  A wave parks and goes on by itself: nothing is
  // merged, and no wave waits for another, before the workgroup's last key.
  const int region_floats = kDecodeWaves * g * (2 + d);
  constexpr float kLn2 = 0.6931471805599453f;       // attn_reduce works with natural-log maxima
  auto park = [&](int n) __attribute__((always_inline)) {
    float* ml_s = dsm + (WALKS ? n * region_floats : 0);
    const float l_all = xor32_sum(xor16_sum(l_run));
    if (l16 < g) {
      if (lq == 0) {
        ml_s[(wave * g + l16) * 2] = m_run;
        ml_s[(wave * g + l16) * 2 + 1] = l_all;
      }
      // this lane's dims lq * 4 + r of every block of 16, of its head's row
      float* row = ml_s + kDecodeWaves * g * 2 + (wave * g + l16) * d + lq * 4;
#pragma unroll
      for (int db = 0; db < D / 16; ++db)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (db * 16 + lq * 4 + r < d) row[db * 16 + r] = o_acc[db][r];
    }
  };
  // Partition n, dim j of head hh, over the parked waves in wave order: the sum, the base-2
  // maximum and the denominator.
  auto merged = [&](int n, int hh, int j, float& a, float& big, float& lsum)
                    __attribute__((always_inline)) {
    const float* ml_s = dsm + (WALKS ? n * region_floats : 0);
    const float* acc_s = ml_s + kDecodeWaves * g * 2;
    // Without branches, so that all the reads are issued together: a wave that saw no key has
    // maximum -inf, weight 0 (selected, since -inf - -inf is no number) and sums of zeros.
    float mw[kDecodeWaves], lw[kDecodeWaves], aw[kDecodeWaves];
    big = -INFINITY;
#pragma unroll
    for (int w = 0; w < kDecodeWaves; ++w) {
      mw[w] = ml_s[(w * g + hh) * 2];
      lw[w] = ml_s[(w * g + hh) * 2 + 1];
      aw[w] = acc_s[(w * g + hh) * d + j];
      big = fmaxf(big, mw[w]);
    }
    lsum = 0.f;
    a = 0.f;
#pragma unroll
    for (int w = 0; w < kDecodeWaves; ++w) {
      const float e = (mw[w] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mw[w] - big);
      lsum += lw[w] * e;
      a += aw[w] * e;
    }
  };

  // The chunks of one partition after the other (a walked partition is a multiple of two
  // chunks per wave: the caller sees to it).  The page ids asked for in a partition's last
  // round are those of the next one's first chunks, so nothing starts anew at the seam: the
  // wave parks what it has and goes on from nothing.
  int kept = 0;
  int stop = (WALKS && mine > 1) ? kbeg + part : kend;      // where the partition at hand ends
  for (;;) {
    if (one_by_one) {
      // One chunk at a time: at most one for every wave of the workgroup, or a wide head.
      for (; c0 < stop; c0 += kStride) {
        RLIS_DEC_CHUNK(c0, pk_a, pv_a, k_a, v_a);
        RLIS_DEC_PAGES(c0 + kStride, pk_a, pv_a);
        compute(c0, k_a, v_a);
      }
    } else if constexpr (kPairs) {
      for (; c0 < stop; c0 += 2 * kStride) {
        RLIS_DEC_CHUNK(c0, pk_a, pv_a, k_a, v_a);
        RLIS_DEC_CHUNK(c0 + kStride, pk_b, pv_b, k_b, v_b);
        RLIS_DEC_PAGES(c0 + 2 * kStride, pk_a, pv_a);
        RLIS_DEC_PAGES(c0 + 3 * kStride, pk_b, pv_b);
        compute(c0, k_a, v_a);
        if (c0 + kStride < kend) compute(c0 + kStride, k_b, v_b);
      }
    }
    if (!WALKS || stop >= kend) break;
    park(kept);
    ++kept;
    stop = min(stop + part, kend);
    m_run = -INFINITY;
    l_run = 0.f;
#pragma unroll
    for (int db = 0; db < D / 16; ++db) o_acc[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
#undef RLIS_DEC_CHUNK
#undef RLIS_DEC_PAGES

  // ---- the workgroup's last key: merge the waves of every partition, then store ---------
  park(kept);                    // kept = mine - 1
  __syncthreads();
  for (int i = tid; i < g * d; i += 64 * kDecodeWaves) {
    const int hh = i / d, j = i % d;
    const int h = kvh * g + hh;
    float a, big, lsum;
    if (!WALKS || mine == 1) {
      // one partition: the sequence's only one, or one to hand over
      merged(0, hh, j, a, big, lsum);
      if (own == 1) {
        out[(long long)seq * out_stride + h * d + j] = f32_to_bf16(a / lsum);
      } else {
        const long long idx = ((long long)seq * nh + h) * splits + first;
        store_shared_result(part_acc + idx * d + j, a);
        if (j == 0) {
          store_shared_result(part_ml + idx * 2, rounded_product(big, kLn2));
          store_shared_result(part_ml + idx * 2 + 1, lsum);
        }
      }
    } else if (mine == own) {
      // All partitions of the sequence were this workgroup's: it merges them as the last to
      // arrive merges those of other workgroups (below), the same sums in the same order.
      // (the maximum times ln 2 is rounded by itself, as on its way through memory: no fused
      // multiply-add with the subtraction behind it)
      float top = -INFINITY;
      for (int n = 0; n < mine; ++n) {
        merged(n, hh, j, a, big, lsum);
        if (lsum > 0.f) top = fmaxf(top, rounded_product(big, kLn2));
      }
      float l_all = 0.f, a_all = 0.f;
      for (int n = 0; n < mine; ++n) {
        merged(n, hh, j, a, big, lsum);
        const float e = lsum > 0.f ? expf(rounded_product(big, kLn2) - top) : 0.f;
        if (e > 0.f) {
          l_all += lsum * e;
          a_all += a * e;
        }
      }
      out[(long long)seq * out_stride + h * d + j] = f32_to_bf16(a_all / l_all);
    } else {
      const long long idx = ((long long)seq * nh + h) * splits + first;
      for (int n = 0; n < mine; ++n) {
        merged(n, hh, j, a, big, lsum);
        store_shared_result(part_acc + (idx + n) * d + j, a);
        if (j == 0) {
          store_shared_result(part_ml + (idx + n) * 2, rounded_product(big, kLn2));
          store_shared_result(part_ml + (idx + n) * 2 + 1, lsum);
        }
      }
    }
  }
  if (!merge_inside || own == 1 || mine == own) return;

  // ---- the last partition of (sequence, KV head) to arrive merges them all -------------
  // Every thread's stores have arrived before it passes the barrier; thread 0 then counts this
  // workgroup in.  The sums run over the partitions in order, with the arithmetic of
  // attn_reduce_kernel, so the result does not depend on which workgroup came last.
  __shared__ int merges;
  __builtin_amdgcn_s_waitcnt(0);         // all counters at zero: this wave's stores have arrived
  __syncthreads();
  if (tid == 0) {
    unsigned* slot = merge.arrivals + (seq * nkv + kvh);
    const bool last = __hip_atomic_fetch_add(slot, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
                      (unsigned)(sharers - 1);
    if (last) __hip_atomic_store(slot, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    merges = last;
  }
  __syncthreads();
  if (!merges) return;
  for (int i = tid; i < g * d; i += 64 * kDecodeWaves) {
    const int hh = i / d, j = i % d;
    const int h = kvh * g + hh;
    const long long base = ((long long)seq * nh + h) * splits;
    // The first kMergeAhead partitions are loaded at once (a partition past the sequence's own
    // reads its last one and counts as empty), any further ones one after the other.
    float mv[kMergeAhead], lv[kMergeAhead], av[kMergeAhead];
#pragma unroll
    for (int s = 0; s < kMergeAhead; ++s) {
      const long long idx = base + min(s, own - 1);
      mv[s] = load_shared_result(part_ml + idx * 2);
      lv[s] = load_shared_result(part_ml + idx * 2 + 1);
      av[s] = load_shared_result(part_acc + idx * d + j);
    }
    float big = -INFINITY;
#pragma unroll
    for (int s = 0; s < kMergeAhead; ++s) {
      if (s >= own) lv[s] = 0.f;
      if (lv[s] > 0.f) big = fmaxf(big, mv[s]);
    }
    for (int s = kMergeAhead; s < own; ++s) {
      const float m = load_shared_result(part_ml + (base + s) * 2);
      const float l = load_shared_result(part_ml + (base + s) * 2 + 1);
      if (l > 0.f) big = fmaxf(big, m);
    }
    float lsum = 0.f, a = 0.f;
#pragma unroll
    for (int s = 0; s < kMergeAhead; ++s) {
      const float e = lv[s] > 0.f ? expf(mv[s] - big) : 0.f;
      if (e > 0.f) {
        lsum += lv[s] * e;
        a += av[s] * e;
      }
    }
    for (int s = kMergeAhead; s < own; ++s) {
      const float m = load_shared_result(part_ml + (base + s) * 2);
      const float l = load_shared_result(part_ml + (base + s) * 2 + 1);
      const float v = load_shared_result(part_acc + (base + s) * d + j);
      const float e = l > 0.f ? expf(m - big) : 0.f;
      if (e > 0.f) {
        lsum += l * e;
        a += v * e;
      }
    }
    out[(long long)seq * out_stride + h * d + j] = f32_to_bf16(a / lsum);
  }
}

RLIS_API int RLIS_CAT(rlis_attn_decode_mfma_d, RLIS_HEAD_DIM)(
    const void* q, long long q_stride, void* out, long long out_stride, float* part_ml,
    float* part_acc, const void* k_pages, const void* v_pages, const int* block_tables,
    int max_pages, const int* ctx_lens, int S, int nh, int nkv, int d, int page_shift, int window,
    float scale, int splits, int part_keys, int max_parts, int merge_inside, int groups, int cap,
    const DecodeRope* rope, const DecodeMerge* merge, const float* slopes, hipStream_t stream) {
  if (S == 0) return 0;
  if (part_keys % (32 * kDecodeWaves) != 0 || part_keys <= 0) return kUnitBadPartition;
  if (merge_inside && (!merge->arrivals || (long long)S * nkv > merge->slots))
    return kUnitTooManyArrivals;
  const int g = nh / nkv;
  const size_t smem = (size_t)(cap < 1 ? 1 : cap) * kDecodeWaves * g * (2 + d) * sizeof(float);
  // several partitions per workgroup: merging inside, whole pairs of chunks, and parked sums
  // that fit the LDS (up to head size 64 two workgroups share a compute unit's 160 KB)
  constexpr size_t kWalkBytes = D <= 64 ? 64 * 1024 : 159 * 1024;
  if (cap < 1 || groups < 1 || (cap > 1 && (!merge_inside || part_keys % (64 * kDecodeWaves) != 0 ||
                                            smem > kWalkBytes)))
    return kUnitBadWalk;
  if (smem > 64 * 1024) {
    // more dynamic LDS than a kernel gets unasked: asked for once on every device
    constexpr int kDevices = 64;
    static bool granted[kDevices];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return kUnitLaunchFailed + (int)e;
    if (dev < 0 || dev >= kDevices || !granted[dev]) {
      const void* forms[] = {reinterpret_cast<const void*>(&DECODE_KERNEL_NAME<true, false>),
                             reinterpret_cast<const void*>(&DECODE_KERNEL_NAME<true, true>),
                             reinterpret_cast<const void*>(&DECODE_KERNEL_NAME<true, false, true>)};
      for (const void* form : forms) {
        e = hipFuncSetAttribute(form, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kWalkBytes);
        if (e != hipSuccess) return kUnitLaunchFailed + (int)e;
      }
      if (dev >= 0 && dev < kDevices) granted[dev] = true;
    }
  }
  // rotation inside the kernel needs head_dim = rotated width = 64, 128 or 256
  if (rope->positions && rope->cos && !(D % 64 == 0 && rope->rot == D && d == D))
    return kUnitBadRotation;
  // deep enough for the sequence with the most partitions, whichever rule binds for it
  const int by_cap = (splits + cap - 1) / cap;
  dim3 grid(nkv, S, cap > 1 ? (groups > by_cap ? (groups < splits ? groups : splits) : by_cap)
                            : splits);
#define RLIS_DEC_LAUNCH(WALKS, EXACT, BIAS)                                                       \
  DECODE_KERNEL_NAME<WALKS, EXACT, BIAS><<<grid, 64 * kDecodeWaves, smem, stream>>>(             \
      (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, part_ml, part_acc,                   \
      (const bf16_t*)k_pages, (const bf16_t*)v_pages, block_tables, max_pages, ctx_lens, nh, nkv, \
      d, page_shift, scale, window, splits, part_keys, max_parts, merge_inside, groups, cap,   \
      *rope, *merge, slopes)
  const bool exact = d == D && page_shift == kExactPageShift && window <= 0;
  if (slopes && cap > 1) RLIS_DEC_LAUNCH(true, false, true);
  else if (slopes) RLIS_DEC_LAUNCH(false, false, true);
  else if (cap > 1 && exact) RLIS_DEC_LAUNCH(true, true, false);
  else if (cap > 1) RLIS_DEC_LAUNCH(true, false, false);
  else if (exact) RLIS_DEC_LAUNCH(false, true, false);
  else RLIS_DEC_LAUNCH(false, false, false);
#undef RLIS_DEC_LAUNCH
  RLIS_UNIT_LAUNCH_CHECK();
  return 0;
}
