// bfloat16 products with more than 64 rows (and the ones of 17 to 64 rows that do not join the
// residual stream) are the library's: hipBLASLt, called here directly.  The reference uses a
// library matmul for every projection (crates/model/src/layers.rs:30-46, candle's matmul).
//
// Why not through the tensor library's matmul: a step that mixes a portion of a prompt with
// decoding requests launches four products per layer, and 20 us of host time per call (operator
// dispatch, output allocation, a heuristics lookup) against 5 us here decide whether the host
// keeps ahead of the device at 500 tokens a step.
//
// The library is not linked: the process already holds one copy (the tensor library's own),
// and a second copy with its own kernels would answer the same symbols.  rlis_lt_open takes
// the path of the copy to use, opens it and looks the entry points up.  A plan (operation and
// layout descriptors, an algorithm) is made once per shape and kept: the algorithm that the
// library's heuristics rank first, or, when the caller asks for the shape to be tried out
// before its first product (rlis_lt_tune), the fastest of the heuristics' first candidates as
// timed on the spot.  At 33 to 1,024 rows the heuristics' order is erratic (3B shape: q/k/v at
// 256 rows 33 us with the first candidate, 21 us with the sixth; output at 192 rows 27 against
// 17 us; down at 192 rows 60 against 35; 1B shape: q/k/v at 64 rows 12.1 against 9.6 us); at
// 2,048 rows the first is the fastest.  A shape's algorithm never changes once a product has
// used it, so that a step computes the same bits whenever it is run.
#include <dlfcn.h>
#include <hipblaslt/hipblaslt.h>

#include <string.h>

#include <algorithm>
#include <map>
#include <mutex>
#include <tuple>

#include "common.h"

namespace {

struct LtApi {
  void* lib = nullptr;
  decltype(&hipblasLtCreate) create = nullptr;
  decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
  decltype(&hipblasLtMatmulDescSetAttribute) desc_set = nullptr;
  decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
  decltype(&hipblasLtMatrixLayoutSetAttribute) layout_set = nullptr;
  decltype(&hipblasLtMatmulPreferenceCreate) pref_create = nullptr;
  decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set = nullptr;
  decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy = nullptr;
  decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
  decltype(&hipblasLtMatmul) matmul = nullptr;
};

struct LtPlan {
  hipblasLtMatmulDesc_t op = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
};

// (device, T, N, K, ldx, ldw, ldy, float32 result, workspace limit, k slices)
using LtKey = std::tuple<int, int, int, int, long long, long long, long long, int, size_t, int>;

std::mutex lt_mutex;
LtApi lt;
std::map<int, hipblasLtHandle_t> lt_handles;      // per device
std::map<LtKey, LtPlan> lt_plans;

template <typename F>
bool lookup(F& fn, const char* name) {
  fn = (F)dlsym(lt.lib, name);
  return fn != nullptr;
}

}  // namespace

// Opens the copy of hipBLASLt at `path` (the one the process has loaded already, if it has) and
// finds its entry points.  Calling it again is harmless.
RLIS_API int rlis_lt_open(const char* path) {
  std::lock_guard<std::mutex> lock(lt_mutex);
  if (lt.lib) return 0;
  RLIS_REQUIRE(path && *path, "lt_open: no path to the library");
  void* lib = dlopen(path, RTLD_NOW | RTLD_LOCAL | RTLD_NOLOAD);
  if (!lib) lib = dlopen(path, RTLD_NOW | RTLD_LOCAL);
  RLIS_REQUIRE(lib != nullptr, "lt_open: cannot open %s: %s", path, dlerror());
  lt.lib = lib;
  const bool ok = lookup(lt.create, "hipblasLtCreate") &&
                  lookup(lt.desc_create, "hipblasLtMatmulDescCreate") &&
                  lookup(lt.desc_set, "hipblasLtMatmulDescSetAttribute") &&
                  lookup(lt.layout_create, "hipblasLtMatrixLayoutCreate") &&
                  lookup(lt.layout_set, "hipblasLtMatrixLayoutSetAttribute") &&
                  lookup(lt.pref_create, "hipblasLtMatmulPreferenceCreate") &&
                  lookup(lt.pref_set, "hipblasLtMatmulPreferenceSetAttribute") &&
                  lookup(lt.pref_destroy, "hipblasLtMatmulPreferenceDestroy") &&
                  lookup(lt.heuristic, "hipblasLtMatmulAlgoGetHeuristic") &&
                  lookup(lt.matmul, "hipblasLtMatmul");
  if (!ok) {
    lt = LtApi();
    rlis_set_error("lt_open: %s lacks an entry point of hipBLASLt", path);
    return 1;
  }
  return 0;
}

RLIS_API int rlis_lt_is_open() {
  std::lock_guard<std::mutex> lock(lt_mutex);
  return lt.lib != nullptr;
}

// The descriptors of one product (K: the k of one slice) into `made`, and up to `want` of the
// heuristics' candidates whose workspace fits, in the library's order, into `found`.
static int describe(hipblasLtHandle_t handle, LtPlan& made, hipblasLtMatmulHeuristicResult_t* found,
                    int want, int* count, int out_f32, int T, int N, int K, long long ldx,
                    long long ldw, long long ldy, int slices, long long y_stride,
                    size_t workspace_bytes) {
  // Column-major view: y^T (N, T) = W^T-as-stored transposed (N, K) times x-as-stored (K, T).
  const hipDataType out_type = out_f32 ? HIP_R_32F : HIP_R_16BF;
  bool ok = lt.desc_create(&made.op, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS;
  const int32_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
  ok = ok && lt.desc_set(made.op, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && lt.desc_set(made.op, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && lt.layout_create(&made.a, HIP_R_16BF, K, N, ldw) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && lt.layout_create(&made.b, HIP_R_16BF, K, T, ldx) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && lt.layout_create(&made.c, out_type, N, T, ldy) == HIPBLAS_STATUS_SUCCESS;
  if (slices > 1) {
    // slice s: k from s * K on in both operands, its result y_stride further on
    const int32_t batch = slices;
    const int64_t k_step = K, y_step = y_stride;
    for (hipblasLtMatrixLayout_t m : {made.a, made.b, made.c}) {
      ok = ok && lt.layout_set(m, HIPBLASLT_MATRIX_LAYOUT_BATCH_COUNT, &batch, sizeof(batch)) ==
                     HIPBLAS_STATUS_SUCCESS;
      ok = ok && lt.layout_set(m, HIPBLASLT_MATRIX_LAYOUT_STRIDED_BATCH_OFFSET,
                               m == made.c ? &y_step : &k_step, sizeof(int64_t)) ==
                     HIPBLAS_STATUS_SUCCESS;
    }
  }
  RLIS_REQUIRE(ok, "lt_gemm: cannot describe the product T=%d N=%d K=%d", T, N, K);
  hipblasLtMatmulPreference_t pref = nullptr;
  ok = lt.pref_create(&pref) == HIPBLAS_STATUS_SUCCESS;
  const uint64_t limit = workspace_bytes;
  ok = ok && lt.pref_set(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &limit, sizeof(limit)) ==
                 HIPBLAS_STATUS_SUCCESS;
  *count = 0;
  ok = ok && lt.heuristic(handle, made.op, made.a, made.b, made.c, made.c, pref, want, found,
                          count) == HIPBLAS_STATUS_SUCCESS;
  if (pref) lt.pref_destroy(pref);
  RLIS_REQUIRE(ok && *count > 0 && found[0].state == HIPBLAS_STATUS_SUCCESS,
               "lt_gemm: the library has no algorithm for T=%d N=%d K=%d", T, N, K);
  RLIS_REQUIRE(found[0].workspaceSize <= workspace_bytes,
               "lt_gemm: the algorithm wants %zu bytes of workspace, %zu are there",
               found[0].workspaceSize, workspace_bytes);
  return 0;
}

// The device's handle, made at first use (under lt_mutex).
static int handle_of(int device, hipblasLtHandle_t* handle) {
  auto h = lt_handles.find(device);
  if (h == lt_handles.end()) {
    hipblasLtHandle_t made = nullptr;
    RLIS_REQUIRE(lt.create(&made) == HIPBLAS_STATUS_SUCCESS, "lt_gemm: cannot create a handle");
    h = lt_handles.emplace(device, made).first;
  }
  *handle = h->second;
  return 0;
}

// y (T, N) = x (T, K) W^T for W (N, K), all row-major with rows ldx, ldw, ldy elements apart;
// x and W bfloat16, y bfloat16 or float32 (out_f32), float32 accumulation.  `workspace` is
// device memory of workspace_bytes that the caller keeps for these calls (none: 0).
// slices > 1: k is cut into that many equal slices, one batched call, and slice s leaves its
// float32 partial sums at Y + s * y_stride (a stack for a consumer that adds them in order).
static int lt_gemm(const void* X, const void* W, void* Y, int out_f32, int T, int N, int K,
                   long long ldx, long long ldw, long long ldy, int slices, long long y_stride,
                   void* workspace, size_t workspace_bytes, hipStream_t stream) {
  RLIS_REQUIRE(T >= 0 && N > 0 && K > 0 && ldx >= K && ldw >= K && ldy >= N,
               "lt_gemm: bad sizes T=%d N=%d K=%d ldx=%lld ldw=%lld ldy=%lld", T, N, K, ldx, ldw,
               ldy);
  RLIS_REQUIRE(slices >= 1 && K % slices == 0 && (slices == 1 || (out_f32 && y_stride >= (long long)T * ldy)),
               "lt_gemm: %d slices of k=%d with results %lld apart", slices, K, y_stride);
  RLIS_REQUIRE(workspace || workspace_bytes == 0, "lt_gemm: a workspace size without a workspace");
  if (T == 0) return 0;
  const int full_k = K;
  K /= slices;
  int device = 0;
  hipError_t he = hipGetDevice(&device);
  RLIS_REQUIRE(he == hipSuccess, "lt_gemm: %s", hipGetErrorString(he));
  hipblasLtHandle_t handle = nullptr;
  LtPlan plan;
  // One lock from the look-up to the launch: the device's handle is shared by all threads, and
  // the library's launch path is not known to take two calls on one handle at once (two
  // runners on two threads did get wrong products and a failed call that way).  The launch is
  // asynchronous, so what is serialised is the host's part of it.
  std::lock_guard<std::mutex> lock(lt_mutex);
  {
    RLIS_REQUIRE(lt.lib != nullptr, "lt_gemm: the library has not been opened");
    if (handle_of(device, &handle)) return 1;
    const LtKey key(device, T, N, full_k, ldx, ldw, ldy, out_f32 ? 1 : 0, workspace_bytes, slices);
    auto p = lt_plans.find(key);
    if (p == lt_plans.end()) {
      LtPlan made;
      hipblasLtMatmulHeuristicResult_t found;
      int count = 0;
      if (describe(handle, made, &found, 1, &count, out_f32, T, N, K, ldx, ldw, ldy, slices,
                   y_stride, workspace_bytes))
        return 1;
      made.algo = found.algo;
      made.workspace = found.workspaceSize;
      p = lt_plans.emplace(key, made).first;
    }
    plan = p->second;
  }
  const float one = 1.f, zero = 0.f;
  const hipblasStatus_t st =
      lt.matmul(handle, plan.op, &one, W, plan.a, X, plan.b, &zero, Y, plan.c, Y, plan.c,
                &plan.algo, workspace, workspace_bytes, stream);
  RLIS_REQUIRE(st == HIPBLAS_STATUS_SUCCESS, "lt_gemm: the product T=%d N=%d K=%d failed (%d)", T,
               N, K, (int)st);
  return 0;
}

RLIS_API int rlis_lt_gemm_bf16(const void* X, const void* W, void* Y, int out_f32, int T, int N,
                               int K, long long ldx, long long ldw, long long ldy,
                               void* workspace, size_t workspace_bytes, hipStream_t stream) {
  return lt_gemm(X, W, Y, out_f32, T, N, K, ldx, ldw, ldy, 1, 0, workspace, workspace_bytes, stream);
}

// The same product as a stack of `slices` float32 partial sums (slices, T, N), y_stride
// elements apart: one batched call over equal slices of k.
RLIS_API int rlis_lt_gemm_bf16_slices(const void* X, const void* W, float* Y, int T, int N, int K,
                                      long long ldx, long long ldw, long long ldy, int slices,
                                      long long y_stride, void* workspace, size_t workspace_bytes,
                                      hipStream_t stream) {
  return lt_gemm(X, W, Y, 1, T, N, K, ldx, ldw, ldy, slices, y_stride, workspace, workspace_bytes,
                 stream);
}

// Tries the shape out before its first product: the heuristics' first `max_candidates`
// algorithms (at most 16, those whose workspace fits) each compute the product once untimed and
// then `runs` times over every one of the `num_w` weights of that shape in turn (other layers'
// weights, so that no candidate finds the weights in a cache that a step would not find them
// in; 32 products at most); the fastest by the median of its products' times becomes the shape's algorithm if it beats the heuristics' first by more than
// `margin` (a fraction), else the first does.  Y is written by every candidate.  Nothing
// happens when the shape has a plan already (an algorithm in use is never changed) or the
// stream is capturing (*chosen = -1).  *chosen: the index taken; us[0], us[1]: the times of
// the first and of the one taken.  Waits for the stream.
RLIS_API int rlis_lt_tune(const void* X, const void* const* Ws, int num_w, void* Y, int out_f32,
                          int T, int N, int K, long long ldx, long long ldw, long long ldy,
                          int slices, long long y_stride, void* workspace, size_t workspace_bytes,
                          int max_candidates, int runs, float margin, int* chosen, float* us,
                          hipStream_t stream) {
  constexpr int kMost = 16;
  RLIS_REQUIRE(T > 0 && N > 0 && K > 0 && ldx >= K && ldw >= K && ldy >= N && num_w >= 1 && Ws &&
                   chosen && us && runs >= 1,
               "lt_tune: bad arguments T=%d N=%d K=%d", T, N, K);
  RLIS_REQUIRE(slices >= 1 && K % slices == 0 && (slices == 1 || (out_f32 && y_stride >= (long long)T * ldy)),
               "lt_tune: %d slices of k=%d with results %lld apart", slices, K, y_stride);
  RLIS_REQUIRE(workspace || workspace_bytes == 0, "lt_tune: a workspace size without a workspace");
  *chosen = -1;
  us[0] = us[1] = 0.f;
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  hipError_t he = hipStreamIsCapturing(stream, &capturing);
  RLIS_REQUIRE(he == hipSuccess, "lt_tune: %s", hipGetErrorString(he));
  if (capturing != hipStreamCaptureStatusNone) return 0;
  const int full_k = K;
  K /= slices;
  int device = 0;
  he = hipGetDevice(&device);
  RLIS_REQUIRE(he == hipSuccess, "lt_tune: %s", hipGetErrorString(he));
  std::lock_guard<std::mutex> lock(lt_mutex);
  RLIS_REQUIRE(lt.lib != nullptr, "lt_tune: the library has not been opened");
  hipblasLtHandle_t handle = nullptr;
  if (handle_of(device, &handle)) return 1;
  const LtKey key(device, T, N, full_k, ldx, ldw, ldy, out_f32 ? 1 : 0, workspace_bytes, slices);
  if (lt_plans.count(key)) return 0;
  LtPlan made;
  hipblasLtMatmulHeuristicResult_t found[kMost];
  int count = 0;
  const int want = max_candidates < 1 ? 1 : (max_candidates > kMost ? kMost : max_candidates);
  if (describe(handle, made, found, want, &count, out_f32, T, N, K, ldx, ldw, ldy, slices,
               y_stride, workspace_bytes))
    return 1;
  // Every timed product stands between two events of its own, and a candidate's time is the
  // median of its products': what passes between one product's events is the device's time for
  // it, whereas a loop timed from end to end is bound by the host's launches where a product
  // takes less than they do (and then says nothing about the candidates).
  constexpr int kTimed = 32;
  const int timed = runs * num_w < kTimed ? runs * num_w : kTimed;
  hipEvent_t marks[2 * kTimed] = {};
  for (int i = 0; i < 2 * timed; ++i) {
    he = hipEventCreate(&marks[i]);
    if (he != hipSuccess) {
      for (int j = 0; j < i; ++j) (void)hipEventDestroy(marks[j]);
      RLIS_REQUIRE(false, "lt_tune: %s", hipGetErrorString(he));
    }
  }
  const float one = 1.f, zero = 0.f;
  float best = 0.f, first = 0.f;
  int taken = 0;
  for (int c = 0; c < count; ++c) {
    if (found[c].state != HIPBLAS_STATUS_SUCCESS || found[c].workspaceSize > workspace_bytes)
      continue;
    auto product = [&](const void* W) {
      return lt.matmul(handle, made.op, &one, W, made.a, X, made.b, &zero, Y, made.c, Y, made.c,
                       &found[c].algo, workspace, workspace_bytes, stream) == HIPBLAS_STATUS_SUCCESS;
    };
    bool ok = product(Ws[0]);
    for (int i = 0; ok && i < timed; ++i) {
      ok = hipEventRecord(marks[2 * i], stream) == hipSuccess && product(Ws[i % num_w]) &&
           hipEventRecord(marks[2 * i + 1], stream) == hipSuccess;
    }
    ok = ok && hipEventSynchronize(marks[2 * timed - 1]) == hipSuccess;
    float each[kTimed];
    for (int i = 0; ok && i < timed; ++i)
      ok = hipEventElapsedTime(&each[i], marks[2 * i], marks[2 * i + 1]) == hipSuccess;
    if (!ok) {
      (void)hipGetLastError();              // a candidate that cannot run is left out
      (void)hipStreamSynchronize(stream);
      if (c == 0) break;                    // ... but without the first there is no yardstick
      continue;
    }
    std::sort(each, each + timed);
    const float t = each[timed / 2] * 1e3f;
    if (c == 0) first = best = t;
    else if (t < best && t < first * (1.f - margin)) {
      best = t;
      taken = c;
    }
  }
  for (int i = 0; i < 2 * timed; ++i) (void)hipEventDestroy(marks[i]);
  RLIS_REQUIRE(first > 0.f, "lt_tune: the heuristics' first algorithm for T=%d N=%d K=%d did not run",
               T, N, K);
  made.algo = found[taken].algo;
  made.workspace = found[taken].workspaceSize;
  lt_plans.emplace(key, made);
  *chosen = taken;
  us[0] = first;
  us[1] = best;
  return 0;
}

// Gives the shape of T rows the algorithm that the shape of T_like rows has (the same N, K and
// kinds of operands; x rows ldx_like apart there): among the heuristics' first sixteen
// candidates for T, the one that names the same kernel, if there is one; else the heuristics'
// first.  For row counts next to one that has been tried out: the same kernel does as well
// there, and nothing is timed.  Nothing happens when T has a plan already (*taken = -2);
// *taken = -1: T_like has no plan or none of T's candidates is its algorithm (T then takes the
// heuristics' first), else the candidate's index.
RLIS_API int rlis_lt_adopt(int T, int T_like, int out_f32, int N, int K, long long ldx,
                           long long ldx_like, long long ldw, long long ldy, int slices,
                           long long y_stride, size_t workspace_bytes, int* taken) {
  constexpr int kMost = 16;
  RLIS_REQUIRE(T > 0 && T_like > 0 && N > 0 && K > 0 && ldx >= K && ldx_like >= K && ldw >= K &&
                   ldy >= N && slices >= 1 && K % slices == 0 && taken,
               "lt_adopt: bad arguments T=%d like %d N=%d K=%d", T, T_like, N, K);
  *taken = -2;
  const int full_k = K;
  K /= slices;
  int device = 0;
  hipError_t he = hipGetDevice(&device);
  RLIS_REQUIRE(he == hipSuccess, "lt_adopt: %s", hipGetErrorString(he));
  std::lock_guard<std::mutex> lock(lt_mutex);
  RLIS_REQUIRE(lt.lib != nullptr, "lt_adopt: the library has not been opened");
  hipblasLtHandle_t handle = nullptr;
  if (handle_of(device, &handle)) return 1;
  const LtKey key(device, T, N, full_k, ldx, ldw, ldy, out_f32 ? 1 : 0, workspace_bytes, slices);
  if (lt_plans.count(key)) return 0;
  const LtKey like(device, T_like, N, full_k, ldx_like, ldw, ldy, out_f32 ? 1 : 0, workspace_bytes,
                   slices);
  auto model = lt_plans.find(like);
  LtPlan made;
  hipblasLtMatmulHeuristicResult_t found[kMost];
  int count = 0;
  if (describe(handle, made, found, kMost, &count, out_f32, T, N, K, ldx, ldw, ldy, slices,
               y_stride, workspace_bytes))
    return 1;
  int pick = -1;
  if (model != lt_plans.end()) {
    for (int c = 0; c < count && pick < 0; ++c)
      if (found[c].state == HIPBLAS_STATUS_SUCCESS && found[c].workspaceSize <= workspace_bytes &&
          memcmp(found[c].algo.data, model->second.algo.data, sizeof(found[c].algo.data)) == 0)
        pick = c;
  }
  made.algo = found[pick < 0 ? 0 : pick].algo;
  made.workspace = found[pick < 0 ? 0 : pick].workspaceSize;
  lt_plans.emplace(key, made);
  *taken = pick;
  return 0;
}
