// Plain bf16 matrix products of many rows (prompt portions, decode steps of more than 64 requests) handed to
// hipBLASLt, as the reference hands its products to cuBLASLt (v3/crates/rvllm-cutlass/src/cublaslt.rs:184-277:
// one descriptor set and one chosen algorithm per shape, a workspace the caller owns).
//
//   out[M, N] (bf16, or 32-bit with out_f32: logits; row stride ldc) = x[M, K] (row stride ldx) * w[N, K]^T (row
//   stride ldw), x and w in bf16, sums in 32 bits.
//
// The library counts in columns: the row-major out[M, N] is its column-major [N, M], so the call is
// D(N x M) = op_T(A = w as K x N) * (B = x as K x M).
//
// Every shape (M, N, K and the three strides) keeps its descriptors and its algorithm once made: a call is then
// one hipblasLtMatmul, which is what a step of a few hundred launches can afford on the host (through a general
// tensor library's product each call cost 19 us of host time, more than the GPU took for it).  The algorithm is
// the library's first suggestion unless the shape has been tuned: rv_lt_tune times every algorithm that the
// library has for the types and that takes the shape (hipblaslt_ext::getAllAlgos, matmulIsAlgoSupported) on the
// caller's operands and keeps the fastest; a shape that was never tuned runs on the algorithm of its tuned neighbour
// in rows (borrow_from_a_neighbour); tuned choices can be listed (rv_lt_tuned_plan) and taken back by their index
// (rv_lt_take_plan), which is how a file of them survives the process.  Nothing here allocates device memory: the
// workspace is the caller's.  Calls are serialised by one lock; calls that overlap on a device share the caller's
// workspace, so they belong on one stream.
#include <hipblaslt/hipblaslt-ext.hpp>
#include <hipblaslt/hipblaslt.h>

#include <algorithm>
#include <cstdio>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "common.h"

namespace {

struct LtShape {
  int dev, M, N, K;
  long long ldx, ldw, ldc;
  int out_f32;  // the result is stored in 32 bits (logits) instead of bf16
  bool operator<(const LtShape& o) const {
    return std::tie(dev, M, N, K, ldx, ldw, ldc, out_f32) < std::tie(o.dev, o.M, o.N, o.K, o.ldx, o.ldw, o.ldc, o.out_f32);
  }
};

struct LtPlan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, d = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
  bool tuned = false;
  bool none = false;  // the library has no algorithm for this shape: asked once, remembered
  int borrowed_rows = 0;  // > 0: the algorithm is the one a tuned shape of that many rows and the same matrix runs on
  long long looked_round = 0;  // g_tuned_round when this shape last looked for a tuned neighbour
  int algo_index = -1;
  float tuned_us = 0.f;
};

std::mutex g_lock;
std::map<int, hipblasLtHandle_t> g_handles;  // by device
std::map<LtShape, LtPlan> g_plans;
long long g_tuned_round = 1;  // goes up whenever a shape becomes tuned: untuned shapes then look at their neighbours again

const char* status_name(hipblasStatus_t s) {
  switch (s) {
    case HIPBLAS_STATUS_SUCCESS: return "success";
    case HIPBLAS_STATUS_NOT_INITIALIZED: return "not initialized";
    case HIPBLAS_STATUS_ALLOC_FAILED: return "allocation failed";
    case HIPBLAS_STATUS_INVALID_VALUE: return "invalid value";
    case HIPBLAS_STATUS_ARCH_MISMATCH: return "architecture mismatch";
    case HIPBLAS_STATUS_EXECUTION_FAILED: return "execution failed";
    case HIPBLAS_STATUS_NOT_SUPPORTED: return "not supported";
    default: return "error";
  }
}

#define LT_CHECK(call, what)                                                                     \
  do {                                                                                           \
    hipblasStatus_t s_ = (call);                                                                 \
    if (s_ != HIPBLAS_STATUS_SUCCESS) return rv_fail("library product: %s: %s", what, status_name(s_)); \
  } while (0)

int handle_for(int dev, hipblasLtHandle_t* out) {
  auto it = g_handles.find(dev);
  if (it == g_handles.end()) {
    hipblasLtHandle_t h = nullptr;
    LT_CHECK(hipblasLtCreate(&h), "hipblasLtCreate");
    it = g_handles.emplace(dev, h).first;
  }
  *out = it->second;
  return 0;
}

// A shape that was never tuned takes the algorithm of the tuned shape nearest in rows (at most RV_LT_NEIGHBOUR
// times more or fewer) with the same matrix (columns, depth, its row stride), if the library says that the algorithm
// takes this shape too: the steps of an engine bring every number of rows, and tuning can only have met a few.
// What the library suggests first for a shape is often a fifth slower than what tuning finds for its neighbour.
#define RV_LT_NEIGHBOUR 1.5
void borrow_from_a_neighbour(hipblasLtHandle_t handle, const LtShape& shape, size_t workspace_bytes, LtPlan& plan) {
  const LtPlan* nearest = nullptr;
  int nearest_rows = 0;
  double nearest_ratio = RV_LT_NEIGHBOUR;
  for (const auto& kv : g_plans) {
    const LtShape& o = kv.first;
    if (o.dev != shape.dev || o.N != shape.N || o.K != shape.K || o.ldw != shape.ldw || o.out_f32 != shape.out_f32) continue;
    if (!kv.second.tuned || kv.second.none) continue;
    const double ratio = o.M > shape.M ? (double)o.M / shape.M : (double)shape.M / o.M;
    if (ratio <= nearest_ratio) nearest = &kv.second, nearest_rows = o.M, nearest_ratio = ratio;
  }
  if (!nearest) return;
  hipblasLtMatmulAlgo_t algo = nearest->algo;
  const float one = 1.f, zero = 0.f;
  size_t room = 0;
  if (hipblaslt_ext::matmulIsAlgoSupported(handle, plan.desc, &one, plan.a, plan.b, &zero, plan.d, plan.d, algo, room) !=
          HIPBLAS_STATUS_SUCCESS ||
      room > workspace_bytes)
    return;
  plan.algo = algo;
  plan.workspace = room;
  plan.algo_index = hipblaslt_ext::getIndexFromAlgo(algo);
  plan.borrowed_rows = nearest_rows;
}
// ... when it has not looked since the last shape was tuned
void look_for_a_neighbour(hipblasLtHandle_t handle, const LtShape& shape, size_t workspace_bytes, LtPlan& plan) {
  if (plan.tuned || plan.none || plan.looked_round == g_tuned_round) return;
  plan.looked_round = g_tuned_round;
  borrow_from_a_neighbour(handle, shape, workspace_bytes, plan);
}

// The plan of a shape, made at its first sight with the library's first suggestion, or with a tuned neighbour's
// algorithm.  g_lock is held.
int plan_for(hipblasLtHandle_t handle, const LtShape& shape, size_t workspace_bytes, LtPlan** out) {
  auto it = g_plans.find(shape);
  if (it != g_plans.end()) {
    look_for_a_neighbour(handle, shape, workspace_bytes, it->second);
    *out = &it->second;
    return 0;
  }
  // what has been created is given back if the plan is not kept (an error on the way)
  struct Making {
    LtPlan plan;
    bool kept = false;
    ~Making() {
      if (kept) return;
      if (plan.a) hipblasLtMatrixLayoutDestroy(plan.a);
      if (plan.b) hipblasLtMatrixLayoutDestroy(plan.b);
      if (plan.d) hipblasLtMatrixLayoutDestroy(plan.d);
      if (plan.desc) hipblasLtMatmulDescDestroy(plan.desc);
    }
  } making;
  LtPlan& plan = making.plan;
  LT_CHECK(hipblasLtMatmulDescCreate(&plan.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F), "hipblasLtMatmulDescCreate");
  const hipblasOperation_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
  LT_CHECK(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof(op_t)), "transpose of w");
  LT_CHECK(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n)), "transpose of x");
  // as stored (before the transposition): w is K x N in columns, x is K x M, out is N x M
  LT_CHECK(hipblasLtMatrixLayoutCreate(&plan.a, HIP_R_16BF, shape.K, shape.N, shape.ldw), "layout of w");
  LT_CHECK(hipblasLtMatrixLayoutCreate(&plan.b, HIP_R_16BF, shape.K, shape.M, shape.ldx), "layout of x");
  LT_CHECK(hipblasLtMatrixLayoutCreate(&plan.d, shape.out_f32 ? HIP_R_32F : HIP_R_16BF, shape.N, shape.M, shape.ldc),
           "layout of out");
  hipblasLtMatmulPreference_t pref = nullptr;
  LT_CHECK(hipblasLtMatmulPreferenceCreate(&pref), "hipblasLtMatmulPreferenceCreate");
  const uint64_t room = workspace_bytes;
  hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &room, sizeof(room));
  hipblasLtMatmulHeuristicResult_t first[1];
  int found = 0;
  const hipblasStatus_t s =
      hipblasLtMatmulAlgoGetHeuristic(handle, plan.desc, plan.a, plan.b, plan.d, plan.d, pref, 1, first, &found);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (s != HIPBLAS_STATUS_SUCCESS || found < 1) {
    plan.none = true;
  } else {
    plan.algo = first[0].algo;
    plan.workspace = first[0].workspaceSize;
    plan.algo_index = hipblaslt_ext::getIndexFromAlgo(plan.algo);
  }
  look_for_a_neighbour(handle, shape, workspace_bytes, plan);
  *out = &g_plans.emplace(shape, plan).first->second;
  making.kept = true;
  return 0;
}

int check_operands(const void* x, const void* w, void* out, int M, int N, int K, long long ldx, long long ldw,
                   long long ldc) {
  RV_CHECK(M > 0 && N > 0 && K > 0 && x && w && out, "library product: bad arguments M=%d N=%d K=%d", M, N, K);
  RV_CHECK(ldx >= K && ldw >= K && ldc >= N, "library product: row strides too small");
  return 0;
}

}  // namespace

// What rv_lt_gemm returns for a shape that the library takes no algorithm for (nothing ran; the caller has another
// kernel for it).
#define RV_LT_NO_ALGORITHM 2
// An algorithm replaces the library's first suggestion only if it is this much faster.
#define RV_LT_CLEARLY 0.03f

// out = x w^T on `stream`; 0, RV_LT_NO_ALGORITHM or -1 (an error); `workspace` (workspace_bytes of device memory, the caller's) is what the algorithm may use.
extern "C" int rv_lt_gemm(hipStream_t stream, const void* x, const void* w, void* out, int M, int N, int K,
                          long long ldx, long long ldw, long long ldc, void* workspace, long long workspace_bytes,
                          int out_f32) {
  if (check_operands(x, w, out, M, N, K, ldx, ldw, ldc)) return -1;
  int dev = 0;
  RV_CHECK(hipGetDevice(&dev) == hipSuccess, "library product: no current device");
  std::lock_guard<std::mutex> guard(g_lock);
  hipblasLtHandle_t handle;
  if (handle_for(dev, &handle)) return -1;
  LtPlan* plan;
  if (plan_for(handle, LtShape{dev, M, N, K, ldx, ldw, ldc, out_f32 != 0}, (size_t)workspace_bytes, &plan)) return -1;
  if (plan->none) {
    rv_fail("library product: the library has no algorithm for M=%d N=%d K=%d (strides %lld %lld %lld)", M, N, K, ldx,
            ldw, ldc);
    return RV_LT_NO_ALGORITHM;
  }
  RV_CHECK(plan->workspace <= (size_t)workspace_bytes && (plan->workspace == 0 || workspace),
           "library product: the algorithm wants %zu bytes of workspace, %lld are there", plan->workspace, workspace_bytes);
  const float one = 1.f, zero = 0.f;
  LT_CHECK(hipblasLtMatmul(handle, plan->desc, &one, w, plan->a, x, plan->b, &zero, out, plan->d, out, plan->d,
                           &plan->algo, workspace, plan->workspace, stream),
           "hipblasLtMatmul");
  return 0;
}

// Times every algorithm the library has for this shape on the given operands (their contents do not matter; `out`
// is overwritten) and keeps the fastest for rv_lt_gemm.  Waits for the device.  Returns the number of algorithms
// timed, or -1; a shape that was tuned before returns 0 at once.  `budget_ms` bounds the time spent.
// `w_others` (num_others of them, may be none): other matrices of the same shape and stride, a model's other layers'.
// The timed calls then take them in turn, so that a call reads its matrix from memory as a step's calls do, layer
// after layer, and not from the cache that the same matrix called over and over would stay in: the algorithm that
// is fastest on a matrix in the cache is not always the one that streams it fastest.
extern "C" int rv_lt_tune(hipStream_t stream, const void* x, const void* w, void* out, int M, int N, int K,
                          long long ldx, long long ldw, long long ldc, void* workspace, long long workspace_bytes,
                          int budget_ms, const void* const* w_others, int num_others, int out_f32) {
  if (check_operands(x, w, out, M, N, K, ldx, ldw, ldc)) return -1;
  int dev = 0;
  RV_CHECK(hipGetDevice(&dev) == hipSuccess, "library product: no current device");
  std::lock_guard<std::mutex> guard(g_lock);
  hipblasLtHandle_t handle;
  if (handle_for(dev, &handle)) return -1;
  LtPlan* plan;
  if (plan_for(handle, LtShape{dev, M, N, K, ldx, ldw, ldc, out_f32 != 0}, (size_t)workspace_bytes, &plan)) return -1;
  if (plan->tuned || plan->none) return 0;
  std::vector<hipblasLtMatmulHeuristicResult_t> all;
  LT_CHECK(hipblaslt_ext::getAllAlgos(handle, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, HIPBLAS_OP_T, HIPBLAS_OP_N,
                                      HIP_R_16BF, HIP_R_16BF, out_f32 ? HIP_R_32F : HIP_R_16BF,
                                      out_f32 ? HIP_R_32F : HIP_R_16BF, HIPBLAS_COMPUTE_32F, all),
           "getAllAlgos");
  const float one = 1.f, zero = 0.f;
  struct Events {
    hipEvent_t t0 = nullptr, t1 = nullptr, begin = nullptr;
    ~Events() {
      if (t0) hipEventDestroy(t0);
      if (t1) hipEventDestroy(t1);
      if (begin) hipEventDestroy(begin);
    }
  } events;
  RV_CHECK(hipEventCreate(&events.t0) == hipSuccess && hipEventCreate(&events.t1) == hipSuccess &&
               hipEventCreate(&events.begin) == hipSuccess,
           "library product: hipEventCreate failed");
  const hipEvent_t t0 = events.t0, t1 = events.t1, begin = events.begin;
  RV_CHECK(num_others >= 0 && (num_others == 0 || w_others), "library product: bad list of other matrices");
  long long turn = 0;
  auto run = [&](hipblasLtMatmulAlgo_t& algo, size_t ws) {
    const void* w_now = num_others > 0 ? w_others[turn++ % num_others] : w;
    return hipblasLtMatmul(handle, plan->desc, &one, w_now, plan->a, x, plan->b, &zero, out, plan->d, out, plan->d,
                           &algo, workspace, ws, stream);
  };
  // the time of `runs` calls in a row, per call (microseconds); negative if a call failed
  auto time_of = [&](hipblasLtMatmulAlgo_t& algo, size_t ws, int runs) -> float {
    if (run(algo, ws) != HIPBLAS_STATUS_SUCCESS) return -1.f;  // a first call apart: it may load the kernel
    hipEventRecord(t0, stream);
    for (int i = 0; i < runs; ++i)
      if (run(algo, ws) != HIPBLAS_STATUS_SUCCESS) return -1.f;
    hipEventRecord(t1, stream);
    if (hipEventSynchronize(t1) != hipSuccess) return -1.f;
    float ms = 0.f;
    hipEventElapsedTime(&ms, t0, t1);
    return ms * 1000.f / runs;
  };
  hipEventRecord(begin, stream);
  int timed = 1;
  // first pass: every algorithm that takes the shape, a few calls each; second pass: the best ones again, longer
  std::vector<std::pair<float, size_t>> ranked;  // (time, place in `all`)
  std::vector<size_t> room(all.size(), 0);
  for (size_t i = 0; i < all.size(); ++i) {
    size_t ws = 0;
    if (hipblaslt_ext::matmulIsAlgoSupported(handle, plan->desc, &one, plan->a, plan->b, &zero, plan->d, plan->d,
                                             all[i].algo, ws) != HIPBLAS_STATUS_SUCCESS)
      continue;
    if (ws > (size_t)workspace_bytes) continue;
    room[i] = ws;
    const float us = time_of(all[i].algo, ws, 3);
    ++timed;
    if (us > 0.f) ranked.emplace_back(us, i);
    hipEventRecord(t1, stream);
    hipEventSynchronize(t1);
    float spent = 0.f;
    hipEventElapsedTime(&spent, begin, t1);
    if (spent > (float)budget_ms) break;
  }
  std::sort(ranked.begin(), ranked.end());
  // The first suggestion stays unless another algorithm beats it clearly: each is timed twice, the suggestion
  // between the others, and the smaller time counts; times of one run differ by a few percent on their own.
  auto twice = [&](hipblasLtMatmulAlgo_t& algo, size_t ws) {
    const float a = time_of(algo, ws, 20), b = time_of(algo, ws, 20);
    return (a > 0.f && b > 0.f) ? std::min(a, b) : -1.f;
  };
  hipblasLtMatmulAlgo_t suggested = plan->algo;
  const size_t suggested_room = plan->workspace;
  float best_us = twice(suggested, suggested_room);
  float to_beat = best_us > 0.f ? best_us * (1.f - RV_LT_CLEARLY) : 0.f;
  for (size_t r = 0; r < ranked.size() && r < 8; ++r) {
    const size_t i = ranked[r].second;
    const float us = twice(all[i].algo, room[i]);
    if (us > 0.f && (best_us <= 0.f || us < to_beat)) {
      best_us = to_beat = us;
      plan->algo = all[i].algo;
      plan->workspace = room[i];
      plan->algo_index = hipblaslt_ext::getIndexFromAlgo(all[i].algo);
    }
  }
  RV_CHECK(best_us > 0.f, "library product: no algorithm ran for M=%d N=%d K=%d", M, N, K);
  plan->tuned = true;
  plan->tuned_us = best_us;
  ++g_tuned_round;
  return timed;
}

// What is kept for a shape: 1 if it has been tuned, 2 if it runs on a tuned neighbour's algorithm, 0 if it runs on the
// library's first suggestion, -1 if it has not been seen; the algorithm's index in the library and the time it was tuned to (microseconds) if asked for.
extern "C" int rv_lt_plan_info(int M, int N, int K, long long ldx, long long ldw, long long ldc, int* algo_index,
                               float* tuned_us, int out_f32) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return -1;
  std::lock_guard<std::mutex> guard(g_lock);
  auto it = g_plans.find(LtShape{dev, M, N, K, ldx, ldw, ldc, out_f32 != 0});
  if (it == g_plans.end()) return -1;
  if (algo_index) *algo_index = it->second.algo_index;
  if (tuned_us) *tuned_us = it->second.tuned_us;
  if (!it->second.tuned && it->second.borrowed_rows > 0) return 2;
  return it->second.tuned ? 1 : 0;
}

// The library's version (its number, as hipblasLtGetVersion gives it): an algorithm's index means something only
// to the version that gave it.  -1 on an error.
extern "C" int rv_lt_version(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return -1;
  std::lock_guard<std::mutex> guard(g_lock);
  hipblasLtHandle_t handle;
  if (handle_for(dev, &handle)) return -1;
  int version = -1;
  if (hipblasLtGetVersion(handle, &version) != HIPBLAS_STATUS_SUCCESS) return -1;
  return version;
}

// What kind of device the current one is, for the file of plans: its architecture's name and its number of compute
// units, as text in `out` (at most `room` bytes with the final 0).  0 or -1.
extern "C" int rv_lt_device_kind(char* out, int room) {
  int dev = 0;
  hipDeviceProp_t prop;
  RV_CHECK(out && room > 0, "library product: no room for the device's kind");
  RV_CHECK(hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess,
           "library product: the current device's properties cannot be read");
  snprintf(out, (size_t)room, "%s/%d", prop.gcnArchName, prop.multiProcessorCount);
  return 0;
}

// The `i`-th tuned shape of the current device, in no particular order: 1 and the shape, its algorithm's index and
// its time; 0 when there are fewer.
extern "C" int rv_lt_tuned_plan(int i, int* M, int* N, int* K, long long* ldx, long long* ldw, long long* ldc,
                                int* algo_index, float* tuned_us, int* out_f32) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  std::lock_guard<std::mutex> guard(g_lock);
  for (const auto& kv : g_plans) {
    if (kv.first.dev != dev || !kv.second.tuned || kv.second.none) continue;
    if (i-- > 0) continue;
    *M = kv.first.M, *N = kv.first.N, *K = kv.first.K;
    *ldx = kv.first.ldx, *ldw = kv.first.ldw, *ldc = kv.first.ldc;
    *algo_index = kv.second.algo_index;
    *tuned_us = kv.second.tuned_us;
    *out_f32 = kv.first.out_f32;
    return 1;
  }
  return 0;
}

// Takes an algorithm that an earlier run of the same library tuned this shape to, by its index, instead of tuning
// again: 0 if it is taken (the shape then counts as tuned), RV_LT_NO_ALGORITHM if the library does not know the index
// or the algorithm does not take the shape (nothing changes: the shape runs on the first suggestion and can be
// tuned), -1 on an error.
extern "C" int rv_lt_take_plan(int M, int N, int K, long long ldx, long long ldw, long long ldc, int algo_index,
                               float tuned_us, long long workspace_bytes, int out_f32) {
  RV_CHECK(M > 0 && N > 0 && K > 0 && ldx >= K && ldw >= K && ldc >= N && algo_index >= 0,
           "library product: bad plan M=%d N=%d K=%d index=%d", M, N, K, algo_index);
  int dev = 0;
  RV_CHECK(hipGetDevice(&dev) == hipSuccess, "library product: no current device");
  std::lock_guard<std::mutex> guard(g_lock);
  hipblasLtHandle_t handle;
  if (handle_for(dev, &handle)) return -1;
  LtPlan* plan;
  if (plan_for(handle, LtShape{dev, M, N, K, ldx, ldw, ldc, out_f32 != 0}, (size_t)workspace_bytes, &plan)) return -1;
  if (plan->tuned) return 0;
  if (plan->none) return RV_LT_NO_ALGORITHM;
  std::vector<int> wanted{algo_index};
  std::vector<hipblasLtMatmulHeuristicResult_t> found;
  if (hipblaslt_ext::getAlgosFromIndex(handle, wanted, found) != HIPBLAS_STATUS_SUCCESS || found.empty())
    return RV_LT_NO_ALGORITHM;
  const float one = 1.f, zero = 0.f;
  size_t room = 0;
  if (hipblaslt_ext::matmulIsAlgoSupported(handle, plan->desc, &one, plan->a, plan->b, &zero, plan->d, plan->d,
                                           found[0].algo, room) != HIPBLAS_STATUS_SUCCESS ||
      room > (size_t)workspace_bytes)
    return RV_LT_NO_ALGORITHM;
  plan->algo = found[0].algo;
  plan->workspace = room;
  plan->algo_index = hipblaslt_ext::getIndexFromAlgo(plan->algo);
  plan->tuned = true;
  plan->tuned_us = tuned_us;
  ++g_tuned_round;
  return 0;
}
