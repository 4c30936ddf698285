// The library matrix product for many rows: out[M, N] = x[M, K] . W[N, K]^T through
// hipBLASLt, bfloat16 inputs, 32-bit accumulation (where the reference calls
// torch's nn.Linear: miniserve/model/qwen3.py:174-176, 366-382).
//
// The process has one hipBLASLt already: the one torch loaded, bound to the HIP
// runtime whose streams and pointers arrive here.  This file binds to that same
// copy at run time (ms_gemm_library_open gets its path) instead of linking a second
// one; only the header's types are used at compile time.  Descriptors and the
// chosen algorithm are kept per shape, so a call costs one hipblasLtMatmul.
//
// Row-major operands are column-major ones transposed: out^T[N, M] = W[K, N]^T . x^T[K, M],
// i.e. A = W with transpose, B = x without, leading dimensions K, K and N.
#include <dlfcn.h>
#include <hipblaslt/hipblaslt.h>

#include <cstring>
#include <map>
#include <mutex>
#include <tuple>

#include "common.hpp"

namespace {

struct Api {
  void* library = nullptr;
  decltype(&hipblasLtCreate) create = nullptr;
  decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
  decltype(&hipblasLtMatmulDescSetAttribute) desc_set = nullptr;
  decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
  decltype(&hipblasLtMatmulPreferenceCreate) pref_create = nullptr;
  decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set = nullptr;
  decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy = nullptr;
  decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
  decltype(&hipblasLtMatmul) matmul = nullptr;
  decltype(&hipblasLtMatmulDescDestroy) desc_destroy = nullptr;
  decltype(&hipblasLtMatrixLayoutDestroy) layout_destroy = nullptr;
};

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
};

std::mutex g_mutex;
Api g_api;
std::map<int, hipblasLtHandle_t> g_handles;                             // by device
std::map<std::tuple<int, int, int, int, int>, Plan> g_plans;            // (device, m, n, k, out is float)
constexpr size_t kMaxPlans = 4096;

constexpr int kCandidates = 8;
// Row counts that share one choice of algorithm: few rows, where a decode step is
// nothing but these products, in fine buckets; many rows in buckets of 256.
int tune_bucket(int m) {
  if (m <= 8) return 0;
  if (m <= 16) return 1;
  if (m <= 32) return 2;
  if (m <= 64) return 3;
  if (m <= 128) return 4;
  if (m < 256) return 5;
  return 5 + m / 256;
}
// Which of the library's candidates runs a product is a fixed rule, so that the same
// model gives the same 32-bit sums in every process: the solution that was pinned for
// (n, k, out is float, tune_bucket(m)) where the library offers it among its candidates
// for the shape, else the library's own first choice.  Nothing is timed while the engine
// serves; the pins come from a table that was measured once (ms_gemm_library_time) and
// is kept with the sources.
std::map<std::tuple<int, int, int, int>, int> g_pinned;

// What the library itself calls the index of an algorithm: the first integer of its
// opaque data.  Used only to recognise a candidate among those offered for a shape.
int solution_index(const hipblasLtMatmulAlgo_t& algo) {
  int index = 0;
  std::memcpy(&index, algo.data, sizeof(index));
  return index;
}

struct Candidates {
  hipblasLtMatmulHeuristicResult_t result[kCandidates];
  int count = 0;
};

// Descriptors of out[m, n] = x[m, k] . w[n, k]^T and the library's candidates for it.
int describe(hipblasLtHandle_t handle, int m, int n, int k, int out_float, size_t workspace_bytes, Plan& plan,
             Candidates& candidates) {
  const hipDataType out_type = out_float ? HIP_R_32F : HIP_R_16BF;
  const int32_t transpose = HIPBLAS_OP_T, keep = HIPBLAS_OP_N;
  bool ok = g_api.desc_create(&plan.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && g_api.desc_set(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transpose, sizeof(transpose)) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && g_api.desc_set(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &keep, sizeof(keep)) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && g_api.layout_create(&plan.a, HIP_R_16BF, k, n, k) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && g_api.layout_create(&plan.b, HIP_R_16BF, k, m, k) == HIPBLAS_STATUS_SUCCESS;
  ok = ok && g_api.layout_create(&plan.c, out_type, n, m, n) == HIPBLAS_STATUS_SUCCESS;
  MS_REQUIRE(ok, "gemm_library: cannot describe %d x %d x %d", m, n, k);
  hipblasLtMatmulPreference_t preference = nullptr;
  MS_REQUIRE(g_api.pref_create(&preference) == HIPBLAS_STATUS_SUCCESS, "gemm_library: no preference object");
  const uint64_t limit = workspace_bytes;
  g_api.pref_set(preference, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &limit, sizeof(limit));
  const hipblasStatus_t status = g_api.heuristic(handle, plan.desc, plan.a, plan.b, plan.c, plan.c, preference,
                                                 kCandidates, candidates.result, &candidates.count);
  g_api.pref_destroy(preference);
  MS_REQUIRE(status == HIPBLAS_STATUS_SUCCESS && candidates.count > 0, "gemm_library: no algorithm for %d x %d x %d", m, n, k);
  return 0;
}

int handle_of_current_device(hipblasLtHandle_t** out) {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return ms_fail("gemm_library: no current device");
  MS_REQUIRE(g_api.library != nullptr, "gemm_library: ms_gemm_library_open was not called");
  hipblasLtHandle_t& handle = g_handles[device];
  if (handle == nullptr && g_api.create(&handle) != HIPBLAS_STATUS_SUCCESS) {
    g_handles.erase(device);
    return ms_fail("gemm_library: hipblasLtCreate failed");
  }
  *out = &handle;
  return 0;
}

template <typename F>
bool resolve(F& slot, const char* name) {
  slot = reinterpret_cast<F>(dlsym(g_api.library, name));
  return slot != nullptr;
}

}  // namespace

// path: the hipBLASLt shared library that the process already uses.
extern "C" int ms_gemm_library_open(const char* path) {
  std::lock_guard<std::mutex> guard(g_mutex);
  if (g_api.library != nullptr) return 0;
  MS_REQUIRE(path != nullptr, "gemm_library: no library path");
  void* library = dlopen(path, RTLD_NOW | RTLD_LOCAL);
  MS_REQUIRE(library != nullptr, "gemm_library: cannot open %s: %s", path, dlerror());
  g_api.library = library;
  const bool ok = resolve(g_api.create, "hipblasLtCreate") && resolve(g_api.desc_create, "hipblasLtMatmulDescCreate") &&
                  resolve(g_api.desc_set, "hipblasLtMatmulDescSetAttribute") &&
                  resolve(g_api.layout_create, "hipblasLtMatrixLayoutCreate") &&
                  resolve(g_api.pref_create, "hipblasLtMatmulPreferenceCreate") &&
                  resolve(g_api.pref_set, "hipblasLtMatmulPreferenceSetAttribute") &&
                  resolve(g_api.pref_destroy, "hipblasLtMatmulPreferenceDestroy") &&
                  resolve(g_api.heuristic, "hipblasLtMatmulAlgoGetHeuristic") && resolve(g_api.matmul, "hipblasLtMatmul") &&
                  resolve(g_api.desc_destroy, "hipblasLtMatmulDescDestroy") &&
                  resolve(g_api.layout_destroy, "hipblasLtMatrixLayoutDestroy");
  if (!ok) {
    g_api = Api{};
    return ms_fail("gemm_library: %s lacks a hipBLASLt entry point", path);
  }
  return 0;
}

// Pins the solution for products against a matrix [n, k] with row counts of `bucket`
// (ms_gemm_library_bucket) and the given output type.  Plans made before the call keep
// what they chose, so pins are set before the first product.
extern "C" int ms_gemm_library_pin(int n, int k, int out_float, int bucket, int solution) {
  std::lock_guard<std::mutex> guard(g_mutex);
  g_pinned[std::make_tuple(n, k, out_float != 0, bucket)] = solution;
  return 0;
}

// The bucket of row counts that m falls into (a plain number, not a status).
extern "C" int ms_gemm_library_bucket(int m) { return tune_bucket(m); }

// x: bfloat16 [m, k]; w: bfloat16 [n, k]; out: [m, n], bfloat16 or (out_float) float.
// accumulate (float output only): out += product.  workspace: device memory of
// workspace_bytes for the library's use, the caller's for the duration of the call
// on this stream.  The call allocates no device memory and waits for nothing.
extern "C" int ms_gemm_library(const void* x, const void* w, void* out, int m, int n, int k, int out_float,
                               int accumulate, void* workspace, size_t workspace_bytes, hipStream_t stream) {
  MS_REQUIRE(m > 0 && n > 0 && k > 0, "gemm_library: empty shape %d x %d x %d", m, n, k);
  MS_REQUIRE(x && w && out, "gemm_library: null operand");
  MS_REQUIRE(!accumulate || out_float, "gemm_library: accumulation needs a float output");
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return ms_fail("gemm_library: no current device");

  std::lock_guard<std::mutex> guard(g_mutex);
  hipblasLtHandle_t* handle = nullptr;
  if (const int failed = handle_of_current_device(&handle)) return failed;

  const auto key = std::make_tuple(device, m, n, k, out_float);
  auto found = g_plans.find(key);
  if (found == g_plans.end()) {
    if (g_plans.size() >= kMaxPlans) g_plans.clear();   // descriptors of shapes long gone; a few hundred bytes each
    Plan plan;
    Candidates candidates;
    if (const int failed = describe(*handle, m, n, k, out_float, workspace_bytes, plan, candidates)) return failed;
    int best = -1;
    const auto pinned = g_pinned.find(std::make_tuple(n, k, out_float != 0, tune_bucket(m)));
    for (int i = 0; i < candidates.count; ++i) {
      const auto& candidate = candidates.result[i];
      if (candidate.state != HIPBLAS_STATUS_SUCCESS || candidate.workspaceSize > workspace_bytes) continue;
      if (best < 0) best = i;                           // the library's first usable choice
      if (pinned != g_pinned.end() && solution_index(candidate.algo) == pinned->second) {
        best = i;
        break;
      }
    }
    MS_REQUIRE(best >= 0, "gemm_library: no usable algorithm for %d x %d x %d", m, n, k);
    plan.algo = candidates.result[best].algo;
    plan.workspace = candidates.result[best].workspaceSize;
    found = g_plans.emplace(key, plan).first;
  }
  const Plan& plan = found->second;
  MS_REQUIRE(plan.workspace <= workspace_bytes, "gemm_library: the algorithm wants %zu bytes of workspace, %zu given",
             plan.workspace, workspace_bytes);
  const float alpha = 1.0f, beta = accumulate ? 1.0f : 0.0f;
  const hipblasStatus_t status = g_api.matmul(*handle, plan.desc, &alpha, w, plan.a, x, plan.b, &beta, out, plan.c, out,
                                              plan.c, &plan.algo, workspace, workspace_bytes, stream);
  MS_REQUIRE(status == HIPBLAS_STATUS_SUCCESS, "gemm_library: hipblasLtMatmul failed with status %d for %d x %d x %d",
             static_cast<int>(status), m, n, k);
  return 0;
}

// For the tool that measures the table of pins, never called while the engine serves:
// times the library's candidates for x[m, k] . w[n, k]^T -> scratch_out [m, n] (memory of
// the caller's, not the product's true output) and reports, per candidate, its solution
// and the least of three timed runs in milliseconds (0 = not usable), each run after
// `flush` (flush_bytes of the caller's memory, more than the caches hold, or null) has
// been overwritten: a decode step meets every matrix in memory, not in the caches, and
// among candidates that are timed warm the wrong one wins.  solutions and milliseconds
// hold `capacity` entries; *count receives how many were filled.  Waits for the stream.
extern "C" int ms_gemm_library_time(const void* x, const void* w, void* scratch_out, int m, int n, int k, int out_float,
                                    void* workspace, size_t workspace_bytes, void* flush, size_t flush_bytes,
                                    int* solutions, float* milliseconds, int capacity, int* count, hipStream_t stream) {
  MS_REQUIRE(m > 0 && n > 0 && k > 0 && x && w && scratch_out && solutions && milliseconds && count && capacity > 0,
             "gemm_library_time: bad arguments");
  std::lock_guard<std::mutex> guard(g_mutex);
  hipblasLtHandle_t* handle = nullptr;
  if (const int failed = handle_of_current_device(&handle)) return failed;
  Plan plan;
  Candidates candidates;
  if (const int failed = describe(*handle, m, n, k, out_float, workspace_bytes, plan, candidates)) return failed;
  hipEvent_t begin = nullptr, end = nullptr;
  MS_REQUIRE(hipEventCreate(&begin) == hipSuccess && hipEventCreate(&end) == hipSuccess, "gemm_library_time: no events");
  const float alpha = 1.0f, beta = 0.0f;
  const auto run = [&](int i) {
    return g_api.matmul(*handle, plan.desc, &alpha, w, plan.a, x, plan.b, &beta, scratch_out, plan.c, scratch_out, plan.c,
                        &candidates.result[i].algo, workspace, workspace_bytes, stream) == HIPBLAS_STATUS_SUCCESS;
  };
  const int filled = candidates.count < capacity ? candidates.count : capacity;
  for (int i = 0; i < filled; ++i) {
    solutions[i] = solution_index(candidates.result[i].algo);
    milliseconds[i] = 0.f;
    bool usable = candidates.result[i].state == HIPBLAS_STATUS_SUCCESS &&
                  candidates.result[i].workspaceSize <= workspace_bytes && run(i);      // one run that is not counted
    for (int trial = 0; usable && trial < 3; ++trial) {
      float ms = 0.f;
      usable = (flush == nullptr || hipMemsetAsync(flush, trial, flush_bytes, stream) == hipSuccess) &&
               hipEventRecord(begin, stream) == hipSuccess && run(i) && hipEventRecord(end, stream) == hipSuccess &&
               hipEventSynchronize(end) == hipSuccess && hipEventElapsedTime(&ms, begin, end) == hipSuccess;
      if (usable && (milliseconds[i] == 0.f || ms < milliseconds[i])) milliseconds[i] = ms;
    }
    if (!usable) {
      milliseconds[i] = 0.f;
      (void)hipGetLastError();
    }
  }
  *count = filled;
  g_api.desc_destroy(plan.desc);
  g_api.layout_destroy(plan.a);
  g_api.layout_destroy(plan.b);
  g_api.layout_destroy(plan.c);
  (void)hipEventDestroy(begin);
  (void)hipEventDestroy(end);
  (void)hipStreamSynchronize(stream);
  return 0;
}
