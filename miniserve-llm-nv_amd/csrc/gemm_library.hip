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
// Row counts that share one timing: the solution that was fastest for the first row
// count of a bucket is taken for the others where the library offers it for them, so
// that a stream of ever new row counts (portions of prompts beside decode tokens) does
// not stop to time each of them.  Few rows, where a decode step is nothing but these
// products, in fine buckets; many rows in buckets of 256.
int tune_bucket(int m) {
  if (m <= 8) return 0;
  if (m <= 16) return 1;
  if (m <= 32) return 2;
  if (m <= 64) return 3;
  if (m <= 128) return 4;
  if (m < 256) return 5;
  return 5 + m / 256;
}
// The solution that timing chose for (device, n, k, out is float, tune_bucket(m)).
std::map<std::tuple<int, int, int, int, int>, int> g_tuned;
// What is written between two timed runs so that each finds the matrix in memory, not
// in the caches (the last-level cache holds 256 MiB): a decode step meets every matrix
// cold, and among candidates that are timed warm the wrong one wins.
constexpr size_t kFlushBytes = static_cast<size_t>(384) << 20;

// What the library itself calls the index of an algorithm: the first integer of its
// opaque data.  Used only to recognise a candidate among those offered for a shape.
int solution_index(const hipblasLtMatmulAlgo_t& algo) {
  int index = 0;
  std::memcpy(&index, algo.data, sizeof(index));
  return index;
}

// Index of the candidate that runs this product fastest: the least of three timed runs
// each, after one that is not counted, the caches flushed before every timed run (where
// the memory for that is to be had).  The output goes to memory of its own, so that
// `out` is written once, by the call.
int fastest_candidate(hipblasLtHandle_t handle, const Plan& plan, const hipblasLtMatmulHeuristicResult_t* candidates,
                      int count, const void* x, const void* w, int m, int n, int out_float, void* workspace,
                      size_t workspace_bytes, hipStream_t stream) {
  void* scratch = nullptr;
  const size_t bytes = static_cast<size_t>(m) * n * (out_float ? 4 : 2);
  if (hipMalloc(&scratch, bytes) != hipSuccess) return 0;
  void* flush = nullptr;
  if (hipMalloc(&flush, kFlushBytes) != hipSuccess) {
    flush = nullptr;
    (void)hipGetLastError();      // timed warm then
  }
  hipEvent_t begin = nullptr, end = nullptr;
  int best = 0;
  if (hipEventCreate(&begin) == hipSuccess && hipEventCreate(&end) == hipSuccess) {
    const float alpha = 1.0f, beta = 0.0f;
    float least[kCandidates];
    bool usable[kCandidates];
    const auto run = [&](int i) {
      return g_api.matmul(handle, plan.desc, &alpha, w, plan.a, x, plan.b, &beta, scratch, plan.c, scratch, plan.c,
                          &candidates[i].algo, workspace, workspace_bytes, stream) == HIPBLAS_STATUS_SUCCESS;
    };
    for (int i = 0; i < count && i < kCandidates; ++i) {
      least[i] = 0.f;
      usable[i] = candidates[i].state == HIPBLAS_STATUS_SUCCESS && candidates[i].workspaceSize <= workspace_bytes && run(i);
    }
    for (int trial = 0; trial < 3; ++trial) {
      for (int i = 0; i < count && i < kCandidates; ++i) {
        if (!usable[i]) continue;
        float ms = 0.f;
        bool ok = flush == nullptr || hipMemsetAsync(flush, trial, kFlushBytes, stream) == hipSuccess;
        ok = ok && hipEventRecord(begin, stream) == hipSuccess && run(i) && hipEventRecord(end, stream) == hipSuccess &&
             hipEventSynchronize(end) == hipSuccess && hipEventElapsedTime(&ms, begin, end) == hipSuccess;
        if (!ok) {
          usable[i] = false;
          (void)hipGetLastError();
        } else if (least[i] == 0.f || ms < least[i]) {
          least[i] = ms;
        }
      }
    }
    float best_ms = 0.f;
    for (int i = 0; i < count && i < kCandidates; ++i) {
      if (usable[i] && least[i] > 0.f && (best_ms == 0.f || least[i] < best_ms)) {
        best_ms = least[i];
        best = i;
      }
    }
  }
  if (begin) hipEventDestroy(begin);
  if (end) hipEventDestroy(end);
  hipStreamSynchronize(stream);
  if (flush) hipFree(flush);
  hipFree(scratch);
  return best;
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
                  resolve(g_api.heuristic, "hipblasLtMatmulAlgoGetHeuristic") && resolve(g_api.matmul, "hipblasLtMatmul");
  if (!ok) {
    g_api = Api{};
    return ms_fail("gemm_library: %s lacks a hipBLASLt entry point", path);
  }
  return 0;
}

// x: bfloat16 [m, k]; w: bfloat16 [n, k]; out: [m, n], bfloat16 or (out_float) float.
// accumulate (float output only): out += product.  workspace: device memory of
// workspace_bytes for the library's use, the caller's for the duration of the call
// on this stream.
extern "C" int ms_gemm_library(const void* x, const void* w, void* out, int m, int n, int k, int out_float,
                               int accumulate, void* workspace, size_t workspace_bytes, hipStream_t stream) {
  MS_REQUIRE(m > 0 && n > 0 && k > 0, "gemm_library: empty shape %d x %d x %d", m, n, k);
  MS_REQUIRE(x && w && out, "gemm_library: null operand");
  MS_REQUIRE(!accumulate || out_float, "gemm_library: accumulation needs a float output");
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return ms_fail("gemm_library: no current device");

  std::lock_guard<std::mutex> guard(g_mutex);
  MS_REQUIRE(g_api.library != nullptr, "gemm_library: ms_gemm_library_open was not called");
  hipblasLtHandle_t& handle = g_handles[device];
  if (handle == nullptr && g_api.create(&handle) != HIPBLAS_STATUS_SUCCESS) {
    g_handles.erase(device);
    return ms_fail("gemm_library: hipblasLtCreate failed");
  }

  const auto key = std::make_tuple(device, m, n, k, out_float);
  auto found = g_plans.find(key);
  if (found == g_plans.end()) {
    if (g_plans.size() >= kMaxPlans) g_plans.clear();   // descriptors of shapes long gone; a few hundred bytes each
    Plan plan;
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
    hipblasLtMatmulHeuristicResult_t result[kCandidates];
    int returned = 0;
    const hipblasStatus_t status =
        g_api.heuristic(handle, plan.desc, plan.a, plan.b, plan.c, plan.c, preference, kCandidates, result, &returned);
    g_api.pref_destroy(preference);
    MS_REQUIRE(status == HIPBLAS_STATUS_SUCCESS && returned > 0, "gemm_library: no algorithm for %d x %d x %d", m, n, k);
    int best = 0;
    // The library's first choice is not always its fastest (25600 x 5120 against 8 rows:
    // 138 us, its third candidate 58).  The candidates are timed once for a bucket of row
    // counts, on scratch output, unless the stream is recording (no waiting there).
    if (returned > 1) {
      const auto bucket = std::make_tuple(device, n, k, out_float, tune_bucket(m));
      const auto tuned = g_tuned.find(bucket);
      hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
      if (tuned != g_tuned.end()) {
        for (int i = 0; i < returned; ++i) {
          if (result[i].state == HIPBLAS_STATUS_SUCCESS && result[i].workspaceSize <= workspace_bytes &&
              solution_index(result[i].algo) == tuned->second) {
            best = i;
            break;
          }
        }
      } else if (hipStreamIsCapturing(stream, &capture) == hipSuccess && capture == hipStreamCaptureStatusNone) {
        best = fastest_candidate(handle, plan, result, returned, x, w, m, n, out_float, workspace, workspace_bytes, stream);
        g_tuned[bucket] = solution_index(result[best].algo);
      }
    }
    plan.algo = result[best].algo;
    plan.workspace = result[best].workspaceSize;
    found = g_plans.emplace(key, plan).first;
  }
  const Plan& plan = found->second;
  MS_REQUIRE(plan.workspace <= workspace_bytes, "gemm_library: the algorithm wants %zu bytes of workspace, %zu given",
             plan.workspace, workspace_bytes);
  const float alpha = 1.0f, beta = accumulate ? 1.0f : 0.0f;
  const hipblasStatus_t status = g_api.matmul(handle, plan.desc, &alpha, w, plan.a, x, plan.b, &beta, out, plan.c, out,
                                              plan.c, &plan.algo, workspace, workspace_bytes, stream);
  MS_REQUIRE(status == HIPBLAS_STATUS_SUCCESS, "gemm_library: hipblasLtMatmul failed with status %d for %d x %d x %d",
             static_cast<int>(status), m, n, k);
  return 0;
}
