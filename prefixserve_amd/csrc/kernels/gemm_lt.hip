// The library product for large bfloat16 steps: out[M, N] = x[M, K] * w[N, K]^T (out bfloat16,
// or float32 for logits) through hipBLASLt, called directly. The reference's engine calls a library for these products too
// (torch.nn.functional.linear, prefixserve/model/llama.py:113-121); going through torch.mm costs
// 18 us of host time per call (descriptors and the heuristic search are redone every time),
// which makes a step of a few hundred tokens host-bound. Here the descriptors and the chosen
// algorithm are kept per (M, N, K), so that a call is one hipblasLtMatmul.
//
// Returns 0, 1 for an error, or 2 if the library has no algorithm for the shape under the
// given conditions (the caller then takes another path).
// use_workspace = 0 asks for an algorithm that needs no workspace: what a caller under stream
// capture wants, since algorithms with a workspace may clear it with a memset, and memset nodes
// of a captured graph are not to be relied on when the graph is replayed.
//
// The library is looked up at run time (the copy already in the process, which is torch's, else
// the system's): nothing links against it, and if it or one of its entry points is missing
// psamd_gemm_lt_available() says so and the caller keeps using torch.mm.
//
// The library's heuristic picks an algorithm without running anything. psamd_gemm_lt_tune() times
// every algorithm that supports a shape on the caller's buffers and keeps the fastest for that
// shape and, where they support them, for row counts within a quarter of it. What it finds depends
// on the copy of the library in the process: the one that ships with torch here has 4,626
// algorithms for bfloat16, 230 of them for the products of the Llama 3.2 1B sizes, and its
// heuristic already returns the fastest of them (one shape of eight gained 5%); ROCm 7.2's own copy
// has 20,141 (2,084), and its heuristic's first choice is 6 to 30% slower than its best (2,048 rows:
// q/k/v 30 -> 26 us, o 31 -> 21, gate/up 114 -> 102, down 84 -> 66), which is about where the other
// copy's heuristic is. So the tuning is off unless asked for. It is meant for warm-up: it takes a
// quarter of a second per shape and waits for the stream.
//
// No kernels in this file.

#include <dlfcn.h>
#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>

#include <algorithm>
#include <cstdlib>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "api.h"
#include "common.h"

namespace psamd {
namespace {

constexpr size_t kWorkspaceBytes = 64u << 20;      // what stream-K algorithms may ask for
constexpr size_t kMaxPlans = 4096;                 // every token count is a shape of its own
constexpr int kMaxDevices = 16;

struct Api {
  bool ok = false;
  decltype(&hipblasLtCreate) create = nullptr;
  decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
  decltype(&hipblasLtMatmulDescDestroy) desc_destroy = nullptr;
  decltype(&hipblasLtMatmulDescSetAttribute) desc_set = nullptr;
  decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
  decltype(&hipblasLtMatrixLayoutDestroy) layout_destroy = nullptr;
  decltype(&hipblasLtMatmulPreferenceCreate) pref_create = nullptr;
  decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy = nullptr;
  decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set = nullptr;
  decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
  decltype(&hipblasLtMatmul) matmul = nullptr;
  // The extension interface (C++ entry points of the same library), for tuning only.
  bool ext = false;
  decltype(&hipblaslt_ext::getAllAlgos) all_algos = nullptr;
  decltype(&hipblaslt_ext::matmulIsAlgoSupported) is_supported = nullptr;
};

template <typename F>
bool bind(void* lib, const char* name, F& fn) {
  fn = reinterpret_cast<F>(dlsym(lib, name));
  return fn != nullptr;
}

const Api& api() {
  static const Api loaded = [] {
    Api a;
    void* lib = dlopen("libhipblaslt.so.1", RTLD_NOW | RTLD_NOLOAD);    // the copy torch brought, if any
    if (lib == nullptr) lib = dlopen("libhipblaslt.so.1", RTLD_NOW | RTLD_LOCAL);
    if (lib == nullptr) lib = dlopen("libhipblaslt.so", RTLD_NOW | RTLD_LOCAL);
    if (lib == nullptr) return a;
    a.ok = bind(lib, "hipblasLtCreate", a.create) && bind(lib, "hipblasLtMatmulDescCreate", a.desc_create) &&
           bind(lib, "hipblasLtMatmulDescDestroy", a.desc_destroy) &&
           bind(lib, "hipblasLtMatmulDescSetAttribute", a.desc_set) &&
           bind(lib, "hipblasLtMatrixLayoutCreate", a.layout_create) &&
           bind(lib, "hipblasLtMatrixLayoutDestroy", a.layout_destroy) &&
           bind(lib, "hipblasLtMatmulPreferenceCreate", a.pref_create) &&
           bind(lib, "hipblasLtMatmulPreferenceDestroy", a.pref_destroy) &&
           bind(lib, "hipblasLtMatmulPreferenceSetAttribute", a.pref_set) &&
           bind(lib, "hipblasLtMatmulAlgoGetHeuristic", a.heuristic) && bind(lib, "hipblasLtMatmul", a.matmul);
    a.ext = bind(lib,
                 "_ZN13hipblaslt_ext11getAllAlgosEPvNS_8GemmTypeE18hipblasOperation_tS2_11hipDataTypeS3_S3_S3_"
                 "20hipblasComputeType_tRSt6vectorI33_hipblasLtMatmulHeuristicResult_tSaIS6_EE",
                 a.all_algos) &&
            bind(lib,
                 "_ZN13hipblaslt_ext21matmulIsAlgoSupportedEPvP27hipblasLtMatmulDescOpaque_tPKvP29hipblasLtMatrixLayoutOpaque_t"
                 "S6_S4_S6_S6_R22_hipblasLtMatmulAlgo_tRm",
                 a.is_supported);
    return a;
  }();
  return loaded;
}

struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, x = nullptr, out = nullptr;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
};

struct Tuned {            // the fastest algorithm found for [M, K] x [N, K]^T by timing
  int64_t M;
  int N, K;
  bool float_out;
  hipblasLtMatmulAlgo_t algo;
  size_t workspace;
};

struct Device {
  hipblasLtHandle_t handle = nullptr;
  void* workspace = nullptr;
  std::map<std::tuple<int64_t, int, int, bool, bool>, Plan> plans;
  std::vector<Tuned> tuned;
  std::vector<hipblasLtMatmulHeuristicResult_t> all[2];     // every algorithm for bfloat16 / float32 output
  bool all_asked[2] = {false, false};
};

std::mutex g_lock;
Device g_devices[kMaxDevices];

void drop(const Api& a, Plan& p) {
  if (p.w) a.layout_destroy(p.w);
  if (p.x) a.layout_destroy(p.x);
  if (p.out) a.layout_destroy(p.out);
  if (p.desc) a.desc_destroy(p.desc);
  p = Plan{};
}

// Row-major out[M, N] = x[M, K] * w[N, K]^T is, in the library's column-major terms,
// C[N x M] = A^T * B with A = w seen as [K x N] (leading dimension K) and B = x seen as [K x M].
int make_plan(const Api& a, Device& dev, int64_t M, int N, int K, bool use_workspace, bool float_out, Plan& p) {
  const hipblasOperation_t trans = HIPBLAS_OP_T, none = HIPBLAS_OP_N;
  bool ok = a.desc_create(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS &&
            a.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &trans, sizeof(trans)) == HIPBLAS_STATUS_SUCCESS &&
            a.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &none, sizeof(none)) == HIPBLAS_STATUS_SUCCESS &&
            a.layout_create(&p.w, HIP_R_16BF, K, N, K) == HIPBLAS_STATUS_SUCCESS &&
            a.layout_create(&p.x, HIP_R_16BF, K, M, K) == HIPBLAS_STATUS_SUCCESS &&
            a.layout_create(&p.out, float_out ? HIP_R_32F : HIP_R_16BF, N, M, N) == HIPBLAS_STATUS_SUCCESS;
  hipblasLtMatmulPreference_t pref = nullptr;
  ok = ok && a.pref_create(&pref) == HIPBLAS_STATUS_SUCCESS;
  const uint64_t room = use_workspace ? kWorkspaceBytes : 0;
  ok = ok && a.pref_set(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &room, sizeof(room)) == HIPBLAS_STATUS_SUCCESS;
  hipblasLtMatmulHeuristicResult_t found;
  int count = 0;
  ok = ok && a.heuristic(dev.handle, p.desc, p.w, p.x, p.out, p.out, pref, 1, &found, &count) == HIPBLAS_STATUS_SUCCESS &&
       count > 0 && found.state == HIPBLAS_STATUS_SUCCESS && found.workspaceSize <= room;
  if (pref) a.pref_destroy(pref);
  if (!ok) {
    drop(a, p);
    return fail("psamd_gemm_lt: the library has no algorithm for [" + std::to_string(M) + ", " + std::to_string(K) +
                "] x [" + std::to_string(N) + ", " + std::to_string(K) + "]^T");
  }
  p.algo = found.algo;
  p.workspace = found.workspaceSize;
  if (use_workspace && a.ext) {
    // A tuned algorithm of the nearest row count within a quarter, if it supports this one.
    const Tuned* best = nullptr;
    for (const Tuned& t : dev.tuned) {
      if (t.N != N || t.K != K || t.float_out != float_out || 4 * t.M > 5 * M || 4 * M > 5 * t.M) continue;
      if (best == nullptr || std::llabs(t.M - M) < std::llabs(best->M - M)) best = &t;
    }
    if (best != nullptr) {
      const float one = 1.f, zero = 0.f;
      hipblasLtMatmulAlgo_t algo = best->algo;
      size_t need = 0;
      if (a.is_supported(dev.handle, p.desc, &one, p.w, p.x, &zero, p.out, p.out, algo, need) == HIPBLAS_STATUS_SUCCESS &&
          need <= kWorkspaceBytes) {
        p.algo = algo;
        p.workspace = need;
      }
    }
  }
  return 0;
}

}  // namespace
}  // namespace psamd

using namespace psamd;

extern "C" {

// 1 if the library is there and ready on the current device (first call per device: creates
// the handle and takes the workspace, so call it outside any stream capture), else 0.
int psamd_gemm_lt_available() {
  const Api& a = api();
  int id = 0;
  if (!a.ok || hipGetDevice(&id) != hipSuccess || id < 0 || id >= kMaxDevices) return 0;
  std::lock_guard<std::mutex> guard(g_lock);
  Device& dev = g_devices[id];
  if (dev.handle != nullptr) return 1;
  hipblasLtHandle_t handle = nullptr;
  if (a.create(&handle) != HIPBLAS_STATUS_SUCCESS) return 0;
  void* room = nullptr;
  if (hipMalloc(&room, kWorkspaceBytes) != hipSuccess) return 0;     // kept until the process ends
  dev.handle = handle;
  dev.workspace = room;
  return 1;
}

int psamd_gemm_lt(void* stream, const void* x, const void* w, void* out, int out_dtype, int64_t M, int N, int K,
                  int use_workspace) {
  PSAMD_REQUIRE(M > 0 && N > 0 && K > 0 && M <= INT32_MAX, "bad sizes");
  PSAMD_REQUIRE(out_dtype == kBF16 || out_dtype == kF32, "the output is bfloat16 or float32");
  const bool float_out = out_dtype == kF32;
  const Api& a = api();
  int id = 0;
  PSAMD_REQUIRE(a.ok && hipGetDevice(&id) == hipSuccess && id >= 0 && id < kMaxDevices, "hipBLASLt is not available");
  std::lock_guard<std::mutex> guard(g_lock);
  Device& dev = g_devices[id];
  PSAMD_REQUIRE(dev.handle != nullptr, "call psamd_gemm_lt_available() on this device first");
  const bool roomy = use_workspace != 0;
  const auto key = std::make_tuple(M, N, K, roomy, float_out);
  auto it = dev.plans.find(key);
  if (it == dev.plans.end()) {
    if (dev.plans.size() >= kMaxPlans) {
      for (auto& kv : dev.plans) drop(a, kv.second);
      dev.plans.clear();
    }
    Plan p;
    make_plan(a, dev, M, N, K, roomy, float_out, p);      // on failure p stays empty, and is kept: the answer will not change
    it = dev.plans.emplace(key, p).first;
  }
  const Plan& p = it->second;
  if (p.desc == nullptr) return 2;                         // the message of make_plan is the last error
  const float one = 1.f, zero = 0.f;
  const hipblasStatus_t st = a.matmul(dev.handle, p.desc, &one, w, p.w, x, p.x, &zero, out, p.out, out, p.out, &p.algo,
                                      roomy ? dev.workspace : nullptr, roomy ? kWorkspaceBytes : 0,
                                      static_cast<hipStream_t>(stream));
  if (st != HIPBLAS_STATUS_SUCCESS) return fail("psamd_gemm_lt: hipblasLtMatmul returned " + std::to_string(st));
  return 0;
}

// Times every algorithm of the library that supports out[M, N] = x[M, K] * w[N, K]^T (with a
// workspace) on the given buffers, w being each of the n_ws matrices of that shape in turn, and keeps the fastest for this shape from now on, if it beats
// the heuristic's choice by 3% or more. out receives the product by the kept algorithm and
// ref_out by the heuristic's, for the caller to compare; us_before and us_after their times.
// Waits for the stream. Returns 0, 1 for an error, 2 if the library or its extension interface
// is not there (nothing changes then).
int psamd_gemm_lt_tune(void* stream, const void* x, const void* const* ws, int n_ws, void* out, void* ref_out, int out_dtype,
                       int64_t M, int N, int K, float* us_before, float* us_after) {
  PSAMD_REQUIRE(M > 0 && N > 0 && K > 0 && M <= INT32_MAX, "bad sizes");
  PSAMD_REQUIRE(out_dtype == kBF16 || out_dtype == kF32, "the output is bfloat16 or float32");
  PSAMD_REQUIRE(us_before != nullptr && us_after != nullptr && out != nullptr && ref_out != nullptr, "missing outputs");
  PSAMD_REQUIRE(ws != nullptr && n_ws >= 1, "at least one matrix");
  const bool float_out = out_dtype == kF32;
  const Api& a = api();
  int id = 0;
  if (!a.ok || !a.ext || hipGetDevice(&id) != hipSuccess || id < 0 || id >= kMaxDevices) return 2;
  std::lock_guard<std::mutex> guard(g_lock);
  Device& dev = g_devices[id];
  PSAMD_REQUIRE(dev.handle != nullptr, "call psamd_gemm_lt_available() on this device first");
  hipStream_t s = static_cast<hipStream_t>(stream);

  // The plan of the heuristic's choice, made anew so that an earlier tuning does not count as "before".
  const auto key = std::make_tuple(M, N, K, true, float_out);
  auto it = dev.plans.find(key);
  if (it != dev.plans.end()) {
    drop(a, it->second);
    dev.plans.erase(it);
  }
  dev.tuned.erase(std::remove_if(dev.tuned.begin(), dev.tuned.end(),
                                 [&](const Tuned& t) { return t.M == M && t.N == N && t.K == K && t.float_out == float_out; }),
                  dev.tuned.end());
  Plan p;
  {
    std::vector<Tuned> none;
    none.swap(dev.tuned);                                   // no borrowing from neighbours either
    const int rc = make_plan(a, dev, M, N, K, true, float_out, p);
    none.swap(dev.tuned);
    if (rc != 0) return 2;
  }
  const hipblasLtMatmulAlgo_t first = p.algo;

  const int which = float_out ? 1 : 0;
  if (!dev.all_asked[which]) {
    dev.all_asked[which] = true;
    const hipDataType out_type = float_out ? HIP_R_32F : HIP_R_16BF;
    if (a.all_algos(dev.handle, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, HIPBLAS_OP_T, HIPBLAS_OP_N, HIP_R_16BF, HIP_R_16BF,
                    out_type, out_type, HIPBLAS_COMPUTE_32F, dev.all[which]) != HIPBLAS_STATUS_SUCCESS)
      dev.all[which].clear();
  }

  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
    drop(a, p);
    return fail("psamd_gemm_lt_tune: no events");
  }
  const float one = 1.f, zero = 0.f;
  // Microseconds per call over `reps` calls into `dst`, or a negative number if the call fails.
  // The matrices are taken in turn (a model's layers): each call then reads its matrix from
  // memory, as a step does, not from the caches the call before it left warm.
  int turn = 0;
  auto timed = [&](hipblasLtMatmulAlgo_t& algo, void* dst, int reps) -> float {
    if (a.matmul(dev.handle, p.desc, &one, ws[0], p.w, x, p.x, &zero, dst, p.out, dst, p.out, &algo, dev.workspace,
                 kWorkspaceBytes, s) != HIPBLAS_STATUS_SUCCESS)
      return -1.f;
    if (hipEventRecord(e0, s) != hipSuccess) return -1.f;
    for (int i = 0; i < reps; ++i) {
      turn = (turn + 1) % n_ws;
      if (a.matmul(dev.handle, p.desc, &one, ws[turn], p.w, x, p.x, &zero, dst, p.out, dst, p.out, &algo, dev.workspace,
                   kWorkspaceBytes, s) != HIPBLAS_STATUS_SUCCESS)
        return -1.f;
    }
    if (hipEventRecord(e1, s) != hipSuccess || hipEventSynchronize(e1) != hipSuccess) return -1.f;
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess) return -1.f;
    return ms * 1000.f / static_cast<float>(reps);
  };

  // A first pass over all that support the shape, three calls each; the leaders again, with the
  // heuristic's choice among them, in three rounds of ten (the lowest round counts).
  std::vector<std::pair<float, size_t>> screened;
  for (size_t i = 0; i < dev.all[which].size(); ++i) {
    hipblasLtMatmulAlgo_t algo = dev.all[which][i].algo;
    size_t need = 0;
    if (a.is_supported(dev.handle, p.desc, &one, p.w, p.x, &zero, p.out, p.out, algo, need) != HIPBLAS_STATUS_SUCCESS ||
        need > kWorkspaceBytes)
      continue;
    const float us = timed(algo, out, 3);
    if (us > 0.f) screened.push_back({us, i});
  }
  std::sort(screened.begin(), screened.end());
  if (screened.size() > 12) screened.resize(12);
  std::vector<hipblasLtMatmulAlgo_t> finalists{first};
  for (const auto& sc : screened) finalists.push_back(dev.all[which][sc.second].algo);
  std::vector<float> best(finalists.size(), 1e30f);
  for (int round = 0; round < 3; ++round)
    for (size_t i = 0; i < finalists.size(); ++i) {
      const float us = timed(finalists[i], out, 10);
      if (us > 0.f) best[i] = std::min(best[i], us);
    }
  size_t winner = 0;
  for (size_t i = 1; i < finalists.size(); ++i)
    if (best[i] < best[winner]) winner = i;
  if (best[winner] > 0.97f * best[0]) winner = 0;
  *us_before = best[0];
  *us_after = best[winner];

  hipblasLtMatmulAlgo_t ref_algo = first;
  n_ws = 1;                                              // both products by the first matrix
  const bool ran = timed(ref_algo, ref_out, 1) > 0.f && timed(finalists[winner], out, 1) > 0.f;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (!ran) {
    drop(a, p);
    return fail("psamd_gemm_lt_tune: the product failed");
  }
  if (winner != 0) {
    size_t need = 0;
    hipblasLtMatmulAlgo_t algo = finalists[winner];
    (void)a.is_supported(dev.handle, p.desc, &one, p.w, p.x, &zero, p.out, p.out, algo, need);
    p.algo = algo;
    p.workspace = need;
    dev.tuned.push_back(Tuned{M, N, K, float_out, algo, need});
    // Plans of neighbouring row counts made before now may borrow it: they are made again when next asked for.
    for (auto pit = dev.plans.begin(); pit != dev.plans.end();) {
      const auto& k = pit->first;
      const int64_t m2 = std::get<0>(k);
      if (std::get<1>(k) == N && std::get<2>(k) == K && std::get<3>(k) && std::get<4>(k) == float_out && 4 * m2 <= 5 * M &&
          4 * M <= 5 * m2) {
        drop(a, pit->second);
        pit = dev.plans.erase(pit);
      } else {
        ++pit;
      }
    }
  }
  dev.plans.emplace(key, p);
  return 0;
}

// Forgets what psamd_gemm_lt_tune() kept for a shape (a caller that found its result wrong).
int psamd_gemm_lt_untune(int out_dtype, int64_t M, int N, int K) {
  const bool float_out = out_dtype == kF32;
  const Api& a = api();
  int id = 0;
  if (!a.ok || hipGetDevice(&id) != hipSuccess || id < 0 || id >= kMaxDevices) return 2;
  std::lock_guard<std::mutex> guard(g_lock);
  Device& dev = g_devices[id];
  dev.tuned.erase(std::remove_if(dev.tuned.begin(), dev.tuned.end(),
                                 [&](const Tuned& t) { return t.M == M && t.N == N && t.K == K && t.float_out == float_out; }),
                  dev.tuned.end());
  for (auto pit = dev.plans.begin(); pit != dev.plans.end();) {
    const auto& k = pit->first;
    if (std::get<1>(k) == N && std::get<2>(k) == K && std::get<3>(k) && std::get<4>(k) == float_out) {
      drop(a, pit->second);
      pit = dev.plans.erase(pit);
    } else {
      ++pit;
    }
  }
  return 0;
}

}  // extern "C"
