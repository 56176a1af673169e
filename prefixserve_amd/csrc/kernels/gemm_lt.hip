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
// No kernels in this file.

#include <dlfcn.h>
#include <hipblaslt/hipblaslt.h>

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

struct Device {
  hipblasLtHandle_t handle = nullptr;
  void* workspace = nullptr;
  std::map<std::tuple<int64_t, int, int, bool, bool>, Plan> plans;
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
                  int use_workspace, int accumulate) {
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
  const hipblasStatus_t st = a.matmul(dev.handle, p.desc, &one, w, p.w, x, p.x, accumulate ? &one : &zero, out, p.out, out, p.out, &p.algo,
                                      roomy ? dev.workspace : nullptr, roomy ? kWorkspaceBytes : 0,
                                      static_cast<hipStream_t>(stream));
  if (st != HIPBLAS_STATUS_SUCCESS) return fail("psamd_gemm_lt: hipblasLtMatmul returned " + std::to_string(st));
  return 0;
}

}  // extern "C"
