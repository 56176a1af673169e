// Next-token choice from float32 logits: greedy (lowest index among equal maxima) and
// temperature sampling by inverse CDF of softmax(logits / T) in vocabulary order. The
// uniform number of each row comes from the host, a function of (seed, request, output
// index) only, so a recomputed request draws the same token.
//
// Two kernels, because one workgroup per row reads a 128k-entry row far below what the
// memory can deliver: the first cuts every row into up to 32 runs of the vocabulary, one
// workgroup each, and leaves per run (maximum, its first index, sum of exp((x - max) / T));
// the second, one workgroup per row, combines the runs (that is already the greedy answer),
// finds the run in which the cumulative sum passes the target and scans only that run.

#include <algorithm>
#include <mutex>

#include "api.h"
#include "common.h"

namespace psamd {

constexpr int kSampleThreads = 256;
constexpr int kMaxRuns = 32;

struct RunStat {
  float max;
  int32_t arg;
  float sum;
  float pad;
};

// A NaN never wins (both comparisons are false for it): a row of NaNs, or of -inf, keeps the
// index the search started from, so callers start from an index of the row, never from a
// sentinel outside it. The token is fed to the next step's embedding on the device.
__device__ __forceinline__ void take_max(float v, int32_t i, float& best, int32_t& best_i) {
  if (v > best || (v == best && i < best_i)) {
    best = v;
    best_i = i;
  }
}

// Block-wide (max, first index) by shuffles and one LDS round.
__device__ __forceinline__ void block_argmax(float& best, int32_t& best_i, float* red, int32_t* red_i) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o, kWave);
    const int32_t oi = __shfl_xor(best_i, o, kWave);
    take_max(ob, oi, best, best_i);
  }
  const int tid = threadIdx.x;
  if ((tid & (kWave - 1)) == 0) {
    red[tid / kWave] = best;
    red_i[tid / kWave] = best_i;
  }
  __syncthreads();
  best = red[0];
  best_i = red_i[0];
#pragma unroll
  for (int w = 1; w < kSampleThreads / kWave; ++w) take_max(red[w], red_i[w], best, best_i);
  __syncthreads();
}

__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  const int tid = threadIdx.x;
  if ((tid & (kWave - 1)) == 0) red[tid / kWave] = v;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int w = 0; w < kSampleThreads / kWave; ++w) total += red[w];   // every thread the same order
  __syncthreads();
  return total;
}

// Applies f(value, index) to row[lo, hi): aligned groups of four as 16-byte loads, several in
// flight per thread, the ragged ends one by one. A run need not start on a 16-byte boundary.
template <typename F>
__device__ __forceinline__ void for_each_in_run(const float* __restrict__ row, int lo, int hi, F f) {
  const int tid = threadIdx.x;
  const int head = min(hi - lo, static_cast<int>((4 - ((reinterpret_cast<uintptr_t>(row + lo) >> 2) & 3)) & 3));
  const int quads = (hi - lo - head) / 4;
  if (tid < head) f(row[lo + tid], lo + tid);
  const float4* body = reinterpret_cast<const float4*>(row + lo + head);
  constexpr int kInFlight = 4;
  for (int q0 = tid; q0 < quads; q0 += kSampleThreads * kInFlight) {
    float4 v[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) v[u] = body[min(q0 + u * kSampleThreads, quads - 1)];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const int q = q0 + u * kSampleThreads;
      if (q < quads) {
        const int i = lo + head + 4 * q;
        f(v[u].x, i);
        f(v[u].y, i + 1);
        f(v[u].z, i + 2);
        f(v[u].w, i + 3);
      }
    }
  }
  for (int i = lo + head + 4 * quads + tid; i < hi; i += kSampleThreads) f(row[i], i);
}

// grid (runs, rows): statistics of one run of one row.
__global__ __launch_bounds__(kSampleThreads) void sample_runs_kernel(const float* __restrict__ logits,
                                                                    const float* __restrict__ temperature,
                                                                    RunStat* __restrict__ stats, int vocab, int run_len) {
  __shared__ float red[kSampleThreads / kWave];
  __shared__ int32_t red_i[kSampleThreads / kWave];
  const int run = blockIdx.x, r = blockIdx.y;
  const float* row = logits + static_cast<int64_t>(r) * vocab;
  const int lo = run * run_len, hi = min(lo + run_len, vocab);
  float best = -INFINITY;
  int32_t best_i = lo;
  for_each_in_run(row, lo, hi, [&](float v, int32_t i) { take_max(v, i, best, best_i); });
  block_argmax(best, best_i, red, red_i);
  const float temp = temperature[r];
  float total = 0.f;
  if (temp > 0.f) {
    const float inv_t = 1.f / temp;
    float mine = 0.f;
    // The run was just read: this second pass comes from cache.
    for_each_in_run(row, lo, hi, [&](float v, int32_t) { mine += expf((v - best) * inv_t); });
    total = block_sum(mine, red);
  }
  if (threadIdx.x == 0) stats[static_cast<int64_t>(r) * gridDim.x + run] = RunStat{best, best_i, total, 0.f};
}

// grid (rows): combines the runs; for a positive temperature walks the cumulative sum.
__global__ __launch_bounds__(kSampleThreads) void sample_pick_kernel(const float* __restrict__ logits,
                                                                    const float* __restrict__ temperature,
                                                                    const float* __restrict__ uniform,
                                                                    const RunStat* __restrict__ stats,
                                                                    int32_t* __restrict__ out, int vocab, int run_len,
                                                                    int runs) {
  __shared__ float seg_sum[kSampleThreads];
  __shared__ int32_t chosen;
  const int tid = threadIdx.x, r = blockIdx.x;
  const RunStat* st = stats + static_cast<int64_t>(r) * runs;
  float best = -INFINITY;
  int32_t best_i = 0;
  for (int c = 0; c < runs; ++c) take_max(st[c].max, st[c].arg, best, best_i);   // runs in index order: first wins
  const float temp = temperature[r];
  if (!(temp > 0.f)) {
    if (tid == 0) out[r] = best_i;
    return;
  }
  const float inv_t = 1.f / temp;
  // Mass of every run relative to the row's maximum, summed in index order.
  float total = 0.f;
  for (int c = 0; c < runs; ++c) total += st[c].sum * expf((st[c].max - best) * inv_t);
  const float target = uniform[r] * total;
  float before = 0.f;
  int pick_run = runs - 1;
  for (int c = 0; c < runs; ++c) {
    const float mass = st[c].sum * expf((st[c].max - best) * inv_t);
    if (target < before + mass) {
      pick_run = c;
      break;
    }
    if (c < runs - 1) before += mass;
  }
  // Within the run: thread t owns the contiguous segment [lo + t * seg, lo + (t + 1) * seg).
  const float* row = logits + static_cast<int64_t>(r) * vocab;
  const int lo = pick_run * run_len, hi = min(lo + run_len, vocab);
  const int seg = (hi - lo + kSampleThreads - 1) / kSampleThreads;
  const int s_lo = min(lo + tid * seg, hi), s_hi = min(s_lo + seg, hi);
  float mine = 0.f;
  for (int i = s_lo; i < s_hi; ++i) mine += expf((row[i] - best) * inv_t);
  seg_sum[tid] = mine;
  if (tid == 0) chosen = hi - 1;
  __syncthreads();
  float start = before;
  for (int t = 0; t < tid; ++t) start += seg_sum[t];          // exclusive prefix, every thread in index order
  if (start <= target && target < start + mine) {
    float run_sum = start;
    int pick = s_hi - 1;
    for (int i = s_lo; i < s_hi; ++i) {
      run_sum += expf((row[i] - best) * inv_t);
      if (run_sum > target) {
        pick = i;
        break;
      }
    }
    atomicMin(&chosen, pick);
  }
  __syncthreads();
  if (tid == 0) out[r] = min(max(chosen, 0), vocab - 1);
}

// ---- the entry point that allocates nothing --------------------------------------------
//
// The run statistics of psamd_sample_static live in this array instead of a buffer the caller
// brings: kStaticMaxRows rows x kMaxRuns runs x 16 bytes = 128 KiB, held by every GPU the
// library runs on until the process ends. Host code never uses the array's name as an
// address: it asks the runtime once per device for the device's own copy and passes that
// pointer on.
constexpr int kStaticMaxRows = 256;
static __device__ __align__(256) RunStat scratch[kStaticMaxRows * kMaxRuns];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static RunStat* g_scratch_ptr[kMaxDevices] = {};

// The address of `scratch` on the current device, looked up on the first call there.
static int static_scratch(RunStat** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(std::string("psamd_sample_static: hipGetDevice: ") + hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail("psamd_sample_static: device index beyond " + std::to_string(kMaxDevices));
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return fail(std::string("psamd_sample_static: hipGetSymbolAddress: ") + hipGetErrorString(e));
    g_scratch_ptr[dev] = static_cast<RunStat*>(p);
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

static int launch_sample(hipStream_t s, const float* logits, const float* temperature, const float* uniform,
                         int32_t* out, RunStat* stats, int rows, int vocab) {
  // Runs of at least 1024 entries, a multiple of 4 long, at most kMaxRuns of them.
  int run_len = static_cast<int>(ceil_div(vocab, kMaxRuns));
  run_len = std::max(1024, (run_len + 3) & ~3);
  const int runs = static_cast<int>(ceil_div(vocab, run_len));
  sample_runs_kernel<<<dim3(runs, rows), dim3(kSampleThreads), 0, s>>>(logits, temperature, stats, vocab, run_len);
  if (int rc = check_launch("psamd_sample(runs)")) return rc;
  sample_pick_kernel<<<dim3(rows), dim3(kSampleThreads), 0, s>>>(logits, temperature, uniform, stats, out, vocab, run_len,
                                                                runs);
  return check_launch("psamd_sample(pick)");
}

}  // namespace psamd

using namespace psamd;

extern "C" {

// Floats of scratch ``psamd_sample`` needs for this many rows.
int64_t psamd_sample_scratch_floats(int rows) { return static_cast<int64_t>(rows) * kMaxRuns * 4; }

int psamd_sample(void* stream, const float* logits, const float* temperature, const float* uniform, int32_t* out,
                 float* scratch, int rows, int vocab) {
  PSAMD_REQUIRE(rows >= 0 && vocab > 0, "bad sizes");
  PSAMD_REQUIRE(rows <= 65535, "too many rows for one launch");
  if (rows == 0) return 0;
  PSAMD_REQUIRE(scratch != nullptr, "sampling needs its scratch buffer");
  return launch_sample(static_cast<hipStream_t>(stream), logits, temperature, uniform, out,
                       reinterpret_cast<RunStat*>(scratch), rows, vocab);
}

int psamd_sample_static_max_rows(void) { return kStaticMaxRows; }

int psamd_sample_static(void* stream, const float* logits, const float* temperature, const float* uniform,
                        int32_t* out, int rows, int vocab) {
  PSAMD_REQUIRE(rows >= 0 && vocab > 0, "bad sizes");
  PSAMD_REQUIRE(rows <= kStaticMaxRows,
                "at most " + std::to_string(kStaticMaxRows) + " rows fit the built-in scratch array, got " +
                    std::to_string(rows) + " (psamd_sample takes a buffer of any size)");
  if (rows == 0) return 0;
  RunStat* stats = nullptr;
  if (int rc = static_scratch(&stats)) return rc;
  // Nothing has to be cleared: the first kernel writes the statistics of every (row, run) of this
  // call before the second reads exactly those; what an earlier call left beyond them is not read.
  return launch_sample(static_cast<hipStream_t>(stream), logits, temperature, uniform, out, stats, rows, vocab);
}

}  // extern "C"
