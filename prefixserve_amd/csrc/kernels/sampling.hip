// Next-token choice from float32 logits: greedy (lowest index among equal maxima) and
// temperature sampling by inverse CDF of softmax(logits / T) in vocabulary order. The
// uniform number of each row comes from the host, a function of (seed, request, output
// index) only, so a recomputed request draws the same token.

#include "api.h"
#include "common.h"

namespace psamd {

constexpr int kSampleThreads = 1024;

// One block per row. Thread t owns the contiguous segment [t * seg, (t + 1) * seg).
__global__ __launch_bounds__(kSampleThreads) void sample_kernel(const float* __restrict__ logits,
                                                                const float* __restrict__ temperature,
                                                                const float* __restrict__ uniform,
                                                                int32_t* __restrict__ out, int vocab) {
  __shared__ float red[kSampleThreads / kWave];
  __shared__ int32_t red_i[kSampleThreads / kWave];
  __shared__ float seg_sum[kSampleThreads];
  __shared__ int32_t chosen;
  const int tid = threadIdx.x;
  const float* row = logits + static_cast<int64_t>(blockIdx.x) * vocab;
  const float temp = temperature[blockIdx.x];

  // ---- max and its first index. The body of the row is read as aligned groups of four,
  // several loads in flight per thread; a row need not start on a 16-byte boundary.
  float best = -INFINITY;
  int32_t best_i = 0x7fffffff;
  auto take = [&](float v, int32_t i) {
    if (v > best || (v == best && i < best_i)) {
      best = v;
      best_i = i;
    }
  };
  const int head = min(vocab, static_cast<int>((4 - ((reinterpret_cast<uintptr_t>(row) >> 2) & 3)) & 3));
  const int quads = (vocab - head) / 4;
  if (tid < head) take(row[tid], tid);
  const float4* body = reinterpret_cast<const float4*>(row + head);
  constexpr int kInFlight = 4;
  for (int q0 = tid; q0 < quads; q0 += kSampleThreads * kInFlight) {
    float4 v[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const int q = q0 + u * kSampleThreads;
      v[u] = body[min(q, quads - 1)];
    }
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const int q = q0 + u * kSampleThreads;
      if (q < quads) {
        const int i = head + 4 * q;
        take(v[u].x, i);
        take(v[u].y, i + 1);
        take(v[u].z, i + 2);
        take(v[u].w, i + 3);
      }
    }
  }
  for (int i = head + 4 * quads + tid; i < vocab; i += kSampleThreads) take(row[i], i);
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o, kWave);
    const int32_t oi = __shfl_xor(best_i, o, kWave);
    if (ob > best || (ob == best && oi < best_i)) {
      best = ob;
      best_i = oi;
    }
  }
  if ((tid & (kWave - 1)) == 0) {
    red[tid / kWave] = best;
    red_i[tid / kWave] = best_i;
  }
  __syncthreads();
  best = red[0];
  best_i = red_i[0];
  for (int w = 1; w < kSampleThreads / kWave; ++w) {
    if (red[w] > best || (red[w] == best && red_i[w] < best_i)) {
      best = red[w];
      best_i = red_i[w];
    }
  }
  if (!(temp > 0.f)) {
    if (tid == 0) out[blockIdx.x] = best_i;
    return;
  }

  // ---- segment sums of exp((x - max) / T)
  const float inv_t = 1.f / temp;
  const int seg = (vocab + kSampleThreads - 1) / kSampleThreads;
  const int lo = min(tid * seg, vocab), hi = min(lo + seg, vocab);
  float mine = 0.f;
  for (int i = lo; i < hi; ++i) mine += expf((row[i] - best) * inv_t);
  seg_sum[tid] = mine;
  if (tid == 0) chosen = vocab - 1;
  __syncthreads();
  // Exclusive prefix over the 1024 segment sums, in index order (every thread the same way).
  float before = 0.f, total = 0.f;
  for (int t = 0; t < kSampleThreads; ++t) {
    if (t == tid) before = total;
    total += seg_sum[t];
  }
  const float target = uniform[blockIdx.x] * total;
  // The segment in which the running sum first exceeds the target rescans itself.
  if (before <= target && target < before + mine) {
    float run = before;
    int pick = hi - 1;
    for (int i = lo; i < hi; ++i) {
      run += expf((row[i] - best) * inv_t);
      if (run > target) {
        pick = i;
        break;
      }
    }
    atomicMin(&chosen, pick);
  }
  __syncthreads();
  if (tid == 0) out[blockIdx.x] = chosen;
}

}  // namespace psamd

using namespace psamd;

extern "C" int psamd_sample(void* stream, const float* logits, const float* temperature, const float* uniform,
                            int32_t* out, int rows, int vocab) {
  PSAMD_REQUIRE(rows >= 0 && vocab > 0, "bad sizes");
  if (rows == 0) return 0;
  sample_kernel<<<dim3(rows), dim3(kSampleThreads), 0, static_cast<hipStream_t>(stream)>>>(logits, temperature,
                                                                                           uniform, out, vocab);
  return check_launch("psamd_sample");
}
