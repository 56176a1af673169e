// A kernel a test's own part brings along: logits capped in place, x <- cap * tanh(x / cap).
// Built by the test with prefixserve_amd.build.build_extension and loaded through
// HipOps.load_extension; nothing in the package knows of it.

#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

__global__ __launch_bounds__(256) void soft_cap_kernel(float* __restrict__ x, int64_t n, float cap) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

}  // namespace

// Returns 0, or 1 for arguments it refuses, or 2 if the launch failed.
extern "C" int toy_soft_cap(void* stream, float* x, int64_t n, float cap) {
  if (x == nullptr || n < 0 || !(cap > 0.f)) return 1;
  if (n == 0) return 0;
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
  soft_cap_kernel<<<dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(x, n, cap);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}
