// Shared device helpers for the gfx950 kernels: bfloat16 <-> float, wave64 reductions,
// error reporting across the C interface.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

namespace psamd {

constexpr int kWave = 64;   // CDNA wavefront
constexpr int kPage = 16;   // tokens per cache page

enum DType : int { kF32 = 0, kBF16 = 1 };

typedef uint16_t bf16_t;    // raw bits; arithmetic is always done in float

__device__ __forceinline__ float bf16_to_float(bf16_t v) { return __uint_as_float(static_cast<uint32_t>(v) << 16); }

// Round to nearest even; NaN stays NaN.
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<bf16_t>((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<bf16_t>(u >> 16);
}

template <typename T> __device__ __forceinline__ float to_float(T v);
template <> __device__ __forceinline__ float to_float<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_float<bf16_t>(bf16_t v) { return bf16_to_float(v); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return float_to_bf16(v); }

// A value read through a pointer whose element type is only known at run time.
__device__ __forceinline__ float load_as_float(const void* p, int dtype, int64_t i) {
  return dtype == kBF16 ? bf16_to_float(static_cast<const bf16_t*>(p)[i]) : static_cast<const float*>(p)[i];
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

// Sum over a block of `nwaves` waves; every thread gets the result. `scratch` holds nwaves floats.
__device__ __forceinline__ float block_sum(float v, float* scratch, int nwaves) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  __syncthreads();
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nwaves; ++i) t += scratch[i];
  return t;
}

__device__ __forceinline__ float block_max(float v, float* scratch, int nwaves) {
  v = wave_max(v);
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  __syncthreads();
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  float t = scratch[0];
  for (int i = 1; i < nwaves; ++i) t = fmaxf(t, scratch[i]);
  return t;
}

// ---- host side ----

void set_error(const std::string& msg);

inline int fail(const std::string& msg) {
  set_error(msg);
  return 1;
}

inline int check_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(std::string(what) + ": " + hipGetErrorString(e));
  return 0;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace psamd

#define PSAMD_REQUIRE(cond, msg) \
  do {                           \
    if (!(cond)) return psamd::fail(std::string(__func__) + ": " + (msg)); \
  } while (0)
