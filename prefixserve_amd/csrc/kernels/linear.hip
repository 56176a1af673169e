// Matrix products out[M,N] = x[M,K] * w[N,K]^T (weights are stored [out, in], no bias).
//
// * gemm_tiled: LDS-tiled FMA kernel for any element types with float accumulation. With
//   float everywhere it is the true 32-bit product of the exact path (plain v_fma_f32: no
//   reduced-precision matrix mode is involved); it is also the fallback for shapes the
//   bfloat16 kernels below refuse.
// * skinny_mfma: bfloat16 product for M <= 64 rows (decode steps and small portions). It is
//   bound by reading w once from HBM, so each wave streams 16 rows of w through the
//   16x16x32 matrix-core instruction with the M tokens as the other operand. Optional
//   epilogue: SwiGLU over a fused [gate; up] matrix, or float32 output for logits.

#include "api.h"
#include "common.h"

namespace psamd {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// ------------------------------------------------------------------ tiled FMA GEMM

template <typename TX, typename TW, typename TO>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const TX* __restrict__ x, const TW* __restrict__ w,
                                                         TO* __restrict__ out, int64_t M, int N, int K) {
  constexpr int BM = 64, BN = 64, BK = 16;
  __shared__ float xs[BK][BM + 1];
  __shared__ float wsm[BK][BN + 1];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int64_t m0 = static_cast<int64_t>(blockIdx.y) * BM;
  const int n0 = blockIdx.x * BN;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = tid + i * 256;
      const int r = e / BK, k = e % BK;
      const bool kin = k0 + k < K;
      xs[k][r] = (kin && m0 + r < M) ? to_float<TX>(x[(m0 + r) * K + k0 + k]) : 0.f;
      wsm[k][r] = (kin && n0 + r < N) ? to_float<TW>(w[static_cast<int64_t>(n0 + r) * K + k0 + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = wsm[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) out[m * N + n] = from_float<TO>(acc[i][j]);
    }
  }
}

template <typename TX, typename TW, typename TO>
static int launch_tiled(hipStream_t s, const void* x, const void* w, void* out, int64_t M, int N, int K) {
  dim3 grid(static_cast<unsigned>(ceil_div(N, 64)), static_cast<unsigned>(ceil_div(M, 64)));
  gemm_tiled_kernel<TX, TW, TO><<<grid, dim3(256), 0, s>>>(static_cast<const TX*>(x), static_cast<const TW*>(w),
                                                           static_cast<TO*>(out), M, N, K);
  return check_launch("psamd_linear");
}

// ------------------------------------------------------------------ skinny bf16 (MFMA)

__device__ __forceinline__ bf16x8 load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = static_cast<__bf16>(0.f);
  return z;
}

__device__ __forceinline__ float silu_f(float g) { return g / (1.f + __expf(-g)); }

// Each wave owns 16 output columns (rows of w) and walks all of K. Operand layout of
// v_mfma_f32_16x16x32_bf16: lane l supplies row (l % 16), k = 8 * (l / 16) + [0, 8) of both
// operands, and receives C[4 * (l / 16) + v][l % 16], v = 0..3, where C rows are rows of w
// and C columns are tokens.
// MT = number of 16-token column tiles. SWIGLU: w is [gate; up] with `n_out` rows each and
// the wave computes silu(gate) * up for its 16 columns.
template <int MT, bool SWIGLU, typename TO>
__global__ __launch_bounds__(256) void skinny_mfma_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                          TO* __restrict__ out, int M, int n_out, int K) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * 4 + wave) * 16;
  if (n0 >= n_out) return;
  const int r = lane & 15, g = lane >> 4;
  const int row = min(n0 + r, n_out - 1);
  const bf16_t* wrow = w + static_cast<int64_t>(row) * K;
  const bf16_t* wrow_up = SWIGLU ? w + static_cast<int64_t>(n_out + row) * K : nullptr;
  const bf16_t* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) xrow[mt] = x + static_cast<int64_t>(min(mt * 16 + r, M - 1)) * K;

  f32x4 acc[MT], acc_up[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    acc_up[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int kfull = K & ~31;
#pragma unroll 4
  for (int k0 = 0; k0 < kfull; k0 += 32) {
    const int k = k0 + 8 * g;
    const bf16x8 a = load8(wrow + k);
    bf16x8 a_up;
    if (SWIGLU) a_up = load8(wrow_up + k);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const bf16x8 b = load8(xrow[mt] + k);
      acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[mt], 0, 0, 0);
      if (SWIGLU) acc_up[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_up, b, acc_up[mt], 0, 0, 0);
    }
  }
  if (kfull < K) {  // K % 32 in {8, 16, 24}: lane groups past the end contribute zeros
    const int k = kfull + 8 * g;
    const bool in = k < K;
    const bf16x8 a = in ? load8(wrow + k) : zero8();
    bf16x8 a_up = zero8();
    if (SWIGLU && in) a_up = load8(wrow_up + k);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const bf16x8 b = in ? load8(xrow[mt] + k) : zero8();
      acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[mt], 0, 0, 0);
      if (SWIGLU) acc_up[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_up, b, acc_up[mt], 0, 0, 0);
    }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r;
    if (m >= M) continue;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int n = n0 + 4 * g + v;
      if (n >= n_out) continue;
      float val = acc[mt][v];
      if (SWIGLU) val = silu_f(val) * acc_up[mt][v];
      out[static_cast<int64_t>(m) * n_out + n] = from_float<TO>(val);
    }
  }
}

template <int MT>
static int launch_skinny(hipStream_t s, const void* x, const void* w, void* out, int out_dtype, int M, int n_out,
                         int K, int epilogue) {
  const dim3 grid(static_cast<unsigned>(ceil_div(ceil_div(n_out, 16), 4))), block(256);
  const bf16_t* xp = static_cast<const bf16_t*>(x);
  const bf16_t* wp = static_cast<const bf16_t*>(w);
  if (epilogue == 1) {
    if (out_dtype != kBF16) return fail("psamd_linear_skinny: the SwiGLU epilogue writes bfloat16");
    skinny_mfma_kernel<MT, true, bf16_t><<<grid, block, 0, s>>>(xp, wp, static_cast<bf16_t*>(out), M, n_out, K);
  } else if (out_dtype == kBF16) {
    skinny_mfma_kernel<MT, false, bf16_t><<<grid, block, 0, s>>>(xp, wp, static_cast<bf16_t*>(out), M, n_out, K);
  } else {
    skinny_mfma_kernel<MT, false, float><<<grid, block, 0, s>>>(xp, wp, static_cast<float*>(out), M, n_out, K);
  }
  return check_launch("psamd_linear_skinny");
}

}  // namespace psamd

using namespace psamd;

extern "C" {

int psamd_linear(void* stream, const void* x, int x_dtype, const void* w, int w_dtype, void* out, int out_dtype,
                 int64_t M, int N, int K) {
  PSAMD_REQUIRE(M >= 0 && N > 0 && K > 0, "bad sizes");
  PSAMD_REQUIRE(ceil_div(M, 64) <= 65535, "too many rows for one launch");
  if (M == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (x_dtype == kF32 && w_dtype == kF32 && out_dtype == kF32) return launch_tiled<float, float, float>(s, x, w, out, M, N, K);
  if (x_dtype == kBF16 && w_dtype == kBF16 && out_dtype == kBF16) return launch_tiled<bf16_t, bf16_t, bf16_t>(s, x, w, out, M, N, K);
  if (x_dtype == kBF16 && w_dtype == kBF16 && out_dtype == kF32) return launch_tiled<bf16_t, bf16_t, float>(s, x, w, out, M, N, K);
  return fail("psamd_linear: supported types are (f32,f32)->f32, (bf16,bf16)->bf16 and (bf16,bf16)->f32");
}

// out[M, n_out]; epilogue 0: n_out = rows of w; epilogue 1 (SwiGLU): w has 2 * n_out rows.
int psamd_linear_skinny(void* stream, const void* x, const void* w, void* out, int out_dtype, int M, int n_out, int K,
                        int epilogue) {
  PSAMD_REQUIRE(M >= 1 && M <= 64, "M must be in [1, 64]");
  PSAMD_REQUIRE(n_out > 0 && K > 0 && K % 8 == 0, "K must be a positive multiple of 8");
  PSAMD_REQUIRE(epilogue == 0 || epilogue == 1, "unknown epilogue");
  PSAMD_REQUIRE(out_dtype == kBF16 || out_dtype == kF32, "output must be bfloat16 or float32");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int mt = static_cast<int>(ceil_div(M, 16));
  switch (mt) {
    case 1: return launch_skinny<1>(s, x, w, out, out_dtype, M, n_out, K, epilogue);
    case 2: return launch_skinny<2>(s, x, w, out, out_dtype, M, n_out, K, epilogue);
    case 3: return launch_skinny<3>(s, x, w, out, out_dtype, M, n_out, K, epilogue);
    default: return launch_skinny<4>(s, x, w, out, out_dtype, M, n_out, K, epilogue);
  }
}

}  // extern "C"
