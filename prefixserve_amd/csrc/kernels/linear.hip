// Matrix products out[M,N] = x[M,K] * w[N,K]^T (weights are stored [out, in], no bias).
//
// * gemm_tiled: LDS-tiled FMA kernel for any element types with float accumulation. With
//   float everywhere it is the true 32-bit product of the exact path (plain v_fma_f32: no
//   reduced-precision matrix mode is involved); it is also the fallback for shapes the
//   bfloat16 kernels below refuse.
// * rows_f32: the 32-bit product for up to 16 tokens (decode steps), in the tiled kernel's order of summation.
// * skinny_mfma: bfloat16 product for M <= 64 rows (decode steps and small portions). It is
//   bound by reading w once from HBM, so each wave streams 16 rows of w through the
//   16x16x32 matrix-core instruction with the M tokens as the other operand. Optional
//   epilogue: SwiGLU over a fused [gate; up] matrix, or float32 output for logits.

#include <algorithm>
#include <string>

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

// ------------------------------------------------------------------ float32, a few tokens

// The 32-bit product for up to 16 tokens (decode steps), where the tiled kernel above would
// leave most of its 64-token tile and most of the chip idle. A workgroup owns 16 rows of w;
// thread (row, token) sums its products over k in ascending order with one fused multiply-add
// each, exactly the order of the tiled kernel: a position's 32-bit result is the same bit for
// bit whether its step had 1 token or 1,000, which is what lets tests of the 32-bit path
// demand equality between different ways of cutting a sequence. The next 64-wide piece of
// w and x is on its way from memory while the current one is summed from LDS. K % 4 == 0.
__global__ __launch_bounds__(256) void rows_f32_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                       float* __restrict__ out, int M, int N, int K) {
  constexpr int BK = 64, LD = BK + 4;
  __shared__ __align__(16) float ws[16][LD];
  __shared__ __align__(16) float xs[16][LD];
  const int tid = threadIdx.x;
  const int r = tid & 15, m = tid >> 4;            // the output this thread sums
  const int lr = tid >> 4, lc = (tid & 15) * 4;    // the 16-byte piece this thread brings in
  const int n0 = blockIdx.x * 16;
  const float4 zero = float4{0.f, 0.f, 0.f, 0.f};
  const float* wsrc = w + static_cast<int64_t>(min(n0 + lr, N - 1)) * K + lc;
  const float* xsrc = x + static_cast<int64_t>(min(lr, M - 1)) * K + lc;
  float4 wv = lc < K ? *reinterpret_cast<const float4*>(wsrc) : zero;
  float4 xv = lc < K ? *reinterpret_cast<const float4*>(xsrc) : zero;
  float acc = 0.f;
  for (int k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();                               // the previous piece has been summed
    *reinterpret_cast<float4*>(&ws[lr][lc]) = wv;
    *reinterpret_cast<float4*>(&xs[lr][lc]) = xv;
    __syncthreads();
    const int kn = k0 + BK + lc;
    wv = kn < K ? *reinterpret_cast<const float4*>(wsrc + k0 + BK) : zero;
    xv = kn < K ? *reinterpret_cast<const float4*>(xsrc + k0 + BK) : zero;
#pragma unroll
    for (int kk = 0; kk < BK; kk += 4) {
      const float4 a = *reinterpret_cast<const float4*>(&ws[r][kk]);
      const float4 b = *reinterpret_cast<const float4*>(&xs[m][kk]);
      acc = fmaf(b.x, a.x, acc);
      acc = fmaf(b.y, a.y, acc);
      acc = fmaf(b.z, a.z, acc);
      acc = fmaf(b.w, a.w, acc);
    }
  }
  if (m < M && n0 + r < N) out[static_cast<int64_t>(m) * N + n0 + r] = acc;
}

static int launch_rows_f32(hipStream_t s, const void* x, const void* w, void* out, int M, int N, int K) {
  const dim3 grid(static_cast<unsigned>(ceil_div(N, 16)));
  rows_f32_kernel<<<grid, dim3(256), 0, s>>>(static_cast<const float*>(x), static_cast<const float*>(w),
                                             static_cast<float*>(out), M, N, K);
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

// *p += v, done by the memory side, nothing returned: the way K-slices of different workgroups,
// on any die, add into one float32 sum.
__device__ __forceinline__ void add_to(float* p, float v) { (void)unsafeAtomicAdd(p, v); }
template <typename T>
__device__ __forceinline__ void add_to(T*, float) {}

// Streams rows of w through v_mfma_f32_16x16x32_bf16 with the M tokens as the other operand.
// Two ways to lay the work over a workgroup's 4 waves:
//  * SPLIT (few output columns): the workgroup owns 16 rows of w and a range of K; its waves
//    take the 32-wide k-steps of that range in turn and their partial tiles are summed
//    through LDS. With gridDim.y > 1 the K range is also split over workgroups and float
//    partial sums go to out[blockIdx.y][M][n_out] for the consumer (the fused add+norm) to add
//    up: that is how a product with few output columns still fills the chip.
//  * !SPLIT (many output columns): every wave owns 16 rows of its own over all of K; the 4
//    waves read the same tokens at the same time, so x comes from L1 rather than L2.
// Loads are issued U steps ahead of the matrix instructions that use them: the kernel is
// bound by memory latency unless many loads are in flight.
//
// Operand layout: lane l supplies row (l % 16), k = 8 * (l / 16) + [0, 8) of both operands
// and receives C[4 * (l / 16) + v][l % 16], v = 0..3; C rows are rows of w, C columns are
// tokens. MT = number of 16-token column tiles. SWIGLU: w is [gate; up] with n_out rows each
// and the result is silu(gate) * up.
// RT = 16-row tiles of w per wave (2 when there are more than 16 tokens: the tokens loaded
// for a k-step then serve twice as many rows, halving the traffic for x, which for 64 tokens
// would otherwise be four times that for w).
// WV = waves of a workgroup (8 with many tokens: more k-slices in flight per workgroup).
// U = k-steps whose loads are in flight together.
constexpr int skinny_depth(int mt, int rt) { return mt == 1 ? 8 : (mt * rt <= 2 ? 4 : (mt * rt <= 8 ? 2 : 1)); }

// ATOMIC (float32 output, plain epilogue): every K-slice adds its partial sums into the one
// out[M][n_out] with float atomics that return nothing, instead of writing a slice of its own:
// out is the residual stream, and no kernel has to add the slices up afterwards. The order of
// the additions, and with it the last bit of the sums, differs from run to run.
template <int MT, int RT, int WV, bool SWIGLU, bool SPLIT, typename TO, int U = skinny_depth(MT, RT), bool ATOMIC = false>
__global__ __launch_bounds__(64 * WV) void skinny_mfma_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                          TO* __restrict__ out, int M, int n_out, int K) {
  constexpr int NACC = SWIGLU ? 2 * MT : MT;
  __shared__ f32x4 red[SPLIT ? WV : 1][NACC][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile0 = (SPLIT ? blockIdx.x : blockIdx.x * WV + wave) * RT;
  if (!SPLIT && tile0 * 16 >= n_out) return;
  const int r = lane & 15, g = lane >> 4;
  const bf16_t* wrow[RT];
  const bf16_t* wrow_up[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int row = min((tile0 + rt) * 16 + r, n_out - 1);
    wrow[rt] = w + static_cast<int64_t>(row) * K + 8 * g;
    wrow_up[rt] = SWIGLU ? w + static_cast<int64_t>(n_out + row) * K + 8 * g : nullptr;
  }
  const bf16_t* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) xrow[mt] = x + static_cast<int64_t>(min(mt * 16 + r, M - 1)) * K + 8 * g;

  f32x4 acc[RT][NACC];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[rt][i] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int steps = (K + 31) >> 5;
  const int per_wg = (steps + gridDim.y - 1) / gridDim.y;
  const int s_begin = blockIdx.y * per_wg;
  const int s_end = min(s_begin + per_wg, steps);
  const int s_full = min(s_end, K >> 5);          // steps that lie wholly inside K
  const int stride = SPLIT ? WV : 1;
  for (int base = s_begin + (SPLIT ? wave : 0); base < s_full; base += stride * U) {
    bf16x8 a[RT][U], a_up[RT][U], b[MT][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = base + stride * u;
      if (s < s_full) {
        const int k = s << 5;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          a[rt][u] = load8(wrow[rt] + k);
          if (SWIGLU) a_up[rt][u] = load8(wrow_up[rt] + k);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) b[mt][u] = load8(xrow[mt] + k);
      } else {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          a[rt][u] = zero8();
          if (SWIGLU) a_up[rt][u] = zero8();
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) b[mt][u] = zero8();
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          acc[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rt][u], b[mt][u], acc[rt][mt], 0, 0, 0);
          if (SWIGLU)
            acc[rt][MT + mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_up[rt][u], b[mt][u], acc[rt][MT + mt], 0, 0, 0);
        }
      }
    }
  }
  // K % 32 in {8, 16, 24}: the last step is partial; lane groups past the end contribute zeros.
  if (s_full < s_end && (!SPLIT || ((s_full - s_begin) % WV) == wave)) {
    const int k = s_full << 5;
    const bool in = k + 8 * g < K;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const bf16x8 a = in ? load8(wrow[rt] + k) : zero8();
      bf16x8 a_up = zero8();
      if (SWIGLU && in) a_up = load8(wrow_up[rt] + k);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const bf16x8 b = in ? load8(xrow[mt] + k) : zero8();
        acc[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[rt][mt], 0, 0, 0);
        if (SWIGLU) acc[rt][MT + mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_up, b, acc[rt][MT + mt], 0, 0, 0);
      }
    }
  }

  auto finish = [&](int rt, int mt, f32x4 sum, f32x4 up) {
    if (SWIGLU) {
#pragma unroll
      for (int v = 0; v < 4; ++v) sum[v] = silu_f(sum[v]) * up[v];
    }
    const int m = mt * 16 + r;
    if (m >= M) return;
    TO* dst = out + (static_cast<int64_t>(ATOMIC ? 0 : blockIdx.y) * M + m) * n_out;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int n = (tile0 + rt) * 16 + 4 * g + v;
      if (n >= n_out) continue;
      if constexpr (ATOMIC) add_to(dst + n, sum[v]);
      else dst[n] = from_float<TO>(sum[v]);
    }
  };

  if (!SPLIT) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) finish(rt, mt, acc[rt][mt], SWIGLU ? acc[rt][MT + mt] : acc[rt][mt]);
    return;
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    if (rt > 0) __syncthreads();
#pragma unroll
    for (int i = 0; i < NACC; ++i) red[wave][i][lane] = acc[rt][i];
    __syncthreads();
    // Wave `wave` finishes column tile `wave` (MT <= 4: at most one each).
    if (wave < MT) {
      const int mt = wave;
      f32x4 sum = red[0][mt][lane];
#pragma unroll
      for (int w2 = 1; w2 < WV; ++w2) sum += red[w2][mt][lane];
      f32x4 up = sum;
      if (SWIGLU) {
        up = red[0][MT + mt][lane];
#pragma unroll
        for (int w2 = 1; w2 < WV; ++w2) up += red[w2][MT + mt][lane];
      }
      finish(rt, mt, sum, up);
    }
  }
}

// Where the tokens of a small step come from: bfloat16 rows x[M][K], or (x == nullptr) rows of the
// float32 residual stream that the kernel normalizes itself on the way in (RMS norm: statistics
// in 32-bit, eps inside the root, times the norm's weight), row rows[m] for token m (rows ==
// nullptr: row m). A kernel that reads its tokens this way needs no norm kernel in front of it.
struct Tokens {
  const bf16_t* x;
  const float* resid;
  const void* norm_w;
  const int32_t* rows;
  float eps;
  int norm_w_bf16;      // the norm's weight is bfloat16 (else float32)
};

// Stages the M <= ROWS tokens of a small step in LDS for a workgroup of WV waves, from rows of
// the float32 residual stream: xs[row][k] = bfloat16(resid[row][k] * norm_w[k]), and the rows'
// sums of squares, from which stage_scale() gives 1 / sqrt(mean(resid[row]^2) + eps) once a
// barrier has passed. The caller multiplies its sums by that (the product is linear in the tokens,
// so a row's scale may wait until the end). With few tokens a row is dealt out to several waves
// (8 for one token, 4 for two, 2 up to four), so that a single token's row is not one wave's
// work while seven wait; each leaves its part of the row's sum in ss[row][part]. Rows from M on
// are zeros. K must be a multiple of 8.
template <int WV>
__device__ __forceinline__ int stage_waves_per_row(int M) {
  return M <= 1 ? WV : (M <= 2 ? WV / 2 : (M <= 4 ? WV / 4 : 1));
}

template <int ROWS, int WV>
__device__ __forceinline__ void stage_normed(const Tokens& tk, bf16_t* xs, int XS, float* ss, int M, int K, int wave,
                                             int lane) {
  const int wpr = stage_waves_per_row<WV>(M);
  const int pieces = K >> 3;                               // 8 elements each
  for (int i = threadIdx.x; i < (ROWS - M) * pieces; i += 64 * WV) {
    const int row = M + i / pieces, c = i - (row - M) * pieces;
    *reinterpret_cast<bf16x8*>(xs + row * XS + 8 * c) = zero8();
  }
  const int per_part = (pieces + wpr - 1) / wpr;
  for (int job = wave; job < ROWS * wpr; job += WV) {
    const int row = job / wpr, part = job - row * wpr;
    if (row >= M) break;
    bf16_t* dst = xs + row * XS;
    const float* src = tk.resid + static_cast<int64_t>(tk.rows != nullptr ? tk.rows[row] : row) * K;
    const int c_end = min(pieces, (part + 1) * per_part);
    float sum = 0.f;
#pragma unroll 4
    for (int c = part * per_part + lane; c < c_end; c += 64) {
      const float4 a = *reinterpret_cast<const float4*>(src + 8 * c);
      const float4 b = *reinterpret_cast<const float4*>(src + 8 * c + 4);
      float wn[8];
      if (tk.norm_w_bf16) {
        const bf16x8 wv = load8(static_cast<const bf16_t*>(tk.norm_w) + 8 * c);
#pragma unroll
        for (int i = 0; i < 8; ++i) wn[i] = static_cast<float>(wv[i]);
      } else {
        const float4 w0 = *reinterpret_cast<const float4*>(static_cast<const float*>(tk.norm_w) + 8 * c);
        const float4 w1 = *reinterpret_cast<const float4*>(static_cast<const float*>(tk.norm_w) + 8 * c + 4);
        wn[0] = w0.x, wn[1] = w0.y, wn[2] = w0.z, wn[3] = w0.w, wn[4] = w1.x, wn[5] = w1.y, wn[6] = w1.z, wn[7] = w1.w;
      }
      const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
      bf16x8 o;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        sum = fmaf(v[i], v[i], sum);
        o[i] = static_cast<__bf16>(v[i] * wn[i]);
      }
      *reinterpret_cast<bf16x8*>(dst + 8 * c) = o;
    }
    sum = wave_sum(sum);
    if (lane == 0) ss[row * WV + part] = sum;
  }
}

// The scale of token `row` (after the barrier behind stage_normed).
template <int WV>
__device__ __forceinline__ float stage_scale(const Tokens& tk, const float* ss, int row, int M, int K) {
  if (row >= M) return 0.f;
  const int wpr = stage_waves_per_row<WV>(M);
  float sum = 0.f;
  for (int p = 0; p < wpr; ++p) sum += ss[row * WV + p];
  return rsqrtf(sum / static_cast<float>(K) + tk.eps);
}

// Up to 16 tokens as workgroups that stay: each stages its tokens in LDS once (ROWS = 8 or 16
// rows of its slice of K; in the kernel above every workgroup reads them again from L2 for its
// one or two row tiles, as many bytes as the rows themselves at two tiles) and then takes groups
// of RT row tiles in turn, gridDim.x apart. Its eight waves split the slice as above, a wave's
// k-steps of all RT tiles in flight together; the partial sums meet in LDS and wave rt finishes
// tile rt. gridDim.y slices of K give partial sums out[blockIdx.y][M][n_out], as above. SWIGLU:
// w is [gate; up] and a group is RT pairs of tiles. K must be a multiple of 32.
// NORMED: the tokens are rows of the float32 residual stream, normalized while they are staged
// (gridDim.y must be 1: a row's statistics need the whole row). ATOMIC: the K-slices add into one
// out[M][n_out] (see skinny_mfma_kernel).
template <int RT, int ROWS, bool SWIGLU, typename TO, bool NORMED = false, bool ATOMIC = false>
__global__ __launch_bounds__(512) void stream_kernel(Tokens tk, const bf16_t* __restrict__ w,
                                                  TO* __restrict__ out, int M, int n_out, int K, int groups) {
  constexpr int WV = 8, U = 8, NACC = SWIGLU ? 2 : 1;
  extern __shared__ __align__(16) unsigned char stream_smem[];
  const int steps_all = K >> 5;
  const int per_slice = (steps_all + gridDim.y - 1) / gridDim.y;
  const int s_begin = blockIdx.y * per_slice;
  const int steps = max(0, min(per_slice, steps_all - s_begin));   // k-steps of this workgroup's slice (none: it writes zeros)
  const int XS = per_slice * 32 + 8;                          // elements per token row in LDS (padded: rows on different banks)
  bf16_t* xs = reinterpret_cast<bf16_t*>(stream_smem);
  f32x4* red = reinterpret_cast<f32x4*>(stream_smem + static_cast<size_t>(ROWS) * XS * sizeof(bf16_t));   // [WV][RT][NACC][64]
  float* ss = reinterpret_cast<float*>(red + WV * RT * NACC * 64);                                         // [ROWS][WV] (NORMED)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  // (Asking for the first group's rows of w before or while the tokens are staged was measured
  // and lost: the registers that hold them cost the second workgroup of a compute unit, or spill.)
  if constexpr (NORMED) {
    stage_normed<ROWS, WV>(tk, xs, XS, ss, M, K, wave, lane);
  } else {
    const int pieces = steps * 4;                             // 16-byte pieces of a row's slice
    const bf16_t* x0 = tk.x + (static_cast<int64_t>(s_begin) << 5);
    for (int p = threadIdx.x; p < ROWS * pieces; p += blockDim.x) {
      const int row = p / pieces, c = p - row * pieces;
      bf16x8 v = zero8();
      if (row < M) v = load8(x0 + static_cast<int64_t>(row) * K + 8 * c);
      *reinterpret_cast<bf16x8*>(xs + row * XS + 8 * c) = v;
    }
  }
  __syncthreads();
  // With ROWS = 8, lanes 8..15 of a group repeat tokens 0..7: their columns of the result are not stored.
  const bf16_t* xl = xs + (r % ROWS) * XS + 8 * g;
  const bf16_t* w0 = w + (static_cast<int64_t>(s_begin) << 5) + 8 * g;
  const float row_scale = NORMED ? stage_scale<WV>(tk, ss, r % ROWS, M, K) : 1.f;
  for (int grp = blockIdx.x; grp < groups; grp += gridDim.x) {
    const int tile0 = grp * RT;
    const bf16_t* wrow[RT];
    const bf16_t* wrow_up[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int row = min((tile0 + rt) * 16 + r, n_out - 1);
      wrow[rt] = w0 + static_cast<int64_t>(row) * K;
      wrow_up[rt] = SWIGLU ? w0 + static_cast<int64_t>(n_out + row) * K : nullptr;
    }
    f32x4 acc[RT][NACC];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < NACC; ++i) acc[rt][i] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int base = wave; base < steps; base += WV * U) {
      bf16x8 a[RT][U], a_up[RT][U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int st = base + WV * u;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          a[rt][u] = st < steps ? load8(wrow[rt] + (st << 5)) : zero8();
          if (SWIGLU) a_up[rt][u] = st < steps ? load8(wrow_up[rt] + (st << 5)) : zero8();
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int st = min(base + WV * u, steps - 1);      // past the end: the row tiles are zeros
        const bf16x8 b = *reinterpret_cast<const bf16x8*>(xl + (st << 5));
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          acc[rt][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rt][u], b, acc[rt][0], 0, 0, 0);
          if (SWIGLU) acc[rt][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_up[rt][u], b, acc[rt][1], 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < NACC; ++i) red[((wave * RT + rt) * NACC + i) * 64 + lane] = acc[rt][i];
    __syncthreads();
    if (wave < RT) {
      const int rt = wave;
      f32x4 sum = red[(rt * NACC) * 64 + lane];
#pragma unroll
      for (int w2 = 1; w2 < WV; ++w2) sum += red[((w2 * RT + rt) * NACC) * 64 + lane];
      if (NORMED) sum *= row_scale;
      if (SWIGLU) {
        f32x4 up = red[(rt * NACC + 1) * 64 + lane];
#pragma unroll
        for (int w2 = 1; w2 < WV; ++w2) up += red[((w2 * RT + rt) * NACC + 1) * 64 + lane];
        if (NORMED) up *= row_scale;
#pragma unroll
        for (int v = 0; v < 4; ++v) sum[v] = silu_f(sum[v]) * up[v];
      }
      if (r < M) {
        TO* dst = out + (static_cast<int64_t>(ATOMIC ? 0 : blockIdx.y) * M + r) * n_out;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int n = (tile0 + rt) * 16 + 4 * g + v;
          if (n >= n_out) continue;
          if constexpr (ATOMIC) add_to(dst + n, sum[v]);
          else dst[n] = from_float<TO>(sum[v]);
        }
      }
    }
    __syncthreads();      // the sums are read before the next group's are written
  }
}

// Bytes of LDS stream_kernel needs.
static size_t stream_smem_bytes(int rt, int rows, bool swiglu, int K, int ksplit) {
  const int per_slice = static_cast<int>(ceil_div(K >> 5, ksplit));
  return static_cast<size_t>(rows) * (per_slice * 32 + 8) * sizeof(bf16_t) + sizeof(f32x4) * 8 * rt * (swiglu ? 2 : 1) * 64 +
         sizeof(float) * rows * 8;
}

static Tokens plain_tokens(const void* x) { return Tokens{static_cast<const bf16_t*>(x), nullptr, nullptr, nullptr, 0.f, 0}; }

// workgroups: how many may stay per K-slice; the groups are dealt out evenly over them.
template <int RT, int ROWS, bool SWIGLU, bool NORMED = false, bool ATOMIC = false>
static int launch_stream(hipStream_t s, const Tokens& tk, const void* w, void* out, int out_dtype, int M, int n_out, int K,
                         int ksplit, int workgroups) {
  const int groups = static_cast<int>(ceil_div(ceil_div(n_out, 16), RT));
  const size_t smem = stream_smem_bytes(RT, ROWS, SWIGLU, K, ksplit);
  const int rounds = static_cast<int>(ceil_div(groups, workgroups));
  const dim3 grid(static_cast<unsigned>(ceil_div(groups, rounds)), static_cast<unsigned>(ksplit)), block(512);
  const bf16_t* wp = static_cast<const bf16_t*>(w);
  auto run = [&](auto kernel, auto* dst) {
    if (smem > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                static_cast<int>(smem)) != hipSuccess) {
      set_error("psamd_linear_skinny: " + std::to_string(smem) + " bytes of LDS were refused");
      return -1;
    }
    kernel<<<grid, block, smem, s>>>(tk, wp, dst, M, n_out, K, groups);
    return check_launch("psamd_linear_skinny");
  };
  if constexpr (ATOMIC) {
    return run(stream_kernel<RT, ROWS, false, float, NORMED, true>, static_cast<float*>(out));
  } else {
    if (SWIGLU || out_dtype == kBF16) return run(stream_kernel<RT, ROWS, SWIGLU, bf16_t, NORMED>, static_cast<bf16_t*>(out));
    return run(stream_kernel<RT, ROWS, false, float, NORMED>, static_cast<float*>(out));
  }
}

template <int MT, int RT, int WV, bool SWIGLU, bool SPLIT>
static int launch_skinny2(hipStream_t s, const void* x, const void* w, void* out, int out_dtype, int M, int n_out,
                          int K, int ksplit) {
  const int64_t groups = ceil_div(ceil_div(n_out, 16), RT);
  const dim3 grid(static_cast<unsigned>(SPLIT ? groups : ceil_div(groups, WV)), static_cast<unsigned>(ksplit)), block(64 * WV);
  const bf16_t* xp = static_cast<const bf16_t*>(x);
  const bf16_t* wp = static_cast<const bf16_t*>(w);
  if constexpr (SWIGLU) {
    skinny_mfma_kernel<MT, RT, WV, true, SPLIT, bf16_t><<<grid, block, 0, s>>>(xp, wp, static_cast<bf16_t*>(out), M, n_out, K);
  } else if (out_dtype == kBF16) {
    skinny_mfma_kernel<MT, RT, WV, false, SPLIT, bf16_t><<<grid, block, 0, s>>>(xp, wp, static_cast<bf16_t*>(out), M, n_out, K);
  } else {
    skinny_mfma_kernel<MT, RT, WV, false, SPLIT, float><<<grid, block, 0, s>>>(xp, wp, static_cast<float*>(out), M, n_out, K);
  }
  return check_launch("psamd_linear_skinny");
}

// Row tiles per wave and waves per workgroup for MT column tiles of tokens. With more than
// 32 tokens the tokens are most of a k-step's loads: a wave then takes four row tiles (the
// SwiGLU form two of gate and two of up) and a workgroup eight k-slices.
constexpr int skinny_rt(int mt, bool swiglu) { return mt == 1 ? 1 : (mt == 2 || swiglu ? 2 : 4); }
constexpr int skinny_wv(int mt) { return mt <= 2 ? 4 : 8; }

// A product with very many output columns (the output matrix over the vocabulary) has row
// groups to spare: from 9 tokens on a wave then takes more row tiles, so that the tokens, which
// every workgroup reads again from L2, are a smaller share of its loads (measured at 128,256
// columns: 137 -> 121 us at 16 tokens, 160 -> 130 at 32, 168 -> 152 at 64).
constexpr int kManyRowTiles = 4096;
constexpr int wide_rt(int mt) { return mt == 1 ? 4 : 8; }
constexpr int wide_wv(int mt) { return (mt == 1 || mt == 3) ? 8 : 4; }
constexpr int wide_depth(int mt) { return mt <= 2 ? 2 : 1; }

template <int MT, bool SWIGLU>
static int launch_skinny1(hipStream_t s, const void* x, const void* w, void* out, int out_dtype, int M, int n_out,
                          int K, int ksplit) {
  if constexpr (!SWIGLU && MT == 1) {
    // Up to 8 tokens and row groups to spare (the output matrix): one row tile (two from 5 tokens
    // on) per workgroup of eight waves that split K, every wave's eight k-steps in flight at once.
    // Against four waves with a row tile each over all of K, at 128,256 columns and K = 2,048:
    // 93 -> 84 us at 1 token, 95 -> 87 at 2, 101 -> 96 at 4, 113 -> 111 at 8; the same order at
    // K = 4,096 (193 -> 172 us at 1 token).
    // From 2 tokens on the workgroups that stay and keep the tokens in LDS are faster (128,256
    // columns, K = 2,048: 93 -> 92 us at 2 tokens, 102 -> 94 at 4, 112 -> 98 at 8, 125 -> 108
    // at 16; K = 4,096: 202 -> 175 at 4, 221 -> 181 at 8): two row tiles per group and two
    // workgroups per compute unit while the tokens are 32 KB, else one and four.
    if (M >= (K <= 2048 ? 4 : 2) && M <= 16 && ksplit == 1 && ceil_div(n_out, 16) >= 2048 && K % 32 == 0) {
      const int rows = M <= 8 ? 8 : 16;
      const bool small = static_cast<int64_t>(rows) * K <= 8 * 2048;
      if (stream_smem_bytes(small ? 2 : 1, rows, false, K, 1) <= 160 * 1024) {
        if (rows == 8) {
          if (small) return launch_stream<2, 8, false>(s, plain_tokens(x), w, out, out_dtype, M, n_out, K, 1, 512);
          return launch_stream<1, 8, false>(s, plain_tokens(x), w, out, out_dtype, M, n_out, K, 1, 1024);
        }
        if (small) return launch_stream<2, 16, false>(s, plain_tokens(x), w, out, out_dtype, M, n_out, K, 1, 512);
        return launch_stream<1, 16, false>(s, plain_tokens(x), w, out, out_dtype, M, n_out, K, 1, 1024);
      }
    }
    if (M <= 8 && ksplit == 1 && ceil_div(n_out, 16) >= 2048) {
      const bf16_t* xp = static_cast<const bf16_t*>(x);
      const bf16_t* wp = static_cast<const bf16_t*>(w);
      const dim3 block(64 * 8);
      if (M <= 4) {
        const dim3 grid(static_cast<unsigned>(ceil_div(n_out, 16)), 1u);
        if (out_dtype == kBF16) skinny_mfma_kernel<1, 1, 8, false, true, bf16_t, 8><<<grid, block, 0, s>>>(xp, wp, static_cast<bf16_t*>(out), M, n_out, K);
        else skinny_mfma_kernel<1, 1, 8, false, true, float, 8><<<grid, block, 0, s>>>(xp, wp, static_cast<float*>(out), M, n_out, K);
      } else {
        const dim3 grid(static_cast<unsigned>(ceil_div(ceil_div(n_out, 16), 2)), 1u);
        if (out_dtype == kBF16) skinny_mfma_kernel<1, 2, 8, false, true, bf16_t, 8><<<grid, block, 0, s>>>(xp, wp, static_cast<bf16_t*>(out), M, n_out, K);
        else skinny_mfma_kernel<1, 2, 8, false, true, float, 8><<<grid, block, 0, s>>>(xp, wp, static_cast<float*>(out), M, n_out, K);
      }
      return check_launch("psamd_linear_skinny");
    }
  }
  if constexpr (!SWIGLU) {
    if (M > 8 && ksplit == 1 && ceil_div(n_out, 16) >= kManyRowTiles) {
      constexpr int RT = wide_rt(MT), WV = wide_wv(MT), U = wide_depth(MT);
      const dim3 grid(static_cast<unsigned>(ceil_div(ceil_div(n_out, 16), RT)), 1u), block(64 * WV);
      const bf16_t* xp = static_cast<const bf16_t*>(x);
      const bf16_t* wp = static_cast<const bf16_t*>(w);
      if (out_dtype == kBF16) {
        skinny_mfma_kernel<MT, RT, WV, false, true, bf16_t, U><<<grid, block, 0, s>>>(xp, wp, static_cast<bf16_t*>(out), M, n_out, K);
      } else {
        skinny_mfma_kernel<MT, RT, WV, false, true, float, U><<<grid, block, 0, s>>>(xp, wp, static_cast<float*>(out), M, n_out, K);
      }
      return check_launch("psamd_linear_skinny");
    }
  }
  if constexpr (SWIGLU) {
    // A wide feed-forward (896 tiles of gate/up pairs at an intermediate size of 14,336) has
    // workgroups to spare at four pairs of tiles per wave, and the tokens are then read half as
    // often: 66 -> 56 us at 32 tokens, 78 -> 65 at 64. At 8,192 (512 tiles) it would leave half
    // the compute units idle, and two pairs stay the best.
    if (M > 8 && ceil_div(n_out, 16) >= 4 * 200) {
      const dim3 grid(static_cast<unsigned>(ceil_div(ceil_div(n_out, 16), 4)), 1u), block(64 * 8);
      skinny_mfma_kernel<MT, 4, 8, true, true, bf16_t, 1><<<grid, block, 0, s>>>(
          static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<bf16_t*>(out), M, n_out, K);
      return check_launch("psamd_linear_skinny");
    }
    if constexpr (MT == 1) {
      // 9 to 16 tokens: two pairs per wave where that leaves 200 workgroups (27.6 -> 23.3 us at
      // 16 tokens, intermediate size 8,192, K = 3,072).
      if (M > 8 && ceil_div(n_out, 16) >= 2 * 200) {
        const dim3 grid(static_cast<unsigned>(ceil_div(ceil_div(n_out, 16), 2)), 1u), block(64 * 8);
        skinny_mfma_kernel<1, 2, 8, true, true, bf16_t, 1><<<grid, block, 0, s>>>(
            static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<bf16_t*>(out), M, n_out, K);
        return check_launch("psamd_linear_skinny");
      }
    }
  }
  if constexpr (MT == 1) {
    // Workgroups that stay (stream_kernel) pay where each has two or more groups of tiles to go
    // through with the tokens it staged, us per product at 8 / 16 tokens:
    //  * products whose K is split over workgroups (o, down), 512 workgroups in all: down of the
    //    1B shape (2,048 x 8,192) 9.6 -> 9.0 / 12.1 -> 10.3, of the 3B shape 14.6 -> 11.9 /
    //    17.0 -> 13.9, of the 8B shape (4,096 x 14,336) 30.5 -> 24.5 / 36.4 -> 26.8; o of the 8B
    //    shape 9.5 -> 9.0 / 11.7 -> 10.1. With one group each (o of the smaller shapes) they lose.
    //  * gate/up with K from 4,096 on, 256 workgroups: 8B shape 54.8 -> 51.8 at 8 tokens; at
    //    K = 2,048 or 3,072 the workgroups that come and go are faster (17.7 vs 19.7).
    const int64_t groups = ceil_div(n_out, 16);
    if (M >= 4 && K % 32 == 0) {
      if constexpr (!SWIGLU) {
        const int wgs = ksplit > 1 ? 512 / ksplit : 0;
        if (wgs > 0 && groups >= 2 * wgs && stream_smem_bytes(1, 16, false, K, ksplit) <= 160 * 1024) {
          if (M <= 8) return launch_stream<1, 8, false>(s, plain_tokens(x), w, out, out_dtype, M, n_out, K, ksplit, wgs);
          return launch_stream<1, 16, false>(s, plain_tokens(x), w, out, out_dtype, M, n_out, K, ksplit, wgs);
        }
      } else {
        if (M <= 8 && ksplit == 1 && K >= 4096 && groups >= 768 && stream_smem_bytes(1, 8, true, K, 1) <= 160 * 1024)
          return launch_stream<1, 8, true>(s, plain_tokens(x), w, out, out_dtype, M, n_out, K, 1, 256);
      }
    }
  }
  constexpr int RT = skinny_rt(MT, SWIGLU), WV = SWIGLU ? 8 : skinny_wv(MT);
  // Enough row groups to fill the chip with one wave each: no need to split K inside a workgroup.
  if (ceil_div(ceil_div(n_out, 16), RT) >= 2048)
    return launch_skinny2<MT, RT, WV, SWIGLU, false>(s, x, w, out, out_dtype, M, n_out, K, ksplit);
  return launch_skinny2<MT, RT, WV, SWIGLU, true>(s, x, w, out, out_dtype, M, n_out, K, ksplit);
}

template <int MT>
static int launch_skinny(hipStream_t s, const void* x, const void* w, void* out, int out_dtype, int M, int n_out,
                         int K, int epilogue, int ksplit) {
  if (epilogue == 1) return launch_skinny1<MT, true>(s, x, w, out, out_dtype, M, n_out, K, ksplit);
  return launch_skinny1<MT, false>(s, x, w, out, out_dtype, M, n_out, K, ksplit);
}

// The q/k/v projection of a small step fused with what follows it: rotary encoding of q and
// k, and the write of k and v into their cache pages. Same streaming scheme as skinny_mfma
// (one workgroup = 16 rows of w over all of K, 4 waves taking k-steps in turn), but the 16
// rows are chosen so that a rotation pair lies in one tile: 8 columns of a head's first half
// and their 8 partners in the second half. After the product, lane groups 0-1 hold
// first-half elements and groups 2-3 their partners, one shuffle apart.
// qkv_out[m] receives the rotated q and k and v (the layout the attention kernels read q
// from); k and v also go to page slot write_slot[m] when a cache is given.
// RT such tiles per workgroup and WV waves, as in skinny_mfma_kernel.
// ROWS > 0 (MT == 1, K a multiple of 32): the tokens are ROWS rows of the float32 residual stream,
// normalized and staged in LDS once per workgroup as in stream_kernel; the matrix instructions
// then read them from there.
template <int MT, int RT, int WV, int ROWS = 0>
__global__ __launch_bounds__(64 * WV) void qkv_rope_append_kernel(
    Tokens tk, const bf16_t* __restrict__ w, bf16_t* __restrict__ qkv_out, int M, int K, int hq,
    int hkv, int d, const int32_t* __restrict__ positions, const float2* __restrict__ table,
    bf16_t* __restrict__ kv, const int32_t* __restrict__ write_slot) {
  constexpr bool NORMED = ROWS > 0;
  static_assert(!NORMED || MT == 1, "staged tokens: one tile of up to 16");
  __shared__ f32x4 red[WV][MT][64];
  extern __shared__ __align__(16) unsigned char qkv_smem[];     // NORMED: xs[ROWS][K + 8] bfloat16, ss[ROWS][WV]
  const bf16_t* x = tk.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int half = d >> 1;
  const int tiles_per_head = d >> 4;
  const int n_tiles = (hq + 2 * hkv) * tiles_per_head;
  const bf16_t* wrow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int t = min(static_cast<int>(blockIdx.x) * RT + rt, n_tiles - 1);
    const int head = t / tiles_per_head;
    const int p = (t - head * tiles_per_head) << 3;                 // first of 8 pair indices
    const int row = head * d + (r < 8 ? p + r : half + p + r - 8);
    wrow[rt] = w + static_cast<int64_t>(row) * K + 8 * g;
  }
  const bf16_t* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) xrow[mt] = x + static_cast<int64_t>(min(mt * 16 + r, M - 1)) * K + 8 * g;
  f32x4 acc[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[rt][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  // What the finishing waves (wave < MT: one 16-token tile each) need from memory after the
  // product is asked for now, so that it arrives behind the weights instead of after them: the
  // token's position, its rotation (a second, dependent trip) and its cache slot.
  float2 cs_early[RT][4];
  int slot_early = 0;
  if (wave < MT) {
    const int mc = min(wave * 16 + r, M - 1);
    const int pos = positions[mc];
    if (kv != nullptr) slot_early = write_slot[mc];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int t = min(static_cast<int>(blockIdx.x) * RT + rt, n_tiles - 1);
      const int head = t / tiles_per_head;
      const int p = (t - head * tiles_per_head) << 3;
      const bool rotate = table != nullptr && head < hq + hkv;
#pragma unroll
      for (int v = 0; v < 4; ++v)
        cs_early[rt][v] = rotate ? table[static_cast<int64_t>(pos) * half + p + 4 * (g & 1) + v] : float2{1.f, 0.f};
    }
  }
  const int s_full = K >> 5;
  constexpr int U = MT == 1 ? 8 : (MT * RT <= 2 ? 4 : 2);   // steps whose loads are in flight together
  const int XS = K + 8;
  bf16_t* xs = reinterpret_cast<bf16_t*>(qkv_smem);
  float* ss = reinterpret_cast<float*>(qkv_smem + static_cast<size_t>(NORMED ? ROWS : 0) * XS * sizeof(bf16_t));   // [ROWS][WV]
  float row_scale = 1.f;
  bf16x8 pre[RT][U];
  if constexpr (NORMED) {
    // The rows of w for the first k-steps are asked for before the tokens are staged: both trips
    // to memory are then under way together (7.8 against 8.1 us at 8 tokens of the 1B shape).
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) pre[rt][u] = wave + WV * u < s_full ? load8(wrow[rt] + ((wave + WV * u) << 5)) : zero8();
    stage_normed<ROWS, WV>(tk, xs, XS, ss, M, K, wave, lane);
    __syncthreads();
    row_scale = stage_scale<WV>(tk, ss, r % ROWS, M, K);
  }
  const bf16_t* xl = xs + (NORMED ? (r % ROWS) * XS + 8 * g : 0);
  for (int base = wave; base < s_full; base += WV * U) {
    bf16x8 a[RT][U], b[MT][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = base + WV * u;
      if (NORMED && base == wave) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) a[rt][u] = pre[rt][u];
      } else if (s < s_full) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) a[rt][u] = load8(wrow[rt] + (s << 5));
        if constexpr (!NORMED) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) b[mt][u] = load8(xrow[mt] + (s << 5));
        }
      } else {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) a[rt][u] = zero8();
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) b[mt][u] = zero8();
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if constexpr (NORMED) b[0][u] = *reinterpret_cast<const bf16x8*>(xl + (min(base + WV * u, s_full - 1) << 5));
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rt][u], b[mt][u], acc[rt][mt], 0, 0, 0);
    }
  }
  if (!NORMED && (K & 31) != 0 && (s_full % WV) == wave) {
    const int k = s_full << 5;
    const bool in = k + 8 * g < K;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const bf16x8 a = in ? load8(wrow[rt] + k) : zero8();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const bf16x8 b = in ? load8(xrow[mt] + k) : zero8();
        acc[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[rt][mt], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    if (rt > 0) __syncthreads();
#pragma unroll
    for (int i = 0; i < MT; ++i) red[wave][i][lane] = acc[rt][i];
    __syncthreads();
    const int t = static_cast<int>(blockIdx.x) * RT + rt;
    if (wave >= MT || t >= n_tiles) continue;
    const int head = t / tiles_per_head;
    const int p = (t - head * tiles_per_head) << 3;
    const int mt = wave;
    f32x4 own = red[0][mt][lane];
#pragma unroll
    for (int w2 = 1; w2 < WV; ++w2) own += red[w2][mt][lane];
    if (NORMED) own *= row_scale;
    const int m = mt * 16 + r;
    const int mc = min(m, M - 1);
    const bool second = g >= 2;
    f32x4 res;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const float other = __shfl_xor(own[v], 32, kWave);              // the pair's other half
      const float2 cs = cs_early[rt][v];                              // (1, 0) where nothing rotates
      res[v] = second ? own[v] * cs.x + other * cs.y : own[v] * cs.x - other * cs.y;
    }
    if (m >= M) continue;
    const int e0 = (second ? half : 0) + p + 4 * (g & 1);              // element of the head, 4 consecutive
    ushort4 pk;
    pk.x = float_to_bf16(res[0]);
    pk.y = float_to_bf16(res[1]);
    pk.z = float_to_bf16(res[2]);
    pk.w = float_to_bf16(res[3]);
    *reinterpret_cast<ushort4*>(qkv_out + static_cast<int64_t>(m) * ((hq + 2 * hkv) * d) + head * d + e0) = pk;
    if (kv == nullptr || head < hq) continue;
    const int slot = slot_early;
    const int64_t page_elems = 2LL * hkv * kPage * d;
    bf16_t* page = kv + static_cast<int64_t>(slot / kPage) * page_elems;
    const int off = slot % kPage;
    if (head < hq + hkv) {                                             // key row [16][D]
      *reinterpret_cast<ushort4*>(page + (static_cast<int64_t>(head - hq) * kPage + off) * d + e0) = pk;
    } else {                                                           // value, transposed [D][16]
      bf16_t* vp = page + static_cast<int64_t>(hkv) * kPage * d + (static_cast<int64_t>(head - hq - hkv) * d + e0) * kPage + off;
      vp[0] = pk.x;
      vp[kPage] = pk.y;
      vp[2 * kPage] = pk.z;
      vp[3 * kPage] = pk.w;
    }
  }
}

// One tile per workgroup keeps the most workgroups, and K cannot be split over workgroups
// here (the rotation needs whole sums); two tiles halve the traffic for the tokens, which pays
// from 9 tokens on where 320 tiles or more leave every compute unit a workgroup (at 384 tiles
// and K = 4,096: 28 -> 22 us at 32 tokens, 45 -> 31 at 64; at 192 tiles one tile stays the
// best). Eight waves per workgroup beat four at every size tried.
template <int MT>
static void launch_qkv(hipStream_t s, const bf16_t* x, const bf16_t* w, bf16_t* out, int M, int K, int hq, int hkv, int d,
                       const int32_t* positions, const float2* table, bf16_t* kv, const int32_t* write_slot) {
  const int n_tiles = (hq + 2 * hkv) * (d / 16);
  const Tokens tk = plain_tokens(x);
  if (M > 8 && n_tiles >= 320) {
    qkv_rope_append_kernel<MT, 2, 8><<<dim3(static_cast<unsigned>(ceil_div(n_tiles, 2))), dim3(512), 0, s>>>(
        tk, w, out, M, K, hq, hkv, d, positions, table, kv, write_slot);
  } else {
    qkv_rope_append_kernel<MT, 1, 8><<<dim3(static_cast<unsigned>(n_tiles)), dim3(512), 0, s>>>(
        tk, w, out, M, K, hq, hkv, d, positions, table, kv, write_slot);
  }
}

// LDS the staged form needs beside the kernel's static array.
static size_t qkv_staged_smem(int rows, int K) { return static_cast<size_t>(rows) * (K + 8) * sizeof(bf16_t) + sizeof(float) * rows * 8; }

// Up to 16 tokens read from the residual stream and normalized in the kernel (K a multiple of 32).
template <int RT, int ROWS>
static int launch_qkv_normed(hipStream_t s, const Tokens& tk, const bf16_t* w, bf16_t* out, int M, int K, int hq, int hkv, int d,
                             const int32_t* positions, const float2* table, bf16_t* kv, const int32_t* write_slot) {
  const int n_tiles = (hq + 2 * hkv) * (d / 16);
  const size_t smem = qkv_staged_smem(ROWS, K);
  auto kernel = qkv_rope_append_kernel<1, RT, 8, ROWS>;
  if (smem + sizeof(f32x4) * 8 * 64 > 64 * 1024 &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                          static_cast<int>(smem)) != hipSuccess)
    return fail("psamd_qkv_rope_append_normed: " + std::to_string(smem) + " bytes of LDS were refused");
  kernel<<<dim3(static_cast<unsigned>(ceil_div(n_tiles, RT))), dim3(512), smem, s>>>(tk, w, out, M, K, hq, hkv, d, positions,
                                                                                   table, kv, write_slot);
  return check_launch("psamd_qkv_rope_append_normed");
}

// Whether the kernels that normalize their tokens themselves take a step of M tokens of width K:
// up to 16 tokens, whole 32-wide k-steps, and the staged tokens fit in LDS beside the partial sums.
static bool normed_ok(int M, int K) {
  return M >= 1 && M <= 16 && K >= 32 && K % 32 == 0 && stream_smem_bytes(1, M <= 8 ? 8 : 16, true, K, 1) <= 160 * 1024;
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
  if (x_dtype == kF32 && w_dtype == kF32 && out_dtype == kF32) {
    const bool aligned = (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) % 16 == 0;
    if (M <= 16 && K % 4 == 0 && aligned) return launch_rows_f32(s, x, w, out, static_cast<int>(M), N, K);
    return launch_tiled<float, float, float>(s, x, w, out, M, N, K);
  }
  if (x_dtype == kBF16 && w_dtype == kBF16 && out_dtype == kBF16) return launch_tiled<bf16_t, bf16_t, bf16_t>(s, x, w, out, M, N, K);
  if (x_dtype == kBF16 && w_dtype == kBF16 && out_dtype == kF32) return launch_tiled<bf16_t, bf16_t, float>(s, x, w, out, M, N, K);
  return fail("psamd_linear: supported types are (f32,f32)->f32, (bf16,bf16)->bf16 and (bf16,bf16)->f32");
}

// The K-split that fills the chip for a linear product of M <= 64 tokens whose float32 partial
// sums a consumer adds up: as many workgroups as there are compute units to spare.
int psamd_linear_skinny_ksplit(int M, int n_out, int K) {
  if (M < 1 || M > 64 || n_out < 1 || K < 1) return 1;
  const int mt = static_cast<int>(ceil_div(M, 16));
  const int64_t groups = ceil_div(ceil_div(n_out, 16), skinny_rt(mt, false));
  const int64_t steps = ceil_div(K, 32);
  // Up to 32 tokens a wave keeps at least two k-steps; above, one is enough (measured).
  // Workgroups of 4 waves: two per compute unit; of 8 waves: one (4,096 x 4,096 at 64 tokens:
  // 16.2 us with 8 slices, 14.3 with 4).
  if (mt == 1) {
    // Up to 16 tokens: as many slices as give a wave about eight k-steps, all of which it has
    // in flight at once, whatever the number of workgroups up to 2,048 (measured at 1 and 8
    // tokens: 2,048 x 8,192 10.0 -> 8.6 us with 8 slices instead of 4, 3,072 x 8,192 15.3 -> 12.0,
    // 4,096 x 14,336 27.9 -> 24 us; 2,048 x 2,048 4.0 -> 3.8 us with 2 instead of 4).
    const int64_t per_slice = 8 * skinny_wv(mt);
    const int64_t split = std::min<int64_t>({8, std::max<int64_t>(2048 / std::max<int64_t>(groups, 1), 1), (steps + per_slice / 2) / per_slice});
    return static_cast<int>(std::max<int64_t>(split, 1));
  }
  const int64_t wanted = skinny_wv(mt) == 8 ? 256 : 512;
  const int64_t split = std::min<int64_t>({8, wanted / std::max<int64_t>(groups, 1), steps / ((mt <= 2 ? 2 : 1) * skinny_wv(mt))});
  return static_cast<int>(std::max<int64_t>(split, 1));
}

// out[ksplit][M, n_out]; epilogue 0: n_out = rows of w; epilogue 1 (SwiGLU): w has 2 * n_out rows.
// ksplit > 1 splits K over workgroups: out then holds ksplit float32 partial sums to be added.
int psamd_linear_skinny(void* stream, const void* x, const void* w, void* out, int out_dtype, int M, int n_out, int K,
                        int epilogue, int ksplit) {
  PSAMD_REQUIRE(M >= 1 && M <= 64, "M must be in [1, 64]");
  PSAMD_REQUIRE(n_out > 0 && K > 0 && K % 8 == 0, "K must be a positive multiple of 8");
  PSAMD_REQUIRE(epilogue == 0 || epilogue == 1, "unknown epilogue");
  PSAMD_REQUIRE(out_dtype == kBF16 || out_dtype == kF32, "output must be bfloat16 or float32");
  PSAMD_REQUIRE(epilogue == 0 || out_dtype == kBF16, "the SwiGLU epilogue writes bfloat16");
  PSAMD_REQUIRE(ksplit >= 1 && ksplit <= 64, "ksplit must be in [1, 64]");
  PSAMD_REQUIRE(ksplit == 1 || (epilogue == 0 && out_dtype == kF32), "partial sums are float32 and linear");
  PSAMD_REQUIRE(ceil_div(n_out, 16) <= 2147483647LL, "too many columns");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int mt = static_cast<int>(ceil_div(M, 16));
  switch (mt) {
    case 1: return launch_skinny<1>(s, x, w, out, out_dtype, M, n_out, K, epilogue, ksplit);
    case 2: return launch_skinny<2>(s, x, w, out, out_dtype, M, n_out, K, epilogue, ksplit);
    case 3: return launch_skinny<3>(s, x, w, out, out_dtype, M, n_out, K, epilogue, ksplit);
    default: return launch_skinny<4>(s, x, w, out, out_dtype, M, n_out, K, epilogue, ksplit);
  }
}


// qkv_out[M, (hq + 2 hkv) * d] = x[M, K] * w^T with q and k rotated by table[positions[m]] (NULL: no rotation);
// k and v are also written to page slot write_slot[m] of kv (NULL: no cache write).
int psamd_qkv_rope_append(void* stream, const void* x, const void* w, void* qkv_out, int M, int K, int hq, int hkv,
                          int head_dim, const int32_t* positions, const float* table, void* kv,
                          const int32_t* write_slot) {
  PSAMD_REQUIRE(M >= 1 && M <= 64, "M must be in [1, 64]");
  PSAMD_REQUIRE(K > 0 && K % 8 == 0, "K must be a positive multiple of 8");
  PSAMD_REQUIRE(hq > 0 && hkv > 0 && head_dim >= 16 && head_dim % 16 == 0, "head_dim must be a multiple of 16");
  PSAMD_REQUIRE(positions != nullptr, "positions are needed");
  PSAMD_REQUIRE(kv == nullptr || write_slot != nullptr, "a cache needs write slots");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bf16_t* xp = static_cast<const bf16_t*>(x);
  const bf16_t* wp = static_cast<const bf16_t*>(w);
  bf16_t* op = static_cast<bf16_t*>(qkv_out);
  const float2* tab = reinterpret_cast<const float2*>(table);
  bf16_t* kvp = static_cast<bf16_t*>(kv);
  switch (static_cast<int>(ceil_div(M, 16))) {
    case 1: launch_qkv<1>(s, xp, wp, op, M, K, hq, hkv, head_dim, positions, tab, kvp, write_slot); break;
    case 2: launch_qkv<2>(s, xp, wp, op, M, K, hq, hkv, head_dim, positions, tab, kvp, write_slot); break;
    case 3: launch_qkv<3>(s, xp, wp, op, M, K, hq, hkv, head_dim, positions, tab, kvp, write_slot); break;
    default: launch_qkv<4>(s, xp, wp, op, M, K, hq, hkv, head_dim, positions, tab, kvp, write_slot); break;
  }
  return check_launch("psamd_qkv_rope_append");
}

// 1 if psamd_linear_normed and psamd_qkv_rope_append_normed take M tokens of width K.
int psamd_normed_supports(int M, int K) { return normed_ok(M, K) ? 1 : 0; }

// out[M, n_out] (float32, the residual stream) += x[M, K] * w[n_out, K]^T for M <= 16: K is split
// over as many workgroups as fill the chip, and every slice adds its partial sums with float
// atomics that return nothing. The order of the additions is not fixed: results differ in the
// last bit from run to run.
int psamd_linear_skinny_add(void* stream, const void* x, const void* w, float* out, int M, int n_out, int K) {
  PSAMD_REQUIRE(M >= 1 && M <= 16, "M must be in [1, 16]");
  PSAMD_REQUIRE(n_out > 0 && K > 0 && K % 8 == 0, "K must be a positive multiple of 8");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int ksplit = psamd_linear_skinny_ksplit(M, n_out, K);
  const int64_t groups = ceil_div(n_out, 16);
  const int wgs = ksplit > 1 ? 512 / ksplit : 0;
  if (M >= 4 && K % 32 == 0 && wgs > 0 && groups >= 2 * wgs && stream_smem_bytes(1, 16, false, K, ksplit) <= 160 * 1024) {
    if (M <= 8) return launch_stream<1, 8, false, false, true>(s, plain_tokens(x), w, out, kF32, M, n_out, K, ksplit, wgs);
    return launch_stream<1, 16, false, false, true>(s, plain_tokens(x), w, out, kF32, M, n_out, K, ksplit, wgs);
  }
  const dim3 grid(static_cast<unsigned>(groups), static_cast<unsigned>(ksplit)), block(64 * 4);
  skinny_mfma_kernel<1, 1, 4, false, true, float, 8, true><<<grid, block, 0, s>>>(
      static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), out, M, n_out, K);
  return check_launch("psamd_linear_skinny_add");
}

// out[M, n_out] = norm(resid[rows[m]]) * w^T for M <= 16 tokens, where norm is the RMS norm with
// weight norm_w [K] (bfloat16 or float32) and eps, computed inside the kernel from the float32
// residual rows (rows == NULL: row m). epilogue 0: out bfloat16 or float32; epilogue 1 (SwiGLU):
// w = [gate; up] with n_out rows each, out = silu(gate) * up in bfloat16.
int psamd_linear_normed(void* stream, const float* resid, const int32_t* rows, const void* norm_w, int norm_w_dtype,
                        float eps, const void* w, void* out, int out_dtype, int M, int n_out, int K, int epilogue) {
  PSAMD_REQUIRE(normed_ok(M, K), "M must be in [1, 16] and K a multiple of 32 that fits in LDS");
  PSAMD_REQUIRE(n_out > 0 && (epilogue == 0 || epilogue == 1), "bad sizes");
  PSAMD_REQUIRE(out_dtype == kBF16 || out_dtype == kF32, "output must be bfloat16 or float32");
  PSAMD_REQUIRE(epilogue == 0 || out_dtype == kBF16, "the SwiGLU epilogue writes bfloat16");
  PSAMD_REQUIRE(norm_w_dtype == kBF16 || norm_w_dtype == kF32, "the norm's weight is bfloat16 or float32");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Tokens tk{nullptr, resid, norm_w, rows, eps, norm_w_dtype == kBF16 ? 1 : 0};
  const int64_t groups = ceil_div(n_out, 16);
  const bool eight = M <= 8;
  if (epilogue == 1) {
    // One pair of gate/up tiles per group; as many workgroups as give each one or two groups.
    // 512 pairs of tiles (an intermediate size of 8,192) and up to 8 tokens: a workgroup per pair
    // (17.9 us at 8 tokens against 19.0 with two pairs each); more tokens (the staged rows then
    // leave a compute unit room for one workgroup) or more pairs: 256 workgroups that stay for two
    // or more (16 tokens: 25.4 -> 21.1 us; 896 pairs at K = 4,096, 8 tokens: 56.4 -> 53.0).
    const int wgs = (eight && groups < 768) ? 512 : 256;
    if (eight) return launch_stream<1, 8, true, true>(s, tk, w, out, out_dtype, M, n_out, K, 1, wgs);
    return launch_stream<1, 16, true, true>(s, tk, w, out, out_dtype, M, n_out, K, 1, wgs);
  }
  // Two row tiles per group while the staged tokens are small (two workgroups per compute unit).
  const bool small = static_cast<int64_t>(eight ? 8 : 16) * K <= 8 * 2048 && groups >= 2048;
  if (eight) {
    if (small) return launch_stream<2, 8, false, true>(s, tk, w, out, out_dtype, M, n_out, K, 1, 512);
    return launch_stream<1, 8, false, true>(s, tk, w, out, out_dtype, M, n_out, K, 1, 1024);
  }
  if (small) return launch_stream<2, 16, false, true>(s, tk, w, out, out_dtype, M, n_out, K, 1, 512);
  return launch_stream<1, 16, false, true>(s, tk, w, out, out_dtype, M, n_out, K, 1, 1024);
}

// psamd_qkv_rope_append with the tokens read from the float32 residual stream and normalized in
// the kernel (RMS norm with weight norm_w and eps), for M <= 16.
int psamd_qkv_rope_append_normed(void* stream, const float* resid, const void* norm_w, int norm_w_dtype, float eps,
                                 const void* w, void* qkv_out, int M, int K, int hq, int hkv, int head_dim,
                                 const int32_t* positions, const float* table, void* kv, const int32_t* write_slot) {
  PSAMD_REQUIRE(normed_ok(M, K), "M must be in [1, 16] and K a multiple of 32 that fits in LDS");
  PSAMD_REQUIRE(hq > 0 && hkv > 0 && head_dim >= 16 && head_dim % 16 == 0, "head_dim must be a multiple of 16");
  PSAMD_REQUIRE(positions != nullptr, "positions are needed");
  PSAMD_REQUIRE(kv == nullptr || write_slot != nullptr, "a cache needs write slots");
  PSAMD_REQUIRE(norm_w_dtype == kBF16 || norm_w_dtype == kF32, "the norm's weight is bfloat16 or float32");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Tokens tk{nullptr, resid, norm_w, nullptr, eps, norm_w_dtype == kBF16 ? 1 : 0};
  const bf16_t* wp = static_cast<const bf16_t*>(w);
  bf16_t* op = static_cast<bf16_t*>(qkv_out);
  const float2* tab = reinterpret_cast<const float2*>(table);
  bf16_t* kvp = static_cast<bf16_t*>(kv);
  const int n_tiles = (hq + 2 * hkv) * (head_dim / 16);
  if (M <= 8) return launch_qkv_normed<1, 8>(s, tk, wp, op, M, K, hq, hkv, head_dim, positions, tab, kvp, write_slot);
  if (n_tiles >= 320) return launch_qkv_normed<2, 16>(s, tk, wp, op, M, K, hq, hkv, head_dim, positions, tab, kvp, write_slot);
  return launch_qkv_normed<1, 16>(s, tk, wp, op, M, K, hq, hkv, head_dim, positions, tab, kvp, write_slot);
}

}  // extern "C"
