// Memory-bound kernels around the matrix products: token gather, fused residual-add +
// RMSNorm, SwiGLU, and rotary encoding fused with the write of keys and values into their
// cache pages. Each is templated on the activation type (bfloat16 or float); statistics,
// rotation and the residual sum are always float.

#include <algorithm>

#include "api.h"
#include "common.h"

namespace psamd {

static thread_local std::string g_error;
void set_error(const std::string& msg) { g_error = msg; }

// ------------------------------------------------------------------ embed

template <typename W>
__global__ void embed_kernel(const int32_t* __restrict__ ids, const W* __restrict__ table,
                             float* __restrict__ out, int hidden, int vocab) {
  const int64_t t = blockIdx.x;
  // Ids are checked on the host, except those a previous step sampled and left on the device:
  // an id outside the table reads its nearest row instead of memory that is not the table's.
  const int id = min(max(ids[t], 0), vocab - 1);
  const W* row = table + static_cast<int64_t>(id) * hidden;
  float* o = out + t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = to_float<W>(row[i]);
}

// ------------------------------------------------------------------ add + rmsnorm

// One block per output row. x = residual + sum of the delta slices; out = weight * x *
// rsqrt(mean(x^2) + eps), everything in float. `delta` is either [rows, hidden] in the
// activation type or n_partials float slices [n_partials][rows, hidden] (partial sums of a
// K-split product). Without `rows` the block handles row blockIdx.x and stores x back as the
// new residual; with `rows` it handles residual row rows[blockIdx.x] and leaves it as it is.
// Rows up to kCache * kThreads wide stay in registers between the two passes, and all loads
// of a pass are independent of each other (clamped addresses, no branches around them), so
// they are in flight together: with one row per block the kernel is pure latency.
template <typename A, typename DT, int kThreads, int kCache>
__global__ __launch_bounds__(kThreads) void add_rmsnorm_kernel(
    float* __restrict__ residual, const DT* __restrict__ delta, int n_partials, int64_t partial_stride,
    const int32_t* __restrict__ rows, const void* __restrict__ weight, int weight_dtype, float eps,
    A* __restrict__ out, int hidden) {
  __shared__ float scratch[kThreads / kWave];
  const int64_t src = rows != nullptr ? rows[blockIdx.x] : blockIdx.x;
  float* r = residual + src * hidden;
  const DT* d0 = delta != nullptr ? delta + src * hidden : nullptr;
  A* o = out + static_cast<int64_t>(blockIdx.x) * hidden;
  const bool store = rows == nullptr && delta != nullptr;
  const int np = delta != nullptr ? n_partials : 0;

  if (hidden <= kCache * kThreads) {
    float v[kCache], wv[kCache];
    int idx[kCache];
#pragma unroll
    for (int j = 0; j < kCache; ++j) {
      idx[j] = min(static_cast<int>(threadIdx.x) + j * kThreads, hidden - 1);
      v[j] = r[idx[j]];
      wv[j] = load_as_float(weight, weight_dtype, idx[j]);
    }
    for (int p = 0; p < np; ++p) {
      const DT* dp = d0 + p * partial_stride;
      float t[kCache];
#pragma unroll
      for (int j = 0; j < kCache; ++j) t[j] = to_float<DT>(dp[idx[j]]);
#pragma unroll
      for (int j = 0; j < kCache; ++j) v[j] += t[j];
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kCache; ++j) {
      const bool in = static_cast<int>(threadIdx.x) + j * kThreads < hidden;
      ss += in ? v[j] * v[j] : 0.f;
    }
    ss = block_sum(ss, scratch, kThreads / kWave);
    const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
#pragma unroll
    for (int j = 0; j < kCache; ++j) {
      if (static_cast<int>(threadIdx.x) + j * kThreads < hidden) {
        if (store) r[idx[j]] = v[j];
        o[idx[j]] = from_float<A>(wv[j] * (v[j] * inv));
      }
    }
    return;
  }

  auto value = [&](int i) {
    float x = r[i];
    for (int p = 0; p < np; ++p) x += to_float<DT>(d0[p * partial_stride + i]);
    return x;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += kThreads) {
    const float x = value(i);
    if (store) r[i] = x;
    ss += x * x;
  }
  ss = block_sum(ss, scratch, kThreads / kWave);
  const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
  for (int i = threadIdx.x; i < hidden; i += kThreads) {
    const float x = store ? r[i] : value(i);
    o[i] = from_float<A>(load_as_float(weight, weight_dtype, i) * (x * inv));
  }
}

// The same operation for bfloat16 activations and rows that are a multiple of 8 wide: every
// thread owns runs of 8 consecutive elements, moved as 16- and 32-byte accesses. kIter runs
// per thread stay in registers (hidden <= 8 * kThreads * kIter).
template <typename DT, int kThreads, int kIter>
__global__ __launch_bounds__(kThreads) void add_rmsnorm_vec8_kernel(
    float* __restrict__ residual, const DT* __restrict__ delta, int n_partials, int64_t partial_stride,
    const int32_t* __restrict__ rows, const void* __restrict__ weight, int weight_dtype, float eps,
    bf16_t* __restrict__ out, int hidden) {
  __shared__ float scratch[kThreads / kWave];
  const int64_t src = rows != nullptr ? rows[blockIdx.x] : blockIdx.x;
  float* r = residual + src * hidden;
  const DT* d0 = delta != nullptr ? delta + src * hidden : nullptr;
  bf16_t* o = out + static_cast<int64_t>(blockIdx.x) * hidden;
  const bool store = rows == nullptr && delta != nullptr;
  const int np = delta != nullptr ? n_partials : 0;
  const int chunks = hidden >> 3;

  float v[kIter][8];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < kIter; ++j) {
    const int cidx = threadIdx.x + j * kThreads;
    const int e = min(cidx, chunks - 1) << 3;
    const float4 a = *reinterpret_cast<const float4*>(r + e);
    const float4 b = *reinterpret_cast<const float4*>(r + e + 4);
    v[j][0] = a.x; v[j][1] = a.y; v[j][2] = a.z; v[j][3] = a.w;
    v[j][4] = b.x; v[j][5] = b.y; v[j][6] = b.z; v[j][7] = b.w;
    for (int p = 0; p < np; ++p) {
      const DT* dp = d0 + p * partial_stride + e;
      if (sizeof(DT) == 2) {
        const uint4 q = *reinterpret_cast<const uint4*>(dp);
        const uint32_t w4[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[j][2 * i] += __uint_as_float(w4[i] << 16);
          v[j][2 * i + 1] += __uint_as_float(w4[i] & 0xffff0000u);
        }
      } else {
        // Up to eight slices are asked for together (one trip to memory, not one per slice) and
        // added in ascending order; slots past the last slice repeat it and are not added.
        float4 x0[8], x1[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const DT* du = d0 + min(p + u, np - 1) * partial_stride + e;
          x0[u] = *reinterpret_cast<const float4*>(du);
          x1[u] = *reinterpret_cast<const float4*>(du + 4);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (p + u < np) {
            v[j][0] += x0[u].x; v[j][1] += x0[u].y; v[j][2] += x0[u].z; v[j][3] += x0[u].w;
            v[j][4] += x1[u].x; v[j][5] += x1[u].y; v[j][6] += x1[u].z; v[j][7] += x1[u].w;
          }
        }
        p += 7;
      }
    }
    if (cidx < chunks) {
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += v[j][i] * v[j][i];
    }
  }
  ss = block_sum(ss, scratch, kThreads / kWave);
  const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
#pragma unroll
  for (int j = 0; j < kIter; ++j) {
    const int cidx = threadIdx.x + j * kThreads;
    if (cidx >= chunks) continue;
    const int e = cidx << 3;
    if (store) {
      *reinterpret_cast<float4*>(r + e) = make_float4(v[j][0], v[j][1], v[j][2], v[j][3]);
      *reinterpret_cast<float4*>(r + e + 4) = make_float4(v[j][4], v[j][5], v[j][6], v[j][7]);
    }
    float w[8];
    if (weight_dtype == kBF16) {
      const uint4 q = *reinterpret_cast<const uint4*>(static_cast<const bf16_t*>(weight) + e);
      const uint32_t w4[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        w[2 * i] = __uint_as_float(w4[i] << 16);
        w[2 * i + 1] = __uint_as_float(w4[i] & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) w[i] = static_cast<const float*>(weight)[e + i];
    }
    uint32_t pk[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pk[i] = static_cast<uint32_t>(float_to_bf16(w[2 * i] * (v[j][2 * i] * inv))) |
              (static_cast<uint32_t>(float_to_bf16(w[2 * i + 1] * (v[j][2 * i + 1] * inv))) << 16);
    }
    *reinterpret_cast<uint4*>(o + e) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
  }
}

// ------------------------------------------------------------------ swiglu

template <typename A>
__global__ void swiglu_kernel(const A* __restrict__ gate_up, A* __restrict__ out, int64_t tokens, int inter) {
  const int64_t n = tokens * inter;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t t = i / inter, c = i - t * inter;
    const float g = to_float<A>(gate_up[t * 2 * inter + c]);
    const float u = to_float<A>(gate_up[t * 2 * inter + inter + c]);
    out[i] = from_float<A>(g / (1.f + __expf(-g)) * u);
  }
}

// bfloat16, intermediate size a multiple of 8: 16-byte accesses, 8 elements per thread.
__global__ void swiglu_vec8_kernel(const bf16_t* __restrict__ gate_up, bf16_t* __restrict__ out, int64_t tokens,
                                   int inter) {
  const int chunks = inter >> 3;
  const int64_t n = tokens * chunks;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t t = i / chunks;
    const int e = static_cast<int>(i - t * chunks) << 3;
    const uint4 g = *reinterpret_cast<const uint4*>(gate_up + t * 2 * inter + e);
    const uint4 u = *reinterpret_cast<const uint4*>(gate_up + t * 2 * inter + inter + e);
    const uint32_t g4[4] = {g.x, g.y, g.z, g.w}, u4[4] = {u.x, u.y, u.z, u.w};
    uint32_t pk[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float g0 = __uint_as_float(g4[k] << 16), g1 = __uint_as_float(g4[k] & 0xffff0000u);
      const float u0 = __uint_as_float(u4[k] << 16), u1 = __uint_as_float(u4[k] & 0xffff0000u);
      pk[k] = static_cast<uint32_t>(float_to_bf16(g0 / (1.f + __expf(-g0)) * u0)) |
              (static_cast<uint32_t>(float_to_bf16(g1 / (1.f + __expf(-g1)) * u1)) << 16);
    }
    *reinterpret_cast<uint4*>(out + t * inter + e) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
  }
}

// ------------------------------------------------------------------ rope + kv append

// One block per token. q and k heads of the fused qkv row are rotated in place (pair
// (i, i + D/2), angle table [pos][i] = (cos, sin)); the rotated keys go to their page as
// [16, D] rows and the values to the page's second half transposed, [D, 16].
template <typename A>
__global__ void rope_kv_append_kernel(A* __restrict__ qkv, int hq, int hkv, int d,
                                      const int32_t* __restrict__ positions,
                                      const float2* __restrict__ table,
                                      A* __restrict__ kv, const int32_t* __restrict__ write_slot) {
  const int64_t t = blockIdx.x;
  const int half = d / 2;
  A* row = qkv + t * static_cast<int64_t>((hq + 2 * hkv) * d);
  const int pos = positions[t];
  int64_t page = 0;
  int off = 0;
  if (kv != nullptr) {
    const int slot = write_slot[t];
    page = slot / kPage;
    off = slot % kPage;
  }
  const int64_t page_elems = 2LL * hkv * kPage * d;
  A* kpage = kv != nullptr ? kv + page * page_elems : nullptr;
  A* vpage = kv != nullptr ? kpage + static_cast<int64_t>(hkv) * kPage * d : nullptr;

  const int n_rot = (hq + hkv) * half;
  for (int idx = threadIdx.x; idx < n_rot; idx += blockDim.x) {
    const int h = idx / half, i = idx - h * half;
    A* x = row + h * d;
    float a = to_float<A>(x[i]), b = to_float<A>(x[i + half]);
    if (table != nullptr) {
      const float2 cs = table[static_cast<int64_t>(pos) * half + i];
      const float ra = a * cs.x - b * cs.y;
      const float rb = b * cs.x + a * cs.y;
      a = ra;
      b = rb;
      x[i] = from_float<A>(a);
      x[i + half] = from_float<A>(b);
    }
    if (kpage != nullptr && h >= hq) {
      A* dst = kpage + (static_cast<int64_t>(h - hq) * kPage + off) * d;
      dst[i] = from_float<A>(a);
      dst[i + half] = from_float<A>(b);
    }
  }
  if (vpage != nullptr) {
    const A* v = row + (hq + hkv) * d;
    for (int idx = threadIdx.x; idx < hkv * d; idx += blockDim.x) {
      const int h = idx / d, c = idx - h * d;
      vpage[(static_cast<int64_t>(h) * d + c) * kPage + off] = v[idx];
    }
  }
}

// bfloat16 with a head size that is a multiple of 16: one block per 16 tokens of the step.
// q and k are rotated eight pairs per thread with 16-byte accesses. The values of the 16
// tokens pass through LDS so that lanes 0..15 write the same (head, dim) of 16 tokens: when
// the tokens follow each other in one page, as the tokens of a prompt do, that is one 32-byte
// run of the transposed page instead of 16 scattered 2-byte stores.
__global__ __launch_bounds__(256) void rope_kv_append_vec_kernel(bf16_t* __restrict__ qkv, int tokens, int hq, int hkv,
                                                                 int d, const int32_t* __restrict__ positions,
                                                                 const float2* __restrict__ table,
                                                                 bf16_t* __restrict__ kv,
                                                                 const int32_t* __restrict__ write_slot) {
  extern __shared__ __align__(16) bf16_t v_lds[];        // [16][hkv * d + 8]
  const int t0 = blockIdx.x * 16;
  const int nt = min(16, tokens - t0);
  const int half = d >> 1;
  const int width = (hq + 2 * hkv) * d;
  const int64_t page_elems = 2LL * hkv * kPage * d;
  const int chunks_per_head = half >> 3;                 // groups of 8 pairs
  const int chunks_per_token = (hq + hkv) * chunks_per_head;
  const int vw = hkv * d;
  const int c_lo = static_cast<int>(static_cast<int64_t>(vw >> 3) * blockIdx.y / gridDim.y);      // 8-element columns
  const int c_hi = static_cast<int>(static_cast<int64_t>(vw >> 3) * (blockIdx.y + 1) / gridDim.y);
  const int nc = c_hi - c_lo, vs = 8 * nc + 8;
  // The values are asked for first: they are on their way into LDS while q and k are rotated.
  for (int idx = threadIdx.x; kv != nullptr && idx < nt * nc; idx += blockDim.x) {
    const int j = idx / nc, c = idx - j * nc;
    *reinterpret_cast<uint4*>(v_lds + j * vs + 8 * c) =
        *reinterpret_cast<const uint4*>(qkv + static_cast<int64_t>(t0 + j) * width + (hq + hkv) * d + 8 * (c_lo + c));
  }
  // blockIdx.y takes its share of the rotation work and of the value columns.
  const int rot_total = nt * chunks_per_token;
  const int rot_lo = static_cast<int>(static_cast<int64_t>(rot_total) * blockIdx.y / gridDim.y);
  const int rot_hi = static_cast<int>(static_cast<int64_t>(rot_total) * (blockIdx.y + 1) / gridDim.y);
  for (int idx = rot_lo + threadIdx.x; idx < rot_hi; idx += blockDim.x) {
    const int j = idx / chunks_per_token, c = idx - j * chunks_per_token;
    const int h = c / chunks_per_head, i = (c - h * chunks_per_head) << 3;
    const int64_t t = t0 + j;
    bf16_t* x = qkv + t * width + h * d + i;
    uint4 lo = *reinterpret_cast<const uint4*>(x), hi = *reinterpret_cast<const uint4*>(x + half);
    if (table != nullptr) {
      const float2* cs = table + static_cast<int64_t>(positions[t]) * half + i;
      const uint32_t* lw = reinterpret_cast<const uint32_t*>(&lo);
      const uint32_t* hw = reinterpret_cast<const uint32_t*>(&hi);
      uint32_t lo_out[4], hi_out[4];
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float a0 = bf16_to_float(static_cast<bf16_t>(lw[w] & 0xffffu)), a1 = bf16_to_float(static_cast<bf16_t>(lw[w] >> 16));
        const float b0 = bf16_to_float(static_cast<bf16_t>(hw[w] & 0xffffu)), b1 = bf16_to_float(static_cast<bf16_t>(hw[w] >> 16));
        const float2 c0 = cs[2 * w], c1 = cs[2 * w + 1];
        lo_out[w] = static_cast<uint32_t>(float_to_bf16(a0 * c0.x - b0 * c0.y)) |
                    (static_cast<uint32_t>(float_to_bf16(a1 * c1.x - b1 * c1.y)) << 16);
        hi_out[w] = static_cast<uint32_t>(float_to_bf16(b0 * c0.x + a0 * c0.y)) |
                    (static_cast<uint32_t>(float_to_bf16(b1 * c1.x + a1 * c1.y)) << 16);
      }
      lo = make_uint4(lo_out[0], lo_out[1], lo_out[2], lo_out[3]);
      hi = make_uint4(hi_out[0], hi_out[1], hi_out[2], hi_out[3]);
      *reinterpret_cast<uint4*>(x) = lo;
      *reinterpret_cast<uint4*>(x + half) = hi;
    }
    if (kv != nullptr && h >= hq) {
      const int slot = write_slot[t];
      bf16_t* dst = kv + static_cast<int64_t>(slot / kPage) * page_elems +
                    (static_cast<int64_t>(h - hq) * kPage + slot % kPage) * d + i;
      *reinterpret_cast<uint4*>(dst) = lo;
      *reinterpret_cast<uint4*>(dst + half) = hi;
    }
  }
  if (kv == nullptr) return;
  __syncthreads();
  const int j = threadIdx.x & 15;
  if (j < nt) {
    const int slot = write_slot[t0 + j];
    bf16_t* vpage = kv + static_cast<int64_t>(slot / kPage) * page_elems + static_cast<int64_t>(hkv) * kPage * d + slot % kPage;
    for (int e = threadIdx.x >> 4; e < 8 * nc; e += blockDim.x >> 4)
      vpage[static_cast<int64_t>(8 * c_lo + e) * kPage] = v_lds[j * vs + e];
  }
}

}  // namespace psamd

using namespace psamd;

extern "C" {

const char* psamd_last_error(void) { return g_error.c_str(); }

int psamd_embed(void* stream, const int32_t* ids, const void* table, int table_dtype, float* out, int64_t tokens,
                int hidden, int vocab) {
  PSAMD_REQUIRE(tokens >= 0 && hidden > 0 && vocab > 0, "bad sizes");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (table_dtype == kBF16) {
    embed_kernel<bf16_t><<<dim3(tokens), dim3(256), 0, s>>>(ids, static_cast<const bf16_t*>(table), out, hidden, vocab);
  } else if (table_dtype == kF32) {
    embed_kernel<float><<<dim3(tokens), dim3(256), 0, s>>>(ids, static_cast<const float*>(table), out, hidden, vocab);
  } else {
    return fail("psamd_embed: table dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_embed");
}

int psamd_add_rmsnorm(void* stream, float* residual, const void* delta, int delta_dtype, int n_partials,
                      int64_t partial_stride, const int32_t* rows, const void* weight, int weight_dtype, float eps,
                      void* out, int act_dtype, int64_t out_rows, int hidden) {
  PSAMD_REQUIRE(out_rows >= 0 && hidden > 0, "bad sizes");
  PSAMD_REQUIRE(weight_dtype == kF32 || weight_dtype == kBF16, "weight dtype must be float32 or bfloat16");
  PSAMD_REQUIRE(delta == nullptr || delta_dtype == kF32 || delta_dtype == kBF16, "delta dtype");
  PSAMD_REQUIRE(delta == nullptr || (n_partials >= 1 && (n_partials == 1 || delta_dtype == kF32)),
                "partial sums must be float32");
  if (out_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  constexpr int kThreads = 256, kCache = 16;
  const dim3 grid(static_cast<unsigned>(out_rows)), block(kThreads);
#define PSAMD_NORM(A_, D_)                                                                                      \
  add_rmsnorm_kernel<A_, D_, kThreads, kCache><<<grid, block, 0, s>>>(                                          \
      residual, static_cast<const D_*>(delta), n_partials, partial_stride, rows, weight, weight_dtype, eps, \
      static_cast<A_*>(out), hidden)
  const bool delta_f32 = delta == nullptr || delta_dtype == kF32;
  if (act_dtype == kBF16 && hidden % 8 == 0 && hidden <= 8 * kThreads * 4) {
    bf16_t* o16 = static_cast<bf16_t*>(out);
#define PSAMD_NORM8(D_, IT_)                                                                                 \
  add_rmsnorm_vec8_kernel<D_, kThreads, IT_><<<grid, block, 0, s>>>(                                         \
      residual, static_cast<const D_*>(delta), n_partials, partial_stride, rows, weight, weight_dtype, eps, \
      o16, hidden)
    const int iters = static_cast<int>(ceil_div(hidden / 8, kThreads));
    if (delta_f32) {
      if (iters <= 1) PSAMD_NORM8(float, 1); else if (iters <= 2) PSAMD_NORM8(float, 2); else PSAMD_NORM8(float, 4);
    } else {
      if (iters <= 1) PSAMD_NORM8(bf16_t, 1); else if (iters <= 2) PSAMD_NORM8(bf16_t, 2); else PSAMD_NORM8(bf16_t, 4);
    }
#undef PSAMD_NORM8
    return check_launch("psamd_add_rmsnorm");
  }
  if (act_dtype == kBF16) {
    if (delta_f32) PSAMD_NORM(bf16_t, float); else PSAMD_NORM(bf16_t, bf16_t);
  } else if (act_dtype == kF32) {
    if (delta_f32) PSAMD_NORM(float, float); else PSAMD_NORM(float, bf16_t);
  } else {
    return fail("psamd_add_rmsnorm: activation dtype must be float32 or bfloat16");
  }
#undef PSAMD_NORM
  return check_launch("psamd_add_rmsnorm");
}

int psamd_swiglu(void* stream, const void* gate_up, void* out, int act_dtype, int64_t tokens, int inter) {
  PSAMD_REQUIRE(tokens >= 0 && inter > 0, "bad sizes");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t n = tokens * inter;
  const int blocks = static_cast<int>(std::min<int64_t>(ceil_div(n, 256), 65536));
  if (act_dtype == kBF16 && inter % 8 == 0) {
    const int vblocks = static_cast<int>(std::min<int64_t>(ceil_div(n / 8, 256), 65536));
    swiglu_vec8_kernel<<<dim3(vblocks), dim3(256), 0, s>>>(static_cast<const bf16_t*>(gate_up),
                                                           static_cast<bf16_t*>(out), tokens, inter);
  } else if (act_dtype == kBF16) {
    swiglu_kernel<bf16_t><<<dim3(blocks), dim3(256), 0, s>>>(static_cast<const bf16_t*>(gate_up),
                                                            static_cast<bf16_t*>(out), tokens, inter);
  } else if (act_dtype == kF32) {
    swiglu_kernel<float><<<dim3(blocks), dim3(256), 0, s>>>(static_cast<const float*>(gate_up),
                                                           static_cast<float*>(out), tokens, inter);
  } else {
    return fail("psamd_swiglu: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_swiglu");
}

int psamd_rope_kv_append(void* stream, void* qkv, int act_dtype, int64_t tokens, int hq, int hkv, int head_dim,
                         const int32_t* positions, const float* table, void* kv, const int32_t* write_slot) {
  PSAMD_REQUIRE(tokens >= 0 && hq > 0 && hkv > 0, "bad sizes");
  PSAMD_REQUIRE(head_dim > 0 && head_dim % 2 == 0, "head_dim must be even");
  PSAMD_REQUIRE(kv == nullptr || write_slot != nullptr, "a cache needs write slots");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float2* tab = reinterpret_cast<const float2*>(table);
  if (act_dtype == kBF16 && head_dim % 16 == 0 && static_cast<size_t>(16) * (hkv * head_dim + 8) * sizeof(bf16_t) <= 64 * 1024) {
    const size_t smem = static_cast<size_t>(16) * (hkv * head_dim + 8) * sizeof(bf16_t);
    // Enough blocks for every compute unit, each with at least a round of work for its threads.
    const int64_t groups = ceil_div(tokens, 16);
    const int64_t rot_rounds = ceil_div(static_cast<int64_t>(16) * (hq + hkv) * (head_dim / 16), 256);
    const unsigned split = static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>({rot_rounds, 16, ceil_div(1024, groups)})));
    rope_kv_append_vec_kernel<<<dim3(static_cast<unsigned>(groups), split), dim3(256), smem, s>>>(
        static_cast<bf16_t*>(qkv), static_cast<int>(tokens), hq, hkv, head_dim, positions, tab, static_cast<bf16_t*>(kv),
        write_slot);
  } else if (act_dtype == kBF16) {
    rope_kv_append_kernel<bf16_t><<<dim3(tokens), dim3(256), 0, s>>>(static_cast<bf16_t*>(qkv), hq, hkv, head_dim,
                                                                    positions, tab, static_cast<bf16_t*>(kv), write_slot);
  } else if (act_dtype == kF32) {
    rope_kv_append_kernel<float><<<dim3(tokens), dim3(256), 0, s>>>(static_cast<float*>(qkv), hq, hkv, head_dim,
                                                                   positions, tab, static_cast<float*>(kv), write_slot);
  } else {
    return fail("psamd_rope_kv_append: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_rope_kv_append");
}

}  // extern "C"
