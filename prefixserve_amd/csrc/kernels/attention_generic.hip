// Causal grouped-query attention over the paged cache, the straightforward way: one wave
// per (new token, query head), float arithmetic throughout, any head size that is a
// multiple of 2 up to 256, any number of heads and groups, optional sliding window.
// It is the attention of the exact 32-bit path and the fallback for shapes the
// matrix-core kernels do not take.
//
// Page layout (per layer): [num_blocks][2][kv_heads][16 * D]; half 0 = keys [16][D],
// half 1 = values transposed [D][16].

#include "api.h"
#include "common.h"

namespace psamd {

template <typename A>
__global__ __launch_bounds__(64) void attention_generic_kernel(
    const A* __restrict__ qkv, int q_stride, A* __restrict__ out, const A* __restrict__ kv,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ tok_item,
    const int32_t* __restrict__ table_off, const int32_t* __restrict__ block_ids,
    int hq, int hkv, int d, float scale, int window) {
  __shared__ float q_s[256];
  __shared__ float p_s[kWave];
  __shared__ int32_t base_s[kWave];   // element offset of (page, kv head) for each key of the chunk
  __shared__ int32_t off_s[kWave];
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int kvh = h / (hq / hkv);
  const int pos = positions[t];
  const int item = tok_item[t];
  const int32_t* table = block_ids + table_off[item];
  const int k_lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int64_t page_elems = 2LL * hkv * kPage * d;
  const int64_t half_elems = static_cast<int64_t>(hkv) * kPage * d;

  const A* q = qkv + t * q_stride + h * d;
  for (int i = lane; i < d; i += kWave) q_s[i] = to_float<A>(q[i]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};   // dims lane, lane+64, lane+128, lane+192
  for (int c0 = k_lo; c0 <= pos; c0 += kWave) {
    const int j = c0 + lane;
    float s = -INFINITY;
    if (j <= pos) {
      const int64_t page = table[j / kPage];
      const int off = j % kPage;
      const int64_t base = page * page_elems + static_cast<int64_t>(kvh) * kPage * d;
      const A* kr = kv + base + static_cast<int64_t>(off) * d;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot = fmaf(q_s[i], to_float<A>(kr[i]), dot);
      s = dot * scale;
      base_s[lane] = static_cast<int32_t>(page);
      off_s[lane] = off;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = j <= pos ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);   // m = -inf on the first chunk gives 0
    l = l * alpha + wave_sum(p);
    m = m_new;
    p_s[lane] = p;
    __syncthreads();
    const int cnt = min(kWave, pos - c0 + 1);
#pragma unroll
    for (int dd = 0; dd < 4; ++dd) {
      const int i = lane + dd * kWave;
      if (i < d) {
        float a = acc[dd] * alpha;
        for (int jj = 0; jj < cnt; ++jj) {
          const int64_t vb = static_cast<int64_t>(base_s[jj]) * page_elems + half_elems +
                             (static_cast<int64_t>(kvh) * d + i) * kPage + off_s[jj];
          a = fmaf(p_s[jj], to_float<A>(kv[vb]), a);
        }
        acc[dd] = a;
      }
    }
    __syncthreads();
  }
  const float inv = 1.f / l;
  A* o = out + t * (static_cast<int64_t>(hq) * d) + h * d;
#pragma unroll
  for (int dd = 0; dd < 4; ++dd) {
    const int i = lane + dd * kWave;
    if (i < d) o[i] = from_float<A>(acc[dd] * inv);
  }
}

}  // namespace psamd

using namespace psamd;

extern "C" int psamd_attention_generic(void* stream, const void* qkv, int q_stride, void* out, const void* kv,
                                       int act_dtype, int64_t tokens, const int32_t* positions,
                                       const int32_t* tok_item, const int32_t* table_off, const int32_t* block_ids,
                                       int hq, int hkv, int head_dim, float scale, int window) {
  PSAMD_REQUIRE(tokens >= 0 && hq > 0 && hkv > 0 && hq % hkv == 0, "bad head counts");
  PSAMD_REQUIRE(head_dim > 0 && head_dim <= 256, "head_dim must be in [1, 256]");
  PSAMD_REQUIRE(hq <= 65535, "too many heads for one launch");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(tokens), static_cast<unsigned>(hq));
  if (act_dtype == kBF16) {
    attention_generic_kernel<bf16_t><<<grid, dim3(64), 0, s>>>(
        static_cast<const bf16_t*>(qkv), q_stride, static_cast<bf16_t*>(out), static_cast<const bf16_t*>(kv),
        positions, tok_item, table_off, block_ids, hq, hkv, head_dim, scale, window);
  } else if (act_dtype == kF32) {
    attention_generic_kernel<float><<<grid, dim3(64), 0, s>>>(
        static_cast<const float*>(qkv), q_stride, static_cast<float*>(out), static_cast<const float*>(kv),
        positions, tok_item, table_off, block_ids, hq, hkv, head_dim, scale, window);
  } else {
    return fail("psamd_attention_generic: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_attention_generic");
}
