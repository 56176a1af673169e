// All layers of a small decode step (at most 16 requests, one token each, bfloat16) in ONE
// kernel: a persistent grid of one workgroup per compute unit that walks through the phases
// of every layer with a software barrier between them.
//
// Why: launched one by one, a decode step of this size is bound by what every kernel pays
// before it streams (launch, first trip to memory, drain): 8 kernels per layer, 4 to 7 us
// each, for 2 to 15 us worth of bytes. Here a layer is 5 phases,
//   1. RMSNorm (folded into the operand load) + q/k/v product + rotation + cache write
//   2. attention over the cache, keys split over workgroups, the last split of a
//      (request, kv head) to finish merges them
//   3. output projection, added into the residual stream
//   4. RMSNorm (folded) + gate/up product + SiLU gate
//   5. down projection, added into the residual stream
// the workgroups stay resident, and the weights of the next phase are requested while a
// workgroup waits at the barrier, so the memory pipe does not drain between phases.
//
// The barrier has two levels because the chip has eight dies with an L2 each: workgroups
// first count in per die (their stores are then in that die's L2); the last one of a die
// writes the die's L2 back once (release at device scope) and counts the die in; everybody
// waits for all dies and invalidates its caches (acquire). One write-back per die and barrier,
// not one per workgroup. Which die a workgroup runs on is read from the hardware register,
// and how many workgroups each die got is counted at the start of the kernel, so nothing
// is assumed about how the dispatcher spreads workgroups.
//
// Every wait is bounded: a workgroup that spins longer than `spin_limit` polls sets the error
// flag, and from then on no barrier of the launch waits, so the grid always drains; the host
// reads the flag with the step's results. The state the barriers count in is left zeroed by
// the last workgroup to leave.
//
// Products are laid out as in skinny_mfma (v_mfma_f32_16x16x32_bf16, weights streamed once, the
// 8 waves of a workgroup take the k-steps in turn and are summed through LDS), with two
// differences: a workgroup owns whole output rows over all of K, so that it can finish them
// (rotation, residual add) without a second kernel; and the normalisation is applied as
// y = (W (x * g)) / rms(x): the operand is residual * norm weight, rounded to bfloat16, the
// sum of squares is gathered in the same pass and the scale is applied to the sums.

#include <algorithm>

#include "api.h"
#include "common.h"

namespace psamd {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kWaves = 8;            // waves of a workgroup
constexpr int kThreads = 64 * kWaves;
constexpr int kMaxTokens = 16;
constexpr int kMaxDies = 16;
constexpr int kMaxGroups = 4;        // layer groups a step can bring block tables for

__device__ __forceinline__ bf16x8 ld8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x4 ld4(const bf16_t* p) { return *reinterpret_cast<const bf16x4*>(p); }
__device__ __forceinline__ bf16x8 zeros8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = static_cast<__bf16>(0.f);
  return z;
}
__device__ __forceinline__ bf16x8 join(bf16x4 a, bf16x4 b) {
  bf16x8 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    r[i] = a[i];
    r[i + 4] = b[i];
  }
  return r;
}
__device__ __forceinline__ float silu_f(float g) { return g / (1.f + __expf(-g)); }

}  // namespace

// One per layer run, in device memory (the host writes the array once per model).
struct FusedLayer {
  const bf16_t* w_qkv;       // [(hq + 2 hkv) * D, H]
  const bf16_t* w_o;         // [H, hq * D]
  const bf16_t* w_gate_up;   // [2 I, H]
  const bf16_t* w_down;      // [H, I]
  const void* norm1;         // [H], norm_dtype
  const void* norm2;
  bf16_t* kv;                // pages of this run's cache entry
  const float2* rope;        // [positions, D / 2] (cos, sin), or null: no rotation
  float eps1, eps2;
  int32_t norm_dtype;
  int32_t group;             // which of the step's block tables
  int32_t writes_cache;
  int32_t pad;
};
static_assert(sizeof(FusedLayer) == 88, "the host packs this layout");

// Barrier state, zero before the first launch and left zero by every launch that ends well.
struct SyncState {
  unsigned registered;       // workgroups that have announced their die
  unsigned top;              // dies counted in, summed over the barriers so far
  unsigned exited;
  unsigned pad0[29];
  unsigned members[kMaxDies];            // workgroups per die
  unsigned pad1[32 - kMaxDies];
  unsigned arrived[kMaxDies][32];        // per die, a cache line of its own
  unsigned pair_done[1];                 // [tokens * kv heads]: splits that have written their partial result
};

struct FusedArgs {
  const FusedLayer* layers;
  int n_layers;
  float* residual;           // [T, H] float32, in and out
  bf16_t* qkv;               // [T, (hq + 2 hkv) * D]
  bf16_t* attn_out;          // [T, hq * D]
  bf16_t* act;               // [T, I]
  float* part_o;             // [T * hq * nsplit * D]
  float* part_ml;            // [T * hq * nsplit * 2]
  SyncState* sync;
  int* error;
  const int32_t* positions;  // [T]
  const int32_t* dec_items;  // [T] items that bring one token (all of them here)
  const int32_t* item_start;
  const int32_t* item_end;
  const int32_t* table_off[kMaxGroups];
  const int32_t* block_ids[kMaxGroups];
  const int32_t* write_slot[kMaxGroups];
  int T, H, I, hq, hkv, nsplit;
  float scale;
  unsigned spin_limit;
  long long* trace;          // null, or [n_layers][10] times (100 MHz) at which workgroup 0 ended each phase and passed each barrier
};

namespace {

// What a workgroup knows about the grid; in LDS, written by thread 0.
struct GridInfo {
  unsigned die_index;   // this workgroup's die among the dies that got workgroups, 0..dies-1
  unsigned die_slot;    // the hardware's id of the die (index into SyncState)
  unsigned rank;        // this workgroup among those of its die
  unsigned per_die;     // workgroups of its die
  unsigned dies;
  unsigned passed;      // barriers passed
  int failed;           // a wait ran out: no barrier waits any more
};

__device__ __forceinline__ unsigned die_id() {
  // XCC_ID, bits 3:0 of hardware register 20
  return __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & (kMaxDies - 1);
}

__device__ __forceinline__ unsigned load_relaxed(unsigned* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Every workgroup announces the die it runs on and waits until all have.
__device__ void grid_register(const FusedArgs& a, GridInfo* gi) {
  if (threadIdx.x == 0) {
    SyncState* st = a.sync;
    const unsigned die = die_id();
    const unsigned rank = __hip_atomic_fetch_add(&st->members[die], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // The count of registered workgroups must not become visible before the die's count: the
    // operand depends on the first result, so the second atomic waits for it.
    __hip_atomic_fetch_add(&st->registered, 1u + (rank >> 31), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    unsigned polls = 0;
    int failed = 0;
    while (load_relaxed(&st->registered) < gridDim.x) {
      if (++polls > a.spin_limit) {
        failed = 1;
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
    unsigned dies = 0, index = 0;
    for (unsigned d = 0; d < kMaxDies; ++d) {
      const unsigned n = load_relaxed(&st->members[d]);
      if (n > 0) {
        if (d < die) ++index;
        ++dies;
      }
    }
    gi->die_index = index;
    gi->die_slot = die;
    gi->rank = rank;
    gi->per_die = load_relaxed(&st->members[die]);
    gi->dies = dies;
    gi->passed = 0;
    gi->failed = failed;
    if (failed) atomicExch(a.error, 1);
  }
  __syncthreads();
}

// All stores of all workgroups before the barrier are visible to all loads after it.
__device__ void grid_barrier(const FusedArgs& a, GridInfo* gi) {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");   // this wave's stores have reached the die's L2
  __syncthreads();
  if (threadIdx.x == 0 && !gi->failed) {
    SyncState* st = a.sync;
    const unsigned k = gi->passed;
    const unsigned old = __hip_atomic_fetch_add(&st->arrived[gi->die_slot][0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (old + 1 == (k + 1) * gi->per_die)      // last of this die: one write-back of its L2 for all of them
      __hip_atomic_fetch_add(&st->top, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned want = (k + 1) * gi->dies;
    unsigned polls = 0;
    while (load_relaxed(&st->top) < want) {
      if (++polls > a.spin_limit) {
        gi->failed = 1;
        atomicExch(a.error, 2);
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    gi->passed = k + 1;
  }
  __syncthreads();
}

// The last workgroup to leave zeroes the barrier state for the next launch.
__device__ void grid_leave(const FusedArgs& a, const GridInfo* gi) {
  __syncthreads();
  if (threadIdx.x != 0 || gi->failed) return;     // after a failure the host clears the state
  SyncState* st = a.sync;
  const unsigned old = __hip_atomic_fetch_add(&st->exited, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (old + 1 != gridDim.x) return;
  for (unsigned d = 0; d < kMaxDies; ++d) {
    __hip_atomic_store(&st->members[d], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&st->arrived[d][0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __hip_atomic_store(&st->registered, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(&st->top, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(&st->exited, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---------------------------------------------------------------- operands

// Tokens as the B operand of a k-step: lane (r, g) supplies token min(r, T-1), k = 32 s + 8 g + [0, 8).
// `in` is false for the lane groups of a last, partial k-step that lie past K: they supply zeros.
struct TokensBf16 {
  const bf16_t* row;      // this lane's token row + 8 g
  struct Raw { bf16x8 v; };
  __device__ __forceinline__ Raw load(int k, bool in) const { return Raw{in ? ld8(row + k) : zeros8()}; }
  __device__ __forceinline__ bf16x8 use(const Raw& raw, float&) const { return raw.v; }
};

// The same from the float32 residual stream times the norm weight; gathers the sum of squares.
template <bool NORM_BF16>
struct TokensNormed {
  const float* row;       // residual row of this lane's token + 8 g
  const void* weight;     // norm weight + 8 g
  struct Raw { float4 x0, x1; float4 w0, w1; bf16x8 wb; };
  __device__ __forceinline__ Raw load(int k, bool in) const {
    Raw raw;
    const float4 zero = float4{0.f, 0.f, 0.f, 0.f};
    raw.x0 = in ? *reinterpret_cast<const float4*>(row + k) : zero;
    raw.x1 = in ? *reinterpret_cast<const float4*>(row + k + 4) : zero;
    if (NORM_BF16) {
      raw.wb = in ? ld8(static_cast<const bf16_t*>(weight) + k) : zeros8();
    } else {
      raw.w0 = in ? *reinterpret_cast<const float4*>(static_cast<const float*>(weight) + k) : zero;
      raw.w1 = in ? *reinterpret_cast<const float4*>(static_cast<const float*>(weight) + k + 4) : zero;
    }
    return raw;
  }
  __device__ __forceinline__ bf16x8 use(const Raw& raw, float& ssq) const {
    const float x[8] = {raw.x0.x, raw.x0.y, raw.x0.z, raw.x0.w, raw.x1.x, raw.x1.y, raw.x1.z, raw.x1.w};
    float w[8];
    if (NORM_BF16) {
#pragma unroll
      for (int i = 0; i < 8; ++i) w[i] = static_cast<float>(raw.wb[i]);
    } else {
      w[0] = raw.w0.x; w[1] = raw.w0.y; w[2] = raw.w0.z; w[3] = raw.w0.w;
      w[4] = raw.w1.x; w[5] = raw.w1.y; w[6] = raw.w1.z; w[7] = raw.w1.w;
    }
    bf16x8 out;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      ssq = fmaf(x[i], x[i], ssq);
      out[i] = static_cast<__bf16>(x[i] * w[i]);
    }
    return out;
  }
};

// acc[i] += rows wrow[i] (this lane's row + 8 g, or null for a lane without a row) x tokens, over the
// k-steps wave, wave + 8, ... of K (a multiple of 8; `g` = lane / 16 tells which 8 of a step's 32
// this lane brings). U steps of loads are in flight together.
template <int NA, int U, typename Tokens>
__device__ __forceinline__ void stream_product(const bf16_t* const (&wrow)[NA], const Tokens& tok, int K, int wave, int g,
                                               f32x4 (&acc)[NA], float& ssq) {
  const int steps = (K + 31) >> 5;
  for (int base = wave; base < steps; base += kWaves * U) {
    bf16x8 av[NA][U];
    typename Tokens::Raw raw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = base + kWaves * u;
      if (s < steps) {
        const bool in = (s << 5) + 8 * g < K;
#pragma unroll
        for (int i = 0; i < NA; ++i) av[i][u] = (in && wrow[i] != nullptr) ? ld8(wrow[i] + (s << 5)) : zeros8();
        raw[u] = tok.load(s << 5, in);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = base + kWaves * u;
      if (s < steps) {
        const bf16x8 b = tok.use(raw[u], ssq);
#pragma unroll
        for (int i = 0; i < NA; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[i][u], b, acc[i], 0, 0, 0);
      }
    }
  }
}

// LDS of a workgroup: partial tiles of the waves, their sums of squares, the attention merge.
struct Shared {
  f32x4 red[kWaves][4][64];         // 32 KB
  float ssq[kWaves][16];
  GridInfo grid;
  int last[2];                      // per half of the workgroup: its split was the last of its pair
};

// Sum of a tile over the waves; every wave may call it for a different i after the barrier.
__device__ __forceinline__ f32x4 sum_waves(const Shared& sh, int i, int lane) {
  f32x4 s = sh.red[0][i][lane];
#pragma unroll
  for (int w = 1; w < kWaves; ++w) s += sh.red[w][i][lane];
  return s;
}

// 1 / rms of the token this lane holds results for (token = lane % 16), from the waves' sums of squares.
__device__ __forceinline__ float inv_rms(const Shared& sh, int r, int H, float eps) {
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) t += sh.ssq[w][r];
  return rsqrtf(t / static_cast<float>(H) + eps);
}

__device__ __forceinline__ void put_partials(Shared& sh, int wave, int lane, float ssq, bool with_ssq) {
  if (with_ssq) {
    ssq += __shfl_xor(ssq, 16, kWave);
    ssq += __shfl_xor(ssq, 32, kWave);
    if (lane < 16) sh.ssq[wave][lane] = ssq;
  }
}

// ---------------------------------------------------------------- phase 1: norm + q/k/v + rotation + cache write

template <bool NORM_BF16>
__device__ void phase_qkv(const FusedArgs& a, const FusedLayer& L, Shared& sh, int d) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int half = d >> 1, tiles_per_head = d >> 4;
  const int n_tiles = (a.hq + 2 * a.hkv) * tiles_per_head;
  const int tok = min(r, a.T - 1);
  TokensNormed<NORM_BF16> tokens{a.residual + static_cast<int64_t>(tok) * a.H + 8 * g,
                                 NORM_BF16 ? static_cast<const void*>(static_cast<const bf16_t*>(L.norm1) + 8 * g)
                                           : static_cast<const void*>(static_cast<const float*>(L.norm1) + 8 * g)};
  const int32_t* write_slot = a.write_slot[L.group];
  for (int t = blockIdx.x; t < n_tiles; t += gridDim.x) {
    // 8 columns of a head's first half and their 8 rotation partners
    const int head = t / tiles_per_head;
    const int p = (t - head * tiles_per_head) << 3;
    const int row = head * d + (r < 8 ? p + r : half + p + r - 8);
    const bf16_t* wrow[1] = {L.w_qkv + static_cast<int64_t>(row) * a.H + 8 * g};
    f32x4 acc[1] = {f32x4{0.f, 0.f, 0.f, 0.f}};
    float ssq = 0.f;
    stream_product<1, 8>(wrow, tokens, a.H, wave, g, acc, ssq);
    sh.red[wave][0][lane] = acc[0];
    put_partials(sh, wave, lane, ssq, true);
    __syncthreads();
    if (wave == 0) {
      const float rinv = inv_rms(sh, r, a.H, L.eps1);
      f32x4 own = sum_waves(sh, 0, lane);
      const bool second = g >= 2;
      const bool rotate = L.rope != nullptr && head < a.hq + a.hkv;
      const int pos = a.positions[tok];
      f32x4 res;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float mine = own[v] * rinv;
        const float other = __shfl_xor(mine, 32, kWave);
        float val = mine;
        if (rotate) {
          const float2 cs = L.rope[static_cast<int64_t>(pos) * half + p + 4 * (g & 1) + v];
          val = second ? mine * cs.x + other * cs.y : mine * cs.x - other * cs.y;
        }
        res[v] = val;
      }
      if (r < a.T) {
        const int e0 = (second ? half : 0) + p + 4 * (g & 1);
        ushort4 pk;
        pk.x = float_to_bf16(res[0]);
        pk.y = float_to_bf16(res[1]);
        pk.z = float_to_bf16(res[2]);
        pk.w = float_to_bf16(res[3]);
        *reinterpret_cast<ushort4*>(a.qkv + static_cast<int64_t>(r) * ((a.hq + 2 * a.hkv) * d) + head * d + e0) = pk;
        if (L.writes_cache && head >= a.hq) {
          const int slot = write_slot[r];
          const int64_t page_elems = 2LL * a.hkv * kPage * d;
          bf16_t* page = L.kv + static_cast<int64_t>(slot / kPage) * page_elems;
          const int off = slot % kPage;
          if (head < a.hq + a.hkv) {
            *reinterpret_cast<ushort4*>(page + (static_cast<int64_t>(head - a.hq) * kPage + off) * d + e0) = pk;
          } else {
            bf16_t* vp = page + static_cast<int64_t>(a.hkv) * kPage * d +
                         (static_cast<int64_t>(head - a.hq - a.hkv) * d + e0) * kPage + off;
            vp[0] = pk.x;
            vp[kPage] = pk.y;
            vp[2 * kPage] = pk.z;
            vp[3 * kPage] = pk.w;
          }
        }
      }
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------- phase 2: attention over the cache

// A half of the workgroup (4 waves) takes one (request, kv head, split of the keys); the pairs
// are dealt to the dies, so that all splits of a pair run on one die and meet in its L2.
template <int NS>
__device__ void phase_attention(const FusedArgs& a, const FusedLayer& L, Shared& sh, float* smem_attn) {
  constexpr int D = 16 * NS;
  constexpr int KS = (D + 31) / 32;
  const GridInfo& gi = sh.grid;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int hf = wave >> 2, w4 = wave & 3, tid_h = threadIdx.x & 255;
  const int r = lane & 15, g4 = lane >> 4;
  const int group = a.hq / a.hkv;
  const int pairs = a.T * a.hkv;
  const int my_pairs = pairs > static_cast<int>(gi.die_index) ? (pairs - gi.die_index + gi.dies - 1) / gi.dies : 0;
  const int my_items = my_pairs * a.nsplit;
  const int workers = 2 * gi.per_die;
  const int rounds = (my_items + workers - 1) / workers;
  float* smem = smem_attn + hf * (8 * group + 4 * group * D);
  float* sm_m = smem;
  float* sm_l = smem + 4 * group;
  float* sm_o = smem + 8 * group;
  const int32_t* table_off = a.table_off[L.group];
  const int32_t* block_ids = a.block_ids[L.group];
  const int64_t page_elems = 2LL * a.hkv * kPage * D;
  const int nsplit = a.nsplit;

  for (int round = 0; round < rounds; ++round) {
    const int j = round * workers + 2 * gi.rank + hf;
    const bool valid = j < my_items;
    int di = 0, kvh = 0, split = 0, pair = 0;
    if (valid) {
      const int lp = j / nsplit;
      split = j - lp * nsplit;
      pair = lp * gi.dies + gi.die_index;
      di = pair / a.hkv;
      kvh = pair - di * a.hkv;
    }
    int64_t t = 0;
    if (valid) {
      const int item = a.dec_items[di];
      t = a.item_start[item];
      const int pos = a.item_end[item] - 1;
      const int32_t* table = block_ids + table_off[item];
      const int tile_hi = pos >> 5;
      const int tps = (tile_hi + nsplit) / nsplit;
      const int my_lo = split * tps;
      const int my_hi = min(my_lo + tps, tile_hi + 1);
      const int64_t khead = static_cast<int64_t>(kvh) * kPage * D;
      const int64_t vhead = static_cast<int64_t>(a.hkv) * kPage * D + static_cast<int64_t>(kvh) * D * kPage;

      bf16x8 qf[KS];
      {
        const bf16_t* qp = a.qkv + t * ((a.hq + 2 * a.hkv) * D) + static_cast<int64_t>(kvh * group + min(r, group - 1)) * D + 8 * g4;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bool in = r < group && 32 * ks + 8 * g4 < D;
          qf[ks] = in ? ld8(qp + 32 * ks) : zeros8();
        }
      }
      f32x4 o[NS];
      float m = -INFINITY, l = 0.f;
#pragma unroll
      for (int ds = 0; ds < NS; ++ds) o[ds] = f32x4{0.f, 0.f, 0.f, 0.f};

      for (int tile = my_lo + w4; tile < my_hi; tile += 4) {
        const int k0 = tile << 5;
        const int64_t page0 = table[min(k0, pos) >> 4];
        const int64_t page1 = table[min(k0 + 16, pos) >> 4];
        const bf16_t* kp0 = L.kv + page0 * page_elems + khead + r * D + 8 * g4;
        const bf16_t* kp1 = L.kv + page1 * page_elems + khead + r * D + 8 * g4;
        bf16x8 ka0[KS], ka1[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bool in = 32 * ks + 8 * g4 < D;
          ka0[ks] = in ? ld8(kp0 + 32 * ks) : zeros8();
          ka1[ks] = in ? ld8(kp1 + 32 * ks) : zeros8();
        }
        const bf16_t* vp0 = L.kv + page0 * page_elems + vhead + 4 * g4;
        const bf16_t* vp1 = L.kv + page1 * page_elems + vhead + 4 * g4;
        bf16x8 va[NS];
#pragma unroll
        for (int ds = 0; ds < NS; ++ds) {
          const int drow = 16 * ds + r;
          va[ds] = join(ld4(vp0 + drow * kPage), ld4(vp1 + drow * kPage));
        }
        f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka0[ks], qf[ks], s0, 0, 0, 0);
          s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka1[ks], qf[ks], s1, 0, 0, 0);
        }
        float sv[8];
        float mx = -INFINITY;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int key0 = k0 + 4 * g4 + v, key1 = key0 + 16;
          sv[v] = key0 <= pos ? s0[v] * a.scale : -INFINITY;
          sv[v + 4] = key1 <= pos ? s1[v] * a.scale : -INFINITY;
          mx = fmaxf(mx, fmaxf(sv[v], sv[v + 4]));
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
        mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
        const float m_new = fmaxf(m, mx);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __expf(m - m_use);
        float rowsum = 0.f;
        bf16x8 pb;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float p = __expf(sv[e] - m_use);
          rowsum += p;
          pb[e] = static_cast<__bf16>(p);
        }
        rowsum += __shfl_xor(rowsum, 16, kWave);
        rowsum += __shfl_xor(rowsum, 32, kWave);
        l = l * alpha + rowsum;
        m = m_new;
#pragma unroll
        for (int ds = 0; ds < NS; ++ds) {
          o[ds] *= alpha;
          // Keys past the request's last position and slots of a page nobody has written yet
          // may hold anything; their probability is zero, and so is what they add.
          o[ds] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[ds], pb, o[ds], 0, 0, 0);
        }
      }
      // the 4 waves of this half meet in LDS
      if (r < group) {
        if (g4 == 0) {
          sm_m[w4 * group + r] = m;
          sm_l[w4 * group + r] = l;
        }
#pragma unroll
        for (int ds = 0; ds < NS; ++ds)
#pragma unroll
          for (int v = 0; v < 4; ++v) sm_o[(static_cast<int64_t>(w4) * group + r) * D + 16 * ds + 4 * g4 + v] = o[ds][v];
      }
    }
    __syncthreads();
    if (valid) {
      for (int idx = tid_h; idx < group * D; idx += 256) {
        const int hh = idx / D, dd = idx - hh * D;
        float mm = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w) mm = fmaxf(mm, sm_m[w * group + hh]);
        float acc = 0.f, ll = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const float mw = sm_m[w * group + hh];
          const float wgt = mw == -INFINITY ? 0.f : __expf(mw - mm);
          acc += wgt * sm_o[(static_cast<int64_t>(w) * group + hh) * D + dd];
          ll += wgt * sm_l[w * group + hh];
        }
        if (nsplit == 1) {
          a.attn_out[t * (static_cast<int64_t>(a.hq) * D) + static_cast<int64_t>(kvh * group + hh) * D + dd] = float_to_bf16(acc / ll);
        } else {
          const int64_t slot = (static_cast<int64_t>(di) * a.hq + kvh * group + hh) * nsplit + split;
          a.part_o[slot * D + dd] = acc;
          if (dd == 0) {
            a.part_ml[slot * 2 + 0] = mm;
            a.part_ml[slot * 2 + 1] = ll;
          }
        }
      }
    }
    if (nsplit == 1) {
      __syncthreads();          // sm_* are free for the next round
      continue;
    }
    // The split that finds all others done merges the pair. Partial results are in this die's
    // L2 once the stores are acknowledged; the counter is only touched by workgroups of this die.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (tid_h == 0) {
      int last = 0;
      if (valid) {
        const unsigned old = __hip_atomic_fetch_add(&a.sync->pair_done[pair], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last = old + 1 == static_cast<unsigned>(nsplit);
        if (last) __hip_atomic_store(&a.sync->pair_done[pair], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      sh.last[hf] = last;
    }
    __syncthreads();
    if (sh.last[hf]) {
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
      for (int idx = tid_h; idx < group * D; idx += 256) {
        const int hh = idx / D, dd = idx - hh * D;
        const int64_t base = (static_cast<int64_t>(di) * a.hq + kvh * group + hh) * nsplit;
        float mm = -INFINITY;
        for (int s = 0; s < nsplit; ++s) mm = fmaxf(mm, a.part_ml[(base + s) * 2]);
        float acc = 0.f, ll = 0.f;
        for (int s = 0; s < nsplit; ++s) {
          const float ms = a.part_ml[(base + s) * 2];
          const float wgt = ms == -INFINITY ? 0.f : __expf(ms - mm);
          acc += wgt * a.part_o[(base + s) * D + dd];
          ll += wgt * a.part_ml[(base + s) * 2 + 1];
        }
        a.attn_out[t * (static_cast<int64_t>(a.hq) * D) + static_cast<int64_t>(kvh * group + hh) * D + dd] = float_to_bf16(acc / ll);
      }
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------- phases 3 and 5: product added into the residual

// residual[t, n] += sum_k x[t, k] w[n, k] for all n < N: a workgroup owns `rpt` rows of w over all
// of K (rpt <= 16, chosen so that every workgroup has rows), so the sums are whole and are
// added in place by their only owner.
__device__ void phase_rows(const FusedArgs& a, const bf16_t* w, const bf16_t* x, int N, int K, Shared& sh) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int rpt = min(16, max(1, (N + static_cast<int>(gridDim.x) - 1) / static_cast<int>(gridDim.x)));
  const int n_tiles = (N + rpt - 1) / rpt;
  TokensBf16 tokens{x + static_cast<int64_t>(min(r, a.T - 1)) * K + 8 * g};
  for (int t = blockIdx.x; t < n_tiles; t += gridDim.x) {
    const int row0 = t * rpt;
    const int row = row0 + r;
    const bf16_t* wrow[1] = {(r < rpt && row < N) ? w + static_cast<int64_t>(row) * K + 8 * g : nullptr};
    f32x4 acc[1] = {f32x4{0.f, 0.f, 0.f, 0.f}};
    float unused = 0.f;
    stream_product<1, 8>(wrow, tokens, K, wave, g, acc, unused);
    sh.red[wave][0][lane] = acc[0];
    __syncthreads();
    if (wave == 0 && r < a.T) {
      const f32x4 sum = sum_waves(sh, 0, lane);
      float* dst = a.residual + static_cast<int64_t>(r) * a.H + row0;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int i = 4 * g + v;
        if (i < rpt && row0 + i < N) dst[i] += sum[v];
      }
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------- phase 4: norm + gate/up + SiLU gate

template <bool NORM_BF16>
__device__ void phase_gate_up(const FusedArgs& a, const FusedLayer& L, Shared& sh) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n_pt = a.I >> 4;                    // tiles of 16 gate/up pairs
  const int units = (n_pt + 1) >> 1;            // two tiles per workgroup and pass
  const int tok = min(r, a.T - 1);
  TokensNormed<NORM_BF16> tokens{a.residual + static_cast<int64_t>(tok) * a.H + 8 * g,
                                 NORM_BF16 ? static_cast<const void*>(static_cast<const bf16_t*>(L.norm2) + 8 * g)
                                           : static_cast<const void*>(static_cast<const float*>(L.norm2) + 8 * g)};
  for (int u = blockIdx.x; u < units; u += gridDim.x) {
    const int pt0 = 2 * u, pt1 = 2 * u + 1;
    const bool two = pt1 < n_pt;
    const bf16_t* g0 = L.w_gate_up + static_cast<int64_t>(16 * pt0 + r) * a.H + 8 * g;
    const bf16_t* wrow[4] = {g0, g0 + static_cast<int64_t>(a.I) * a.H, two ? g0 + 16LL * a.H : nullptr,
                             two ? g0 + (static_cast<int64_t>(a.I) + 16) * a.H : nullptr};
    f32x4 acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    float ssq = 0.f;
    stream_product<4, NORM_BF16 ? 4 : 2>(wrow, tokens, a.H, wave, g, acc, ssq);   // float32 norm weights: twice the registers per step
#pragma unroll
    for (int i = 0; i < 4; ++i) sh.red[wave][i][lane] = acc[i];
    put_partials(sh, wave, lane, ssq, true);
    __syncthreads();
    if (wave < 2 && (wave == 0 || two) && r < a.T) {
      const float rinv = inv_rms(sh, r, a.H, L.eps2);
      const f32x4 gate = sum_waves(sh, 2 * wave, lane);
      const f32x4 up = sum_waves(sh, 2 * wave + 1, lane);
      ushort4 pk;
      pk.x = float_to_bf16(silu_f(gate[0] * rinv) * (up[0] * rinv));
      pk.y = float_to_bf16(silu_f(gate[1] * rinv) * (up[1] * rinv));
      pk.z = float_to_bf16(silu_f(gate[2] * rinv) * (up[2] * rinv));
      pk.w = float_to_bf16(silu_f(gate[3] * rinv) * (up[3] * rinv));
      *reinterpret_cast<ushort4*>(a.act + static_cast<int64_t>(r) * a.I + 16 * (wave == 0 ? pt0 : pt1) + 4 * g) = pk;
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------- the kernel

template <int NS, bool NORM_BF16>
__global__ __launch_bounds__(kThreads) void decode_layers_kernel(const FusedArgs a) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  Shared& sh = *reinterpret_cast<Shared*>(lds_raw);
  float* smem_attn = reinterpret_cast<float*>(lds_raw + sizeof(Shared));
  constexpr int D = 16 * NS;
  grid_register(a, &sh.grid);
  const bool tracing = a.trace != nullptr && blockIdx.x == 0 && threadIdx.x == 0;
  auto mark = [&](int li, int i) {
    if (tracing) a.trace[li * 10 + i] = wall_clock64();
  };
  for (int li = 0; li < a.n_layers; ++li) {
    const FusedLayer L = a.layers[li];
    phase_qkv<NORM_BF16>(a, L, sh, D);
    mark(li, 0);
    grid_barrier(a, &sh.grid);
    mark(li, 1);
    phase_attention<NS>(a, L, sh, smem_attn);
    mark(li, 2);
    grid_barrier(a, &sh.grid);
    mark(li, 3);
    phase_rows(a, L.w_o, a.attn_out, a.H, a.hq * D, sh);
    mark(li, 4);
    grid_barrier(a, &sh.grid);
    mark(li, 5);
    phase_gate_up<NORM_BF16>(a, L, sh);
    mark(li, 6);
    grid_barrier(a, &sh.grid);
    mark(li, 7);
    phase_rows(a, L.w_down, a.act, a.H, a.I, sh);
    mark(li, 8);
    grid_barrier(a, &sh.grid);
    mark(li, 9);
  }
  grid_leave(a, &sh.grid);
}

size_t fused_lds_bytes(int hq, int hkv, int d) {
  const int group = hq / hkv;
  return sizeof(Shared) + 2 * sizeof(float) * (8 * static_cast<size_t>(group) + 4 * static_cast<size_t>(group) * d);
}

int g_compute_units = 0;

int compute_units() {
  if (g_compute_units == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
    g_compute_units = prop.multiProcessorCount;
  }
  return g_compute_units;
}

template <int NS, bool NORM_BF16>
int launch_fused(hipStream_t s, const FusedArgs& a, int d, int grid) {
  const size_t lds = fused_lds_bytes(a.hq, a.hkv, d);
  auto kernel = decode_layers_kernel<NS, NORM_BF16>;
  // Checked once per kernel and LDS size: every workgroup of the grid must be resident at once,
  // or the barrier would wait for workgroups that cannot start.
  static size_t checked_lds = 0;
  if (checked_lds != lds) {
    if (lds > 64 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(lds)) != hipSuccess)
      return fail("psamd_decode_layers: cannot have that much LDS");
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kThreads, lds) != hipSuccess || per_cu < 1)
      return fail("psamd_decode_layers: a workgroup does not fit a compute unit");
    checked_lds = lds;
  }
  kernel<<<dim3(static_cast<unsigned>(grid)), dim3(kThreads), lds, s>>>(a);
  return check_launch("psamd_decode_layers");
}

}  // namespace

}  // namespace psamd

using namespace psamd;

extern "C" {

// Bytes of barrier state for steps of up to max_tokens requests (zeroed by the caller once).
int64_t psamd_decode_layers_sync_bytes(int max_tokens, int hkv) {
  return static_cast<int64_t>(sizeof(SyncState)) + 4LL * std::max(max_tokens, 1) * std::max(hkv, 1);
}

int psamd_decode_layers_layer_bytes(void) { return static_cast<int>(sizeof(FusedLayer)); }

// 1 if the fused decode step takes these sizes, else 0 (the caller then runs the layers kernel by kernel).
int psamd_decode_layers_supports(int tokens, int hidden, int inter, int hq, int hkv, int head_dim, int norm_dtype) {
  if (tokens < 1 || tokens > kMaxTokens) return 0;
  if (hq <= 0 || hkv <= 0 || hq % hkv || hq / hkv > 16) return 0;
  if (!(head_dim == 16 || head_dim == 32 || head_dim == 64 || head_dim == 128)) return 0;
  if (hidden % 8 || inter % 16) return 0;        // 16-byte rows; whole tiles of 16 gate/up pairs
  if (norm_dtype != kF32 && norm_dtype != kBF16) return 0;
  if (fused_lds_bytes(hq, hkv, head_dim) > 96 * 1024) return 0;
  return compute_units() > 0;
}

int psamd_decode_layers(void* stream, const void* layers, int n_layers, float* residual, void* qkv, void* attn_out,
                        void* act, float* part_o, float* part_ml, void* sync, int* error, const int32_t* positions,
                        const int32_t* dec_items, const int32_t* item_start, const int32_t* item_end,
                        const int32_t* const* table_off, const int32_t* const* block_ids,
                        const int32_t* const* write_slot, int n_groups, int tokens, int hidden, int inter, int hq, int hkv,
                        int head_dim, int norm_dtype, int nsplit, float scale, int64_t spin_limit, int64_t* trace) {
  PSAMD_REQUIRE(psamd_decode_layers_supports(tokens, hidden, inter, hq, hkv, head_dim, norm_dtype),
                "sizes not taken by the fused decode step");
  PSAMD_REQUIRE(n_layers >= 1 && n_groups >= 1 && n_groups <= kMaxGroups, "1 to 4 layer groups");
  PSAMD_REQUIRE(nsplit >= 1 && nsplit <= 64, "nsplit must be in [1, 64]");
  PSAMD_REQUIRE(spin_limit >= 1 && spin_limit <= 0x7fffffffLL, "spin_limit must be positive");
  FusedArgs a;
  a.layers = static_cast<const FusedLayer*>(layers);
  a.n_layers = n_layers;
  a.residual = residual;
  a.qkv = static_cast<bf16_t*>(qkv);
  a.attn_out = static_cast<bf16_t*>(attn_out);
  a.act = static_cast<bf16_t*>(act);
  a.part_o = part_o;
  a.part_ml = part_ml;
  a.sync = static_cast<SyncState*>(sync);
  a.error = error;
  a.positions = positions;
  a.dec_items = dec_items;
  a.item_start = item_start;
  a.item_end = item_end;
  for (int g = 0; g < kMaxGroups; ++g) {
    a.table_off[g] = g < n_groups ? table_off[g] : nullptr;
    a.block_ids[g] = g < n_groups ? block_ids[g] : nullptr;
    a.write_slot[g] = g < n_groups ? write_slot[g] : nullptr;
  }
  a.T = tokens;
  a.H = hidden;
  a.I = inter;
  a.hq = hq;
  a.hkv = hkv;
  a.nsplit = nsplit;
  a.scale = scale;
  a.spin_limit = static_cast<unsigned>(spin_limit);
  a.trace = reinterpret_cast<long long*>(trace);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int grid = compute_units();
  const bool nb = norm_dtype == kBF16;
#define PSAMD_FUSED(NS_)                                                          \
  return nb ? launch_fused<NS_, true>(s, a, head_dim, grid) : launch_fused<NS_, false>(s, a, head_dim, grid)
  switch (head_dim / 16) {
    case 1: PSAMD_FUSED(1);
    case 2: PSAMD_FUSED(2);
    case 4: PSAMD_FUSED(4);
    default: PSAMD_FUSED(8);
  }
#undef PSAMD_FUSED
}

}  // extern "C"
