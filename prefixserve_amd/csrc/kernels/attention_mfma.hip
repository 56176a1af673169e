// bfloat16 causal grouped-query attention over the paged cache on the CDNA4 matrix cores.
//
// Both kernels compute the score tile TRANSPOSED, S^T = K * Q^T (keys are rows), because the
// accumulator layout of S^T is, lane for lane, the B-operand layout of the next product
// O^T = V^T * P^T: probabilities go from the first product's registers straight into the
// second without passing through LDS. The cache stores values transposed per page
// ([D][16], see elementwise.hip) so that V^T rows are contiguous 8-byte runs.
//
//  * prefill: one workgroup per (32 new tokens, query head), its 4 waves splitting the keys;
//    v_mfma_f32_32x32x16_bf16; online softmax per query column held redundantly in lanes l
//    and l^32; log-sum-exp merge of the waves in LDS.
//  * decode: one workgroup per (request, kv head, split of the key range); the `group`
//    query heads sharing the kv head are the columns of a 16x16x32 tile, so every key and
//    value byte is read once for all of them; 4 waves interleave 32-key tiles and merge by
//    log-sum-exp in LDS; a second small kernel merges the splits (a device-wide fence inside
//    the kernel would be far dearer than a launch on this multi-die part).
//
// Softmax statistics, scaling and masks are float. Page layout per layer:
// [num_blocks][2][kv_heads][16 * D], half 0 keys [16][D], half 1 values [D][16].

#include <algorithm>

#include "api.h"
#include "common.h"

namespace psamd {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
// A 16-byte piece in registers. A plain vector: HIP's uint4 is a struct, and copies of it in
// arrays were compiled to copies through scratch memory.
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

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

// Values of keys no query of the tile can see get probability zero, but zero times what lies in
// a slot nobody of this request has written (the rest of its last page, a page a window gave
// back and somebody else took) is NaN if that is a NaN or an infinity: such values are set to
// zero in the tiles that touch those slots. `keep(e)` tells whether element e's key is visible.
template <typename Keep>
__device__ __forceinline__ bf16x8 zero_unless(bf16x8 v, Keep keep) {
#pragma unroll
  for (int e = 0; e < 8; ++e)
    if (!keep(e)) v[e] = static_cast<__bf16>(0.f);
  return v;
}

// ------------------------------------------------------------------ prefill

constexpr int kMinSplitKeys = 512;   // a workgroup's share of a tile's keys is not cut below this

// NS = D / 16. A workgroup owns 32 consecutive queries of one item and one query head; its
// 4 waves take the 32-key tiles in turn and merge by log-sum-exp through LDS. Splitting the
// keys (not the queries) over the waves keeps the longest dependent chain of tiles four
// times shorter, which is what bounds a causal prompt's last rows.
// Per wave the loop is unrolled by two with two register sets: the keys and values of the
// wave's next tile are loaded before the current one is computed. The block table is staged
// in LDS once (a page id fetched from global memory inside the loop would put a second,
// unhidden latency in front of every tile's loads). Only tiles that touch the diagonal (or a
// window's edge) pay for masking; the softmax uses exp2 with the scale folded into one
// multiply-add per score.
template <int NS>
__global__ __launch_bounds__(256) void attn_prefill_mfma_kernel(
    const bf16_t* __restrict__ qkv, int q_stride, bf16_t* __restrict__ out, const bf16_t* __restrict__ kv,
    const int32_t* __restrict__ pf_tiles, const int32_t* __restrict__ item_start,
    const int32_t* __restrict__ item_pos0, const int32_t* __restrict__ table_off,
    const int32_t* __restrict__ block_ids, int hq, int hkv, float scale, int window,
    float* __restrict__ part_o, float* __restrict__ part_ml) {
  constexpr int D = 16 * NS;
  constexpr int DT = (D + 31) / 32;
  constexpr int DTC = DT < 2 ? DT : 2;      // d-tiles merged per pass (bounds the LDS buffer)
  __shared__ float sm_m[4][32], sm_l[4][32];
  __shared__ float sm_o[3 * DTC * 16 * 64];
  extern __shared__ int32_t table[];
  // Late tiles of a prompt see the most keys: start them first. Workgroups are handed out in
  // the order x + gridDim.x * y, round robin over the dies: x runs over the kv heads first and
  // then over the query heads of each, so that with a multiple of 8 kv heads all workgroups of
  // a kv head run on one die and share its keys and values in that die's L2.
  const int tile = gridDim.y - 1 - blockIdx.y;
  const int h = (blockIdx.x % hkv) * (hq / hkv) + blockIdx.x / hkv;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int item = pf_tiles[2 * tile];
  const int q_off = pf_tiles[2 * tile + 1];
  const int t0 = item_start[item];
  const int n = item_start[item + 1] - t0;
  const int pos0 = item_pos0[item];
  const int kvh = h / (hq / hkv);
  const int col = lane & 31, hi = lane >> 5;

  const int qi = min(q_off + col, n - 1);          // lanes past the end repeat the last query
  const bool q_valid = q_off + col < n;
  const int q_pos = pos0 + qi;
  const int first_pos = pos0 + q_off;
  const int last_pos = pos0 + min(q_off + 31, n - 1);
  const int max_key = pos0 + n - 1;
  const int k_lo_q = window > 0 ? max(0, q_pos - window + 1) : 0;
  const int k_begin_vis = window > 0 ? max(0, first_pos - window + 1) : 0;   // the first key any query of the tile sees
  const int k_begin = k_begin_vis & ~31;
  const float c = scale * 1.44269504088896340736f;  // scores are exponentiated in base 2
  // With gridDim.z > 1 the tile's keys are dealt out to that many workgroups in runs of whole
  // rounds of the four waves, at least kMinSplitKeys each, for the merge kernel to put together
  // (see the grouped kernel below); a tile with too few keys leaves the last runs empty.
  const int nsplit = gridDim.z;
  int k_first = k_begin, k_last = last_pos;
  int64_t part_slot = 0;
  if (nsplit > 1) {
    const int rounds = (last_pos - k_begin) / 128 + 1;
    const int per = max((rounds + nsplit - 1) / nsplit, kMinSplitKeys / 128);
    k_first = k_begin + static_cast<int>(blockIdx.z) * per * 128;
    k_last = min(last_pos, k_first + per * 128 - 1);
    part_slot = (static_cast<int64_t>(tile * 32 + col) * hq + h) * nsplit + blockIdx.z;
    if (k_first > last_pos) {
      if (wave == 0 && q_valid && hi == 0) {
        part_ml[2 * part_slot] = -INFINITY;
        part_ml[2 * part_slot + 1] = 0.f;
      }
      return;
    }
  }
  {
    const int32_t* gtable = block_ids + table_off[item];
    for (int i = threadIdx.x; i <= (last_pos >> 4); i += blockDim.x) table[i] = gtable[i];
  }
  __syncthreads();

  bf16x8 qf[NS];
  {
    const bf16_t* qp = qkv + static_cast<int64_t>(t0 + qi) * q_stride + h * D + 8 * hi;
#pragma unroll
    for (int s = 0; s < NS; ++s) qf[s] = ld8(qp + 16 * s);
  }

  f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[dt][v] = 0.f;
  float m = -INFINITY, l = 0.f;       // m in base-2 units (score * c)

  const int64_t page_elems = 2LL * hkv * kPage * D;
  const int64_t khead = static_cast<int64_t>(kvh) * kPage * D;
  const int64_t vhead = static_cast<int64_t>(hkv) * kPage * D + static_cast<int64_t>(kvh) * D * kPage;

  struct Tile {
    bf16x8 k[NS];        // A operand of S^T = K.Q^T: key row (k0 + col), 8 dims per 16-wide step
    bf16x8 v[2][DT];     // A operand of O^T += V^T.P^T: page c of the tile, V^T row d
  };
  auto load_tile = [&](Tile& t, int k0) {
    const int key_a = min(k0 + col, last_pos);
    const bf16_t* kp = kv + static_cast<int64_t>(table[key_a >> 4]) * page_elems + khead + (key_a & 15) * D + 8 * hi;
#pragma unroll
    for (int i = 0; i < NS; ++i) t.k[i] = ld8(kp + 16 * i);
#pragma unroll
    for (int cpage = 0; cpage < 2; ++cpage) {
      const int key_p = min(k0 + 16 * cpage, last_pos);
      const bf16_t* vp = kv + static_cast<int64_t>(table[key_p >> 4]) * page_elems + vhead + 4 * hi;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const bf16_t* vr = vp + min(32 * dt + col, D - 1) * kPage;
        t.v[cpage][dt] = join(ld4(vr), ld4(vr + 8));
      }
    }
    if (k0 + 31 > max_key || k0 < k_begin_vis) {
#pragma unroll
      for (int cpage = 0; cpage < 2; ++cpage)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
          t.v[cpage][dt] = zero_unless(t.v[cpage][dt], [&](int e) {
            const int key = k0 + 16 * cpage + 8 * (e >> 2) + 4 * hi + (e & 3);
            return key <= max_key && key >= k_begin_vis;
          });
    }
  };
  auto compute = [&](const Tile& t, int k0) {
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    f32x16 s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(t.k[0], qf[0], zero, 0, 0, 0);
#pragma unroll
    for (int i = 1; i < NS; ++i) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(t.k[i], qf[i], s, 0, 0, 0);
    // A tile whose last key is not after the first query, with no window, needs no mask.
    if (window > 0 || k0 + 31 > first_pos) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int key = k0 + 8 * (v >> 2) + 4 * hi + (v & 3);
        s[v] = (key <= q_pos && key >= k_lo_q) ? s[v] : -INFINITY;
      }
    }
    float mx = s[0];
#pragma unroll
    for (int v = 1; v < 16; ++v) mx = fmaxf(mx, s[v]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave)) * c;
    // The running maximum is only raised (and the accumulators rescaled) when some query's
    // scores outgrow it by more than 2^8: probabilities stay below 256, nothing overflows,
    // the final division by the sum is exact either way, and most tiles skip the rescale of
    // the whole accumulator.
    if (__any(mx > m + 8.f)) {
      const float m_new = fmaxf(m, mx);
      const float alpha = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m - m_new);
      l *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[dt][v] *= alpha;
      m = m_new;
    }
    const float m_use = m == -INFINITY ? 0.f : m;
    float rowsum = 0.f;
    bf16x8 pb[2];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const float p = __builtin_amdgcn_exp2f(fmaf(s[v], c, -m_use));
      rowsum += p;
      pb[v >> 3][v & 7] = static_cast<__bf16>(p);
    }
    l += rowsum + __shfl_xor(rowsum, 32, kWave);
#pragma unroll
    for (int cpage = 0; cpage < 2; ++cpage)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(t.v[cpage][dt], pb[cpage], o[dt], 0, 0, 0);
  };

  {
    Tile ta, tb;
    int k0 = k_first + 32 * wave;
    if (k0 <= k_last) {
      load_tile(ta, k0);
      while (true) {
        // The next tile is loaded whether or not it exists (addresses are clamped to the last
        // key): with no branch around the loads, the wait in front of the matrix instructions
        // counts exactly the loads of the current tile and leaves the next tile's in flight.
        load_tile(tb, k0 + 128);
        compute(ta, k0);
        k0 += 128;
        if (k0 > k_last) break;
        load_tile(ta, k0 + 128);
        compute(tb, k0);
        k0 += 128;
        if (k0 > k_last) break;
      }
    }
  }

  // ---- merge the 4 waves' partial results for the 32 queries
  if (hi == 0) {
    sm_m[wave][col] = m;
    sm_l[wave][col] = l;
  }
  __syncthreads();
  float mm = sm_m[0][col];
#pragma unroll
  for (int w = 1; w < 4; ++w) mm = fmaxf(mm, sm_m[w][col]);
  float ll = 0.f, mine = 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const float mw = sm_m[w][col];
    const float f = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - mm);
    ll += f * sm_l[w][col];
    if (w == wave) mine = f;
  }
  // One run of several: the sum, the maximum and the output as it is go to the merge kernel.
  const float inv = nsplit > 1 ? 1.f : 1.f / ll;
  if (nsplit > 1 && wave == 0 && q_valid && hi == 0) {
    part_ml[2 * part_slot] = mm;
    part_ml[2 * part_slot + 1] = ll;
  }
  bf16_t* op = out + static_cast<int64_t>(t0 + qi) * (static_cast<int64_t>(hq) * D) + h * D;
#pragma unroll
  for (int d0 = 0; d0 < DT; d0 += DTC) {
    if (wave > 0) {
#pragma unroll
      for (int dt = 0; dt < DTC; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          if (d0 + dt < DT) sm_o[(((wave - 1) * DTC + dt) * 16 + v) * 64 + lane] = o[d0 + dt][v] * mine;
    }
    __syncthreads();
    if (wave == 0 && q_valid) {
#pragma unroll
      for (int dt = 0; dt < DTC; ++dt) {
        if (d0 + dt >= DT) continue;
        float r[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          r[v] = o[d0 + dt][v] * mine;
#pragma unroll
          for (int w = 0; w < 3; ++w) r[v] += sm_o[((w * DTC + dt) * 16 + v) * 64 + lane];
        }
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) {
          const int d = 32 * (d0 + dt) + 8 * v4 + 4 * hi;
          if (d < D && nsplit > 1) {
            *reinterpret_cast<float4*>(part_o + part_slot * D + d) =
                float4{r[4 * v4 + 0], r[4 * v4 + 1], r[4 * v4 + 2], r[4 * v4 + 3]};
          } else if (d < D) {
            ushort4 pk;
            pk.x = float_to_bf16(r[4 * v4 + 0] * inv);
            pk.y = float_to_bf16(r[4 * v4 + 1] * inv);
            pk.z = float_to_bf16(r[4 * v4 + 2] * inv);
            pk.w = float_to_bf16(r[4 * v4 + 3] * inv);
            *reinterpret_cast<ushort4*>(op + d) = pk;
          }
        }
      }
    }
    if (d0 + DTC < DT) __syncthreads();
  }
}

// ------------------------------------------------------------------ prefill, query heads of a kv head together

// The same 32 queries for up to 4 query heads that share a kv head: one head per wave, all
// keys, no merge. The 32-key tile of K and of V^T is brought into LDS ONCE per workgroup
// (16-byte loads, whole contiguous pages) and read from there by the 4 waves: the texture
// path, which bounded the kernel above (a wave's operand loads there touch 32 rows of 32
// bytes each, and every head loads the same keys again), carries a quarter of the bytes in
// full lines. Two LDS stages: the next tile's global loads are in flight while the current
// tile is multiplied, one barrier per tile.
// LDS rows are padded (keys by 8 elements, V^T rows by 4) so that a wave's operand reads
// spread over all banks.
// Up to head size 64 the kernel is held to 128 registers (four waves per SIMD, the second
// argument of the launch bounds): at 131 only one workgroup of eight waves fitted a compute unit.
// With two, a prompt of 8,192 tokens, whose 256 tiles are more workgroups than compute units,
// runs 5% faster (8 layers of the 1B shape: 10.6 -> 10.0 ms).
// The pieces on their way from global memory to LDS are held as plain 4-word vectors: as
// arrays of HIP's uint4 (a struct) the compiler kept them in scratch memory whenever a thread
// has two or more pieces (head sizes from 96 on), waiting for each load right after issuing
// it; without that a 2,048-token prompt at head size 128 went from 75 to 55 us a layer.
// Measured and not kept: the scores of the next iteration issued before the softmax of the
// current one (correct, no faster at head size 128, slower at 64 where it costs the second
// workgroup per compute unit its registers), and the stores to LDS issued behind the barrier.
template <int NS, int KT, int KP>
__global__ __launch_bounds__(256 * KP, NS <= 4 ? 4 : 2) void attn_prefill_grouped_kernel(
    const bf16_t* __restrict__ qkv, int q_stride, bf16_t* __restrict__ out, const bf16_t* __restrict__ kv,
    const int32_t* __restrict__ pf_tiles, const int32_t* __restrict__ item_start,
    const int32_t* __restrict__ item_pos0, const int32_t* __restrict__ table_off,
    const int32_t* __restrict__ block_ids, int n_tiles, int hq, int hkv, int table_pages, float scale,
    int window, float* __restrict__ part_o, float* __restrict__ part_ml, int pair_tiles, int tiles_per_wg,
    const int32_t* __restrict__ pf_blocks, int n_blocks) {
  constexpr int D = 16 * NS;
  constexpr int DT = (D + 31) / 32;
  constexpr int KS = D + 8;                      // elements per key row in LDS
  constexpr int VS = kPage + 4;                  // elements per V^T row of one page in LDS
  constexpr int THREADS = 256 * KP;
  constexpr int KEYS = 32 * KT * KP;             // keys per iteration
  constexpr int CHUNKS = 4 * D * KT * KP;        // 16-byte pieces of an iteration's keys (and of its values)
  constexpr int CPT = (CHUNKS + THREADS - 1) / THREADS;   // pieces per thread
  constexpr int K_STAGE = KEYS * KS, V_STAGE = (KEYS / kPage) * D * VS;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  bf16_t* k_lds = reinterpret_cast<bf16_t*>(smem_raw);
  bf16_t* v_lds = k_lds + 2 * K_STAGE;
  int32_t* table = reinterpret_cast<int32_t*>(v_lds + 2 * V_STAGE);

  // A workgroup's four head slots (wave & 3) are four query heads of the kv head on one tile of
  // queries, or, with fewer query heads per kv head, two heads on two consecutive tiles or one
  // head on four (tiles_per_wg = 1, 2, 4): the keys and values a workgroup stages are then still
  // used by four waves. Its tiles are those of one item: pf_blocks lists the first tile of every
  // run of up to four consecutive tiles of an item, and gridDim.y is the number of those runs
  // times the workgroups that share one (two with two tiles each).
  const int group = hq / hkv;
  const int heads_per_wg = 4 / tiles_per_wg;
  const int wg_per_kv = (group + heads_per_wg - 1) / heads_per_wg;
  // Grid: x = (kv head, block of 4 query heads), y = tile, the late tiles (which see the most
  // keys) first. Workgroups are handed out in the order x + gridDim.x * y and go round robin over
  // the dies: the heaviest tiles of every head start first, so no head's long tiles are left
  // running alone at the end, and with a multiple of 8 workgroups in x a kv head's tiles all run
  // on one die, whose L2 then holds that head's keys and values for all of them (a 2,048-token
  // prompt at head size 64 fetched 20 MB from memory with the tile in x and 7 MB this way).
  const int kvh = blockIdx.x / wg_per_kv;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int part = wave >> 2;                           // which of the iteration's KP runs of keys
  const int slot = wave & 3;
  const int head_in_group = (blockIdx.x - kvh * wg_per_kv) * heads_per_wg + slot % heads_per_wg;
  const int tile_in_wg = slot / heads_per_wg;
  bool head_valid = head_in_group < group;             // a spare wave repeats the last head and writes nothing
  const int h = kvh * group + min(head_in_group, group - 1);
  // pair_tiles (the whole grid runs at once, two workgroups to a compute unit): the second half
  // of the workgroups, which join the first half's on their compute units, take the early tiles in
  // ascending order, so that the longest tile shares its compute unit with the shortest and every
  // compute unit has about the same number of keys to go through.
  const int by = static_cast<int>(blockIdx.y), first_half = (n_tiles + 1) >> 1;
  int wg_tile = (pair_tiles && by >= first_half) ? by - first_half : n_tiles - 1 - by;
  int wg_q_off_more = 0;
  if (tiles_per_wg > 1) {
    const int sub = 4 / tiles_per_wg;                  // workgroups per run of four tiles
    const int at = n_blocks * sub - 1 - by;            // late tiles first
    wg_tile = pf_blocks[at / sub] + tiles_per_wg * (at % sub);
    wg_q_off_more = 32 * tiles_per_wg * (at % sub);
  }
  const int item = pf_tiles[2 * (wg_tile - (wg_q_off_more >> 5))];
  const int wg_q_off = pf_tiles[2 * (wg_tile - (wg_q_off_more >> 5)) + 1] + wg_q_off_more;
  const int t0 = item_start[item];
  const int n = item_start[item + 1] - t0;
  if (wg_q_off >= n) return;                           // the run ends before this workgroup's tiles
  const int pos0 = item_pos0[item];
  const int col = lane & 31, hi = lane >> 5;

  // This wave's tile: a block's tiles past the end of the item do not exist, the wave then
  // repeats the block's first tile and writes nothing.
  int tile = wg_tile, q_off = wg_q_off;
  if (tile_in_wg > 0) {
    if (wg_q_off + 32 * tile_in_wg < n) {
      tile = wg_tile + tile_in_wg;
      q_off = wg_q_off + 32 * tile_in_wg;
    } else {
      head_valid = false;
    }
  }
  const int qi = min(q_off + col, n - 1);          // lanes past the end repeat the last query
  const bool q_valid = q_off + col < n;
  const int q_pos = pos0 + qi;
  const int first_pos = pos0 + q_off;                          // of this wave's tile
  const int last_pos = pos0 + min(q_off + 31, n - 1);
  const int wg_last_pos = pos0 + min(wg_q_off + 32 * tiles_per_wg - 1, n - 1);   // of the block
  const int k_lo_q = window > 0 ? max(0, q_pos - window + 1) : 0;
  const int max_key = pos0 + n - 1;
  const int k_begin_vis = window > 0 ? max(0, pos0 + wg_q_off - window + 1) : 0;   // the first key any query of the block sees
  const int k_begin = k_begin_vis & ~(KEYS - 1);
  const float c = scale * 1.44269504088896340736f;  // scores are exponentiated in base 2
  // With gridDim.z > 1 the tile's keys are dealt out to that many workgroups in runs of whole
  // pairs of iterations, at least kMinSplitKeys each; every workgroup leaves its sum, its
  // maximum and its unnormalized output in part_ml / part_o for the merge kernel. A tile with
  // too few keys for all of them leaves the last ones nothing: they write an empty sum.
  const int nsplit = gridDim.z;
  int k_first = k_begin, k_last = wg_last_pos;
  int64_t part_slot = 0;
  if (nsplit > 1) {
    constexpr int PAIR = 2 * KEYS;
    const int pairs = (wg_last_pos - k_begin) / PAIR + 1;
    const int per = max((pairs + nsplit - 1) / nsplit, kMinSplitKeys / PAIR);
    k_first = k_begin + static_cast<int>(blockIdx.z) * per * PAIR;
    k_last = min(wg_last_pos, k_first + per * PAIR - 1);
    part_slot = (static_cast<int64_t>(tile * 32 + col) * hq + h) * nsplit + blockIdx.z;
    if (k_first > wg_last_pos) {
      if (part == 0 && head_valid && q_valid && hi == 0) {
        part_ml[2 * part_slot] = -INFINITY;
        part_ml[2 * part_slot + 1] = 0.f;
      }
      return;
    }
  }
  {
    const int32_t* gtable = block_ids + table_off[item];
    for (int i = threadIdx.x; i <= (wg_last_pos >> 4); i += blockDim.x) table[i] = gtable[i];
  }
  __syncthreads();

  bf16x8 qf[NS];
  {
    const bf16_t* qp = qkv + static_cast<int64_t>(t0 + qi) * q_stride + h * D + 8 * hi;
#pragma unroll
    for (int s = 0; s < NS; ++s) qf[s] = ld8(qp + 16 * s);
  }
  f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[dt][v] = 0.f;
  float m = -INFINITY, l = 0.f;       // m in base-2 units (score * c)

  const int64_t page_elems = 2LL * hkv * kPage * D;
  const int64_t khead = static_cast<int64_t>(kvh) * kPage * D;
  const int64_t vhead = static_cast<int64_t>(hkv) * kPage * D + static_cast<int64_t>(kvh) * D * kPage;

  // Piece p of a tile lies in page p / (2 D) at element 8 * (p % (2 D)) of the head's keys
  // (and likewise of its values): both halves of a page are contiguous per head.
  struct Pieces {
    u32x4 k[CPT], v[CPT];
  };
  auto load_global = [&](Pieces& r, int k0) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int p = threadIdx.x + THREADS * i;
      if (CHUNKS % THREADS == 0 || p < CHUNKS) {
        const int page = p / (2 * D), rem = p - page * 2 * D;
        const int64_t base = static_cast<int64_t>(table[min(k0 + 16 * page, wg_last_pos) >> 4]) * page_elems;
        const bf16_t* src = kv + base + 8 * rem;
        r.k[i] = *reinterpret_cast<const u32x4*>(src + khead);
        r.v[i] = *reinterpret_cast<const u32x4*>(src + vhead);
      }
    }
  };
  auto store_lds = [&](const Pieces& r, int stage, int k0) {
    bf16_t* kd = k_lds + stage * K_STAGE;
    bf16_t* vd = v_lds + stage * V_STAGE;
    const bool edge = k0 + KEYS - 1 > max_key || k0 < k_begin_vis;   // slots nobody of this request wrote
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int p = threadIdx.x + THREADS * i;
      if (CHUNKS % THREADS == 0 || p < CHUNKS) {
        const int key = p / (D / 8), part = p - key * (D / 8);
        *reinterpret_cast<u32x4*>(kd + key * KS + 8 * part) = r.k[i];
        const int row = p >> 1, half = p & 1;                     // row = page * D + d
        u32x4 v = r.v[i];
        if (edge) {
          const int key0 = k0 + 16 * (row / D) + 8 * half;        // the piece holds the values of keys key0 .. key0 + 7
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (key0 + e > max_key || key0 + e < k_begin_vis) v[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
        }
        uint2* dst = reinterpret_cast<uint2*>(vd + row * VS + 8 * half);
        dst[0] = uint2{v[0], v[1]};
        dst[1] = uint2{v[2], v[3]};
      }
    }
  };
  auto compute = [&](int stage, int k_iter) {
    const int k0 = k_iter + 32 * KT * part;          // this wave's keys of the iteration
    if (k0 > last_pos) return;                       // all after the last query (the loads were clamped)
    const bf16_t* kd = k_lds + stage * K_STAGE + (32 * KT * part + col) * KS + 8 * hi;
    const bf16_t* vd = v_lds + stage * V_STAGE + 2 * KT * part * D * VS + 4 * hi;
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // The KT score tiles are independent chains of matrix instructions: one runs while the
    // other's results are being exponentiated.
    f32x16 s[KT];
#pragma unroll
    for (int t = 0; t < KT; ++t) {
      s[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ld8(kd + t * 32 * KS), qf[0], zero, 0, 0, 0);
#pragma unroll
      for (int i = 1; i < NS; ++i)
        s[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ld8(kd + t * 32 * KS + 16 * i), qf[i], s[t], 0, 0, 0);
    }
    // Keys that are not after the first query, with no window, need no mask.
    if (window > 0 || k0 + 32 * KT - 1 > first_pos) {
#pragma unroll
      for (int t = 0; t < KT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int key = k0 + 32 * t + 8 * (v >> 2) + 4 * hi + (v & 3);
          s[t][v] = (key <= q_pos && key >= k_lo_q) ? s[t][v] : -INFINITY;
        }
    }
    float mx = s[0][0];
#pragma unroll
    for (int t = 0; t < KT; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[t][v]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave)) * c;
    // The running maximum is only raised (and the accumulators rescaled) when some query's
    // scores outgrow it by more than 2^8 (see the kernel above).
    if (__any(mx > m + 8.f)) {
      const float m_new = fmaxf(m, mx);
      const float alpha = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m - m_new);
      l *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[dt][v] *= alpha;
      m = m_new;
    }
    const float m_use = m == -INFINITY ? 0.f : m;
    float rowsum = 0.f;
#pragma unroll
    for (int t = 0; t < KT; ++t) {
      bf16x8 pb[2];
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s[t][v], c, -m_use));
        rowsum += p;
        pb[v >> 3][v & 7] = static_cast<__bf16>(p);
      }
#pragma unroll
      for (int cpage = 0; cpage < 2; ++cpage)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const bf16_t* vr = vd + ((2 * t + cpage) * D + min(32 * dt + col, D - 1)) * VS;
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(join(ld4(vr), ld4(vr + 8)), pb[cpage], o[dt], 0, 0, 0);
        }
    }
    l += rowsum + __shfl_xor(rowsum, 32, kWave);
  };

  {
    // Global loads run two iterations ahead in two register sets, issued whether or not the
    // keys exist (page lookups are clamped to the last key): memory that missed the L2 takes
    // longer than one iteration, and with no branch around the loads the wait in front of a
    // store to LDS counts exactly the older set and leaves the newer one in flight.
    Pieces ra, rb;
    int k0 = k_first, stage = 0;
    load_global(ra, k0);
    load_global(rb, k0 + KEYS);
    auto iteration = [&](Pieces& r) {
      store_lds(r, stage, k0);
      load_global(r, k0 + 2 * KEYS);
      // Every wave is past the iteration that last used this stage: it had to finish it to
      // reach the previous barrier.
      __syncthreads();
      compute(stage, k0);
      stage ^= 1;
      k0 += KEYS;
    };
    // Always two iterations per turn, the second perhaps on keys past the last query (its
    // loads are clamped, its stores go to a free stage and compute() skips it): a way out of
    // the loop between the two would, as the compiler lays the loop out, also be a way back to
    // its head, and the wait in front of the first store would then be for all loads but one
    // instead of all but three, which waits for the set that has just been asked for.
    do {
      iteration(ra);
      iteration(rb);
    } while (k0 <= k_last);
  }

  if (KP > 1) {
    // Merge the KP runs of keys by log-sum-exp; the K/V stages are free now.
    constexpr int O_FLOATS = DT * 16 * 64;
    float* mg = reinterpret_cast<float*>(smem_raw);
    __syncthreads();
    if (part > 0) {
      float* dst = mg + ((part - 1) * 4 + (wave & 3)) * (O_FLOATS + 64);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) dst[(dt * 16 + v) * 64 + lane] = o[dt][v];
      if (hi == 0) {
        dst[O_FLOATS + col] = m;
        dst[O_FLOATS + 32 + col] = l;
      }
    }
    __syncthreads();
    if (part == 0) {
    float mm = m;
#pragma unroll
    for (int p = 1; p < KP; ++p) mm = fmaxf(mm, mg[((p - 1) * 4 + wave) * (O_FLOATS + 64) + O_FLOATS + col]);
    const float f0 = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - mm);
    l *= f0;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[dt][v] *= f0;
#pragma unroll
    for (int p = 1; p < KP; ++p) {
      const float* src = mg + ((p - 1) * 4 + wave) * (O_FLOATS + 64);
      const float mp = src[O_FLOATS + col];
      const float f = mp == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mp - mm);
      l += f * src[O_FLOATS + 32 + col];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[dt][v] += f * src[(dt * 16 + v) * 64 + lane];
    }
    m = mm;
    }
  }
  if (part != 0 || !head_valid || !q_valid) return;
  if (nsplit > 1) {
    // m is in units of the base-2 exponent; a query with no key in this run has m = -inf, l = 0.
    if (hi == 0) {
      part_ml[2 * part_slot] = m;
      part_ml[2 * part_slot + 1] = l;
    }
    float* po = part_o + part_slot * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int v4 = 0; v4 < 4; ++v4) {
        const int d = 32 * dt + 8 * v4 + 4 * hi;
        if (d < D)
          *reinterpret_cast<float4*>(po + d) =
              float4{o[dt][4 * v4 + 0], o[dt][4 * v4 + 1], o[dt][4 * v4 + 2], o[dt][4 * v4 + 3]};
      }
    return;
  }
  const float inv = 1.f / l;
  bf16_t* op = out + static_cast<int64_t>(t0 + qi) * (static_cast<int64_t>(hq) * D) + h * D;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const int d = 32 * dt + 8 * v4 + 4 * hi;
      if (d < D) {
        ushort4 pk;
        pk.x = float_to_bf16(o[dt][4 * v4 + 0] * inv);
        pk.y = float_to_bf16(o[dt][4 * v4 + 1] * inv);
        pk.z = float_to_bf16(o[dt][4 * v4 + 2] * inv);
        pk.w = float_to_bf16(o[dt][4 * v4 + 3] * inv);
        *reinterpret_cast<ushort4*>(op + d) = pk;
      }
    }
}

// Puts together the runs that the two kernels above cut a tile's keys into: for each (query,
// head) the unnormalized outputs are weighed by 2^(m_s - max m), added in the order of the runs,
// divided by the weighed sum and written as bfloat16. A thread owns four dimensions of one
// (query, head) pair, D / 4 threads a pair, the pairs of a workgroup next to each other in
// memory; the statistics of all runs are asked for at once, then all partial outputs. A run that
// held no key this query sees (m = -inf) counts as nothing whatever its output holds: it was
// never written.
constexpr int kMaxPrefillSplit = 16;

__global__ __launch_bounds__(256) void attn_prefill_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, bf16_t* __restrict__ out,
    const int32_t* __restrict__ pf_tiles, const int32_t* __restrict__ item_start, int64_t pairs, int hq, int d,
    int nsplit) {
  const int per_pair = d >> 2;                         // threads per pair
  const int pairs_per_block = 256 / per_pair;
  const int sub = threadIdx.x / per_pair, chunk = threadIdx.x - sub * per_pair;
  const int64_t pair = static_cast<int64_t>(blockIdx.x) * pairs_per_block + sub;
  if (sub >= pairs_per_block || pair >= pairs) return;
  const int row = static_cast<int>(pair / hq), h = static_cast<int>(pair - static_cast<int64_t>(row) * hq);
  const int tile = row >> 5, col = row & 31;
  const int item = pf_tiles[2 * tile];
  const int q = pf_tiles[2 * tile + 1] + col;
  const int t0 = item_start[item];
  if (q >= item_start[item + 1] - t0) return;
  const float2* ml = reinterpret_cast<const float2*>(part_ml) + pair * nsplit;
  const float4* po = reinterpret_cast<const float4*>(part_o + pair * nsplit * d) + chunk;
  float2 st[kMaxPrefillSplit];
#pragma unroll
  for (int s = 0; s < kMaxPrefillSplit; ++s) st[s] = s < nsplit ? ml[s] : float2{-INFINITY, 0.f};
  float4 part[kMaxPrefillSplit];
#pragma unroll
  for (int s = 0; s < kMaxPrefillSplit; ++s)
    if (s < nsplit) part[s] = po[s * per_pair];
  float mm = -INFINITY;
#pragma unroll
  for (int s = 0; s < kMaxPrefillSplit; ++s) mm = fmaxf(mm, st[s].x);
  float4 acc = {0.f, 0.f, 0.f, 0.f};
  float ll = 0.f;
#pragma unroll
  for (int s = 0; s < kMaxPrefillSplit; ++s) {
    if (s < nsplit && st[s].x != -INFINITY) {
      const float w = __builtin_amdgcn_exp2f(st[s].x - mm);
      ll += w * st[s].y;
      acc.x += w * part[s].x;
      acc.y += w * part[s].y;
      acc.z += w * part[s].z;
      acc.w += w * part[s].w;
    }
  }
  const float inv = 1.f / ll;
  ushort4 pk;
  pk.x = float_to_bf16(acc.x * inv);
  pk.y = float_to_bf16(acc.y * inv);
  pk.z = float_to_bf16(acc.z * inv);
  pk.w = float_to_bf16(acc.w * inv);
  *reinterpret_cast<ushort4*>(out + static_cast<int64_t>(t0 + q) * (static_cast<int64_t>(hq) * d) +
                              static_cast<int64_t>(h) * d + 4 * chunk) = pk;
}

// ------------------------------------------------------------------ decode (split keys)

// NS = D / 16, CT = ceil(group / 16) column tiles of query heads.
// part_o[dec][head][split][D], part_ml[dec][head][split][2] = (max, sum).
template <int NS, int CT>
__global__ __launch_bounds__(256) void attn_decode_mfma_kernel(
    const bf16_t* __restrict__ qkv, int q_stride, const bf16_t* __restrict__ kv, bf16_t* __restrict__ out,
    float* __restrict__ part_o, float* __restrict__ part_ml, const int32_t* __restrict__ dec_items,
    const int32_t* __restrict__ item_start,
    const int32_t* __restrict__ item_end, const int32_t* __restrict__ table_off,
    const int32_t* __restrict__ block_ids, int hq, int hkv, int nsplit, float scale, int window, int min_tiles,
    int n_dec) {
  constexpr int D = 16 * NS;
  constexpr int KS = (D + 31) / 32;
  extern __shared__ float smem[];
  // Workgroups are handed out in the order of blockIdx.x, round robin over the eight dies. The
  // (request, split) pairs are laid out eight at a time, one per die, with the kv heads of a pair
  // 8 apart, so on the same die (a die's address translation then sees an eighth of the
  // requests' pages; with the heads of a pair on eight dies a batch of 64 was 4% slower). The
  // pairs follow each other request by request, the splits of a request turned by its number:
  // the splits of one request go to different dies, and so do the first splits (the only ones
  // with keys where a request is short) of different requests. With the request as the fast
  // index of a three-dimensional grid and a multiple of eight requests, all workgroups of a
  // request ran on one die, and a request with a long context among short ones was read at an
  // eighth of the memory bandwidth (31 requests of 1,024 keys and one of 60,000 at head size
  // 128: 687 us whatever the number of splits). The grid is rounded up to whole groups of eight
  // pairs; the workgroups of the pairs that do not exist leave at once.
  // Grid: x = die slot + 8 * kv head, y = group of eight pairs.
  const int kvh = blockIdx.x >> 3;
  const int at = blockIdx.y * 8 + (blockIdx.x & 7);
  const int di = at / nsplit;
  if (di >= n_dec) return;
  const int turned = at - di * nsplit + nsplit - (di < nsplit ? di : di % nsplit);     // in [1, 2 nsplit)
  const int split = turned >= nsplit ? turned - nsplit : turned;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, g4 = lane >> 4;
  const int item = dec_items[di];
  const int64_t t = item_start[item];
  const int pos = item_end[item] - 1;
  const int group = hq / hkv;
  const int32_t* table = block_ids + table_off[item];
  const int k_lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int tile_lo = k_lo >> 5, tile_hi = pos >> 5;
  // ceil(ntiles / nsplit), but no fewer than min_tiles: a short request beside a long one is
  // not cut into as many runs as the long one needs, and leaves the last splits empty.
  const int tps = max((tile_hi - tile_lo + nsplit) / nsplit, min_tiles);
  const int my_lo = tile_lo + split * tps;
  const int my_hi = min(my_lo + tps, tile_hi + 1);
  if (my_lo >= my_hi) {
    // No keys left for this split (only with nsplit > 1): an empty sum and an output of zeros,
    // which the merge kernel multiplies by a weight of zero (what lay there before might be NaN).
    for (int idx = threadIdx.x; idx < group * D; idx += blockDim.x) {
      const int hh = idx / D, d = idx - hh * D;
      const int64_t slot = (static_cast<int64_t>(di) * hq + kvh * group + hh) * nsplit + split;
      part_o[slot * D + d] = 0.f;
      if (d == 0) {
        part_ml[slot * 2 + 0] = -INFINITY;
        part_ml[slot * 2 + 1] = 0.f;
      }
    }
    return;
  }

  const int64_t page_elems = 2LL * hkv * kPage * D;
  const int64_t khead = static_cast<int64_t>(kvh) * kPage * D;
  const int64_t vhead = static_cast<int64_t>(hkv) * kPage * D + static_cast<int64_t>(kvh) * D * kPage;

  bf16x8 qf[CT][KS];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int hh = ct * 16 + r;
    const bf16_t* qp = qkv + t * q_stride + static_cast<int64_t>(kvh * group + min(hh, group - 1)) * D + 8 * g4;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bool in = hh < group && 32 * ks + 8 * g4 < D;
      qf[ct][ks] = in ? ld8(qp + 32 * ks) : zeros8();
    }
  }

  f32x4 o[CT][NS];
  float m[CT], l[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    m[ct] = -INFINITY;
    l[ct] = 0.f;
#pragma unroll
    for (int ds = 0; ds < NS; ++ds) o[ct][ds] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  for (int tile = my_lo + wave; tile < my_hi; tile += 4) {
    // The tile is the same for all lanes of a wave: said so, its page ids come through the scalar
    // cache instead of as vector loads that every lane repeats (32 requests x 8 kv heads, 2,048
    // keys: 25.9 -> 22.0 us). Asking for the next tile's keys and values before multiplying the
    // current one, on top of that, was measured and lost (22.0 -> 23.4 us; 64 requests 44 -> 53).
    const int k0 = __builtin_amdgcn_readfirstlane(tile) << 5;
    // Each 16-key half of the tile is exactly one page.
    const int64_t page0 = table[min(k0, pos) >> 4];
    const int64_t page1 = table[min(k0 + 16, pos) >> 4];
    const bf16_t* kp0 = kv + page0 * page_elems + khead + r * D + 8 * g4;
    const bf16_t* kp1 = kv + page1 * page_elems + khead + r * D + 8 * g4;
    bf16x8 ka0[KS], ka1[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bool in = 32 * ks + 8 * g4 < D;
      ka0[ks] = in ? ld8(kp0 + 32 * ks) : zeros8();
      ka1[ks] = in ? ld8(kp1 + 32 * ks) : zeros8();
    }
    const bf16_t* vp0 = kv + page0 * page_elems + vhead + 4 * g4;
    const bf16_t* vp1 = kv + page1 * page_elems + vhead + 4 * g4;
    bf16x8 va[NS];
#pragma unroll
    for (int ds = 0; ds < NS; ++ds) {
      const int drow = 16 * ds + r;
      va[ds] = join(ld4(vp0 + drow * kPage), ld4(vp1 + drow * kPage));
    }
    if (k0 + 31 > pos || k0 < k_lo) {
#pragma unroll
      for (int ds = 0; ds < NS; ++ds)
        va[ds] = zero_unless(va[ds], [&](int e) {
          const int key = k0 + 16 * (e >> 2) + 4 * g4 + (e & 3);
          return key <= pos && key >= k_lo;
        });
    }
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka0[ks], qf[ct][ks], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka1[ks], qf[ct][ks], s1, 0, 0, 0);
      }
      float sv[8];
      float mx = -INFINITY;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int key0 = k0 + 4 * g4 + v, key1 = key0 + 16;
        sv[v] = (key0 <= pos && key0 >= k_lo) ? s0[v] * scale : -INFINITY;
        sv[v + 4] = (key1 <= pos && key1 >= k_lo) ? s1[v] * scale : -INFINITY;
        mx = fmaxf(mx, fmaxf(sv[v], sv[v + 4]));
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
      mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
      const float m_new = fmaxf(m[ct], mx);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = __expf(m[ct] - m_use);
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
      l[ct] = l[ct] * alpha + rowsum;
      m[ct] = m_new;
#pragma unroll
      for (int ds = 0; ds < NS; ++ds) {
        o[ct][ds] *= alpha;
        o[ct][ds] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[ds], pb, o[ct][ds], 0, 0, 0);
      }
    }
  }

  // ---- merge the 4 waves: smem = m[4][group], l[4][group], o[4][group][D]
  float* sm_m = smem;
  float* sm_l = smem + 4 * group;
  float* sm_o = smem + 8 * group;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int hh = ct * 16 + r;
    if (hh < group) {
      if (g4 == 0) {
        sm_m[wave * group + hh] = m[ct];
        sm_l[wave * group + hh] = l[ct];
      }
#pragma unroll
      for (int ds = 0; ds < NS; ++ds)
#pragma unroll
        for (int v = 0; v < 4; ++v)
          sm_o[(static_cast<int64_t>(wave) * group + hh) * D + 16 * ds + 4 * g4 + v] = o[ct][ds][v];
    }
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < group * D; idx += blockDim.x) {
    const int hh = idx / D, d = idx - hh * D;
    float mm = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) mm = fmaxf(mm, sm_m[w * group + hh]);
    float acc = 0.f, ll = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = sm_m[w * group + hh];
      const float wgt = mw == -INFINITY ? 0.f : __expf(mw - mm);
      acc += wgt * sm_o[(static_cast<int64_t>(w) * group + hh) * D + d];
      ll += wgt * sm_l[w * group + hh];
    }
    if (nsplit == 1) {   // nothing to merge with: this is the result
      out[t * (static_cast<int64_t>(hq) * D) + static_cast<int64_t>(kvh * group + hh) * D + d] = float_to_bf16(acc / ll);
      continue;
    }
    const int64_t slot = (static_cast<int64_t>(di) * hq + kvh * group + hh) * nsplit + split;
    part_o[slot * D + d] = acc;
    if (d == 0) {
      part_ml[slot * 2 + 0] = mm;
      part_ml[slot * 2 + 1] = ll;
    }
  }
}

// One block (64 threads) per (decode item, head): merges the splits and writes bfloat16.
// Lane s first loads the statistics of split s, so the weights of all splits come from one
// round of loads; then every lane sums its dimensions over the splits with loads that do
// not depend on each other.
__global__ __launch_bounds__(64) void attn_decode_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, bf16_t* __restrict__ out,
    const int32_t* __restrict__ dec_items, const int32_t* __restrict__ item_start, int hq, int d, int nsplit) {
  __shared__ float wgt_s[64];
  const int di = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int64_t t = item_start[dec_items[di]];
  const int64_t base = (static_cast<int64_t>(di) * hq + h) * nsplit;
  const bool has = lane < nsplit;                       // nsplit <= 64
  const float ms = has ? part_ml[(base + lane) * 2] : -INFINITY;
  const float ls = has ? part_ml[(base + lane) * 2 + 1] : 0.f;
  // The first splits' partial outputs are asked for together with the statistics, not after them.
  constexpr int kEarly = 8;
  float early[kEarly];
#pragma unroll
  for (int s = 0; s < kEarly; ++s) early[s] = (s < nsplit && lane < d) ? part_o[(base + s) * d + lane] : 0.f;
  const float mm = wave_max(ms);
  const float w = ms == -INFINITY ? 0.f : __expf(ms - mm);
  const float ll = wave_sum(w * ls);
  wgt_s[lane] = w / ll;
  __syncthreads();
  for (int i = lane; i < d; i += kWave) {
    float acc = 0.f;
    int s0 = 0;
    if (i == lane) {
#pragma unroll
      for (int s = 0; s < kEarly; ++s) acc += (s < nsplit ? wgt_s[s] : 0.f) * early[s];
      s0 = kEarly;
    }
#pragma unroll 8
    for (int s = s0; s < nsplit; ++s) acc += wgt_s[s] * part_o[(base + s) * d + i];
    out[t * (static_cast<int64_t>(hq) * d) + h * d + i] = float_to_bf16(acc);
  }
}

// Bytes of LDS the grouped kernel needs for head size D, kt 32-key tiles per wave and
// iteration, kp waves per head and a block table of table_pages entries.
static size_t grouped_smem(int D, int kt, int kp, int table_pages) {
  const size_t stages = sizeof(bf16_t) * 2 * kt * kp * (32 * static_cast<size_t>(D + 8) + 2 * static_cast<size_t>(D) * (kPage + 4)) +
                        sizeof(int32_t) * static_cast<size_t>(table_pages);
  const size_t merge = sizeof(float) * (kp - 1) * 4 * (static_cast<size_t>((D + 31) / 32) * 16 * 64 + 64);
  return std::max(stages, merge);
}

// More than 64 KB of dynamic LDS has to be asked for, kernel by kernel.
template <typename Kernel>
static bool lds_allowed(Kernel kernel, size_t bytes) {
  if (bytes <= 64 * 1024) return true;
  if (bytes > 160 * 1024) return false;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                             static_cast<int>(bytes)) == hipSuccess;
}

// Which kernel a step's portions go to, when two or more query heads share a kv head
// (measured on 256 compute units with 32 query heads on 8 kv heads; us per layer, per-head /
// grouped, at head size 64 and at head size 128):
//   256 on 1,792 cached     18 / 30      31 / 43       384 on 3,712 cached     48 / 53      94 / 78
//   512 from position 0     11 / 12      21 / 18       512 on 7,680 cached     91 / 101    180 / 148
//   768 on 2,304 cached     50 / 42     104 / 63       1,024 on 3,072 cached   84 / 56     176 / 88
//   2,048 from position 0   57 / 36     142 / 58       8,192 from 0             - / 355      - / 655
// The per-head kernel, whose grid is four times as large, fills the chip better while the grouped
// one has few workgroups: up to 128 of them at head sizes up to 64, up to 80 above (the grouped
// kernel's advantage, every key and value read once for four heads, grows with the head size).
// Two tiles per workgroup (the b-th from the end and the b-th from the start of a causal prompt,
// to even out the triangle) were measured against the order of workgroups described in the kernel
// and dropped: within 3% at best, 12% slower at 3,072 tokens, up to 15% slower on top of a cached
// prefix.
enum class PrefillForm { kPerHead, kGrouped };

// With one or two query heads per kv head a workgroup of the grouped kernel takes four or two
// consecutive tiles of queries, so that four waves still share the keys and values it stages.
static int prefill_tiles_per_wg(int group) { return group == 1 ? 4 : (group == 2 ? 2 : 1); }

// Workgroups of the grouped kernel for a step of n_tiles tiles (a run of tiles that ends early
// adds one per item: the estimate is for choosing a form, not for a grid).
static int64_t grouped_workgroups(int n_tiles, int hq, int hkv) {
  const int group = hq / hkv;
  const int tiles = prefill_tiles_per_wg(group), heads = 4 / tiles;
  return ceil_div(n_tiles, tiles) * hkv * ceil_div(group, heads);
}

// Few enough of them that the per-head kernel, with four times as many, does better.
static bool few_grouped_workgroups(int n_tiles, int hq, int hkv, int head_dim) {
  return grouped_workgroups(n_tiles, hq, hkv) <= (head_dim <= 64 ? 128 : 80);
}

static PrefillForm prefill_form(int n_tiles, int hq, int hkv, int head_dim) {
  return few_grouped_workgroups(n_tiles, hq, hkv, head_dim) ? PrefillForm::kPerHead : PrefillForm::kGrouped;
}

static int launch_prefill_merge(hipStream_t s, const float* part_o, const float* part_ml, void* out,
                                const int32_t* pf_tiles, const int32_t* item_start, int n_tiles, int hq, int head_dim,
                                int nsplit) {
  const int64_t pairs = 32LL * n_tiles * hq;
  const int pairs_per_block = 256 / (head_dim / 4);
  attn_prefill_merge_kernel<<<dim3(static_cast<unsigned>(ceil_div(pairs, pairs_per_block))), dim3(256), 0, s>>>(
      part_o, part_ml, static_cast<bf16_t*>(out), pf_tiles, item_start, pairs, hq, head_dim, nsplit);
  return check_launch("psamd_attention_prefill(merge)");
}

// Into how many runs the grouped kernel cuts a tile's keys (1: not at all). Few query tiles on
// many keys (a portion of a long prompt, a short tail behind a long context) are too few
// workgroups for 256 compute units: their keys are then dealt out to more of them, up to as many
// workgroups as run at once (two per compute unit up to head size 64, one above), each run no
// shorter than 512 keys, and a merge kernel puts the runs together. Measured with 32 query heads
// on 8 kv heads, us per layer at head size 64 / 128, no cut -> cut: 512 tokens on 7,680 cached
// 92 -> 60 / 148 -> 94; 512 on 60,000 625 -> 332 / 1,045 -> 590; 128 on 8,064 48 -> 27 / 92 -> 37;
// 20 on 16,000 88 -> 23 / 170 -> 32. Where the per-head kernel would run (few workgroups), fewer
// than four runs lose to it, and so do runs of under 1,024 keys once it has a workgroup per
// compute unit itself (256 on 1,792: 17 -> 20 with four); where the grouped kernel would run
// without a cut, two runs pay from 4,096 keys on (512 on 3,584 at head size 128: 78 -> 58) and,
// above 128 workgroups, from 8,192 on (1,024 on 3,072: 56 -> 60; on 15,000: 199 -> 183).
static int grouped_nsplit(int n_tiles, int max_kv_len, int hq, int hkv, int head_dim) {
  const int64_t workgroups = grouped_workgroups(n_tiles, hq, hkv);
  const int at_once = head_dim <= 64 ? 512 : 256;
  if (2 * workgroups > at_once) return 1;
  if (grouped_smem(head_dim, 1, 1, static_cast<int>(ceil_div(max_kv_len, kPage))) > 160 * 1024) return 1;
  // 65 to 128 workgroups on 2,048 to 4,095 keys: two runs (512 tokens on 2,560 cached at head size
  // 64 / 128: 43 -> 36 / 70 -> 54 us; on 1,536 cached 30 -> 28 / 44 -> 41).
  if (workgroups > 64 && workgroups <= 128 && max_kv_len >= 2048 && max_kv_len < 4096) return 2;
  const int nsplit = static_cast<int>(std::min<int64_t>({at_once / workgroups, max_kv_len / kMinSplitKeys, kMaxPrefillSplit}));
  const bool per_head_else = few_grouped_workgroups(n_tiles, hq, hkv, head_dim);
  if (per_head_else) {
    if (nsplit < 4 || (static_cast<int64_t>(n_tiles) * hq >= 256 && max_kv_len < 4096)) return 1;
  } else if (max_kv_len < (workgroups <= 128 ? 4096 : 8192)) {
    return 1;
  }
  return std::max(nsplit, 1);
}

// The same for the per-head kernel, a workgroup per (tile, query head), which takes the steps
// with one or two query heads per kv head that the grouped kernel (four or two tiles of queries
// per workgroup then) neither cuts nor has enough workgroups for: runs of 1,024 keys or more, up
// to one workgroup per compute unit (more lost again). 32 heads on 32 at head size 128: 64 tokens
// on 4,032 cached 51 -> 26 us, 20 on 16,000 172 -> 56; 16 heads on 8: 256 on 7,936 93 -> 57,
// 256 on 60,000 622 -> 323.
static int per_head_nsplit(int n_tiles, int max_kv_len, int hq) {
  const int64_t workgroups = static_cast<int64_t>(n_tiles) * hq;
  if (2 * workgroups > 256) return 1;
  return static_cast<int>(std::max<int64_t>(1, std::min<int64_t>({256 / workgroups, max_kv_len / 1024, 16})));
}

static int prefill_nsplit(int n_tiles, int max_kv_len, int hq, int hkv, int head_dim) {
  const int cut = grouped_nsplit(n_tiles, max_kv_len, hq, hkv, head_dim);
  if (hq / hkv > 2 || cut > 1 || !few_grouped_workgroups(n_tiles, hq, hkv, head_dim)) return cut;
  return per_head_nsplit(n_tiles, max_kv_len, hq);
}

template <int NS>
static int launch_prefill(hipStream_t s, const void* qkv, int q_stride, void* out, const void* kv,
                          const int32_t* pf_tiles, int n_tiles, const int32_t* pf_blocks, int n_blocks, int max_kv_len,
                          const int32_t* item_start, const int32_t* item_pos0,
                          const int32_t* table_off, const int32_t* block_ids, int hq, int hkv, float scale, int window,
                          float* part_o, float* part_ml, int nsplit) {
  const int group = hq / hkv;
  const int table_pages = static_cast<int>(ceil_div(max_kv_len, kPage));
  // One or two query heads per kv head: the per-head kernel without the list of runs of tiles, and
  // where the keys are cut by its rule and not by the grouped kernel's.
  const bool small_per_head =
      group <= 2 && (n_blocks == 0 || (nsplit > 1 && grouped_nsplit(n_tiles, max_kv_len, hq, hkv, 16 * NS) == 1));
  const PrefillForm form = nsplit > 1 || small_per_head ? (small_per_head ? PrefillForm::kPerHead : PrefillForm::kGrouped)
                                                        : prefill_form(n_tiles, hq, hkv, 16 * NS);
  // The heads of a kv head share its keys and values through LDS, two waves per head (each its
  // own run of keys) if the stages fit, else one.
  if (form != PrefillForm::kPerHead) {
    const int tiles_per_wg = prefill_tiles_per_wg(group), heads_per_wg = 4 / tiles_per_wg;
    const dim3 grid(hkv * ((group + heads_per_wg - 1) / heads_per_wg), tiles_per_wg == 1 ? n_tiles : n_blocks * heads_per_wg,
                    nsplit);
    // More than one workgroup per compute unit but no more than run at once (two of eight waves
    // up to head size 64): see pair_tiles in the kernel.
    const int64_t wgs = static_cast<int64_t>(grid.x) * grid.y;
    // (2,048 tokens at head size 64, 32 heads on 8: 37.6 -> 35.1 us; on 2,048 cached keys 80 -> 74.)
    const int pair = (NS <= 4 && nsplit == 1 && tiles_per_wg == 1 && wgs > 256 && wgs <= 512 && grid.x % 8 == 0) ? 1 : 0;
#define PSAMD_GROUPED(KP_)                                                                                         \
  {                                                                                                               \
    const size_t smem = grouped_smem(16 * NS, 1, KP_, table_pages);                                               \
    if (lds_allowed(attn_prefill_grouped_kernel<NS, 1, KP_>, smem)) {                                             \
      attn_prefill_grouped_kernel<NS, 1, KP_><<<grid, dim3(256 * KP_), smem, s>>>(                                \
          static_cast<const bf16_t*>(qkv), q_stride, static_cast<bf16_t*>(out), static_cast<const bf16_t*>(kv),   \
          pf_tiles, item_start, item_pos0, table_off, block_ids, n_tiles, hq, hkv, table_pages, scale, window,   \
          part_o, part_ml, pair, tiles_per_wg, pf_blocks, n_blocks);                                              \
      const int rc = check_launch("psamd_attention_prefill");                                                     \
      if (rc != 0 || nsplit == 1) return rc;                                                                      \
      return launch_prefill_merge(s, part_o, part_ml, out, pf_tiles, item_start, n_tiles, hq, 16 * NS, nsplit);   \
    }                                                                                                             \
  }
    // From head size 96 on, where a compute unit holds one workgroup of eight waves, four
    // workgroups per compute unit's worth of tiles run 5% faster as two workgroups of four waves
    // (one wave per head): two barriers' worth of waves that do not wait for each other
    // (head size 128: 4,096 tokens 181 -> 171 us, 8,192 tokens 657 -> 623 us; 2,048 tokens 56 -> 67).
    if (NS < 6 || wgs * grid.z < 1024) PSAMD_GROUPED(2)
    PSAMD_GROUPED(1)
#undef PSAMD_GROUPED
  }
  attn_prefill_mfma_kernel<NS><<<dim3(hq, n_tiles, nsplit), dim3(256), sizeof(int32_t) * static_cast<size_t>(table_pages), s>>>(
      static_cast<const bf16_t*>(qkv), q_stride, static_cast<bf16_t*>(out), static_cast<const bf16_t*>(kv), pf_tiles,
      item_start, item_pos0, table_off, block_ids, hq, hkv, scale, window, part_o, part_ml);
  const int rc = check_launch("psamd_attention_prefill");
  if (rc != 0 || nsplit == 1) return rc;
  return launch_prefill_merge(s, part_o, part_ml, out, pf_tiles, item_start, n_tiles, hq, 16 * NS, nsplit);
}

template <int NS, int CT>
static int launch_decode(hipStream_t s, const void* qkv, int q_stride, const void* kv, void* out, float* part_o,
                         float* part_ml, const int32_t* dec_items, int n_dec, const int32_t* item_start, const int32_t* item_end,
                         const int32_t* table_off, const int32_t* block_ids, int hq, int hkv, int nsplit, float scale,
                         int window, int min_tiles) {
  const int group = hq / hkv;
  const size_t smem = sizeof(float) * (8 * group + 4 * static_cast<size_t>(group) * 16 * NS);
  const int64_t groups_of_8 = ceil_div(static_cast<int64_t>(n_dec) * nsplit, 8);
  attn_decode_mfma_kernel<NS, CT><<<dim3(8 * hkv, static_cast<unsigned>(groups_of_8)), dim3(256), smem, s>>>(
      static_cast<const bf16_t*>(qkv), q_stride, static_cast<const bf16_t*>(kv), static_cast<bf16_t*>(out), part_o,
      part_ml, dec_items, item_start, item_end, table_off, block_ids, hq, hkv, nsplit, scale, window, min_tiles, n_dec);
  return check_launch("psamd_attention_decode");
}

template <int NS>
static int dispatch_decode_ct(int ct, hipStream_t s, const void* qkv, int q_stride, const void* kv, void* out,
                              float* part_o, float* part_ml, const int32_t* dec_items, int n_dec, const int32_t* item_start,
                              const int32_t* item_end, const int32_t* table_off, const int32_t* block_ids, int hq,
                              int hkv, int nsplit, float scale, int window, int min_tiles) {
#define PSAMD_DEC(CT_)                                                                                             \
  return launch_decode<NS, CT_>(s, qkv, q_stride, kv, out, part_o, part_ml, dec_items, n_dec, item_start, item_end, \
                                table_off, block_ids, hq, hkv, nsplit, scale, window, min_tiles)
  switch (ct) {
    case 1: PSAMD_DEC(1);
    case 2: PSAMD_DEC(2);
    default: PSAMD_DEC(4);
  }
#undef PSAMD_DEC
}

}  // namespace psamd

using namespace psamd;

extern "C" {

// 1 if the matrix-core kernels take this shape, else 0 (the caller then uses the generic kernel).
int psamd_attention_mfma_supports(int hq, int hkv, int head_dim) {
  if (hq <= 0 || hkv <= 0 || hq % hkv) return 0;
  const int group = hq / hkv;
  const bool dim_ok = head_dim % 16 == 0 && ((head_dim >= 16 && head_dim <= 128) || head_dim == 160 || head_dim == 192 ||
                                             head_dim == 256);
  const size_t smem = sizeof(float) * (8 * group + 4 * static_cast<size_t>(group) * head_dim);
  return dim_ok && group <= 64 && smem <= 64 * 1024 && hq <= 65535 && hkv <= 65535;
}

// Into how many runs psamd_attention_prefill may cut the keys of this step's query tiles; from 2
// on it needs part_o and part_ml.
int psamd_attention_prefill_nsplit(int n_tiles, int max_kv_len, int hq, int hkv, int head_dim) {
  if (!psamd_attention_mfma_supports(hq, hkv, head_dim) || n_tiles <= 0) return 1;
  return prefill_nsplit(n_tiles, max_kv_len, hq, hkv, head_dim);
}

// Rows of part_o / part_ml (32 * n_tiles * nsplit) that no step of this shape exceeds while
// nsplit > 1: the runs are dealt out so that the workgroups fill the chip once, which bounds
// (tiles x runs) whatever the step. A caller that keeps the buffers at this size never grows them.
int psamd_attention_prefill_part_rows(int hq, int hkv, int head_dim) {
  if (!psamd_attention_mfma_supports(hq, hkv, head_dim)) return 0;
  const int group = hq / hkv;
  // grouped kernel: tiles * runs * hkv * ceil(group / 4) <= 512 (256 above head size 64; two runs
  // for up to 128 workgroups stay below it too); per-head kernel: tiles * runs * hq <= 256.
  // With one or two query heads per kv head the grouped kernel's workgroups take four or two tiles:
  // tiles * runs * hq <= 4 * 512 (4 * 256 above head size 64).
  const int tiles_times_runs = group <= 2 ? std::max(1, 4 * (head_dim <= 64 ? 512 : 256) / hq)
                                          : std::max(1, 512 / (hkv * ((group + 3) / 4)));
  return 32 * tiles_times_runs;
}

// pf_tiles: (item, first query) of every tile of 32 queries; pf_blocks: the first tile of every run
// of up to four consecutive tiles of one item, in the order of the tiles (n_blocks = 0: no such
// list; steps with one or two query heads per kv head then run a slower form).
// max_kv_len: the longest request of the step after it (sizes the block table staged in LDS).
// nsplit: 1, or what psamd_attention_prefill_nsplit gave for these sizes (or less); part_o then
// has room for 32 * n_tiles * hq * nsplit * head_dim floats and part_ml for 32 * n_tiles * hq * nsplit * 2.
int psamd_attention_prefill(void* stream, const void* qkv, int q_stride, void* out, const void* kv,
                            const int32_t* pf_tiles, int n_tiles, const int32_t* pf_blocks, int n_blocks, int max_kv_len,
                            const int32_t* item_start,
                            const int32_t* item_pos0, const int32_t* table_off, const int32_t* block_ids, int hq,
                            int hkv, int head_dim, float scale, int window, float* part_o, float* part_ml, int nsplit) {
  PSAMD_REQUIRE(psamd_attention_mfma_supports(hq, hkv, head_dim), "shape not supported by the matrix-core kernels");
  PSAMD_REQUIRE(q_stride % 8 == 0, "query row stride must be a multiple of 8 elements");
  PSAMD_REQUIRE(max_kv_len >= 1 && max_kv_len <= 8192 * kPage, "context too long for the block table staged in LDS");
  if (n_tiles == 0) return 0;
  PSAMD_REQUIRE(n_tiles <= 65535, "too many query tiles for one launch");
  PSAMD_REQUIRE(n_blocks >= 0 && n_blocks <= n_tiles && (n_blocks == 0 || (pf_blocks != nullptr && 4LL * n_blocks >= n_tiles)),
                "the runs of tiles must cover the tiles, four at most each");
  PSAMD_REQUIRE(nsplit >= 1 && nsplit <= kMaxPrefillSplit, "nsplit must be in [1, 16]");
  PSAMD_REQUIRE(nsplit == 1 || (part_o != nullptr && part_ml != nullptr), "split keys need part_o and part_ml");
  hipStream_t s = static_cast<hipStream_t>(stream);
#define PSAMD_PF(NS_)                                                                                           \
  return launch_prefill<NS_>(s, qkv, q_stride, out, kv, pf_tiles, n_tiles, pf_blocks, n_blocks, max_kv_len, item_start, \
                             item_pos0, table_off, block_ids, hq, hkv, scale, window, part_o, part_ml, nsplit)
  switch (head_dim / 16) {
    case 1: PSAMD_PF(1);
    case 2: PSAMD_PF(2);
    case 3: PSAMD_PF(3);
    case 4: PSAMD_PF(4);
    case 5: PSAMD_PF(5);
    case 6: PSAMD_PF(6);
    case 7: PSAMD_PF(7);
    case 8: PSAMD_PF(8);
    case 10: PSAMD_PF(10);
    case 12: PSAMD_PF(12);
    default: PSAMD_PF(16);
  }
#undef PSAMD_PF
}

// Whether the single-token items of a step have one context far longer than the rest: more than
// four times their mean and 4,096 tokens beyond that. The keys are then cut into runs of 1,024 or
// more, as many as the longest request needs, instead of as many as fill the chip with requests of
// equal length; a long request among short ones is otherwise read by a few workgroups while the
// rest of the chip waits (31 requests of 1,024 tokens and one of 60,000: 429 -> 55 us a layer at
// head size 64). Steps of equal lengths pay 10 to 25 us a layer for the extra runs, so it is
// decided step by step. Tuned on 256 compute units.
int psamd_attention_decode_skewed(int n_dec, int longest, int64_t total) {
  return n_dec > 1 && static_cast<int64_t>(longest) * n_dec > 4 * total + 4096LL * n_dec;
}

// How psamd_attention_decode should cut the keys of a step of n_dec single-token items whose
// longest context is kv_len (for a captured step: the longest there can be): *nsplit runs per
// request, none shorter than *min_run keys. Two workgroups per compute unit; from one per compute
// unit on, no split and no merge kernel (32 requests x 8 kv heads at head size 128: 48 -> 41 us).
int psamd_attention_decode_plan(int n_dec, int kv_len, int skewed, int hkv, int window, int* nsplit, int* min_run) {
  PSAMD_REQUIRE(n_dec >= 1 && kv_len >= 1 && hkv >= 1 && nsplit != nullptr && min_run != nullptr, "decode plan: bad sizes");
  if (window > 0) kv_len = std::min(kv_len, window);
  const int64_t pairs = static_cast<int64_t>(n_dec) * hkv;
  int n = pairs >= 256 ? 1 : static_cast<int>(std::max<int64_t>(1, std::min<int64_t>({64, 512 / pairs, ceil_div(kv_len, 128)})));
  int run = 128;
  if (skewed && window <= 0) {
    n = std::max(n, static_cast<int>(std::min<int64_t>({64, 4096 / n_dec, ceil_div(kv_len, 1024)})));
    run = 1024;
  }
  *nsplit = std::max(n, 1);
  *min_run = run;
  return 0;
}

// (requests x runs) of any plan for up to max_requests single-token items: room for the partial
// results of every decode step, so that the buffers never grow.
int psamd_attention_decode_max_parts(int max_requests) { return std::max({4096, 512, max_requests}); }

// part_o needs n_dec * hq * nsplit * head_dim floats, part_ml n_dec * hq * nsplit * 2.
// min_split_keys: a request's keys are cut into runs no shorter than this (a multiple of 32), so
// that nsplit can follow the longest request of a step without cutting the short ones to pieces.
int psamd_attention_decode(void* stream, const void* qkv, int q_stride, void* out, const void* kv, float* part_o,
                           float* part_ml, const int32_t* dec_items, int n_dec, const int32_t* item_start,
                           const int32_t* item_end, const int32_t* table_off, const int32_t* block_ids, int hq,
                           int hkv, int head_dim, int nsplit, float scale, int window, int min_split_keys) {
  PSAMD_REQUIRE(psamd_attention_mfma_supports(hq, hkv, head_dim), "shape not supported by the matrix-core kernels");
  PSAMD_REQUIRE(q_stride % 8 == 0, "query row stride must be a multiple of 8 elements");
  PSAMD_REQUIRE(nsplit >= 1 && nsplit <= 64, "nsplit must be in [1, 64]");
  PSAMD_REQUIRE(min_split_keys >= 32 && min_split_keys % 32 == 0, "min_split_keys must be a positive multiple of 32");
  const int min_tiles = min_split_keys / 32;
  PSAMD_REQUIRE(static_cast<int64_t>(n_dec) * nsplit <= 8 * 65535, "too many (request, split) pairs for one launch");
  if (n_dec == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int group = hq / hkv;
  const int ct = group <= 16 ? 1 : (group <= 32 ? 2 : 4);
  int rc;
#define PSAMD_DEC_NS(NS_)                                                                                          \
  rc = dispatch_decode_ct<NS_>(ct, s, qkv, q_stride, kv, out, part_o, part_ml, dec_items, n_dec, item_start,    \
                               item_end, table_off, block_ids, hq, hkv, nsplit, scale, window, min_tiles);       \
  break
  switch (head_dim / 16) {
    case 1: PSAMD_DEC_NS(1);
    case 2: PSAMD_DEC_NS(2);
    case 3: PSAMD_DEC_NS(3);
    case 4: PSAMD_DEC_NS(4);
    case 5: PSAMD_DEC_NS(5);
    case 6: PSAMD_DEC_NS(6);
    case 7: PSAMD_DEC_NS(7);
    case 8: PSAMD_DEC_NS(8);
    case 10: PSAMD_DEC_NS(10);
    case 12: PSAMD_DEC_NS(12);
    default: PSAMD_DEC_NS(16);
  }
#undef PSAMD_DEC_NS
  if (rc != 0 || nsplit == 1) return rc;
  attn_decode_merge_kernel<<<dim3(n_dec, hq), dim3(64), 0, s>>>(part_o, part_ml, static_cast<bf16_t*>(out), dec_items,
                                                               item_start, hq, head_dim, nsplit);
  return check_launch("psamd_attention_decode(merge)");
}

}  // extern "C"
