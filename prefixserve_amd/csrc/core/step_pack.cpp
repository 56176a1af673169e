#include "step_pack.hpp"

#include <algorithm>

#include "page_pool.hpp"

namespace psamd {

namespace {

int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

std::string range(int64_t lo, int64_t hi) { return "[" + std::to_string(lo) + ", " + std::to_string(hi) + ")"; }

}  // namespace

PackLayout plan_step(const std::vector<PackItem>& items, const std::vector<PackGroup>& groups,
                     const PackLimits& lim) {
  if (items.empty()) throw PackError(-1, "empty step");
  PackLayout lay;
  lay.items = static_cast<int64_t>(items.size());
  const int64_t max_slot = std::max<int64_t>(lim.num_slots, 1);
  for (int64_t i = 0; i < lay.items; ++i) {
    const PackItem& it = items[static_cast<size_t>(i)];
    const int64_t n = it.tokens.size;
    if (n < 1) throw PackError(i, "an item has no tokens");
    const int64_t end = it.start + n;
    if (it.start < 0 || end > lim.max_position)
      throw PackError(i, "positions " + range(it.start, end) + " outside " + range(0, lim.max_position));
    if (it.slot < 0 || it.slot >= max_slot)
      throw PackError(i, "state slot " + std::to_string(it.slot) + " outside " + range(0, lim.num_slots));
    if (it.tables.size() != groups.size())
      throw PackError(i, std::to_string(it.tables.size()) + " block tables for " + std::to_string(groups.size()) +
                             " layer groups");
    for (int64_t w = 0; w < it.want.size; ++w)
      if (it.want.data[w] < 0 || it.want.data[w] >= n)
        throw PackError(i, "wanted place " + std::to_string(it.want.data[w]) + " outside its " + std::to_string(n) +
                               " tokens");
    const int64_t pages = ceil_div(end, kBlockSize);
    if (lim.static_pages >= 0 && pages > lim.static_pages)
      throw PackError(i, "needs " + std::to_string(pages) + " pages, static layout has " +
                             std::to_string(lim.static_pages));
    for (size_t g = 0; g < groups.size(); ++g)
      if (it.tables[g].size < pages)
        throw PackError(i, std::to_string(it.tables[g].size) + " blocks in group " + std::to_string(g) + " for " +
                               std::to_string(end) + " tokens");
    lay.tokens += n;
    lay.logit_rows += it.want.size;
    if (n == 1) {
      lay.decode_items += 1;
      lay.decode_max_kv = std::max(lay.decode_max_kv, end);
      lay.decode_sum_kv += end;
    } else {
      lay.prefill_tiles += ceil_div(n, lim.prefill_tile);
      lay.prefill_blocks += ceil_div(n, lim.prefill_tile * kTilesPerBlock);
    }
    lay.pages += lim.static_pages >= 0 ? lim.static_pages : pages;
    lay.max_kv_len = std::max(lay.max_kv_len, end);
  }
  int64_t off = 0;
  auto take = [&off](int64_t n) {
    const int64_t at = off;
    off += n;
    return at;
  };
  lay.token_ids = take(lay.tokens);
  lay.positions = take(lay.tokens);
  lay.tok_item = take(lay.tokens);
  lay.item_start = take(lay.items + 1);
  lay.item_pos0 = take(lay.items);
  lay.item_end = take(lay.items);
  lay.slots = take(lay.items);
  lay.logit_rows_off = take(lay.logit_rows);
  lay.dec_items = take(lay.decode_items);
  lay.pf_tiles = take(2 * lay.prefill_tiles);
  lay.pf_blocks = take(lay.prefill_blocks);
  lay.groups.resize(groups.size());
  for (GroupLayout& g : lay.groups) {
    g.table_off = take(lay.items + 1);
    g.write_slot = take(lay.tokens);
    g.block_ids = take(lay.pages);
  }
  lay.total = off;
  if (lay.total > INT32_MAX) throw PackError(-1, "step too large for 32-bit offsets");
  return lay;
}

void fill_step(const std::vector<PackItem>& items, const std::vector<PackGroup>& groups, const PackLimits& lim,
               const PackLayout& lay, int32_t* buf) {
  int32_t* ids = buf + lay.token_ids;
  int32_t* pos = buf + lay.positions;
  int32_t* tok_item = buf + lay.tok_item;
  int32_t* item_start = buf + lay.item_start;
  int32_t* item_pos0 = buf + lay.item_pos0;
  int32_t* item_end = buf + lay.item_end;
  int32_t* slots = buf + lay.slots;
  int32_t* rows = buf + lay.logit_rows_off;
  int32_t* dec = buf + lay.dec_items;
  int32_t* tiles = buf + lay.pf_tiles;
  int32_t* blocks = buf + lay.pf_blocks;
  int64_t tile_count = 0;

  int64_t t0 = 0;
  item_start[0] = 0;
  for (int64_t i = 0; i < lay.items; ++i) {
    const PackItem& it = items[static_cast<size_t>(i)];
    const int64_t n = it.tokens.size;
    for (int64_t j = 0; j < n; ++j) {
      const int64_t id = it.tokens.data[j];
      if (id < 0 || id >= lim.vocab_size)
        throw PackError(i, "token id " + std::to_string(id) + " outside " + range(0, lim.vocab_size));
      ids[t0 + j] = static_cast<int32_t>(id);
      // Absolute positions: a request that reused a prefix or resumes after preemption does
      // not restart at 0 (prefixserve/llama_engine.py:190-193).
      pos[t0 + j] = static_cast<int32_t>(it.start + j);
      tok_item[t0 + j] = static_cast<int32_t>(i);
    }
    if (n == 1) {
      *dec++ = static_cast<int32_t>(i);
    } else {
      for (int64_t q = 0; q < n; q += lim.prefill_tile) {
        if (q % (lim.prefill_tile * kTilesPerBlock) == 0) *blocks++ = static_cast<int32_t>(tile_count);
        *tiles++ = static_cast<int32_t>(i);
        *tiles++ = static_cast<int32_t>(q);
        ++tile_count;
      }
    }
    for (int64_t w = 0; w < it.want.size; ++w) *rows++ = static_cast<int32_t>(t0 + it.want.data[w]);
    item_pos0[i] = static_cast<int32_t>(it.start);
    item_end[i] = static_cast<int32_t>(it.start + n);
    slots[i] = static_cast<int32_t>(it.slot);
    t0 += n;
    item_start[i + 1] = static_cast<int32_t>(t0);
  }

  for (size_t g = 0; g < groups.size(); ++g) {
    int32_t* table_off = buf + lay.groups[g].table_off;
    int32_t* wslot = buf + lay.groups[g].write_slot;
    int32_t* bids = buf + lay.groups[g].block_ids;
    int64_t p0 = 0;
    t0 = 0;
    table_off[0] = 0;
    for (int64_t i = 0; i < lay.items; ++i) {
      const PackItem& it = items[static_cast<size_t>(i)];
      const Span& table = it.tables[g];
      const int64_t n = it.tokens.size, end = it.start + n;
      const int64_t pages = ceil_div(end, kBlockSize);
      const int64_t cap = lim.static_pages >= 0 ? lim.static_pages : pages;
      // Pages a token of this step can see or writes: all of them, or in a window group
      // those from the window of the first new token on. Earlier entries may be -1 (given
      // back); they are never read and go out as 0.
      const int64_t first_needed =
          groups[g].window < 0 ? 0 : std::max<int64_t>(0, it.start - groups[g].window + 1) / kBlockSize;
      for (int64_t p = 0; p < first_needed; ++p) bids[p0 + p] = 0;
      for (int64_t p = first_needed; p < pages; ++p) {
        const int64_t id = table.data[p];
        if (id < 0 || id >= groups[g].num_blocks)
          throw PackError(i, "block id " + std::to_string(id) + " outside the pool of group " + std::to_string(g) +
                                 " (0.." + std::to_string(groups[g].num_blocks - 1) + ")");
        bids[p0 + p] = static_cast<int32_t>(id);
      }
      for (int64_t p = pages; p < cap; ++p) bids[p0 + p] = 0;
      for (int64_t j = 0; j < n; ++j) {
        const int64_t at = it.start + j;
        wslot[t0 + j] = bids[p0 + at / kBlockSize] * kBlockSize + static_cast<int32_t>(at % kBlockSize);
      }
      p0 += cap;
      t0 += n;
      table_off[i + 1] = static_cast<int32_t>(p0);
    }
  }
}

}  // namespace psamd
