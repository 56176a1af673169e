// The integer arrays of one step, laid out in one buffer.
//
// A step is a list of items (a request, its next tokens, where they start, its block table
// in every layer group, its state slot, the places whose logits are wanted). All tokens lie
// back to back. The kernels read: per token its id, absolute position, item and the cache
// slot its key and value are written to; per item its first flat token, first position,
// length after the step and state slot; the flat rows whose logits are wanted; the items
// that bring one token (decode kernel) and the query tiles of the others (prefill kernel);
// per layer group the items' block tables back to back. The reference packs its arrays the
// same way, one pinned buffer and one copy (prefixserve/llama_engine.py:152-227), and checks
// them on the host first, because a bad page id on the device is an out-of-bounds write
// (llama_engine.py:270-287).
#pragma once

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

namespace psamd {

struct Span {
  const int64_t* data = nullptr;
  int64_t size = 0;
};

struct PackItem {
  Span tokens;
  int64_t start = 0;
  int64_t slot = 0;
  std::vector<Span> tables;  // one per layer group
  Span want;
};

struct PackGroup {
  int64_t num_blocks = 0;
  int64_t window = -1;  // < 0: every earlier position stays visible
};

struct PackLimits {
  int64_t vocab_size = 0;
  int64_t max_position = 0;
  int64_t num_slots = 0;
  int64_t prefill_tile = 1;
  int64_t static_pages = -1;  // >= 0: every item's table takes exactly this many entries
};

inline constexpr int64_t kTilesPerBlock = 4;   // tiles of queries in a block of the prefill list

struct GroupLayout {
  int64_t table_off = 0, write_slot = 0, block_ids = 0;
};

struct PackLayout {
  int64_t total = 0;
  int64_t tokens = 0, items = 0, logit_rows = 0, decode_items = 0, prefill_tiles = 0, pages = 0;
  // runs of up to kTilesPerBlock consecutive tiles of one item (a kernel whose workgroups take
  // several tiles of queries at once finds its tiles through them)
  int64_t prefill_blocks = 0;
  int64_t max_kv_len = 0;
  // over the items that bring one token: the longest context after the step and the sum of them
  int64_t decode_max_kv = 0, decode_sum_kv = 0;
  // offsets into the buffer, in 32-bit words
  int64_t token_ids = 0, positions = 0, tok_item = 0, item_start = 0, item_pos0 = 0, item_end = 0, slots = 0;
  int64_t logit_rows_off = 0, dec_items = 0, pf_tiles = 0, pf_blocks = 0;
  std::vector<GroupLayout> groups;
};

// A batch that must not run. ``item`` is the index of the offending item, or -1.
struct PackError : std::runtime_error {
  PackError(int64_t item_index, const std::string& what) : std::runtime_error(what), item(item_index) {}
  int64_t item;
};

// Checks everything that does not need the buffer and computes the layout.
PackLayout plan_step(const std::vector<PackItem>& items, const std::vector<PackGroup>& groups,
                     const PackLimits& lim);

// Fills ``buf`` (at least layout.total words) and checks token and page ids on the way.
void fill_step(const std::vector<PackItem>& items, const std::vector<PackGroup>& groups, const PackLimits& lim,
               const PackLayout& layout, int32_t* buf);

}  // namespace psamd
