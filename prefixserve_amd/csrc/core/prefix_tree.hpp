// The prefix cache: an index from token prefixes, one full page (16 tokens) at a time, to the
// KV pages that hold them, so that a request whose tokens start like an earlier one's reuses
// those pages instead of computing them again.
//
// What a caller can observe is the reference's RadixTree (csrc/radix_tree.hpp:36-144,
// csrc/radix_tree.cpp:130-297):
//   * a page is found by ALL its 16 tokens and its place in the prefix, and only after the
//     tokens were compared: two pages after the same prefix may start with the same token,
//     and the same 16 tokens after another prefix are another entry;
//   * the index is one owner of every page it holds and a request using the page is another,
//     so a page with a single owner is held by the index alone and may be evicted;
//   * match_prefix makes the caller an owner of every page it returns;
//   * insert takes all of its new pages or none, never replaces a page that is already held
//     for the same tokens, and ignores a trailing partial page;
//   * evict gives up the pages used longest ago that nobody else owns, leaves first; a page
//     whose last continuation went can go in the same call;
//   * nothing allocates after the constructor.
//
// How it is built here: entries live in one array; children are found through a hash table
// with chaining (bucket heads plus a link per entry, so removal is a list unlink and there
// are no tombstones and nothing to shift); recency is a doubly linked list through all
// entries, oldest first, with no clock: whenever an entry is used, it and then each of its
// ancestors move to the young end, so an entry always stands before its ancestors and a walk
// from the old end meets the leaves of a stale prefix before the prefix itself.
// One thread at a time, like the scheduler that owns it.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

#include "page_pool.hpp"

namespace psamd {

class PrefixIndex {
 public:
  // `pool` must outlive the index. The destructor returns the pages the index owns.
  PrefixIndex(PagePool& pool, uint64_t seed);
  ~PrefixIndex();
  PrefixIndex(const PrefixIndex&) = delete;
  PrefixIndex& operator=(const PrefixIndex&) = delete;

  static uint64_t random_seed();

  // Longest held prefix of tokens[0, n), in whole pages: page ids into out[0 .. result / 16)
  // (room for n / 16 entries), the caller becomes an owner of each, and the prefix counts as
  // used now. Returns the number of tokens matched.
  int64_t lookup(const int32_t* tokens, int64_t n, BlockId* out) noexcept;

  // Holds the full pages of tokens[0, n); pages[i] has tokens [16 i, 16 i + 16). *added = how
  // many pages the index took (those not held before).
  Fault hold(const int32_t* tokens, int64_t n, const BlockId* pages, int64_t num_pages, int32_t* added) noexcept;

  // Gives up to `want` pages back to the pool; returns how many.
  int32_t release_oldest(int32_t want) noexcept;

  int32_t size() const noexcept { return held_; }
  bool holds(BlockId id) const noexcept { return pool_.valid(id) && shared_[static_cast<size_t>(id)] != 0; }

  bool consistent(std::string* why) const;

 private:
  using Ref = int32_t;                       // index of an entry; 0 is the empty prefix
  static constexpr Ref kTop = 0, kNil = -1;

  struct Entry {
    Ref parent = kNil;                       // the prefix this page continues
    BlockId page = kNoBlock;
    int32_t continuations = 0;               // entries whose parent this is
    Ref same_bucket = kNil;                  // next entry of the hash bucket
    Ref older = kNil, younger = kNil;        // recency list
    uint64_t hash = 0;
  };

  uint64_t hash_of(Ref parent, const int32_t* page_tokens) const noexcept;
  Ref find(Ref parent, const int32_t* page_tokens, uint64_t h) const noexcept;
  const int32_t* text(Ref e) const noexcept { return &text_[static_cast<size_t>(e) * kBlockSize]; }
  void unlink_recency(Ref e) noexcept;
  void make_youngest(Ref e) noexcept;
  void used(Ref deepest) noexcept;           // the entry and its ancestors, in that order
  void forget(Ref leaf) noexcept;

  PagePool& pool_;
  uint64_t seed_;
  std::vector<Entry> entry_;                 // pages + 1
  std::vector<int32_t> text_;                // 16 tokens per entry
  std::vector<Ref> bucket_;                  // power of two many heads
  std::vector<Ref> unused_;                  // entries not in use
  std::vector<uint8_t> shared_;              // per page: the index owns it
  std::vector<uint32_t> seen_in_call_;       // per page: the insert call that last looked at it
  uint32_t call_ = 0;
  Ref oldest_ = kNil, youngest_ = kNil;
  int32_t held_ = 0;
};

}  // namespace psamd
