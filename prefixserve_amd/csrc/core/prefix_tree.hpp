// Prefix cache over KV pages: a tree with one node per full 16-token page. A path from
// the root spells a cached prompt prefix page by page, so a new request whose tokens
// start the same way can reuse those pages instead of recomputing them.
//
// Behaviour follows the reference's RadixTree (csrc/radix_tree.hpp:36-144,
// csrc/radix_tree.cpp:130-297):
//   * a child is found by hashing ALL tokens of its page together with the parent id and
//     is accepted only after comparing the tokens: two siblings may start with the same
//     token, and the same tokens at another depth are another node;
//   * the tree owns one reference on every cached page; a request using the page owns
//     one more, so "count == 1" means only the tree holds it and it may be evicted;
//   * match_prefix takes one reference per matched page for the caller;
//   * insert is all-or-nothing, never replaces a page that is already cached for the
//     same tokens, and ignores a trailing partial page;
//   * evict removes least-recently-used leaves nobody else holds; a parent that loses
//     its last child becomes a leaf and may go in the same call;
//   * nothing allocates after the constructor.
// Single-threaded by design, like its owner, the scheduler.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

#include "block_pool.hpp"

namespace psamd {

class PrefixTree {
 public:
  // `pool` must outlive the tree. The destructor gives the tree's references back.
  PrefixTree(BlockPool& pool, uint64_t hash_seed);
  ~PrefixTree();
  PrefixTree(const PrefixTree&) = delete;
  PrefixTree& operator=(const PrefixTree&) = delete;

  static uint64_t random_seed();

  // Longest cached prefix of tokens[0, n) in whole pages. Writes the page ids to
  // out[0 .. matched/16) (out must hold n/16 entries), takes one reference on each for
  // the caller, marks the path as used now. Returns the matched token count.
  int64_t match_prefix(const int32_t* tokens, int64_t n, BlockId* out) noexcept;

  // Caches the full pages of tokens[0, n); blocks[i] holds tokens [16i, 16i+16).
  Status insert(const int32_t* tokens, int64_t n, const BlockId* blocks, int64_t num_blocks,
                int32_t* added) noexcept;

  // Frees up to `want` pages, least recently used first. Returns how many were freed.
  int32_t evict(int32_t want) noexcept;

  int32_t num_cached_blocks() const noexcept { return capacity_ - 1 - static_cast<int32_t>(spare_.size()); }
  int32_t max_blocks() const noexcept { return pool_.num_blocks(); }
  bool is_cached(BlockId id) const noexcept { return pool_.valid(id) && owned_[static_cast<size_t>(id)] != 0; }

  bool check_invariants(std::string* why) const;

 private:
  using Node = int32_t;
  static constexpr Node kRoot = 0;
  static constexpr Node kNone = -1;

  uint64_t edge_hash(Node parent, const int32_t* page_tokens) const noexcept;
  // Slot of the child of `parent` spelling `page_tokens`, or -1.
  int64_t find_edge(Node parent, const int32_t* page_tokens, uint64_t h) const noexcept;
  void table_put(uint64_t h, Node node) noexcept;
  void table_remove(size_t slot) noexcept;
  const int32_t* tokens_of(Node n) const noexcept { return &page_tokens_[static_cast<size_t>(n) * kBlockSize]; }

  // Indexed min-heap of leaves by (last use, node id); each node knows its position.
  bool older(Node a, Node b) const noexcept;
  void heap_set(size_t pos, Node n) noexcept;
  void heap_up(size_t pos) noexcept;
  void heap_down(size_t pos) noexcept;
  void heap_add(Node n) noexcept;
  void heap_drop(Node n) noexcept;

  void drop_leaf(Node leaf) noexcept;

  BlockPool& pool_;
  int32_t capacity_;                 // nodes including the root: num_blocks + 1
  uint32_t key_[kBlockSize];         // random per-position hash keys
  uint64_t clock_ = 0;               // logical time of the last match/insert

  std::vector<Node> parent_;
  std::vector<BlockId> block_;       // kNoBlock for the root and for spare nodes
  std::vector<int32_t> children_;
  std::vector<int32_t> heap_pos_;    // -1 when not in the heap
  std::vector<uint64_t> used_at_;
  std::vector<int32_t> page_tokens_; // [capacity_][kBlockSize]
  std::vector<Node> spare_;

  std::vector<uint64_t> slot_hash_;  // open addressing, power-of-two size, <= 50 % load
  std::vector<Node> slot_node_;      // kNone = empty
  size_t mask_ = 0;

  std::vector<Node> heap_;
  size_t heap_size_ = 0;
  std::vector<Node> held_back_;      // evict(): leaves somebody still uses, re-added after
  std::vector<uint8_t> owned_;       // owned_[page] = the tree holds a reference on it
};

}  // namespace psamd
