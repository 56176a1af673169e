#include "prefix_tree.hpp"

#include <cstring>
#include <random>

namespace psamd {

namespace {

inline uint64_t finalize64(uint64_t z) noexcept {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

inline size_t sz(int64_t v) noexcept { return static_cast<size_t>(v); }

}  // namespace

uint64_t PrefixTree::random_seed() {
  std::random_device rd;
  return (static_cast<uint64_t>(rd()) << 32) ^ rd();
}

PrefixTree::PrefixTree(BlockPool& pool, uint64_t hash_seed)
    : pool_(pool), capacity_(pool.num_blocks() + 1) {
  uint64_t s = hash_seed;
  for (int32_t i = 0; i < kBlockSize; ++i) {
    s = finalize64(s);
    key_[i] = static_cast<uint32_t>(s >> 32);
  }
  const size_t cap = sz(capacity_);
  parent_.assign(cap, kNone);
  block_.assign(cap, kNoBlock);
  children_.assign(cap, 0);
  heap_pos_.assign(cap, -1);
  used_at_.assign(cap, 0);
  page_tokens_.assign(cap * kBlockSize, 0);
  spare_.reserve(cap);
  for (Node n = capacity_ - 1; n >= 1; --n) spare_.push_back(n);

  size_t slots = 16;
  while (slots < 2 * cap) slots <<= 1;
  slot_hash_.assign(slots, 0);
  slot_node_.assign(slots, kNone);
  mask_ = slots - 1;

  heap_.assign(cap, kNone);
  held_back_.reserve(cap);
  owned_.assign(sz(pool.num_blocks()), 0);
}

PrefixTree::~PrefixTree() {
  for (Node n = 1; n < capacity_; ++n) {
    if (block_[sz(n)] != kNoBlock) (void)pool_.decref(block_[sz(n)]);
  }
}

// NH-style hash over the page: sum of (t[2i]+k[2i]) * (t[2i+1]+k[2i+1]) with 32-bit
// wrapping adds and a 64-bit product, mixed with the parent id and finalized
// (csrc/radix_tree.cpp:65-87 of the reference describes the same family).
uint64_t PrefixTree::edge_hash(Node parent, const int32_t* t) const noexcept {
  uint64_t acc = 0;
  for (int32_t i = 0; i < kBlockSize; i += 2) {
    const uint32_t a = static_cast<uint32_t>(t[i]) + key_[i];
    const uint32_t b = static_cast<uint32_t>(t[i + 1]) + key_[i + 1];
    acc += static_cast<uint64_t>(a) * static_cast<uint64_t>(b);
  }
  return finalize64(acc ^ (static_cast<uint64_t>(static_cast<uint32_t>(parent)) << 32));
}

int64_t PrefixTree::find_edge(Node parent, const int32_t* t, uint64_t h) const noexcept {
  for (size_t s = h & mask_;; s = (s + 1) & mask_) {
    const Node n = slot_node_[s];
    if (n == kNone) return -1;
    // A hash hit alone never returns a page: parent and all tokens must agree.
    if (slot_hash_[s] == h && parent_[sz(n)] == parent &&
        std::memcmp(tokens_of(n), t, sizeof(int32_t) * kBlockSize) == 0) {
      return static_cast<int64_t>(s);
    }
  }
}

void PrefixTree::table_put(uint64_t h, Node node) noexcept {
  size_t s = h & mask_;
  while (slot_node_[s] != kNone) s = (s + 1) & mask_;
  slot_hash_[s] = h;
  slot_node_[s] = node;
}

// Linear-probing deletion by shifting later entries back, so no tombstones pile up.
void PrefixTree::table_remove(size_t hole) noexcept {
  size_t s = hole;
  for (;;) {
    s = (s + 1) & mask_;
    if (slot_node_[s] == kNone) break;
    const size_t home = slot_hash_[s] & mask_;
    // Move the entry at s into the hole unless its home lies cyclically in (hole, s].
    const bool stays = (hole <= s) ? (home > hole && home <= s) : (home > hole || home <= s);
    if (!stays) {
      slot_hash_[hole] = slot_hash_[s];
      slot_node_[hole] = slot_node_[s];
      hole = s;
    }
  }
  slot_node_[hole] = kNone;
  slot_hash_[hole] = 0;
}

int64_t PrefixTree::match_prefix(const int32_t* tokens, int64_t n, BlockId* out) noexcept {
  if (n <= 0 || tokens == nullptr) return 0;
  const uint64_t now = ++clock_;
  used_at_[kRoot] = now;
  Node cur = kRoot;
  int64_t pages = 0;
  for (int64_t b = 0; b < n / kBlockSize; ++b) {
    const int32_t* t = tokens + b * kBlockSize;
    const int64_t s = find_edge(cur, t, edge_hash(cur, t));
    if (s < 0) break;
    const Node child = slot_node_[sz(s)];
    if (pool_.incref(block_[sz(child)]) != Status::kOk) break;  // cannot fail while the tree owns it
    out[pages++] = block_[sz(child)];
    used_at_[sz(child)] = now;
    cur = child;
  }
  // Only leaves sit in the heap; the last node's key just grew.
  if (heap_pos_[sz(cur)] >= 0) heap_down(sz(heap_pos_[sz(cur)]));
  return pages * kBlockSize;
}

Status PrefixTree::insert(const int32_t* tokens, int64_t n, const BlockId* blocks, int64_t num_blocks,
                          int32_t* added) noexcept {
  if (added != nullptr) *added = 0;
  if (n < 0 || num_blocks < 0 || (n > 0 && tokens == nullptr) || (num_blocks > 0 && blocks == nullptr)) {
    return Status::kInvalidArgument;
  }
  const int64_t full = n / kBlockSize;
  if (num_blocks < full) return Status::kInvalidArgument;

  // 1. Walk what is cached already (read only).
  Node cur = kRoot;
  int64_t depth = 0;
  for (; depth < full; ++depth) {
    const int32_t* t = tokens + depth * kBlockSize;
    const int64_t s = find_edge(cur, t, edge_hash(cur, t));
    if (s < 0) break;
    cur = slot_node_[sz(s)];
  }
  const int64_t fresh = full - depth;
  if (fresh > static_cast<int64_t>(spare_.size())) return Status::kOutOfNodes;

  // 2. Check every new page before anything changes; marking as we go also catches the
  //    same id given twice in one call. Marks are rolled back on refusal.
  for (int64_t i = depth; i < full; ++i) {
    const BlockId id = blocks[i];
    Status bad = Status::kOk;
    if (!pool_.valid(id)) bad = Status::kInvalidBlockId;
    else if (pool_.ref_count(id) == 0) bad = Status::kBlockNotAllocated;
    else if (pool_.ref_count(id) == INT32_MAX) bad = Status::kRefCountOverflow;
    else if (owned_[sz(id)]) bad = Status::kBlockAlreadyCached;
    if (bad != Status::kOk) {
      for (int64_t j = depth; j < i; ++j) owned_[sz(blocks[j])] = 0;
      return bad;
    }
    owned_[sz(id)] = 1;
  }

  // 3. Commit; nothing below can fail.
  const uint64_t now = ++clock_;
  if (fresh > 0 && heap_pos_[sz(cur)] >= 0) heap_drop(cur);  // gains a child: no longer a leaf
  for (Node x = cur; x != kNone; x = parent_[sz(x)]) used_at_[sz(x)] = now;
  if (fresh == 0) {
    if (heap_pos_[sz(cur)] >= 0) heap_down(sz(heap_pos_[sz(cur)]));
    return Status::kOk;
  }
  for (int64_t i = depth; i < full; ++i) {
    const Node child = spare_.back();
    spare_.pop_back();
    const int32_t* t = tokens + i * kBlockSize;
    parent_[sz(child)] = cur;
    block_[sz(child)] = blocks[i];
    children_[sz(child)] = 0;
    heap_pos_[sz(child)] = -1;
    used_at_[sz(child)] = now;
    std::memcpy(&page_tokens_[sz(child) * kBlockSize], t, sizeof(int32_t) * kBlockSize);
    table_put(edge_hash(cur, t), child);
    ++children_[sz(cur)];
    (void)pool_.incref(blocks[i]);
    cur = child;
  }
  heap_add(cur);  // only the deepest new node is a leaf
  if (added != nullptr) *added = static_cast<int32_t>(fresh);
  return Status::kOk;
}

int32_t PrefixTree::evict(int32_t want) noexcept {
  int32_t freed = 0;
  held_back_.clear();
  while (freed < want && heap_size_ > 0) {
    const Node leaf = heap_[0];
    heap_drop(leaf);
    if (pool_.ref_count(block_[sz(leaf)]) > 1) {  // a request still reads it
      held_back_.push_back(leaf);
      continue;
    }
    drop_leaf(leaf);
    ++freed;
  }
  for (const Node n : held_back_) heap_add(n);
  held_back_.clear();
  return freed;
}

void PrefixTree::drop_leaf(Node leaf) noexcept {
  const Node parent = parent_[sz(leaf)];
  const int32_t* t = tokens_of(leaf);
  const int64_t s = find_edge(parent, t, edge_hash(parent, t));
  if (s >= 0) table_remove(sz(s));
  owned_[sz(block_[sz(leaf)])] = 0;
  (void)pool_.decref(block_[sz(leaf)]);  // count was 1: the page returns to the pool
  parent_[sz(leaf)] = kNone;
  block_[sz(leaf)] = kNoBlock;
  children_[sz(leaf)] = 0;
  heap_pos_[sz(leaf)] = -1;
  used_at_[sz(leaf)] = 0;
  spare_.push_back(leaf);
  if (--children_[sz(parent)] == 0 && parent != kRoot) heap_add(parent);
}

bool PrefixTree::older(Node a, Node b) const noexcept {
  const uint64_t ta = used_at_[sz(a)], tb = used_at_[sz(b)];
  return ta < tb || (ta == tb && a < b);  // ties by id: eviction order is deterministic
}

void PrefixTree::heap_set(size_t pos, Node n) noexcept {
  heap_[pos] = n;
  heap_pos_[sz(n)] = static_cast<int32_t>(pos);
}

void PrefixTree::heap_up(size_t pos) noexcept {
  const Node n = heap_[pos];
  while (pos > 0) {
    const size_t up = (pos - 1) / 2;
    if (!older(n, heap_[up])) break;
    heap_set(pos, heap_[up]);
    pos = up;
  }
  heap_set(pos, n);
}

void PrefixTree::heap_down(size_t pos) noexcept {
  const Node n = heap_[pos];
  for (;;) {
    size_t kid = 2 * pos + 1;
    if (kid >= heap_size_) break;
    if (kid + 1 < heap_size_ && older(heap_[kid + 1], heap_[kid])) ++kid;
    if (!older(heap_[kid], n)) break;
    heap_set(pos, heap_[kid]);
    pos = kid;
  }
  heap_set(pos, n);
}

void PrefixTree::heap_add(Node n) noexcept {
  heap_[heap_size_] = n;
  heap_pos_[sz(n)] = static_cast<int32_t>(heap_size_);
  ++heap_size_;
  heap_up(heap_size_ - 1);
}

void PrefixTree::heap_drop(Node n) noexcept {
  const size_t pos = sz(heap_pos_[sz(n)]);
  heap_pos_[sz(n)] = -1;
  --heap_size_;
  if (pos == heap_size_) return;
  const Node moved = heap_[heap_size_];
  heap_set(pos, moved);
  heap_up(pos);
  heap_down(sz(heap_pos_[sz(moved)]));
}

bool PrefixTree::check_invariants(std::string* why) const {
  auto fail = [&](const std::string& m) {
    if (why != nullptr) *why = m;
    return false;
  };
  std::vector<uint8_t> seen_block(sz(pool_.num_blocks()), 0);
  std::vector<int32_t> kids(sz(capacity_), 0);
  int32_t live = 0;
  for (Node n = 1; n < capacity_; ++n) {
    const BlockId b = block_[sz(n)];
    if (b == kNoBlock) {
      if (heap_pos_[sz(n)] != -1) return fail("spare node in heap");
      continue;
    }
    ++live;
    if (!pool_.valid(b)) return fail("node holds invalid block");
    if (seen_block[sz(b)]) return fail("block in two nodes");
    seen_block[sz(b)] = 1;
    if (!owned_[sz(b)]) return fail("node's block not marked cached");
    if (pool_.ref_count(b) < 1) return fail("cached block has no reference");
    const Node p = parent_[sz(n)];
    if (p < 0 || p >= capacity_ || (p != kRoot && block_[sz(p)] == kNoBlock)) return fail("dangling parent");
    ++kids[sz(p)];
    if (used_at_[sz(p)] < used_at_[sz(n)]) return fail("parent used before child");
    const int64_t s = find_edge(p, tokens_of(n), edge_hash(p, tokens_of(n)));
    if (s < 0 || slot_node_[sz(s)] != n) return fail("node not reachable through the table");
  }
  if (live != num_cached_blocks()) return fail("live nodes != cached count");
  for (int32_t b = 0; b < pool_.num_blocks(); ++b) {
    if (owned_[sz(b)] && !seen_block[sz(b)]) return fail("cached mark without a node");
  }
  size_t in_heap = 0;
  for (Node n = 0; n < capacity_; ++n) {
    if (kids[sz(n)] != children_[sz(n)]) return fail("child count wrong");
    const bool leaf = n != kRoot && block_[sz(n)] != kNoBlock && children_[sz(n)] == 0;
    if (leaf != (heap_pos_[sz(n)] >= 0)) return fail("heap membership != leaf");
    if (heap_pos_[sz(n)] >= 0) {
      ++in_heap;
      if (sz(heap_pos_[sz(n)]) >= heap_size_ || heap_[sz(heap_pos_[sz(n)])] != n) return fail("heap position stale");
    }
  }
  if (in_heap != heap_size_) return fail("heap size wrong");
  for (size_t i = 1; i < heap_size_; ++i) {
    if (older(heap_[i], heap_[(i - 1) / 2])) return fail("heap order broken");
  }
  size_t filled = 0;
  for (size_t s = 0; s <= mask_; ++s) filled += slot_node_[s] != kNone;
  if (filled != static_cast<size_t>(live)) return fail("table entries != live nodes");
  return true;
}

}  // namespace psamd
