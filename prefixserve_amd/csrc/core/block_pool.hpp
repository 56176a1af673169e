// Host-side page bookkeeping for the KV cache: which page ids are free, and how many
// owners each live page has. A page id is the index of a page in every device pool of
// its layer group; nothing here touches device memory.
//
// Behaviour follows the reference's BlockManager (csrc/block_manager.hpp:49-119,
// csrc/block_manager.cpp:29-66): a fixed pool, LIFO reuse, reference counts, no direct
// "free" call (a page is free only when its count drops to zero), and misuse reported
// as a status value rather than an exception so the per-step path never unwinds.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace psamd {

using BlockId = int32_t;

inline constexpr int32_t kBlockSize = 16;      // tokens per page
inline constexpr BlockId kNoBlock = -1;
inline constexpr int32_t kMaxBlocks = 1 << 26;  // keeps every index well inside int32

enum class Status : uint8_t {
  kOk = 0,
  kInvalidBlockId,      // id outside [0, num_blocks)
  kBlockNotAllocated,   // count operation on a free page: double free or use-after-free
  kRefCountOverflow,
  kBlockAlreadyCached,  // page already belongs to a prefix-tree node
  kOutOfNodes,          // prefix tree ran out of nodes (an invariant is broken)
  kInvalidArgument,
};

const char* status_name(Status s) noexcept;

class BlockPool {
 public:
  // Throws std::invalid_argument unless 1 <= num_blocks <= kMaxBlocks.
  explicit BlockPool(int32_t num_blocks);
  BlockPool(const BlockPool&) = delete;
  BlockPool& operator=(const BlockPool&) = delete;

  // A page with count 1, or kNoBlock when none is free (normal under load).
  BlockId allocate() noexcept {
    if (free_top_ == 0) return kNoBlock;
    const BlockId id = free_[--free_top_];
    refs_[static_cast<size_t>(id)] = 1;
    return id;
  }

  // n pages into out[0..n), or false with nothing taken.
  bool allocate_many(int32_t n, BlockId* out) noexcept {
    if (n < 0 || n > free_top_) return false;
    for (int32_t i = 0; i < n; ++i) out[i] = allocate();
    return true;
  }

  Status incref(BlockId id) noexcept {
    if (!valid(id)) return Status::kInvalidBlockId;
    int32_t& r = refs_[static_cast<size_t>(id)];
    if (r == 0) return Status::kBlockNotAllocated;
    if (r == INT32_MAX) return Status::kRefCountOverflow;
    ++r;
    return Status::kOk;
  }

  // The last owner's decref returns the page to the free stack. A decref of a free
  // page is refused in every build: letting it through would list the page twice and
  // two requests would later write the same memory.
  Status decref(BlockId id) noexcept {
    if (!valid(id)) return Status::kInvalidBlockId;
    int32_t& r = refs_[static_cast<size_t>(id)];
    if (r == 0) return Status::kBlockNotAllocated;
    if (--r == 0) free_[free_top_++] = id;
    return Status::kOk;
  }

  bool valid(BlockId id) const noexcept { return id >= 0 && id < num_blocks_; }
  // 0 for a free page, -1 for an invalid id.
  int32_t ref_count(BlockId id) const noexcept { return valid(id) ? refs_[static_cast<size_t>(id)] : -1; }
  int32_t num_free() const noexcept { return free_top_; }
  int32_t num_blocks() const noexcept { return num_blocks_; }

  // O(n) consistency check for tests: every page is either counted or listed free, once.
  bool check_invariants(std::string* why) const;

 private:
  int32_t num_blocks_;
  int32_t free_top_;             // free_[0, free_top_) are the free ids, top = next out
  std::vector<int32_t> refs_;
  std::vector<BlockId> free_;    // sized once; never reallocates
};

// Slots for per-request state of a fixed size (recurrent state, running sums): one slot
// per live request, taken at admission and returned when the request leaves. The
// reference has no such state; the slot id travels in the step batch next to the block
// table so that a mixer with state of its own finds it. bytes_per_slot may be 0 (no
// mixer of the model keeps state): ids are still handed out so the batch format is one.
class StateSlots {
 public:
  StateSlots(int32_t num_slots, int64_t bytes_per_slot);
  int32_t acquire() noexcept {
    if (free_.empty()) return -1;
    const int32_t s = free_.back();
    free_.pop_back();
    used_[static_cast<size_t>(s)] = 1;
    return s;
  }
  Status release(int32_t slot) noexcept {
    if (slot < 0 || slot >= num_slots_) return Status::kInvalidBlockId;
    if (!used_[static_cast<size_t>(slot)]) return Status::kBlockNotAllocated;
    used_[static_cast<size_t>(slot)] = 0;
    free_.push_back(slot);
    return Status::kOk;
  }
  bool in_use(int32_t slot) const noexcept {
    return slot >= 0 && slot < num_slots_ && used_[static_cast<size_t>(slot)] != 0;
  }
  int32_t num_slots() const noexcept { return num_slots_; }
  int32_t num_free() const noexcept { return static_cast<int32_t>(free_.size()); }
  int64_t bytes_per_slot() const noexcept { return bytes_per_slot_; }

 private:
  int32_t num_slots_;
  int64_t bytes_per_slot_;
  std::vector<uint8_t> used_;
  std::vector<int32_t> free_;
};

}  // namespace psamd
