// Which KV pages are free and how many owners every page in use has. A page id is the index
// of a page in each device pool of its layer group; nothing here touches device memory.
//
// What a caller can observe is the reference's BlockManager (csrc/block_manager.hpp:49-119,
// csrc/block_manager.cpp:29-66): a pool of fixed size whose first pages come out as
// 0, 1, 2, ...; the page given back last is handed out first; a page has owners, not a
// "free" call, and returns to the pool when its last owner lets go; misuse (a second free,
// an id out of range) is answered with a value, never with an exception, so that the
// per-step path cannot unwind.
//
// One array holds everything: the entry of a page in use is its owner count, the entry of a
// free page is a link to the next free page (tagged in the top bit), so the free pages form
// a list threaded through the array and the pool needs no second container.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace psamd {

using BlockId = int32_t;

inline constexpr int32_t kBlockSize = 16;       // tokens per page
inline constexpr BlockId kNoBlock = -1;
inline constexpr int32_t kMaxBlocks = 1 << 26;

// What went wrong in a call that changes counts; kNone = nothing.
enum class Fault : uint8_t {
  kNone = 0,
  kBadPage,          // id outside the pool
  kNotInUse,         // the page has no owner: freed twice, or used after it was freed
  kTooManyOwners,
  kAlreadyShared,    // the prefix index holds this page already
  kIndexFull,        // the prefix index has no node left (cannot happen while counts are right)
  kBadArgument,
};

// The text Python sees in a CoreError.
const char* describe(Fault f) noexcept;

class PagePool {
 public:
  // std::invalid_argument unless 1 <= pages <= kMaxBlocks.
  explicit PagePool(int32_t pages);
  PagePool(const PagePool&) = delete;
  PagePool& operator=(const PagePool&) = delete;

  int32_t num_blocks() const noexcept { return static_cast<int32_t>(cell_.size()); }
  int32_t num_free() const noexcept { return free_count_; }
  bool valid(BlockId id) const noexcept { return id >= 0 && id < num_blocks(); }

  // A page with one owner, or kNoBlock if the pool is empty (ordinary under load).
  BlockId take() noexcept;
  // n pages into out, or false and nothing taken.
  bool take_many(int32_t n, BlockId* out) noexcept;
  // One owner more / one less. The last owner's drop returns the page to the pool. Dropping
  // a free page is refused in every build: accepted, the page would be in the free list
  // twice and two requests would end up writing the same memory.
  Fault share(BlockId id) noexcept;
  Fault drop(BlockId id) noexcept;
  // Owners of a page: 0 if it is free, -1 if the id is no page.
  int32_t owners(BlockId id) const noexcept;

  // For tests, O(pages): every page is in use or in the free list, exactly once.
  bool check_invariants(std::string* why) const;

 private:
  static constexpr uint32_t kFreeTag = 0x80000000u;   // entry = kFreeTag | (next free page + 1), 0 ends the list
  static constexpr uint32_t kMaxOwners = 0x7fffffffu;

  bool in_use(BlockId id) const noexcept { return (cell_[static_cast<size_t>(id)] & kFreeTag) == 0; }

  std::vector<uint32_t> cell_;
  BlockId first_free_ = kNoBlock;
  int32_t free_count_ = 0;
};

// Places for per-request state of a fixed size (a recurrent state, running sums): a request
// takes one when it starts to run and returns it when it leaves. The reference has nothing
// of the kind; the slot id travels in the step batch beside the block tables so that a mixer
// with state of its own finds its row. bytes_per_slot may be 0 (no mixer of the model keeps
// state): ids are handed out all the same, so every batch looks alike.
class StateSlots {
 public:
  StateSlots(int32_t num_slots, int64_t bytes_per_slot);
  int32_t acquire() noexcept;                  // -1 if all are taken
  Fault release(int32_t slot) noexcept;
  bool in_use(int32_t slot) const noexcept {
    return slot >= 0 && slot < num_slots() && next_[static_cast<size_t>(slot)] == kTaken;
  }
  int32_t num_slots() const noexcept { return static_cast<int32_t>(next_.size()); }
  int32_t num_free() const noexcept { return free_count_; }
  int64_t bytes_per_slot() const noexcept { return bytes_per_slot_; }

 private:
  static constexpr int32_t kTaken = -2, kEnd = -1;
  std::vector<int32_t> next_;                  // free slots chained, kTaken for a slot in use
  int32_t first_free_ = kEnd;
  int32_t free_count_ = 0;
  int64_t bytes_per_slot_;
};

}  // namespace psamd
