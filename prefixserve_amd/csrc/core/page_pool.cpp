#include "page_pool.hpp"

#include <stdexcept>

namespace psamd {

const char* describe(Fault f) noexcept {
  switch (f) {
    case Fault::kNone: return "no fault";
    case Fault::kBadPage: return "invalid block id";
    case Fault::kNotInUse: return "block is not allocated: a double free, or use after the free";
    case Fault::kTooManyOwners: return "too many references on one block";
    case Fault::kAlreadyShared: return "block is already cached in the prefix tree";
    case Fault::kIndexFull: return "the prefix tree has no node left";
    case Fault::kBadArgument: return "invalid argument";
  }
  return "unknown fault";
}

PagePool::PagePool(int32_t pages) {
  if (pages < 1 || pages > kMaxBlocks)
    throw std::invalid_argument("a pool holds between 1 and " + std::to_string(kMaxBlocks) + " blocks");
  cell_.resize(static_cast<size_t>(pages));
  // 0 -> 1 -> 2 -> ...: the first pages handed out are 0, 1, 2, ...
  for (int32_t id = 0; id < pages; ++id)
    cell_[static_cast<size_t>(id)] = kFreeTag | static_cast<uint32_t>(id + 1 < pages ? id + 2 : 0);
  first_free_ = 0;
  free_count_ = pages;
}

BlockId PagePool::take() noexcept {
  const BlockId id = first_free_;
  if (id == kNoBlock) return kNoBlock;
  const uint32_t link = cell_[static_cast<size_t>(id)] & ~kFreeTag;
  first_free_ = link == 0 ? kNoBlock : static_cast<BlockId>(link - 1);
  cell_[static_cast<size_t>(id)] = 1;
  --free_count_;
  return id;
}

bool PagePool::take_many(int32_t n, BlockId* out) noexcept {
  if (n < 0 || n > free_count_) return false;
  for (int32_t i = 0; i < n; ++i) out[i] = take();
  return true;
}

Fault PagePool::share(BlockId id) noexcept {
  if (!valid(id)) return Fault::kBadPage;
  if (!in_use(id)) return Fault::kNotInUse;
  uint32_t& owners = cell_[static_cast<size_t>(id)];
  if (owners >= kMaxOwners) return Fault::kTooManyOwners;
  ++owners;
  return Fault::kNone;
}

Fault PagePool::drop(BlockId id) noexcept {
  if (!valid(id)) return Fault::kBadPage;
  if (!in_use(id)) return Fault::kNotInUse;
  uint32_t& entry = cell_[static_cast<size_t>(id)];
  if (--entry == 0) {
    entry = kFreeTag | static_cast<uint32_t>(first_free_ == kNoBlock ? 0 : first_free_ + 1);
    first_free_ = id;
    ++free_count_;
  }
  return Fault::kNone;
}

int32_t PagePool::owners(BlockId id) const noexcept {
  if (!valid(id)) return -1;
  return in_use(id) ? static_cast<int32_t>(cell_[static_cast<size_t>(id)]) : 0;
}

bool PagePool::check_invariants(std::string* why) const {
  auto broken = [why](std::string what) {
    if (why != nullptr) *why = std::move(what);
    return false;
  };
  // Walk the free list: it must visit free_count_ distinct free pages and end.
  std::vector<uint8_t> seen(cell_.size(), 0);
  int32_t walked = 0;
  for (BlockId id = first_free_; id != kNoBlock;) {
    if (!valid(id)) return broken("the free list leaves the pool");
    if (in_use(id)) return broken("block " + std::to_string(id) + " is in the free list and has owners");
    if (seen[static_cast<size_t>(id)]) return broken("block " + std::to_string(id) + " is in the free list twice");
    seen[static_cast<size_t>(id)] = 1;
    if (++walked > num_blocks()) return broken("the free list does not end");
    const uint32_t link = cell_[static_cast<size_t>(id)] & ~kFreeTag;
    id = link == 0 ? kNoBlock : static_cast<BlockId>(link - 1);
  }
  if (walked != free_count_) return broken("free count and free list disagree");
  for (BlockId id = 0; id < num_blocks(); ++id) {
    if (!in_use(id) && !seen[static_cast<size_t>(id)])
      return broken("block " + std::to_string(id) + " is lost: no owner and not in the free list");
    if (in_use(id) && cell_[static_cast<size_t>(id)] == 0) return broken("a block in use has no owner");
  }
  return true;
}

StateSlots::StateSlots(int32_t num_slots, int64_t bytes_per_slot) : bytes_per_slot_(bytes_per_slot) {
  if (num_slots < 1 || num_slots > kMaxBlocks) throw std::invalid_argument("num_slots must be in [1, 2^26]");
  if (bytes_per_slot < 0) throw std::invalid_argument("bytes_per_slot must not be negative");
  next_.resize(static_cast<size_t>(num_slots));
  for (int32_t s = 0; s < num_slots; ++s) next_[static_cast<size_t>(s)] = s + 1 < num_slots ? s + 1 : kEnd;
  first_free_ = 0;
  free_count_ = num_slots;
}

int32_t StateSlots::acquire() noexcept {
  const int32_t s = first_free_;
  if (s == kEnd) return -1;
  first_free_ = next_[static_cast<size_t>(s)];
  next_[static_cast<size_t>(s)] = kTaken;
  --free_count_;
  return s;
}

Fault StateSlots::release(int32_t slot) noexcept {
  if (slot < 0 || slot >= num_slots()) return Fault::kBadPage;
  if (next_[static_cast<size_t>(slot)] != kTaken) return Fault::kNotInUse;
  next_[static_cast<size_t>(slot)] = first_free_;
  first_free_ = slot;
  ++free_count_;
  return Fault::kNone;
}

}  // namespace psamd
