#include "block_pool.hpp"

#include <stdexcept>

namespace psamd {

const char* status_name(Status s) noexcept {
  switch (s) {
    case Status::kOk: return "ok";
    case Status::kInvalidBlockId: return "invalid block id";
    case Status::kBlockNotAllocated: return "block not allocated (double free or use-after-free)";
    case Status::kRefCountOverflow: return "ref count overflow";
    case Status::kBlockAlreadyCached: return "block already cached";
    case Status::kOutOfNodes: return "out of tree nodes";
    case Status::kInvalidArgument: return "invalid argument";
  }
  return "unknown status";
}

BlockPool::BlockPool(int32_t num_blocks) : num_blocks_(num_blocks), free_top_(0) {
  if (num_blocks < 1 || num_blocks > kMaxBlocks) {
    throw std::invalid_argument("num_blocks must be in [1, " + std::to_string(kMaxBlocks) + "]");
  }
  refs_.assign(static_cast<size_t>(num_blocks), 0);
  free_.resize(static_cast<size_t>(num_blocks));
  // Highest id at the bottom, so the first pages handed out are 0, 1, 2, ...
  for (int32_t i = 0; i < num_blocks; ++i) free_[static_cast<size_t>(i)] = num_blocks - 1 - i;
  free_top_ = num_blocks;
}

bool BlockPool::check_invariants(std::string* why) const {
  auto fail = [&](const std::string& m) {
    if (why != nullptr) *why = m;
    return false;
  };
  if (free_top_ < 0 || free_top_ > num_blocks_) return fail("free count out of range");
  std::vector<uint8_t> listed(static_cast<size_t>(num_blocks_), 0);
  for (int32_t i = 0; i < free_top_; ++i) {
    const BlockId id = free_[static_cast<size_t>(i)];
    if (!valid(id)) return fail("invalid id on the free stack");
    if (listed[static_cast<size_t>(id)]) return fail("block " + std::to_string(id) + " listed free twice");
    listed[static_cast<size_t>(id)] = 1;
    if (refs_[static_cast<size_t>(id)] != 0) return fail("free block " + std::to_string(id) + " has a ref count");
  }
  int32_t live = 0;
  for (int32_t id = 0; id < num_blocks_; ++id) {
    const int32_t r = refs_[static_cast<size_t>(id)];
    if (r < 0) return fail("negative ref count");
    if (r > 0) ++live;
    if (r == 0 && !listed[static_cast<size_t>(id)]) return fail("block " + std::to_string(id) + " lost: count 0 but not free");
  }
  if (live + free_top_ != num_blocks_) return fail("live + free != total");
  return true;
}

StateSlots::StateSlots(int32_t num_slots, int64_t bytes_per_slot)
    : num_slots_(num_slots), bytes_per_slot_(bytes_per_slot) {
  if (num_slots < 1 || num_slots > kMaxBlocks) throw std::invalid_argument("num_slots must be in [1, 2^26]");
  if (bytes_per_slot < 0) throw std::invalid_argument("bytes_per_slot must be >= 0");
  used_.assign(static_cast<size_t>(num_slots), 0);
  free_.reserve(static_cast<size_t>(num_slots));
  for (int32_t i = num_slots - 1; i >= 0; --i) free_.push_back(i);
}

}  // namespace psamd
