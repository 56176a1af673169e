#include "prefix_tree.hpp"

#include <cstring>
#include <random>

namespace psamd {

namespace {

size_t buckets_for(int32_t entries) {
  size_t n = 16;
  while (n < 2 * static_cast<size_t>(entries)) n <<= 1;
  return n;
}

}  // namespace

PrefixIndex::PrefixIndex(PagePool& pool, uint64_t seed) : pool_(pool), seed_(seed) {
  const int32_t pages = pool.num_blocks();
  entry_.resize(static_cast<size_t>(pages) + 1);
  text_.assign((static_cast<size_t>(pages) + 1) * kBlockSize, 0);
  bucket_.assign(buckets_for(pages + 1), kNil);
  shared_.assign(static_cast<size_t>(pages), 0);
  seen_in_call_.assign(static_cast<size_t>(pages), 0);
  unused_.reserve(static_cast<size_t>(pages));
  for (Ref e = pages; e >= 1; --e) unused_.push_back(e);      // entry 1 is used first
}

PrefixIndex::~PrefixIndex() {
  for (Ref e = oldest_; e != kNil; e = entry_[static_cast<size_t>(e)].younger)
    pool_.drop(entry_[static_cast<size_t>(e)].page);
}

uint64_t PrefixIndex::random_seed() {
  std::random_device device;
  return (static_cast<uint64_t>(device()) << 32) ^ device();
}

// Two tokens at a time through a multiply-and-fold; the prefix enters through the start value.
// Quality only matters for speed: a hit is confirmed by comparing the tokens.
uint64_t PrefixIndex::hash_of(Ref parent, const int32_t* t) const noexcept {
  uint64_t h = seed_ + 0x9E3779B97F4A7C15ull * (static_cast<uint64_t>(parent) + 1);
  for (int i = 0; i < kBlockSize; i += 2) {
    const uint64_t two = static_cast<uint32_t>(t[i]) | (static_cast<uint64_t>(static_cast<uint32_t>(t[i + 1])) << 32);
    h = (h ^ two) * 0xD6E8FEB86659FD93ull;
    h ^= h >> 32;
  }
  return h;
}

PrefixIndex::Ref PrefixIndex::find(Ref parent, const int32_t* t, uint64_t h) const noexcept {
  for (Ref e = bucket_[h & (bucket_.size() - 1)]; e != kNil; e = entry_[static_cast<size_t>(e)].same_bucket) {
    const Entry& x = entry_[static_cast<size_t>(e)];
    if (x.hash == h && x.parent == parent && std::memcmp(text(e), t, sizeof(int32_t) * kBlockSize) == 0) return e;
  }
  return kNil;
}

void PrefixIndex::unlink_recency(Ref e) noexcept {
  Entry& x = entry_[static_cast<size_t>(e)];
  if (x.older != kNil) entry_[static_cast<size_t>(x.older)].younger = x.younger; else oldest_ = x.younger;
  if (x.younger != kNil) entry_[static_cast<size_t>(x.younger)].older = x.older; else youngest_ = x.older;
  x.older = x.younger = kNil;
}

void PrefixIndex::make_youngest(Ref e) noexcept {
  Entry& x = entry_[static_cast<size_t>(e)];
  x.older = youngest_;
  x.younger = kNil;
  if (youngest_ != kNil) entry_[static_cast<size_t>(youngest_)].younger = e; else oldest_ = e;
  youngest_ = e;
}

void PrefixIndex::used(Ref deepest) noexcept {
  for (Ref e = deepest; e != kTop; e = entry_[static_cast<size_t>(e)].parent) {
    unlink_recency(e);
    make_youngest(e);
  }
}

int64_t PrefixIndex::lookup(const int32_t* tokens, int64_t n, BlockId* out) noexcept {
  const int64_t full = n / kBlockSize;
  Ref at = kTop;
  int64_t matched = 0;
  for (; matched < full; ++matched) {
    const int32_t* t = tokens + matched * kBlockSize;
    const Ref next = find(at, t, hash_of(at, t));
    if (next == kNil) break;
    const BlockId page = entry_[static_cast<size_t>(next)].page;
    if (pool_.share(page) != Fault::kNone) break;          // owner count at its limit: stop here
    out[matched] = page;
    at = next;
  }
  used(at);
  return matched * kBlockSize;
}

Fault PrefixIndex::hold(const int32_t* tokens, int64_t n, const BlockId* pages, int64_t num_pages,
                         int32_t* added) noexcept {
  if (added != nullptr) *added = 0;
  const int64_t full = n / kBlockSize;
  if (n < 0 || num_pages < full) return Fault::kBadArgument;
  // What is held already.
  Ref at = kTop;
  int64_t known = 0;
  for (; known < full; ++known) {
    const int32_t* t = tokens + known * kBlockSize;
    const Ref next = find(at, t, hash_of(at, t));
    if (next == kNil) break;
    at = next;
  }
  // Every new page is looked at before anything changes.
  if (static_cast<int64_t>(unused_.size()) < full - known) return Fault::kIndexFull;
  if (++call_ == 0) {                                        // the counter wrapped: old marks mean nothing now
    std::fill(seen_in_call_.begin(), seen_in_call_.end(), 0u);
    call_ = 1;
  }
  for (int64_t i = known; i < full; ++i) {
    const BlockId page = pages[i];
    const int32_t owners = pool_.owners(page);
    if (owners < 0) return Fault::kBadPage;
    if (owners == 0) return Fault::kNotInUse;
    if (owners == INT32_MAX) return Fault::kTooManyOwners;
    if (shared_[static_cast<size_t>(page)] || seen_in_call_[static_cast<size_t>(page)] == call_)
      return Fault::kAlreadyShared;                          // held elsewhere, or given twice in this call
    seen_in_call_[static_cast<size_t>(page)] = call_;
  }
  for (int64_t i = known; i < full; ++i) {
    const int32_t* t = tokens + i * kBlockSize;
    const Ref e = unused_.back();
    unused_.pop_back();
    Entry& x = entry_[static_cast<size_t>(e)];
    x.parent = at;
    x.page = pages[i];
    x.continuations = 0;
    x.hash = hash_of(at, t);
    std::memcpy(&text_[static_cast<size_t>(e) * kBlockSize], t, sizeof(int32_t) * kBlockSize);
    Ref& head = bucket_[x.hash & (bucket_.size() - 1)];
    x.same_bucket = head;
    head = e;
    entry_[static_cast<size_t>(at)].continuations += 1;
    pool_.share(x.page);
    shared_[static_cast<size_t>(x.page)] = 1;
    make_youngest(e);
    at = e;
  }
  held_ += static_cast<int32_t>(full - known);
  if (added != nullptr) *added = static_cast<int32_t>(full - known);
  used(at);                                                  // new pages, then their prefix, youngest last
  return Fault::kNone;
}

void PrefixIndex::forget(Ref leaf) noexcept {
  Entry& x = entry_[static_cast<size_t>(leaf)];
  unlink_recency(leaf);
  Ref* link = &bucket_[x.hash & (bucket_.size() - 1)];
  while (*link != leaf) link = &entry_[static_cast<size_t>(*link)].same_bucket;
  *link = x.same_bucket;
  entry_[static_cast<size_t>(x.parent)].continuations -= 1;
  shared_[static_cast<size_t>(x.page)] = 0;
  pool_.drop(x.page);
  x = Entry{};
  unused_.push_back(leaf);
  --held_;
}

int32_t PrefixIndex::release_oldest(int32_t want) noexcept {
  int32_t freed = 0;
  // From the old end. An entry stands before its ancestors, so a prefix whose last
  // continuation goes is met later in the same walk.
  for (Ref e = oldest_; e != kNil && freed < want;) {
    const Ref next = entry_[static_cast<size_t>(e)].younger;
    const Entry& x = entry_[static_cast<size_t>(e)];
    if (x.continuations == 0 && pool_.owners(x.page) == 1) {
      forget(e);
      ++freed;
    }
    e = next;
  }
  return freed;
}

bool PrefixIndex::consistent(std::string* why) const {
  auto broken = [why](std::string what) {
    if (why != nullptr) *why = std::move(what);
    return false;
  };
  const size_t n = entry_.size();
  std::vector<int32_t> place(n, -1), kids(n, 0);
  int32_t count = 0;
  Ref before = kNil;
  for (Ref e = oldest_; e != kNil; e = entry_[static_cast<size_t>(e)].younger) {
    if (e <= kTop || static_cast<size_t>(e) >= n) return broken("the recency list leaves the entries");
    if (place[static_cast<size_t>(e)] >= 0) return broken("an entry is in the recency list twice");
    if (entry_[static_cast<size_t>(e)].older != before) return broken("recency links disagree");
    place[static_cast<size_t>(e)] = count++;
    before = e;
  }
  if (before != youngest_) return broken("the young end of the recency list is wrong");
  if (count != held_) return broken("held count and recency list disagree");
  if (static_cast<size_t>(held_) + unused_.size() + 1 != n) return broken("entries in use + unused != all");
  int32_t marks = 0;
  for (uint8_t m : shared_) marks += m;
  if (marks != held_) return broken("page marks and entries disagree");
  for (size_t e = 1; e < n; ++e) {
    if (place[e] < 0) continue;
    const Entry& x = entry_[e];
    if (x.parent != kTop && (x.parent < 0 || place[static_cast<size_t>(x.parent)] < 0))
      return broken("an entry continues a prefix that is not held");
    if (x.parent != kTop && place[static_cast<size_t>(x.parent)] < place[e])
      return broken("an entry stands after its prefix in the recency list");
    kids[static_cast<size_t>(x.parent)] += 1;
    if (!pool_.valid(x.page) || !shared_[static_cast<size_t>(x.page)]) return broken("an entry's page is not marked");
    if (pool_.owners(x.page) < 1) return broken("the index holds a page that has no owner");
    if (x.hash != hash_of(x.parent, text(static_cast<Ref>(e)))) return broken("a stored hash is stale");
    if (find(x.parent, text(static_cast<Ref>(e)), x.hash) != static_cast<Ref>(e))
      return broken("an entry cannot be found through its bucket");
  }
  for (size_t e = 0; e < n; ++e) {
    if ((e == 0 || place[e] >= 0) && entry_[e].continuations != kids[e]) return broken("a continuation count is wrong");
  }
  return true;
}

}  // namespace psamd
