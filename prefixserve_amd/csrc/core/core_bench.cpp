// Times the host cache core's calls on the per-step path, without Python in between:
//
//  1. looking up a fully held 2,048-token prompt (128 pages) among 300 other held prompts and
//     dropping the pages again: the workload of the reference's own micro-benchmark
//     (bench/micro_core.cpp:1-66, whose bar is 10 microseconds a call);
//  2. taking and dropping 128 pages;
//  3. holding a finished 2,048-token prompt (all of its pages new to the index) and letting the
//     index give them back;
//  4. laying out and filling the integer buffer of a decode step of 64 requests of 4,096 tokens.
//
// Prints one line per measurement ("<name>: <ns> ns/call ...") and exits 0, or 1 if the lookup
// is over the reference's bar.

#include <chrono>
#include <cstdint>
#include <cstdio>
#include <vector>

#include "page_pool.hpp"
#include "prefix_tree.hpp"
#include "step_pack.hpp"

using namespace psamd;

namespace {

using Clock = std::chrono::steady_clock;

template <typename F>
double ns_per_call(int iters, F&& call) {
  for (int i = 0; i < iters / 20 + 1; ++i) call();
  const auto t0 = Clock::now();
  for (int i = 0; i < iters; ++i) call();
  return std::chrono::duration<double, std::nano>(Clock::now() - t0).count() / iters;
}

std::vector<int32_t> prompt(int64_t n, uint32_t salt) {
  std::vector<int32_t> t(static_cast<size_t>(n));
  for (int64_t i = 0; i < n; ++i)
    t[static_cast<size_t>(i)] = static_cast<int32_t>((static_cast<uint32_t>(i) * 2654435761u + salt * 40503u) % 50000u);
  return t;
}

}  // namespace

int main() {
  constexpr int64_t kTokens = 2048, kPages = kTokens / kBlockSize;
  PagePool pool(1 << 16);
  PrefixIndex index(pool, 12345);
  int64_t sink = 0;

  const std::vector<int32_t> toks = prompt(kTokens, 0);
  std::vector<BlockId> pages(static_cast<size_t>(kPages));
  if (!pool.take_many(static_cast<int32_t>(kPages), pages.data())) return 2;
  int32_t added = 0;
  if (index.hold(toks.data(), kTokens, pages.data(), kPages, &added) != Fault::kNone || added != kPages) return 2;
  for (BlockId id : pages) (void)pool.drop(id);
  // Other held prompts, so that the table is neither tiny nor all in the nearest cache.
  for (uint32_t p = 1; p <= 300; ++p) {
    const std::vector<int32_t> t = prompt(256, p);
    BlockId ids[16];
    if (!pool.take_many(16, ids)) return 2;
    (void)index.hold(t.data(), 256, ids, 16, &added);
    for (BlockId id : ids) (void)pool.drop(id);
  }

  std::vector<BlockId> out(static_cast<size_t>(kPages));
  const double lookup = ns_per_call(200000, [&] {
    const int64_t matched = index.lookup(toks.data(), kTokens, out.data());
    sink += matched;
    for (int64_t i = 0; i < matched / kBlockSize; ++i) (void)pool.drop(out[static_cast<size_t>(i)]);
  });
  std::printf("lookup of 2048 held tokens (128 pages) + drop: %.0f ns/call, %.1f ns/page (the reference's bar: 10000 ns/call)\n",
              lookup, lookup / static_cast<double>(kPages));

  const double take = ns_per_call(200000, [&] {
    if (pool.take_many(static_cast<int32_t>(kPages), out.data()))
      for (BlockId id : out) sink += static_cast<int64_t>(pool.drop(id) == Fault::kNone);
  });
  std::printf("take and drop 128 pages: %.0f ns/call, %.1f ns/page\n", take, take / static_cast<double>(kPages));

  uint32_t salt = 1000;
  const double hold = ns_per_call(20000, [&] {
    const std::vector<int32_t> t = prompt(kTokens, ++salt);          // (its cost is in the figure: about a tenth)
    if (!pool.take_many(static_cast<int32_t>(kPages), out.data())) return;
    int32_t took = 0;
    (void)index.hold(t.data(), kTokens, out.data(), kPages, &took);
    for (BlockId id : out) (void)pool.drop(id);
    sink += index.release_oldest(took);
  });
  std::printf("hold 2048 new tokens (128 pages) + give them back: %.0f ns/call, %.1f ns/page\n", hold,
              hold / static_cast<double>(kPages));

  // A decode step: 64 requests, one token each, behind 4,096 tokens (257 pages in each table).
  constexpr int64_t kRequests = 64, kContext = 4096, kTablePages = kContext / kBlockSize + 1;
  std::vector<std::vector<int64_t>> tables(static_cast<size_t>(kRequests));
  std::vector<int64_t> token{7}, want{0};
  std::vector<PackItem> items(static_cast<size_t>(kRequests));
  for (int64_t r = 0; r < kRequests; ++r) {
    auto& table = tables[static_cast<size_t>(r)];
    for (int64_t p = 0; p < kTablePages; ++p) table.push_back((r * kTablePages + p) % 60000);
    PackItem& it = items[static_cast<size_t>(r)];
    it.tokens = Span{token.data(), 1};
    it.start = kContext;
    it.slot = r;
    it.tables = {Span{table.data(), kTablePages}};
    it.want = Span{want.data(), 1};
  }
  const std::vector<PackGroup> groups{PackGroup{60000, -1}};
  PackLimits lim;
  lim.vocab_size = 128256;
  lim.max_position = 131072;
  lim.num_slots = kRequests;
  lim.prefill_tile = 32;
  std::vector<int32_t> buffer(static_cast<size_t>(plan_step(items, groups, lim).total));
  const double pack = ns_per_call(20000, [&] {
    const PackLayout lay = plan_step(items, groups, lim);
    fill_step(items, groups, lim, lay, buffer.data());
    sink += buffer[static_cast<size_t>(lay.token_ids)];
  });
  std::printf("lay out and fill a decode step of 64 requests x 257 pages: %.0f ns/call, %.0f ns/request\n", pack,
              pack / static_cast<double>(kRequests));

  return (sink > 0 && lookup < 10000.0) ? 0 : 1;
}
