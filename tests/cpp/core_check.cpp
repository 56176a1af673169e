// A check of the host cache core that runs without Python, built twice by the tests: plain,
// and with the address and undefined-behaviour sanitizers (every warning an error in both).
//
// 1. No allocation on the per-step path. The global operator new is replaced by one that
//    counts; after construction, taking / sharing / dropping pages, looking up, holding and
//    evicting prefixes, taking and returning state slots, and filling a step's integer
//    buffer must not allocate at all (the reference checks its own core the same way,
//    tests/cpp/test_no_alloc.cpp:79-144, self-test of the counter included). plan_step
//    returns its per-group offsets in a vector: one allocation per call, counted here so
//    that a second one would show.
// 2. A random workload of requests over a small pool against a model of the counts kept in
//    this file: no page lost, held twice or freed twice, the index and the pool agree after
//    every operation. Under the sanitizers this is also the run that would show a read or
//    write outside the core's arrays.
//
// Prints "ok: ..." lines and exits 0, or prints what failed and exits 1.

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <new>
#include <string>
#include <vector>

#include "page_pool.hpp"
#include "prefix_tree.hpp"
#include "step_pack.hpp"

namespace {
long g_news = 0;
}

// noinline: inlined, the compiler sees malloc paired with a delete expression and warns.
#define KEEP_OUT __attribute__((noinline))

KEEP_OUT void* operator new(std::size_t n) {
  ++g_news;
  void* p = std::malloc(n ? n : 1);
  if (p == nullptr) throw std::bad_alloc();
  return p;
}
KEEP_OUT void* operator new[](std::size_t n) {
  ++g_news;
  void* p = std::malloc(n ? n : 1);
  if (p == nullptr) throw std::bad_alloc();
  return p;
}
KEEP_OUT void operator delete(void* p) noexcept { std::free(p); }
KEEP_OUT void operator delete[](void* p) noexcept { std::free(p); }
KEEP_OUT void operator delete(void* p, std::size_t) noexcept { std::free(p); }
KEEP_OUT void operator delete[](void* p, std::size_t) noexcept { std::free(p); }

using namespace psamd;

namespace {

int g_failures = 0;

void expect(bool cond, const char* what, int line) {
  if (!cond) {
    std::printf("FAILED line %d: %s\n", line, what);
    ++g_failures;
  }
}
#define EXPECT(c) expect((c), #c, __LINE__)

struct Rng {
  uint64_t s;
  uint32_t next() {
    s = s * 6364136223846793005ULL + 1442695040888963407ULL;
    return static_cast<uint32_t>(s >> 33);
  }
  int32_t below(int32_t n) { return static_cast<int32_t>(next() % static_cast<uint32_t>(n)); }
};

// ---------------------------------------------------------------- 1. allocation counting

void counter_counts() {
  const long before = g_news;
  int* p = new int(3);
  std::vector<int>* v = new std::vector<int>(10);
  const long seen = g_news - before;
  delete p;
  delete v;
  EXPECT(seen == 3);                       // the int, the vector object, its storage
  std::printf("ok: the counter counts (%ld allocations seen for 3 made)\n", seen);
}

void hot_paths_do_not_allocate() {
  constexpr int32_t kPages = 96;
  PagePool pool(kPages);
  PrefixIndex index(pool, 1234);
  StateSlots slots(8, 64);
  std::vector<int32_t> tokens(20 * kBlockSize);
  std::vector<BlockId> pages(kPages), found(kPages);
  Rng rng{7};
  // Step packing: operands prepared before the counted region, as the engine keeps them.
  std::vector<int64_t> toks64(40), table64(8), want64(1, 0);
  for (size_t i = 0; i < toks64.size(); ++i) toks64[i] = static_cast<int64_t>(i % 50);
  for (size_t i = 0; i < table64.size(); ++i) table64[i] = static_cast<int64_t>(i);
  std::vector<PackItem> items(2);
  items[0].tokens = Span{toks64.data(), 40};
  items[0].start = 16;
  items[0].tables = {Span{table64.data(), 8}};
  items[0].want = Span{want64.data(), 1};
  items[1].tokens = Span{toks64.data(), 1};
  items[1].start = 70;
  items[1].slot = 1;
  items[1].tables = {Span{table64.data(), 8}};
  items[1].want = Span{want64.data(), 1};
  std::vector<PackGroup> groups(1);
  groups[0].num_blocks = kPages;
  PackLimits lim;
  lim.vocab_size = 50;
  lim.max_position = 128;
  lim.num_slots = 8;
  lim.prefill_tile = 32;
  std::vector<int32_t> buf(4096);

  const long before = g_news;
  long plan_news = 0;
  for (int round = 0; round < 200; ++round) {
    for (int32_t& t : tokens) t = rng.below(3);                   // few distinct tokens: prefixes repeat
    const int32_t n_pages = 1 + rng.below(20);
    const int64_t n_tok = static_cast<int64_t>(n_pages) * kBlockSize;
    const int64_t hit = index.lookup(tokens.data(), n_tok, found.data());
    const int32_t have = static_cast<int32_t>(hit / kBlockSize);
    const int32_t need = n_pages - have;
    if (pool.num_free() < need) index.release_oldest(need - pool.num_free());
    if (pool.take_many(need, pages.data())) {
      // the request's table: matched pages first, then its own
      std::vector<BlockId>& all = found;                          // reuse: [0, have) are the matched ones already
      for (int32_t i = 0; i < need; ++i) all[static_cast<size_t>(have + i)] = pages[static_cast<size_t>(i)];
      int32_t added = 0;
      EXPECT(index.hold(tokens.data(), n_tok, all.data(), n_pages, &added) == Fault::kNone);
      EXPECT(pool.share(all[0]) == Fault::kNone);
      EXPECT(pool.drop(all[0]) == Fault::kNone);
      for (int32_t i = 0; i < n_pages; ++i) EXPECT(pool.drop(all[static_cast<size_t>(i)]) == Fault::kNone);
    } else {
      for (int32_t i = 0; i < have; ++i) EXPECT(pool.drop(found[static_cast<size_t>(i)]) == Fault::kNone);
    }
    const int32_t s = slots.acquire();
    EXPECT(s >= 0 && slots.release(s) == Fault::kNone);
    EXPECT(pool.drop(kPages + 5) == Fault::kBadPage);             // a refusal does not allocate either
    const long p0 = g_news;
    const PackLayout lay = plan_step(items, groups, lim);
    plan_news += g_news - p0;
    fill_step(items, groups, lim, lay, buf.data());
  }
  const long total = g_news - before;
  EXPECT(plan_news == 200);                                       // the per-group offsets of each plan, nothing else
  EXPECT(total - plan_news == 0);
  std::string why;
  EXPECT(pool.check_invariants(&why));
  EXPECT(index.consistent(&why));
  std::printf("ok: 200 rounds of lookup/take/hold/share/drop/evict/slots/fill_step allocated %ld times "
              "(plan_step: %ld, one per call)\n", total - plan_news, plan_news);
}

// ---------------------------------------------------------------- 2. random workload against a model

struct Live {
  std::vector<BlockId> pages;
  std::vector<int32_t> tokens;
  int32_t slot;
};

// The model: how many live requests hold each page, and which pages the index held when it
// was last asked. A page's owners in the pool must be the sum of the two at every moment.
struct Model {
  std::vector<int32_t> requests;
  std::vector<uint8_t> indexed;
  explicit Model(int32_t pages) : requests(static_cast<size_t>(pages), 0), indexed(static_cast<size_t>(pages), 0) {}
  // Brings `indexed` up to date; returns (pages newly held) - (pages given up).
  int32_t refresh(const PrefixIndex& index) {
    int32_t change = 0;
    for (size_t p = 0; p < indexed.size(); ++p) {
      const uint8_t now = index.holds(static_cast<BlockId>(p)) ? 1 : 0;
      change += static_cast<int32_t>(now) - static_cast<int32_t>(indexed[p]);
      indexed[p] = now;
    }
    return change;
  }
  int32_t owners(BlockId p) const { return requests[static_cast<size_t>(p)] + indexed[static_cast<size_t>(p)]; }
};

void random_workload(uint64_t seed) {
  constexpr int32_t kPages = 40;
  PagePool pool(kPages);
  StateSlots slots(6, 0);
  Model model(kPages);
  std::vector<Live> live;
  std::string why;
  Rng rng{seed};
  long evicted = 0, hits = 0, refused = 0;
  {
    PrefixIndex index(pool, seed * 977 + 1);
    std::vector<BlockId> got(kPages);
    for (int op = 0; op < 4000; ++op) {
      const int32_t what = rng.below(10);
      if (what < 5 && live.size() < 6) {          // a request arrives
        Live r;
        const int32_t n_pages = 1 + rng.below(9);
        r.tokens.resize(static_cast<size_t>(n_pages * kBlockSize + rng.below(kBlockSize)));
        // One of three families up to a random depth (so that prefixes are found again), then its own tokens.
        const int32_t family = rng.below(3), shared = rng.below(n_pages + 1) * kBlockSize;
        for (size_t i = 0; i < r.tokens.size(); ++i)
          r.tokens[i] = static_cast<int32_t>(i) < shared ? family * 100 + static_cast<int32_t>(i % 7) : 1000 + rng.below(500);
        const int64_t n = static_cast<int64_t>(r.tokens.size());
        const int64_t hit = index.lookup(r.tokens.data(), n, got.data());
        EXPECT(hit % kBlockSize == 0 && hit <= n);
        const int32_t have = static_cast<int32_t>(hit / kBlockSize);
        hits += have;
        for (int32_t i = 0; i < have; ++i) {
          EXPECT(index.holds(got[static_cast<size_t>(i)]));
          model.requests[static_cast<size_t>(got[static_cast<size_t>(i)])] += 1;
        }
        r.pages.assign(got.begin(), got.begin() + have);
        const int32_t need = static_cast<int32_t>((n + kBlockSize - 1) / kBlockSize) - have;
        if (pool.num_free() < need) {
          const int32_t free_before = pool.num_free();
          const int32_t gone = index.release_oldest(need - free_before);
          EXPECT(pool.num_free() == free_before + gone);
          EXPECT(model.refresh(index) == -gone);
          evicted += gone;
        }
        std::vector<BlockId> fresh(static_cast<size_t>(need));
        const int32_t free_before = pool.num_free();
        if (pool.take_many(need, fresh.data())) {
          for (BlockId p : fresh) {
            EXPECT(pool.valid(p) && model.owners(p) == 0);                    // never a page somebody holds
            model.requests[static_cast<size_t>(p)] = 1;
            r.pages.push_back(p);
          }
          r.slot = slots.acquire();
          EXPECT(r.slot >= 0);
          live.push_back(r);
        } else {
          ++refused;
          EXPECT(pool.num_free() == free_before);                             // all or nothing
          for (BlockId p : r.pages) {
            EXPECT(pool.drop(p) == Fault::kNone);
            model.requests[static_cast<size_t>(p)] -= 1;
          }
        }
      } else if (!live.empty()) {                 // a request ends: its full pages go to the index, then it lets go
        const size_t k = static_cast<size_t>(rng.below(static_cast<int32_t>(live.size())));
        Live r = live[k];
        live.erase(live.begin() + static_cast<std::ptrdiff_t>(k));
        if (rng.below(4) != 0) {
          const int64_t full = static_cast<int64_t>(r.tokens.size()) / kBlockSize;
          int32_t added = 0;
          EXPECT(index.hold(r.tokens.data(), static_cast<int64_t>(r.tokens.size()), r.pages.data(), full, &added) == Fault::kNone);
          EXPECT(model.refresh(index) == added);
        }
        for (BlockId p : r.pages) {
          EXPECT(pool.drop(p) == Fault::kNone);
          model.requests[static_cast<size_t>(p)] -= 1;
        }
        EXPECT(slots.release(r.slot) == Fault::kNone);
        EXPECT(slots.release(r.slot) != Fault::kNone);                         // a second release is refused
      }
      int32_t free_model = 0;
      for (int32_t p = 0; p < kPages; ++p) {
        EXPECT(pool.owners(p) == model.owners(p));
        free_model += model.owners(p) == 0;
      }
      EXPECT(pool.num_free() == free_model);
      if (op % 64 == 0) {
        EXPECT(pool.check_invariants(&why));
        EXPECT(index.consistent(&why));
      }
      if (g_failures) return;
    }
    for (int32_t p = 0; p < kPages; ++p)          // a page that is free cannot be dropped again
      if (model.owners(p) == 0) {
        EXPECT(pool.drop(p) == Fault::kNotInUse);
        break;
      }
    for (const Live& r : live)
      for (BlockId p : r.pages) EXPECT(pool.drop(p) == Fault::kNone);
  }                                               // the index returns what it owns
  EXPECT(pool.num_free() == kPages);
  EXPECT(pool.check_invariants(&why));
  EXPECT(evicted > 0 && hits > 0);                // the workload reached eviction and prefix hits
  std::printf("ok: random workload, seed %llu: %ld pages found in the index, %ld evicted, %ld arrivals refused\n",
              static_cast<unsigned long long>(seed), hits, evicted, refused);
}

}  // namespace

int main() {
  counter_counts();
  hot_paths_do_not_allocate();
  for (uint64_t seed = 1; seed <= 5 && g_failures == 0; ++seed) random_workload(seed);
  if (g_failures) {
    std::printf("%d check(s) failed\n", g_failures);
    return 1;
  }
  std::printf("all core checks passed\n");
  return 0;
}
