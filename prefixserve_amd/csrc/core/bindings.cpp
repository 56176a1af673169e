// The Python module prefixserve_amd._core: the host side of the cache (page pool, prefix
// index, state slots) and the packing of a step's integers.
//
// Python sees the reference's names with the reference's meanings (prefixserve/_core.pyi:9-36,
// csrc/bindings.cpp:96-171): BLOCK_SIZE, CoreError, BlockManager, RadixTree. StateSlots and
// pack_step are additions. Arguments are only read during the call; results are new Python
// lists, never views of memory that a later call writes again.

#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <deque>
#include <stdexcept>
#include <string>
#include <vector>

#include "page_pool.hpp"
#include "prefix_tree.hpp"
#include "step_pack.hpp"

namespace py = pybind11;
using namespace psamd;

namespace {

// Misuse of the counts (a double free, an id out of range, ...) as a Python exception.
struct CoreError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

[[noreturn]] void raise_fault(const std::string& where, Fault f) { throw CoreError(where + ": " + describe(f)); }

void require(const std::string& where, Fault f) {
  if (f != Fault::kNone) raise_fault(where, f);
}

using IntArray = py::array_t<int32_t, py::array::c_style | py::array::forcecast>;

void require_flat(const IntArray& a, const char* what) {
  if (a.ndim() != 1) throw py::value_error(std::string(what) + " must be one-dimensional");
}

py::list python_list(const std::vector<BlockId>& ids, size_t count) {
  py::list result(count);
  for (size_t i = 0; i < count; ++i) result[i] = ids[i];
  return result;
}

// ---- BlockManager

py::object pool_allocate(PagePool& pool) {
  const BlockId id = pool.take();
  if (id == kNoBlock) return py::none();
  return py::int_(id);
}

py::object pool_allocate_many(PagePool& pool, int32_t n) {
  if (n < 0) throw py::value_error("cannot allocate a negative number of blocks");
  std::vector<BlockId> ids(static_cast<size_t>(n));
  if (!pool.take_many(n, ids.data())) return py::none();       // fewer than n free: nothing was taken
  return python_list(ids, ids.size());
}

void pool_decref_many(PagePool& pool, const IntArray& ids) {
  require_flat(ids, "block_ids");
  for (py::ssize_t i = 0; i < ids.size(); ++i) {
    const Fault f = pool.drop(ids.at(i));
    if (f != Fault::kNone)
      raise_fault("decref_many, block " + std::to_string(ids.at(i)) + " at index " + std::to_string(i), f);
  }
}

int32_t pool_ref_count(const PagePool& pool, BlockId id) {
  const int32_t owners = pool.owners(id);
  if (owners < 0) raise_fault("ref_count", Fault::kBadPage);
  return owners;
}

void pool_check(const PagePool& pool) {
  std::string why;
  if (!pool.check_invariants(&why)) throw CoreError("the block manager is inconsistent: " + why);
}

// ---- RadixTree: the index and a result buffer made once, so that a lookup allocates nothing
// but its Python result.

class Index {
 public:
  Index(PagePool& pool, const py::object& seed)
      : tree_(pool, seed.is_none() ? PrefixIndex::random_seed() : seed.cast<uint64_t>()),
        scratch_(static_cast<size_t>(pool.num_blocks())) {}

  py::tuple lookup(const IntArray& tokens) {
    require_flat(tokens, "tokens");
    // However long the prompt, no more pages can match than the pool has.
    const int64_t usable = std::min<int64_t>(tokens.size(), static_cast<int64_t>(scratch_.size()) * kBlockSize);
    const int64_t matched = tree_.lookup(tokens.data(), usable, scratch_.data());
    return py::make_tuple(matched, python_list(scratch_, static_cast<size_t>(matched / kBlockSize)));
  }

  int32_t insert(const IntArray& tokens, const IntArray& pages) {
    require_flat(tokens, "tokens");
    require_flat(pages, "block_ids");
    int32_t added = 0;
    require("insert", tree_.hold(tokens.data(), tokens.size(), pages.data(), pages.size(), &added));
    return added;
  }

  int32_t evict(int32_t count) {
    if (count < 0) throw py::value_error("cannot evict a negative number of blocks");
    return tree_.release_oldest(count);
  }

  bool is_cached(BlockId id) const { return tree_.holds(id); }
  int32_t num_cached_blocks() const { return tree_.size(); }

  void check() const {
    std::string why;
    if (!tree_.consistent(&why)) throw CoreError("the prefix tree is inconsistent: " + why);
  }

 private:
  PrefixIndex tree_;
  std::vector<BlockId> scratch_;
};

// ---- pack_step

using Longs = py::array_t<int64_t, py::array::c_style | py::array::forcecast>;

// Integer sequences of a call as 64-bit spans: arrays are borrowed (converted if their type
// differs), lists and tuples are copied. Everything lives until the holder dies.
struct Borrowed {
  std::vector<Longs> arrays;
  std::deque<std::vector<int64_t>> copies;

  Span of(const py::handle& seq, const char* name) {
    PyObject* o = seq.ptr();
    if (PyList_Check(o) || PyTuple_Check(o)) {
      const Py_ssize_t n = PySequence_Fast_GET_SIZE(o);
      PyObject** elems = PySequence_Fast_ITEMS(o);
      std::vector<int64_t>& v = copies.emplace_back(static_cast<size_t>(n));
      for (Py_ssize_t i = 0; i < n; ++i) {
        v[static_cast<size_t>(i)] = PyLong_AsLongLong(elems[i]);
        if (v[static_cast<size_t>(i)] == -1 && PyErr_Occurred()) {
          PyErr_Clear();
          // Not plain Python integers (numpy scalars, say): let numpy convert the lot.
          copies.pop_back();
          return of_array(seq, name);
        }
      }
      return Span{v.data(), static_cast<int64_t>(n)};
    }
    return of_array(seq, name);
  }

  Span of_array(const py::handle& seq, const char* name) {
    Longs a = Longs::ensure(seq);
    if (!a) {
      PyErr_Clear();
      throw py::value_error(std::string(name) + " must be a sequence of integers");
    }
    if (a.ndim() != 1) a = a.attr("reshape")(-1).cast<Longs>();
    arrays.push_back(a);
    return Span{a.data(), static_cast<int64_t>(a.size())};
  }
};

// pack_step(buffer, items, groups, vocab_size, max_position, num_slots, prefill_tile,
// static_pages) -> None if the buffer is too small, in which case only the first number
// of the result counts, else the layout as a tuple of integers.
py::tuple pack_step(py::array_t<int32_t, py::array::c_style> buffer, const py::sequence& items,
                    const std::vector<std::pair<int64_t, py::object>>& groups, int64_t vocab_size,
                    int64_t max_position, int64_t num_slots, int64_t prefill_tile, const py::object& static_pages) {
  std::vector<PackGroup> gs;
  for (const auto& g : groups) gs.push_back(PackGroup{g.first, g.second.is_none() ? -1 : g.second.cast<int64_t>()});
  PackLimits lim;
  lim.vocab_size = vocab_size;
  lim.max_position = max_position;
  lim.num_slots = num_slots;
  lim.prefill_tile = prefill_tile;
  lim.static_pages = static_pages.is_none() ? -1 : static_pages.cast<int64_t>();

  Borrowed keep;
  std::vector<PackItem> its;
  const size_t n_items = py::len(items);
  its.reserve(n_items);
  keep.arrays.reserve(n_items * (2 + gs.size()));
  // Attribute names as Python strings made once: this runs for every item of every step.
  // They are never released: a static object's destructor would run after the interpreter.
  static const py::handle k_tokens = py::str("tokens").release(), k_start = py::str("start").release(),
                          k_slot = py::str("slot").release(), k_tables = py::str("block_tables").release(),
                          k_want = py::str("want").release();
  for (const py::handle& obj : items) {
    PackItem it;
    it.tokens = keep.of(obj.attr(k_tokens), "tokens");
    it.start = obj.attr(k_start).cast<int64_t>();
    it.slot = obj.attr(k_slot).cast<int64_t>();
    it.tables.reserve(gs.size());
    for (const py::handle& table : obj.attr(k_tables)) it.tables.push_back(keep.of(table, "a block table"));
    it.want = keep.of(obj.attr(k_want), "want");
    its.push_back(std::move(it));
  }
  try {
    const PackLayout lay = plan_step(its, gs, lim);
    const bool fits = lay.total <= buffer.size();
    if (fits) fill_step(its, gs, lim, lay, buffer.mutable_data());
    py::list group_offsets;
    for (const GroupLayout& g : lay.groups) group_offsets.append(py::make_tuple(g.table_off, g.write_slot, g.block_ids));
    return py::make_tuple(fits, lay.total, lay.tokens, lay.items, lay.logit_rows, lay.decode_items,
                          lay.prefill_tiles, lay.prefill_blocks, lay.pages, lay.max_kv_len, lay.decode_max_kv,
                          lay.decode_sum_kv,
                          py::make_tuple(lay.token_ids, lay.positions, lay.tok_item, lay.item_start, lay.item_pos0,
                                         lay.item_end, lay.slots, lay.logit_rows_off, lay.dec_items, lay.pf_tiles,
                                         lay.pf_blocks),
                          group_offsets);
  } catch (const PackError& e) {
    std::string who;
    if (e.item >= 0) who = py::str(items[static_cast<size_t>(e.item)].attr("key")).cast<std::string>() + ": ";
    throw py::value_error(who + e.what());
  }
}

}  // namespace

PYBIND11_MODULE(_core, m) {
  m.doc() = "Host side of the paged KV cache: page pool, prefix index, state slots, step packing.";
  m.attr("BLOCK_SIZE") = kBlockSize;
  py::register_exception<CoreError>(m, "CoreError", PyExc_RuntimeError);

  py::class_<PagePool> pool(m, "BlockManager");
  pool.def(py::init<int32_t>(), py::arg("num_blocks"));
  pool.def("allocate", &pool_allocate, "A block with one reference, or None if none is free.");
  pool.def("allocate_many", &pool_allocate_many, py::arg("n"), "n blocks, or None and nothing taken.");
  pool.def("incref", [](PagePool& p, BlockId id) { require("incref", p.share(id)); }, py::arg("block_id"));
  pool.def("decref", [](PagePool& p, BlockId id) { require("decref", p.drop(id)); }, py::arg("block_id"));
  pool.def("decref_many", &pool_decref_many, py::arg("block_ids"));
  pool.def("ref_count", &pool_ref_count, py::arg("block_id"));
  pool.def_property_readonly("num_free", &PagePool::num_free);
  pool.def_property_readonly("num_blocks", &PagePool::num_blocks);
  pool.def("check_invariants", &pool_check);

  py::class_<Index> index(m, "RadixTree");
  // The index points into the pool: it keeps the pool's Python object alive.
  index.def(py::init<PagePool&, const py::object&>(), py::arg("block_manager"), py::arg("hash_seed") = py::none(),
            py::keep_alive<1, 2>());
  index.def("match_prefix", &Index::lookup, py::arg("tokens"),
            "(matched tokens, block ids); the caller holds one reference on each block.");
  index.def("insert", &Index::insert, py::arg("tokens"), py::arg("block_ids"),
            "Holds the full blocks of tokens; returns how many it took.");
  index.def("evict", &Index::evict, py::arg("num_blocks"), "Frees up to num_blocks blocks nobody uses, oldest first.");
  index.def("is_cached", &Index::is_cached, py::arg("block_id"));
  index.def_property_readonly("num_cached_blocks", &Index::num_cached_blocks);
  index.def("check_invariants", &Index::check);

  py::class_<StateSlots> slots(m, "StateSlots");
  slots.def(py::init<int32_t, int64_t>(), py::arg("num_slots"), py::arg("bytes_per_slot") = 0);
  slots.def("acquire", [](StateSlots& s) -> py::object {
    const int32_t id = s.acquire();
    if (id < 0) return py::none();
    return py::int_(id);
  }, "A free slot, or None if all are taken.");
  slots.def("release", [](StateSlots& s, int32_t slot) { require("release", s.release(slot)); }, py::arg("slot"));
  slots.def("in_use", &StateSlots::in_use, py::arg("slot"));
  slots.def_property_readonly("num_slots", &StateSlots::num_slots);
  slots.def_property_readonly("num_free", &StateSlots::num_free);
  slots.def_property_readonly("bytes_per_slot", &StateSlots::bytes_per_slot);

  m.def("pack_step", &pack_step, py::arg("buffer"), py::arg("items"), py::arg("groups"), py::arg("vocab_size"),
        py::arg("max_position"), py::arg("num_slots"), py::arg("prefill_tile"), py::arg("static_pages") = py::none(),
        "Checks a step's items and lays their integer arrays out in one buffer.");
}
