// Python module prefixserve_amd._core: the host-side cache bookkeeping.
//
// The Python names and meanings are the reference's (prefixserve/_core.pyi:9-36,
// csrc/bindings.cpp:96-171): BLOCK_SIZE, CoreError, BlockManager, RadixTree; StateSlots is
// new. Inputs are borrowed for the length of a call; outputs are fresh Python lists, never
// views of memory the next call reuses.

#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <deque>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "block_pool.hpp"
#include "prefix_tree.hpp"
#include "step_pack.hpp"

namespace py = pybind11;
using namespace psamd;

namespace {

struct CoreError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

void expect_ok(Status s, const std::string& what) {
  if (s != Status::kOk) throw CoreError(what + ": " + status_name(s));
}

using Ints = py::array_t<int32_t, py::array::c_style | py::array::forcecast>;

const Ints& one_dim(const Ints& a, const char* name) {
  if (a.ndim() != 1) throw py::value_error(std::string(name) + " must be 1-D");
  return a;
}

py::list as_list(const BlockId* v, size_t n) {
  py::list out(n);
  for (size_t i = 0; i < n; ++i) out[i] = py::int_(v[i]);
  return out;
}

// The tree plus a result buffer sized once, so a match allocates nothing on this side.
class TreeHandle {
 public:
  TreeHandle(BlockPool& pool, py::object seed)
      : tree_(pool, seed.is_none() ? PrefixTree::random_seed() : seed.cast<uint64_t>()),
        found_(static_cast<size_t>(pool.num_blocks())) {}

  py::tuple match_prefix(const Ints& tokens) {
    one_dim(tokens, "tokens");
    // At most one page per pool page can match, whatever the prompt's length.
    const int64_t n = std::min<int64_t>(tokens.size(), static_cast<int64_t>(found_.size()) * kBlockSize);
    const int64_t matched = tree_.match_prefix(tokens.data(), n, found_.data());
    return py::make_tuple(matched, as_list(found_.data(), static_cast<size_t>(matched / kBlockSize)));
  }
  int32_t insert(const Ints& tokens, const Ints& blocks) {
    one_dim(tokens, "tokens");
    one_dim(blocks, "block_ids");
    int32_t added = 0;
    expect_ok(tree_.insert(tokens.data(), tokens.size(), blocks.data(), blocks.size(), &added), "insert");
    return added;
  }
  int32_t evict(int32_t n) {
    if (n < 0) throw py::value_error("num_blocks must be >= 0");
    return tree_.evict(n);
  }
  int32_t cached() const { return tree_.num_cached_blocks(); }
  bool is_cached(BlockId id) const { return tree_.is_cached(id); }
  void check() const {
    std::string why;
    if (!tree_.check_invariants(&why)) throw CoreError("RadixTree invariant broken: " + why);
  }

 private:
  PrefixTree tree_;
  std::vector<BlockId> found_;
};

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
                          lay.prefill_tiles, lay.pages, lay.max_kv_len,
                          py::make_tuple(lay.token_ids, lay.positions, lay.tok_item, lay.item_start, lay.item_pos0,
                                         lay.item_end, lay.slots, lay.logit_rows_off, lay.dec_items, lay.pf_tiles),
                          group_offsets);
  } catch (const PackError& e) {
    std::string who;
    if (e.item >= 0) who = py::str(items[static_cast<size_t>(e.item)].attr("key")).cast<std::string>() + ": ";
    throw py::value_error(who + e.what());
  }
}

}  // namespace

PYBIND11_MODULE(_core, m) {
  m.doc() = "Paged KV block manager, block-granular radix prefix cache and per-request state slots.";
  m.attr("BLOCK_SIZE") = kBlockSize;
  py::register_exception<CoreError>(m, "CoreError", PyExc_RuntimeError);

  py::class_<BlockPool>(m, "BlockManager")
      .def(py::init<int32_t>(), py::arg("num_blocks"))
      .def("allocate",
           [](BlockPool& p) -> py::object {
             const BlockId id = p.allocate();
             return id == kNoBlock ? py::object(py::none()) : py::object(py::int_(id));
           },
           "One block with ref_count 1, or None when the pool is empty.")
      .def("allocate_many",
           [](BlockPool& p, int32_t n) -> py::object {
             if (n < 0) throw py::value_error("n must be >= 0");
             if (p.num_free() < n) return py::none();  // all-or-nothing
             std::vector<BlockId> ids(static_cast<size_t>(n));
             (void)p.allocate_many(n, ids.data());
             return as_list(ids.data(), ids.size());
           },
           py::arg("n"), "n blocks, or None (nothing allocated) if fewer than n are free.")
      .def("incref", [](BlockPool& p, BlockId id) { expect_ok(p.incref(id), "incref"); }, py::arg("block_id"))
      .def("decref", [](BlockPool& p, BlockId id) { expect_ok(p.decref(id), "decref"); }, py::arg("block_id"))
      .def("decref_many",
           [](BlockPool& p, const Ints& ids) {
             one_dim(ids, "block_ids");
             const int32_t* v = ids.data();
             for (py::ssize_t i = 0; i < ids.size(); ++i) {
               const Status s = p.decref(v[i]);
               if (s != Status::kOk) {
                 throw CoreError("decref_many: block " + std::to_string(v[i]) + " at index " + std::to_string(i) +
                                 ": " + status_name(s));
               }
             }
           },
           py::arg("block_ids"))
      .def("ref_count",
           [](const BlockPool& p, BlockId id) {
             if (!p.valid(id)) expect_ok(Status::kInvalidBlockId, "ref_count");
             return p.ref_count(id);
           },
           py::arg("block_id"))
      .def_property_readonly("num_free", &BlockPool::num_free)
      .def_property_readonly("num_blocks", &BlockPool::num_blocks)
      .def("check_invariants", [](const BlockPool& p) {
        std::string why;
        if (!p.check_invariants(&why)) throw CoreError("BlockManager invariant broken: " + why);
      });

  py::class_<TreeHandle>(m, "RadixTree")
      // keep_alive: the tree points into the pool, so it keeps the pool's Python object alive.
      .def(py::init<BlockPool&, py::object>(), py::arg("block_manager"), py::arg("hash_seed") = py::none(),
           py::keep_alive<1, 2>())
      .def("match_prefix", &TreeHandle::match_prefix, py::arg("tokens"),
           "(matched_tokens, block_ids). Takes 1 ref per block for the caller.")
      .def("insert", &TreeHandle::insert, py::arg("tokens"), py::arg("block_ids"),
           "Caches full blocks. Returns how many new blocks the tree now holds.")
      .def("evict", &TreeHandle::evict, py::arg("num_blocks"),
           "Frees up to num_blocks unused blocks, LRU first. Returns how many were freed.")
      .def("is_cached", &TreeHandle::is_cached, py::arg("block_id"))
      .def_property_readonly("num_cached_blocks", &TreeHandle::cached)
      .def("check_invariants", &TreeHandle::check);

  m.def("pack_step", &pack_step, py::arg("buffer"), py::arg("items"), py::arg("groups"), py::arg("vocab_size"),
        py::arg("max_position"), py::arg("num_slots"), py::arg("prefill_tile"), py::arg("static_pages") = py::none(),
        "Checks a step's items and lays their integer arrays out in one buffer.");

  py::class_<StateSlots>(m, "StateSlots")
      .def(py::init<int32_t, int64_t>(), py::arg("num_slots"), py::arg("bytes_per_slot") = 0)
      .def("acquire",
           [](StateSlots& s) -> py::object {
             const int32_t id = s.acquire();
             return id < 0 ? py::object(py::none()) : py::object(py::int_(id));
           },
           "A free slot id, or None when every slot is taken.")
      .def("release", [](StateSlots& s, int32_t id) { expect_ok(s.release(id), "release"); }, py::arg("slot"))
      .def("in_use", &StateSlots::in_use, py::arg("slot"))
      .def_property_readonly("num_slots", &StateSlots::num_slots)
      .def_property_readonly("num_free", &StateSlots::num_free)
      .def_property_readonly("bytes_per_slot", &StateSlots::bytes_per_slot);
}
