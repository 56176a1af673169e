"""Host-side cache bookkeeping: page pool, prefix tree, state slots, cache manager.

The behaviours and vectors are those of the reference's tests (tests/cpp/test_core.cpp:64-389,
tests/test_core_bindings.py:29-178); the randomized tests check that no page is lost, held
twice or freed twice under random orders of requests."""

from __future__ import annotations

import random

import numpy as np
import pytest

from prefixserve_amd.cache import BLOCK_SIZE, BlockManager, CacheManager, CoreError, RadixTree, StateSlots


def seq(n, start=0):
    return np.arange(start, start + n, dtype=np.int32)


def prefill(bm, tree, toks):
    """What a request does: match, allocate the rest, insert. Returns the blocks it holds."""
    matched, held = tree.match_prefix(toks)
    need = -(-len(toks) // BLOCK_SIZE) - len(held)
    new = bm.allocate_many(need)
    assert new is not None
    held = held + new
    tree.insert(toks, held)
    return held


def match_len(bm, tree, toks):
    n, ids = tree.match_prefix(toks)
    bm.decref_many(ids)
    return n


def ok(bm, tree):
    bm.check_invariants()
    tree.check_invariants()


# ------------------------------------------------------------- block manager

def test_block_manager_sizes_and_order():
    assert BLOCK_SIZE == 16
    for bad in (0, -5, (1 << 26) + 1):
        with pytest.raises(ValueError):
            BlockManager(bad)
    bm = BlockManager(4)
    assert [bm.allocate() for _ in range(4)] == [0, 1, 2, 3]      # first ids in order
    assert bm.allocate() is None and bm.num_free == 0
    assert all(bm.ref_count(i) == 1 for i in range(4))


def test_ref_counting_and_double_free():
    bm = BlockManager(2)
    b = bm.allocate()
    bm.incref(b)
    assert bm.ref_count(b) == 2
    bm.decref(b)
    assert bm.num_free == 1
    bm.decref(b)
    assert bm.num_free == 2
    with pytest.raises(CoreError, match="double free"):
        bm.decref(b)
    assert bm.num_free == 2                                        # not listed twice
    with pytest.raises(CoreError):
        bm.incref(b)
    for bad in (-1, 2, 99):
        with pytest.raises(CoreError, match="invalid block id"):
            bm.decref(bad)
        with pytest.raises(CoreError):
            bm.ref_count(bad)
    bm.check_invariants()


def test_lifo_reuse_and_all_or_nothing():
    bm = BlockManager(8)
    a = bm.allocate()
    bm.allocate()
    bm.decref(a)
    assert bm.allocate() == a
    assert bm.allocate_many(7) is None and bm.num_free == 6       # nothing taken
    got = bm.allocate_many(6)
    assert len(got) == 6 and bm.num_free == 0
    with pytest.raises(CoreError, match="index 1"):
        bm.decref_many([got[0], got[0]])
    with pytest.raises(ValueError):
        bm.allocate_many(-1)
    with pytest.raises(ValueError):
        bm.decref_many(np.zeros((2, 2), dtype=np.int32))


# ----------------------------------------------------------------- radix tree

def test_full_blocks_only():
    bm = BlockManager(8)
    tree = RadixTree(bm, 1)
    assert match_len(bm, tree, seq(64)) == 0
    toks = seq(40)
    held = prefill(bm, tree, toks)
    assert len(held) == 3 and tree.num_cached_blocks == 2 and not tree.is_cached(held[2])
    n, out = tree.match_prefix(toks)
    assert n == 32 and out == held[:2]
    assert bm.ref_count(held[0]) == 3                              # tree + request + this match
    bm.decref_many(out)
    bm.decref_many(held)
    assert bm.ref_count(held[0]) == 1
    ok(bm, tree)
    bm2 = BlockManager(4)
    t2 = RadixTree(bm2, 1)
    h = prefill(bm2, t2, seq(15))
    assert t2.num_cached_blocks == 0
    bm2.decref_many(h)
    assert bm2.num_free == 4


def test_siblings_with_the_same_first_token_and_same_tokens_at_other_depth():
    bm = BlockManager(16)
    tree = RadixTree(bm, 2)
    a = seq(32)
    b = a.copy()
    b[17] = 999
    ha = prefill(bm, tree, a)
    assert match_len(bm, tree, b) == 16
    hb = prefill(bm, tree, b)
    assert tree.num_cached_blocks == 3 and ha[0] == hb[0] and ha[1] != hb[1]
    n, out = tree.match_prefix(b)
    assert n == 32 and out[1] == hb[1]
    bm.decref_many(out + ha + hb)
    ok(bm, tree)
    chunk = seq(16, 100)
    twice = np.concatenate([chunk, chunk])
    h = prefill(bm, tree, twice)
    assert match_len(bm, tree, chunk) == 16 and match_len(bm, tree, twice) == 32
    assert len(set(h)) == 2
    bm.decref_many(h)
    ok(bm, tree)


def test_duplicate_content_keeps_the_tree_copy():
    bm = BlockManager(8)
    tree = RadixTree(bm, 3)
    toks = seq(32)
    first = prefill(bm, tree, toks)
    mine = bm.allocate_many(2)
    assert tree.insert(toks, mine) == 0
    assert not tree.is_cached(mine[0]) and bm.ref_count(mine[0]) == 1
    bm.decref_many(mine + first)
    ok(bm, tree)


def test_insert_refusals_change_nothing():
    bm = BlockManager(8)
    tree = RadixTree(bm, 4)
    held = prefill(bm, tree, seq(16))
    other = seq(32, 500)
    extra = bm.allocate()
    with pytest.raises(CoreError, match="already cached"):
        tree.insert(other, [held[0], extra])
    fresh = bm.allocate()
    with pytest.raises(CoreError, match="already cached"):
        tree.insert(other, [fresh, fresh])                         # same id twice: mark rolled back
    assert not tree.is_cached(fresh)
    assert bm.ref_count(7) == 0
    with pytest.raises(CoreError, match="not allocated"):
        tree.insert(other, [7, 6])
    with pytest.raises(CoreError, match="invalid block id"):
        tree.insert(other, [fresh, 1000])
    with pytest.raises(CoreError, match="invalid argument"):
        tree.insert(other, [fresh])
    assert tree.num_cached_blocks == 1
    ok(bm, tree)
    assert tree.insert(other, [fresh, extra]) == 2
    bm.decref_many([fresh, extra] + held)
    ok(bm, tree)


def test_eviction_order_pins_and_chains():
    bm = BlockManager(8)
    tree = RadixTree(bm, 5)
    a, b, c = seq(16, 0), seq(16, 100), seq(16, 200)
    for t in (a, b, c):
        bm.decref_many(prefill(bm, tree, t))
    assert match_len(bm, tree, a) == 16                            # a is now the most recent
    assert tree.evict(1) == 1
    assert match_len(bm, tree, b) == 0 and match_len(bm, tree, a) == 16 and match_len(bm, tree, c) == 16
    ok(bm, tree)

    bm = BlockManager(8)
    tree = RadixTree(bm, 5)
    held = prefill(bm, tree, a)                                    # still in use
    bm.decref_many(prefill(bm, tree, b))
    assert tree.evict(8) == 1 and match_len(bm, tree, a) == 16     # only b could go
    bm.decref_many(held)
    assert tree.evict(8) == 1 and bm.num_free == 8
    ok(bm, tree)

    bm = BlockManager(8)
    tree = RadixTree(bm, 5)
    bm.decref_many(prefill(bm, tree, seq(48)))
    assert tree.evict(10) == 3 and tree.num_cached_blocks == 0 and bm.num_free == 8
    with pytest.raises(ValueError):
        tree.evict(-1)


def test_tree_returns_its_refs_and_keeps_its_pool_alive():
    bm = BlockManager(8)
    tree = RadixTree(bm)
    bm.decref_many(prefill(bm, tree, seq(64)))
    assert bm.num_free == 4
    del tree
    assert bm.num_free == 8
    bm.check_invariants()
    tree = RadixTree(BlockManager(4))                              # pool object only reachable through the tree
    assert tree.match_prefix(seq(16)) == (0, [])


def test_inputs_are_copied_and_lists_accepted():
    bm = BlockManager(8)
    tree = RadixTree(bm, 6)
    toks = seq(32)
    held = bm.allocate_many(2)
    assert tree.insert(list(toks), np.asarray(held, dtype=np.int64)) == 2
    toks[:] = 0                                                    # caller's array changes afterwards
    assert match_len(bm, tree, seq(32)) == 32
    n, ids = tree.match_prefix(seq(32))
    ids.append(123)                                                # a fresh list, not a view
    assert tree.match_prefix(seq(32))[1] == held
    with pytest.raises(ValueError):
        tree.match_prefix(np.zeros((2, 16), dtype=np.int32))


def test_randomized_ref_count_model():
    """rc(b) == holders(b) + is_cached(b) after every operation; everything returns at the end."""
    rng = random.Random(7)
    bm = BlockManager(24)
    tree = RadixTree(bm, 9)
    live: list[list[int]] = []
    prefixes = [seq(48, 1000 * i) for i in range(3)]
    for _ in range(3000):
        op = rng.random()
        if op < 0.5:
            toks = np.concatenate([rng.choice(prefixes)[: rng.choice([16, 32, 48])], seq(rng.randint(1, 40), rng.randint(0, 5) * 77)])
            matched, held = tree.match_prefix(toks)
            need = -(-len(toks) // 16) - len(held)
            new = bm.allocate_many(need)
            if new is None:
                tree.evict(need - bm.num_free)
                new = bm.allocate_many(need)
            if new is None:
                bm.decref_many(held)
            else:
                held = held + new
                if rng.random() < 0.8:
                    tree.insert(toks, held)
                live.append(held)
        elif op < 0.85 and live:
            bm.decref_many(live.pop(rng.randrange(len(live))))
        else:
            tree.evict(rng.randint(0, 4))
        holders = np.zeros(24, dtype=int)
        for h in live:
            for b in h:
                holders[b] += 1
        for b in range(24):
            assert bm.ref_count(b) == holders[b] + int(tree.is_cached(b))
        ok(bm, tree)
    for h in live:
        bm.decref_many(h)
    tree.evict(24)
    assert bm.num_free == 24 and tree.num_cached_blocks == 0


# ---------------------------------------------------------------- state slots

def test_state_slots():
    s = StateSlots(3, 128)
    assert s.bytes_per_slot == 128 and s.num_slots == 3
    got = [s.acquire() for _ in range(3)]
    assert sorted(got) == [0, 1, 2] and s.acquire() is None and s.num_free == 0
    s.release(1)
    assert not s.in_use(1) and s.in_use(0)
    with pytest.raises(CoreError):
        s.release(1)                                               # freed twice
    with pytest.raises(CoreError):
        s.release(7)
    assert s.acquire() == 1
    z = StateSlots(2)                                              # size 0: ids are still handed out
    assert z.bytes_per_slot == 0 and z.acquire() == 0
    with pytest.raises(ValueError):
        StateSlots(0)


# --------------------------------------------------------------- cache manager

def test_manager_groups_windows_and_prefix_cache():
    m = CacheManager([8, 6], windows=[None, 32], num_slots=2)
    assert not m.prefix_cache                                      # a windowed group switches it off
    tables = m.allocate([5, 5])
    assert tables is not None and m.num_free(0) == 3 and m.num_free(1) == 1
    assert m.allocate([4, 1]) is None and m.num_free(0) == 3 and m.num_free(1) == 1   # all-or-nothing across groups
    # 80 tokens computed: the next token (position 80) sees 49..80 in the window group, so pages 0..2 go.
    assert m.trim_windows(tables, 80) == 3
    assert tables[1][:3] == [-1, -1, -1] and tables[1][3] >= 0 and tables[0][0] >= 0
    assert m.num_free(1) == 4
    assert m.trim_windows(tables, 80) == 0                         # not freed twice
    m.release(tables)
    assert m.num_free(0) == 8 and m.num_free(1) == 6
    m.check_invariants()
    assert m.pages_needed(0, 1000, 64) == 63 and m.pages_needed(1, 1000, 64) == 7

    m = CacheManager([8, 8], num_slots=2)                          # two full groups: one tree each
    toks = seq(40)
    t = m.allocate([3, 3])
    m.cache(toks, t)
    m.release(t)
    matched, got = m.match_prefix(toks)
    assert matched == 32 and [len(g) for g in got] == [2, 2]
    m.release(got)
    assert m.evict_all() == 4 and m.num_free(0) == 8 and m.num_free(1) == 8
    a, b = m.acquire_slot(), m.acquire_slot()
    assert {a, b} == {0, 1} and m.acquire_slot() is None
    m.release_slot(a)
    assert m.acquire_slot() == a


def test_manager_random_requests_lose_nothing():
    rng = random.Random(3)
    m = CacheManager([20], num_slots=4)
    live = []
    for _ in range(2000):
        if rng.random() < 0.55 and len(live) < 4:
            toks = np.concatenate([seq(32, 500 * rng.randint(0, 2)), seq(rng.randint(1, 60), rng.randint(0, 9))])
            matched, tables = m.match_prefix(toks[:-1])
            need = -(-len(toks) // 16) - len(tables[0])
            fresh = m.allocate([need])
            slot = m.acquire_slot()
            if fresh is None or slot is None:
                m.release(tables)
                if slot is not None:
                    m.release_slot(slot)
                continue
            tables[0].extend(fresh[0])
            live.append((toks, tables, slot))
        elif live:
            toks, tables, slot = live.pop(rng.randrange(len(live)))
            if rng.random() < 0.7:
                m.cache(toks, tables)
            m.release(tables)
            m.release_slot(slot)
        distinct = {b for t in live for b in t[1][0]}                # shared prefix pages count once
        assert len(distinct) + m.num_free(0) + m.num_cached(0) >= 20 and len(distinct) + m.num_free(0) <= 20
        m.check_invariants()
    for toks, tables, slot in live:
        m.release(tables)
        m.release_slot(slot)
    m.evict_all()
    assert m.num_free(0) == 20 and m.slots.num_free == 4
