"""Host-side cache manager: pages of every layer group, the prefix cache, state slots.

For each layer group it owns a ``BlockManager`` (ref-counted page ids) and, when prefix
caching is possible, a ``RadixTree``. A request holds one reference on every page in its
block tables and, while it lives, one state slot. Pages come back when a request ends or
is preempted, when a window has passed them, and when cached prefixes are evicted to make
room; they are then used again.

Prefix caching needs every key of the prefix to be present, so it is active only when no
group is windowed; and it needs everything a request has computed to be in pages, so it is
off when requests keep state in slots (``bytes_per_slot > 0``): a request that started
behind a cached prefix would run with a state that never saw the prefix. With several groups each has a tree of its own; a match is the shortest
of the groups' matches.
"""

from __future__ import annotations

from typing import Sequence

import numpy as np

from prefixserve_amd.build import ensure_core

_core = ensure_core()
BLOCK_SIZE: int = _core.BLOCK_SIZE
BlockManager = _core.BlockManager
RadixTree = _core.RadixTree
StateSlots = _core.StateSlots
CoreError = _core.CoreError


def blocks_for(num_tokens: int) -> int:
    return -(-num_tokens // BLOCK_SIZE)


class CacheManager:
    def __init__(self, num_blocks: Sequence[int], windows: Sequence[int | None] | None = None, num_slots: int = 64,
                 bytes_per_slot: int = 0, enable_prefix_cache: bool = True, hash_seed: int | None = None) -> None:
        self.num_groups = len(num_blocks)
        if self.num_groups < 1:
            raise ValueError("at least one layer group")
        self.windows = list(windows) if windows is not None else [None] * self.num_groups
        if len(self.windows) != self.num_groups:
            raise ValueError("one window entry per group")
        self.pools = [BlockManager(int(n)) for n in num_blocks]
        self.prefix_cache = (bool(enable_prefix_cache) and all(w is None for w in self.windows)
                             and int(bytes_per_slot) == 0)
        self.trees = [RadixTree(p, hash_seed) for p in self.pools] if self.prefix_cache else []
        self.slots = StateSlots(int(num_slots), int(bytes_per_slot))

    # ------------------------------------------------------------- sizes

    def num_blocks(self, g: int = 0) -> int:
        return self.pools[g].num_blocks

    def num_free(self, g: int = 0) -> int:
        return self.pools[g].num_free

    def num_cached(self, g: int = 0) -> int:
        return self.trees[g].num_cached_blocks if self.prefix_cache else 0

    def pages_needed(self, g: int, num_tokens: int, longest_step: int) -> int:
        """Most pages a request of ``num_tokens`` holds in group g at any time, when no step
        gives it more than ``longest_step`` tokens."""
        w = self.windows[g]
        if w is None:
            return blocks_for(num_tokens)
        return min(blocks_for(num_tokens), blocks_for(w + longest_step) + 1)

    # ------------------------------------------------------------- pages

    def match_prefix(self, tokens: np.ndarray) -> tuple[int, list[list[int]]]:
        """(matched token count, block tables per group); one reference per page is taken."""
        if not self.prefix_cache:
            return 0, [[] for _ in range(self.num_groups)]
        found = [t.match_prefix(tokens) for t in self.trees]
        matched = min(m for m, _ in found)
        keep = matched // BLOCK_SIZE
        tables = []
        for pool, (_, ids) in zip(self.pools, found):
            if len(ids) > keep:
                pool.decref_many(ids[keep:])
            tables.append(list(ids[:keep]))
        return matched, tables

    def allocate(self, counts: Sequence[int]) -> list[list[int]] | None:
        """``counts[g]`` fresh pages in every group, or None with nothing taken. Cached
        prefixes nobody uses are evicted, least recently used first, when a pool is short
        (prefixserve/scheduler.py:395-402 of the reference)."""
        for g, n in enumerate(counts):
            short = n - self.pools[g].num_free
            if short > 0 and self.prefix_cache:
                self.trees[g].evict(short)
        if any(n > self.pools[g].num_free for g, n in enumerate(counts)):
            return None
        out = []
        for g, n in enumerate(counts):
            ids = self.pools[g].allocate_many(int(n)) if n > 0 else []
            assert ids is not None
            out.append(list(ids))
        return out

    def release(self, tables: Sequence[Sequence[int]]) -> None:
        """Gives back the request's reference on every page it still holds (-1 = already gone)."""
        for pool, table in zip(self.pools, tables):
            live = [b for b in table if b >= 0]
            if live:
                pool.decref_many(live)

    def cache(self, tokens: np.ndarray, tables: Sequence[Sequence[int]]) -> None:
        """Puts the full pages of ``tokens`` into the prefix cache (no-op when it is off)."""
        if not self.prefix_cache or len(tokens) < BLOCK_SIZE:
            return
        for tree, table in zip(self.trees, tables):
            tree.insert(tokens, table)

    def trim_windows(self, tables: list[list[int]], next_position: int) -> int:
        """Releases pages of window groups that no token at or after ``next_position`` can see.
        Entries become -1 so positions keep their index. Returns how many pages went back."""
        freed = 0
        for g, w in enumerate(self.windows):
            if w is None:
                continue
            first_visible = next_position - w + 1
            last_dead_page = first_visible // BLOCK_SIZE  # pages [0, last_dead_page) lie wholly before it
            table = tables[g]
            # Pages go back in order, so the entries already given back are a prefix of the
            # table: walk down from the newest dead page until one of them.
            j = min(max(last_dead_page, 0), len(table)) - 1
            while j >= 0 and table[j] >= 0:
                self.pools[g].decref(table[j])
                table[j] = -1
                freed += 1
                j -= 1
        return freed

    def evict_all(self) -> int:
        return sum(t.evict(p.num_blocks) for t, p in zip(self.trees, self.pools))

    # ------------------------------------------------------------- slots

    def acquire_slot(self) -> int | None:
        return self.slots.acquire()

    def release_slot(self, slot: int) -> None:
        self.slots.release(slot)

    def check_invariants(self) -> None:
        for p in self.pools:
            p.check_invariants()
        for t in self.trees:
            t.check_invariants()
