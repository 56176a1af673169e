"""The batch of one step: for each request its next tokens, where they start, its block
tables and state slot, and the places whose logits are wanted.

All tokens of all requests lie back to back (``[T]``, no padding). Every integer array
the kernels need is laid out in ONE pinned host buffer and goes to the device in one copy
(prefixserve/llama_engine.py:152-227 of the reference packs its seven arrays the same way);
the arrays are checked on the host first, because a bad page id on the device is an
out-of-bounds write, not an error (llama_engine.py:270-287).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Hashable, Sequence

import numpy as np
import torch

PAGE = 16  # tokens per page; equals the cache core's BLOCK_SIZE


class EngineError(RuntimeError):
    """The engine was given a batch it cannot run: a configuration or scheduler bug."""


@dataclass
class StepItem:
    """``tokens`` = seq[start : start+n] of one request. ``block_tables[g]`` is the request's
    block table in layer group g (entry j covers positions [16j, 16j+16); entries wholly
    outside a window group's window may be -1). ``want`` lists indices into ``tokens``."""

    key: Hashable
    tokens: Any
    start: int
    block_tables: Sequence[Sequence[int]]
    slot: int = 0
    want: Sequence[int] = ()


@dataclass(frozen=True)
class GroupMeta:
    num_blocks: int
    window: int | None = None


@dataclass
class GroupArrays:
    table_off: torch.Tensor    # [B+1] start of each item's table in block_ids
    block_ids: torch.Tensor    # [P]
    write_slot: torch.Tensor   # [T]   page * 16 + offset where each new token's K/V goes
    table_off_host: np.ndarray
    block_ids_host: np.ndarray


@dataclass
class StepContext:
    num_tokens: int
    num_items: int
    num_logit_rows: int
    num_decode: int            # items with exactly one token (served by the decode kernel)
    num_prefill_tiles: int
    max_kv_len: int
    token_ids: torch.Tensor    # [T]
    positions: torch.Tensor    # [T] absolute
    tok_item: torch.Tensor     # [T] item of each token
    item_start: torch.Tensor   # [B+1] first flat token of each item
    item_pos0: torch.Tensor    # [B] absolute position of the item's first token
    item_end: torch.Tensor     # [B] kv length after this step
    slots: torch.Tensor        # [B]
    logit_rows: torch.Tensor   # [S] flat token rows
    dec_items: torch.Tensor    # [num_decode] item indices
    pf_tiles: torch.Tensor     # [num_prefill_tiles, 2] (item, first query of the tile within the item)
    groups: list[GroupArrays]
    keys: list[Hashable]
    want_counts: list[int]
    host: dict[str, np.ndarray] = field(default_factory=dict)


class StepPacker:
    """Owns the host staging buffer and its device twin. ``pack`` must not be called again
    before the previous step's kernels were enqueued; it waits for the previous copy itself."""

    def __init__(self, device: torch.device, groups: Sequence[GroupMeta], vocab_size: int, max_position: int,
                 num_slots: int, prefill_tile: int, capacity: int = 1 << 16) -> None:
        self.device = torch.device(device)
        self.groups = list(groups)
        self.vocab_size, self.max_position, self.num_slots = int(vocab_size), int(max_position), int(num_slots)
        self.prefill_tile = int(prefill_tile)
        self.on_gpu = self.device.type == "cuda"
        self._copied = torch.cuda.Event() if self.on_gpu else None
        self._alloc(capacity)

    def _alloc(self, capacity: int) -> None:
        self.capacity = int(capacity)
        self._host = torch.empty(self.capacity, dtype=torch.int32, pin_memory=self.on_gpu)
        self._host_np = self._host.numpy()
        self._dev = torch.empty(self.capacity, dtype=torch.int32, device=self.device) if self.on_gpu else self._host
        self.version = getattr(self, "version", 0) + 1

    def pack(self, items: Sequence[StepItem], static_pages: int | None = None) -> StepContext:
        """``static_pages``: give every item's table exactly this many entries (padded), so
        that the layout depends only on the batch's shape: what a captured graph needs."""
        if not items:
            raise EngineError("empty step")
        b = len(items)
        g_n = len(self.groups)
        toks = [np.asarray(it.tokens, dtype=np.int64).reshape(-1) for it in items]
        lens = [int(t.size) for t in toks]
        if min(lens) < 1:
            raise EngineError("an item has no tokens")
        t_n = sum(lens)
        s_n = sum(len(it.want) for it in items)
        ends = [int(it.start) + n for it, n in zip(items, lens)]
        pages = [-(-e // PAGE) for e in ends]
        tile = self.prefill_tile
        n_dec = sum(1 for n in lens if n == 1)
        n_tiles = sum(-(-n // tile) for n in lens if n > 1)
        p_caps = [static_pages if static_pages is not None else p for p in pages]
        p_total = sum(p_caps)

        # ---- host checks (per item: cheap scalar ones; ranges of ids and pages: once per array below) ----
        max_slot = max(self.num_slots, 1)
        for it, n, e, pg in zip(items, lens, ends, pages):
            if it.start < 0 or e > self.max_position:
                raise EngineError(f"{it.key}: positions [{it.start}, {e}) outside [0, {self.max_position})")
            if not 0 <= it.slot < max_slot:
                raise EngineError(f"{it.key}: state slot {it.slot} outside [0, {self.num_slots})")
            if len(it.block_tables) != g_n:
                raise EngineError(f"{it.key}: {len(it.block_tables)} block tables for {g_n} layer groups")
            for w in it.want:
                if not 0 <= w < n:
                    raise EngineError(f"{it.key}: wanted place {w} outside its {n} tokens")
            if static_pages is not None and pg > static_pages:
                raise EngineError(f"{it.key}: needs {pg} pages, static layout has {static_pages}")
            for gi, table in enumerate(it.block_tables):
                if len(table) < pg:
                    raise EngineError(f"{it.key}: {len(table)} blocks in group {gi} for {e} tokens")

        # ---- layout ----
        off = 0

        def take(n: int) -> slice:
            nonlocal off
            s = slice(off, off + n)
            off += n
            return s

        sl = {
            "token_ids": take(t_n), "positions": take(t_n), "tok_item": take(t_n),
            "item_start": take(b + 1), "item_pos0": take(b), "item_end": take(b), "slots": take(b),
            "logit_rows": take(s_n), "dec_items": take(n_dec), "pf_tiles": take(2 * n_tiles),
        }
        gsl = [{"table_off": take(b + 1), "write_slot": take(t_n), "block_ids": take(p_total)} for _ in range(g_n)]
        total = off
        if total > self.capacity:
            if self._copied is not None:
                self._copied.synchronize()
            if self.on_gpu:
                torch.cuda.synchronize()
            self._alloc(max(total, 2 * self.capacity))
        if self._copied is not None:
            self._copied.synchronize()  # the previous copy must have left the staging buffer
        buf = self._host_np

        ids, pos, tok_item = buf[sl["token_ids"]], buf[sl["positions"]], buf[sl["tok_item"]]
        item_start, item_pos0 = buf[sl["item_start"]], buf[sl["item_pos0"]]
        item_end, slots = buf[sl["item_end"]], buf[sl["slots"]]
        rows, dec, tiles = buf[sl["logit_rows"]], buf[sl["dec_items"]], buf[sl["pf_tiles"]]
        # Absolute positions: a request that reused a prefix or resumes after preemption does
        # not restart at 0 (prefixserve/llama_engine.py:190-193).
        starts = [int(it.start) for it in items]
        item_start[0] = 0
        item_start[1:] = np.cumsum(lens)
        item_pos0[:], item_end[:], slots[:] = starts, ends, [it.slot for it in items]
        if n_dec == b:
            ids[:] = [tk[0] for tk in toks]
            pos[:] = starts
            tok_item[:] = np.arange(b, dtype=np.int32)
        else:
            ids[:] = np.concatenate(toks)
            tok_item[:] = np.repeat(np.arange(b, dtype=np.int32), lens)
            pos[:] = item_pos0[tok_item] + (np.arange(t_n, dtype=np.int32) - item_start[tok_item])
        dec[:] = [i for i, n in enumerate(lens) if n == 1]
        tiles[:] = [x for i, n in enumerate(lens) if n > 1 for q in range(0, n, tile) for x in (i, q)]
        rows[:] = [t0 + w for t0, it in zip(item_start[:-1].tolist(), items) for w in it.want]
        if int(ids.min()) < 0 or int(ids.max()) >= self.vocab_size:
            bad = next(it.key for it, tk in zip(items, toks) if int(tk.min()) < 0 or int(tk.max()) >= self.vocab_size)
            raise EngineError(f"{bad}: token id outside [0, {self.vocab_size})")

        for gi, (gm, gs) in enumerate(zip(self.groups, gsl)):
            table_off, wslot, bids = buf[gs["table_off"]], buf[gs["write_slot"]], buf[gs["block_ids"]]
            table_off[0] = 0
            table_off[1:] = np.cumsum(p_caps)
            if static_pages is not None:
                bids[:] = 0
            p0 = 0
            for it, s0, pg, cap in zip(items, starts, pages, p_caps):
                table = it.block_tables[gi]
                if not isinstance(table, np.ndarray):
                    table = np.asarray(table[:pg], dtype=np.int64)
                # Pages a token of this step can see or writes: all of them, or for a window
                # group those from the window of the first new token on; earlier entries may be
                # -1 (given back) and are never read.
                if gm.window is None:
                    bids[p0:p0 + pg] = table[:pg]
                else:
                    first_needed = max(0, s0 - gm.window + 1) // PAGE
                    bids[p0:p0 + first_needed] = 0
                    bids[p0 + first_needed:p0 + pg] = table[first_needed:pg]
                p0 += cap
            if int(bids.min()) < 0 or int(bids.max()) >= gm.num_blocks:
                p0 = 0
                for it, pg, cap in zip(items, pages, p_caps):        # name the request that brought it
                    row = bids[p0:p0 + pg]
                    if row.size and (int(row.min()) < 0 or int(row.max()) >= gm.num_blocks):
                        raise EngineError(f"{it.key}: block id outside the pool of group {gi} (0..{gm.num_blocks - 1})")
                    p0 += cap
            wslot[:] = bids[table_off[tok_item] + pos // PAGE] * PAGE + pos % PAGE

        # ---- one copy ----
        if self.on_gpu:
            self._dev[:total].copy_(self._host[:total], non_blocking=True)
            assert self._copied is not None
            self._copied.record()
        dev = self._dev

        def d(s: slice) -> torch.Tensor:
            return dev[s]

        groups = [GroupArrays(d(gs["table_off"]), d(gs["block_ids"]), d(gs["write_slot"]),
                              buf[gs["table_off"]], buf[gs["block_ids"]]) for gs in gsl]
        return StepContext(
            num_tokens=t_n, num_items=b, num_logit_rows=s_n, num_decode=n_dec, num_prefill_tiles=n_tiles,
            max_kv_len=max(ends),
            token_ids=d(sl["token_ids"]), positions=d(sl["positions"]), tok_item=d(sl["tok_item"]),
            item_start=d(sl["item_start"]), item_pos0=d(sl["item_pos0"]), item_end=d(sl["item_end"]),
            slots=d(sl["slots"]), logit_rows=d(sl["logit_rows"]), dec_items=d(sl["dec_items"]),
            pf_tiles=d(sl["pf_tiles"]).view(n_tiles, 2), groups=groups,
            keys=[it.key for it in items], want_counts=[len(it.want) for it in items],
            host={k: buf[v] for k, v in sl.items()},
        )
