"""The batch of one step: for each request its next tokens, where they start, its block
tables and state slot, and the places whose logits are wanted.

All tokens of all requests lie back to back (``[T]``, no padding). Every integer array
the kernels need is laid out in ONE pinned host buffer and goes to the device in one copy
(prefixserve/llama_engine.py:152-227 of the reference packs its seven arrays the same way);
the arrays are checked on the host first, because a bad page id on the device is an
out-of-bounds write, not an error (llama_engine.py:270-287). Checking and filling run in
the cache core (csrc/core/step_pack.cpp): they are on the critical path of every step.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Hashable, Sequence

import numpy as np
import torch

from ..build import ensure_core

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
    num_prefill_blocks: int
    max_kv_len: int
    decode_skewed: bool        # the kernels' verdict on the single-token items' context lengths (one far longer than the rest)
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
    pf_blocks: torch.Tensor    # [num_prefill_blocks] the first tile of each run of up to four consecutive tiles of an item
    groups: list[GroupArrays]
    keys: list[Hashable]
    want_counts: list[int]
    host: dict[str, np.ndarray] = field(default_factory=dict)
    # The step's residual stream (float32 [T, hidden]), set by the model before the layers run: a
    # part may add its output into it itself instead of handing back what is to be added.
    residual: Any = None


class StepPacker:
    """Owns the host staging buffer and its device twin. ``pack`` must not be called again
    before the previous step's kernels were enqueued; it waits for the previous copy itself."""

    def __init__(self, device: torch.device, groups: Sequence[GroupMeta], vocab_size: int, max_position: int,
                 num_slots: int, prefill_tile: int, capacity: int = 1 << 16, skew_rule: Any = None) -> None:
        """``skew_rule(count, longest, total) -> bool``: the kernel library's rule for when the
        context lengths of a step's single-token items count as skewed (it cuts their keys
        another way then, and a captured step is keyed by it); without one, never."""
        self.device = torch.device(device)
        self.groups = list(groups)
        self.vocab_size, self.max_position, self.num_slots = int(vocab_size), int(max_position), int(num_slots)
        self.prefill_tile = int(prefill_tile)
        self._skew_rule = skew_rule
        self.on_gpu = self.device.type == "cuda"
        self._copied = torch.cuda.Event() if self.on_gpu else None
        self._pack_step = ensure_core().pack_step
        self._group_args = [(int(g.num_blocks), None if g.window is None else int(g.window)) for g in self.groups]
        self._alloc(capacity)

    def _alloc(self, capacity: int) -> None:
        self.capacity = int(capacity)
        self._host = torch.empty(self.capacity, dtype=torch.int32, pin_memory=self.on_gpu)
        self._host_np = self._host.numpy()
        self._dev = torch.empty(self.capacity, dtype=torch.int32, device=self.device) if self.on_gpu else self._host
        self.version = getattr(self, "version", 0) + 1
        self._views = None

    def pack(self, items: Sequence[StepItem], static_pages: int | None = None) -> StepContext:
        """``static_pages``: give every item's table exactly this many entries (padded), so
        that the layout depends only on the batch's shape: what a captured graph needs.
        Checking and filling are the cache core's ``pack_step``."""
        if self._copied is not None:
            self._copied.synchronize()  # the previous copy must have left the staging buffer
        try:
            res = self._pack_step(self._host_np, items, self._group_args, self.vocab_size, self.max_position,
                                  self.num_slots, self.prefill_tile, static_pages)
            if not res[0]:
                if self.on_gpu:
                    torch.cuda.synchronize()
                self._alloc(max(res[1], 2 * self.capacity))
                res = self._pack_step(self._host_np, items, self._group_args, self.vocab_size, self.max_position,
                                      self.num_slots, self.prefill_tile, static_pages)
        except ValueError as e:
            raise EngineError(str(e)) from None
        _, total, t_n, b, s_n, n_dec, n_tiles, n_blocks, p_total, max_kv_len, dec_max_kv, dec_sum_kv, offs, group_offs = res
        o_ids, o_pos, o_item, o_start, o_pos0, o_end, o_slots, o_rows, o_dec, o_tiles, o_blocks = offs

        if self.on_gpu:
            self._dev[:total].copy_(self._host[:total], non_blocking=True)
            assert self._copied is not None
            self._copied.record()
        # The views depend on the layout only, and a decoding batch keeps its layout for many steps.
        sig = (self.version, t_n, b, s_n, n_dec, n_tiles, n_blocks, p_total, offs, tuple(group_offs))
        if self._views is None or self._views[0] != sig:
            dev, buf = self._dev, self._host_np
            named = {"token_ids": (o_ids, t_n), "positions": (o_pos, t_n), "tok_item": (o_item, t_n),
                     "item_start": (o_start, b + 1), "item_pos0": (o_pos0, b), "item_end": (o_end, b),
                     "slots": (o_slots, b), "logit_rows": (o_rows, s_n), "dec_items": (o_dec, n_dec),
                     "pf_tiles": (o_tiles, 2 * n_tiles), "pf_blocks": (o_blocks, n_blocks)}
            on_dev = {k: dev[o:o + n] for k, (o, n) in named.items()}
            on_dev["pf_tiles"] = on_dev["pf_tiles"].view(n_tiles, 2)
            host = {k: buf[o:o + n] for k, (o, n) in named.items()}
            groups = [GroupArrays(dev[o_t:o_t + b + 1], dev[o_b:o_b + p_total], dev[o_w:o_w + t_n],
                                  buf[o_t:o_t + b + 1], buf[o_b:o_b + p_total]) for o_t, o_w, o_b in group_offs]
            self._views = (sig, on_dev, host, groups)
        _, on_dev, host, groups = self._views
        skewed = bool(self._skew_rule(n_dec, dec_max_kv, dec_sum_kv)) if self._skew_rule is not None and n_dec > 1 else False
        return StepContext(
            num_tokens=t_n, num_items=b, num_logit_rows=s_n, num_decode=n_dec, num_prefill_tiles=n_tiles,
            num_prefill_blocks=n_blocks, max_kv_len=max_kv_len, decode_skewed=skewed, groups=groups,
            keys=[it.key for it in items],
            want_counts=[len(it.want) for it in items], host=host, **on_dev,
        )
