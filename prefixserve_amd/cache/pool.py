"""Device memory of the cache: one page pool per layer group, and per-request state.

Layers whose mixers need the same thing (same kv heads, head size and window) form a
group. A group has its own pages and every request has one block table per group; a page
id addresses the same page in every layer of its group, so the host-side bookkeeping is
per group, not per layer (the reference has a single group: one id addresses the page in
all layers, prefixserve/llama_engine.py:110-117).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Mapping

import torch

from prefixserve_amd.engine.batch import PAGE
from prefixserve_amd.parts.attention import LayerCache
from prefixserve_amd.parts.base import CacheNeed, StateNeed


@dataclass(frozen=True)
class LayerGroup:
    need: CacheNeed
    entries: tuple[int, ...]      # cache entries (see LayerRun.cache) stored in this group

    def bytes_per_block(self, itemsize: int) -> int:
        return 2 * PAGE * self.need.kv_heads * self.need.head_dim * itemsize * len(self.entries)


def plan_groups(needs: Mapping[int, CacheNeed]) -> list[LayerGroup]:
    by_need: dict[CacheNeed, list[int]] = {}
    for entry in sorted(needs):
        by_need.setdefault(needs[entry], []).append(entry)
    return [LayerGroup(need, tuple(entries)) for need, entries in by_need.items()]


class KVPools:
    """``tensors[g]`` is ``[entries, num_blocks, 2, kv_heads, 16 * head_dim]`` in the activation
    dtype, allocated once and never grown (growing would copy every live page)."""

    def __init__(self, groups: list[LayerGroup], num_blocks: list[int], dtype: torch.dtype,
                 device: torch.device) -> None:
        self.groups = groups
        self.num_blocks = list(num_blocks)
        self.tensors = [
            torch.zeros((len(g.entries), nb, 2, g.need.kv_heads, PAGE * g.need.head_dim), dtype=dtype, device=device)
            for g, nb in zip(groups, num_blocks)
        ]

    def layer_caches(self) -> dict[int, LayerCache]:
        out: dict[int, LayerCache] = {}
        for gi, (g, t) in enumerate(zip(self.groups, self.tensors)):
            for j, entry in enumerate(g.entries):
                out[entry] = LayerCache(kv=t[j], group=gi, window=g.need.window)
        return out

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.tensors)


def make_states(needs: Mapping[int, StateNeed], num_slots: int, device: torch.device) -> dict[int, torch.Tensor]:
    """run index -> ``[num_slots, *shape]`` zero-initialised."""
    return {i: torch.zeros((num_slots, *n.shape), dtype=n.dtype, device=device) for i, n in needs.items()}
