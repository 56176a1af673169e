"""Grouped-query causal attention over the paged cache."""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import TYPE_CHECKING, Any, Mapping

import torch

from .base import CacheNeed, Mixer, PositionEncoding, RotaryTable, Runtime, WeightWant, register_mixer

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


@dataclass
class LayerCache:
    """One cache entry as a run sees it: the pages of its layer group.

    ``kv`` is ``[num_blocks, 2, kv_heads, 16 * head_dim]``. Half 0 of a page holds the keys
    of its 16 positions as ``[16, head_dim]`` (after rotation); half 1 holds the values
    transposed, ``[head_dim, 16]``, which is the operand order the matrix cores want for
    probabilities x values. ``group`` selects the block tables of the step batch."""

    kv: torch.Tensor
    group: int
    window: int | None


class PagedAttention(Mixer):
    """q/k/v projection (one fused product), position encoding on q and k, keys and values
    written to their pages, causal attention of every new token over the request's cache,
    output projection. Query head h reads kv head h // (heads / kv_heads); scores are
    q.k / sqrt(head_dim) unless ``scale`` is given; softmax in 32-bit
    (prefixserve/model/llama.py:113-117, prefixserve/model/attention.py:103-120)."""

    takes_normed_rows = True

    def __init__(self, hidden_size: int, positions: Mapping[str, PositionEncoding], num_heads: int,
                 num_kv_heads: int, head_dim: int, names: Mapping[str, str], position: str | None = None,
                 window: int | None = None, scale: float | None = None) -> None:
        if num_kv_heads < 1 or num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads not divisible by {num_kv_heads} kv heads")
        if head_dim % 16 or not 16 <= head_dim <= 256:
            raise ValueError(f"head_dim must be a multiple of 16 in [16, 256], got {head_dim}")
        self.hidden_size = int(hidden_size)
        self.num_heads, self.num_kv_heads, self.head_dim = int(num_heads), int(num_kv_heads), int(head_dim)
        self.names = dict(names)
        self.window = None if window is None else int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.pos = positions[position] if position is not None else None
        if self.pos is not None and not isinstance(self.pos, RotaryTable):
            raise ValueError("PagedAttention applies rotation tables; other encodings belong to their own mixer")
        if isinstance(self.pos, RotaryTable) and self.pos.head_dim != self.head_dim:
            raise ValueError("rotary head_dim differs from the attention head_dim")
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim

    def weights(self) -> dict[str, WeightWant]:
        h, n = self.hidden_size, self.names
        return {
            n["q"]: WeightWant((self.q_size, h)),
            n["k"]: WeightWant((self.kv_size, h)),
            n["v"]: WeightWant((self.kv_size, h)),
            n["o"]: WeightWant((h, self.q_size)),
        }

    def cache_need(self) -> CacheNeed:
        return CacheNeed(self.num_kv_heads, self.head_dim, self.window)

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        super().bind(tensors, rt)
        n = self.names
        # Rows of q, then k, then v: one product per layer instead of three
        # (prefixserve/model/weights.py:115-119). No permutation: checkpoints are laid
        # out for the rotate-half pairing already.
        self.w_qkv = rt.ops.prepare_matrix(torch.cat([tensors[n["q"]], tensors[n["k"]], tensors[n["v"]]], dim=0), rt)
        self.w_o = rt.ops.prepare_matrix(tensors[n["o"]], rt)

    def weight_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_qkv, self.w_o))

    def forward(self, x: torch.Tensor, ctx: "StepContext", cache: Any, state: torch.Tensor | None,
                writes_cache: bool) -> torch.Tensor:
        rt, ops, ws = self.rt, self.rt.ops, self.rt.workspace
        t = x.shape[0]
        qkv = ws.get("attn.qkv", (t, self.q_size + 2 * self.kv_size), rt.dtype)
        table = self.pos.table if self.pos is not None else None
        ops.qkv_rope_append(x, self.w_qkv, qkv, self.num_heads, self.num_kv_heads, self.head_dim, ctx.positions, table,
                            cache.kv if writes_cache else None, ctx.groups[cache.group].write_slot)
        out = ws.get("attn.out", (t, self.q_size), rt.dtype)
        ops.paged_attention(qkv, out, cache.kv, ctx, cache.group, self.num_heads, self.num_kv_heads,
                            self.head_dim, self.scale, cache.window)
        return ops.linear_to_residual(out, self.w_o, "attn.delta", getattr(ctx, "residual", None))


register_mixer("paged_attention", PagedAttention)
