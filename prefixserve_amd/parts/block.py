"""How a layer's parts are arranged."""

from __future__ import annotations

from typing import TYPE_CHECKING, Any

import torch

from .base import FeedForward, Mixer, Norm, Part, register_block

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


class PreNormBlock:
    """norm -> mixer -> add, norm -> feed-forward -> add (prefixserve/model/llama.py:111-121).

    The residual stream is float32. Each sub-layer's output is not added at once: it is
    handed on as ``pending`` and summed into the residual by the next norm's fused
    add+norm, so the stream is read and written once per sub-layer."""

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, feed_forward_norm: Norm) -> None:
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm

    def parts(self) -> list[Part]:
        return [self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward]

    def forward(self, residual: torch.Tensor, pending: torch.Tensor | None, ctx: "StepContext", cache: Any,
                state: torch.Tensor | None, writes_cache: bool) -> torch.Tensor:
        x = self.mixer_norm.add_norm(residual, pending, "block.x")
        mixed = self.mixer.forward(x, ctx, cache, state, writes_cache)
        x = self.feed_forward_norm.add_norm(residual, mixed, "block.x")
        return self.feed_forward.forward(x, ctx)


    def fused_decode_layer(self, cache: Any, writes_cache: bool) -> dict | None:
        """What the fused decode step needs to run this layer, if it can: the layer must be
        exactly RMSNorm, rotary (or unrotated) attention over pages without a window, RMSNorm,
        SwiGLU, each of the package's own classes and bound. None otherwise; the layer then
        runs part by part."""
        from .attention import PagedAttention
        from .mlp import SwiGLU
        from .norm import RMSNorm

        m, ff, n1, n2 = self.mixer, self.feed_forward, self.mixer_norm, self.feed_forward_norm
        if type(m) is not PagedAttention or type(ff) is not SwiGLU or type(n1) is not RMSNorm or type(n2) is not RMSNorm:
            return None
        if cache is None or cache.window is not None or m.window is not None or n1.weight.dtype != n2.weight.dtype:
            return None
        return dict(w_qkv=m.w_qkv, w_o=m.w_o, w_gate_up=ff.w_gate_up, w_down=ff.w_down, norm1=n1.weight, norm2=n2.weight,
                    eps1=n1.eps, eps2=n2.eps, kv=cache.kv, rope=None if m.pos is None else m.pos.table, group=cache.group,
                    writes_cache=bool(writes_cache), hq=m.num_heads, hkv=m.num_kv_heads, d=m.head_dim, scale=m.scale,
                    inter=ff.intermediate_size, hidden=m.hidden_size)


register_block("prenorm", PreNormBlock)
