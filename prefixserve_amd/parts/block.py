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
    add+norm, so the stream is read and written once per sub-layer. A sub-layer may also add its
    output into the stream itself and hand on None; and where a sub-layer's kernels normalize
    their tokens themselves (``takes_normed_rows``), the norm in front of it may hand over the
    rows of the stream instead of running a kernel. An arrangement that needs a sub-layer's
    output itself (to normalize it before it is added, say) sets ``ctx.residual = None`` first:
    the sub-layers then hand their output back in every step."""

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, feed_forward_norm: Norm) -> None:
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm

    def parts(self) -> list[Part]:
        return [self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward]

    def forward(self, residual: torch.Tensor, pending: torch.Tensor | None, ctx: "StepContext", cache: Any,
                state: torch.Tensor | None, writes_cache: bool) -> torch.Tensor:
        if self.mixer.takes_normed_rows:
            x = self.mixer_norm.add_norm(residual, pending, "block.x", lazy=True)
        else:
            x = self.mixer_norm.add_norm(residual, pending, "block.x")
        mixed = self.mixer.forward(x, ctx, cache, state, writes_cache)
        if self.feed_forward.takes_normed_rows:
            x = self.feed_forward_norm.add_norm(residual, mixed, "block.x", lazy=True)
        else:
            x = self.feed_forward_norm.add_norm(residual, mixed, "block.x")
        return self.feed_forward.forward(x, ctx)


register_block("prenorm", PreNormBlock)
