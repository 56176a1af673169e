"""Dense gated feed-forward (SwiGLU)."""

from __future__ import annotations

from typing import TYPE_CHECKING, Mapping

import torch

from .base import FeedForward, Runtime, WeightWant, register_feed_forward

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


class SwiGLU(FeedForward):
    """down( silu(gate(x)) * up(x) ), no biases; gate and up are one fused product whose
    first ``intermediate_size`` columns are the gate (prefixserve/model/llama.py:120-121,
    prefixserve/model/weights.py:120-123)."""

    takes_normed_rows = True

    def __init__(self, hidden_size: int, intermediate_size: int, names: Mapping[str, str],
                 activation: str = "silu") -> None:
        if activation != "silu":
            raise ValueError(f"the gated feed-forward kernels apply SiLU to the gate; {activation!r} is not implemented")
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.names = dict(names)

    def weights(self) -> dict[str, WeightWant]:
        h, i, n = self.hidden_size, self.intermediate_size, self.names
        return {n["gate"]: WeightWant((i, h)), n["up"]: WeightWant((i, h)), n["down"]: WeightWant((h, i))}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        super().bind(tensors, rt)
        n = self.names
        self.w_gate_up = rt.ops.prepare_matrix(torch.cat([tensors[n["gate"]], tensors[n["up"]]], dim=0), rt)
        self.w_down = rt.ops.prepare_matrix(tensors[n["down"]], rt)

    def weight_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_gate_up, self.w_down))

    def forward(self, x: torch.Tensor, ctx: "StepContext") -> torch.Tensor:
        rt, ops, ws = self.rt, self.rt.ops, self.rt.workspace
        t = x.shape[0]
        act = ws.get("mlp.act", (t, self.intermediate_size), rt.dtype)
        ops.linear_swiglu(x, self.w_gate_up, act)
        return ops.linear_to_residual(act, self.w_down, "mlp.delta", getattr(ctx, "residual", None))


register_feed_forward("swiglu", SwiGLU)
