"""RMSNorm fused with the residual sum in front of it."""

from __future__ import annotations

from typing import Mapping

import torch

from .base import Norm, NormedRows, Runtime, WeightWant, register_norm


class RMSNorm(Norm):
    """weight * x * rsqrt(mean(x^2) + eps), eps inside the root; statistics, scale and the
    residual sum in 32-bit (prefixserve/model/llama.py:63-69 of the reference upcasts the
    same way). The weight is used in the dtype it is stored in."""

    def __init__(self, hidden_size: int, eps: float, name: str = "weight") -> None:
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        self.name = name

    def weights(self) -> dict[str, WeightWant]:
        return {self.name: WeightWant((self.hidden_size,), "norm")}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        super().bind(tensors, rt)
        w = tensors[self.name]
        if w.dtype not in (torch.bfloat16, torch.float32):
            w = w.to(torch.float32)
        self.weight = w.to(rt.device).contiguous()

    def weight_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()

    def _lazy(self, count: int) -> bool:
        """Whether the kernels of this runtime normalize ``count`` rows of this width themselves."""
        fuses = getattr(self.rt.ops, "fuses_norm", None)
        return fuses is not None and fuses(count, self.hidden_size, self.rt.dtype)

    def add_norm(self, residual: torch.Tensor, delta: torch.Tensor | None, out_name: str,
                 lazy: bool = False) -> torch.Tensor | NormedRows:
        rt = self.rt
        if lazy and delta is None and self._lazy(residual.shape[0]):
            return NormedRows(residual, self.weight, self.eps, rt.dtype)
        out = rt.workspace.get(out_name, (residual.shape[0], self.hidden_size), rt.dtype)
        rt.ops.add_rmsnorm(residual, delta, self.weight, self.eps, out)
        return out

    def add_norm_rows(self, residual: torch.Tensor, delta: torch.Tensor | None, rows: torch.Tensor,
                      out_name: str, lazy: bool = False) -> torch.Tensor | NormedRows:
        rt = self.rt
        if lazy and delta is None and self._lazy(rows.shape[0]):
            return NormedRows(residual, self.weight, self.eps, rt.dtype, rows)
        out = rt.workspace.get(out_name, (rows.shape[0], self.hidden_size), rt.dtype)
        rt.ops.add_rmsnorm_rows(residual, delta, rows, self.weight, self.eps, out)
        return out


register_norm("rmsnorm", RMSNorm)
