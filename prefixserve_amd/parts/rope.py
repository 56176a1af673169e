"""Rotary position encoding (rotate-half layout) with optional llama3 frequency scaling."""

from __future__ import annotations

import math
from typing import Any, Mapping

import torch

from .base import RotaryTable, Runtime, register_position


def rope_inv_freq(head_dim: int, theta: float, scaling: Mapping[str, Any] | None) -> torch.Tensor:
    """inv_freq[i] = 1 / theta^(2i/D), i < D/2, then the llama3 three bands by wavelength:
    long waves divided by ``factor``, short ones unchanged, the middle blended
    (prefixserve/model/llama.py:24-46 of the reference). Evaluated in float64 and rounded
    once to float32, which agrees with the reference's float32 evaluation to one ulp and
    does not depend on a library's ``pow``."""
    i = torch.arange(0, head_dim, 2, dtype=torch.float64)
    inv = 1.0 / (torch.tensor(float(theta), dtype=torch.float64) ** (i / head_dim))
    if scaling is not None:
        factor = float(scaling["factor"])
        low = float(scaling["low_freq_factor"])
        high = float(scaling["high_freq_factor"])
        old = float(scaling["original_max_position_embeddings"])
        low_wavelen, high_wavelen = old / low, old / high
        wavelen = 2.0 * math.pi / inv
        scaled = torch.where(wavelen > low_wavelen, inv / factor, inv)
        smooth = (old / wavelen - low) / (high - low)
        smoothed = (1.0 - smooth) * scaled / factor + smooth * scaled
        medium = ~(wavelen < high_wavelen) & ~(wavelen > low_wavelen)
        inv = torch.where(medium, smoothed, scaled)
    return inv.to(torch.float32)


class RotaryEmbedding(RotaryTable):
    """Pairs (i, i + D/2) of every head are rotated by angle = position * inv_freq[i]
    (prefixserve/model/llama.py:72-77). The angle is a float32 product as in the
    reference's table (llama.py:56-58); its cosine and sine are kept in float32 whatever
    the activation dtype. The table is ``[max_position, D/2, 2]`` = (cos, sin) and is
    read by the kernel that also writes keys and values into their pages."""

    def __init__(self, head_dim: int, theta: float, scaling: Mapping[str, Any] | None = None) -> None:
        if head_dim % 2:
            raise ValueError(f"rotary head_dim must be even, got {head_dim}")
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.scaling = dict(scaling) if scaling is not None else None
        self.table: torch.Tensor | None = None

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        super().bind(tensors, rt)

    def prepare(self, max_position: int) -> None:
        inv = rope_inv_freq(self.head_dim, self.theta, self.scaling)
        pos = torch.arange(max_position, dtype=torch.float32)
        angle = torch.outer(pos, inv)  # float32 product, exactly rounded
        a64 = angle.to(torch.float64)
        table = torch.stack((a64.cos(), a64.sin()), dim=-1).to(torch.float32)
        self.table = table.contiguous().to(self.rt.device)
        self.max_position = int(max_position)


register_position("rope", RotaryEmbedding)
