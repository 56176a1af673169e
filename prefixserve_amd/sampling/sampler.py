"""Greedy and temperature sampling.

The reference samples greedily only (prefixserve/llama_engine.py:146; its server refuses a
temperature, prefixserve/server.py:427-428). Here a request may carry a temperature:
p = softmax(logits / T) in float32 and a draw by inverse CDF in vocabulary order. The
uniform number is a function of (seed, request, index of the output token) alone, never of
the step or the batch slot, so a request that was preempted and recomputed, or batched
differently, draws the same tokens. Temperature 0 is greedy with the lowest index winning
ties. The draw itself runs in a device kernel over the step's logits.
"""

from __future__ import annotations

import zlib
from typing import Any, Sequence

import torch

_M64 = (1 << 64) - 1


def _mix64(z: int) -> int:
    z = (z + 0x9E3779B97F4A7C15) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def request_key(req_id: str) -> int:
    """A stable 64-bit key of a request id (Python's own hash() differs between runs)."""
    data = req_id.encode()
    return (zlib.crc32(data) << 32) | zlib.adler32(data)


def uniform_for(seed: int, key: int, output_index: int) -> float:
    """u in [0, 1) with 24 random bits: a chain of splitmix64 finalizers over the three inputs."""
    z = _mix64(seed & _M64)
    z = _mix64(z ^ (key & _M64))
    z = _mix64(z ^ (output_index & _M64))
    return (z >> 40) / float(1 << 24)


class Sampler:
    """Draws one token per logits row on the device and brings the ids to the host in one copy."""

    def __init__(self, ops: Any, device: torch.device, max_rows: int = 1024) -> None:
        self.ops = ops
        self.device = torch.device(device)
        self._alloc(max_rows)

    def _alloc(self, rows: int) -> None:
        pin = self.device.type == "cuda"
        # Temperatures, then uniform numbers: one contiguous host-to-device copy.
        self._host = torch.empty(2 * rows, dtype=torch.float32, pin_memory=pin)
        self._host_np = self._host.numpy()
        self._dev = torch.zeros(2 * rows, dtype=torch.float32, device=self.device)
        self._out = torch.empty(rows, dtype=torch.int32, device=self.device)
        self._out_host = torch.empty(rows, dtype=torch.int32, pin_memory=pin)
        self._out_np = self._out_host.numpy()
        self.max_rows = rows
        self._greedy_rows = rows     # leading rows of the device copy known to hold temperature 0

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], uniforms: Sequence[float]) -> list[int]:
        rows = logits.shape[0]
        if len(temperatures) != rows or len(uniforms) != rows:
            raise ValueError("one temperature and one uniform number per logits row")
        if rows > self.max_rows:
            self._alloc(max(rows, 2 * self.max_rows))
        n = self.max_rows
        greedy = not any(t > 0 for t in temperatures)
        if not (greedy and self._greedy_rows >= rows):     # an all-greedy batch reads zeros already there
            self._host_np[:rows] = temperatures
            self._host_np[n:n + rows] = uniforms
            if self.device.type == "cuda":
                self._dev[:n + rows].copy_(self._host[:n + rows], non_blocking=True)
            else:
                self._dev[:n + rows] = self._host[:n + rows]
            self._greedy_rows = rows if greedy else 0
        out = self._out[:rows]
        self.ops.sample(logits, self._dev[:rows], self._dev[n:n + rows], out)
        # The step's one device-to-host wait.
        if self.device.type == "cuda":
            self._out_host[:rows].copy_(out, non_blocking=True)
            torch.cuda.current_stream(self.device).synchronize()
            return self._out_np[:rows].tolist()
        return out.tolist()

    # ---- several steps in a row: nothing here waits for the device but ``fetch``

    def stage_steps(self, temperatures: Sequence[float], uniforms: Sequence[Sequence[float]]):
        """Device copies of the temperatures and of one row of uniform numbers per step, made
        with one host-to-device copy; and a device buffer for ``len(uniforms)`` rows of tokens."""
        rows, steps = len(temperatures), len(uniforms)
        need = (steps + 1) * rows
        if getattr(self, "_steps_cap", 0) < need:
            pin = self.device.type == "cuda"
            self._steps_host = torch.empty(need, dtype=torch.float32, pin_memory=pin)
            self._steps_dev = torch.zeros(need, dtype=torch.float32, device=self.device)
            self._steps_out = torch.empty(need, dtype=torch.int32, device=self.device)
            self._steps_out_host = torch.empty(need, dtype=torch.int32, pin_memory=pin)
            self._steps_cap = need
            self._steps_greedy = need
        greedy = not any(t > 0 for t in temperatures)
        if not (greedy and self._steps_greedy >= need):
            host = self._steps_host.numpy()
            host[:rows] = temperatures
            for j, u in enumerate(uniforms):
                host[(j + 1) * rows:(j + 2) * rows] = u
            self._steps_dev[:need].copy_(self._steps_host[:need], non_blocking=True)
            self._steps_greedy = need if greedy else 0
        temps = self._steps_dev[:rows]
        return temps, [self._steps_dev[(j + 1) * rows:(j + 2) * rows] for j in range(steps)], \
            [self._steps_out[j * rows:(j + 1) * rows] for j in range(steps)]

    def sample_into(self, logits: torch.Tensor, temperatures: torch.Tensor, uniforms: torch.Tensor,
                    out: torch.Tensor) -> None:
        self.ops.sample(logits, temperatures, uniforms, out)

    def fetch(self, steps: int, rows: int) -> list[list[int]]:
        """The tokens of ``stage_steps``' output rows: the one device-to-host wait."""
        n = steps * rows
        if self.device.type == "cuda":
            self._steps_out_host[:n].copy_(self._steps_out[:n], non_blocking=True)
            torch.cuda.current_stream(self.device).synchronize()
            flat = self._steps_out_host.numpy()[:n]
        else:
            flat = self._steps_out[:n].numpy()
        return flat.reshape(steps, rows).tolist()
