"""Weights from safetensors by tensor name.

The whole checkpoint is checked against what the model wants from the files' headers alone;
tensors are then read one at a time, when a part asks for them, across shards
(``model.safetensors.index.json`` or a single ``model.safetensors``;
prefixserve/model/weights.py:62-70 of the reference) and kept as stored: bfloat16 stays bfloat16, a tensor stored in 32-bit stays 32-bit, integer tables
become int32, other float widths are widened to float32. Everything that is wrong with a
checkpoint is reported in ONE error that lists missing tensors, unexpected tensors and
wrong shapes (the reference stops at the first, weights.py:91-96,137-143).
"""

from __future__ import annotations

import json
from contextlib import ExitStack
from pathlib import Path
from typing import Mapping, Sequence

import torch
from safetensors import safe_open

from prefixserve_amd.parts.base import WeightWant


class WeightLoadError(RuntimeError):
    def __init__(self, message: str, missing: Sequence[str] = (), unexpected: Sequence[str] = (),
                 wrong_shape: Sequence[tuple[str, tuple[int, ...], tuple[int, ...]]] = ()) -> None:
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)


def shard_files(model_dir: Path) -> list[Path]:
    index = model_dir / "model.safetensors.index.json"
    if index.exists():
        names = sorted(set(json.loads(index.read_text())["weight_map"].values()))
        return [model_dir / n for n in names]
    single = model_dir / "model.safetensors"
    if single.exists():
        return [single]
    raise WeightLoadError(f"no safetensors weights in {model_dir}")


def _as_kept(t: torch.Tensor) -> torch.Tensor:
    if t.dtype in (torch.bfloat16, torch.float32, torch.int32):
        return t
    if t.dtype.is_floating_point:
        return t.to(torch.float32)
    if t.dtype == torch.bool:
        return t
    return t.to(torch.int32)


class CheckpointTensors(Mapping[str, torch.Tensor]):
    """name -> tensor on the host, read from its file when asked for and not kept: a part that
    binds takes its tensors to the device and lets go of the host copies, so the host holds
    one part's tensors at a time, not the checkpoint (the reference reads tensor by tensor for
    the same reason, prefixserve/model/weights.py:9-12). ``close()`` lets go of the files."""

    def __init__(self, stack: ExitStack, where: Mapping[str, object], names: Sequence[str]) -> None:
        self._stack, self._where, self._names = stack, where, list(names)
        self._wanted = frozenset(self._names)

    def __getitem__(self, name: str) -> torch.Tensor:
        if name not in self._where or name not in self._wanted:
            raise KeyError(name)
        return _as_kept(self._where[name].get_tensor(name))  # type: ignore[attr-defined]

    def __iter__(self):
        return iter(self._names)

    def __len__(self) -> int:
        return len(self._names)

    def close(self) -> None:
        self._stack.close()
        self._where = {}

    def __enter__(self) -> "CheckpointTensors":
        return self

    def __exit__(self, *exc) -> None:
        self.close()


def load_weights(model_dir: str | Path, wanted: Mapping[str, WeightWant],
                 ignored_suffixes: Sequence[str] = ()) -> CheckpointTensors:
    """name -> tensor (on the host, read on demand) for every wanted name, after checking the
    whole checkpoint against ``wanted``: names and shapes come from the files' headers."""
    model_dir = Path(model_dir)
    stack = ExitStack()
    try:
        where: dict[str, object] = {}
        for f in shard_files(model_dir):
            if not f.exists():
                raise WeightLoadError(f"shard {f} named by the index is missing")
            handle = stack.enter_context(safe_open(str(f), framework="pt", device="cpu"))
            for name in handle.keys():
                where[name] = handle

        missing = [n for n in wanted if n not in where]
        unexpected = [n for n in where if n not in wanted and not any(n.endswith(s) for s in ignored_suffixes)]
        wrong: list[tuple[str, tuple[int, ...], tuple[int, ...]]] = []
        for name, want in wanted.items():
            h = where.get(name)
            if h is None:
                continue
            shape = tuple(h.get_slice(name).get_shape())  # type: ignore[attr-defined]
            if shape != tuple(want.shape):
                wrong.append((name, shape, tuple(want.shape)))
        if missing or unexpected or wrong:
            lines = [f"checkpoint in {model_dir} does not fit the model:"]
            if missing:
                lines.append(f"  missing ({len(missing)}): " + ", ".join(sorted(missing)))
            if unexpected:
                lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(sorted(unexpected)))
            if wrong:
                lines.append(f"  wrong shape ({len(wrong)}): " + ", ".join(
                    f"{n} is {list(got)}, expected {list(exp)}" for n, got, exp in sorted(wrong)))
            raise WeightLoadError("\n".join(lines), missing, unexpected, wrong)
        return CheckpointTensors(stack, where, list(wanted))
    except BaseException:
        stack.close()
        raise
