"""Random-weights mode: writes a model folder (config.json, model.safetensors) from a
configuration and a seed, which then loads like any checkpoint.

The reference has no such mode (its tests let another library build and save a random
model, tests/test_llama_exact.py:50-87). Matrices and the token table are N(0, std),
norm weights 1 + N(0, norm_std) so that a forgotten weight multiply shows. Each tensor has
its own generator seeded from (seed, tensor name): the values do not depend on the order
or on which other tensors exist.
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path
from typing import Any, Mapping

import torch
from safetensors.torch import save_file

from prefixserve_amd.config.registry import architecture_of
from prefixserve_amd.parts.base import WeightWant
from prefixserve_amd.parts.model import DecoderModel

STORE_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def _seed_for(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & ((1 << 63) - 1)


def random_tensors(wanted: Mapping[str, WeightWant], seed: int, std: float = 0.02, norm_std: float = 0.1,
                   dtype: torch.dtype = torch.bfloat16) -> dict[str, torch.Tensor]:
    out: dict[str, torch.Tensor] = {}
    for name, want in wanted.items():
        g = torch.Generator().manual_seed(_seed_for(seed, name))
        t = torch.empty(want.shape, dtype=torch.float32).normal_(0.0, 1.0, generator=g)
        if want.init == "norm":
            t = 1.0 + norm_std * t
        else:
            t = std * t
        out[name] = t.to(dtype).contiguous()
    return out


def write_random_model(model_dir: str | Path, config_json: Mapping[str, Any], seed: int, std: float = 0.02,
                       norm_std: float = 0.1, store_dtype: str = "bfloat16") -> Path:
    """Writes ``config.json`` and ``model.safetensors`` for the architecture that
    ``config_json`` names. Returns the folder."""
    import prefixserve_amd.models  # noqa: F401  (fills the registry)

    model_dir = Path(model_dir)
    model_dir.mkdir(parents=True, exist_ok=True)
    arch = architecture_of(config_json)
    cfg = arch.config_cls.from_dicts(config_json, {})
    model = DecoderModel(arch.build_spec(cfg))
    tensors = random_tensors(model.weights(), seed, std, norm_std, STORE_DTYPES[store_dtype])
    (model_dir / "config.json").write_text(json.dumps(dict(config_json), indent=2))
    save_file(tensors, str(model_dir / "model.safetensors"), metadata={"format": "pt", "seed": str(seed)})
    return model_dir
