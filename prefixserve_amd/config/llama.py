"""Typed Llama configuration read from the architecture's own ``config.json`` keys.

Key names, defaults and refusals follow prefixserve/model/config.py:54-120 of the
reference: both the transformers-4 layout (top-level ``rope_theta`` + ``rope_scaling``)
and the transformers-5 layout (one ``rope_parameters`` dict); stop ids from
``generation_config.json`` first; anything not understood raises instead of being
ignored, because a silently dropped ``rope_scaling`` loads fine and writes garbage at
long positions.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Mapping


class UnsupportedModelError(ValueError):
    """The folder describes a model this engine cannot run."""


@dataclass(frozen=True)
class Llama3RopeScaling:
    """The "llama3" three-band frequency scaling (prefixserve/model/config.py:20-27)."""

    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int


@dataclass(frozen=True)
class LlamaConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: Llama3RopeScaling | None
    max_position_embeddings: int
    tie_word_embeddings: bool
    stop_token_ids: frozenset[int]

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @classmethod
    def from_dir(cls, path: str | Path) -> "LlamaConfig":
        path = Path(path)
        raw = json.loads((path / "config.json").read_text())
        gen_path = path / "generation_config.json"
        gen = json.loads(gen_path.read_text()) if gen_path.exists() else {}
        return cls.from_dicts(raw, gen)

    @classmethod
    def from_dicts(cls, raw: Mapping[str, Any], gen: Mapping[str, Any] | None = None) -> "LlamaConfig":
        if raw.get("model_type") != "llama":
            raise UnsupportedModelError(f"model_type {raw.get('model_type')!r} is not 'llama'")
        heads = int(raw["num_attention_heads"])
        kv_heads = int(raw.get("num_key_value_heads", heads))
        if kv_heads < 1 or heads % kv_heads:
            raise UnsupportedModelError(f"{heads} query heads not divisible by {kv_heads} KV heads")
        hidden = int(raw["hidden_size"])
        head_dim = int(raw.get("head_dim") or hidden // heads)
        rope_params = raw.get("rope_parameters") or {}
        rope = raw.get("rope_parameters") or raw.get("rope_scaling")
        theta_raw = rope_params.get("rope_theta", raw.get("rope_theta"))
        theta = float(theta_raw) if theta_raw is not None else 10000.0
        if raw.get("attention_bias") or raw.get("mlp_bias"):
            raise UnsupportedModelError("biases in attention/MLP are not supported")
        eos = (gen or {}).get("eos_token_id", raw.get("eos_token_id"))
        stop = frozenset(int(t) for t in (eos if isinstance(eos, list) else [eos]) if t is not None)
        return cls(
            vocab_size=int(raw["vocab_size"]),
            hidden_size=hidden,
            intermediate_size=int(raw["intermediate_size"]),
            num_layers=int(raw["num_hidden_layers"]),
            num_heads=heads,
            num_kv_heads=kv_heads,
            head_dim=head_dim,
            rms_norm_eps=float(raw["rms_norm_eps"]),
            rope_theta=theta,
            rope_scaling=_parse_rope_scaling(rope),
            max_position_embeddings=int(raw["max_position_embeddings"]),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            stop_token_ids=stop,
        )

    def to_config_json(self) -> dict[str, Any]:
        """The ``config.json`` this configuration is read back from (used by the
        random-weights mode to write a model folder)."""
        raw: dict[str, Any] = {
            "architectures": ["LlamaForCausalLM"],
            "model_type": "llama",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_layers,
            "num_attention_heads": self.num_heads,
            "num_key_value_heads": self.num_kv_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": None,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "attention_bias": False,
            "mlp_bias": False,
        }
        if self.rope_scaling is not None:
            rs = self.rope_scaling
            raw["rope_scaling"] = {
                "rope_type": "llama3",
                "factor": rs.factor,
                "low_freq_factor": rs.low_freq_factor,
                "high_freq_factor": rs.high_freq_factor,
                "original_max_position_embeddings": rs.original_max_position_embeddings,
            }
        if self.stop_token_ids:
            ids = sorted(self.stop_token_ids)
            raw["eos_token_id"] = ids[0] if len(ids) == 1 else ids
        return raw


def _parse_rope_scaling(rs: Mapping[str, Any] | None) -> Llama3RopeScaling | None:
    if rs is None:
        return None
    kind = rs.get("rope_type", rs.get("type"))
    if kind in (None, "default"):
        return None
    if kind != "llama3":
        raise UnsupportedModelError(f"rope_scaling type {kind!r} is not supported")
    return Llama3RopeScaling(
        factor=float(rs["factor"]),
        low_freq_factor=float(rs["low_freq_factor"]),
        high_freq_factor=float(rs["high_freq_factor"]),
        original_max_position_embeddings=int(rs["original_max_position_embeddings"]),
    )
