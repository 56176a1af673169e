"""The Llama architecture's configuration, typed, from its own ``config.json`` keys.

Which keys are read, their defaults and what is refused are those of the reference's
parser (prefixserve/model/config.py:54-120): the rope base and scaling may stand at the
top level (``rope_theta``, ``rope_scaling``) or together in one ``rope_parameters`` dict
(the newer layout of the same checkpoints); stop ids come from ``generation_config.json``
when it has them. A key that changes the arithmetic and is not understood raises: a
scaling rule dropped without a word would load and then write nonsense at long positions.
"""

from __future__ import annotations

import json
from dataclasses import dataclass, fields
from pathlib import Path
from typing import Any, Mapping

ARCHITECTURE = "LlamaForCausalLM"
MODEL_TYPE = "llama"
DEFAULT_ROPE_THETA = 10000.0
HIDDEN_ACT = "silu"          # the gate of the feed-forward; the one activation the kernels implement

# dataclass field -> config.json key, for the sizes that must be there and are plain integers
_INT_KEYS = {
    "vocab_size": "vocab_size",
    "hidden_size": "hidden_size",
    "intermediate_size": "intermediate_size",
    "num_layers": "num_hidden_layers",
    "num_heads": "num_attention_heads",
    "max_position_embeddings": "max_position_embeddings",
}
_SCALING_KEYS = ("factor", "low_freq_factor", "high_freq_factor", "original_max_position_embeddings")


class UnsupportedModelError(ValueError):
    """config.json describes something this engine does not run."""


@dataclass(frozen=True)
class Llama3RopeScaling:
    """The "llama3" rule: long waves are slowed by ``factor``, short ones kept, those between
    blended; the bands are set by the two frequency factors and the original context length."""

    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int

    @classmethod
    def from_json(cls, entry: Mapping[str, Any] | None) -> "Llama3RopeScaling | None":
        """None for no entry and for the kind "default"; any other kind but "llama3" is refused."""
        if not entry:
            return None
        kind = entry["rope_type"] if "rope_type" in entry else entry.get("type")
        if kind is None or kind == "default":
            return None
        if kind != "llama3":
            raise UnsupportedModelError(f"rope scaling of kind {kind!r}: only 'llama3' is implemented")
        values = [entry[k] for k in _SCALING_KEYS]          # KeyError names what is missing
        return cls(float(values[0]), float(values[1]), float(values[2]), int(values[3]))

    def to_json(self) -> dict[str, Any]:
        return {"rope_type": "llama3", **{k: getattr(self, k) for k in _SCALING_KEYS}}


@dataclass(frozen=True)
class LlamaConfig:
    # sizes
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    max_position_embeddings: int
    # attention
    num_heads: int
    num_kv_heads: int
    head_dim: int
    # constants
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: Llama3RopeScaling | None
    tie_word_embeddings: bool
    stop_token_ids: frozenset[int]
    hidden_act: str = HIDDEN_ACT

    @property
    def q_size(self) -> int:
        """Columns of the query projection."""
        return self.head_dim * self.num_heads

    @property
    def kv_size(self) -> int:
        """Columns of the key projection, and of the value projection."""
        return self.head_dim * self.num_kv_heads

    # ------------------------------------------------------------------ reading

    @classmethod
    def from_dir(cls, model_dir: str | Path) -> "LlamaConfig":
        folder = Path(model_dir)
        generation = folder / "generation_config.json"
        return cls.from_dicts(json.loads((folder / "config.json").read_text()),
                              json.loads(generation.read_text()) if generation.exists() else None)

    @classmethod
    def from_dicts(cls, raw: Mapping[str, Any], gen: Mapping[str, Any] | None = None) -> "LlamaConfig":
        """``raw`` = config.json, ``gen`` = generation_config.json or None."""
        _refuse_what_is_not_llama(raw)
        sizes = {name: int(raw[key]) for name, key in _INT_KEYS.items()}
        heads = sizes["num_heads"]
        kv_heads = int(raw["num_key_value_heads"]) if "num_key_value_heads" in raw else heads
        if kv_heads < 1 or heads % kv_heads != 0:
            raise UnsupportedModelError(f"{heads} attention heads cannot share {kv_heads} key/value heads")
        theta, scaling = _rope_of(raw)
        return cls(
            **sizes,
            num_kv_heads=kv_heads,
            # 3.2-1B states its head size; older checkpoints leave it to hidden / heads.
            head_dim=int(raw.get("head_dim") or sizes["hidden_size"] // heads),
            rms_norm_eps=float(raw["rms_norm_eps"]),
            rope_theta=theta,
            rope_scaling=scaling,
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            stop_token_ids=_stop_ids(raw, gen),
            # The reference never reads this key and always applies SiLU (prefixserve/model/llama.py:121);
            # a file that names another activation is refused above rather than run with the wrong one.
            hidden_act=str(raw.get("hidden_act") or HIDDEN_ACT),
        )

    # ------------------------------------------------------------------ writing

    def to_config_json(self) -> dict[str, Any]:
        """A config.json that reads back as this configuration: what the random-weights mode
        writes next to its model.safetensors."""
        out: dict[str, Any] = {"architectures": [ARCHITECTURE], "model_type": MODEL_TYPE}
        out.update({key: getattr(self, name) for name, key in _INT_KEYS.items()})
        out.update(num_key_value_heads=self.num_kv_heads, head_dim=self.head_dim, rms_norm_eps=self.rms_norm_eps,
                   rope_theta=self.rope_theta, tie_word_embeddings=self.tie_word_embeddings, hidden_act=self.hidden_act,
                   attention_bias=False, mlp_bias=False,
                   rope_scaling=self.rope_scaling.to_json() if self.rope_scaling is not None else None)
        stops = sorted(self.stop_token_ids)
        if stops:
            out["eos_token_id"] = stops if len(stops) > 1 else stops[0]
        return out


assert {f.name for f in fields(LlamaConfig)} >= set(_INT_KEYS)


def _refuse_what_is_not_llama(raw: Mapping[str, Any]) -> None:
    kind = raw.get("model_type")
    if kind != MODEL_TYPE:
        raise UnsupportedModelError(f"model_type is {kind!r}, expected {MODEL_TYPE!r}")
    act = raw.get("hidden_act")
    if act is not None and act != HIDDEN_ACT:
        raise UnsupportedModelError(f"hidden_act is {act!r}: only the {HIDDEN_ACT!r} gate is implemented")
    for key in ("attention_bias", "mlp_bias"):
        if raw.get(key):
            raise UnsupportedModelError(f"{key} is set: projections with a bias are not implemented")


def _rope_of(raw: Mapping[str, Any]) -> tuple[float, Llama3RopeScaling | None]:
    """(theta, scaling) from ``rope_parameters`` if the file has that dict, else from the
    top-level ``rope_theta`` and ``rope_scaling``."""
    joint = raw.get("rope_parameters")
    if joint:
        theta = joint.get("rope_theta", raw.get("rope_theta"))
        entry = joint
    else:
        theta = raw.get("rope_theta")
        entry = raw.get("rope_scaling")
    return (DEFAULT_ROPE_THETA if theta is None else float(theta)), Llama3RopeScaling.from_json(entry)


def _stop_ids(raw: Mapping[str, Any], gen: Mapping[str, Any] | None) -> frozenset[int]:
    """eos_token_id, an integer or a list of them, from the generation config first."""
    found = gen.get("eos_token_id") if gen and "eos_token_id" in gen else raw.get("eos_token_id")
    if found is None:
        return frozenset()
    many = found if isinstance(found, (list, tuple)) else [found]
    return frozenset(int(t) for t in many if t is not None)
