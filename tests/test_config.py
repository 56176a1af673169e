"""Configuration parsing and the architecture registry. Vectors are the reference's
(tests/test_llama_config.py:18-64)."""

from __future__ import annotations

import json

import pytest

import prefixserve_amd.models  # noqa: F401
from prefixserve_amd.config import (Llama3RopeScaling, LlamaConfig, UnknownArchitectureError, UnsupportedModelError,
                                    architecture_of, read_model_dir, registered_architectures)
from prefixserve_amd.parts import DecoderModel

SCALING = {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
           "original_max_position_embeddings": 8192, "rope_type": "llama3"}
WANT = Llama3RopeScaling(8.0, 1.0, 4.0, 8192)


def base(**kw):
    cfg = {"model_type": "llama", "vocab_size": 128256, "hidden_size": 4096, "intermediate_size": 14336,
           "num_hidden_layers": 32, "num_attention_heads": 32, "num_key_value_heads": 8, "rms_norm_eps": 1e-5,
           "max_position_embeddings": 131072, "eos_token_id": 128001}
    cfg.update(kw)
    return cfg


def test_transformers4_layout():
    c = LlamaConfig.from_dicts(base(rope_theta=500000.0, rope_scaling=SCALING), {"eos_token_id": [128001, 128008, 128009]})
    assert c.rope_theta == 500000.0 and c.rope_scaling == WANT
    assert c.head_dim == 128 and c.q_size == 4096 and c.kv_size == 1024
    assert c.stop_token_ids == {128001, 128008, 128009}


def test_transformers5_layout():
    c = LlamaConfig.from_dicts(base(rope_parameters={**SCALING, "rope_theta": 500000.0}))
    assert c.rope_theta == 500000.0 and c.rope_scaling == WANT


def test_no_scaling_and_defaults():
    for raw in (base(rope_theta=500000.0), base(rope_parameters={"rope_type": "default", "rope_theta": 500000.0})):
        c = LlamaConfig.from_dicts(raw)
        assert c.rope_theta == 500000.0 and c.rope_scaling is None
    c = LlamaConfig.from_dicts(base())
    assert c.rope_theta == 10000.0 and not c.tie_word_embeddings
    assert LlamaConfig.from_dicts(base(rope_theta=1.0)).stop_token_ids == {128001}
    assert LlamaConfig.from_dicts(base(head_dim=64)).head_dim == 64
    assert LlamaConfig.from_dicts(base(head_dim=None)).head_dim == 128
    c = LlamaConfig.from_dicts({k: v for k, v in base().items() if k != "num_key_value_heads"})
    assert c.num_kv_heads == 32


@pytest.mark.parametrize("bad", [
    {"model_type": "mistral"}, {"rope_scaling": {"rope_type": "yarn", "factor": 4.0}},
    {"attention_bias": True}, {"mlp_bias": True}, {"num_key_value_heads": 5},
])
def test_refuses_what_it_cannot_run(bad):
    with pytest.raises(UnsupportedModelError):
        LlamaConfig.from_dicts(base(**bad))


def test_missing_required_key_raises():
    raw = base()
    del raw["rms_norm_eps"]
    with pytest.raises(KeyError):
        LlamaConfig.from_dicts(raw)
    with pytest.raises(KeyError):
        LlamaConfig.from_dicts(base(rope_scaling={"rope_type": "llama3", "factor": 8.0}))


def test_roundtrip_through_config_json():
    c = LlamaConfig.from_dicts(base(rope_theta=500000.0, rope_scaling=SCALING, tie_word_embeddings=True))
    assert LlamaConfig.from_dicts(c.to_config_json()) == c


def test_registry(tmp_path):
    assert "LlamaForCausalLM" in registered_architectures()
    with pytest.raises(UnknownArchitectureError, match="LlamaForCausalLM"):
        architecture_of({"architectures": ["MysteryForCausalLM"]})
    with pytest.raises(UnknownArchitectureError):
        architecture_of({"model_type": "llama"})
    raw = base(architectures=["LlamaForCausalLM"], rope_theta=500000.0, rope_scaling=SCALING)
    (tmp_path / "config.json").write_text(json.dumps(raw))
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [1, 2]}))
    arch, cfg, _ = read_model_dir(tmp_path)
    assert arch.name == "LlamaForCausalLM" and cfg.stop_token_ids == {1, 2}


def test_spec_has_no_size_of_its_own():
    """Every size of the built model comes from the configuration."""
    from configs import TINY

    for raw in TINY.values():
        cfg = LlamaConfig.from_dicts(raw)
        arch = architecture_of(raw)
        spec = arch.build_spec(cfg)
        model = DecoderModel(spec)
        want = model.weights()
        h, q, kv, i = cfg.hidden_size, cfg.q_size, cfg.kv_size, cfg.intermediate_size
        assert want["model.embed_tokens.weight"].shape == (cfg.vocab_size, h)
        assert want["model.layers.0.self_attn.q_proj.weight"].shape == (q, h)
        assert want["model.layers.0.self_attn.k_proj.weight"].shape == (kv, h)
        assert want["model.layers.0.self_attn.o_proj.weight"].shape == (h, q)
        assert want["model.layers.0.mlp.gate_proj.weight"].shape == (i, h)
        assert want["model.layers.0.mlp.down_proj.weight"].shape == (h, i)
        assert want["model.norm.weight"].shape == (h,)
        assert ("lm_head.weight" in want) == (not cfg.tie_word_embeddings)
        assert len(spec.layers) == cfg.num_layers and len(spec.order) == cfg.num_layers
        n = 9 * cfg.num_layers + 2 + (0 if cfg.tie_word_embeddings else 1)
        assert len(want) == n
