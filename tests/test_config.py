"""Reading config.json into the typed configuration, and the registry from architecture names
to models. The 8B numbers and the four refusals are those of the reference's own test
(tests/test_llama_config.py:18-64)."""

from __future__ import annotations

import json

import pytest

import prefixserve_amd.models  # noqa: F401
from prefixserve_amd.config import (Llama3RopeScaling, LlamaConfig, UnknownArchitectureError, UnsupportedModelError,
                                    architecture_of, read_model_dir, registered_architectures)
from prefixserve_amd.parts import DecoderModel

LLAMA3_RULE = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                   original_max_position_embeddings=8192)
SCALING = LLAMA3_RULE


def base(**changes):
    """config.json of the 8B model without its rope entries, plus ``changes``."""
    raw = dict(model_type="llama", vocab_size=128256, hidden_size=4096, intermediate_size=14336, num_hidden_layers=32,
               num_attention_heads=32, num_key_value_heads=8, rms_norm_eps=1e-5, max_position_embeddings=131072,
               eos_token_id=128001)
    raw.update(changes)
    return raw


def parse(gen=None, **changes):
    return LlamaConfig.from_dicts(base(**changes), gen)


@pytest.mark.parametrize("layout", ["top-level keys", "one rope_parameters dict"])
def test_rope_entries_in_either_layout(layout):
    if layout == "top-level keys":
        cfg = parse(rope_theta=500000.0, rope_scaling=LLAMA3_RULE)
    else:
        cfg = parse(rope_parameters=dict(LLAMA3_RULE, rope_theta=500000.0))
    assert cfg.rope_theta == 500000.0
    assert cfg.rope_scaling == Llama3RopeScaling(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                                 original_max_position_embeddings=8192)


def test_sizes_that_follow_from_the_keys():
    cfg = parse()
    assert (cfg.head_dim, cfg.q_size, cfg.kv_size) == (128, 4096, 1024)
    assert parse(head_dim=64).head_dim == 64 and parse(head_dim=None).head_dim == 128
    without_kv = base()
    without_kv.pop("num_key_value_heads")
    assert LlamaConfig.from_dicts(without_kv).num_kv_heads == 32


def test_defaults_and_stop_ids():
    cfg = parse()
    assert cfg.rope_theta == 10000.0 and cfg.rope_scaling is None and cfg.tie_word_embeddings is False
    assert cfg.stop_token_ids == {128001}
    assert parse(gen={"eos_token_id": [128001, 128008, 128009]}).stop_token_ids == {128001, 128008, 128009}
    for no_rule in (dict(rope_theta=500000.0), dict(rope_parameters={"rope_type": "default", "rope_theta": 500000.0})):
        cfg = parse(**no_rule)
        assert cfg.rope_theta == 500000.0 and cfg.rope_scaling is None


@pytest.mark.parametrize("change", [dict(model_type="mistral"), dict(rope_scaling={"rope_type": "yarn", "factor": 4.0}),
                                    dict(attention_bias=True), dict(mlp_bias=True), dict(num_key_value_heads=5),
                                    dict(hidden_act="gelu")])
def test_what_cannot_run_is_refused(change):
    with pytest.raises(UnsupportedModelError):
        parse(**change)


def test_a_key_that_is_needed_and_missing_is_named():
    incomplete = base()
    incomplete.pop("rms_norm_eps")
    with pytest.raises(KeyError, match="rms_norm_eps"):
        LlamaConfig.from_dicts(incomplete)
    with pytest.raises(KeyError, match="low_freq_factor"):
        parse(rope_scaling={"rope_type": "llama3", "factor": 8.0})


def test_what_is_written_reads_back():
    cfg = parse(rope_theta=500000.0, rope_scaling=LLAMA3_RULE, tie_word_embeddings=True)
    assert LlamaConfig.from_dicts(cfg.to_config_json()) == cfg
    plain = parse()
    assert LlamaConfig.from_dicts(plain.to_config_json()) == plain


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
