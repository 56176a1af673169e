"""Weight loading: by name, stored dtype kept, one error that lists everything wrong."""

from __future__ import annotations

import json

import pytest
import torch
from safetensors.torch import load_file, save_file

import prefixserve_amd.models  # noqa: F401
from configs import TINY
from prefixserve_amd.config import architecture_of
from prefixserve_amd.parts import DecoderModel
from prefixserve_amd.weights import WeightLoadError, load_weights, write_random_model


def wanted(name="A"):
    raw = TINY[name]
    arch = architecture_of(raw)
    spec = arch.build_spec(arch.config_cls.from_dicts(raw, {}))
    return DecoderModel(spec).weights(), spec


def test_random_model_loads_and_is_reproducible(tmp_path):
    a = write_random_model(tmp_path / "a", TINY["B"], seed=3)
    b = write_random_model(tmp_path / "b", TINY["B"], seed=3)
    c = write_random_model(tmp_path / "c", TINY["B"], seed=4)
    want, spec = wanted("B")
    ta, tb, tc = (load_weights(d, want, spec.ignored_weights) for d in (a, b, c))
    assert set(ta) == set(want)
    assert all(torch.equal(ta[k], tb[k]) for k in ta)
    assert any(not torch.equal(ta[k], tc[k]) for k in ta)
    assert all(t.dtype == torch.bfloat16 for t in ta.values())
    norm = ta["model.layers.1.input_layernorm.weight"].float()
    assert 0.05 < (norm - 1).abs().max() < 1.0                       # 1 + N(0, 0.1)
    mat = ta["model.layers.1.mlp.down_proj.weight"].float()
    assert abs(float(mat.std()) - 0.02) < 0.004 and abs(float(mat.mean())) < 0.002
    assert json.loads((a / "config.json").read_text())["architectures"] == ["LlamaForCausalLM"]


def test_stored_dtypes_are_kept(tmp_path):
    d = write_random_model(tmp_path / "m", TINY["A"], seed=1)
    t = load_file(str(d / "model.safetensors"))
    t["model.norm.weight"] = t["model.norm.weight"].float()           # a 32-bit tensor stays 32-bit
    t["model.layers.0.mlp.up_proj.weight"] = t["model.layers.0.mlp.up_proj.weight"].to(torch.float16)
    save_file(t, str(d / "model.safetensors"))
    want, spec = wanted("A")
    got = load_weights(d, want, spec.ignored_weights)
    assert got["model.norm.weight"].dtype == torch.float32
    assert got["model.embed_tokens.weight"].dtype == torch.bfloat16
    assert got["model.layers.0.mlp.up_proj.weight"].dtype == torch.float32   # other widths widen


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = write_random_model(tmp_path / "m", TINY["A"], seed=1)
    t = load_file(str(d / "model.safetensors"))
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(3, 5, dtype=torch.bfloat16)
    t["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(4, dtype=torch.bfloat16)
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)            # recomputed: tolerated
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()                  # tied: tolerated
    save_file(t, str(d / "model.safetensors"))
    want, spec = wanted("A")
    with pytest.raises(WeightLoadError) as e:
        load_weights(d, want, spec.ignored_weights)
    err = e.value
    assert sorted(err.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.q_norm.weight"]
    assert err.wrong_shape == [("model.layers.0.self_attn.q_proj.weight", (3, 5), (64, 64))]
    msg = str(err)
    for needle in ("missing (2)", "unexpected (1)", "wrong shape (1)", "q_norm", "up_proj", "[3, 5]", "[64, 64]"):
        assert needle in msg


def test_untied_model_requires_its_head(tmp_path):
    d = write_random_model(tmp_path / "m", TINY["B"], seed=1)
    t = load_file(str(d / "model.safetensors"))
    del t["lm_head.weight"]
    save_file(t, str(d / "model.safetensors"))
    want, spec = wanted("B")
    with pytest.raises(WeightLoadError, match="lm_head.weight"):
        load_weights(d, want, spec.ignored_weights)


def test_sharded_checkpoint_and_no_weights(tmp_path):
    d = write_random_model(tmp_path / "m", TINY["A"], seed=1)
    t = load_file(str(d / "model.safetensors"))
    names = sorted(t)
    half = len(names) // 2
    save_file({k: t[k] for k in names[:half]}, str(d / "model-00001-of-00002.safetensors"))
    save_file({k: t[k] for k in names[half:]}, str(d / "model-00002-of-00002.safetensors"))
    index = {"weight_map": {k: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
                            for i, k in enumerate(names)}}
    (d / "model.safetensors.index.json").write_text(json.dumps(index))
    (d / "model.safetensors").unlink()
    want, spec = wanted("A")
    got = load_weights(d, want, spec.ignored_weights)
    assert all(torch.equal(got[k], t[k]) for k in names)
    empty = tmp_path / "empty"
    empty.mkdir()
    with pytest.raises(WeightLoadError, match="no safetensors"):
        load_weights(empty, want)


def test_tensors_are_read_when_asked_for_and_not_kept(tmp_path):
    """The loader checks the checkpoint from the headers and hands out a mapping that reads a
    tensor from its file on every access (the host never holds the whole checkpoint); closed,
    it lets go of the files."""
    from configs import TINY
    from prefixserve_amd.config import read_model_dir
    from prefixserve_amd.parts import DecoderModel

    d = write_random_model(tmp_path, TINY["A"], seed=3, std=0.1)
    arch, cfg, _ = read_model_dir(d)
    spec = arch.build_spec(cfg)
    want = DecoderModel(spec).weights()
    got = load_weights(d, want, spec.ignored_weights)
    assert not isinstance(got, dict) and set(got) == set(want) and len(got) == len(want)
    name = "model.layers.0.mlp.down_proj.weight"
    first, second = got[name], got[name]
    assert first is not second and torch.equal(first, second)
    with pytest.raises(KeyError):
        got["no.such.tensor"]
    got.close()
    with pytest.raises(KeyError):
        got[name]
