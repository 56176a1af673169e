"""A toy architecture defined in the tests alone: a mixer that keeps fixed-size state per
request (a running mean over the request's tokens, no pages) alternating with attention
layers, one layer run twice and one reading another layer's cache. It is registered through
the package's public registries without touching the package's files, and is no model of
anyone's."""

from __future__ import annotations

import json
from pathlib import Path

import torch

from prefixserve_amd.config import register_architecture, registered_architectures
from prefixserve_amd.parts import (DecoderModel, LayerRun, LayerSpec, Mixer, ModelSpec, PartSpec, StateNeed, WeightWant,
                                   register_mixer)

TOY_MEAN_CONFIG = {"architectures": ["ToyMeanForCausalLM"], "hidden_size": 64, "inner": 96, "vocab_size": 100}


class RunningMean(Mixer):
    """out_t = W . mean(x_0..x_t); the state is (sum [hidden], count [1]) per request. It never
    clears its slot: the runner hands a request that starts at position 0 a zeroed one."""

    def __init__(self, hidden_size, positions, name):
        self.h, self.name = hidden_size, name

    def weights(self):
        return {self.name: WeightWant((self.h, self.h))}

    def state_need(self):
        return StateNeed((self.h + 1,), torch.float32)

    def bind(self, tensors, rt):
        super().bind(tensors, rt)
        self.w = rt.ops.prepare_matrix(tensors[self.name], rt)

    def forward(self, x, ctx, cache, state, writes_cache):
        assert cache is None and state is not None
        out = self.rt.workspace.get("toy.mean", tuple(x.shape), x.dtype)
        starts = ctx.host["item_start"].tolist()
        for i in range(ctx.num_items):
            slot = int(ctx.host["slots"][i])
            seg = x[starts[i]:starts[i + 1]].float()
            sums = state[slot, : self.h] + torch.cumsum(seg, 0)
            counts = state[slot, self.h] + torch.arange(1, seg.shape[0] + 1, device=x.device)
            out[starts[i]:starts[i + 1]] = (sums / counts[:, None]).to(x.dtype)
            state[slot, : self.h] = sums[-1]
            state[slot, self.h] = counts[-1]
        delta = self.rt.workspace.get("toy.delta", tuple(x.shape), x.dtype)
        self.rt.ops.linear(out, self.w, delta)
        return delta


class ToyConfig:
    def __init__(self, raw):
        self.raw = raw

    @classmethod
    def from_dicts(cls, raw, gen=None):
        return cls(dict(raw))


def build_toy_mean(cfg):
    r = cfg.raw
    h = r["hidden_size"]
    attn = PartSpec("paged_attention", {"num_heads": 4, "num_kv_heads": 2, "head_dim": 16, "position": "rope",
                                        "names": {"q": "q.weight", "k": "k.weight", "v": "v.weight", "o": "o.weight"}})
    mean = PartSpec("test_running_mean", {"name": "mix.weight"})
    ff = PartSpec("swiglu", {"intermediate_size": r["inner"], "names": {"gate": "g.weight", "up": "u.weight", "down": "d.weight"}})
    norm = lambda n: PartSpec("rmsnorm", {"eps": 1e-5, "name": n})
    layers = tuple(LayerSpec(prefix=f"l{i}.", mixer=mean if i % 2 else attn, feed_forward=ff,
                             mixer_norm=norm("n1.weight"), feed_forward_norm=norm("n2.weight")) for i in range(3))
    # layer 1 (the toy mixer) runs twice; layer 2 reads the keys and values layer 0 wrote
    order = (LayerRun(0, 0), LayerRun(1, 1), LayerRun(2, 0, writes_cache=False), LayerRun(1, 2))
    return ModelSpec(vocab_size=r["vocab_size"], hidden_size=h, embedding="emb.weight", layers=layers, order=order,
                     final_norm=norm("norm.weight"), final_norm_prefix="", head=None,
                     positions={"rope": PartSpec("rope", {"head_dim": 16, "theta": 10000.0})}, max_position=512)


def write_toy_mean_model(folder: Path, seed: int = 5, std: float = 0.1) -> Path:
    """Registers the toy architecture (once) and writes a model folder of it with random weights."""
    from safetensors.torch import save_file

    from prefixserve_amd.weights import random_tensors

    if "ToyMeanForCausalLM" not in registered_architectures():
        register_mixer("test_running_mean", RunningMean)
        register_architecture("ToyMeanForCausalLM", ToyConfig, build_toy_mean)
    folder = Path(folder)
    (folder / "config.json").write_text(json.dumps(TOY_MEAN_CONFIG))
    model = DecoderModel(build_toy_mean(ToyConfig(TOY_MEAN_CONFIG)))
    save_file(random_tensors(model.weights(), seed=seed, std=std), str(folder / "model.safetensors"))
    return folder
