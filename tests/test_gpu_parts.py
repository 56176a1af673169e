"""Each part of a layer alone against the plain implementation's function for it, and the
openness of the part registries: a toy mixer with state of its own, defined here, is
registered, built into a model and stepped without touching the package's files."""

from __future__ import annotations

import math
import tempfile
from pathlib import Path

import numpy as np
import pytest
import torch

from plain import llama_plain as P
from prefixserve_amd.engine.batch import GroupMeta, StepItem, StepPacker

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def runtime(dtype):
    from prefixserve_amd.kernels.ops import HipOps
    from prefixserve_amd.parts.base import Runtime, Workspace

    ws = Workspace(DEV)
    return Runtime(DEV, dtype, HipOps(DEV, ws), ws)


def rel(got, want):
    got = got.detach().float().cpu().numpy().astype(np.float64)
    return float(np.abs(got - want).max() / np.abs(want).max())


TOL = {torch.float32: 5e-6, torch.bfloat16: 2e-2}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_part(dtype):
    from prefixserve_amd.parts.norm import RMSNorm

    rt = runtime(dtype)
    part = RMSNorm(hidden_size=200, eps=1e-6, name="w")
    assert part.weights()["w"].shape == (200,)
    w = (1 + 0.1 * torch.randn(200)).to(torch.bfloat16)
    part.bind({"w": w}, rt)
    res = torch.randn(5, 200, device=DEV)
    delta = torch.randn(5, 200, device=DEV).to(dtype)
    want = P.rms_norm((res + delta.float()).cpu().double().numpy(), w.double().numpy(), 1e-6)
    got = part.add_norm(res, delta, "x")
    assert rel(got, want) < TOL[dtype]


def test_rope_part_table():
    from prefixserve_amd.parts.rope import RotaryEmbedding

    scaling = dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64)
    part = RotaryEmbedding(head_dim=32, theta=500000.0, scaling=scaling)
    part.bind({}, runtime(torch.float32))
    part.prepare(300)
    inv = P.rope_inv_freq(32, 500000.0, scaling)
    cos, sin = P.rope_cos_sin(np.arange(300), inv)
    table = part.table.cpu().numpy()
    assert table.shape == (300, 16, 2)
    np.testing.assert_allclose(table[..., 0], cos[:, :16], atol=1e-7)
    np.testing.assert_allclose(table[..., 1], sin[:, :16], atol=1e-7)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_part(dtype):
    from prefixserve_amd.parts.mlp import SwiGLU

    rt = runtime(dtype)
    part = SwiGLU(hidden_size=72, intermediate_size=200, names={"gate": "g", "up": "u", "down": "d"})
    w = {"g": 0.2 * torch.randn(200, 72), "u": 0.2 * torch.randn(200, 72), "d": 0.2 * torch.randn(72, 200)}
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    part.bind(w, rt)
    for t in (3, 100):
        x = torch.randn(t, 72, device=DEV).to(dtype)
        want = P.swiglu_mlp(x.float().cpu().double().numpy(), *(w[k].double().numpy() for k in "gud"))
        o = part.forward(x, None)
        assert rel(o.sum(0) if o.dim() == 3 else o, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv,d", [(6, 2, 32), (5, 5, 16), (8, 2, 64)])
def test_attention_part_whole_and_in_portions(dtype, hq, hkv, d):
    from prefixserve_amd.parts.attention import LayerCache, PagedAttention
    from prefixserve_amd.parts.rope import RotaryEmbedding

    rt = runtime(dtype)
    hidden, n = 80, 75
    rope = RotaryEmbedding(head_dim=d, theta=10000.0)
    rope.bind({}, rt)
    rope.prepare(128)
    names = {"q": "q", "k": "k", "v": "v", "o": "o"}
    part = PagedAttention(hidden_size=hidden, positions={"rope": rope}, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                          names=names, position="rope")
    w = {"q": torch.randn(hq * d, hidden), "k": torch.randn(hkv * d, hidden), "v": torch.randn(hkv * d, hidden),
         "o": torch.randn(hidden, hq * d)}
    w = {k: (0.15 * v).to(torch.bfloat16) for k, v in w.items()}
    part.bind(w, rt)
    x = torch.randn(n, hidden, device=DEV).to(dtype)

    xs = x.float().cpu().double().numpy()
    wd = {k: v.double().numpy() for k, v in w.items()}
    cos, sin = P.rope_cos_sin(np.arange(n), P.rope_inv_freq(d, 10000.0, None))
    q = P.apply_rope((xs @ wd["q"].T).reshape(n, hq, d), cos, sin)
    k = P.apply_rope((xs @ wd["k"].T).reshape(n, hkv, d), cos, sin)
    v = (xs @ wd["v"].T).reshape(n, hkv, d)
    want = P.causal_attention(q, k, v).reshape(n, hq * d) @ wd["o"].T

    pk = StepPacker(DEV, [GroupMeta(8)], 10, 128, 4, rt.ops.PREFILL_TILE_Q)
    table = [5, 2, 7, 0, 3]
    for cuts in ([n], [30, 1, 1, 2, 41]):
        cache = LayerCache(kv=torch.zeros(8, 2, hkv, 16 * d, dtype=dtype, device=DEV), group=0, window=None)
        outs, p0 = [], 0
        for c in cuts:
            ctx = pk.pack([StepItem("a", [1] * c, p0, [table])])
            o = part.forward(x[p0:p0 + c].contiguous(), ctx, cache, None, True)
            outs.append(o.sum(0) if o.dim() == 3 else o.float().clone())   # float32 slices of a K-split
            p0 += c
        assert rel(torch.cat(outs), want) < TOL[dtype] * 2


def test_a_toy_mixer_with_state_of_its_own(tmp_path):
    """A running mean over the request's tokens (fixed-size state per request, no pages),
    alternating with attention layers; defined, registered and run from this test only."""
    from prefixserve_amd.engine.replay import TraceReplayer
    from prefixserve_amd.engine.runner import ModelRunner
    from toy_parts import write_toy_mean_model

    write_toy_mean_model(tmp_path)

    runner = ModelRunner(tmp_path, dtype="float32", device="cuda:0", num_blocks=16, max_seq_len=128, max_num_seqs=4,
                         use_graphs=True)
    # Asked for or not, no graphs for a model that keeps state: capturing a step runs it twice.
    assert runner.use_graphs is False
    assert runner.state_bytes_per_slot == 2 * 65 * 4 and len(runner.states) == 2
    assert len(runner.layer_groups) == 1 and runner.layer_groups[0].entries == (0,)
    toks = np.random.default_rng(0).integers(0, 100, 60).tolist()
    other = np.random.default_rng(1).integers(0, 100, 33).tolist()
    rp = TraceReplayer(runner)
    whole = rp.run_step({"step": 0, "entries": [{"id": "a", "tokens": toks, "want": list(range(60))}], "end": ["a"]})
    # the same request in portions, beside another request that keeps its own state
    outs, p0 = [], 0
    for k, c in enumerate([7, 2, 30, 1, 1, 19]):
        entries = [{"id": "b", "tokens": toks[p0:p0 + c], "want": list(range(c))}]
        if k < 3:
            entries.insert(0, {"id": "c", "tokens": other[11 * k:11 * k + 11], "want": []})
        got = rp.run_step({"step": k + 1, "entries": entries, "end": ["c"] if k == 2 else []})
        outs.append(got)
        p0 += c
    cut = np.concatenate(outs)
    assert np.abs(cut - whole).max() / np.abs(whole).max() < 1e-5
    assert np.abs(whole).max() > 0.1 and np.isfinite(whole).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_prenorm_block_is_one_plain_layer(dtype, model_dirs, plain_models):
    """The block arrangement alone: norm -> mixer -> add, norm -> feed-forward -> add, with the
    sums handed on as pending deltas, against the plain model's layer function."""
    from configs import TINY
    from prefixserve_amd.config import architecture_of
    from prefixserve_amd.parts import DecoderModel
    from prefixserve_amd.parts.attention import LayerCache
    from prefixserve_amd.weights import load_weights

    name = "B"
    raw = TINY[name]
    arch = architecture_of(raw)
    spec = arch.build_spec(arch.config_cls.from_dicts(raw, {}))
    model = DecoderModel(spec)
    rt = runtime(dtype)
    model.bind(load_weights(model_dirs[name], model.weights(), spec.ignored_weights), rt, 128)
    plain = plain_models[name]
    n, hidden = 50, raw["hidden_size"]
    h0 = (0.5 * torch.randn(n, hidden)).to(torch.bfloat16).float()
    cos, sin = P.rope_cos_sin(np.arange(n), plain.inv_freq)
    want = plain.layer(1, h0.double().numpy(), cos, sin)

    pk = StepPacker(DEV, [GroupMeta(8)], 10, 128, 4, rt.ops.PREFILL_TILE_Q)
    hkv, d = raw["num_key_value_heads"], raw["head_dim"]
    cache = LayerCache(kv=torch.zeros(8, 2, hkv, 16 * d, dtype=dtype, device=DEV), group=0, window=None)
    block = model.blocks[1]
    got, p0 = [], 0
    for c in (33, 1, 16):                                         # a portion, a decode token, a portion
        ctx = pk.pack([StepItem("a", [1] * c, p0, [[3, 1, 4, 6]])])
        residual = h0[p0:p0 + c].to(DEV).contiguous()
        pending = block.forward(residual, None, ctx, cache, None, True)
        pend = pending.sum(0) if pending.dim() == 3 else pending.float()
        got.append((residual + pend).clone())                     # the last add is the next block's
        p0 += c
    assert rel(torch.cat(got), want) < TOL[dtype] * 2


def test_windowed_attention_through_the_engine(tmp_path):
    """A toy architecture whose layers keep different things: one layer attends over a window
    of 24 positions (its pages are given back as the window passes), one over everything.
    Replayed whole, in portions and token by token, with a window-group pool too small for a
    whole request; compared with the plain functions in both dtypes."""
    import json

    from safetensors.torch import save_file

    from prefixserve_amd.config import register_architecture, registered_architectures
    from prefixserve_amd.engine.replay import TraceReplayer
    from prefixserve_amd.engine.runner import ModelRunner
    from prefixserve_amd.parts import DecoderModel, LayerRun, LayerSpec, ModelSpec, PartSpec
    from prefixserve_amd.weights import random_tensors

    WINDOW, H, HQ, HKV, D, INNER, V = 24, 64, 4, 2, 16, 96, 120

    class Cfg:
        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dicts(cls, raw, gen=None):
            return cls(dict(raw))

    def build(cfg):
        def attn(window):
            return PartSpec("paged_attention", {"num_heads": HQ, "num_kv_heads": HKV, "head_dim": D, "position": "rope",
                                                "window": window,
                                                "names": {"q": "q.weight", "k": "k.weight", "v": "v.weight", "o": "o.weight"}})
        ff = PartSpec("swiglu", {"intermediate_size": INNER, "names": {"gate": "g.weight", "up": "u.weight", "down": "d.weight"}})
        norm = lambda nm: PartSpec("rmsnorm", {"eps": 1e-5, "name": nm})
        layers = tuple(LayerSpec(prefix=f"l{i}.", mixer=attn(WINDOW if i == 0 else None), feed_forward=ff,
                                 mixer_norm=norm("n1.weight"), feed_forward_norm=norm("n2.weight")) for i in range(2))
        return ModelSpec(vocab_size=V, hidden_size=H, embedding="emb.weight", layers=layers,
                         order=(LayerRun(0, 0), LayerRun(1, 1)), final_norm=norm("norm.weight"), final_norm_prefix="",
                         head=None, positions={"rope": PartSpec("rope", {"head_dim": D, "theta": 10000.0})}, max_position=512)

    if "ToyWindowForCausalLM" not in registered_architectures():
        register_architecture("ToyWindowForCausalLM", Cfg, build)
    raw = {"architectures": ["ToyWindowForCausalLM"]}
    (tmp_path / "config.json").write_text(json.dumps(raw))
    tensors = random_tensors(DecoderModel(build(Cfg(raw))).weights(), seed=9, std=0.1)
    save_file(tensors, str(tmp_path / "model.safetensors"))
    w = {k: v.double().numpy() for k, v in tensors.items()}

    toks = np.random.default_rng(3).integers(0, V, 150).tolist()
    n = len(toks)
    cos, sin = P.rope_cos_sin(np.arange(n), P.rope_inv_freq(D, 10000.0, None))
    h = w["emb.weight"][toks]
    for i, window in enumerate((WINDOW, None)):
        p = f"l{i}."
        x = P.rms_norm(h, w[p + "n1.weight"], 1e-5)
        q = P.apply_rope((x @ w[p + "q.weight"].T).reshape(n, HQ, D), cos, sin)
        k = P.apply_rope((x @ w[p + "k.weight"].T).reshape(n, HKV, D), cos, sin)
        v = (x @ w[p + "v.weight"].T).reshape(n, HKV, D)
        h = h + P.causal_attention(q, k, v, window).reshape(n, HQ * D) @ w[p + "o.weight"].T
        x = P.rms_norm(h, w[p + "n2.weight"], 1e-5)
        h = h + P.swiglu_mlp(x, w[p + "g.weight"], w[p + "u.weight"], w[p + "d.weight"])
    want = P.rms_norm(h, w["norm.weight"], 1e-5) @ w["emb.weight"].T

    for dtype, tol in (("float32", 1e-5), ("bfloat16", 4e-2)):
        # group of the full layer: 10 pages (150 tokens); group of the window layer: 5 pages only
        runner = ModelRunner(tmp_path, dtype=dtype, device="cuda:0", num_blocks=[5, 10], max_seq_len=160,
                             max_num_seqs=2, use_graphs=True)
        windows = runner.windows
        assert sorted(windows, key=lambda x: (x is None, x)) == [WINDOW, None]
        if windows[0] is None:                                     # group order follows the cache entries
            runner = ModelRunner(tmp_path, dtype=dtype, device="cuda:0", num_blocks=[10, 5], max_seq_len=160,
                                 max_num_seqs=2, use_graphs=True)
        for cuts in ([16] * 9 + [6], [5, 2, 16, 1, 1, 1, 30, 3] + [1] * 40 + [16, 16, 16, 2, 1]):
            assert sum(cuts) == n
            rp = TraceReplayer(runner)
            assert not rp.cache.prefix_cache                       # a window switches the prefix cache off
            p0, worst = 0, 0.0
            for kk, c in enumerate(cuts):
                got = rp.run_step({"step": kk, "entries": [{"id": "a", "tokens": toks[p0:p0 + c], "want": list(range(c))}],
                                   "end": ["a"] if p0 + c == n else []})
                err = np.abs(got - want[p0:p0 + c]).max(-1) / np.abs(want[p0:p0 + c]).max(-1)
                assert err.max() < tol, f"{dtype} positions {p0}..{p0 + c}: {err.max():.3e}"
                p0 += c
            assert all(rp.cache.num_free(g) == rp.cache.num_blocks(g) for g in range(2))

    # The same architecture through the scheduler: pages of the window group go back while the
    # requests run, also when several decode steps are taken per round.
    from prefixserve_amd import Engine, EngineConfig, generate

    prompts = [toks[:70], toks[40:75], toks[90:97]]
    eng = Engine(EngineConfig(model_path=tmp_path, dtype="float32", max_num_seqs=3, max_prefill_tokens=32, max_seq_len=160,
                              num_blocks=12))
    one, _ = generate(eng, prompts, 40, ignore_eos=True)
    four, _ = generate(eng, prompts, 40, ignore_eos=True, decode_steps=4)
    assert [o.tokens for o in one] == [o.tokens for o in four]
    seq = list(prompts[2])
    for tok in one[2].tokens[:6]:                                  # against the plain functions, token by token
        hh = w["emb.weight"][seq]
        nn = len(seq)
        cs, sn = P.rope_cos_sin(np.arange(nn), P.rope_inv_freq(D, 10000.0, None))
        for i, window in enumerate((WINDOW, None)):
            pp = f"l{i}."
            x = P.rms_norm(hh, w[pp + "n1.weight"], 1e-5)
            q = P.apply_rope((x @ w[pp + "q.weight"].T).reshape(nn, HQ, D), cs, sn)
            k = P.apply_rope((x @ w[pp + "k.weight"].T).reshape(nn, HKV, D), cs, sn)
            v = (x @ w[pp + "v.weight"].T).reshape(nn, HKV, D)
            hh = hh + P.causal_attention(q, k, v, window).reshape(nn, HQ * D) @ w[pp + "o.weight"].T
            x = P.rms_norm(hh, w[pp + "n2.weight"], 1e-5)
            hh = hh + P.swiglu_mlp(x, w[pp + "g.weight"], w[pp + "u.weight"], w[pp + "d.weight"])
        row = P.rms_norm(hh[-1:], w["norm.weight"], 1e-5) @ w["emb.weight"].T
        assert tok == int(np.argmax(row[0]))
        seq.append(tok)


def test_a_toy_position_encoding_and_a_routed_feed_forward(tmp_path):
    """Two more parts defined and registered from this test only: a position encoding whose
    rotation angle is position * (i + 1) / 50 (another rule than rope's, through the same
    rotation table), and a feed-forward that sends every token to one of three SwiGLU experts
    by the largest router logit and scales the result by that logit's softmax weight. Layer 0
    uses both; layer 1 is an ordinary rope + dense layer: the parts are chosen per layer.
    Compared with the plain functions, whole and in portions, in both dtypes."""
    import json

    from safetensors.torch import save_file

    from prefixserve_amd.config import register_architecture, registered_architectures
    from prefixserve_amd.engine.replay import TraceReplayer
    from prefixserve_amd.engine.runner import ModelRunner
    from prefixserve_amd.parts import (DecoderModel, FeedForward, LayerRun, LayerSpec, ModelSpec, PartSpec, RotaryTable,
                                       WeightWant, register_feed_forward, register_position)
    from prefixserve_amd.weights import random_tensors

    H, HQ, HKV, D, INNER, V, E = 80, 5, 1, 32, 48, 90, 3

    class LinearAngles(RotaryTable):
        def __init__(self, head_dim, slope):
            self.head_dim, self.slope = int(head_dim), float(slope)

        def prepare(self, max_position):
            i = torch.arange(self.head_dim // 2, dtype=torch.float64)
            angle = torch.outer(torch.arange(max_position, dtype=torch.float64), (i + 1.0) * self.slope)
            self.table = torch.stack((angle.cos(), angle.sin()), -1).float().contiguous().to(self.rt.device)

    class Top1Experts(FeedForward):
        def __init__(self, hidden_size, inner, experts):
            self.h, self.inner, self.e = hidden_size, inner, experts

        def weights(self):
            want = {"router.weight": WeightWant((self.e, self.h))}
            for e in range(self.e):
                want[f"e{e}.gate_up.weight"] = WeightWant((2 * self.inner, self.h))
                want[f"e{e}.down.weight"] = WeightWant((self.h, self.inner))
            return want

        def bind(self, tensors, rt):
            super().bind(tensors, rt)
            self.router = tensors["router.weight"].float().to(rt.device)        # router logits in 32-bit
            self.gate_up = [rt.ops.prepare_matrix(tensors[f"e{e}.gate_up.weight"], rt) for e in range(self.e)]
            self.down = [rt.ops.prepare_matrix(tensors[f"e{e}.down.weight"], rt) for e in range(self.e)]

        def forward(self, x, ctx):
            ops = self.rt.ops
            logits = x.float() @ self.router.T
            weight, choice = torch.softmax(logits, -1).max(-1)
            out = torch.zeros_like(x)
            for e in range(self.e):
                rows = (choice == e).nonzero().flatten()
                if rows.numel() == 0:
                    continue
                xe = x[rows].contiguous()
                act = torch.empty(rows.numel(), self.inner, dtype=x.dtype, device=x.device)
                ops.linear_swiglu(xe, self.gate_up[e], act)
                ye = torch.empty(rows.numel(), self.h, dtype=x.dtype, device=x.device)
                ops.linear(act, self.down[e], ye)
                out[rows] = (ye.float() * weight[rows, None]).to(x.dtype)
            return out

    class Cfg:
        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dicts(cls, raw, gen=None):
            return cls(dict(raw))

    def build(cfg):
        def attn(position):
            return PartSpec("paged_attention", {"num_heads": HQ, "num_kv_heads": HKV, "head_dim": D, "position": position,
                                                "names": {"q": "q.weight", "k": "k.weight", "v": "v.weight", "o": "o.weight"}})
        dense = PartSpec("swiglu", {"intermediate_size": INNER, "names": {"gate": "g.weight", "up": "u.weight", "down": "d.weight"}})
        routed = PartSpec("test_top1_experts", {"inner": INNER, "experts": E})
        norm = lambda nm: PartSpec("rmsnorm", {"eps": 1e-6, "name": nm})
        layers = (LayerSpec(prefix="l0.", mixer=attn("linear"), feed_forward=routed, mixer_norm=norm("n1.weight"),
                            feed_forward_norm=norm("n2.weight")),
                  LayerSpec(prefix="l1.", mixer=attn("rope"), feed_forward=dense, mixer_norm=norm("n1.weight"),
                            feed_forward_norm=norm("n2.weight")))
        return ModelSpec(vocab_size=V, hidden_size=H, embedding="emb.weight", layers=layers,
                         order=(LayerRun(0, 0), LayerRun(1, 1)), final_norm=norm("norm.weight"), final_norm_prefix="",
                         head="head.weight",
                         positions={"rope": PartSpec("rope", {"head_dim": D, "theta": 10000.0}),
                                    "linear": PartSpec("test_linear_angles", {"head_dim": D, "slope": 0.02})},
                         max_position=256)

    if "ToyRoutedForCausalLM" not in registered_architectures():
        register_position("test_linear_angles", LinearAngles)
        register_feed_forward("test_top1_experts", Top1Experts)
        register_architecture("ToyRoutedForCausalLM", Cfg, build)
    raw = {"architectures": ["ToyRoutedForCausalLM"]}
    (tmp_path / "config.json").write_text(json.dumps(raw))
    tensors = random_tensors(DecoderModel(build(Cfg(raw))).weights(), seed=11, std=0.1)
    tensors["l0.router.weight"] = tensors["l0.router.weight"] * 8.0        # clear choices, far from ties
    save_file(tensors, str(tmp_path / "model.safetensors"))
    w = {k: v.double().numpy() for k, v in tensors.items()}

    toks = np.random.default_rng(5).integers(0, V, 100).tolist()
    n = len(toks)
    pos = np.arange(n)
    angle = np.outer(pos, (np.arange(D // 2) + 1.0) * 0.02)
    angle = np.concatenate([angle, angle], -1)                            # both halves of a pair share the angle
    tables = [(np.cos(angle), np.sin(angle)), P.rope_cos_sin(pos, P.rope_inv_freq(D, 10000.0, None))]
    h = w["emb.weight"][toks]
    used = set()
    for i, (cos, sin) in enumerate(tables):
        p = f"l{i}."
        x = P.rms_norm(h, w[p + "n1.weight"], 1e-6)
        q = P.apply_rope((x @ w[p + "q.weight"].T).reshape(n, HQ, D), cos, sin)
        k = P.apply_rope((x @ w[p + "k.weight"].T).reshape(n, HKV, D), cos, sin)
        v = (x @ w[p + "v.weight"].T).reshape(n, HKV, D)
        h = h + P.causal_attention(q, k, v).reshape(n, HQ * D) @ w[p + "o.weight"].T
        x = P.rms_norm(h, w[p + "n2.weight"], 1e-6)
        if i == 0:
            logits = x @ w[p + "router.weight"].T
            prob = np.exp(logits - logits.max(-1, keepdims=True))
            prob /= prob.sum(-1, keepdims=True)
            y = np.zeros_like(x)
            for t in range(n):
                e = int(prob[t].argmax())
                used.add(e)
                gu = w[p + f"e{e}.gate_up.weight"]
                y[t] = prob[t, e] * P.swiglu_mlp(x[t:t + 1], gu[:INNER], gu[INNER:], w[p + f"e{e}.down.weight"])[0]
            h = h + y
        else:
            h = h + P.swiglu_mlp(x, w[p + "g.weight"], w[p + "u.weight"], w[p + "d.weight"])
    assert used == set(range(E))                                           # every expert had tokens
    want = P.rms_norm(h, w["norm.weight"], 1e-6) @ w["head.weight"].T

    for dtype, tol in (("float32", 1e-5), ("bfloat16", 4e-2)):
        runner = ModelRunner(tmp_path, dtype=dtype, device="cuda:0", num_blocks=8, max_seq_len=112, max_num_seqs=2,
                             use_graphs=False)
        for cuts in ([n], [3, 2, 40, 1, 1, 1, 17, 35]):
            assert sum(cuts) == n
            rp = TraceReplayer(runner)
            p0 = 0
            for kk, c in enumerate(cuts):
                got = rp.run_step({"step": kk, "entries": [{"id": "a", "tokens": toks[p0:p0 + c], "want": list(range(c))}],
                                   "end": ["a"] if p0 + c == n else []})
                err = np.abs(got - want[p0:p0 + c]).max(-1) / np.abs(want[p0:p0 + c]).max(-1)
                assert err.max() < tol, f"{dtype} positions {p0}..{p0 + c}: {err.max():.3e}"
                p0 += c


def test_toy_transforms_and_a_block_with_more_norms(tmp_path):
    """Three more things a model may be made of, defined and registered from this test only: the
    residual stream scaled and given a learned row per position right behind the token table,
    the logits capped (cap * tanh(logits / cap)), and a block with a norm behind each sub-layer
    as well as in front of it (``LayerSpec.extra_norms``). The block wants each sub-layer's
    output itself, so it keeps the stream to itself (``ctx.residual = None``). Compared with the
    plain functions whole, in portions and token by token through graphs, in both dtypes."""
    import json

    from safetensors.torch import save_file

    from prefixserve_amd.config import register_architecture, registered_architectures
    from prefixserve_amd.engine.replay import TraceReplayer
    from prefixserve_amd.engine.runner import ModelRunner
    from prefixserve_amd.parts import (DecoderModel, LayerRun, LayerSpec, ModelSpec, PartSpec, Transform, WeightWant,
                                       register_block, register_transform)
    from prefixserve_amd.weights import random_tensors

    H, HQ, HKV, D, INNER, V, CAP, MAXPOS = 64, 4, 2, 16, 96, 110, 3.0, 256

    class Scale(Transform):
        def __init__(self, hidden_size, vocab_size, factor):
            self.factor = float(factor)

        def apply(self, t, ctx, rows):
            t.mul_(self.factor)

    class LearnedPositions(Transform):
        def __init__(self, hidden_size, vocab_size, name, positions):
            self.h, self.name, self.n = hidden_size, name, positions

        def weights(self):
            return {self.name: WeightWant((self.n, self.h))}

        def bind(self, tensors, rt):
            super().bind(tensors, rt)
            self.table = tensors[self.name].to(rt.device, torch.float32)

        def apply(self, t, ctx, rows):
            pos = ctx.positions if rows is None else ctx.positions[rows.long()]
            t.add_(self.table[pos.long()])

    class SoftCap(Transform):
        def __init__(self, hidden_size, vocab_size, cap):
            self.cap = float(cap)

        def apply(self, t, ctx, rows):
            t.copy_(self.cap * torch.tanh(t / self.cap))

    class Sandwich:
        def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm, post_mixer, post_feed_forward):
            self.mixer, self.ff, self.n1, self.n2, self.p1, self.p2 = mixer, feed_forward, mixer_norm, feed_forward_norm, post_mixer, post_feed_forward

        def parts(self):
            return [self.n1, self.mixer, self.p1, self.n2, self.ff, self.p2]

        def _normed(self, norm, delta, name):
            ws = norm.rt.workspace
            t = delta.shape[-2]
            zero = ws.get("sandwich.zero", (t, H), torch.float32)
            zero.zero_()
            return norm.add_norm(zero, delta, name)                # norm(0 + delta)

        def forward(self, residual, pending, ctx, cache, state, writes_cache):
            ctx.residual = None                                    # the sub-layers hand their output back
            x = self.n1.add_norm(residual, pending, "block.x")
            y = self._normed(self.p1, self.mixer.forward(x, ctx, cache, state, writes_cache), "sandwich.y1")
            x = self.n2.add_norm(residual, y, "block.x")
            return self._normed(self.p2, self.ff.forward(x, ctx), "sandwich.y2")

    class Cfg:
        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dicts(cls, raw, gen=None):
            return cls(dict(raw))

    def build(cfg):
        attn = PartSpec("paged_attention", {"num_heads": HQ, "num_kv_heads": HKV, "head_dim": D, "position": "rope",
                                            "names": {"q": "q.weight", "k": "k.weight", "v": "v.weight", "o": "o.weight"}})
        ff = PartSpec("swiglu", {"intermediate_size": INNER, "names": {"gate": "g.weight", "up": "u.weight", "down": "d.weight"}})
        norm = lambda nm: PartSpec("rmsnorm", {"eps": 1e-5, "name": nm})
        layers = tuple(LayerSpec(prefix=f"l{i}.", mixer=attn, feed_forward=ff, mixer_norm=norm("n1.weight"),
                                 feed_forward_norm=norm("n2.weight"), block="test_sandwich",
                                 extra_norms={"post_mixer": norm("p1.weight"), "post_feed_forward": norm("p2.weight")})
                       for i in range(2))
        return ModelSpec(vocab_size=V, hidden_size=H, embedding="emb.weight", layers=layers,
                         order=(LayerRun(0, 0), LayerRun(1, 1)), final_norm=norm("norm.weight"), final_norm_prefix="",
                         head=None, positions={"rope": PartSpec("rope", {"head_dim": D, "theta": 10000.0})}, max_position=MAXPOS,
                         embedding_transforms=(PartSpec("test_scale", {"factor": math.sqrt(H)}),
                                               PartSpec("test_learned_positions", {"name": "pos.weight", "positions": MAXPOS})),
                         logit_transforms=(PartSpec("test_softcap", {"cap": CAP}),))

    if "ToySandwichForCausalLM" not in registered_architectures():
        register_transform("test_scale", Scale)
        register_transform("test_learned_positions", LearnedPositions)
        register_transform("test_softcap", SoftCap)
        register_block("test_sandwich", Sandwich)
        register_architecture("ToySandwichForCausalLM", Cfg, build)
    raw = {"architectures": ["ToySandwichForCausalLM"]}
    (tmp_path / "config.json").write_text(json.dumps(raw))
    tensors = random_tensors(DecoderModel(build(Cfg(raw))).weights(), seed=4, std=0.1)
    assert "pos.weight" in tensors and "l1.p2.weight" in tensors
    save_file(tensors, str(tmp_path / "model.safetensors"))
    w = {k: v.double().numpy() for k, v in tensors.items()}

    toks = np.random.default_rng(5).integers(0, V, 90).tolist()
    n = len(toks)
    cos, sin = P.rope_cos_sin(np.arange(n), P.rope_inv_freq(D, 10000.0, None))
    h = w["emb.weight"][toks] * math.sqrt(H) + w["pos.weight"][:n]
    for i in range(2):
        p = f"l{i}."
        x = P.rms_norm(h, w[p + "n1.weight"], 1e-5)
        q = P.apply_rope((x @ w[p + "q.weight"].T).reshape(n, HQ, D), cos, sin)
        k = P.apply_rope((x @ w[p + "k.weight"].T).reshape(n, HKV, D), cos, sin)
        v = (x @ w[p + "v.weight"].T).reshape(n, HKV, D)
        h = h + P.rms_norm(P.causal_attention(q, k, v).reshape(n, HQ * D) @ w[p + "o.weight"].T, w[p + "p1.weight"], 1e-5)
        x = P.rms_norm(h, w[p + "n2.weight"], 1e-5)
        h = h + P.rms_norm(P.swiglu_mlp(x, w[p + "g.weight"], w[p + "u.weight"], w[p + "d.weight"]), w[p + "p2.weight"], 1e-5)
    want = CAP * np.tanh(P.rms_norm(h, w["norm.weight"], 1e-5) @ w["emb.weight"].T / CAP)
    assert np.abs(want).max() > 0.5 * CAP                          # the cap is felt

    for dtype, tol in (("float32", 2e-5), ("bfloat16", 4e-2)):
        runner = ModelRunner(tmp_path, dtype=dtype, device="cuda:0", num_blocks=16, max_seq_len=128, max_num_seqs=2,
                             use_graphs=True)
        for cuts in ([n], [7, 2, 30, 1, 1, 17] + [1] * 32):
            rp = TraceReplayer(runner)
            p0 = 0
            for kk, c in enumerate(cuts):
                got = rp.run_step({"step": kk, "entries": [{"id": "a", "tokens": toks[p0:p0 + c], "want": list(range(c))}],
                                   "end": ["a"] if p0 + c == n else []})
                err = np.abs(got - want[p0:p0 + c]).max(-1) / np.abs(want[p0:p0 + c]).max(-1)
                assert err.max() < tol, f"{dtype} positions {p0}..{p0 + c}: {err.max():.3e}"
                p0 += c
        assert (1, 1, False) in runner._graphs                    # the single tokens went through a captured graph


def toy_kernel_library():
    """The test's own kernel library, compiled on first use (the build entry point compiles it
    beforehand together with the package's)."""
    from prefixserve_amd.build import build_extension

    here = Path(__file__).resolve().parent / "toy_kernels"
    out = here / "_lib" / "libtoy_soft_cap.so"
    if not out.exists() or out.stat().st_mtime < (here / "soft_cap.hip").stat().st_mtime:
        try:
            build_extension([here / "soft_cap.hip"], out)
        except OSError:                                           # a tree that cannot be written to
            out = Path(tempfile.mkdtemp()) / out.name
            build_extension([here / "soft_cap.hip"], out)
    return out


def test_a_part_with_a_kernel_of_its_own(tmp_path):
    """A part that brings its own device kernel, from test files alone: a transform of the logits
    whose HIP source lies beside this test, built with the package's flags
    (``build.build_extension``) and loaded through ``HipOps.load_extension``; no file of the
    package is touched. The architecture is the Llama builder's specification with that transform
    behind the output matrix. Compared with the plain model's logits, capped, whole and token by
    token through graphs (the kernel is launched on the step's stream, so it is captured with it),
    in both dtypes; and the library's refusals and a missing entry point come back as errors."""
    import ctypes
    import dataclasses
    import json

    from configs import INIT_STD, TINY
    from plain.llama_plain import PlainLlama
    from prefixserve_amd.config import register_architecture, registered_architectures
    from prefixserve_amd.config.llama import LlamaConfig
    from prefixserve_amd.engine.replay import TraceReplayer
    from prefixserve_amd.engine.runner import ModelRunner
    from prefixserve_amd.kernels.ops import KernelError
    from prefixserve_amd.models.llama import build_llama_spec
    from prefixserve_amd.parts import PartSpec, Transform, register_transform
    from prefixserve_amd.weights import write_random_model

    CAP = 2.0
    lib_path = toy_kernel_library()

    class KernelSoftCap(Transform):
        def __init__(self, hidden_size, vocab_size, cap):
            self.cap = float(cap)

        def bind(self, tensors, rt):
            super().bind(tensors, rt)
            self.ops = rt.ops
            self.lib = rt.ops.load_extension(lib_path, {"toy_soft_cap": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_float]})

        def apply(self, t, ctx, rows):
            assert t.dtype == torch.float32 and t.is_contiguous()
            self.ops.check(self.lib.toy_soft_cap(self.ops.stream_pointer(), t.data_ptr(), t.numel(), self.cap), "toy_soft_cap")

    def build(cfg):
        return dataclasses.replace(build_llama_spec(cfg), logit_transforms=(PartSpec("test_kernel_softcap", {"cap": CAP}),))

    if "ToyCappedLlamaForCausalLM" not in registered_architectures():
        register_transform("test_kernel_softcap", KernelSoftCap)
        register_architecture("ToyCappedLlamaForCausalLM", LlamaConfig, build)
    raw = dict(TINY["B"])
    write_random_model(tmp_path / "llama", raw, seed=12, std=INIT_STD)
    plain = PlainLlama(tmp_path / "llama")
    capped = tmp_path / "capped"
    capped.mkdir()
    (capped / "config.json").write_text(json.dumps({**raw, "architectures": ["ToyCappedLlamaForCausalLM"]}))
    (capped / "model.safetensors").write_bytes((tmp_path / "llama" / "model.safetensors").read_bytes())

    toks = np.random.default_rng(3).integers(0, raw["vocab_size"], 60).tolist()
    n = len(toks)
    want = CAP * np.tanh(plain.logits(toks) / CAP)
    assert np.abs(plain.logits(toks)).max() > CAP                  # the cap is felt
    for dtype, tol in (("float32", 2e-5), ("bfloat16", 4e-2)):
        runner = ModelRunner(capped, dtype=dtype, device="cuda:0", num_blocks=16, max_seq_len=128, max_num_seqs=2, use_graphs=True)
        for cuts in ([n], [25] + [1] * 35):
            rp = TraceReplayer(runner)
            p0 = 0
            for kk, c in enumerate(cuts):
                got = rp.run_step({"step": kk, "entries": [{"id": "a", "tokens": toks[p0:p0 + c], "want": list(range(c))}],
                                   "end": ["a"] if p0 + c == n else []})
                err = np.abs(got - want[p0:p0 + c]).max(-1) / np.abs(want[p0:p0 + c]).max(-1)
                assert err.max() < tol, f"{dtype} positions {p0}..{p0 + c}: {err.max():.3e}"
                p0 += c
        assert (1, 1, False) in runner._graphs                    # the single tokens went through a captured graph
        ops = runner.rt.ops
    lib = ops.load_extension(lib_path, {"toy_soft_cap": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_float]})
    with pytest.raises(KernelError, match="code 1"):
        ops.check(lib.toy_soft_cap(ops.stream_pointer(), None, 4, 1.0), "toy_soft_cap")
    with pytest.raises(KernelError, match="no entry point"):
        ops.load_extension(lib_path, {"toy_missing": [ctypes.c_void_p]})
    with pytest.raises(KernelError, match="cannot load"):
        ops.load_extension(tmp_path / "nothing.so", {})
