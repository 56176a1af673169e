"""A decoder built from a ``ModelSpec``: token table, layers run in the listed order,
final norm, output matrix. This is the one forward pass of the package: generation, the
scheduler's engine and trace replay all call ``DecoderModel.step``."""

from __future__ import annotations

import struct
from dataclasses import dataclass
from typing import TYPE_CHECKING, Any, Mapping

import torch

from . import attention as _attention  # noqa: F401  (registers the built-in parts)
from . import block as _block  # noqa: F401
from . import mlp as _mlp  # noqa: F401
from . import norm as _norm  # noqa: F401
from . import rope as _rope  # noqa: F401
from .base import CacheNeed, Part, Runtime, StateNeed, WeightWant, make
from .spec import ModelSpec

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


@dataclass
class FusedDecodePlan:
    """The layer runs of a model as the fused decode step reads them: one record per run in
    device memory (``FusedLayer`` in csrc/kernels/decode_fused.hip) and the sizes all runs share."""

    layers: torch.Tensor       # uint8 [n_layers * record size] on the device
    n_layers: int
    hidden: int
    inter: int
    hq: int
    hkv: int
    d: int
    scale: float
    norm_dtype: torch.dtype
    groups: tuple[int, ...]
    keep: tuple                # the tensors the records point to


class DecoderModel:
    def __init__(self, spec: ModelSpec) -> None:
        spec.validate()
        self.spec = spec
        self.positions = {name: make("position", ps.kind, **ps.params) for name, ps in spec.positions.items()}
        self.blocks = []
        for layer in spec.layers:
            h = spec.hidden_size
            mixer = make("mixer", layer.mixer.kind, hidden_size=h, positions=self.positions, **layer.mixer.params)
            ff = make("feed_forward", layer.feed_forward.kind, hidden_size=h, **layer.feed_forward.params)
            n1 = make("norm", layer.mixer_norm.kind, hidden_size=h, **layer.mixer_norm.params)
            n2 = make("norm", layer.feed_forward_norm.kind, hidden_size=h, **layer.feed_forward_norm.params)
            self.blocks.append(make("block", layer.block, mixer=mixer, feed_forward=ff, mixer_norm=n1,
                                    feed_forward_norm=n2))
        self.final_norm = make("norm", spec.final_norm.kind, hidden_size=spec.hidden_size, **spec.final_norm.params)
        self.caches: dict[int, Any] = {}
        self.states: dict[int, torch.Tensor] = {}
        self.rt: Runtime | None = None
        self._fused_plan: FusedDecodePlan | None | bool = False

    # ---------------------------------------------------------------- weights

    def _named_parts(self) -> list[tuple[str, Part]]:
        out: list[tuple[str, Part]] = []
        for layer, blk in zip(self.spec.layers, self.blocks):
            out += [(layer.prefix, p) for p in blk.parts()]
        out.append((self.spec.final_norm_prefix, self.final_norm))
        return out

    def weights(self) -> dict[str, WeightWant]:
        """Every tensor the model wants, by full name."""
        s = self.spec
        want: dict[str, WeightWant] = {s.embedding: WeightWant((s.vocab_size, s.hidden_size), "embedding")}
        for prefix, part in self._named_parts():
            for rel, w in part.weights().items():
                want[prefix + rel] = w
        if s.head is not None:
            want[s.head] = WeightWant((s.vocab_size, s.hidden_size), "matrix")
        return want

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime, max_position: int) -> None:
        """Hands each part its tensors and builds position tables up to ``max_position``."""
        s = self.spec
        if max_position > s.max_position:
            raise ValueError(f"max_position {max_position} > the model's limit {s.max_position}")
        self.rt = rt
        for pos in self.positions.values():
            pos.bind({}, rt)
            pos.prepare(max_position)
        for prefix, part in self._named_parts():
            part.bind({rel: tensors[prefix + rel] for rel in part.weights()}, rt)
        self.embedding = rt.ops.prepare_matrix(tensors[s.embedding], rt)
        # Tied output matrix = the very same storage (prefixserve/model/weights.py:133-136).
        self.head = self.embedding if s.head is None else rt.ops.prepare_matrix(tensors[s.head], rt)
        self.max_position = int(max_position)

    def step_weight_bytes(self) -> int:
        """Bytes of weights one decode step reads: every layer's matrices and norm weights in
        each run, the final norm and the output matrix. The token table is only gathered from
        (a few rows), unless it is also the output matrix."""
        total = 0
        for run in self.spec.order:
            total += sum(p.weight_bytes() for p in self.blocks[run.layer].parts())
        total += self.final_norm.weight_bytes()
        total += self.head.numel() * self.head.element_size()
        return total

    # ------------------------------------------------------------------ cache

    def cache_needs(self) -> dict[int, CacheNeed]:
        """cache entry -> what its writing run's mixer needs."""
        needs: dict[int, CacheNeed] = {}
        for run in self.spec.order:
            need = self.blocks[run.layer].mixer.cache_need()
            if need is None:
                continue
            if run.writes_cache:
                needs[run.cache] = need
        return needs

    def state_needs(self) -> dict[int, StateNeed]:
        """index into ``spec.order`` -> fixed-size per-request state its mixer keeps."""
        needs: dict[int, StateNeed] = {}
        for i, run in enumerate(self.spec.order):
            need = self.blocks[run.layer].mixer.state_need()
            if need is not None:
                needs[i] = need
        return needs

    def attach(self, caches: Mapping[int, Any], states: Mapping[int, torch.Tensor]) -> None:
        self.caches = dict(caches)
        self.states = dict(states)
        self._fused_plan: FusedDecodePlan | None | bool = False        # False: not looked at yet

    def fused_decode_plan(self) -> FusedDecodePlan | None:
        """The plan for running all layers of a small decode step in one kernel, or None if
        some layer is not of the kind that kernel runs (another mixer, a window, state, sizes
        that differ between layers, a dtype other than bfloat16)."""
        if self._fused_plan is not False:
            return self._fused_plan
        self._fused_plan = None
        rt = self.rt
        if rt is None or rt.dtype != torch.bfloat16 or self.states or not hasattr(rt.ops, "decode_layers"):
            return None
        descs = []
        for run in self.spec.order:
            blk = self.blocks[run.layer]
            desc = blk.fused_decode_layer(self.caches.get(run.cache), run.writes_cache) if hasattr(blk, "fused_decode_layer") else None
            if desc is None:
                return None
            descs.append(desc)
        first = descs[0]
        shared = ("hq", "hkv", "d", "scale", "inter", "hidden")
        if any(d[k] != first[k] for d in descs for k in shared) or any(d["norm1"].dtype != first["norm1"].dtype for d in descs):
            return None
        if not rt.ops.decode_layers_supported(1, first["hidden"], first["inter"], first["hq"], first["hkv"], first["d"],
                                              first["norm1"].dtype):
            return None
        code = 1 if first["norm1"].dtype == torch.bfloat16 else 0
        ptr = lambda t: 0 if t is None else t.data_ptr()
        raw = b"".join(struct.pack("<8Q2f4i", ptr(d["w_qkv"]), ptr(d["w_o"]), ptr(d["w_gate_up"]), ptr(d["w_down"]),
                                   ptr(d["norm1"]), ptr(d["norm2"]), ptr(d["kv"]), ptr(d["rope"]), d["eps1"], d["eps2"],
                                   code, d["group"], int(d["writes_cache"]), 0) for d in descs)
        layers = torch.frombuffer(bytearray(raw), dtype=torch.uint8).to(rt.device)
        keep = tuple(t for d in descs for t in d.values() if isinstance(t, torch.Tensor))
        self._fused_plan = FusedDecodePlan(layers, len(descs), first["hidden"], first["inter"], first["hq"], first["hkv"],
                                           first["d"], float(first["scale"]), first["norm1"].dtype,
                                           tuple(d["group"] for d in descs), keep)
        return self._fused_plan

    # ------------------------------------------------------------------- step

    def step(self, ctx: "StepContext") -> torch.Tensor | None:
        """Runs the tokens of ``ctx`` as one batch from the cache and returns float32 logits
        ``[S, vocab]`` at the wanted rows (None when no row is wanted: nothing to wait for).
        Rows first, then the norm, then the product: only S rows pay for the vocabulary
        (prefixserve/model/llama.py:96-101,123-126)."""
        rt = self.rt
        assert rt is not None, "bind() first"
        s, ws, ops = self.spec, rt.workspace, rt.ops
        t = ctx.num_tokens
        with ops.step_scope():
            residual = ws.get("residual", (t, s.hidden_size), torch.float32)
            ops.embed(ctx.token_ids, self.embedding, residual)
            pending = None
            plan = self.fused_decode_plan() if ctx.num_decode == t == ctx.num_items else None
            if plan is not None and ops.decode_layers_supported(t, plan.hidden, plan.inter, plan.hq, plan.hkv, plan.d,
                                                                 plan.norm_dtype):
                ops.decode_layers(plan, residual, ctx)       # every layer, added into the residual
            else:
                for i, run in enumerate(s.order):
                    pending = self.blocks[run.layer].forward(residual, pending, ctx, self.caches.get(run.cache),
                                                             self.states.get(i), run.writes_cache)
            if ctx.num_logit_rows == 0:
                return None
            x = self.final_norm.add_norm_rows(residual, pending, ctx.logit_rows, "final.x")
            logits = ws.get("logits", (ctx.num_logit_rows, s.vocab_size), torch.float32)
            ops.linear(x, self.head, logits)
            return logits
