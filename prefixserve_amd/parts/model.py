"""A decoder built from a ``ModelSpec``: token table, layers run in the listed order,
final norm, output matrix. This is the one forward pass of the package: generation, the
scheduler's engine and trace replay all call ``DecoderModel.step``."""

from __future__ import annotations

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
            extra = {name: make("norm", ps.kind, hidden_size=h, **ps.params) for name, ps in layer.extra_norms.items()}
            self.blocks.append(make("block", layer.block, mixer=mixer, feed_forward=ff, mixer_norm=n1,
                                    feed_forward_norm=n2, **extra))
        self.final_norm = make("norm", spec.final_norm.kind, hidden_size=spec.hidden_size, **spec.final_norm.params)
        sizes = dict(hidden_size=spec.hidden_size, vocab_size=spec.vocab_size)
        self.embedding_transforms = [make("transform", ps.kind, **sizes, **ps.params) for ps in spec.embedding_transforms]
        self.logit_transforms = [make("transform", ps.kind, **sizes, **ps.params) for ps in spec.logit_transforms]
        self.caches: dict[int, Any] = {}
        self.states: dict[int, torch.Tensor] = {}
        self.rt: Runtime | None = None

    # ---------------------------------------------------------------- weights

    def _named_parts(self) -> list[tuple[str, Part]]:
        out: list[tuple[str, Part]] = []
        for layer, blk in zip(self.spec.layers, self.blocks):
            out += [(layer.prefix, p) for p in blk.parts()]
        out.append((self.spec.final_norm_prefix, self.final_norm))
        out += [("", tr) for tr in self.embedding_transforms + self.logit_transforms]
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
            for tr in self.embedding_transforms:
                tr.apply(residual, ctx, None)
            ctx.residual = residual
            pending = None
            for i, run in enumerate(s.order):
                pending = self.blocks[run.layer].forward(residual, pending, ctx, self.caches.get(run.cache),
                                                         self.states.get(i), run.writes_cache)
            if ctx.num_logit_rows == 0:
                return None
            x = self.final_norm.add_norm_rows(residual, pending, ctx.logit_rows, "final.x", lazy=True)
            logits = ws.get("logits", (ctx.num_logit_rows, s.vocab_size), torch.float32)
            ops.linear(x, self.head, logits)
            for tr in self.logit_transforms:
                tr.apply(logits, ctx, ctx.logit_rows)
            return logits
