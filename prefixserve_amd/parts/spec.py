"""What a model is made of, as data.

An architecture's builder turns its typed configuration into a ``ModelSpec``: a list of
layers, each naming its mixer, feed-forward, norms and block arrangement by *kind* with
their sizes and constants as parameters, plus the order in which layers run. Nothing in
this file or in the parts knows which model it describes; a different architecture is a
different builder producing the same kind of data.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping


@dataclass(frozen=True)
class PartSpec:
    """One part: the registry kind that builds it and the parameters it is built with."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One layer. ``prefix`` is put before every weight name the layer's parts ask for."""

    prefix: str
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec
    block: str = "prenorm"
    # Further norms an arrangement other than "prenorm" may want (norms behind the sub-layers,
    # say): built like the two above and handed to the block's factory by these names.
    extra_norms: Mapping[str, PartSpec] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerRun:
    """One entry of the execution order: run ``layer`` with cache entry ``cache``.

    Two runs with the same ``cache`` share it: the run with ``writes_cache`` fills it and
    the others only read it, which is how a layer reads another layer's keys and values.
    A layer may appear in several runs (the same weights applied twice); each run that
    writes needs a cache entry of its own.
    """

    layer: int
    cache: int
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    vocab_size: int
    hidden_size: int
    embedding: str                       # weight name of the token table [vocab, hidden]
    layers: tuple[LayerSpec, ...]
    order: tuple[LayerRun, ...]
    final_norm: PartSpec
    final_norm_prefix: str
    head: str | None                     # weight name of the output matrix; None = the token table
    positions: Mapping[str, PartSpec]    # named position encodings that mixers refer to
    max_position: int
    stop_token_ids: frozenset[int] = frozenset()
    ignored_weights: tuple[str, ...] = ()  # name suffixes a checkpoint may carry and we recompute
    # Transforms of the residual stream right behind the token table (a scale, an added table by
    # position) and of the logits (a cap, a scale, a bias), in the order they are applied; their
    # weight names are taken as they are, without a prefix.
    embedding_transforms: tuple[PartSpec, ...] = ()
    logit_transforms: tuple[PartSpec, ...] = ()

    def validate(self) -> None:
        writers: dict[int, int] = {}
        for run in self.order:
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"order names layer {run.layer}, model has {len(self.layers)}")
            if run.writes_cache:
                if run.cache in writers:
                    raise ValueError(f"cache entry {run.cache} is written by two runs")
                writers[run.cache] = run.layer
        for i, run in enumerate(self.order):
            if not run.writes_cache:
                seen = [j for j, r in enumerate(self.order[:i]) if r.cache == run.cache and r.writes_cache]
                if not seen:
                    raise ValueError(f"run {i} reads cache entry {run.cache} before any run wrote it")
