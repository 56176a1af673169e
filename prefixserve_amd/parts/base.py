"""Interfaces of the parts a model is put together from, and their registries.

Every part is built from a ``PartSpec`` (its sizes and constants are parameters), says
which weights it wants (names relative to its layer's prefix, with shapes), receives
them in ``bind`` and then runs on the flat ragged batch of a step: all requests' new
tokens back to back, ``[T, ...]``, no padding and no batch dimension.

Adding a part = one class + one ``register_*`` call; a model uses it by naming its kind
in a ``PartSpec``. No part knows which model it is in.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import TYPE_CHECKING, Any, Callable, Mapping

import torch

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


@dataclass(frozen=True)
class WeightWant:
    """A weight a part asks for. ``init`` tells the random-weights mode how to fill it:
    "matrix" = N(0, std), "norm" = 1 + N(0, norm_std), "embedding" = N(0, std)."""

    shape: tuple[int, ...]
    init: str = "matrix"


@dataclass(frozen=True)
class CacheNeed:
    """Keys and values in pages. Layers whose needs are equal share a page pool and a
    block table per request ("layer group"); ``window`` None keeps every key, a number
    keeps only the last ``window`` positions and lets older pages go."""

    kv_heads: int
    head_dim: int
    window: int | None = None


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size (elements of ``dtype``), kept in a slot."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


class Workspace:
    """Named device buffers that live across steps, so a steady-state step allocates
    nothing and captured graphs keep valid addresses. A buffer only ever grows; growth
    bumps ``version`` so that whoever holds addresses (a captured graph) knows to drop them."""

    def __init__(self, device: torch.device) -> None:
        self.device = device
        self.version = 0
        self._bufs: dict[str, torch.Tensor] = {}
        self._views: dict[tuple, torch.Tensor] = {}      # (name, shape, dtype) -> view handed out before

    def get(self, name: str, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        key = (name, tuple(shape), dtype)
        view = self._views.get(key)
        if view is not None:
            return view
        n = 1
        for s in shape:
            n *= int(s)
        buf = self._bufs.get(name)
        if buf is None or buf.dtype != dtype or buf.numel() < n:
            grow = max(n, 1)
            buf = torch.empty(grow, dtype=dtype, device=self.device)
            self._bufs[name] = buf
            self.version += 1
            self._views.clear()                          # views of the buffer this one replaces
        if len(self._views) >= 2048:                     # every token count brings shapes of its own
            self._views.clear()
        view = self._views[key] = buf[:n].view(*shape)
        return view

    def get_zeroed(self, name: str, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        """Like ``get``, but the buffer is zero when first handed out or after it grew. Users
        that need zeros on every call must leave the buffer zero themselves."""
        before = self.version
        out = self.get(name, shape, dtype)
        if self.version != before:
            self._bufs[name].zero_()
        return out

    def nbytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in self._bufs.values())


@dataclass
class NormedRows:
    """Rows of the residual stream with a norm still to be applied: what a norm hands to a
    consumer whose kernel normalizes its tokens itself while it reads them, instead of a tensor a
    norm kernel has written. ``rows`` (int32, on the device) selects rows of ``residual``; None
    means all of them in order. A consumer that cannot take it asks ``ops.normed(x)`` for the
    tensor."""

    residual: torch.Tensor          # [T, hidden] float32
    weight: torch.Tensor            # [hidden]
    eps: float
    dtype: torch.dtype              # the activation dtype the normalized rows stand for
    rows: torch.Tensor | None = None

    @property
    def shape(self) -> tuple[int, int]:
        n = self.rows.numel() if self.rows is not None else self.residual.shape[0]
        return (int(n), int(self.residual.shape[1]))


@dataclass
class Runtime:
    """What every part needs to run: the device, the activation dtype (bfloat16 for
    serving, float32 for the exact path), the kernel bindings and the buffer store."""

    device: torch.device
    dtype: torch.dtype
    ops: Any
    workspace: Workspace


class Part:
    """Base of every part."""

    def weights(self) -> dict[str, WeightWant]:
        """Relative weight name -> what is wanted."""
        return {}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        """Receives the wanted tensors (as stored: bfloat16 stays bfloat16, 32-bit stays
        32-bit) and moves/casts what it needs to the runtime's device and dtype."""
        self.rt = rt

    def weight_bytes(self) -> int:
        """Bytes of weights a step reads from this part (for roofline accounting)."""
        return 0



class Norm(Part):
    """A normalisation fused with the residual sum that precedes it."""

    def add_norm(self, residual: torch.Tensor, delta: torch.Tensor | None, out_name: str,
                 lazy: bool = False) -> "torch.Tensor | NormedRows":
        """residual (float32 [T,H], updated in place) += delta; returns norm(residual) in the
        activation dtype. ``delta`` is [T,H] or [S,T,H] float32 slices to be summed, or None when
        there is nothing to add (the first layer, or a sub-layer that added its output into the
        residual stream itself). The sum and the statistics are 32-bit. ``lazy``: the caller's
        consumer takes ``NormedRows``; the norm may then return that instead of running a kernel
        (only when delta is None: a consumer normalizes, it does not add)."""
        raise NotImplementedError

    def add_norm_rows(self, residual: torch.Tensor, delta: torch.Tensor | None, rows: torch.Tensor,
                      out_name: str, lazy: bool = False) -> "torch.Tensor | NormedRows":
        """The same for the selected rows only; ``residual`` is left as it is."""
        raise NotImplementedError


class PositionEncoding(Part):
    """Position information applied to queries and keys before attention."""

    def prepare(self, max_position: int) -> None:
        """Build tables for positions [0, max_position)."""


class RotaryTable(PositionEncoding):
    """A position encoding that rotates the pairs (i, i + D/2) of every query and key head by
    an angle that depends on the position and on i. It has ``head_dim`` and, once ``prepare``
    ran, ``table``: float32 ``[max_position, head_dim / 2, 2]`` = (cos, sin) on the device.
    How the angles come about is the subclass's business; attention only reads the table."""

    head_dim: int
    table: torch.Tensor | None = None


class Mixer(Part):
    """Mixes information between positions (attention here)."""

    def cache_need(self) -> CacheNeed | None:
        return None

    def state_need(self) -> StateNeed | None:
        return None

    # True: ``forward`` takes ``NormedRows`` for x (it hands x to kernels that normalize their
    # tokens themselves); the block then lets the norm in front of it be lazy.
    takes_normed_rows = False

    def forward(self, x: torch.Tensor, ctx: "StepContext", cache: Any, state: torch.Tensor | None,
                writes_cache: bool) -> torch.Tensor | None:
        """x [T, hidden] (activation dtype) -> what is to be added to the residual: [T, hidden]
        in the activation dtype, or [S, T, hidden] float32 slices whose sum it is, or None if the
        part has added its output into ``ctx.residual`` itself (the three things
        ``ops.linear_to_residual`` returns). ``cache`` is this run's ``LayerCache`` (pages of its group) or None; ``state`` is
        ``[num_slots, *shape]`` or None, indexed by ``ctx.slots``.

        Who clears a slot: the runner does. Before a step runs, every state tensor's rows for
        the items that start at position 0 are set to zero on the stream, so a request (new, or
        sent back by the scheduler and starting over) always meets zeros, whoever held the slot
        before. A mixer only reads and updates its rows; a state whose neutral value is not
        zero must be stored as the difference from it."""
        raise NotImplementedError


class Transform(Part):
    """Changes a float32 tensor of the step in place: the residual stream ``[T, hidden]`` right
    behind the token table, or the logits ``[S, vocab]``. ``rows`` are the flat token rows the
    tensor's rows belong to (all tokens in order for the stream, ``ctx.logit_rows`` for logits),
    for a transform that depends on the position (``ctx.positions[rows]``)."""

    def apply(self, t: torch.Tensor, ctx: "StepContext", rows: torch.Tensor | None) -> None:
        raise NotImplementedError


class FeedForward(Part):
    """Per-position transformation (dense or experts)."""

    takes_normed_rows = False       # as for Mixer

    def forward(self, x: torch.Tensor, ctx: "StepContext") -> torch.Tensor | None:
        """x [T, hidden] -> what is to be added to the residual, as for ``Mixer.forward``."""
        raise NotImplementedError


# ------------------------------------------------------------------ registries

Factory = Callable[..., Any]

_REGISTRIES: dict[str, dict[str, Factory]] = {
    "mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "block": {}, "transform": {},
}


def _register(family: str, kind: str, factory: Factory) -> None:
    table = _REGISTRIES[family]
    if kind in table and table[kind] is not factory:
        raise ValueError(f"{family} kind {kind!r} is already registered")
    table[kind] = factory


def register_mixer(kind: str, factory: Factory) -> None:
    """factory(hidden_size=..., positions={name: PositionEncoding}, **params) -> Mixer"""
    _register("mixer", kind, factory)


def register_feed_forward(kind: str, factory: Factory) -> None:
    """factory(hidden_size=..., **params) -> FeedForward"""
    _register("feed_forward", kind, factory)


def register_norm(kind: str, factory: Factory) -> None:
    """factory(hidden_size=..., **params) -> Norm"""
    _register("norm", kind, factory)


def register_position(kind: str, factory: Factory) -> None:
    """factory(**params) -> PositionEncoding"""
    _register("position", kind, factory)


def register_block(kind: str, factory: Factory) -> None:
    """factory(mixer=..., feed_forward=..., mixer_norm=..., feed_forward_norm=..., **extra_norms) -> Block"""
    _register("block", kind, factory)


def register_transform(kind: str, factory: Factory) -> None:
    """factory(hidden_size=..., vocab_size=..., **params) -> Transform"""
    _register("transform", kind, factory)


def make(family: str, kind: str, **kwargs: Any) -> Any:
    table = _REGISTRIES[family]
    if kind not in table:
        raise KeyError(f"no {family} of kind {kind!r}; registered: {sorted(table)}")
    return table[kind](**kwargs)
