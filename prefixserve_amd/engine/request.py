"""What the scheduler and the engine pass to each other: requests, the items of a step, the
batch, and what a commit reports. The names and their meanings are those of the reference's
Python API (prefixserve/scheduler.py:44-140): a caller of that library finds the same
fields here; sampling options, state slots and per-group block tables are additions.
"""

from __future__ import annotations

import enum
from dataclasses import dataclass, field
from typing import Sequence

import numpy as np


class SchedulerError(RuntimeError):
    """schedule_step and commit were not called in turn, or with the wrong batch."""


class AddResult(enum.Enum):
    """Answer of ``add_request``."""

    ACCEPTED = "accepted"
    INVALID = "invalid"              # empty id, no or non-integer tokens, max_tokens < 1, ...
    DUPLICATE_ID = "duplicate_id"
    TOO_LONG = "too_long"            # prompt + max_tokens exceed the whole pool
    QUEUE_FULL = "queue_full"


class FinishReason(str, enum.Enum):
    STOP = "stop"                    # a stop token was sampled (it is part of the output)
    LENGTH = "length"                # max_tokens reached
    ABORT = "abort"                  # free_request


class ReqState(enum.Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


@dataclass(eq=False)
class Request:
    """One generation. ``prompt + output`` is the sequence; ``num_computed`` counts the tokens
    of it whose keys and values are in the cache. ``arrival`` never changes, so a request keeps
    its place among the running ones through preemptions."""

    req_id: str
    prompt: np.ndarray
    max_tokens: int
    arrival: int
    ignore_eos: bool = False
    temperature: float = 0.0
    seed: int = 0
    state: ReqState = ReqState.WAITING
    output: list[int] = field(default_factory=list)
    # One table per layer group; the request holds one reference on every entry that is >= 0.
    block_tables: list[list[int]] = field(default_factory=list)
    slot: int = -1
    num_computed: int = 0
    cached_tokens: int = 0           # taken from the prefix cache, summed over admissions
    num_preemptions: int = 0
    abort_pending: bool = False
    prompt_cached: bool = False

    @property
    def seq_len(self) -> int:
        return self.prompt.shape[0] + len(self.output)

    @property
    def block_table(self) -> list[int]:
        """Table of the first layer group (all there is for a model with one group)."""
        return self.block_tables[0] if self.block_tables else []

    def seq(self) -> np.ndarray:
        """prompt + output as one int32 array."""
        if self.output:
            return np.concatenate([self.prompt, np.asarray(self.output, dtype=np.int32)])
        return self.prompt

    def tokens(self, start: int, end: int) -> np.ndarray | list[int]:
        """seq[start:end] without building seq: a view of the prompt, a slice of the output
        list (what every decode step asks for), or the two joined."""
        p = self.prompt.shape[0]
        if start >= p:
            return self.output[start - p:end - p]
        if end <= p:
            return self.prompt[start:end]
        return np.concatenate([self.prompt[start:], np.asarray(self.output[:end - p], dtype=np.int32)])


@dataclass(frozen=True)
class WorkItem:
    """Run seq[start:end] of ``req`` in this step."""

    req: Request
    start: int
    end: int

    @property
    def samples(self) -> bool:
        """True if the item ends where the sequence ends: then a token is sampled for it."""
        return self.req.seq_len == self.end


@dataclass(frozen=True)
class Batch:
    """The work of one step. ``decode_steps`` > 1: every item is a decoding request and the
    engine runs that many steps in a row for them (step j of a request starts at
    ``start + j``), handing each step's token to the next on the device; ``commit`` then
    takes a list of tokens per request."""

    work: list[WorkItem]
    preempted: list[str]
    decode_steps: int = 1

    @property
    def num_tokens(self) -> int:
        return sum(item.end - item.start for item in self.work)


@dataclass(frozen=True)
class StepResult:
    """``new_tokens``: the last token each request got in this commit; ``tokens``: all of them
    in order (more than one after a batch of several decode steps)."""

    new_tokens: dict[str, int]
    finished: dict[str, FinishReason]
    tokens: dict[str, list[int]] = field(default_factory=dict)


@dataclass(frozen=True)
class SchedulerStats:
    num_waiting: int
    num_running: int
    free_blocks: int
    cached_blocks: int
    prompt_tokens: int
    cached_prompt_tokens: int        # counted at a request's first admission only
    preemptions: int
    rejected: int

    @property
    def prefix_hit_rate(self) -> float:
        return self.cached_prompt_tokens / self.prompt_tokens if self.prompt_tokens > 0 else 0.0


def as_token_list(value: int | Sequence[int]) -> list[int]:
    """What an engine returned for one request: one token or one per decode step."""
    if isinstance(value, (int, np.integer)):
        return [int(value)]
    return [int(t) for t in value]
