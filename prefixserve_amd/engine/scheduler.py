"""Continuous-batching scheduler over the cache manager.

Every request is a token list ``seq = prompt + output`` and a counter ``num_computed``
(tokens whose keys and values are in the cache). A step runs some of
``seq[num_computed:]`` for each scheduled request; a request that reaches the end of its
``seq`` gets one new token sampled. Decode is "one token left", prefill "more than one
left", recomputation after preemption is prefill again: one code path for all three.

The rules are the reference's (prefixserve/scheduler.py:143-451): running requests first
and oldest first; decodes never use the prefill budget; prompts are cut into portions of
at most ``chunk_size`` under a shared per-step token budget; admission is FIFO, matches the
prefix cache on ``seq[:-1]`` and never preempts; a running request that needs pages evicts
cached prefixes and then preempts the NEWEST running request (recompute, not swap), which
returns to the front of the queue; aborting a request of the batch in flight waits for
``commit``. Added here: a state slot per running request, block tables per layer group,
release of pages a window has passed, and per-request sampling options.

Not thread-safe, on purpose: one owner drives schedule_step -> engine.step -> commit.
"""

from __future__ import annotations

import bisect
import logging
import time
from collections import deque
from dataclasses import dataclass, field
from enum import Enum
from typing import Iterable, Mapping, Sequence

import numpy as np

from prefixserve_amd.cache.manager import BLOCK_SIZE, CacheManager, blocks_for

logger = logging.getLogger(__name__)

DEFAULT_CHUNK_SIZE = 512
SLOW_STEP_SECONDS = 1e-3


class SchedulerError(RuntimeError):
    """The caller broke the schedule -> commit protocol."""


class ReqState(Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


class FinishReason(str, Enum):
    LENGTH = "length"
    STOP = "stop"
    ABORT = "abort"


class AddResult(Enum):
    ACCEPTED = "accepted"
    QUEUE_FULL = "queue_full"
    TOO_LONG = "too_long"          # cannot fit even with the whole pool to itself
    DUPLICATE_ID = "duplicate_id"
    INVALID = "invalid"


@dataclass(eq=False)
class Request:
    req_id: str
    prompt: np.ndarray
    max_tokens: int
    arrival: int                    # fixed for life, so priority survives preemption
    ignore_eos: bool = False
    temperature: float = 0.0
    seed: int = 0
    state: ReqState = ReqState.WAITING
    output: list[int] = field(default_factory=list)
    block_tables: list[list[int]] = field(default_factory=list)   # one per layer group; 1 ref held on each entry
    slot: int = -1
    num_computed: int = 0
    cached_tokens: int = 0          # tokens reused from the prefix cache, summed over admissions
    num_preemptions: int = 0
    abort_pending: bool = False
    prompt_cached: bool = False

    @property
    def seq_len(self) -> int:
        return len(self.prompt) + len(self.output)

    @property
    def block_table(self) -> list[int]:
        """The table of the first layer group (the only one for a single-group model)."""
        return self.block_tables[0] if self.block_tables else []

    def seq(self) -> np.ndarray:
        if not self.output:
            return self.prompt
        return np.concatenate((self.prompt, np.asarray(self.output, dtype=np.int32)))

    def tokens(self, start: int, end: int) -> np.ndarray | list[int]:
        """seq[start:end] without building the whole sequence: an array, or a list when all
        of it is output (every decode step asks for that; a slice of a list costs least)."""
        n = len(self.prompt)
        if end <= n:
            return self.prompt[start:end]
        if start >= n:
            return self.output[start - n:end - n]
        return np.concatenate((self.prompt[start:], np.asarray(self.output[:end - n], dtype=np.int32)))


@dataclass(frozen=True)
class WorkItem:
    req: Request
    start: int      # run seq[start:end]
    end: int

    @property
    def samples(self) -> bool:
        """The item reaches the end of seq, so a token must be sampled for it."""
        return self.end == self.req.seq_len


@dataclass(frozen=True)
class Batch:
    """``decode_steps`` > 1: every item is a decoding request and the engine runs that many
    steps in a row for them (item j of a request starts at ``start + j``), feeding each step's
    token to the next on the device; ``commit`` then takes a list of tokens per request."""

    work: list[WorkItem]
    preempted: list[str]
    decode_steps: int = 1

    @property
    def num_tokens(self) -> int:
        return sum(w.end - w.start for w in self.work)


@dataclass(frozen=True)
class StepResult:
    """``new_tokens``: the last token each request got in this commit; ``tokens``: all of
    them in order (more than one after a batch of several decode steps)."""

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
    cached_prompt_tokens: int
    preemptions: int
    rejected: int

    @property
    def prefix_hit_rate(self) -> float:
        return self.cached_prompt_tokens / self.prompt_tokens if self.prompt_tokens else 0.0


class Scheduler:
    def __init__(self, num_blocks: int | Sequence[int] | None = None, *, max_waiting: int = 1024,
                 chunk_size: int = DEFAULT_CHUNK_SIZE, stop_token_ids: Iterable[int] = (),
                 enable_prefix_cache: bool = True, cache: CacheManager | None = None,
                 num_slots: int = 1024) -> None:
        if max_waiting < 1 or chunk_size < 1:
            raise ValueError("max_waiting and chunk_size must be >= 1")
        if cache is None:
            if num_blocks is None:
                raise ValueError("give num_blocks or a CacheManager")
            sizes = [num_blocks] if isinstance(num_blocks, int) else list(num_blocks)
            cache = CacheManager(sizes, num_slots=num_slots, enable_prefix_cache=enable_prefix_cache)
        self.cache = cache
        self.block_manager = cache.pools[0]
        self.tree = cache.trees[0] if cache.trees else None
        self._max_waiting = max_waiting
        self._chunk_size = chunk_size
        self._stop = frozenset(int(t) for t in stop_token_ids)

        self._requests: dict[str, Request] = {}
        self._waiting: deque[Request] = deque()
        self._running: list[Request] = []     # by arrival, newest last
        self._inflight: Batch | None = None
        self._pending_aborts: list[Request] = []
        self._next_arrival = 0
        self._prompt_tokens = 0
        self._cached_prompt_tokens = 0
        self._preemptions = 0
        self._rejected = 0

    # ---------------------------------------------------------------- API

    def add_request(self, req_id: str, prompt: Iterable[int] | np.ndarray, max_tokens: int, *,
                    ignore_eos: bool = False, temperature: float = 0.0, seed: int = 0) -> AddResult:
        checked = self._validate(req_id, prompt, max_tokens, temperature)
        if isinstance(checked, AddResult):
            self._rejected += 1
            return checked
        req = Request(req_id=req_id, prompt=checked, max_tokens=max_tokens, arrival=self._next_arrival,
                      ignore_eos=ignore_eos, temperature=float(temperature), seed=int(seed))
        self._next_arrival += 1
        self._requests[req_id] = req
        self._waiting.append(req)
        self._prompt_tokens += len(checked)
        return AddResult.ACCEPTED

    def schedule_step(self, max_prefill_tokens: int, max_decode_seqs: int, decode_steps: int = 1) -> Batch:
        """Chooses this step's work. ``commit`` must follow before the next call.

        ``decode_steps`` > 1 lets a batch that holds nothing but decoding requests, with nobody
        waiting, run up to that many steps before the host looks at the tokens (fewer if a
        request would pass its ``max_tokens`` or the free pages do not reach). A request that
        meets a stop token in between finishes there; what was computed for it after that is
        dropped. Nothing else changes: the pages for those positions are taken now."""
        if self._inflight is not None:
            raise SchedulerError("commit() the previous batch before scheduling another")
        if max_prefill_tokens < 1 or max_decode_seqs < 1:
            raise ValueError("max_prefill_tokens and max_decode_seqs must be >= 1")
        started = time.perf_counter()
        work: list[WorkItem] = []
        preempted: list[str] = []
        budget = max_prefill_tokens

        # Running requests, oldest first. A victim of _reserve is always newer than the
        # asker, hence later in this loop and never in `work` already.
        i = 0
        while i < len(self._running):
            req = self._running[i]
            remaining = req.seq_len - req.num_computed
            n = 1 if remaining == 1 else min(self._chunk_size, remaining, budget)
            if n == 0:           # budget used up: this prefill waits a step
                i += 1
                continue
            need = [max(blocks_for(req.num_computed + n) - len(t), 0) for t in req.block_tables]
            if any(need) and not self._reserve(req, need, preempted):
                continue         # req preempted itself; the same index now holds the next request
            if remaining > 1:
                budget -= n
            work.append(WorkItem(req, req.num_computed, req.num_computed + n))
            i += 1

        # Waiting requests, first come first served; the head that cannot start blocks the rest.
        while self._waiting and len(self._running) < max_decode_seqs:
            item = self._admit(self._waiting[0], budget)
            if item is None:
                break
            self._waiting.popleft()
            if item.end - item.start > 1:
                budget -= item.end - item.start
            work.append(item)

        steps = 1
        if (decode_steps > 1 and work and not self._waiting and not preempted
                and all(w.end - w.start == 1 and w.samples for w in work)):
            steps = min(decode_steps, min(w.req.max_tokens - len(w.req.output) for w in work))
            for w in work:
                if steps == 1:
                    break
                need = [max(blocks_for(w.start + steps) - len(t), 0) for t in w.req.block_tables]
                if any(need):
                    fresh = self.cache.allocate(need)
                    if fresh is None:
                        steps = 1        # pages already taken for others stay theirs: they will be used
                    else:
                        for table, new in zip(w.req.block_tables, fresh):
                            table.extend(new)
        batch = Batch(work=work, preempted=preempted, decode_steps=steps)
        self._inflight = batch
        elapsed = time.perf_counter() - started
        if elapsed > SLOW_STEP_SECONDS:
            logger.debug("schedule_step took %.2f ms", elapsed * 1e3)
        return batch

    def commit(self, batch: Batch, sampled: Mapping[str, int]) -> StepResult:
        """Applies the engine's results; ``sampled`` has a token for every item that samples."""
        if batch is not self._inflight:
            raise SchedulerError("commit() got a batch that isn't the one in flight")
        self._inflight = None
        new_tokens: dict[str, int] = {}
        all_tokens: dict[str, list[int]] = {}
        finished: dict[str, FinishReason] = {}
        for w in batch.work:
            req = w.req
            if req.num_computed != w.start:
                raise SchedulerError(f"{req.req_id}: batch is stale")
            if not w.samples:
                req.num_computed = w.end
                self.cache.trim_windows(req.block_tables, req.num_computed)
                continue
            if req.req_id not in sampled:
                raise SchedulerError(f"engine returned no token for {req.req_id}")
            got = sampled[req.req_id]
            tokens = [int(got)] if isinstance(got, (int, np.integer)) else [int(t) for t in got]
            if len(tokens) != batch.decode_steps:
                raise SchedulerError(f"{req.req_id}: {len(tokens)} tokens for {batch.decode_steps} decode steps")
            for j, token in enumerate(tokens):
                req.num_computed = w.end + j
                self.cache.trim_windows(req.block_tables, req.num_computed)
                if not req.prompt_cached:      # prompt complete for the first time: share it now
                    self._cache(req)
                    req.prompt_cached = True
                req.output.append(token)
                new_tokens[req.req_id] = token
                all_tokens.setdefault(req.req_id, []).append(token)
                if req.abort_pending:
                    break
                if token in self._stop and not req.ignore_eos:
                    self._finish(req, FinishReason.STOP)
                    finished[req.req_id] = FinishReason.STOP
                    break
                if len(req.output) >= req.max_tokens:
                    self._finish(req, FinishReason.LENGTH)
                    finished[req.req_id] = FinishReason.LENGTH
                    break
        for req in self._pending_aborts:   # safe now: the batch that wrote their pages is done
            if req.state is ReqState.RUNNING:
                self._finish(req, FinishReason.ABORT)
                finished[req.req_id] = FinishReason.ABORT
        self._pending_aborts.clear()
        return StepResult(new_tokens=new_tokens, finished=finished, tokens=all_tokens)

    def free_request(self, req_id: str) -> bool:
        """Aborts a request. False for an unknown id or a second call."""
        req = self._requests.get(req_id)
        if req is None or req.abort_pending:
            return False
        if req.state is ReqState.WAITING:
            self._waiting.remove(req)
            req.state = ReqState.FINISHED
            del self._requests[req_id]
            return True
        if self._inflight is not None:
            # The device may still be writing this request's pages; give them back at commit.
            req.abort_pending = True
            self._pending_aborts.append(req)
            return True
        self._finish(req, FinishReason.ABORT)
        return True

    def get_request(self, req_id: str) -> Request | None:
        return self._requests.get(req_id)

    def has_work(self) -> bool:
        return bool(self._waiting or self._running)

    def stats(self) -> SchedulerStats:
        return SchedulerStats(
            num_waiting=len(self._waiting), num_running=len(self._running),
            free_blocks=self.cache.num_free(0), cached_blocks=self.cache.num_cached(0),
            prompt_tokens=self._prompt_tokens, cached_prompt_tokens=self._cached_prompt_tokens,
            preemptions=self._preemptions, rejected=self._rejected)

    # ---------------------------------------------------------- internals

    def _validate(self, req_id: str, prompt: Iterable[int] | np.ndarray, max_tokens: int,
                  temperature: float) -> np.ndarray | AddResult:
        if not req_id or not isinstance(max_tokens, int) or isinstance(max_tokens, bool) or max_tokens < 1:
            return AddResult.INVALID
        try:
            if not float(temperature) >= 0.0:
                return AddResult.INVALID
            arr = np.asarray(prompt)
        except (TypeError, ValueError, OverflowError):
            return AddResult.INVALID
        if arr.ndim != 1 or arr.size == 0 or arr.dtype.kind not in "iu":
            return AddResult.INVALID      # floats would be truncated silently
        if int(arr.min()) < 0 or int(arr.max()) > np.iinfo(np.int32).max:
            return AddResult.INVALID
        if req_id in self._requests:
            return AddResult.DUPLICATE_ID
        total = int(arr.size) + max_tokens
        for g in range(self.cache.num_groups):
            if self.cache.pages_needed(g, total, self._chunk_size) > self.cache.num_blocks(g):
                return AddResult.TOO_LONG  # could never finish even alone
        if len(self._waiting) >= self._max_waiting:
            return AddResult.QUEUE_FULL
        return arr.astype(np.int32)       # a copy: later changes by the caller do not reach us

    def _admit(self, req: Request, budget: int) -> WorkItem | None:
        seq = req.seq()
        # At least one token stays to be computed: the model must run something to give logits.
        matched, cached = self.cache.match_prefix(seq[:-1])
        remaining = len(seq) - matched
        n = 1 if remaining == 1 else min(self._chunk_size, remaining, budget)
        fresh = None
        slot = None
        if n > 0:
            slot = self.cache.acquire_slot()
            if slot is not None:
                need = [blocks_for(matched + n) - len(t) for t in cached]
                fresh = self.cache.allocate(need)
        if fresh is None:
            # Admission never preempts: evicting a running request to start a new one only
            # swaps who waits, and under load both keep redoing work.
            self.cache.release(cached)
            if slot is not None:
                self.cache.release_slot(slot)
            return None
        req.block_tables = [c + f for c, f in zip(cached, fresh)]
        req.slot = slot if slot is not None else -1
        req.num_computed = matched
        req.cached_tokens += matched
        if req.num_preemptions == 0:
            self._cached_prompt_tokens += min(matched, len(req.prompt))
        req.state = ReqState.RUNNING
        bisect.insort(self._running, req, key=lambda r: r.arrival)
        return WorkItem(req, matched, matched + n)

    def _reserve(self, req: Request, need: list[int], preempted: list[str]) -> bool:
        """More pages for a running request: evict cached prefixes, then preempt the newest
        running request, until it fits. False if ``req`` itself had to go. The oldest request
        can take from everyone newer and nothing admitted exceeds the pool, so it finishes."""
        while True:
            fresh = self.cache.allocate(need)
            if fresh is not None:
                for table, new in zip(req.block_tables, fresh):
                    table.extend(new)
                return True
            victim = self._running[-1]
            self._preempt(victim)
            preempted.append(victim.req_id)
            if victim is req:
                return False

    def _release(self, req: Request) -> None:
        self.cache.release(req.block_tables)
        req.block_tables = []
        if req.slot >= 0:
            self.cache.release_slot(req.slot)
            req.slot = -1

    def _preempt(self, req: Request) -> None:
        # Recompute, not swap; but what it computed is cached first, so coming back is
        # usually a prefix hit on its own pages.
        self._cache(req)
        self._release(req)
        req.num_computed = 0
        req.num_preemptions += 1
        req.state = ReqState.WAITING
        self._running.remove(req)
        self._waiting.appendleft(req)
        self._preemptions += 1

    def _finish(self, req: Request, reason: FinishReason) -> None:
        self._cache(req)
        self._release(req)
        req.state = ReqState.FINISHED
        self._running.remove(req)
        del self._requests[req.req_id]
        logger.debug("finished %s: %s", req.req_id, reason.value)

    def _cache(self, req: Request) -> None:
        if req.num_computed >= BLOCK_SIZE:
            self.cache.cache(req.seq()[:req.num_computed], req.block_tables)
