"""Python entry point: run prompts to completion through the scheduler and the engine.

The loop is the reference's driver loop (README.md:321-336, prefixserve/server.py:209-243):
``add_request`` ... ``while has_work(): batch = schedule_step(); sampled = engine.step(batch);
commit(batch, sampled)``.
"""

from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Iterable, Sequence

from prefixserve_amd.engine.engine import Engine
from prefixserve_amd.engine.scheduler import AddResult, FinishReason, Scheduler, SchedulerStats


@dataclass
class Generation:
    req_id: str
    prompt: list[int]
    tokens: list[int] = field(default_factory=list)
    finish_reason: FinishReason | None = None
    cached_tokens: int = 0
    preemptions: int = 0


@dataclass
class LoopTimes:
    """Where the loop's time goes, summed over its steps: the same three intervals the
    reference's serving loop keeps (prefixserve/server.py:104-115, 221-237). ``engine_s`` is
    the whole of ``engine.step``: packing the step's arrays, the device's work and the wait
    for the sampled tokens."""

    steps: int = 0
    schedule_s: float = 0.0
    engine_s: float = 0.0
    commit_s: float = 0.0

    @property
    def scheduler_overhead(self) -> float:
        """schedule / (schedule + engine), the reference's "scheduler overhead" figure."""
        both = self.schedule_s + self.engine_s
        return self.schedule_s / both if both > 0 else 0.0

    def as_dict(self) -> dict[str, float]:
        return {"steps": self.steps, "schedule_s": self.schedule_s, "engine_s": self.engine_s,
                "commit_s": self.commit_s, "scheduler_overhead": self.scheduler_overhead}


def generate(engine: Engine, prompts: Sequence[Iterable[int]], max_tokens: int, *, temperature: float = 0.0,
             seed: int = 0, ignore_eos: bool = False, scheduler: Scheduler | None = None,
             max_prefill_tokens: int | None = None, max_running_requests: int | None = None,
             enable_prefix_cache: bool = True, decode_steps: int | None = None,
             times: LoopTimes | None = None) -> tuple[list[Generation], SchedulerStats]:
    """Generates up to ``max_tokens`` tokens for every prompt (token ids in, token ids out).
    ``decode_steps``: how many decode steps a batch of decoding requests may run before the
    host looks at the tokens (default: the engine configuration's). ``times``, if given, is
    added to step by step."""
    steps = decode_steps if decode_steps is not None else engine.cfg.decode_steps
    budget = max_prefill_tokens if max_prefill_tokens is not None else engine.cfg.max_prefill_tokens
    running = max_running_requests if max_running_requests is not None else engine.cfg.max_num_seqs
    sched = scheduler if scheduler is not None else engine.make_scheduler(
        chunk_size=budget, enable_prefix_cache=enable_prefix_cache)
    results: dict[str, Generation] = {}
    for i, p in enumerate(prompts):
        rid = f"req-{i}"
        ids = [int(t) for t in p]
        if len(ids) + max_tokens > engine.max_seq_len:
            raise ValueError(f"{rid}: {len(ids)} prompt + {max_tokens} new tokens exceed max_seq_len {engine.max_seq_len}")
        res = sched.add_request(rid, ids, max_tokens, ignore_eos=ignore_eos, temperature=temperature, seed=seed)
        if res is not AddResult.ACCEPTED:
            raise ValueError(f"{rid} rejected: {res.value}")
        results[rid] = Generation(rid, ids)
    clock = time.perf_counter
    while sched.has_work():
        t0 = clock()
        batch = sched.schedule_step(budget, running, steps)
        if not batch.work:
            raise RuntimeError("the scheduler has work but could schedule none of it (pool too small?)")
        tracked = {w.req.req_id: w.req for w in batch.work}
        t1 = clock()
        sampled = engine.step(batch)
        t2 = clock()
        step = sched.commit(batch, sampled)
        if times is not None:
            times.steps += 1
            times.schedule_s += t1 - t0
            times.engine_s += t2 - t1
            times.commit_s += clock() - t2
        for rid, toks in step.tokens.items():
            results[rid].tokens.extend(toks)
        for rid, why in step.finished.items():
            g, r = results[rid], tracked.get(rid)
            g.finish_reason = why
            if r is not None:
                g.cached_tokens, g.preemptions = r.cached_tokens, r.num_preemptions
    return [results[f"req-{i}"] for i in range(len(prompts))], sched.stats()
