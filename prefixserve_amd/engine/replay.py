"""Trace replay: feeds given token ids through the model step by step and hands back the
logits that were asked for. It samples nothing and has no forward pass, cache or loader of
its own: it drives the same ``ModelRunner.step`` and ``CacheManager`` that generation uses.

A step is ``{"step": k, "entries": [{"id", "tokens", "want"}...], "end": [ids]}``: all
entries form one batch (portions of prompts beside single decoded tokens); requests named
in ``end`` give back their pages and slot after the step. The reference's nearest
relatives are its test drivers (tests/test_llama_exact.py:130-167, teacher forcing in
tests/gpu/test_engine_flashinfer.py:45-83).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping

import numpy as np

from prefixserve_amd.cache.manager import CacheManager, blocks_for
from prefixserve_amd.engine.batch import EngineError, StepItem
from prefixserve_amd.engine.runner import ModelRunner


@dataclass
class _Live:
    slot: int
    tables: list[list[int]]
    length: int = 0
    tokens: list[int] = field(default_factory=list)


class TraceReplayer:
    def __init__(self, runner: ModelRunner, cache: CacheManager | None = None) -> None:
        self.runner = runner
        # Prefix caching stays off: a trace says which tokens a step runs, so none may be
        # skipped. Pages still come from the real allocator and are used again once freed.
        self.cache = cache if cache is not None else CacheManager(
            runner.num_blocks_per_group, runner.windows, runner.max_num_seqs, runner.state_bytes_per_slot,
            enable_prefix_cache=False)
        self.live: dict[Any, _Live] = {}

    def run_step(self, step: Mapping[str, Any]) -> np.ndarray | None:
        """Runs one step; returns float32 ``[wanted, vocab]`` or None if nothing was wanted."""
        entries = step.get("entries", [])
        items: list[StepItem] = []
        seen: set[Any] = set()
        for e in entries:
            rid = e["id"]
            if rid in seen:
                raise EngineError(f"request {rid!r} appears twice in step {step.get('step')}")
            seen.add(rid)
            toks = [int(t) for t in e["tokens"]]
            if not toks:
                raise EngineError(f"request {rid!r} brings no tokens in step {step.get('step')}")
            st = self.live.get(rid)
            if st is None:
                slot = self.cache.acquire_slot()
                if slot is None:
                    raise EngineError(f"no free state slot for request {rid!r}")
                st = _Live(slot=slot, tables=[[] for _ in range(self.cache.num_groups)])
                self.live[rid] = st
            need = [blocks_for(st.length + len(toks)) - len(t) for t in st.tables]
            fresh = self.cache.allocate([max(n, 0) for n in need])
            if fresh is None:
                raise EngineError(f"out of pages: request {rid!r} needs {need} more; --max-tokens is too small")
            for table, new in zip(st.tables, fresh):
                table.extend(new)
            items.append(StepItem(key=rid, tokens=toks, start=st.length, block_tables=st.tables, slot=st.slot,
                                  want=[int(w) for w in e.get("want", [])]))
        logits = self.runner.step(items) if items else None
        for it in items:
            st = self.live[it.key]
            st.length += len(it.tokens)
            self.cache.trim_windows(st.tables, st.length)
        out = None
        if logits is not None:
            out = logits.detach().to("cpu").numpy().astype(np.float32, copy=True)
        for rid in step.get("end", []):
            st = self.live.pop(rid, None)
            if st is None:
                raise EngineError(f"step {step.get('step')} ends unknown request {rid!r}")
            self.cache.release(st.tables)
            self.cache.release_slot(st.slot)
        return out
