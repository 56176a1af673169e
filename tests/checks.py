"""Assertions that several test files share."""

from __future__ import annotations

from typing import Any

PAGE = 16


class CacheWriteWatch:
    """Wraps an engine's step function and asserts, at every step, that no token is written
    into a page the prefix cache holds: such a page may be shared with other requests, now or
    later (the reference asserts the same per step, tests/test_llama_exact.py:145-151).
    ``writes`` counts the token writes that were looked at."""

    def __init__(self, engine: Any, scheduler: Any) -> None:
        self.writes = 0
        self.steps = 0
        inner = engine.runner.step
        cache = scheduler.cache

        def step(items, *args, **kwargs):
            self.steps += 1
            if cache.prefix_cache:
                for it in items:
                    for g, tree in enumerate(cache.trees):
                        table = it.block_tables[g]
                        for pos in range(it.start, it.start + len(it.tokens)):
                            page = int(table[pos // PAGE])
                            assert not tree.is_cached(page), (
                                f"step {self.steps}: {it.key} writes position {pos} into page {page}, "
                                f"which the prefix cache holds")
                            self.writes += 1
            return inner(items, *args, **kwargs)

        engine.runner.step = step


def logit_errors(trace, prompts, outs, plain) -> list[float]:
    """Every row of an engine's ``logit_trace`` against the plain model run over the tokens the
    engine itself produced (so each row is judged given the same tokens before it, whatever
    the engine sampled): per row, max |difference| / max |truth|. Requests are "req-<index>".
    Rows a round of decode steps computed past a request's last token are skipped."""
    import numpy as np

    truth = {}
    errors = []
    for rid, pos, row in trace:
        i = int(rid.split("-")[1])
        if i not in truth:
            truth[i] = plain.logits(list(prompts[i]) + list(outs[i].tokens[:-1]))
        if pos >= len(truth[i]):
            continue
        want = truth[i][pos]
        errors.append(float(np.abs(row.numpy() - want).max() / np.abs(want).max()))
    return errors
