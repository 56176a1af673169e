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


def logit_errors(trace, prompts, outs, plain, traced_rows_only: bool = False) -> list[float]:
    """Every row of an engine's ``logit_trace`` against the plain model run over the tokens the
    engine itself produced (so each row is judged given the same tokens before it, whatever
    the engine sampled): per row, max |difference| / max |truth|. Requests are "req-<index>".
    Rows a round of decode steps computed past a request's last token are skipped.
    ``traced_rows_only``: the plain model's logits at the traced positions only (a large
    vocabulary times every position of a long prompt is most of the work otherwise)."""
    import numpy as np

    truth = {}
    errors = []
    for rid, pos, row in trace:
        i = int(rid.split("-")[1])
        if i not in truth:
            seq = list(prompts[i]) + list(outs[i].tokens[:-1])
            if traced_rows_only:
                places = sorted({p for r, p, _ in trace if r == rid and p < len(seq)})
                truth[i] = dict(zip(places, plain.logits_at(seq, places)))
            else:
                truth[i] = dict(enumerate(plain.logits(seq)))
        if pos not in truth[i]:
            continue
        want = truth[i][pos]
        errors.append(float(np.abs(row.numpy() - want).max() / np.abs(want).max()))
    return errors


def plain_bf16_bars(model_dir, plain, reqs=None, truth=None, vocab=None) -> tuple[float, float]:
    """(mean row error, bar for a single row) of bfloat16 logits for the model in ``model_dir``:
    a plain run of it with every result rounded to bfloat16 against ``plain`` (the same model in
    float64), over ``reqs`` (whose float64 logits may be given as ``truth``) or over four random
    sequences of 130 tokens. The bar for a row is BF16_ROW_FACTOR x that run's worst row: how far
    8-bit rounding moves a row is the model's property, and the engine may do no worse than a
    plain implementation does."""
    import numpy as np

    from configs import BF16_ROW_FACTOR
    from plain.llama_plain import PlainLlama

    rough = PlainLlama(model_dir, bf16=True, weights=plain.w)
    if reqs is None:
        rng = np.random.default_rng(77)
        reqs = [rng.integers(0, vocab, 130).tolist() for _ in range(4)]
    rows = []
    for i, toks in enumerate(reqs):
        want = truth[i] if truth is not None else plain.logits(toks)
        rows.append(np.abs(rough.logits(toks) - want).max(-1) / np.abs(want).max(-1))
    rows = np.concatenate(rows)
    return float(rows.mean()), BF16_ROW_FACTOR * float(rows.max())
