"""Builds replay traces: the same requests cut in different ways. Every builder returns
``(steps, expect)`` where ``steps`` are the JSON objects a replay program reads and
``expect[k]`` lists, for step k, the (request, position) of each logits row it writes."""

from __future__ import annotations

import random
from typing import Sequence

Steps = list[dict]
Expect = list[list[tuple[int, int]]]


def whole(reqs: Sequence[Sequence[int]]) -> tuple[Steps, Expect]:
    """Each request alone and whole, logits at every position."""
    steps, expect = [], []
    for i, toks in enumerate(reqs):
        steps.append({"step": len(steps), "entries": [{"id": f"r{i}", "tokens": list(toks), "want": list(range(len(toks)))}],
                      "end": [f"r{i}"]})
        expect.append([(i, p) for p in range(len(toks))])
    return steps, expect


def decode_tail(reqs: Sequence[Sequence[int]], tail: int = 32) -> tuple[Steps, Expect]:
    """Most of a request in one step, its last ``tail`` tokens one by one."""
    steps, expect = [], []
    for i, toks in enumerate(reqs):
        n = len(toks)
        head = max(1, n - tail)
        steps.append({"step": len(steps), "entries": [{"id": f"r{i}", "tokens": list(toks[:head]), "want": [head - 1]}],
                      "end": []})
        expect.append([(i, head - 1)])
        for p in range(head, n):
            steps.append({"step": len(steps), "entries": [{"id": f"r{i}", "tokens": [toks[p]], "want": [0]}],
                          "end": [f"r{i}"] if p == n - 1 else []})
            expect.append([(i, p)])
        if head == n:
            steps[-1]["end"] = [f"r{i}"]
    return steps, expect


def portions(reqs: Sequence[Sequence[int]], sizes: Sequence[int] = (7, 2, 16, 3, 31, 2, 1, 5, 17, 2, 33, 4)) -> tuple[Steps, Expect]:
    """Portions of changing size, down to two tokens (and one); every page offset is crossed."""
    steps, expect = [], []
    for i, toks in enumerate(reqs):
        p, k = 0, i
        while p < len(toks):
            c = min(sizes[k % len(sizes)], len(toks) - p)
            k += 1
            last = p + c == len(toks)
            steps.append({"step": len(steps), "entries": [{"id": f"r{i}", "tokens": list(toks[p:p + c]), "want": list(range(c))}],
                          "end": [f"r{i}"] if last else []})
            expect.append([(i, q) for q in range(p, p + c)])
            p += c
    return steps, expect


def mixed(reqs: Sequence[Sequence[int]], max_live: int = 4, seed: int = 0, prompt_frac: float = 0.6) -> tuple[Steps, Expect, int]:
    """Up to ``max_live`` live requests per step: portions of some prompts beside single
    decoded tokens of others; a request may sit a step out. Also returns the most tokens live
    requests hold at any time (each rounded up to 64): a pool of that size is reused."""
    rng = random.Random(seed)
    state = [{"pos": 0, "prompt": max(1, int(len(t) * prompt_frac))} for t in reqs]
    waiting = list(range(len(reqs)))
    live: list[int] = []
    steps, expect = [], []
    peak = 0
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            live.append(waiting.pop(0))
        entries, exp, ended = [], [], []
        for i in list(live):
            st, toks = state[i], reqs[i]
            if len(live) > 1 and rng.random() < 0.15:
                continue                                    # left out of this step, goes on later
            if st["pos"] < st["prompt"]:
                c = min(rng.choice([2, 3, 5, 8, 13, 16, 21, 40]), st["prompt"] - st["pos"])
            else:
                c = 1
            c = min(c, len(toks) - st["pos"])
            want = list(range(c)) if rng.random() < 0.8 else [c - 1]
            entries.append({"id": f"r{i}", "tokens": list(toks[st["pos"]:st["pos"] + c]), "want": want})
            exp += [(i, st["pos"] + w) for w in want]
            st["pos"] += c
            if st["pos"] == len(toks):
                ended.append(i)
        peak = max(peak, sum(-(-state[i]["pos"] // 64) * 64 for i in live))
        if not entries:
            continue
        steps.append({"step": len(steps), "entries": entries, "end": [f"r{i}" for i in ended]})
        expect.append(exp)
        for i in ended:
            live.remove(i)
    return steps, expect, peak


def compare(run_step, steps: Steps, expect: Expect, truth: Sequence, tol: float, errors: list | None = None) -> float:
    """Runs the steps and checks every row against ``truth[req][pos]``. Returns the worst
    relative error (and appends every row's to ``errors``); fails naming the first wrong place."""
    import numpy as np

    worst = 0.0
    for step, exp in zip(steps, expect):
        got = run_step(step)
        if not exp:
            assert got is None
            continue
        assert got is not None and got.shape[0] == len(exp), f"step {step['step']}: {None if got is None else got.shape} rows for {len(exp)} wanted"
        for row, (i, p) in zip(got, exp):
            want = truth[i][p]
            err = float(np.abs(row - want).max() / np.abs(want).max())
            assert np.isfinite(err) and err <= tol, (
                f"step {step['step']}: request {i} position {p}: relative error {err:.3e} > {tol:.1e} "
                f"(entries {[(e['id'], len(e['tokens'])) for e in step['entries']]})")
            worst = max(worst, err)
            if errors is not None:
                errors.append(err)
    return worst
