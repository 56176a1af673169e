"""The scheduler's decisions, one rule per test, with a fake engine (a fresh token for every
item that samples). The vectors are the reference's (tests/test_scheduler.py:55-262,
tests/test_invariants.py:23-108); window groups, slots and sampling options are added."""

from __future__ import annotations

import itertools
import random

import numpy as np
import pytest

from prefixserve_amd import (BLOCK_SIZE, AddResult, Batch, FinishReason, Scheduler, SchedulerError)
from prefixserve_amd.cache import CacheManager

_tok = itertools.count(1000)


def sample(batch):
    return {w.req.req_id: next(_tok) for w in batch.work if w.samples}


def step(s, budget=2048, max_seqs=8):
    batch = s.schedule_step(budget, max_seqs)
    return batch, s.commit(batch, sample(batch))


def run_until_done(s, budget=2048, max_seqs=8, cap=10_000):
    batches = []
    for _ in range(cap):
        if not s.has_work():
            return batches
        batches.append(step(s, budget, max_seqs)[0])
    raise AssertionError("scheduler did not finish: possible livelock")


def assert_clean(s):
    s.cache.check_invariants()
    s.cache.evict_all()
    for g in range(s.cache.num_groups):
        assert s.cache.num_free(g) == s.cache.num_blocks(g)
    assert s.cache.slots.num_free == s.cache.slots.num_slots


def toks(n, start=0):
    return list(range(start, start + n))


def test_every_decode_runs_every_step():
    s = Scheduler(64)
    for i in range(4):
        assert s.add_request(f"r{i}", toks(16, 100 * i), max_tokens=10) is AddResult.ACCEPTED
    step(s)
    for _ in range(5):
        batch, _ = step(s)
        assert sorted(w.req.req_id for w in batch.work) == ["r0", "r1", "r2", "r3"]
        assert all(w.end - w.start == 1 for w in batch.work)
    run_until_done(s)
    assert_clean(s)


def test_decodes_ignore_the_prefill_budget():
    s = Scheduler(256)
    s.add_request("short", toks(16), max_tokens=50)
    step(s)
    s.add_request("long", toks(2000, 5000), max_tokens=1)
    batch, _ = step(s, budget=1)
    by_id = {w.req.req_id: w for w in batch.work}
    assert by_id["short"].end - by_id["short"].start == 1
    assert by_id["long"].end - by_id["long"].start == 1


def test_portions_of_512_and_shared_budget():
    s = Scheduler(256)
    s.add_request("big", toks(1300), max_tokens=1)
    sizes = []
    for _ in range(3):
        batch, result = step(s)
        sizes.append(batch.work[0].end - batch.work[0].start)
    assert sizes == [512, 512, 276] and result.finished == {"big": FinishReason.LENGTH}
    s = Scheduler(256)
    s.add_request("a", toks(1000), max_tokens=1)
    s.add_request("b", toks(1000, 5000), max_tokens=1)
    batch, _ = step(s, budget=600)
    assert [(w.req.req_id, w.end - w.start) for w in batch.work] == [("a", 512), ("b", 88)]
    assert batch.num_tokens == 600


def test_shared_prefix_is_reused_and_identical_prompt_still_computes():
    s = Scheduler(128)
    system = toks(256, 7000)
    s.add_request("first", system + toks(20), max_tokens=2)
    run_until_done(s)
    free_before = s.block_manager.num_free
    s.add_request("second", system + toks(30, 900), max_tokens=2)
    batch, _ = step(s)
    req = batch.work[0].req
    assert req.cached_tokens == 256 and batch.work[0].start == 256
    assert free_before - s.block_manager.num_free == 2             # only the 30-token tail
    assert s.stats().prefix_hit_rate > 0
    run_until_done(s)
    assert_clean(s)
    s = Scheduler(64)
    s.add_request("a", toks(64), max_tokens=1)
    run_until_done(s)
    s.add_request("b", toks(64), max_tokens=1)
    batch, result = step(s)
    assert (batch.work[0].start, batch.work[0].end) == (48, 64)    # matched on seq[:-1]
    assert "b" in result.new_tokens
    assert_clean(s)


def test_out_of_pages_preempts_the_newest_and_all_finish():
    s = Scheduler(12)
    for name in ("a", "b", "c"):
        assert s.add_request(name, toks(48, ord(name) * 100), max_tokens=60) is AddResult.ACCEPTED
    batches = run_until_done(s)
    preempted = [rid for b in batches for rid in b.preempted]
    assert preempted and "a" not in preempted                      # the oldest is never preempted
    assert s.stats().preemptions == len(preempted)
    assert_clean(s)


def test_preempted_request_finds_its_own_pages_again():
    s = Scheduler(10)
    s.add_request("a", toks(64, 0), max_tokens=40)
    s.add_request("b", toks(64, 5000), max_tokens=40)
    b = s.get_request("b")
    run_until_done(s)
    assert b.num_preemptions >= 1 and b.cached_tokens > 0
    assert_clean(s)


def test_admission_never_preempts():
    s = Scheduler(6)
    s.add_request("a", toks(80), max_tokens=10)                    # 5 pages, 6 at the end
    step(s)
    s.add_request("b", toks(40, 900), max_tokens=4)                # needs 3, only 1 free
    batch, _ = step(s)
    assert [w.req.req_id for w in batch.work] == ["a"] and not batch.preempted
    assert s.stats().num_waiting == 1
    run_until_done(s)
    assert_clean(s)


def test_abort_in_flight_waits_for_commit():
    s = Scheduler(16)
    s.add_request("a", toks(40), max_tokens=10)
    batch = s.schedule_step(512, 8)
    held = list(batch.work[0].req.block_table)
    assert s.free_request("a") is True and s.free_request("a") is False
    assert all(s.block_manager.ref_count(b) >= 1 for b in held)    # the step may still write them
    result = s.commit(batch, sample(batch))
    assert result.finished == {"a": FinishReason.ABORT} and s.get_request("a") is None
    assert_clean(s)


def test_abort_when_idle_and_while_waiting():
    s = Scheduler(16)
    s.add_request("run", toks(20), max_tokens=10)
    step(s)
    assert s.free_request("run") is True
    s.add_request("wait", toks(20), max_tokens=10)
    batch = s.schedule_step(512, 8)
    s.add_request("queued", toks(20, 50), max_tokens=10)
    assert s.free_request("queued") is True
    s.commit(batch, sample(batch))
    assert s.free_request("nope") is False
    s.free_request("wait")
    assert_clean(s)


def test_rejections():
    s = Scheduler(8, max_waiting=2)
    assert s.add_request("", toks(4), 1) is AddResult.INVALID
    assert s.add_request("x", [], 1) is AddResult.INVALID
    assert s.add_request("x", toks(4), 0) is AddResult.INVALID
    assert s.add_request("x", [1, -2], 1) is AddResult.INVALID
    assert s.add_request("x", [1.5, 2.0], 1) is AddResult.INVALID
    assert s.add_request("x", [[1, 2]], 1) is AddResult.INVALID
    assert s.add_request("x", [2 ** 40], 1) is AddResult.INVALID
    assert s.add_request("x", toks(8 * BLOCK_SIZE), 1) is AddResult.TOO_LONG
    assert s.add_request("a", toks(4), 1) is AddResult.ACCEPTED
    assert s.add_request("a", toks(4), 1) is AddResult.DUPLICATE_ID
    assert s.add_request("b", np.arange(4, dtype=np.int64), 1) is AddResult.ACCEPTED
    assert s.add_request("c", toks(4), 1) is AddResult.QUEUE_FULL
    assert s.stats().rejected == 10
    assert s.add_request("t", toks(4), 1, temperature=-1.0) is AddResult.INVALID


def test_prompt_is_copied_and_finish_reasons():
    s = Scheduler(8)
    p = np.arange(20, dtype=np.int32)
    s.add_request("a", p, 1)
    p[:] = 0
    assert s.get_request("a").prompt[5] == 5
    s = Scheduler(32, stop_token_ids={4242})
    s.add_request("len", toks(40), max_tokens=3)
    _, result = step(s)
    assert result.finished == {}
    run_until_done(s)
    s.add_request("eos", toks(40, 300), max_tokens=100)
    batch = s.schedule_step(512, 8)
    result = s.commit(batch, {"eos": 4242})
    assert result.finished == {"eos": FinishReason.STOP} and result.new_tokens == {"eos": 4242}
    assert s.tree.num_cached_blocks >= 4
    s.add_request("ign", toks(40, 600), max_tokens=2, ignore_eos=True)
    batch = s.schedule_step(512, 8)
    assert s.commit(batch, {"ign": 4242}).finished == {}            # runs on to max_tokens
    run_until_done(s)
    assert_clean(s)


def test_protocol_errors_and_bad_arguments():
    s = Scheduler(16)
    s.add_request("a", toks(20), 5)
    batch = s.schedule_step(512, 8)
    with pytest.raises(SchedulerError):
        s.schedule_step(512, 8)
    with pytest.raises(SchedulerError):
        s.commit(Batch(work=[], preempted=[]), {})
    with pytest.raises(SchedulerError, match="no token"):
        s.commit(batch, {})
    s = Scheduler(16)
    with pytest.raises(ValueError):
        s.schedule_step(0, 8)
    with pytest.raises(ValueError):
        s.schedule_step(512, 0)
    with pytest.raises(ValueError):
        Scheduler(16, chunk_size=0)


def test_running_cap_and_slots():
    s = Scheduler(256, num_slots=3)
    for i in range(10):
        s.add_request(f"r{i}", toks(16, i * 100), max_tokens=5)
    for _ in range(20):
        batch = s.schedule_step(2048, 5)                            # slots (3) bind before the cap (5)
        assert s.stats().num_running <= 3
        slots = [w.req.slot for w in batch.work]
        assert len(set(slots)) == len(slots) and all(0 <= x < 3 for x in slots)
        s.commit(batch, sample(batch))
    run_until_done(s, max_seqs=5)
    assert_clean(s)


def test_prefix_cache_can_be_switched_off():
    s = Scheduler(64, enable_prefix_cache=False)
    s.add_request("a", toks(64), max_tokens=1)
    run_until_done(s)
    s.add_request("b", toks(64), max_tokens=1)
    batch, _ = step(s)
    assert (batch.work[0].start, batch.work[0].end) == (0, 64) and s.stats().cached_blocks == 0
    assert_clean(s)


def test_window_group_gives_pages_back_while_running():
    cache = CacheManager([64, 6], windows=[None, 32], num_slots=4)
    s = Scheduler(cache=cache, chunk_size=32)
    assert s.add_request("w", toks(200), max_tokens=40) is AddResult.ACCEPTED   # 15 pages would not fit group 1
    peak = 0
    while s.has_work():
        batch, _ = step(s, budget=32)
        req = batch.work[0].req
        if req.block_tables:
            peak = max(peak, sum(1 for b in req.block_tables[1] if b >= 0))
    assert peak <= 5
    assert_clean(s)


def test_random_load_keeps_the_ref_count_invariant():
    """rc(page) == requests holding it + cached, after every step; all work finishes; nothing leaks."""
    rng = random.Random(11)
    s = Scheduler(24, chunk_size=24)
    shared = toks(32, 9000)
    n_added = 0
    for it in range(1500):
        r = rng.random()
        if r < 0.25 and n_added < 400:
            prompt = (shared if rng.random() < 0.5 else []) + toks(rng.randint(1, 70), rng.randint(0, 50))
            s.add_request(f"q{n_added}", prompt, max_tokens=rng.randint(1, 30))
            n_added += 1
        elif r < 0.3 and s._requests:
            s.free_request(rng.choice(list(s._requests)))
        else:
            batch = s.schedule_step(24, 4)
            if rng.random() < 0.1 and batch.work:
                s.free_request(rng.choice(batch.work).req.req_id)   # abort during the step
            s.commit(batch, sample(batch))
        holders = np.zeros(24, dtype=int)
        for req in s._requests.values():
            for b in req.block_table:
                holders[b] += 1
        for b in range(24):
            assert s.block_manager.ref_count(b) == holders[b] + int(s.tree.is_cached(b))
        s.cache.check_invariants()
    run_until_done(s, budget=24, max_seqs=4)
    assert_clean(s)


def test_several_decode_steps_in_one_batch():
    """A batch of nothing but decodes, nobody waiting: up to decode_steps steps, bounded by
    max_tokens and by the free pages; commit takes that many tokens per request and stops a
    request at its stop token."""
    s = Scheduler(num_blocks=16, stop_token_ids=[7])
    s.add_request("a", toks(20), 9, ignore_eos=True)
    s.add_request("b", toks(30, 50), 30)
    first = s.schedule_step(2048, 8, decode_steps=4)
    assert first.decode_steps == 1                                     # prompts: one step
    s.commit(first, {"a": 1, "b": 1})
    batch = s.schedule_step(2048, 8, decode_steps=4)
    assert batch.decode_steps == 4 and [(w.start, w.end) for w in batch.work] == [(20, 21), (30, 31)]
    assert len(s.get_request("a").block_table) == 2 and len(s.get_request("b").block_table) == 3   # 24 and 34 positions
    res = s.commit(batch, {"a": [2, 3, 4, 5], "b": [2, 7, 8, 9]})      # b meets its stop token at the second step
    assert res.tokens == {"a": [2, 3, 4, 5], "b": [2, 7]} and res.finished == {"b": FinishReason.STOP}
    assert s.get_request("a").num_computed == 24 and s.get_request("a").output == [1, 2, 3, 4, 5]
    batch = s.schedule_step(2048, 8, decode_steps=8)
    assert batch.decode_steps == 4                                     # max_tokens 9, 5 made
    res = s.commit(batch, {"a": [6, 7, 8, 9]})                         # ignore_eos: 7 does not stop it
    assert res.finished == {"a": FinishReason.LENGTH} and not s.has_work()
    assert_clean(s)


def test_decode_steps_fall_back_to_one():
    s = Scheduler(num_blocks=4)                                        # 64 positions in all
    s.add_request("a", toks(30), 20, ignore_eos=True)
    s.add_request("b", toks(30, 40), 20, ignore_eos=True)
    step(s)
    batch = s.schedule_step(2048, 8, decode_steps=8)                   # 32 + 8 positions each: no pages for that
    assert batch.decode_steps == 1
    s.commit(batch, sample(batch))
    s.add_request("c", toks(5, 90), 4)
    batch = s.schedule_step(2048, 1, decode_steps=2)                   # somebody waits: one step at a time
    assert batch.decode_steps == 1 and s.stats().num_waiting == 1
    s.commit(batch, sample(batch))
    run_until_done(s)
    assert_clean(s)
