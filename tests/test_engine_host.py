"""Everything on the host side of a step, without a GPU: the kernel library is replaced by
its torch stand-in (tests/emulated_ops.py), the rest is the product's own code. Compared
with the plain implementation in every way of cutting the work."""

from __future__ import annotations

import numpy as np
import pytest
import torch

import traces
from checks import CacheWriteWatch
from configs import TINY, TOL_F32
from emulated_ops import EmulatedOps
from prefixserve_amd.engine.batch import EngineError, GroupMeta, StepItem, StepPacker
from prefixserve_amd.engine.engine import Engine, EngineConfig
from prefixserve_amd.engine.replay import TraceReplayer
from prefixserve_amd.engine.runner import ModelRunner
from prefixserve_amd.generation import LoopTimes, generate
from prefixserve_amd.sampling import request_key, uniform_for


def make_runner(model_dir, num_blocks=64, max_seq_len=512, **kw):
    return ModelRunner(model_dir, dtype="float32", device="cpu", num_blocks=num_blocks, max_seq_len=max_seq_len,
                       max_num_seqs=8, ops=EmulatedOps(), use_graphs=False, **kw)


def requests_for(name, lengths, seed=0):
    rng = np.random.default_rng(seed)
    return [rng.integers(0, TINY[name]["vocab_size"], n).tolist() for n in lengths]


@pytest.mark.parametrize("name", ["A", "B"])
def test_replay_in_every_cutting(name, model_dirs, plain_models):
    reqs = requests_for(name, [70, 33, 5, 97, 64, 18])
    truth = [plain_models[name].logits(t) for t in reqs]
    runner = make_runner(model_dirs[name])
    for build in (traces.whole, traces.decode_tail, traces.portions):
        steps, expect = build(reqs)
        traces.compare(TraceReplayer(runner).run_step, steps, expect, truth, TOL_F32)
    reqs = requests_for(name, [70, 33, 120, 97, 64, 18, 130, 45, 101, 77, 128, 90], seed=1)
    truth = [plain_models[name].logits(t) for t in reqs]
    steps, expect, peak = traces.mixed(reqs, seed=3)
    assert sum(len(r) for r in reqs) > 1.5 * peak                 # pages must be used again
    small = make_runner(model_dirs[name], num_blocks=peak // 16)
    small.pools.tensors[0].fill_(1e30)                            # stale pages hold junk, never zeros
    rp = TraceReplayer(small)
    traces.compare(rp.run_step, steps, expect, truth, TOL_F32)
    assert rp.cache.num_free(0) == peak // 16 and not rp.live


def test_replay_errors(model_dirs):
    rp = TraceReplayer(make_runner(model_dirs["A"], num_blocks=2))
    with pytest.raises(EngineError, match="out of pages"):
        rp.run_step({"step": 0, "entries": [{"id": "a", "tokens": list(range(40)), "want": []}], "end": []})
    with pytest.raises(EngineError, match="unknown request"):
        rp.run_step({"step": 1, "entries": [], "end": ["zz"]})
    with pytest.raises(EngineError, match="twice"):
        rp.run_step({"step": 2, "entries": [{"id": "b", "tokens": [1], "want": []}, {"id": "b", "tokens": [2], "want": []}], "end": []})


def test_packer_refuses_bad_batches():
    pk = StepPacker(torch.device("cpu"), [GroupMeta(8)], vocab_size=100, max_position=64, num_slots=2, prefill_tile=128)
    good = dict(key="a", tokens=[1, 2, 3], start=0, block_tables=[[0]], slot=0, want=[2])
    pk.pack([StepItem(**good)])
    for change, needle in [
        (dict(block_tables=[[8]]), "outside the pool"), (dict(block_tables=[[-1]]), "outside the pool"),
        (dict(block_tables=[[]]), "blocks in group"), (dict(block_tables=[[0], [0]]), "block tables"),
        (dict(tokens=[100], want=[0]), "token id"), (dict(tokens=[]), "no tokens"), (dict(start=62), "positions"),
        (dict(want=[3]), "wanted place"), (dict(slot=2), "state slot"), (dict(start=-1), "positions"),
    ]:
        with pytest.raises(EngineError, match=needle):
            pk.pack([StepItem(**{**good, **change})])
    with pytest.raises(EngineError, match="empty"):
        pk.pack([])


def test_packer_layout():
    pk = StepPacker(torch.device("cpu"), [GroupMeta(32)], vocab_size=200, max_position=256, num_slots=4, prefill_tile=128)
    items = [StepItem("a", list(range(20)), 30, [[5, 6, 7, 8]], slot=1, want=[19]),
             StepItem("b", [7], 16, [[9, 3]], slot=2, want=[0]),
             StepItem("c", list(range(130)), 0, [list(range(10, 19))], slot=0, want=[])]
    ctx = pk.pack(items)
    assert (ctx.num_tokens, ctx.num_items, ctx.num_logit_rows, ctx.num_decode, ctx.num_prefill_tiles) == (151, 3, 2, 1, 3)
    assert ctx.item_start.tolist() == [0, 20, 21, 151] and ctx.item_pos0.tolist() == [30, 16, 0]
    assert ctx.item_end.tolist() == [50, 17, 130] and ctx.slots.tolist() == [1, 2, 0]
    assert ctx.positions[:20].tolist() == list(range(30, 50)) and ctx.positions[20].item() == 16   # absolute
    assert ctx.logit_rows.tolist() == [19, 20] and ctx.dec_items.tolist() == [1]
    assert ctx.pf_tiles.tolist() == [[0, 0], [2, 0], [2, 128]]
    assert ctx.num_prefill_blocks == 2 and ctx.pf_blocks.tolist() == [0, 1]     # runs of up to four tiles, one item each
    small = StepPacker(torch.device("cpu"), [GroupMeta(32)], vocab_size=200, max_position=256, num_slots=4, prefill_tile=8)
    many = small.pack([StepItem("a", [1] * 70, 0, [list(range(5))], slot=0), StepItem("b", [1], 3, [[9]], slot=1),
                       StepItem("c", [1] * 33, 0, [list(range(10, 13))], slot=2), StepItem("d", [1] * 2, 40, [[20, 21, 22]], slot=3)])
    assert many.num_prefill_tiles == 9 + 5 + 1 and many.pf_blocks.tolist() == [0, 4, 8, 9, 13, 14]
    assert [many.pf_tiles[t].tolist() for t in many.pf_blocks.tolist()] == [[0, 0], [0, 32], [0, 64], [2, 0], [2, 32], [3, 0]]
    g = ctx.groups[0]
    assert g.table_off.tolist() == [0, 4, 6, 15] and g.block_ids[:6].tolist() == [5, 6, 7, 8, 9, 3]
    assert g.write_slot[0].item() == 6 * 16 + 14 and g.write_slot[2].item() == 7 * 16 + 0   # pos 30 -> page 1 (id 6)
    assert g.write_slot[20].item() == 3 * 16 + 0                                             # pos 16 -> second page
    st = pk.pack(items[:2], static_pages=6)                        # fixed-width tables for captured graphs
    assert st.groups[0].table_off.tolist() == [0, 6, 12] and st.groups[0].block_ids.numel() == 12


def test_uniform_numbers_match_the_plain_ones():
    from plain.llama_plain import uniform_for as plain_uniform

    for seed, key, idx in [(0, 0, 0), (3, 99, 5), (2 ** 63 + 5, request_key("req-7"), 41)]:
        assert uniform_for(seed, key, idx) == plain_uniform(seed, key, idx)
    assert request_key("a") != request_key("b") and request_key("a") == request_key("a")


@pytest.mark.parametrize("name", ["A", "B"])
def test_scheduler_driven_greedy_generation_equals_plain(name, model_dirs, plain_models):
    """Chunked prefill, a shared prefix, eviction and preemption (the pool is small) must not
    change a single token."""
    vocab = TINY[name]["vocab_size"]
    rng = np.random.default_rng(4)
    shared = rng.integers(3, vocab, 37).tolist()
    prompts = [shared + rng.integers(3, vocab, n).tolist() for n in (9, 21, 40)] + [rng.integers(3, vocab, 5).tolist()]
    new = 10
    eng = Engine(EngineConfig(model_path=model_dirs[name], dtype="float32", device="cpu", max_num_seqs=4,
                              max_prefill_tokens=24, max_seq_len=256, num_blocks=11, use_graphs=False), ops=EmulatedOps())
    eng.capture_logits = True
    times = LoopTimes()
    sched = eng.make_scheduler(chunk_size=24)
    watch = CacheWriteWatch(eng, sched)
    outs, stats = generate(eng, prompts, new, ignore_eos=True, times=times, scheduler=sched)
    assert watch.writes >= sum(len(p) for p in prompts) - stats.cached_prompt_tokens
    for p, o in zip(prompts, outs):
        want, _ = plain_models[name].greedy(p, new)
        assert o.tokens == want, f"prompt of {len(p)}: {o.tokens} != {want}"
    assert stats.preemptions > 0 and stats.cached_prompt_tokens > 0
    assert times.steps >= new and min(times.schedule_s, times.engine_s, times.commit_s) > 0
    assert 0 < times.scheduler_overhead < 1
    sched_cache = eng.make_cache()
    assert sched_cache.num_free(0) == 11


def test_temperature_sampling_is_reproducible_across_batching(model_dirs):
    eng = Engine(EngineConfig(model_path=model_dirs["B"], dtype="float32", device="cpu", max_num_seqs=4,
                              max_prefill_tokens=64, max_seq_len=256, num_blocks=64, use_graphs=False, sample_seed=5),
                 ops=EmulatedOps())
    rng = np.random.default_rng(8)
    prompts = [rng.integers(3, 512, n).tolist() for n in (12, 30, 7)]
    a, _ = generate(eng, prompts, 8, temperature=0.8, ignore_eos=True)
    b, _ = generate(eng, prompts, 8, temperature=0.8, ignore_eos=True, max_running_requests=1, max_prefill_tokens=5)
    assert [o.tokens for o in a] == [o.tokens for o in b]          # same draws whatever the batching
    c, _ = generate(eng, prompts, 8, temperature=0.8, seed=1, ignore_eos=True)
    assert [o.tokens for o in a] != [o.tokens for o in c]
    g, _ = generate(eng, prompts, 8, temperature=0.0, ignore_eos=True)
    assert [o.tokens for o in g] != [o.tokens for o in a]


def test_stop_token_ends_generation(model_dirs, plain_models):
    prompt = np.random.default_rng(2).integers(3, 256, 20).tolist()
    want, _ = plain_models["A"].greedy(prompt, 6)
    eng = Engine(EngineConfig(model_path=model_dirs["A"], dtype="float32", device="cpu", max_num_seqs=2,
                              max_seq_len=128, num_blocks=16, use_graphs=False), ops=EmulatedOps())
    sched = eng.make_scheduler()
    sched.stop_token_ids = frozenset({want[3]})
    outs, _ = generate(eng, [prompt], 6, scheduler=sched)
    stop_at = want.index(want[3])
    assert outs[0].tokens == want[:stop_at + 1] and outs[0].finish_reason.value == "stop"
    assert eng.stop_token_ids == {2}                               # from config.json's eos_token_id


def test_engine_refuses_without_kernels_on_cpu(model_dirs):
    from prefixserve_amd.kernels.ops import KernelError

    with pytest.raises(KernelError, match="GPU only"):
        ModelRunner(model_dirs["A"], dtype="float32", device="cpu", num_blocks=4, max_seq_len=64)


@pytest.mark.parametrize("temperature", [0.0, 0.8])
def test_several_decode_steps_give_the_same_tokens(temperature, model_dirs, plain_models):
    """Running four decode steps before the host reads the tokens changes no token, greedy or
    sampled: each step's token reaches the next on the device, the draws depend only on
    (seed, request, output index). A stop token inside the four ends the request there."""
    eng = Engine(EngineConfig(model_path=model_dirs["A"], dtype="float32", device="cpu", max_num_seqs=4,
                              max_prefill_tokens=64, max_seq_len=128, num_blocks=32, use_graphs=False, sample_seed=2),
                 ops=EmulatedOps())
    rng = np.random.default_rng(11)
    prompts = [rng.integers(3, 256, n).tolist() for n in (12, 30, 7)]
    one, _ = generate(eng, prompts, 11, temperature=temperature, ignore_eos=True)
    four, _ = generate(eng, prompts, 11, temperature=temperature, ignore_eos=True, decode_steps=4)
    assert [o.tokens for o in one] == [o.tokens for o in four]
    if temperature == 0.0:
        assert one[0].tokens == plain_models["A"].greedy(prompts[0], 11)[0]
        sched = eng.make_scheduler()
        sched.stop_token_ids = frozenset({one[1].tokens[5]})
        stopped, _ = generate(eng, prompts, 11, scheduler=sched, decode_steps=4)
        for o, full in zip(stopped, one):
            cut = next((i for i, t in enumerate(full.tokens) if t in sched.stop_token_ids), None)
            assert o.tokens == (full.tokens if cut is None else full.tokens[:cut + 1])
    assert eng.make_cache().num_free(0) == 32


def test_a_request_id_that_comes_back_gets_its_own_block_tables(model_dirs, plain_models):
    """Runs on one engine and one scheduler reuse the ids req-0, req-1, ...: the second run's
    requests are longer and get other pages than the first run's, whose prompts stay in the
    prefix cache. Were anything of the first run's tables to survive in the engine, the second
    run would write into those cached pages, and the third run, which finds the first prompt
    in the cache again, would read them."""
    eng = Engine(EngineConfig(model_path=model_dirs["A"], dtype="float32", device="cpu", max_num_seqs=4,
                              max_prefill_tokens=64, max_seq_len=256, num_blocks=40, use_graphs=False), ops=EmulatedOps())
    rng = np.random.default_rng(31)
    sched = eng.make_scheduler()
    first = [rng.integers(3, 256, n).tolist() for n in (40, 20)]
    generate(eng, first, 6, ignore_eos=True, scheduler=sched)
    second = [rng.integers(3, 256, n).tolist() for n in (90, 70, 33)]
    outs, _ = generate(eng, second, 9, ignore_eos=True, scheduler=sched)
    for p, o in zip(second, outs):
        assert o.tokens == plain_models["A"].greedy(p, 9)[0]
    again, stats = generate(eng, first, 6, ignore_eos=True, scheduler=sched)
    assert again[0].cached_tokens >= 32                                     # the first prompt came from the cache
    for p, o in zip(first, again):
        assert o.tokens == plain_models["A"].greedy(p, 6)[0]


# ------------------------------------------------------------- a mixer that keeps state

def test_a_state_keeping_mixer_through_the_scheduler(tmp_path):
    """The toy running-mean mixer (state in slots, no pages) through the engine and the
    scheduler with a shared prefix and a pool so small that requests are sent back: a prefix
    hit would start a request behind tokens its state never saw, so the cache manager keeps
    the prefix cache off for such a model, and a request that comes back starts from
    position 0 with a fresh state. Every token equals the model's own whole-sequence choice."""
    from toy_parts import write_toy_mean_model

    write_toy_mean_model(tmp_path)
    rng = np.random.default_rng(3)
    shared = rng.integers(0, 100, 40).tolist()
    prompts = [shared + rng.integers(0, 100, n).tolist() for n in (9, 30, 17)] + [shared[:33]]
    new = 12
    eng = Engine(EngineConfig(model_path=tmp_path, dtype="float32", device="cpu", max_num_seqs=4,
                              max_prefill_tokens=24, max_seq_len=256, num_blocks=12, use_graphs=False), ops=EmulatedOps())
    assert eng.runner.state_bytes_per_slot > 0
    sched = eng.make_scheduler(chunk_size=24)
    assert sched.cache.prefix_cache is False and sched.tree is None
    outs, stats = generate(eng, prompts, new, ignore_eos=True, scheduler=sched)
    assert stats.preemptions > 0 and stats.cached_prompt_tokens == 0
    assert sched.cache.num_free(0) == 12 and sched.cache.slots.num_free == 4
    roomy = make_runner(tmp_path, num_blocks=64)
    for i, (p, o) in enumerate(zip(prompts, outs)):
        seq = p + o.tokens
        rows = TraceReplayer(roomy).run_step(
            {"step": i, "entries": [{"id": "w", "tokens": seq[:-1], "want": list(range(len(p) - 1, len(seq) - 1))}],
             "end": ["w"]})
        assert np.argmax(rows, -1).tolist() == o.tokens, f"request {i}"


def test_a_state_slot_is_cleared_by_the_runner_not_by_the_mixer(tmp_path):
    """The toy mixer never resets its state. Every slot is filled with junk, as a slot's last
    owner leaves it; a request that starts at position 0 must still give its whole-sequence
    logits, first in a fresh slot and then in the slot another request has just given back."""
    from toy_parts import write_toy_mean_model

    runner = make_runner(write_toy_mean_model(tmp_path), num_blocks=32, max_seq_len=128)
    rng = np.random.default_rng(6)
    a, b = rng.integers(0, 100, 40).tolist(), rng.integers(0, 100, 25).tolist()
    clean = TraceReplayer(make_runner(tmp_path, num_blocks=32, max_seq_len=128))
    want_a = clean.run_step({"step": 0, "entries": [{"id": "a", "tokens": a, "want": list(range(40))}], "end": ["a"]})
    want_b = TraceReplayer(make_runner(tmp_path, num_blocks=32, max_seq_len=128)).run_step(
        {"step": 0, "entries": [{"id": "b", "tokens": b, "want": list(range(25))}], "end": ["b"]})
    for state in runner.states.values():
        state.fill_(123.0)
    rp = TraceReplayer(runner)
    got_a = np.concatenate([
        rp.run_step({"step": 0, "entries": [{"id": "a", "tokens": a[:13], "want": list(range(13))}], "end": []}),
        rp.run_step({"step": 1, "entries": [{"id": "a", "tokens": a[13:], "want": list(range(27))}], "end": ["a"]})])
    slot_a = 0 if not rp.live else None
    got_b = rp.run_step({"step": 2, "entries": [{"id": "b", "tokens": b, "want": list(range(25))}], "end": ["b"]})
    assert slot_a == 0 and rp.cache.slots.num_free == 8
    assert np.abs(got_a - want_a).max() <= 1e-5 * np.abs(want_a).max()
    assert np.abs(got_b - want_b).max() <= 1e-5 * np.abs(want_b).max()
    # the slots nobody started in still hold the junk
    assert sum(float(s[-1].abs().max()) == 123.0 for s in runner.states.values()) == len(runner.states)


# ------------------------------------------------------------- faults switched on

class _GateUpSwapped(EmulatedOps):
    def linear_swiglu(self, x, w_gate_up, out) -> None:
        inter = w_gate_up.shape[0] // 2
        super().linear_swiglu(x, torch.cat([w_gate_up[inter:], w_gate_up[:inter]]), out)


class _KvHeadByRemainder(EmulatedOps):
    """Query head h reads kv head h % kv_heads instead of h // (heads / kv_heads)."""

    def expand_kv(self, x, rep):
        return x.repeat(1, rep, 1)


def _relative_positions(runner):
    """The reference's own switchable fault (prefixserve/llama_engine.py:192, ``rope_relative``):
    positions restart at 0 in every portion."""
    inner = runner.packer.pack

    def pack(items, **kw):
        ctx = inner(items, **kw)
        ctx.positions -= ctx.item_pos0[ctx.tok_item.long()]
        return ctx

    runner.packer.pack = pack


@pytest.mark.parametrize("fault", ["relative positions", "gate and up swapped", "kv head by remainder"])
def test_the_cuttings_catch_a_fault_that_is_switched_on(fault, model_dirs, plain_models):
    """What the replay comparisons are worth: each of three plausible faults, switched on in
    the host stand-in, must fail them (the reference checks its own tests the same way,
    tests/test_llama_exact.py:227-241). Positions that restart per portion are right for a
    whole prompt and wrong for every later portion, so only the cut replay sees them."""
    name = "A"                                              # 4 heads on 2 kv heads: the two head maps differ
    reqs = requests_for(name, [70, 33, 97])
    truth = [plain_models[name].logits(t) for t in reqs]
    ops = {"gate and up swapped": _GateUpSwapped, "kv head by remainder": _KvHeadByRemainder}.get(fault, EmulatedOps)()
    runner = ModelRunner(model_dirs[name], dtype="float32", device="cpu", num_blocks=64, max_seq_len=512,
                         max_num_seqs=8, ops=ops, use_graphs=False)
    if fault == "relative positions":
        _relative_positions(runner)
        steps, expect = traces.whole(reqs)
        traces.compare(TraceReplayer(runner).run_step, steps, expect, truth, TOL_F32)     # whole prompts: no difference
    steps, expect = traces.portions(reqs)
    with pytest.raises(AssertionError, match="relative error"):
        traces.compare(TraceReplayer(runner).run_step, steps, expect, truth, TOL_F32)


def test_the_scheduler_refuses_what_the_engine_cannot_address(model_dirs):
    eng = Engine(EngineConfig(model_path=model_dirs["A"], dtype="float32", device="cpu", max_num_seqs=2,
                              max_seq_len=64, num_blocks=32, use_graphs=False), ops=EmulatedOps())
    sched = eng.make_scheduler()
    from prefixserve_amd.engine.scheduler import AddResult

    assert sched.add_request("long", list(range(3, 60)), 8) is AddResult.TOO_LONG      # 57 + 8 > 64, the pool would do
    assert sched.add_request("fits", list(range(3, 59)), 8) is AddResult.ACCEPTED
    assert sched.stats().rejected == 1
