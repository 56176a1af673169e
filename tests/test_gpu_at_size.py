"""The engine against the plain model at the layer sizes the benchmark runs, where the
kernels take the forms that tiny models never reach: products whose inner size is 2,048 to
14,336 (split over workgroups, partial sums added by the norm that follows), 192 and more
tiles of q/k/v columns, the grouped prefill attention at head sizes 64 and 128 with four
query heads per kv head, decode attention split over thousands of keys and merged, and the
output matrix over 128,256 columns. Fewer layers than the real models, the same layers
(the reference tests its attention at real head shapes, tests/gpu/test_flashinfer_vs_ref.py:48,60-67).
And long prompts through two small models with one and with two query heads per kv head, whose
prefill attention takes several tiles of queries per workgroup.
"""

from __future__ import annotations

import numpy as np
import pytest

import traces
from checks import logit_errors, plain_bf16_bars
from configs import TOL_F32
from prefixserve_amd.engine.replay import TraceReplayer
from prefixserve_amd.engine.runner import ModelRunner

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(600)]   # the plain model at these sizes takes its time

LLAMA3 = dict(rope_type="llama3", low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192)

SIZES = {
    # two layers of the 1B shape, its vocabulary and tied output matrix
    "1b": dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=128256, hidden_size=2048,
               intermediate_size=8192, num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
               rms_norm_eps=1e-5, rope_theta=500000.0, rope_scaling=dict(LLAMA3, factor=32.0),
               max_position_embeddings=131072, tie_word_embeddings=True),
    # one layer of the 8B shape; the vocabulary is cut to a quarter (it is no layer size, and
    # two untied matrices of 128,256 x 4,096 would be most of the test's time)
    "8b": dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=32064, hidden_size=4096,
               intermediate_size=14336, num_hidden_layers=1, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
               rms_norm_eps=1e-5, rope_theta=500000.0, rope_scaling=dict(LLAMA3, factor=8.0),
               max_position_embeddings=131072, tie_word_embeddings=False),
}


@pytest.fixture(scope="module", params=list(SIZES))
def sized(request, tmp_path_factory):
    """(name, model folder, plain model in float64 / float32 for the larger one, the mean row error
    of a plain bfloat16 run of it, the bar for a single bfloat16 row: 1.5 x that run's worst row)."""
    from plain.llama_plain import PlainLlama
    from prefixserve_amd.weights import write_random_model

    name = request.param
    d = tmp_path_factory.mktemp(f"size-{name}")
    # 0.02 as in real checkpoints: with the tests' usual 0.1 the logits of 2,048 to 4,096 wide
    # layers would be in the thousands.
    write_random_model(d, SIZES[name], seed=40 + len(name), std=0.02)
    print(f"[{name}] model written", flush=True)
    plain = PlainLlama(d, dtype=np.float64 if name == "1b" else np.float32)
    rng = np.random.default_rng(5)
    yardstick, row_bar = plain_bf16_bars(d, plain, [rng.integers(0, SIZES[name]["vocab_size"], 96).tolist() for _ in range(3)])
    print(f"[{name}] plain model ready, plain bfloat16: mean {yardstick:.3e}, bar for a row {row_bar:.3e}", flush=True)
    return name, d, plain, yardstick, row_bar


def tol(dtype, row_bar):
    return TOL_F32 if dtype == "float32" else row_bar


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cutting_at_the_benchmarked_layer_sizes(dtype, sized):
    name, model_dir, plain, yardstick, row_bar = sized
    rng = np.random.default_rng(8)
    reqs = [rng.integers(0, SIZES[name]["vocab_size"], n).tolist() for n in (70, 33, 120, 97, 64, 18, 101, 45)]
    truth = [plain.logits(t) for t in reqs]
    runner = ModelRunner(model_dir, dtype=dtype, device="cuda:0", num_blocks=64, max_seq_len=256, max_num_seqs=8,
                         use_graphs=True)
    worst, errors = {}, []
    for build in (traces.whole, traces.decode_tail, traces.portions):
        steps, expect = build(reqs[:4])
        worst[build.__name__] = traces.compare(TraceReplayer(runner).run_step, steps, expect, truth, tol(dtype, row_bar), errors)
    # Mixed, in a pool of exactly the pages the live requests hold at their peak: pages are used again.
    steps, expect, peak = traces.mixed(reqs, max_live=3, seed=3)
    assert sum(len(r) for r in reqs) > 1.5 * peak
    del runner
    small = ModelRunner(model_dir, dtype=dtype, device="cuda:0", num_blocks=peak // 16, max_seq_len=256, max_num_seqs=8,
                        use_graphs=True)
    small.pools.tensors[0].fill_(1e30)
    rp = TraceReplayer(small)
    worst["mixed"] = traces.compare(rp.run_step, steps, expect, truth, tol(dtype, row_bar), errors)
    assert rp.cache.num_free(0) == peak // 16
    print(name, dtype, {k: f"{v:.2e}" for k, v in worst.items()}, f"mean {np.mean(errors):.2e} (plain bf16 {yardstick:.2e})",
          flush=True)
    if dtype == "float32":
        assert max(worst.values()) < 2e-5
    else:
        assert np.mean(errors) <= yardstick, f"{np.mean(errors):.3e} > {yardstick:.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_behind_long_prompts_at_the_benchmarked_layer_sizes(dtype, sized):
    """The benchmark's own schedule in small: prompts of more than 2,048 tokens in one step
    each (the prefill kernels over 65 and more query tiles), then decode steps of the
    requests together through captured graphs (keys split over workgroups and merged)."""
    name, model_dir, plain, yardstick, row_bar = sized
    rng = np.random.default_rng(9)
    lengths, new = (2100, 2063, 517, 40, 33), 6        # five requests: the products' forms for 4 to 16 tokens
    seqs = [rng.integers(0, SIZES[name]["vocab_size"], n + new).tolist() for n in lengths]
    runner = ModelRunner(model_dir, dtype=dtype, device="cuda:0", num_blocks=3 * 136, max_seq_len=2176, max_num_seqs=8,
                         use_graphs=True)
    rp = TraceReplayer(runner)
    truth = [plain.logits_at(s, range(n - 1, n + new)) for s, n in zip(seqs, lengths)]
    errors = []
    for i, (s, n) in enumerate(zip(seqs, lengths)):
        got = rp.run_step({"step": i, "entries": [{"id": f"r{i}", "tokens": s[:n], "want": [n - 1]}], "end": []})
        errors.append(float(np.abs(got[0] - truth[i][0]).max() / np.abs(truth[i][0]).max()))
    for k in range(new):
        entries = [{"id": f"r{i}", "tokens": [s[n + k]], "want": [0]} for i, (s, n) in enumerate(zip(seqs, lengths))]
        got = rp.run_step({"step": 10 + k, "entries": entries, "end": []})
        for i in range(len(seqs)):
            want = truth[i][1 + k]
            errors.append(float(np.abs(got[i] - want).max() / np.abs(want).max()))
    if runner.use_graphs:
        assert (5, 5, False) in runner._graphs
    print(name, dtype, f"worst {max(errors):.2e} mean {np.mean(errors):.2e} (plain bf16 {yardstick:.2e})", flush=True)
    assert max(errors) < (2e-5 if dtype == "float32" else row_bar)
    if dtype == "bfloat16":
        assert np.mean(errors) <= yardstick


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_short_portion_behind_a_long_prefix_at_the_benchmarked_layer_sizes(dtype, sized):
    """The tail of a long prompt as a portion of its own, beside a short fresh prompt: seven query
    tiles on 2,250 keys, which the bfloat16 attention deals out to four workgroups per tile and
    merges (the fresh prompt's tiles leave all runs but the first empty)."""
    name, model_dir, plain, yardstick, row_bar = sized
    rng = np.random.default_rng(10)
    vocab = SIZES[name]["vocab_size"]
    long, short = rng.integers(0, vocab, 2250).tolist(), rng.integers(0, vocab, 40).tolist()
    places = [0, 31, 32, 100, 149]
    truth = list(plain.logits_at(long, [2100 + p for p in places])) + [plain.logits_at(short, [39])[0]]
    runner = ModelRunner(model_dir, dtype=dtype, device="cuda:0", num_blocks=160, max_seq_len=2304, max_num_seqs=4)
    rp = TraceReplayer(runner)
    assert rp.run_step({"step": 0, "entries": [{"id": "a", "tokens": long[:2100], "want": []}], "end": []}) is None
    got = rp.run_step({"step": 1, "entries": [{"id": "a", "tokens": long[2100:], "want": places},
                                              {"id": "b", "tokens": short, "want": [39]}], "end": ["a", "b"]})
    errors = [float(np.abs(g - w).max() / np.abs(w).max()) for g, w in zip(got, truth)]
    print(name, dtype, f"worst {max(errors):.2e} mean {np.mean(errors):.2e} (plain bf16 {yardstick:.2e})", flush=True)
    assert max(errors) < (2e-5 if dtype == "float32" else row_bar)
    if dtype == "bfloat16":
        assert np.mean(errors) <= yardstick


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_forty_one_requests_decode_together_at_the_benchmarked_layer_sizes(dtype, sized):
    """What decoding at batch 64 rests on: 41 requests in one step take the small-step products'
    forms for four token tiles (33 to 64 tokens), q/k/v + rotation + cache write included, at
    inner sizes of 2,048 to 14,336, and the decode attention over 41 block tables of which one
    is 2,100 tokens long, through a captured graph. Judged by the logits of every step."""
    name, model_dir, plain, yardstick, row_bar = sized
    rng = np.random.default_rng(11)
    vocab = SIZES[name]["vocab_size"]
    lengths, new = [2100] + [8 + (7 * i) % 40 for i in range(40)], 4
    seqs = [rng.integers(0, vocab, n + new).tolist() for n in lengths]
    blocks = sum(-(-(n + new) // 16) for n in lengths) + 4
    runner = ModelRunner(model_dir, dtype=dtype, device="cuda:0", num_blocks=blocks, max_seq_len=2176, max_num_seqs=48,
                         use_graphs=True)
    runner.pools.tensors[0].fill_(1e30)
    rp = TraceReplayer(runner)
    truth = [plain.logits_at(s, range(n, n + new)) for s, n in zip(seqs, lengths)]
    rp.run_step({"step": 0, "entries": [{"id": "r0", "tokens": seqs[0][:2100], "want": []}], "end": []})
    for at in range(1, 41, 8):      # the short prompts eight at a time
        rp.run_step({"step": at, "entries": [{"id": f"r{i}", "tokens": seqs[i][:lengths[i]], "want": []}
                                             for i in range(at, at + 8)], "end": []})
    errors = []
    for k in range(new):
        entries = [{"id": f"r{i}", "tokens": [s[n + k]], "want": [0]} for i, (s, n) in enumerate(zip(seqs, lengths))]
        got = rp.run_step({"step": 100 + k, "entries": entries, "end": []})
        for i in range(41):
            want = truth[i][k]
            errors.append(float(np.abs(got[i] - want).max() / np.abs(want).max()))
    assert (41, 41, False) in runner._graphs
    print(name, dtype, f"worst {max(errors):.2e} mean {np.mean(errors):.2e} (plain bf16 {yardstick:.2e})", flush=True)
    assert max(errors) < (2e-5 if dtype == "float32" else row_bar)
    if dtype == "bfloat16":
        assert np.mean(errors) <= yardstick


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_scheduler_at_the_benchmarked_layer_sizes(dtype, sized):
    """The engine as it is served, at real layer sizes: four prompts that share their first 512
    tokens, portions of 256, a pool of 70 pages (one request is sent back and recomputed, the
    shared prefix comes from the cache), warm_up() and eight decode steps per round through
    graphs with the sampled token fed on the device. Judged by the logits of every row the
    engine sampled from, given its own tokens."""
    from prefixserve_amd import Engine, EngineConfig, generate
    from checks import CacheWriteWatch

    name, model_dir, plain, yardstick, row_bar = sized
    rng = np.random.default_rng(14)
    vocab = SIZES[name]["vocab_size"]
    shared = rng.integers(3, vocab, 512).tolist()
    prompts = [shared + rng.integers(3, vocab, n).tolist() for n in (100, 300, 200, 50)]
    new = 24
    eng = Engine(EngineConfig(model_path=model_dir, dtype=dtype, max_num_seqs=4, max_prefill_tokens=256, max_seq_len=1024,
                              num_blocks=70, decode_steps=8))
    eng.warm_up()
    captured = set(eng.runner._graphs)
    eng.runner.pools.tensors[0].fill_(1e30)
    eng.logit_trace = []
    sched = eng.make_scheduler(chunk_size=256)
    watch = CacheWriteWatch(eng, sched)
    outs, stats = generate(eng, prompts, new, ignore_eos=True, scheduler=sched)
    assert stats.preemptions > 0 and stats.cached_prompt_tokens >= 512 and watch.writes > 0
    assert all(len(o.tokens) == new for o in outs) and set(eng.runner._graphs) == captured
    assert sched.cache.num_free(0) + sched.stats().cached_blocks == 70
    errors = logit_errors(eng.logit_trace, prompts, outs, plain, traced_rows_only=True)
    assert len(errors) >= 4 * new
    print(name, dtype, f"worst {max(errors):.2e} mean {np.mean(errors):.2e} (plain bf16 {yardstick:.2e}), "
          f"{stats.preemptions} sent back, {stats.cached_prompt_tokens} tokens from the cache", flush=True)
    assert max(errors) < (2e-5 if dtype == "float32" else row_bar)
    if dtype == "bfloat16":
        assert np.mean(errors) <= yardstick


def test_the_pool_sized_from_free_memory_leaves_room_for_the_largest_step(sized):
    """No ``num_blocks``: the runner runs the largest step a scheduler can ask for (a portion of
    512 tokens beside 63 decoding requests, 64 rows of logits) once on a throwaway pool and
    gives the pages what the device then reports free, less the reserve of 1 GiB
    (prefixserve/llama_engine.py:231-267,304-320). With the pool allocated, warm_up() (that step
    again, then a graph capture per batch size) and the same step once more must run, and at
    least half of the reserve must still be free afterwards: an estimate that forgot a buffer
    would have given its bytes to the pages. The last pages of a pool of hundreds of gigabytes
    are used like the first: their byte offsets do not fit 32 bits."""
    import gc

    import torch

    from prefixserve_amd import Engine, EngineConfig

    name, model_dir, plain, yardstick, row_bar = sized
    if name != "1b":
        pytest.skip("one shape is enough for this")
    reserve = 1 << 30
    gc.collect()
    torch.cuda.empty_cache()
    eng = runner = None
    eng = Engine(EngineConfig(model_path=model_dir, dtype="bfloat16", max_num_seqs=64, max_prefill_tokens=512,
                              max_seq_len=4096))
    try:
        runner = eng.runner
        free_after_pool = torch.cuda.mem_get_info("cuda:0")[0]
        assert runner.pools.nbytes() > 100e9, "most of the device's memory goes to pages"
        print(f"free with the pool allocated: {free_after_pool / 1e6:.0f} MB", flush=True)
        # (what the device reports free does not fall by exactly the bytes asked for at this size)
        assert reserve // 2 <= free_after_pool <= 2 * reserve
        eng.warm_up()
        assert len(runner._graphs) == len(eng._batch_sizes())
        assert runner.step(runner.largest_step()).shape == (64, SIZES[name]["vocab_size"])
        torch.cuda.synchronize()
        free = torch.cuda.mem_get_info("cuda:0")[0]
        print(f"pool {runner.pools.nbytes() / 1e9:.1f} GB in {runner.num_blocks} pages, free after warm-up {free / 1e6:.0f} MB", flush=True)
        assert free >= reserve // 2
        # the same prompt through the first and through the last pages of the pool
        toks = np.random.default_rng(2).integers(0, SIZES[name]["vocab_size"], 200).tolist()
        truth = plain.logits_at(toks, [199])[0]
        rows = []
        for first_page in (0, runner.num_blocks - 13):
            rp = TraceReplayer(runner)
            table = list(range(first_page, first_page + 13))
            rp.cache.allocate = lambda need, table=table: [list(table[:n]) for n in need]      # these pages, not the next free ones
            rp.cache.release = lambda tables: None
            got = rp.run_step({"step": 0, "entries": [{"id": "a", "tokens": toks, "want": [199]}], "end": ["a"]})
            rows.append(got[0])
            assert float(np.abs(got[0] - truth).max() / np.abs(truth).max()) < row_bar
        assert np.array_equal(rows[0], rows[1])
    finally:
        del eng, runner
        gc.collect()
        torch.cuda.empty_cache()


FEW_HEADS_PER_KV = {
    # one query head per kv head at head size 64, two at head size 128: long prompts then go to the
    # form of the prefill attention in which a workgroup takes four or two consecutive tiles of queries
    "one": dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=2000, hidden_size=512,
                intermediate_size=1024, num_hidden_layers=2, num_attention_heads=16, num_key_value_heads=16, head_dim=64,
                rms_norm_eps=1e-5, rope_theta=10000.0, max_position_embeddings=4096, tie_word_embeddings=True),
    "two": dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=1500, hidden_size=384,
                intermediate_size=800, num_hidden_layers=2, num_attention_heads=12, num_key_value_heads=6, head_dim=128,
                rms_norm_eps=1e-6, rope_theta=500000.0, rope_scaling=dict(LLAMA3, factor=8.0, original_max_position_embeddings=512),
                max_position_embeddings=4096, tie_word_embeddings=False),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads", list(FEW_HEADS_PER_KV))
def test_long_prompts_with_one_or_two_query_heads_per_kv_head(dtype, heads, tmp_path):
    """Two prompts of 1,500 and 1,107 tokens in one step (47 + 35 tiles of queries: runs of four
    tiles, the last of each prompt shorter, the second prompt's last tile of 19 queries), a third
    in portions on top of what it cached, then all of them decoding together; logits at places
    all over the prompts against the plain model."""
    from plain.llama_plain import PlainLlama
    from prefixserve_amd.weights import write_random_model

    cfg = FEW_HEADS_PER_KV[heads]
    write_random_model(tmp_path, cfg, seed=7, std=0.05)
    plain = PlainLlama(tmp_path)
    rng = np.random.default_rng(12)
    yardstick, row_bar = plain_bf16_bars(tmp_path, plain, [rng.integers(0, cfg["vocab_size"], 130).tolist() for _ in range(3)])
    lengths, new = (1500, 1107, 1300), 4
    seqs = [rng.integers(0, cfg["vocab_size"], n + new).tolist() for n in lengths]
    places = [[0, 31, 32, 127, 128, 129, 700, 1471, 1472, 1499], [5, 1087, 1088, 1106], [1299]]
    truth = [plain.logits_at(s, list(p) + list(range(n, n + new))) for s, n, p in zip(seqs, lengths, places)]
    runner = ModelRunner(tmp_path, dtype=dtype, device="cuda:0", num_blocks=260, max_seq_len=1536, max_num_seqs=4, use_graphs=True)
    rp = TraceReplayer(runner)
    errors = []

    def judge(got, want):
        errors.extend((np.abs(got - want).max(-1) / np.abs(want).max(-1)).tolist())

    got = rp.run_step({"step": 0, "entries": [{"id": "r0", "tokens": seqs[0][:1500], "want": places[0]},
                                              {"id": "r1", "tokens": seqs[1][:1107], "want": places[1]}], "end": []})
    judge(got, np.concatenate([truth[0][:len(places[0])], truth[1][:len(places[1])]]))
    for k, (a, b) in enumerate(((0, 600), (600, 1150), (1150, 1300))):
        got = rp.run_step({"step": 1 + k, "entries": [{"id": "r2", "tokens": seqs[2][a:b], "want": [b - a - 1] if b == 1300 else []}], "end": []})
    judge(got, truth[2][:1])
    for k in range(new):
        entries = [{"id": f"r{i}", "tokens": [s[n + k]], "want": [0]} for i, (s, n) in enumerate(zip(seqs, lengths))]
        got = rp.run_step({"step": 10 + k, "entries": entries, "end": []})
        judge(got, np.stack([truth[i][len(places[i]) + k] for i in range(3)]))
    print(heads, dtype, f"worst {max(errors):.2e} mean {np.mean(errors):.2e} (plain bf16 {yardstick:.2e}, bar for a row {row_bar:.2e})", flush=True)
    assert max(errors) < (2e-5 if dtype == "float32" else row_bar)
    if dtype == "bfloat16":
        assert np.mean(errors) <= yardstick
