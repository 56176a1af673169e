"""The engine against the plain model at the layer sizes the benchmark runs, where the
kernels take the forms that tiny models never reach: products whose inner size is 2,048 to
14,336 (split over workgroups, partial sums added by the norm that follows), 192 and more
tiles of q/k/v columns, the grouped prefill attention at head sizes 64 and 128 with four
query heads per kv head, decode attention split over thousands of keys and merged, and the
output matrix over 128,256 columns. Fewer layers than the real models, the same layers
(the reference tests its attention at real head shapes, tests/gpu/test_flashinfer_vs_ref.py:48,60-67).
"""

from __future__ import annotations

import numpy as np
import pytest

import traces
from configs import TOL_BF16, TOL_F32
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
TOL = {"float32": TOL_F32, "bfloat16": TOL_BF16}


@pytest.fixture(scope="module", params=list(SIZES))
def sized(request, tmp_path_factory):
    """(name, model folder, plain model in float64 / float32 for the larger one, its bfloat16 yardstick)."""
    from plain.llama_plain import PlainLlama
    from prefixserve_amd.weights import write_random_model

    name = request.param
    d = tmp_path_factory.mktemp(f"size-{name}")
    # 0.02 as in real checkpoints: with the tests' usual 0.1 the logits of 2,048 to 4,096 wide
    # layers would be in the thousands.
    write_random_model(d, SIZES[name], seed=40 + len(name), std=0.02)
    print(f"[{name}] model written", flush=True)
    plain = PlainLlama(d, dtype=np.float64 if name == "1b" else np.float32)
    toks = np.random.default_rng(5).integers(0, SIZES[name]["vocab_size"], 96).tolist()
    truth = plain.logits(toks)
    rough = PlainLlama(d, bf16=True, weights=plain.w).logits(toks)
    yardstick = float(np.mean(np.abs(rough - truth).max(-1) / np.abs(truth).max(-1)))
    print(f"[{name}] plain model ready, bfloat16 yardstick {yardstick:.3e}", flush=True)
    return name, d, plain, yardstick


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cutting_at_the_benchmarked_layer_sizes(dtype, sized):
    name, model_dir, plain, yardstick = sized
    rng = np.random.default_rng(8)
    reqs = [rng.integers(0, SIZES[name]["vocab_size"], n).tolist() for n in (70, 33, 120, 97)]
    truth = [plain.logits(t) for t in reqs]
    runner = ModelRunner(model_dir, dtype=dtype, device="cuda:0", num_blocks=64, max_seq_len=256, max_num_seqs=8,
                         use_graphs=True)
    worst, errors = {}, []
    for build in (traces.whole, traces.decode_tail, traces.portions):
        steps, expect = build(reqs)
        worst[build.__name__] = traces.compare(TraceReplayer(runner).run_step, steps, expect, truth, TOL[dtype], errors)
    steps, expect, peak = traces.mixed(reqs, seed=3)
    runner.pools.tensors[0].fill_(1e30)
    worst["mixed"] = traces.compare(TraceReplayer(runner).run_step, steps, expect, truth, TOL[dtype], errors)
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
    name, model_dir, plain, yardstick = sized
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
    assert max(errors) < (2e-5 if dtype == "float32" else TOL_BF16)
    if dtype == "bfloat16":
        assert np.mean(errors) <= yardstick


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_short_portion_behind_a_long_prefix_at_the_benchmarked_layer_sizes(dtype, sized):
    """The tail of a long prompt as a portion of its own, beside a short fresh prompt: seven query
    tiles on 2,250 keys, which the bfloat16 attention deals out to four workgroups per tile and
    merges (the fresh prompt's tiles leave all runs but the first empty)."""
    name, model_dir, plain, yardstick = sized
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
    assert max(errors) < (2e-5 if dtype == "float32" else TOL_BF16)
    if dtype == "bfloat16":
        assert np.mean(errors) <= yardstick
