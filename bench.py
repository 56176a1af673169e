#!/usr/bin/env python3
"""Headline benchmark: Llama 3.2 1B shape, random bfloat16 weights, 4,096-token context.

  python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the scheduler-driven engine (schedule, run, sample, commit)
at batch 8 over 2,048-token prompts. Prints ONE JSON line: decoded tokens per second as
``value``, the 2,048-token prefill under ``prefill``, the decode step's HBM roofline under
``roofline`` and batch 1 / batch 64 decoding under ``points``. Synthetic data: seeded
uniform-random token ids and seeded random weights; nothing is downloaded.
"""

from __future__ import annotations

import argparse
import gc
import json
import sys
import tempfile
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

# MI355X published peaks.
HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}

LLAMA_1B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 128256, "hidden_size": 2048,
    "intermediate_size": 8192, "num_hidden_layers": 16, "num_attention_heads": 32, "num_key_value_heads": 8,
    "head_dim": 64, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
    "max_position_embeddings": 131072, "tie_word_embeddings": True,
}


def _llama3(hidden, inter, layers, heads, kv, dim, factor, tied):
    cfg = dict(LLAMA_1B)
    cfg.update(hidden_size=hidden, intermediate_size=inter, num_hidden_layers=layers, num_attention_heads=heads,
               num_key_value_heads=kv, head_dim=dim, tie_word_embeddings=tied,
               rope_scaling=dict(LLAMA_1B["rope_scaling"], factor=factor))
    return cfg


# The default is the 1B shape; the larger ones show the kernels at another head size and width and with other head counts.
SHAPES = {
    "llama-3.2-1b": LLAMA_1B,
    "llama-3.2-3b": _llama3(3072, 8192, 28, 24, 8, 128, 32.0, True),
    "llama-3.1-8b": _llama3(4096, 14336, 32, 32, 8, 128, 8.0, False),
    # every query head with keys and values of its own, a vocabulary of 32,000, no rope scaling
    "llama-2-7b": {**_llama3(4096, 11008, 32, 32, 32, 128, 1.0, False), "vocab_size": 32000, "rope_theta": 10000.0,
                   "rope_scaling": None},
}


def prefill_flops(cfg: dict, layers: int, tokens: int) -> float:
    h, i, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    hq, hkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    per_token_layer = 2 * h * (hq + 2 * hkv) * d + 2 * hq * d * h + 2 * h * 2 * i + 2 * i * h
    attention = 2 * 2 * (tokens * (tokens + 1) / 2) * hq * d          # causal QK^T and PV
    return layers * (tokens * per_token_layer + attention) + 2 * h * v  # one row through the output matrix


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / batch 64 points")
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--decode-steps", type=int, default=8,
                    help="decode steps per scheduler round (the host reads the tokens once per round)")
    ap.add_argument("--prefill-reps", type=int, default=5, help="timed repetitions of the 2,048-token prefill")
    ap.add_argument("--repeats", type=int, default=3,
                    help="how often the timed region of K steps is run; the line reports the median repeat")
    ap.add_argument("--long-context", type=int, default=16384,
                    help="context of the extra decode point (0: skip it); its prompts fill all but 2,048 tokens of it")
    ap.add_argument("--longer-context", type=int, default=65536, help="context of a second extra decode point (0: skip it)")
    ap.add_argument("--skewed-context", type=int, default=30000,
                    help="extra point: 32 requests decode together, one behind this many tokens, the others behind 200 (0: skip it)")
    ap.add_argument("--other-shape", choices=sorted(SHAPES) + ["none"], default="llama-3.1-8b",
                    help="extra point: some layers of this shape decoding at batch 32 in an 8,192 context")
    ap.add_argument("--other-layers", type=int, default=8, help="how many layers of --other-shape are run")
    ap.add_argument("--no-peaks", action="store_true", help="skip measuring the copy bandwidth and a large library product")
    ap.add_argument("--model", default=None, help="use this model folder instead of writing random weights")
    ap.add_argument("--shape", choices=sorted(SHAPES), default="llama-3.2-1b", help="layer sizes of the random model")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import numpy as np
    import torch

    from prefixserve_amd import Engine, EngineConfig
    from prefixserve_amd.weights import write_random_model

    cfg = dict(SHAPES[args.shape])
    if args.model is not None:
        cfg = json.loads((Path(args.model) / "config.json").read_text())
    layers_full = cfg["num_hidden_layers"]
    if args.layers is not None:
        cfg["num_hidden_layers"] = args.layers
    layers = cfg["num_hidden_layers"]
    tmp = None
    if args.model is None:
        tmp = tempfile.TemporaryDirectory(prefix="psamd_bench_")
        model_dir = write_random_model(tmp.name, cfg, seed=0)
    else:
        model_dir = Path(args.model)
    max_batch = max(args.batch, 1 if args.no_points else 64)
    blocks = max_batch * (args.context // 16) + 64
    engine = Engine(EngineConfig(model_path=model_dir, dtype=args.dtype, max_num_seqs=max_batch,
                                 max_prefill_tokens=args.prompt_len, max_seq_len=args.context, num_blocks=blocks,
                                 use_graphs=not args.no_graphs))
    runner = engine.runner
    rng = np.random.default_rng(0)
    vocab = cfg["vocab_size"]
    weight_bytes = runner.model.step_weight_bytes()
    kv_bytes_per_token = sum(runner.bytes_per_block) // 16

    def sync() -> None:
        torch.cuda.synchronize()

    def decode_run(engine, batch: int, steps: int, warmup: int, prompt_len, context: int, repeats: int = 1) -> dict:
        """``repeats`` timed regions of exactly ``steps`` decode steps each, every one between two
        device synchronisations; the result is the median region. Beside the host clock, the
        device's own time per scheduler round (events on the stream around the round's
        launches) and the host's shares: scheduling, packing the step's integers, commit."""
        runner = engine.runner
        lens = list(prompt_len) if isinstance(prompt_len, (list, tuple)) else [prompt_len] * batch
        prompt_len = max(lens)
        sched = engine.make_scheduler(chunk_size=prompt_len, enable_prefix_cache=False)
        for b in range(batch):
            sched.add_request(f"d{batch}-{b}", rng.integers(0, vocab, lens[b]), context - lens[b] - 1, ignore_eos=True)
        # prompts, untimed: one request's prompt per step
        while any(r.num_computed < len(r.prompt) for r in sched.requests()):
            bt = sched.schedule_step(prompt_len, batch)
            sched.commit(bt, engine.step(bt))
        for _ in range(warmup):
            bt = sched.schedule_step(prompt_len, batch)
            sched.commit(bt, engine.step(bt))
        clock = time.perf_counter
        in_pack = [0.0]
        inner_pack = runner.packer._pack_step          # the cache core's check-and-fill of the step's integers

        def timed_pack(*a, **kw):
            t = clock()
            out = inner_pack(*a, **kw)
            in_pack[0] += clock() - t
            return out

        runner.packer._pack_step = timed_pack
        regions = []
        for _ in range(repeats):
            kv_start = sum(r.num_computed for r in sched.requests())
            events = []
            in_pack[0] = 0.0
            sync()
            t0 = clock()
            done = 0
            in_schedule = in_commit = 0.0
            while done < steps:
                t1 = clock()
                bt = sched.schedule_step(prompt_len, batch, min(args.decode_steps, steps - done))
                assert len(bt.work) == batch and bt.num_tokens == batch
                t2 = clock()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                sampled = engine.step(bt)
                e1.record()
                t3 = clock()
                sched.commit(bt, sampled)
                in_schedule += t2 - t1
                in_commit += clock() - t3
                events.append((e0, e1))
                done += bt.decode_steps
            sync()
            dt = clock() - t0
            kv_end = sum(r.num_computed for r in sched.requests())
            mean_kv_tokens = 0.5 * (kv_start + kv_end) + 0.5 * batch       # keys read per step, summed over requests
            bytes_per_step = weight_bytes + mean_kv_tokens * kv_bytes_per_token
            regions.append({"tok_s": batch * steps / dt, "ms_per_step": 1e3 * dt / steps,
                            "gbs": bytes_per_step * steps / dt / 1e9, "kv_len": mean_kv_tokens / batch,
                            "schedule_us": 1e6 * in_schedule / steps, "commit_us": 1e6 * in_commit / steps,
                            "pack_us": 1e6 * in_pack[0] / steps,
                            "device_us": 1e3 * sum(a.elapsed_time(b) for a, b in events) / steps})
        runner.packer._pack_step = inner_pack
        for rid in [r.req_id for r in sched.requests()]:
            sched.free_request(rid)
        regions.sort(key=lambda r: r["ms_per_step"])
        out = dict(regions[len(regions) // 2])
        out["all_ms_per_step"] = [round(r["ms_per_step"], 4) for r in regions]
        return out

    def prefill_run(reps: int = 5, warm: int = 2, portion: int | None = None) -> dict:
        """A prompt of ``--prompt-len`` tokens in one step, or in steps of ``portion`` tokens
        each over the cache the earlier portions left; the median of ``reps`` timings."""
        from prefixserve_amd.engine.batch import StepItem

        n = args.prompt_len
        portion = portion or n
        table = [list(range(-(-n // 16)))]
        toks = rng.integers(0, vocab, n)
        items = [[StepItem("p", toks[a:min(a + portion, n)], a, table, 0, [min(a + portion, n) - a - 1] if a + portion >= n else [])]
                 for a in range(0, n, portion)]
        times = []
        for rep in range(warm + reps):
            sync()
            t0 = time.perf_counter()
            for item in items:
                runner.step(item)
            sync()
            if rep >= warm:
                times.append(1e3 * (time.perf_counter() - t0))
        ms = sorted(times)[len(times) // 2]
        flops = prefill_flops(cfg, layers, n)
        return {"value": n / (ms / 1e3), "tokens": n, "ms": ms,
                "frac": flops / (ms / 1e3) / (MFMA_PEAK_TFLOPS[args.dtype] * 1e12)}

    def measured_peaks() -> dict:
        """What this GPU delivers on the two simplest workloads, to set beside the published
        peaks: a 1 GiB device copy (bytes read + written per second) and an 8192^3 library product."""
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        a = torch.randn(8192, 8192, device="cuda").to(torch.bfloat16 if args.dtype == "bfloat16" else torch.float32)
        out = {}
        for name, fn, work in (("copy_gbs", lambda: dst.copy_(src), 2 * src.numel() / 1e9),
                               ("product_tflops", lambda: torch.matmul(a, a), 2 * 8192 ** 3 / 1e12)):
            for _ in range(2):
                fn()
            sync()
            t0 = time.perf_counter()
            for _ in range(5):
                fn()
            sync()
            out[name] = work * 5 / (time.perf_counter() - t0)
        return out

    prefill = prefill_run(reps=args.prefill_reps)
    main_run = decode_run(engine, args.batch, args.steps, args.warmup, args.prompt_len, args.context, repeats=max(args.repeats, 1))
    points = {}
    if not args.no_points:
        points["decode_b1"] = decode_run(engine, 1, max(16, args.steps // 2), max(4, args.warmup // 2), args.prompt_len,
                                         args.context)["tok_s"]
        points["decode_b64"] = decode_run(engine, 64, max(16, args.steps // 4), max(4, args.warmup // 4), args.prompt_len,
                                          args.context)["tok_s"]
        if args.prompt_len > 512:
            points["prefill_portions_of_512"] = prefill_run(reps=3, warm=1, portion=512)["value"]
        if args.prompt_len > 1024:
            points["prefill_portions_of_1024"] = prefill_run(reps=3, warm=1, portion=1024)["value"]

    peaks = {} if args.no_peaks else measured_peaks()      # last: a long product changes the clocks of what follows

    def fresh_engine(folder, batch: int, prefill_tokens: int, context: int, blocks: int) -> "Engine":
        """Another engine in place of the current one (its pools go back to the device first)."""
        nonlocal engine, runner, weight_bytes, kv_bytes_per_token
        engine = runner = None
        gc.collect()
        torch.cuda.empty_cache()
        engine = Engine(EngineConfig(model_path=folder, dtype=args.dtype, max_num_seqs=batch, max_prefill_tokens=prefill_tokens,
                                     max_seq_len=context, num_blocks=blocks, use_graphs=not args.no_graphs))
        weight_bytes = engine.runner.model.step_weight_bytes()
        kv_bytes_per_token = sum(engine.runner.bytes_per_block) // 16
        return engine

    steps_q, warm_q = max(16, args.steps // 4), max(4, args.warmup // 4)
    for ctx_len in ([] if args.no_points else [c for c in (args.long_context, args.longer_context) if c > args.context]):
        # The same batch over a long context, where the cache is most of what a step reads.
        fresh_engine(model_dir, args.batch, ctx_len - 2048, ctx_len, args.batch * (ctx_len // 16) + 64)
        long_run = decode_run(engine, args.batch, steps_q, warm_q, ctx_len - 2048, ctx_len)
        points[f"decode_b{args.batch}_context_{ctx_len}"] = long_run["tok_s"]
        points[f"decode_b{args.batch}_context_{ctx_len}_hbm_frac"] = long_run["gbs"] / HBM_PEAK_GBS

    if not args.no_points and args.skewed_context > 0:
        # Contexts of unequal length in one batch: 31 requests behind 200 tokens and one behind
        # args.skewed_context, the attention reading the long one with the whole chip.
        lens = [args.skewed_context] + [200] * 31
        top = args.skewed_context + 512
        fresh_engine(model_dir, 32, args.skewed_context, top, sum(-(-(n + 300) // 16) for n in lens) + 64)
        run = decode_run(engine, 32, steps_q, warm_q, lens, top)
        points[f"decode_b32_one_context_of_{args.skewed_context}_among_200"] = run["tok_s"]
        points[f"decode_b32_one_context_of_{args.skewed_context}_among_200_hbm_frac"] = run["gbs"] / HBM_PEAK_GBS

    if not args.no_points and args.other_shape != "none" and args.model is None:
        # Another width and head size: some of the layers of a larger shape (the name says how
        # many of how many), decoding at batch 32 behind 4,096-token prompts in an 8,192 context.
        other = dict(SHAPES[args.other_shape])
        of = other["num_hidden_layers"]
        other["num_hidden_layers"] = min(args.other_layers, of)
        other_dir = write_random_model(Path(tmp.name) / "other", other, seed=1)
        fresh_engine(other_dir, 32, 4096, 8192, 32 * (8192 // 16) + 64)
        run = decode_run(engine, 32, steps_q, warm_q, 4096, 8192)
        name = f"{args.other_shape}_{other['num_hidden_layers']}_of_{of}_layers_decode_b32_context_8192"
        points[name] = run["tok_s"]
        points[name + "_hbm_frac"] = run["gbs"] / HBM_PEAK_GBS

    line = {
        "metric": "decode_tokens_per_second", "value": main_run["tok_s"], "unit": "tok/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": main_run["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: seeded uniform-random token ids, seeded random weights",
        "config": {
            "model": (args.shape if args.model is None else Path(args.model).name) + "-shape", "layers": layers_full, "layers_run": layers, "hidden": cfg["hidden_size"],
            "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
            "intermediate": cfg["intermediate_size"], "vocab": vocab, "rope_theta": cfg["rope_theta"],
            "rope_factor": (cfg.get("rope_scaling") or {}).get("factor"), "rms_norm_eps": cfg["rms_norm_eps"],
            "tied": cfg.get("tie_word_embeddings", False), "global_batch": args.batch, "seq_len": args.context,
            "prompt_len": args.prompt_len, "kv_len": round(main_run["kv_len"], 1), "page_tokens": 16,
            "decode_steps": args.decode_steps, "parallelism": "none",
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": main_run["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": main_run["gbs"] / HBM_PEAK_GBS},
        "points": points,
        # the timed region was run this often; the line is the median region
        "repeats": {"count": max(args.repeats, 1), "ms_per_step": main_run["all_ms_per_step"]},
        # per decode step inside ms_per_step: the device's own time (events around each round's
        # launches) and the host's shares (the scheduler's two calls, packing the step's integers)
        "us_per_step": {"device": main_run["device_us"], "schedule": main_run["schedule_us"], "pack": main_run["pack_us"],
                        "commit": main_run["commit_us"]},
        "measured_peaks": peaks,
    }
    print(json.dumps(line), flush=True)
    if tmp is not None:
        tmp.cleanup()
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
