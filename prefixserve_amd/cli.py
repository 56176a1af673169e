"""Command line: ``python -m prefixserve_amd.cli <command>``.

Option names and meanings are the reference server's where it has them
(prefixserve/server.py:563-581): ``--model``, ``--dtype``, ``--max-seq-len``, ``--num-blocks``,
``--max-waiting``, ``--max-running-requests``, ``--chunked-prefill-size`` (sets both the
step's token budget and the largest portion of one prompt), ``--disable-prefix-cache``.
The reference's entry is an HTTP server; this one generates from token ids and prints JSON.

  generate       run prompts (given ids or random ids) to completion, print tokens and stats
  random-model   write a model folder (config.json, model.safetensors) from a config and a seed
  bench-core     time the host cache core's calls alone (prefix lookup, pages, step packing)
"""

from __future__ import annotations

import argparse
import json
import logging
import sys
import time
from pathlib import Path


def _add_engine_options(p: argparse.ArgumentParser) -> None:
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--max-seq-len", type=int, default=8192)
    p.add_argument("--num-blocks", type=int, default=None, help="KV blocks; default: sized from free GPU memory")
    p.add_argument("--max-waiting", type=int, default=256)
    p.add_argument("--max-running-requests", type=int, default=64)
    p.add_argument("--chunked-prefill-size", type=int, default=2048,
                   help="prompt tokens per step and per portion of one prompt (the reference's default is 512)")
    p.add_argument("--disable-prefix-cache", action="store_true")
    p.add_argument("--no-graphs", action="store_true", help="do not capture decode steps as HIP graphs")
    p.add_argument("--decode-steps", type=int, default=1,
                   help="decode steps a batch of decoding requests runs before the host looks at the tokens")
    p.add_argument("--warm-up", action="store_true",
                   help="size buffers and capture the decode graphs before the first request (not timed)")


def _generate(args: argparse.Namespace) -> int:
    import numpy as np

    from prefixserve_amd.engine.engine import Engine, EngineConfig
    from prefixserve_amd.generation import LoopTimes, generate

    cfg = EngineConfig(model_path=Path(args.model), dtype=args.dtype, max_num_seqs=args.max_running_requests,
                       max_prefill_tokens=args.chunked_prefill_size, max_seq_len=args.max_seq_len,
                       num_blocks=args.num_blocks, use_graphs=not args.no_graphs, sample_seed=args.sample_seed,
                       decode_steps=args.decode_steps)
    engine = Engine(cfg)
    if args.warm_up:
        engine.warm_up()
    prompts: list[list[int]] = [[int(t) for t in s.split(",") if t.strip()] for s in (args.prompt_ids or [])]
    if args.prompt_len:
        rng = np.random.default_rng(args.seed)
        shared = rng.integers(0, engine.runner.vocab_size, min(args.shared_prefix_len, args.prompt_len)).tolist()
        for i in range(args.num_prompts):
            own = rng.integers(0, engine.runner.vocab_size, args.prompt_len).tolist()
            # every second random prompt starts with the shared prefix
            prompts.append(shared + own[len(shared):] if shared and i % 2 == 0 else own)
    if not prompts:
        print("give --prompt-ids or --prompt-len", file=sys.stderr)
        return 2
    sched = engine.make_scheduler(max_waiting=args.max_waiting, chunk_size=args.chunked_prefill_size,
                                  enable_prefix_cache=not args.disable_prefix_cache)
    times = LoopTimes()
    t0 = time.perf_counter()
    outs, stats = generate(engine, prompts, args.max_tokens, temperature=args.temperature, seed=args.sample_seed,
                           ignore_eos=args.ignore_eos, scheduler=sched,
                           max_prefill_tokens=args.chunked_prefill_size, max_running_requests=args.max_running_requests,
                           times=times)
    dt = time.perf_counter() - t0
    new = sum(len(o.tokens) for o in outs)
    print(json.dumps({
        "outputs": [] if args.quiet else
                   [{"id": o.req_id, "tokens": o.tokens, "finish_reason": o.finish_reason.value if o.finish_reason else None,
                     "cached_tokens": o.cached_tokens, "preemptions": o.preemptions} for o in outs],
        "stats": {"seconds": dt, "new_tokens": new, "tokens_per_second": new / dt if dt > 0 else None,
                  "prompt_tokens": stats.prompt_tokens, "cached_prompt_tokens": stats.cached_prompt_tokens,
                  "prefix_hit_rate": stats.prefix_hit_rate, "preemptions": stats.preemptions,
                  "loop": times.as_dict()},
    }))
    return 0


def _random_model(args: argparse.Namespace) -> int:
    from prefixserve_amd.weights.random_init import write_random_model

    config = json.loads(Path(args.config).read_text())
    out = write_random_model(args.out, config, args.seed, std=args.std, norm_std=args.norm_std,
                             store_dtype=args.store_dtype)
    print(json.dumps({"model": str(out), "seed": args.seed}))
    return 0


def _bench_core(args: argparse.Namespace) -> int:
    """Builds the cache core's micro-benchmark (csrc/core/core_bench.cpp: the reference's
    bench/micro_core.cpp workload and three more) and runs it."""
    import subprocess
    import tempfile

    from prefixserve_amd import build

    with tempfile.TemporaryDirectory() as tmp:
        exe = build.build_core_program(build.CSRC / "core" / "core_bench.cpp", Path(tmp) / "core_bench", what="core benchmark")
        return subprocess.run([str(exe)], check=False).returncode


def main(argv: list[str] | None = None) -> int:
    parser = argparse.ArgumentParser(prog="prefixserve_amd", description=__doc__,
                                     formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--log-level", default="WARNING")
    sub = parser.add_subparsers(dest="command", required=True)

    g = sub.add_parser("generate", help="generate from token ids")
    _add_engine_options(g)
    g.add_argument("--max-tokens", type=int, default=16)
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--sample-seed", type=int, default=0)
    g.add_argument("--ignore-eos", action="store_true")
    g.add_argument("--prompt-ids", action="append", help="comma-separated token ids; may be repeated")
    g.add_argument("--prompt-len", type=int, default=0, help="make random prompts of this many ids")
    g.add_argument("--num-prompts", type=int, default=1)
    g.add_argument("--shared-prefix-len", type=int, default=0,
                   help="every second random prompt starts with the same ids of this length")
    g.add_argument("--quiet", action="store_true", help="print the statistics only, not the tokens")
    g.add_argument("--seed", type=int, default=0, help="seed of the random prompt ids")
    g.set_defaults(run=_generate)

    r = sub.add_parser("random-model", help="write a random-weights model folder")
    r.add_argument("--config", required=True, help="a config.json of the architecture")
    r.add_argument("--out", required=True)
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--std", type=float, default=0.02)
    r.add_argument("--norm-std", type=float, default=0.1)
    r.add_argument("--store-dtype", choices=["bfloat16", "float32"], default="bfloat16")
    r.set_defaults(run=_random_model)

    c = sub.add_parser("bench-core", help="time the host cache core's calls (no GPU)")
    c.set_defaults(run=_bench_core)

    args = parser.parse_args(argv)
    logging.basicConfig(level=getattr(logging, args.log_level.upper(), logging.WARNING))
    return int(args.run(args))


if __name__ == "__main__":
    raise SystemExit(main())
