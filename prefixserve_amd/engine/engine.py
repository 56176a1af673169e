"""The engine a driver loop talks to: runs a scheduler batch on the GPU and returns the
sampled tokens (prefixserve/llama_engine.py:39-150 and prefixserve/engine.py:10-29 of the
reference define the same surface: ``EngineConfig``, ``step(batch)``, ``num_blocks``,
``max_seq_len``, ``stop_token_ids``, ``capture_logits``/``last_logits``).
"""

from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path
from typing import Any

import numpy as np
import torch

from prefixserve_amd.cache.manager import CacheManager
from prefixserve_amd.engine.batch import PAGE, EngineError, StepItem
from prefixserve_amd.engine.runner import ModelRunner
from prefixserve_amd.engine.scheduler import Batch, Scheduler
from prefixserve_amd.sampling.sampler import Sampler, request_key, uniform_for


@dataclass(frozen=True)
class EngineConfig:
    model_path: Path | str
    dtype: str = "bfloat16"              # "bfloat16" (serving) or "float32" (exact)
    device: str = "cuda:0"
    # Must match the scheduler's limits: they size buffers and the slot pool.
    max_num_seqs: int = 64
    # The step's budget of prompt tokens and the largest portion of one prompt. The reference's
    # default is 512 (prefixserve/server.py:48-52: its simulation lost no throughput against 2,048
    # and the time between tokens was lower). On this GPU a step has to be larger to run at the
    # matrix cores' rate: a prompt in portions of 512 / 1,024 / 2,048 tokens prefills at 216,000 /
    # 288,000 / 372,000 tokens a second at the 1B shape, and a step of 2,048 takes 5 ms there.
    max_prefill_tokens: int = 2048
    max_seq_len: int = 8192
    num_blocks: int | None = None        # None = sized from free GPU memory
    reserve_bytes: int = 1 << 30
    use_graphs: bool = True              # replay decode-only steps as captured HIP graphs
    sample_seed: int = 0
    # Decode steps a batch of decoding requests may run before the host looks at the tokens
    # (1 = after every step). More hides the host's work behind the device's; a request that
    # meets a stop token in between has computed up to decode_steps - 1 tokens for nothing, and
    # a request that arrives waits until the running batch has finished its steps.
    decode_steps: int = 1


class Engine:
    def __init__(self, cfg: EngineConfig, ops: Any = None) -> None:
        self.cfg = cfg
        self.runner = ModelRunner(
            cfg.model_path, dtype=cfg.dtype, device=cfg.device, num_blocks=cfg.num_blocks,
            max_seq_len=cfg.max_seq_len, max_num_seqs=cfg.max_num_seqs, max_prefill_tokens=cfg.max_prefill_tokens,
            reserve_bytes=cfg.reserve_bytes, use_graphs=cfg.use_graphs, ops=ops)
        self.sampler = Sampler(self.runner.ops, self.runner.device, max(cfg.max_num_seqs, 1))
        self.capture_logits = False
        self.last_logits: dict[str, torch.Tensor] = {}
        # Set to a list to have every logits row the engine samples from appended to it as
        # (request id, position of the token the row belongs to, float32 row on the host), in
        # single steps and in rounds of several decode steps alike. For tests that judge a run
        # by its logits; it waits for the device at every step.
        self.logit_trace: list[tuple[str, int, torch.Tensor]] | None = None
        # req_id -> (request, preemption count, [(array, filled)] per group): block tables as arrays,
        # extended as the lists grow, so a step does not convert whole lists again.
        self._tables: dict[str, tuple[Any, int, list[list]]] = {}
        self._sizes = self._batch_sizes()

    @property
    def num_blocks(self) -> int:
        return self.runner.num_blocks

    @property
    def max_seq_len(self) -> int:
        return self.cfg.max_seq_len

    @property
    def stop_token_ids(self) -> frozenset[int]:
        return self.runner.stop_token_ids

    def make_cache(self, enable_prefix_cache: bool = True) -> CacheManager:
        """The host-side manager of exactly this engine's pools and slots."""
        r = self.runner
        return CacheManager(r.num_blocks_per_group, r.windows, r.max_num_seqs, r.state_bytes_per_slot,
                            enable_prefix_cache=enable_prefix_cache)

    def make_scheduler(self, *, max_waiting: int = 1024, chunk_size: int | None = None,
                       enable_prefix_cache: bool = True) -> Scheduler:
        return Scheduler(cache=self.make_cache(enable_prefix_cache), max_waiting=max_waiting,
                         chunk_size=chunk_size if chunk_size is not None else self.cfg.max_prefill_tokens,
                         stop_token_ids=self.stop_token_ids, max_seq_len=self.cfg.max_seq_len)

    def _table_arrays(self, req) -> list:
        """The request's block tables as int64 arrays. A request's tables only grow while it
        runs; after a preemption it gets new ones, which the preemption count tells. An entry
        belongs to one request object: an id may come back with another request."""
        entry = self._tables.get(req.req_id)
        if (entry is None or entry[0] is not req or entry[1] != req.num_preemptions
                or len(entry[2]) != len(req.block_tables)):
            entry = (req, req.num_preemptions, [[np.empty(64, dtype=np.int64), 0] for _ in req.block_tables])
            if len(self._tables) > 8 * self.cfg.max_num_seqs:
                self._tables.clear()           # finished requests leave entries behind
            self._tables[req.req_id] = entry
        out = []
        for slot, table in zip(entry[2], req.block_tables):
            arr, filled = slot
            n = len(table)
            if n > arr.size:
                grown = np.empty(max(n, 2 * arr.size), dtype=np.int64)
                grown[:filled] = arr[:filled]
                arr = slot[0] = grown
            if n < filled:
                filled = 0
            if n > filled:
                arr[filled:n] = table[filled:n]
                slot[1] = n
            out.append(arr[:n])
        return out

    def _batch_sizes(self) -> list[int]:
        """The sizes decode batches are filled up to."""
        top = self.cfg.max_num_seqs
        sizes = [n for n in (1, 2, 4, 8) if n <= top] + list(range(16, top + 1, 8))
        return sizes if sizes and sizes[-1] == top else sizes + [top]

    def warm_up(self) -> None:
        """Does before the first request what the first requests would otherwise pay for: the
        largest step there can be (it sizes the buffers that steps share; a buffer that grows
        later drops the captured graphs, which hold its address) and, if steps are replayed as
        graphs, a capture of the decode step at every size batches are filled up to. The steps run on
        token 0 and write into the first pages of every pool, which hold nothing anybody reads
        before writing it. Call it before any request is running."""
        r = self.runner
        r.step(r.largest_step())
        if r.use_graphs:
            one_page = [[0] for _ in r.num_blocks_per_group]
            for size in reversed(self._batch_sizes()):
                items = [StepItem(key=f"warm-up-{i}", tokens=(0,), start=0, block_tables=one_page, slot=0, want=(0,))
                         for i in range(size)]
                r.step(items)
        if r.device.type == "cuda":
            torch.cuda.synchronize(r.device)

    def _padded(self, work: list) -> list:
        """A batch of decoding requests filled up to one of a few sizes (1, 2, 4, 8, then
        multiples of 8) by repeating its last item, when steps are replayed as graphs: a batch
        that loses one request at a time would otherwise meet a new shape, and a capture, at
        every step. The repeated item computes what the original computes and writes the same
        values to the same place; its row of the result is not looked at."""
        n = len(work)
        if not self.runner.use_graphs or n == 0:
            return work
        size = next((s for s in self._sizes if s >= n), n)
        return work + [work[-1]] * (size - n) if size > n else work

    def _decode_steps(self, batch: Batch) -> dict[str, list[int]]:
        """``batch.decode_steps`` steps in a row for a batch of decoding requests. The token a
        step samples stays on the device and is the next step's input there; the host packs
        the next step's integers while the device runs the current one and waits once, at the
        end, for all tokens."""
        k, work = batch.decode_steps, self._padded(batch.work)
        reqs = [w.req for w in work]
        for w in batch.work:
            if w.start + k > self.cfg.max_seq_len:
                raise EngineError(f"{w.req.req_id}: position {w.start + k} > max_seq_len {self.cfg.max_seq_len}")
        temps = [r.temperature for r in reqs]
        uniforms = [[uniform_for(self.cfg.sample_seed ^ r.seed, request_key(r.req_id), len(r.output) + j)
                     if r.temperature > 0 else 0.0 for r in reqs] for j in range(k)]
        t_dev, u_dev, out_dev = self.sampler.stage_steps(temps, uniforms)
        tables = [self._table_arrays(r) for r in reqs]
        first = [r.tokens(w.start, w.end) for r, w in zip(reqs, work)]
        for j in range(k):
            items = [StepItem(key=r.req_id, tokens=first[i] if j == 0 else (0,), start=w.start + j,
                              block_tables=tables[i], slot=max(r.slot, 0), want=(0,))
                     for i, (r, w) in enumerate(zip(reqs, work))]
            logits = self.runner.step(items, token_feed=out_dev[j - 1] if j else None)
            assert logits is not None
            if self.logit_trace is not None:
                host = logits.to("cpu", copy=True)
                self.logit_trace += [(w.req.req_id, w.start + j, host[i]) for i, w in enumerate(batch.work)]
            self.sampler.sample_into(logits, t_dev, u_dev[j], out_dev[j])
        rows = self.sampler.fetch(k, len(reqs))
        return {r.req_id: [rows[j][i] for j in range(k)] for i, r in enumerate(reqs)}

    def step(self, batch: Batch) -> dict[str, int]:
        """Runs one batch; returns req_id -> next token for the items that sample (a list of
        tokens each for a batch of several decode steps)."""
        if not batch.work:
            return {}
        if batch.decode_steps > 1:
            return self._decode_steps(batch)
        if len(batch.work) > self.cfg.max_num_seqs:
            raise EngineError(f"batch of {len(batch.work)} requests is over max_num_seqs {self.cfg.max_num_seqs}")
        work = batch.work
        if all(w.end - w.start == 1 and w.samples for w in work):
            work = self._padded(work)
        items, sampling = [], []
        for w in work:
            req, n = w.req, w.end - w.start
            if w.end > self.cfg.max_seq_len:
                raise EngineError(f"{req.req_id}: position {w.end} > max_seq_len {self.cfg.max_seq_len}")
            items.append(StepItem(key=req.req_id, tokens=req.tokens(w.start, w.end), start=w.start,
                                  block_tables=self._table_arrays(req), slot=max(req.slot, 0),
                                  want=[n - 1] if w.samples else []))
            if w.samples:
                sampling.append(req)
        logits = self.runner.step(items)
        if not sampling:
            return {}             # a portion in the middle of a prompt: nothing to wait for
        assert logits is not None
        if self.capture_logits:
            self.last_logits = {r.req_id: logits[i].to("cpu", copy=True) for i, r in enumerate(sampling)}
        if self.logit_trace is not None:
            host = logits.to("cpu", copy=True)
            # items a batch was filled up with repeat its last request and come last: not traced
            self.logit_trace += [(r.req_id, r.seq_len - 1, host[i]) for i, r in enumerate(sampling[:len(batch.work)])]
        temps = [r.temperature for r in sampling]
        seeds = [uniform_for(self.cfg.sample_seed ^ r.seed, request_key(r.req_id), len(r.output)) if r.temperature > 0
                 else 0.0 for r in sampling]
        tokens = self.sampler.sample(logits, temps, seeds)
        return {r.req_id: t for r, t in zip(sampling, tokens)}


LlamaEngine = Engine   # the reference's name for its engine
