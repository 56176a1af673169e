"""ModelRunner: a model folder made ready to step on one device.

It reads the configuration, picks the model through the registry, loads and binds the
weights, sizes and allocates the page pools and state slots, and exposes the ONE step
function everything above uses: the scheduler-driven engine, generation, the benchmark
and trace replay (prefixserve/llama_engine.py:75-150 of the reference is the counterpart).
"""

from __future__ import annotations

import gc
import logging
from pathlib import Path
from typing import Any, Sequence

import numpy as np
import torch

import prefixserve_amd.models  # noqa: F401  (fills the architecture registry)
from prefixserve_amd.cache.pool import KVPools, make_states, plan_groups
from prefixserve_amd.config.registry import read_model_dir
from prefixserve_amd.engine.batch import PAGE, EngineError, GroupMeta, StepContext, StepItem, StepPacker
from prefixserve_amd.parts.base import Runtime, Workspace
from prefixserve_amd.parts.model import DecoderModel
from prefixserve_amd.weights.loader import load_weights

logger = logging.getLogger(__name__)

DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def _make_ops(device: torch.device, workspace: Workspace) -> Any:
    """The compiled kernels, or an error: there is nothing to fall back to."""
    from prefixserve_amd.kernels.ops import HipOps

    return HipOps(device, workspace)


class ModelRunner:
    def __init__(self, model_dir: str | Path, dtype: str | torch.dtype = "bfloat16", device: str = "cuda:0",
                 num_blocks: int | Sequence[int] | None = None, max_seq_len: int = 8192, max_num_seqs: int = 64,
                 max_prefill_tokens: int = 2048, reserve_bytes: int = 1 << 30, use_graphs: bool = True,
                 ops: Any = None) -> None:
        self.device = torch.device(device)
        self.dtype = DTYPES[dtype] if isinstance(dtype, str) else dtype
        if self.dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"dtype must be bfloat16 or float32, got {dtype}")
        self.max_seq_len, self.max_num_seqs = int(max_seq_len), int(max_num_seqs)
        self.max_prefill_tokens = int(max_prefill_tokens)

        arch, self.config, self.raw_config = read_model_dir(model_dir)
        self.spec = arch.build_spec(self.config)
        if self.max_seq_len > self.spec.max_position:
            raise ValueError(f"max_seq_len {self.max_seq_len} > model limit {self.spec.max_position}")
        self.model = DecoderModel(self.spec)
        self.workspace = Workspace(self.device)
        self.ops = ops if ops is not None else _make_ops(self.device, self.workspace)
        if getattr(self.ops, "ws", None) is None:
            self.ops.ws = self.workspace
        self.rt = Runtime(self.device, self.dtype, self.ops, self.workspace)

        # Read tensor by tensor as the parts bind: the host never holds the whole checkpoint.
        with load_weights(model_dir, self.model.weights(), self.spec.ignored_weights) as tensors:
            self.model.bind(tensors, self.rt, self.max_seq_len)
        logger.info("weights bound: %.2f GB read per decode step", self.model.step_weight_bytes() / 1e9)

        self.layer_groups = plan_groups(self.model.cache_needs())
        itemsize = torch.empty((), dtype=self.dtype).element_size()
        self.bytes_per_block = [g.bytes_per_block(itemsize) for g in self.layer_groups]
        state_needs = self.model.state_needs()
        self.states = make_states(state_needs, self.max_num_seqs, self.device)
        self.state_bytes_per_slot = sum(
            int(torch.empty((), dtype=n.dtype).element_size()) * int(torch.Size(n.shape).numel())
            for n in state_needs.values())
        # A model whose mixers keep state of their own runs eagerly: capturing a step runs it
        # once before and once after the capture, which pages of keys and values do not mind
        # and a state that is added to does.
        self.use_graphs = bool(use_graphs) and self.device.type == "cuda" and not state_needs
        self._graphs: dict[Any, Any] = {}
        if num_blocks is None:
            blocks = self._size_pools(reserve_bytes)
        elif isinstance(num_blocks, int):
            blocks = [num_blocks] * len(self.layer_groups)
        else:
            blocks = [int(n) for n in num_blocks]
        if len(blocks) != len(self.layer_groups):
            raise ValueError(f"{len(blocks)} pool sizes for {len(self.layer_groups)} layer groups")
        self._install_pools(blocks)
        logger.info("KV pools: %s blocks (%.2f GB)", blocks, self.pools.nbytes() / 1e9)

    def _install_pools(self, blocks: Sequence[int]) -> None:
        """Page pools of the given sizes, attached to the model, and the packer that checks page
        ids against them."""
        self.num_blocks_per_group = list(blocks)
        self.pools = KVPools(self.layer_groups, self.num_blocks_per_group, self.dtype, self.device)
        self.model.attach(self.pools.layer_caches(), self.states)
        self.packer = StepPacker(
            self.device, [GroupMeta(nb, g.need.window) for g, nb in zip(self.layer_groups, blocks)],
            self.spec.vocab_size, self.max_seq_len, self.max_num_seqs, self.ops.PREFILL_TILE_Q,
            skew_rule=getattr(self.ops, "decode_is_skewed", None))

    # ------------------------------------------------------------ properties

    @property
    def num_blocks(self) -> int:
        """Pages of the first (for Llama: the only) layer group."""
        return self.num_blocks_per_group[0]

    @property
    def windows(self) -> list[int | None]:
        return [g.need.window for g in self.layer_groups]

    @property
    def stop_token_ids(self) -> frozenset[int]:
        return self.spec.stop_token_ids

    @property
    def vocab_size(self) -> int:
        return self.spec.vocab_size

    # ---------------------------------------------------------------- sizing

    def largest_step(self) -> list[StepItem]:
        """The largest step a scheduler can ask this runner for: a portion of the whole prefill
        budget beside decoding requests in all other places, every item wanting its logits. On
        token 0, in the first pages of every pool and in slot 0: for sizing buffers before any
        request runs (nothing anybody reads before writing it is touched)."""
        groups = self.num_blocks_per_group
        n = min(self.max_prefill_tokens, self.max_seq_len, PAGE * min(groups))
        one_page = [[0] for _ in groups]
        items = [StepItem(key="largest", tokens=np.zeros(n, dtype=np.int32), start=0,
                          block_tables=[list(range(-(-n // PAGE))) for _ in groups], slot=0, want=(n - 1,))]
        items += [StepItem(key=f"largest-{i}", tokens=(0,), start=0, block_tables=one_page, slot=0, want=(0,))
                  for i in range(self.max_num_seqs - 1)]
        return items

    def _size_pools(self, reserve_bytes: int) -> list[int]:
        """Pages that fit in what is free after the weights, after everything the largest step
        really takes, and a reserve. The step is run once on a throwaway pool of a few pages: its
        buffers stay (the workspace keeps them for every later step), so what the device reports
        free afterwards is what is left for pages (prefixserve/llama_engine.py:231-267,304-320
        measures a dummy step on a dummy pool the same way; sizing from free memory alone would
        leave nothing for activations, and an estimate would have to know every part's buffers)."""
        if self.device.type != "cuda":
            raise ValueError("num_blocks must be given when not on a GPU")
        probe = -(-min(self.max_prefill_tokens, self.max_seq_len) // PAGE) + 1
        self._install_pools([probe] * len(self.layer_groups))
        graphs, self.use_graphs = self.use_graphs, False
        try:
            self.step(self.largest_step())
            torch.cuda.synchronize(self.device)
        finally:
            self.use_graphs = graphs
        for state in self.states.values():
            state.zero_()
        self.pools = None
        self.model.attach({}, self.states)
        gc.collect()
        torch.cuda.empty_cache()             # the throwaway pool goes back to the device; the step's buffers are in use
        free, _total = torch.cuda.mem_get_info(self.device)
        usable = free - reserve_bytes
        n = int(usable // sum(self.bytes_per_block))
        n = min(n, (1 << 27) - 1)            # a token's place, page * 16 + offset, is a 32-bit integer
        need = -(-self.max_seq_len // PAGE)
        if n < need:
            raise EngineError(f"only {n} KV blocks fit ({usable / 1e9:.2f} GB usable after a largest step's buffers "
                              f"and a reserve of {reserve_bytes / 1e9:.2f} GB); one request of max_seq_len needs {need}")
        logger.info("pools sized after a measured largest step: %.2f GB of buffers, %.2f GB for pages",
                    self.workspace.nbytes() / 1e9, usable / 1e9)
        return [n] * len(self.layer_groups)

    # ------------------------------------------------------------------ step

    @torch.inference_mode()
    def step(self, items: Sequence[StepItem], token_feed: torch.Tensor | None = None) -> torch.Tensor | None:
        """One step: runs exactly the given tokens as one batch from the cache that earlier
        steps left, and returns float32 logits ``[S, vocab]`` in the order of the items and
        of their ``want`` (None if nothing is wanted). Steps run strictly in order on the
        current stream, so step N+1 reads what step N wrote.

        ``token_feed``: int32 ``[T]`` on the device, taken for the step's token ids instead of
        the items' own (which must still be valid ids): the tokens an earlier step sampled and
        the host has not seen yet."""
        if self.states:
            self._clear_new_slots(items)
        if self.use_graphs and all(len(it.tokens) == 1 for it in items):
            from prefixserve_amd.engine.graphs import graphed_decode_step

            out = graphed_decode_step(self, items, token_feed)
            if out is not NotImplemented:
                return out
        ctx = self.packer.pack(items)
        if token_feed is not None:
            ctx.token_ids.copy_(token_feed)
        return self.model.step(ctx)

    def _clear_new_slots(self, items: Sequence[StepItem]) -> None:
        """Zeroes the state slots of the items that start at position 0, in stream order before
        the step: a slot comes from the allocator with its last owner's contents, and a request
        (new, or sent back and starting over) begins from nothing. Mixers never clear slots."""
        fresh = sorted({int(it.slot) for it in items if it.start == 0})
        if not fresh:
            return
        for s in fresh:
            if not 0 <= s < self.max_num_seqs:
                raise EngineError(f"state slot {s} outside [0, {self.max_num_seqs})")
        index = torch.tensor(fresh, dtype=torch.int64).to(self.device, non_blocking=True)
        for state in self.states.values():
            state.index_fill_(0, index, 0)

    def pack(self, items: Sequence[StepItem]) -> StepContext:
        return self.packer.pack(items)
