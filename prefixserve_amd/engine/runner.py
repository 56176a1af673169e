"""ModelRunner: a model folder made ready to step on one device.

It reads the configuration, picks the model through the registry, loads and binds the
weights, sizes and allocates the page pools and state slots, and exposes the ONE step
function everything above uses: the scheduler-driven engine, generation, the benchmark
and trace replay (prefixserve/llama_engine.py:75-150 of the reference is the counterpart).
"""

from __future__ import annotations

import logging
from pathlib import Path
from typing import Any, Sequence

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
                 max_prefill_tokens: int = 512, reserve_bytes: int = 1 << 30, use_graphs: bool = True,
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
        if num_blocks is None:
            blocks = self._size_pools(reserve_bytes)
        elif isinstance(num_blocks, int):
            blocks = [num_blocks] * len(self.layer_groups)
        else:
            blocks = [int(n) for n in num_blocks]
        if len(blocks) != len(self.layer_groups):
            raise ValueError(f"{len(blocks)} pool sizes for {len(self.layer_groups)} layer groups")
        self.num_blocks_per_group = blocks
        self.pools = KVPools(self.layer_groups, blocks, self.dtype, self.device)
        state_needs = self.model.state_needs()
        self.states = make_states(state_needs, self.max_num_seqs, self.device)
        self.state_bytes_per_slot = sum(
            int(torch.empty((), dtype=n.dtype).element_size()) * int(torch.Size(n.shape).numel())
            for n in state_needs.values())
        self.model.attach(self.pools.layer_caches(), self.states)
        self.packer = StepPacker(
            self.device, [GroupMeta(nb, g.need.window) for g, nb in zip(self.layer_groups, blocks)],
            self.spec.vocab_size, self.max_seq_len, self.max_num_seqs, self.ops.PREFILL_TILE_Q)
        # A model whose mixers keep state of their own runs eagerly: capturing a step runs it
        # once before and once after the capture, which pages of keys and values do not mind
        # and a state that is added to does.
        self.use_graphs = bool(use_graphs) and self.device.type == "cuda" and not self.model.state_needs()
        self._graphs: dict[Any, Any] = {}
        logger.info("KV pools: %s blocks (%.2f GB)", blocks, self.pools.nbytes() / 1e9)

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

    def _size_pools(self, reserve_bytes: int) -> list[int]:
        """Pages that fit in what is free after the weights, the buffers of a worst-case
        step and a reserve (prefixserve/llama_engine.py:231-267 sizes its pool the same way:
        sizing from free memory alone would leave nothing for activations)."""
        if self.device.type != "cuda":
            raise ValueError("num_blocks must be given when not on a GPU")
        t = self.max_prefill_tokens + self.max_num_seqs
        act = self._activation_bytes(t)
        free, _total = torch.cuda.mem_get_info(self.device)
        usable = free - act - reserve_bytes
        per_token_page = sum(self.bytes_per_block)
        n = int(usable // per_token_page)
        need = -(-self.max_seq_len // PAGE)
        if n < need:
            raise EngineError(f"only {n} KV blocks fit ({usable / 1e9:.2f} GB usable); one request of "
                              f"max_seq_len needs {need}")
        return [n] * len(self.layer_groups)

    def _activation_bytes(self, tokens: int) -> int:
        """Device memory the buffers of a step of ``tokens`` tokens take: what the parts say they
        ask for (buffers are shared between layers by name, so the largest layer counts), the
        float32 residual stream, the logits of every request and a margin."""
        s = self.spec
        itemsize = torch.empty((), dtype=self.dtype).element_size()
        widest = max((sum(p.activation_bytes(tokens, itemsize) for p in blk.parts()) for blk in self.model.blocks),
                     default=0)
        return widest + tokens * s.hidden_size * 4 + self.max_num_seqs * s.vocab_size * 4 + (256 << 20)

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
        if self.use_graphs and all(len(it.tokens) == 1 for it in items):
            from prefixserve_amd.engine.graphs import graphed_decode_step

            out = graphed_decode_step(self, items, token_feed)
            if out is not NotImplemented:
                return out
        ctx = self.packer.pack(items)
        if token_feed is not None:
            ctx.token_ids.copy_(token_feed)
        return self.model.step(ctx)

    def pack(self, items: Sequence[StepItem]) -> StepContext:
        return self.packer.pack(items)

    def tune_products(self, token_counts: Sequence[int]) -> list[tuple[int, tuple[int, int], float, float]]:
        """Lets the product library time its algorithms for steps of the given token counts,
        once per distinct matrix shape of the model's parts, and keep the fastest: the library's
        own choice is made without running anything. The same product of every layer shares a
        shape; its matrices are timed in turn, so that each call reads its matrix from memory as
        a step does. Returns (tokens, (out, in), microseconds before, after) per tuned product.
        For warm-up: a second or so per shape."""
        tune = getattr(self.ops, "tune_linear", None)
        done: list[tuple[int, tuple[int, int], float, float]] = []
        if tune is None or self.dtype != torch.bfloat16:
            return done
        by_shape: dict[tuple[int, int], list[torch.Tensor]] = {}
        for blk in self.model.blocks:
            for part in blk.parts():
                for w in part.product_weights():
                    by_shape.setdefault((int(w.shape[0]), int(w.shape[1])), []).append(w)
        for shape, weights in by_shape.items():
            for t in dict.fromkeys(int(t) for t in token_counts):
                res = tune(t, weights)
                if res is not None:
                    done.append((t, shape, res[0], res[1]))
                    logger.info("product of %d tokens by [%d, %d]: %.1f -> %.1f us", t, shape[0], shape[1], *res)
        return done
