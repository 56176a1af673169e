"""Decode-only steps as captured HIP graphs.

A decode step of a small model is a few hundred short kernels; launched one by one the
host is the bottleneck long before HBM is. For a step whose items all bring one token,
the whole launch sequence is captured once per (batch size, wanted rows) and replayed:
the step's integers are copied into the same device buffer at the same offsets (block
tables padded to a fixed width), and the kernels read lengths and tables from there, so
one graph serves every step of that shape. The number of key splits of the decode
attention is fixed from ``max_seq_len`` so the grid does not depend on the step, and a
library product (a batch of more than 64 requests) is asked for an algorithm without a
workspace, which has nothing to clear with a memset node.

Steps with portions of prompts in them were captured by shape as well, as an experiment: the
step times did not move (such steps are bound by their kernels, not by launches), so they run
eagerly.

The graph holds addresses of the packer's device buffer and of workspace buffers; if
either is reallocated (their ``version`` changes) the graph is dropped and captured again.
"""

from __future__ import annotations

import gc
from typing import TYPE_CHECKING, Any, Sequence

import torch

from prefixserve_amd.engine.batch import PAGE, StepItem

if TYPE_CHECKING:
    from prefixserve_amd.engine.runner import ModelRunner


def graphed_decode_step(runner: "ModelRunner", items: Sequence[StepItem], token_feed: Any = None) -> Any:
    wanted = sum(len(it.want) for it in items)
    static_pages = -(-runner.max_seq_len // PAGE)
    ops, ws, packer = runner.ops, runner.workspace, runner.packer
    ctx = packer.pack(items, static_pages=static_pages)
    # The attention's grid follows from the batch size, from max_seq_len and from whether one
    # context is far longer than the others: steps that differ in that are different graphs.
    key = (len(items), wanted, ctx.decode_skewed)
    if token_feed is not None:
        ctx.token_ids.copy_(token_feed)    # in stream order after the packed integers, before the graph
    entry = runner._graphs.get(key)
    if entry is not None and entry[2] == (packer.version, ws.version):
        entry[0].replay()
        return entry[1]

    previous = ops.fixed_kv_len, ops.fixed_skew
    ops.fixed_kv_len, ops.fixed_skew = runner.max_seq_len, ctx.decode_skewed
    try:
        # An eager run first: it sizes every workspace buffer (and is this step's result if
        # capture is not possible). Then capture the same sequence and replay it.
        logits = runner.model.step(ctx)
        versions = (packer.version, ws.version)
        torch.cuda.synchronize(runner.device)
        graph = torch.cuda.CUDAGraph()
        # No garbage collection while the stream is capturing: a collection that runs in the
        # middle of it may destroy what an earlier runner left behind (its graphs, their memory
        # pools), and releasing those is not allowed during a capture: the process aborts.
        # What is unreachable now is collected before, the rest after.
        gc.collect()
        gc_was_on = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph):
                captured = runner.model.step(ctx)
        finally:
            if gc_was_on:
                gc.enable()
        if (packer.version, ws.version) != versions:
            return logits      # something grew during capture; try again on a later step
        runner._graphs[key] = (graph, captured, versions)
        graph.replay()         # idempotent: same inputs, same cache writes as the eager run
        return captured
    finally:
        ops.fixed_kv_len, ops.fixed_skew = previous
