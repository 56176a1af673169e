"""prefixserve_amd: a small, whole inference engine for one AMD MI355X (gfx950).

The package surface follows the reference's (prefixserve/__init__.py:3-32): the cache core
(``BLOCK_SIZE``, ``BlockManager``, ``RadixTree``, ``CoreError``) and the scheduler's names;
plus the engine (``Engine``/``LlamaEngine``, ``EngineConfig``), the step types and
``generate``. Importing the package compiles nothing on the GPU side; the host cache core is
compiled on first import if no built library exists.
"""

from prefixserve_amd.cache.manager import (BLOCK_SIZE, BlockManager, CacheManager, CoreError, RadixTree, StateSlots)
from prefixserve_amd.engine.batch import EngineError, StepItem
from prefixserve_amd.engine.scheduler import (AddResult, Batch, FinishReason, ReqState, Request, Scheduler,
                                              SchedulerError, SchedulerStats, StepResult, WorkItem)

__all__ = [
    "BLOCK_SIZE", "AddResult", "Batch", "BlockManager", "CacheManager", "CoreError", "Engine", "EngineConfig",
    "EngineError", "FinishReason", "LlamaEngine", "LoopTimes", "RadixTree", "ReqState", "Request", "Scheduler", "SchedulerError",
    "SchedulerStats", "StateSlots", "StepItem", "StepResult", "WorkItem", "generate",
]


def __getattr__(name: str):
    # The engine pulls in torch and the kernel bindings; load them only when asked for.
    if name in ("Engine", "LlamaEngine", "EngineConfig"):
        from prefixserve_amd.engine import engine as _engine

        return getattr(_engine, name)
    if name in ("generate", "LoopTimes"):
        from prefixserve_amd import generation as _generation

        return getattr(_generation, name)
    raise AttributeError(f"module 'prefixserve_amd' has no attribute {name!r}")
