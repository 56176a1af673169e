from .batch import PAGE, EngineError, StepContext, StepItem

__all__ = ["PAGE", "EngineError", "StepContext", "StepItem"]
