from .batch import StepBatch, StepEntry
from .engine import Engine, EngineError

__all__ = ["Engine", "EngineError", "StepBatch", "StepEntry"]
