from .batch import DeviceToken, StepBatch, StepEntry
from .engine import Engine, EngineError

__all__ = ["DeviceToken", "Engine", "EngineError", "StepBatch", "StepEntry"]
