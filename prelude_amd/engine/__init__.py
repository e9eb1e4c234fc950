from .batch import GroupStep, StepBatch
from .engine import Engine, StepEntry, StepError

__all__ = ["GroupStep", "StepBatch", "Engine", "StepEntry", "StepError"]
