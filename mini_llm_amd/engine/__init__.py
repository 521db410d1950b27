from .batch import StepBatch, StepEntry
from .step import ModelRunner, StepError

__all__ = ["ModelRunner", "StepBatch", "StepEntry", "StepError"]
