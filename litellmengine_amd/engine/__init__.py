from .batch import SeqInfo, StepEntry, StepState, build_step
from .runner import ModelRunner

__all__ = ["ModelRunner", "SeqInfo", "StepEntry", "StepState", "build_step"]
