from .batch import StepEntry, build_step
from .runner import ModelRunner

__all__ = ["StepEntry", "build_step", "ModelRunner"]
