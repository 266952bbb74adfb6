from .batch import StepContext, StepEntry, build_context
from .runner import ModelRunner

__all__ = ["StepContext", "StepEntry", "build_context", "ModelRunner"]
