"""The step function, the scheduler above it, the engine loop and trace replay."""
from .step import ModelRunner, StepContext, StepEntry, StepError

__all__ = ["ModelRunner", "StepContext", "StepEntry", "StepError"]
