"""The step function and the generation loop above it."""
from .step import Engine, StepEntry

__all__ = ["Engine", "StepEntry"]
