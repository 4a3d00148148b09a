"""The step function and the generation loop above it."""
from .generate import EngineBackend, GenerationLoop, GenerationResult, generate
from .step import Engine, StepEntry

__all__ = ["Engine", "StepEntry", "EngineBackend", "GenerationLoop", "GenerationResult", "generate"]
