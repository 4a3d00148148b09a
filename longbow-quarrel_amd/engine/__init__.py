"""The step function and the generation loop above it."""
from .generate import EngineBackend, GenerationLoop, GenerationResult, generate
from .step import Engine, SequenceTooLong, StepEntry

__all__ = ["Engine", "SequenceTooLong", "StepEntry", "EngineBackend", "GenerationLoop", "GenerationResult", "generate"]
