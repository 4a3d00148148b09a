"""longbow-quarrel on MI355X: a small model library with its own generation.

One architecture (the Llama 3 dense decoder), one GPU, from a model folder
(config.json + model.safetensors) to generated tokens, on hand-written gfx950
kernels.
"""
from . import models  # noqa: F401  (registers the architectures)
from .api import QuarrelEngine, SamplerConfig, new_engine
from .config import ConfigError, LlamaConfig, ModelConfig
from .engine import Engine, GenerationResult, SequenceTooLong, StepEntry, generate
from .loading import load_engine, random_engine
from .sampling import NonFiniteLogits, SamplingParams
from .registry import register_architecture, registered_architectures
from .weights import WeightError, write_model_folder

__all__ = [
    "ConfigError", "LlamaConfig", "ModelConfig", "Engine", "StepEntry", "load_engine", "random_engine",
    "GenerationResult", "generate", "SamplingParams", "NonFiniteLogits", "SequenceTooLong", "QuarrelEngine", "SamplerConfig", "new_engine", "register_architecture", "registered_architectures", "WeightError", "write_model_folder",
]
