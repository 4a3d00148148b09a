"""Typed configurations read from a model folder's config.json."""
from .base import ConfigError, ModelConfig, read_config_json
from .llama import LlamaConfig, RopeScaling

__all__ = ["ConfigError", "ModelConfig", "read_config_json", "LlamaConfig", "RopeScaling"]
