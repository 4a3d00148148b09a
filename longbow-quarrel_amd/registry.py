"""One registry from the architecture's name (config.json's `architectures[0]`)
to its typed configuration and the function that turns it into a `ModelSpec`.

The reference keeps a name -> creator map too (internal/engine/types_base.go:23-39),
keyed by backend; here the key is the architecture."""
from __future__ import annotations

from typing import Any, Callable, Dict, List, Tuple, Type

from .config.base import ConfigError, ModelConfig

_ARCHITECTURES: Dict[str, Tuple[Type[ModelConfig], Callable]] = {}


def register_architecture(name: str, config_cls: Type[ModelConfig], spec_fn: Callable) -> None:
    _ARCHITECTURES[name] = (config_cls, spec_fn)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def registered_architectures() -> List[str]:
    return sorted(_ARCHITECTURES)


def architecture_of(config_dict: Dict[str, Any]) -> str:
    archs = config_dict.get("architectures")
    if not archs or not isinstance(archs, list) or not isinstance(archs[0], str):
        raise ConfigError("config.json: 'architectures' must be a list that names the model class")
    return archs[0]


def lookup(name: str) -> Tuple[Type[ModelConfig], Callable]:
    if name not in _ARCHITECTURES:
        known = ", ".join(registered_architectures()) or "none"
        raise ConfigError(f"architecture {name!r} is not registered; registered: {known}")
    return _ARCHITECTURES[name]


def config_from_dict(config_dict: Dict[str, Any]) -> ModelConfig:
    config_cls, _ = lookup(architecture_of(config_dict))
    return config_cls.from_dict(config_dict)


def spec_from_config(config: ModelConfig):
    _, spec_fn = lookup(config.architecture)
    return spec_fn(config)
