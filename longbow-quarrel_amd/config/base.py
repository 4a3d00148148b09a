"""What every architecture's typed configuration has in common.

A configuration is a frozen dataclass whose fields carry the architecture's own
config.json keys.  `from_dict` reads and validates; `to_dict` writes the same
keys back, so a configuration and a seed are enough to write a model folder.
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict


class ConfigError(ValueError):
    """A config.json that this library cannot run; the message names the key."""


class ModelConfig:
    """Base of the typed configurations.  Subclasses are dataclasses."""

    #: the architecture name as config.json's `architectures[0]` gives it
    architecture: str = ""

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:
        raise NotImplementedError


def read_config_json(folder: str) -> Dict[str, Any]:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {folder!r}")
    with open(path, "r", encoding="utf-8") as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from e
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return d


def require(d: Dict[str, Any], key: str, kind=int):
    if key not in d or d[key] is None:
        raise ConfigError(f"config.json: required key {key!r} is missing")
    return coerce(d[key], key, kind)


def optional(d: Dict[str, Any], key: str, default, kind=int):
    if key not in d or d[key] is None:
        return default
    return coerce(d[key], key, kind)


def coerce(value, key: str, kind):
    if kind is int:
        if isinstance(value, bool) or not isinstance(value, (int, float)) or int(value) != value:
            raise ConfigError(f"config.json: {key!r} must be an integer, found {value!r}")
        return int(value)
    if kind is float:
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"config.json: {key!r} must be a number, found {value!r}")
        return float(value)
    if kind is bool:
        if not isinstance(value, bool):
            raise ConfigError(f"config.json: {key!r} must be true or false, found {value!r}")
        return value
    raise TypeError(kind)
