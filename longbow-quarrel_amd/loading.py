"""From a model folder (or a configuration and a seed) to an `Engine`."""
from __future__ import annotations

from typing import Any, Optional, Union

import torch

from . import models  # noqa: F401  (registers the architectures)
from .config.base import ModelConfig, read_config_json
from .engine.step import Engine
from .model import DecoderModel
from .parts.base import BuildEnv
from .registry import config_from_dict, spec_from_config
from .weights.loader import check_names_and_shapes, load_tensors
from .weights.random_init import random_tensors

_DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
}


def parse_dtype(dtype: Union[str, torch.dtype]) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"run dtype must be bfloat16 or float32, found {dtype}")
        return dtype
    if dtype not in _DTYPES:
        raise ValueError(f"run dtype must be one of {sorted(_DTYPES)}, found {dtype!r}")
    return _DTYPES[dtype]


def _env(dtype, device, kernels) -> BuildEnv:
    device = torch.device(device)
    if kernels is None:
        from .kernels.hip import HipKernels  # raises if the kernel library cannot be had
        kernels = HipKernels()
    return BuildEnv(dtype=parse_dtype(dtype), device=device, kernels=kernels)


def load_engine(folder: str, dtype: Union[str, torch.dtype] = "bfloat16", max_tokens: int = 8192,
                max_slots: int = 256, device: Union[str, torch.device] = "cuda:0",
                kernels: Any = None, max_sequence_tokens: Optional[int] = None) -> Engine:
    """config.json chooses the model class; model.safetensors is bound by tensor name.
    `max_tokens` sizes the cache for all live sequences together; `max_sequence_tokens` bounds one
    sequence (default: what the configuration allows, `max_position_embeddings` for Llama)."""
    config = config_from_dict(read_config_json(folder))
    model = DecoderModel(spec_from_config(config))
    env = _env(dtype, device, kernels)
    tensors = load_tensors(folder, model.tensor_specs(), env.dtype, env.device)
    model.bind(tensors, env, consume=True)
    del tensors
    engine = Engine(model, env, max_tokens, max_slots, max_sequence_tokens)
    engine.config = config
    return engine


def random_engine(config: ModelConfig, seed: int, dtype: Union[str, torch.dtype] = "bfloat16",
                  max_tokens: int = 8192, max_slots: int = 256,
                  device: Union[str, torch.device] = "cuda:0", kernels: Any = None,
                  std: float = 0.02, max_sequence_tokens: Optional[int] = None) -> Engine:
    """Random weights made in memory on the device (nothing is written)."""
    model = DecoderModel(spec_from_config(config))
    env = _env(dtype, device, kernels)
    specs = model.tensor_specs()
    tensors = random_tensors(specs, seed, env.dtype, std, device=env.device)
    for s in specs:  # the same dtype rule as for files
        if s.kind == "vector32":
            tensors[s.name] = tensors[s.name].float()
    check_names_and_shapes(specs, {n: tuple(t.shape) for n, t in tensors.items()}, "random weights")
    model.bind(tensors, env, consume=True)
    del tensors
    engine = Engine(model, env, max_tokens, max_slots, max_sequence_tokens)
    engine.config = config
    return engine
