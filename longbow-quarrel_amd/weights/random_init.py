"""Random weights from a configuration and a seed.

Each tensor is drawn from its own generator keyed by (seed, tensor name), so
its values do not depend on the order in which tensors are made: N(0, std) in
float32, then rounded to the stored dtype; norm gains are 1 + N(0, gain_spread),
so that a gain that is not applied, or applied twice, changes the result.  The
reference's tests write tiny synthetic model files the same way, with constant
values (internal/engine/engine_test.go:17-164).

`write_model_folder` writes config.json and model.safetensors;
`random_tensors` makes the same kind of tensors in memory, on any device (large
shapes are generated on the GPU directly and never touch the disk).
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Optional, Sequence

import torch

from ..config.base import ModelConfig
from ..parts.base import TABLE, TensorSpec
from .safetensors_io import write_safetensors


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensors(specs: Sequence[TensorSpec], seed: int, dtype: torch.dtype, std: float = 0.02,
                   device: Optional[torch.device] = None, gain_spread: float = 0.1) -> Dict[str, torch.Tensor]:
    """name -> tensor; floating tensors in `dtype` (drawn in float32, then rounded), tables int32."""
    device = torch.device(device or "cpu")
    out: Dict[str, torch.Tensor] = {}
    for s in specs:
        gen = torch.Generator(device=device)
        gen.manual_seed(_tensor_seed(seed, s.name))
        if s.kind == TABLE:
            out[s.name] = torch.zeros(s.shape, dtype=torch.int32, device=device)
            continue
        if s.init == "around_one":
            t = torch.empty(s.shape, dtype=torch.float32, device=device).normal_(1.0, gain_spread, generator=gen)
        elif s.init == "zeros":
            t = torch.zeros(s.shape, dtype=torch.float32, device=device)
        elif s.init == "normal":
            t = torch.empty(s.shape, dtype=torch.float32, device=device).normal_(0.0, std, generator=gen)
        else:
            raise ValueError(f"{s.name}: unknown init rule {s.init!r}")
        out[s.name] = t.to(dtype)
    return out


def write_model_folder(folder: str, config: ModelConfig, seed: int, dtype: Optional[torch.dtype] = None,
                       std: float = 0.02, gain_spread: float = 0.1) -> str:
    """Writes config.json and model.safetensors for `config` with weights drawn from `seed`."""
    from ..model import DecoderModel
    from ..registry import spec_from_config

    cfg = config.to_dict()
    if dtype is None:
        dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}[
            cfg.get("torch_dtype", "bfloat16")]
    model = DecoderModel(spec_from_config(config))
    tensors = random_tensors(model.tensor_specs(), seed, dtype, std, gain_spread=gain_spread)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=2)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors, {"format": "pt"})
    return folder
