"""RMSNorm: y = x / sqrt(mean(x^2) + eps) * w, eps inside the root, the weight
after the normalisation (internal/device/kernels.metal:905-942; host twin
internal/device/cpu_ref.go:63-83).  Statistics in 32-bit, weight held in 32-bit
(internal/engine/engine.go:788-792 promotes norm weights the same way)."""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .base import NORMS, VECTOR32, BuildEnv, Norm, StepContext, TensorSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True
    deferrable = True  # a consumer may apply it itself from x, weight, eps and the rows' sums of squares

    def __init__(self, width: int, eps: float, name: str) -> None:
        self.width = int(width)
        self.eps = float(eps)
        self.name = name
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name, (self.width,), kind=VECTOR32, init="around_one")]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        self.weight = tensors[self.name].contiguous()

    def forward(self, x: torch.Tensor, ctx: StepContext, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
        out = ctx.ws.alloc(x.shape, ctx.dtype)
        ctx.kernels.rmsnorm(x, self.weight, self.eps, out, delta=delta)
        return out
