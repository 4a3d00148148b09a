"""Dense SwiGLU feed-forward: down(silu(gate(n)) * up(n)), no biases, no clamps
(internal/device/metal.go:1464-1471; silu(g) = g / (1 + e^-g),
internal/device/cpu_ref.go:132-149).  gate and up are concatenated at bind time
so that one matrix product makes both."""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional

import torch

from .base import (FEED_FORWARDS, BuildEnv, FeedForward, NormedRows, StepContext, TensorSpec, product_weight, project,
                   project_into, project_normed)


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True

    def __init__(self, width: int, inner: int, prefix: str, names: Optional[Mapping[str, str]] = None) -> None:
        self.width, self.inner = int(width), int(inner)
        n = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}
        n.update(names or {})
        self.names: Dict[str, str] = {key: f"{prefix}.{val}" for key, val in n.items()}
        self.fused = False
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [
            TensorSpec(self.names["gate"], (self.inner, self.width)),
            TensorSpec(self.names["up"], (self.inner, self.width)),
            TensorSpec(self.names["down"], (self.width, self.inner)),
        ]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        gate, up = tensors[self.names["gate"]], tensors[self.names["up"]]
        if gate.dtype != up.dtype:
            raise ValueError(f"{self.names['gate']}: gate and up projections are stored in different dtypes")
        kn = env.kernels
        self.fused = gate.dtype == env.dtype and self.inner % 8 == 0 and \
            getattr(kn, "linear_swiglu_supported", lambda *a: False)(gate.dtype, 2 * self.inner, self.width)
        if self.fused:
            # gate and up rows interleaved so that the product's epilogue can apply silu(g) * u itself
            self.w_gate_up = product_weight(env, kn.interleave_gate_up(gate, up))
        else:
            self.w_gate_up = product_weight(env, torch.cat([gate, up], dim=0))
        self.w_down = product_weight(env, tensors[self.names["down"]])

    takes_normed_rows = True
    takes_residual_sink = True

    def forward(self, h, ctx: StepContext, sink=None) -> Optional[torch.Tensor]:
        kn = ctx.kernels
        rows = h.shape[0]
        act = ctx.ws.alloc((rows, self.inner), ctx.dtype)
        if self.fused:
            if not project_normed(kn, ctx, h, self.w_gate_up, act, swiglu=True):
                if isinstance(h, NormedRows):
                    h = h.tensor(ctx)
                kn.linear_swiglu(h, self.w_gate_up, act)
        else:
            gu = ctx.ws.alloc((rows, 2 * self.inner), torch.float32)
            if not project_normed(kn, ctx, h, self.w_gate_up, gu):
                if isinstance(h, NormedRows):
                    h = h.tensor(ctx)
                project(kn, ctx, h, self.w_gate_up, gu)
            kn.swiglu(gu, act)
        return project_into(kn, ctx, act, self.w_down, sink)
