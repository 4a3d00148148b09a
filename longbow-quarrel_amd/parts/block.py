"""The pre-norm decoder block: x += mixer(norm(x)); x += ffn(norm(x))
(internal/device/metal.go:1326-1527: norm :1349, residual :1434, second norm
:1451, residual :1474).  The residual stream stays float32; each add rides on
the norm kernel that follows it."""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Block, BuildEnv, LayerCache, PartSpec,
                   StepContext, TensorSpec, build_part)


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    def __init__(self, mixer: PartSpec, feed_forward: PartSpec, mixer_norm: PartSpec, ffn_norm: PartSpec) -> None:
        self.mixer = build_part(MIXERS, mixer)
        self.ffn = build_part(FEED_FORWARDS, feed_forward)
        self.mixer_norm = build_part(NORMS, mixer_norm)
        self.ffn_norm = build_part(NORMS, ffn_norm)

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in self.parts())

    def parts(self):
        return (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        for p in self.parts():
            p.bind(tensors, env)

    def forward(self, x: torch.Tensor, pending: Optional[torch.Tensor], ctx: StepContext,
                cache: Optional[LayerCache]) -> Optional[torch.Tensor]:
        h = self.mixer_norm.forward(x, ctx, delta=pending)
        mixed = self.mixer.forward(h, ctx, cache)
        h = self.ffn_norm.forward(x, ctx, delta=mixed)
        return self.ffn.forward(h, ctx)
