"""The pre-norm decoder block: x += mixer(norm(x)); x += ffn(norm(x))
(internal/device/metal.go:1326-1527: norm :1349, residual :1434, second norm
:1451, residual :1474).  The residual stream stays float32; each add rides on
the norm kernel that follows it, or, for the few rows of a decoding step, on the projection that
produced it, which then also leaves the statistics for the norm that the next projection folds in."""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Block, BuildEnv, LayerCache, NormedRows, PartSpec,
                   ResidualSink, RowStats, StepContext, TensorSpec, build_part)


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

    takes_next_norm = True

    @property
    def first_norm(self):
        return self.mixer_norm

    @staticmethod
    def _normed(norm, x: torch.Tensor, pending, ctx: StepContext, consumer):
        """The rows for `consumer`: normalised now, or left for it to normalise where it can."""
        if isinstance(pending, RowStats):
            if consumer.takes_normed_rows and pending.norm is norm and pending.scaled is not None:
                return NormedRows(x, norm, pending)
            return norm.forward(x, ctx)
        return norm.forward(x, ctx, delta=pending)

    def forward(self, x: torch.Tensor, pending, ctx: StepContext, cache: Optional[LayerCache], next_norm=None):
        h = self._normed(self.mixer_norm, x, pending, ctx, self.mixer)
        if self.mixer.takes_residual_sink:
            sink = ResidualSink(x, self.ffn_norm)
            pending = self.mixer.forward(h, ctx, cache, sink=sink)
            pending = sink.stats if pending is None else pending
        else:
            pending = self.mixer.forward(h, ctx, cache)
        h = self._normed(self.ffn_norm, x, pending, ctx, self.ffn)
        if self.ffn.takes_residual_sink:
            sink = ResidualSink(x, next_norm)
            pending = self.ffn.forward(h, ctx, sink=sink)
            return sink.stats if pending is None else pending
        return self.ffn.forward(h, ctx)
