"""Sampling options, with the reference's names and meanings
(`SamplerConfig{Temperature, TopK, TopP, RepPenalty, Seed}`, internal/engine/types_base.go:7-15;
defaults of its command line: cmd/quarrel/main_metal.go:31-34)."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0  # 0: greedy arg-max (internal/engine/sampler.go:81-84)
    top_k: int = 0  # keep the k most probable; <= 0 or >= candidates: off (:309-314)
    top_p: float = 1.0  # shortest prefix with mass >= p; <= 0 or >= 1: off (:316-339)
    repetition_penalty: float = 1.0  # active above 1, over the last 64 ids (:77-79, 249-275)
    seed: int = 0  # a real seed: equal seeds give equal draws (the reference turns 0 into the clock)

    def __post_init__(self) -> None:
        if self.temperature < 0:
            raise ValueError(f"temperature must not be negative, found {self.temperature}")
        if self.repetition_penalty <= 0:
            raise ValueError(f"repetition_penalty must be positive, found {self.repetition_penalty}")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0
