"""Fixed-size state of each sequence's sampler, in device arrays indexed by slot:
the random generator (a 64-bit key and a draw counter; draw n of a sequence depends
on its key and n only, so it does not depend on the batch around it) and the ring
of the last 64 token ids that the repetition penalty looks at
(internal/engine/sampler.go:13-26 holds the generator, :249-275 the 64-id window)."""
from __future__ import annotations

from typing import Sequence

import torch

RECENT = 64
_MASK = (1 << 64) - 1


def sequence_key(seed: int, index: int) -> int:
    """The generator key of the `index`-th request of a run with `seed` (splitmix64 of both)."""
    z = (seed * 0x9E3779B97F4A7C15 + (index + 1) * 0xD1B54A32D192ED03) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    z = z ^ (z >> 31)
    return z - (1 << 64) if z >= (1 << 63) else z  # as a signed 64-bit value


class SamplerState:
    def __init__(self, max_slots: int, device: torch.device, window: int = RECENT) -> None:
        """`window`: ids of history that the penalty looks at (the sampling kernels say which width they take)."""
        self.device = device
        self.window = int(window)
        self.rng_key = torch.zeros(max_slots, dtype=torch.int64, device=device)
        self.rng_ctr = torch.zeros(max_slots, dtype=torch.int64, device=device)
        self.recent = torch.full((max_slots, self.window), -1, dtype=torch.int32, device=device)
        self.recent_n = torch.zeros(max_slots, dtype=torch.int32, device=device)
        # what the two stages of the arg-max kernel pass between them: 32 words for each row of a batch
        self.argmax_scratch = torch.zeros(32 * max_slots, dtype=torch.int64, device=device)
        # what the stages of temperature sampling with a small top-k pass between them (made when first asked for)
        self.sample_scratch = None

    def scratch_for_sampling(self, kernels, rows: int):
        need = getattr(kernels, "sample_scratch_bytes", None)
        if need is None:
            return None
        if self.sample_scratch is None:
            self.sample_scratch = torch.zeros(need(self.rng_key.numel()), dtype=torch.uint8, device=self.device)
        return self.sample_scratch if rows <= self.rng_key.numel() else None

    def start(self, slot: int, key: int, history: Sequence[int]) -> None:
        """A sequence starts in `slot`: generator at draw 0, ring holding the end of its prompt."""
        ring = self.window
        tail = list(history[-ring:])
        row = torch.full((ring,), -1, dtype=torch.int32)
        if tail:
            # the ring is written at n % its width; lay the tail out as if it had been pushed one by one
            n = len(history)
            for j, tok in enumerate(tail):
                row[(n - len(tail) + j) % ring] = int(tok)
        self.recent[slot].copy_(row)
        self.recent_n[slot : slot + 1].copy_(torch.tensor([len(history)], dtype=torch.int32))
        self.rng_key[slot : slot + 1].copy_(torch.tensor([key], dtype=torch.int64))
        self.rng_ctr[slot : slot + 1].copy_(torch.tensor([0], dtype=torch.int64))
