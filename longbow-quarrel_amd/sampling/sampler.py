"""Picks the next token of every sequence of a batch from its logits, on the device."""
from __future__ import annotations

from typing import List, Optional

import torch

from .params import SamplingParams
from .state import SamplerState


NO_TOKEN = -1


class NonFiniteLogits(RuntimeError):
    """A row of logits holds a NaN or an infinity.  The reference scans for them and falls back to the
    first finite index (internal/engine/sampler.go:73-75, 107-123); a library that is checked for
    exactness reports the fault instead.  The kernels write `NO_TOKEN` for such a row and leave its
    generator and its ring of recent ids alone; whoever reads the tokens back raises this.  Raised by the
    generation loop it carries `result`: what every request had got by then, the faulty ones with the finish
    "error" and the others run to their own ends."""

    def __init__(self, message: str, result=None) -> None:
        super().__init__(message)
        self.result = result


class Sampler:
    def __init__(self, kernels, state: SamplerState, params: SamplingParams) -> None:
        self.kernels = kernels
        self.state = state
        self.params = params
        # made now, not inside a step: a captured step must not allocate
        self.scratch = None if params.greedy else state.scratch_for_sampling(kernels, state.rng_key.numel())

    def sample(self, logits: torch.Tensor, seq_slot: torch.Tensor, out: torch.Tensor) -> None:
        """logits float32 [batch, vocab] (changed in place by the penalty), seq_slot int32 [batch],
        out int32 [batch].  Launches only; safe inside a graph capture."""
        p, st, kn = self.params, self.state, self.kernels
        if p.repetition_penalty > 1.0:
            kn.apply_penalty(logits, seq_slot, st.recent, st.recent_n, p.repetition_penalty)
        if p.greedy:
            kn.argmax(logits, out, st.argmax_scratch, seq_slot, st.recent, st.recent_n)
        else:
            kn.sample(logits, out, seq_slot, p.temperature, p.top_k, p.top_p, st.rng_key, st.rng_ctr,
                      st.recent, st.recent_n, scratch=self.scratch)

    @staticmethod
    def read_tokens(out: torch.Tensor) -> List[int]:
        """The sampled tokens on the host (waits for them); raises `NonFiniteLogits` naming the rows
        whose logits could not be sampled from."""
        tokens = out.cpu().tolist()
        bad = [r for r, t in enumerate(tokens) if t == NO_TOKEN]
        if bad:
            raise NonFiniteLogits(f"the logits of row(s) {bad} hold a NaN or an infinity; nothing was sampled from them")
        return tokens
