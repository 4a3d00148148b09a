"""Decoding steps captured into HIP graphs.

A decoding step of a batch of B sequences launches a fixed list of kernels whose
arguments do not change from step to step: the step's integer arrays (tokens,
positions, lengths, slots) live in fixed device buffers that the step itself moves
on (the sampler writes the next tokens where the embedding reads them, a small
kernel adds one to positions and lengths).  So the whole step (model, sampler,
state upkeep) is captured once per batch size and replayed; the host only keeps
the block tables ahead of the lengths and reads the sampled tokens back.

A graph bakes in the pointers of its own workspace, logits buffer and integer
arrays; the cache, the weights and the sampler state have fixed addresses for the
life of the engine.  The split grid of the attention kernel depends on an upper
bound of the lengths, so a graph is keyed by (B, bound) and a new one is captured
when a sequence outgrows the bound.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..parts.base import StepContext, Workspace
from ..sampling.sampler import Sampler

LEN_BUCKET = 1024


def _pad4(n: int) -> int:
    return (n + 3) // 4 * 4


class DecodeGraph:
    def __init__(self, engine, batch: int, bound: int) -> None:
        self.engine = engine
        self.batch = batch
        self.bound = bound
        dev = engine.device
        b = batch
        self.sizes = [b, b, b, b, b, b, b + 1, b]  # tokens row_seq row_pos slot start len cu want
        offs, total = [], 0
        for n in self.sizes:
            offs.append(total)
            total += _pad4(n)
        self.meta = torch.zeros(total, dtype=torch.int32, device=dev)
        self.host = torch.zeros(total, dtype=torch.int32, pin_memory=dev.type == "cuda")
        self.views = [self.meta[o : o + n] for o, n in zip(offs, self.sizes)]
        self.offs = offs
        self.ws = Workspace(dev, 1 << 16)
        self.logits = torch.empty((batch, engine.vocab_size), dtype=torch.float32, device=dev)
        self.handle: Optional[int] = None
        self.slots: List[int] = []

    def load(self, slots: Sequence[int], tokens: Sequence[int], starts: Sequence[int]) -> None:
        """Writes the batch's arrays: sequence b sits in slots[b], holds starts[b] tokens and brings tokens[b]."""
        b = self.batch
        h = self.host
        o = self.offs
        h[o[0] : o[0] + b] = torch.tensor(list(tokens), dtype=torch.int32)
        h[o[1] : o[1] + b] = torch.arange(b, dtype=torch.int32)
        h[o[2] : o[2] + b] = torch.tensor(list(starts), dtype=torch.int32)
        h[o[3] : o[3] + b] = torch.tensor(list(slots), dtype=torch.int32)
        h[o[4] : o[4] + b] = torch.tensor(list(starts), dtype=torch.int32)
        h[o[5] : o[5] + b] = torch.tensor([s + 1 for s in starts], dtype=torch.int32)
        h[o[6] : o[6] + b + 1] = torch.arange(b + 1, dtype=torch.int32)
        h[o[7] : o[7] + b] = torch.arange(b, dtype=torch.int32)
        self.meta.copy_(h)
        self.slots = list(slots)

    def context(self) -> StepContext:
        e = self.engine
        t, row_seq, row_pos, slot, start, length, cu, _want = self.views
        return StepContext(
            kernels=e.kernels, dtype=e.dtype, device=e.device, ws=self.ws, rows=self.batch, batch=self.batch,
            tokens=t, row_seq=row_seq, row_pos=row_pos, seq_slot=slot, seq_start=start, seq_len=length,
            cu_rows=cu, host_slots=list(self.slots), host_start=[], host_new=[1] * self.batch,
            max_new=1, max_len=self.bound, decode=True, logits_out=self.logits)

    def run_body(self, sampler: Sampler) -> None:
        """What one decoding step launches; the same calls whether captured or run directly."""
        e = self.engine
        ctx = self.context()
        self.ws.reset()
        e.model.forward(ctx, e.cache.layer_views(), self.views[7], self.batch)
        sampler.sample(self.logits, self.views[3], self.views[0])
        e.kernels.advance(self.views[2], self.views[4], self.views[5], self.batch)

    def capture(self, sampler: Sampler) -> None:
        kn = self.engine.kernels
        # a dry pass sizes the workspace (captures must not allocate)
        self._size_workspace(sampler)
        kn.graph_begin()
        try:
            self.run_body(sampler)
        finally:
            self.handle = kn.graph_end()
        self.ws.frozen = True

    def _size_workspace(self, sampler: Sampler) -> None:
        """Runs the body's allocations without launching, to learn the workspace size."""
        e = self.engine

        queries = ("attention_workspace", "attention_folds_rope", "linear_swiglu_supported", "linear_pieces",
                   "linear_fused_parts")

        class _Null:
            """Answers the size and capability questions truthfully, launches nothing."""

            def __getattr__(self, name):
                if name in queries:
                    return getattr(e.kernels, name)
                return lambda *a, **k: None

        ctx = self.context()
        ctx.kernels = _Null()
        self.ws.reset()
        e.model.forward(ctx, e.cache.layer_views(), self.views[7], self.batch)
        self.ws.reset()  # grows the buffer to the high-water mark

    def launch(self) -> None:
        self.engine.kernels.graph_launch(self.handle)

    def destroy(self) -> None:
        if self.handle is not None:
            self.engine.kernels.graph_destroy(self.handle)
            self.handle = None
