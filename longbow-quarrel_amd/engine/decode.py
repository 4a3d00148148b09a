"""Decoding steps captured into HIP graphs.

A decoding step of a batch of B sequences launches a fixed list of kernels whose
arguments do not change from step to step: the step's integer arrays (tokens,
positions, lengths, slots) live in fixed device buffers that the step itself moves
on (the sampler writes the next tokens where the embedding reads them, a small
kernel adds one to positions and lengths).  So the whole step (model, sampler,
state upkeep) is captured once per batch size and replayed; the host only keeps
the block tables ahead of the lengths and reads the sampled tokens back.

A graph bakes in the pointers of the workspace, the logits buffer and its own integer
arrays; the cache, the weights and the sampler state have fixed addresses for the
life of the engine.  What a mixer's launches depend on beside the batch size (for
attention: an upper bound of the lengths, which shapes its split grid, and whether the
lengths differ much) the mixers say themselves (`Engine.length_bound`,
`Engine.lengths_uneven`); a graph is keyed by (B, bound, uneven) and a new one is
captured when a sequence outgrows the bound.

The graphs of one `DecodeGraphs` replay one at a time on one stream, so they share one
workspace and one logits buffer, as large as the largest of them needs; when a new
graph needs more than there is, the older graphs are dropped (their pointers would
dangle) and captured again when their batch size comes back.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..kernels.dry import DryKernels
from ..parts.base import StepContext, Workspace
from ..sampling.sampler import Sampler


def _pad4(n: int) -> int:
    return (n + 3) // 4 * 4


class DecodeGraph:
    def __init__(self, engine, batch: int, bound: int, ws: Workspace, logits: torch.Tensor,
                 uneven: bool = False) -> None:
        self.engine = engine
        self.batch = batch
        self.bound = bound
        self.uneven = uneven  # the step's hint to the attention kernel (`Engine.lengths_uneven`), fixed at capture
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
        self.ws = ws
        self.logits = logits  # [batch, vocab], rows of the shared buffer
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

    def context(self, dry: bool = False) -> StepContext:
        e = self.engine
        return e.make_context(self.ws, self.views[:7], self.slots or [0] * self.batch, [], [1] * self.batch,
                              self.bound, logits_out=self.logits,
                              kernels=DryKernels(e.kernels) if dry else None, dry=dry, uneven=self.uneven,
                              want_all=True)  # (views[7] lists the rows 0 .. batch - 1)

    def run_body(self, sampler: Sampler) -> None:
        """What one decoding step launches; the same calls whether captured or run directly."""
        e = self.engine
        ctx = self.context()
        self.ws.reset()
        e.forward(ctx, self.views[7], self.batch)
        sampler.sample(self.logits, self.views[3], self.views[0])
        e.kernels.advance(self.views[2], self.views[4], self.views[5], self.batch)

    def walk(self) -> bool:
        """Walks through the body's allocations without launching (the workspace must not be frozen:
        what does not fit comes from the allocator for the walk); False if the workspace was too small."""
        e = self.engine
        self.ws.reset()
        e.forward(self.context(dry=True), self.views[7], self.batch)
        return self.ws.fits()

    def capture(self, sampler: Sampler) -> None:
        kn = self.engine.kernels
        kn.graph_begin()
        try:
            self.run_body(sampler)
        finally:
            self.handle = kn.graph_end()

    def launch(self) -> None:
        self.engine.kernels.graph_launch(self.handle)

    def destroy(self) -> None:
        if self.handle is not None:
            self.engine.kernels.graph_destroy(self.handle)
            self.handle = None


class DecodeGraphs:
    """The captured decoding steps of one backend, keyed by (batch size, length bound, whether the
    lengths are uneven), and the workspace and logits buffer that they share."""

    graph_cls = DecodeGraph

    def __init__(self, engine, sampler: Sampler) -> None:
        self.engine = engine
        self.sampler = sampler
        self.ws = Workspace(engine.device, 1 << 16)
        self.logits: Optional[torch.Tensor] = None
        self.graphs: Dict[Tuple[int, int, bool], DecodeGraph] = {}
        self.captures = 0

    def get(self, batch: int, bound: int, uneven: bool = False) -> Tuple[DecodeGraph, bool]:
        """The graph for this batch size, bound and hint, and whether it is new (then the caller loads its
        arrays and calls `capture`)."""
        key = (batch, bound, bool(uneven))
        g = self.graphs.get(key)
        if g is not None:
            return g, False
        e = self.engine
        if self.logits is None or self.logits.shape[0] < batch:
            self.drop_all()
            self.logits = torch.empty((batch, e.vocab_size), dtype=torch.float32, device=e.device)
        g = self.graph_cls(e, batch, bound, self.ws, self.logits[:batch], bool(uneven))
        self.ws.frozen = False
        if not g.walk():
            self.drop_all()  # the buffers are about to move: the graphs that point into them go
        self.ws.reset()  # grows the buffers to what the walk needed
        self.ws.frozen = True
        self.graphs[key] = g
        self.captures += 1
        return g, True

    def drop_all(self) -> None:
        for g in self.graphs.values():
            g.destroy()
        self.graphs.clear()
        self.ws.frozen = False

    def close(self) -> None:
        self.drop_all()
