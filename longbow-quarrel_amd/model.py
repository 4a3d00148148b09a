"""A decoder model as data (`ModelSpec`) and the object built from it.

`ModelSpec` names the token embedding, the layers (each a block spec), the
order in which layers run, the final norm and the output head.  `DecoderModel`
builds the parts through their registries, declares every tensor they bind,
and runs a step's rows through the schedule.

The schedule is a list of `Run(layer, cache_of)`.  The same layer may appear
more than once: it then runs again with the same weights, and every run has a
cache of its own (its inputs differ, so its keys and values do).  `cache_of = j`
lets a run read what run number j of the schedule (an earlier one) wrote instead
of writing its own.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Mapping, Optional, Sequence

import torch

from .parts.base import (BLOCKS, MATRIX, NORMS, Block, BuildEnv, LayerCache, Norm, PartSpec, RowStats,
                         StepContext, TensorSpec, build_part, project)


@dataclass(frozen=True)
class Run:
    layer: int
    cache_of: Optional[int] = None  # read (never write) the cache of this earlier run of the schedule


@dataclass(frozen=True)
class ModelSpec:
    vocab_size: int
    width: int
    embedding_name: str
    layers: Sequence[PartSpec]  # block specs
    schedule: Sequence[Run]
    final_norm: PartSpec
    head_name: Optional[str]  # None: always the embedding matrix
    tie_head: bool  # use the embedding matrix as the head (a head tensor in the file is then unexpected)
    stop_ids: Sequence[int] = field(default_factory=tuple)
    bos_id: Optional[int] = None


class DecoderModel:
    def __init__(self, spec: ModelSpec) -> None:
        self.spec = spec
        self.blocks: List[Block] = [build_part(BLOCKS, b) for b in spec.layers]
        self.final_norm: Norm = build_part(NORMS, spec.final_norm)
        for i, run in enumerate(spec.schedule):
            if not 0 <= run.layer < len(self.blocks):
                raise ValueError(f"schedule names layer {run.layer}, the model has {len(self.blocks)}")
            if run.cache_of is not None:
                if not 0 <= run.cache_of < i or spec.schedule[run.cache_of].cache_of is not None:
                    raise ValueError(f"run {i} of the schedule reads the cache of run {run.cache_of}, which is "
                                     "not an earlier run with a cache of its own")
        self.embedding: Optional[torch.Tensor] = None
        self.head: Optional[torch.Tensor] = None
        self.env: Optional[BuildEnv] = None

    # ---- tensors ---------------------------------------------------------------
    def tensor_specs(self) -> List[TensorSpec]:
        s = self.spec
        specs = [TensorSpec(s.embedding_name, (s.vocab_size, s.width), kind=MATRIX)]
        for b in self.blocks:
            specs.extend(b.tensor_specs())
        specs.extend(self.final_norm.tensor_specs())
        if s.head_name is not None and not s.tie_head:
            specs.append(TensorSpec(s.head_name, (s.vocab_size, s.width), kind=MATRIX))
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        self.env = env
        s = self.spec
        self.embedding = tensors[s.embedding_name].contiguous()
        for b in self.blocks:
            b.bind(tensors, env)
        self.final_norm.bind(tensors, env)
        if s.head_name is not None and not s.tie_head:
            self.head = tensors[s.head_name].contiguous()
        else:
            # the head is the embedding when the file has none: internal/engine/engine.go:1106-1116
            self.head = self.embedding

    # ---- what the cache has to hold -----------------------------------------------
    def cache_needs(self) -> Dict[int, object]:
        """Run number -> KVNeed / StateNeed, for the runs of the schedule that own a cache."""
        needs = {}
        for i, run in enumerate(self.spec.schedule):
            if run.cache_of is None:
                need = self.blocks[run.layer].mixer.cache_need()
                if need is not None:
                    needs[i] = need
        return needs

    # ---- one step -------------------------------------------------------------------
    def forward(self, ctx: StepContext, caches: Mapping[int, LayerCache], want_rows: torch.Tensor,
                n_want: int) -> Optional[torch.Tensor]:
        """Runs ctx.rows tokens through the schedule; returns float32 logits [n_want, vocab]
        of the rows listed in want_rows (None when nothing is wanted)."""
        kn = ctx.kernels
        s = self.spec
        x = ctx.ws.alloc((ctx.rows, s.width), torch.float32, keep=True)
        kn.embed(self.embedding, ctx.tokens, x)
        pending: Optional[torch.Tensor] = None
        if ctx.observe is not None:
            ctx.observe("embed", x, None)
        for i, run in enumerate(s.schedule):
            ctx.ws.next_run()  # the buffers of the run before the last one are free again
            cache = caches.get(i if run.cache_of is None else run.cache_of)
            if cache is not None and run.cache_of is not None:
                cache = LayerCache(write=False, k=cache.k, v=cache.v, block_table=cache.block_table,
                                   block_size=cache.block_size, state=cache.state)
            block = self.blocks[run.layer]
            if block.takes_next_norm:
                after = self.blocks[s.schedule[i + 1].layer].first_norm if i + 1 < len(s.schedule) else None
                pending = block.forward(x, pending, ctx, cache, next_norm=after)
            else:
                pending = block.forward(x, pending, ctx, cache)
            if ctx.observe is not None:
                ctx.observe(f"run {i}", x, None if isinstance(pending, RowStats) else pending)
        if n_want == 0:
            return None
        ctx.ws.next_run()
        picked = ctx.ws.alloc((n_want, s.width), torch.float32)
        kn.gather_rows(x, want_rows, picked, delta=None if isinstance(pending, RowStats) else pending)
        normed = self.final_norm.forward(picked, ctx)
        logits = ctx.logits_out
        if logits is None:
            logits = torch.empty((n_want, s.vocab_size), dtype=torch.float32, device=ctx.device)
        project(kn, ctx, normed, self.head, logits)
        return logits
