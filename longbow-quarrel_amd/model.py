"""A decoder model as data (`ModelSpec`) and the object built from it.

`ModelSpec` names the embedding (a part: tokens and positions in, residual stream
out), the layers (each a block spec), the order in which layers run, the final
norm, the output head and an optional step on the logits.  `DecoderModel`
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

from .parts.base import (BLOCKS, EMBEDDINGS, LOGIT_STEPS, MATRIX, NORMS, Block, BuildEnv, Embedding, LogitsStep, Norm,
                         NormedRows, PartSpec, RowStats, StepContext, TensorSpec, build_part, product_weight, project,
                         project_normed)


@dataclass(frozen=True)
class Run:
    layer: int
    cache_of: Optional[int] = None  # read (never write) the cache of this earlier run of the schedule


@dataclass(frozen=True)
class ModelSpec:
    vocab_size: int
    width: int
    embedding: PartSpec  # an `Embedding` kind
    layers: Sequence[PartSpec]  # block specs
    schedule: Sequence[Run]
    final_norm: PartSpec
    head_name: Optional[str]  # None: always the embedding's table
    tie_head: bool  # use the embedding's table as the head (a head tensor in the file is then unexpected)
    stop_ids: Sequence[int] = field(default_factory=tuple)
    bos_id: Optional[int] = None
    logits_step: Optional[PartSpec] = None  # a `LogitsStep` kind, applied to the logits after the head
    max_positions: Optional[int] = None  # the longest sequence the architecture's configuration allows


def token_table(name: str, vocab_size: int, width: int) -> PartSpec:
    """The plain embedding: x = E[token]."""
    return PartSpec("token_table", {"name": name, "vocab_size": vocab_size, "width": width})


class DecoderModel:
    def __init__(self, spec: ModelSpec) -> None:
        self.spec = spec
        self.embedding: Embedding = build_part(EMBEDDINGS, spec.embedding)
        self.blocks: List[Block] = [build_part(BLOCKS, b) for b in spec.layers]
        self.final_norm: Norm = build_part(NORMS, spec.final_norm)
        self.logits_step: Optional[LogitsStep] = build_part(LOGIT_STEPS, spec.logits_step) if spec.logits_step else None
        for i, run in enumerate(spec.schedule):
            if not 0 <= run.layer < len(self.blocks):
                raise ValueError(f"schedule names layer {run.layer}, the model has {len(self.blocks)}")
            if run.cache_of is not None:
                if not 0 <= run.cache_of < i or spec.schedule[run.cache_of].cache_of is not None:
                    raise ValueError(f"run {i} of the schedule reads the cache of run {run.cache_of}, which is "
                                     "not an earlier run with a cache of its own")
        self.head: Optional[torch.Tensor] = None
        self.env: Optional[BuildEnv] = None

    def parts(self):
        return (self.embedding, *self.blocks, self.final_norm, *((self.logits_step,) if self.logits_step else ()))

    @property
    def graph_safe(self) -> bool:
        """Whether every part only launches library kernels (then decoding steps can be captured)."""
        return all(getattr(p, "graph_safe", False) for p in self.parts())

    # ---- tensors ---------------------------------------------------------------
    def tensor_specs(self) -> List[TensorSpec]:
        s = self.spec
        specs = list(self.embedding.tensor_specs())
        for b in self.blocks:
            specs.extend(b.tensor_specs())
        specs.extend(self.final_norm.tensor_specs())
        if s.head_name is not None and not s.tie_head:
            specs.append(TensorSpec(s.head_name, (s.vocab_size, s.width), kind=MATRIX))
        if self.logits_step is not None:
            specs.extend(self.logits_step.tensor_specs())
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv, consume: bool = False) -> None:
        """Hands every part its tensors.  With `consume` (tensors a dict that the caller gives up) a part's
        tensors leave the dict as soon as the part is bound: what a part keeps in another form (a packed
        product weight, q, k and v as one matrix) then frees its source at once, and binding a model takes the
        room of its weights plus a layer's, not twice its weights."""
        self.env = env
        s = self.spec
        waiting: Dict[str, int] = {}  # parts that still have to see a tensor (two parts may name one)
        for p in self.parts():
            for spec in p.tensor_specs():
                waiting[spec.name] = waiting.get(spec.name, 0) + 1
        for p in self.parts():
            p.bind(tensors, env)
            for spec in p.tensor_specs():
                waiting[spec.name] -= 1
                if consume and waiting[spec.name] == 0:
                    tensors.pop(spec.name, None)
        if s.head_name is not None and not s.tie_head:
            self.head = product_weight(env, tensors.pop(s.head_name) if consume else tensors[s.head_name])
        else:
            # the head is the embedding when the file has none: internal/engine/engine.go:1106-1116
            table = self.embedding.table
            if table is None or tuple(table.shape) != (s.vocab_size, s.width):
                raise ValueError("the output head is tied to the embedding, which has no [vocab, width] table")
            if getattr(self.embedding, "table_is_for_kernels", False):
                # one copy for both: the embedding's kernel reads the product's form of the table too
                table = self.embedding.table = product_weight(env, table)
            self.head = table

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

    # ---- what a decoding step's launches depend on beside the batch size ---------------
    def _mixers(self):
        return [b.mixer for b in self.blocks if getattr(b, "mixer", None) is not None]

    def length_bound(self, kernels, longest: int) -> int:
        """The largest of the mixers' bounds (`Mixer.length_bound`); `longest` itself without mixers."""
        return max((m.length_bound(kernels, longest) for m in self._mixers()), default=longest)

    def lengths_uneven(self, kernels, lengths) -> bool:
        return any(m.lengths_uneven(kernels, lengths) for m in self._mixers())

    # ---- one step -------------------------------------------------------------------
    def forward(self, ctx: StepContext, caches: Mapping[int, object], want_rows: torch.Tensor,
                n_want: int) -> Optional[torch.Tensor]:
        """Runs ctx.rows tokens through the schedule; returns float32 logits [n_want, vocab]
        of the rows listed in want_rows (None when nothing is wanted)."""
        kn = ctx.kernels
        s = self.spec
        x = self.embedding.forward(ctx)
        pending: Optional[torch.Tensor] = None
        if ctx.observe is not None:
            ctx.observe("embed", x, None)
        for i, run in enumerate(s.schedule):
            ctx.ws.next_run()  # the buffers of the run before the last one are free again
            cache = caches.get(i if run.cache_of is None else run.cache_of)
            if cache is not None and run.cache_of is not None:
                cache = cache.read_only()
            block = self.blocks[run.layer]
            if block.takes_next_norm:
                if i + 1 < len(s.schedule):
                    after = self.blocks[s.schedule[i + 1].layer].first_norm
                else:  # the final norm, where the head can take every row as it stands
                    after = self.final_norm if ctx.want_all and n_want == ctx.rows else None
                pending = block.forward(x, pending, ctx, cache, next_norm=after)
            else:
                pending = block.forward(x, pending, ctx, cache)
            if ctx.observe is not None:
                ctx.observe(f"run {i}", x, None if isinstance(pending, RowStats) else pending)
        if n_want == 0:
            return None
        ctx.ws.next_run()
        logits = ctx.logits_out
        if logits is None:
            logits = torch.empty((n_want, s.vocab_size), dtype=torch.float32, device=ctx.device)
        # every row wanted as it stands, and the last block has left the final norm's statistics: the head
        # applies the norm itself, without a kernel that picks rows and one that normalises them
        folded = ctx.want_all and n_want == ctx.rows and isinstance(pending, RowStats) \
            and pending.norm is self.final_norm \
            and project_normed(kn, ctx, NormedRows(x, self.final_norm, pending), self.head, logits)
        if not folded:
            picked = ctx.ws.alloc((n_want, s.width), torch.float32)
            kn.gather_rows(x, want_rows, picked, delta=None if isinstance(pending, RowStats) else pending)
            normed = self.final_norm.forward(picked, ctx)
            project(kn, ctx, normed, self.head, logits)
        if self.logits_step is not None:
            self.logits_step.forward(logits, ctx)
        return logits
