"""Interfaces of the parts a model is put together from, and their registries.

A model is data: a `ModelSpec` lists, layer by layer, which block, mixer,
feed-forward, norm and position encoding to build and with which sizes and
constants (`PartSpec(kind, params)`), plus the order in which layers run.  Each
kind name maps to a class through a registry; registering another class under a
new name is all it takes to make a new part available to any architecture.

No part knows which model it is in: everything it needs comes through its
constructor parameters, the tensors it declared, and the `StepContext`.
"""
from __future__ import annotations

from dataclasses import dataclass, field, replace
from typing import Any, Callable, Dict, Generic, List, Mapping, Optional, Tuple, TypeVar

import torch

T = TypeVar("T")


class Registry(Generic[T]):
    """Name -> class (or factory).  Unknown names fail with the list of known ones."""

    def __init__(self, what: str) -> None:
        self.what = what
        self._items: Dict[str, T] = {}

    def register(self, name: str, item: Optional[T] = None):
        def put(obj: T) -> T:
            if name in self._items and self._items[name] is not obj:
                raise ValueError(f"{self.what} {name!r} is already registered")
            self._items[name] = obj
            return obj

        return put if item is None else put(item)

    def unregister(self, name: str) -> None:
        self._items.pop(name, None)

    def get(self, name: str) -> T:
        if name not in self._items:
            known = ", ".join(sorted(self._items)) or "none"
            raise KeyError(f"unknown {self.what} {name!r}; registered: {known}")
        return self._items[name]

    def names(self) -> List[str]:
        return sorted(self._items)

    def __contains__(self, name: str) -> bool:
        return name in self._items


MIXERS: Registry = Registry("mixer")
FEED_FORWARDS: Registry = Registry("feed-forward")
NORMS: Registry = Registry("norm")
POSITION_ENCODINGS: Registry = Registry("position encoding")
BLOCKS: Registry = Registry("block")
EMBEDDINGS: Registry = Registry("embedding")
LOGIT_STEPS: Registry = Registry("logits step")


@dataclass(frozen=True)
class PartSpec:
    """Which class to build (`kind`, looked up in the part's registry) and its parameters."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)


# ---- tensors a part binds -------------------------------------------------------

#: follows the file: bfloat16 stays bfloat16, a 32-bit tensor stays 32-bit
#: (float16 becomes bfloat16); everything becomes float32 in the float32 mode
MATRIX = "matrix"
#: always held in float32 (norm weights)
VECTOR32 = "vector32"
#: integer table, held as int32
TABLE = "table"


@dataclass(frozen=True)
class TensorSpec:
    name: str  # the safetensors name
    shape: Tuple[int, ...]
    kind: str = MATRIX
    init: str = "normal"  # random-weights rule: "normal" | "around_one" (a gain) | "zeros"
    optional: bool = False  # may be absent from the file (a tied head)


# ---- what a mixer asks of the cache ----------------------------------------------


class CacheNeed:
    """What a mixer asks of the cache.  Needs are hashable values: runs of the schedule whose mixers
    state equal needs share one group of storage, unequal needs get storage of their own.  A need
    builds its own group, so a new kind of per-sequence storage is a new need class with a group
    class beside it (`cache.CacheGroup` is the interface) and nothing else changes."""

    def make_group(self, runs: List[int], n_blocks: int, max_slots: int, dtype: torch.dtype,
                   device: torch.device):
        """Storage for the runs of the schedule in `runs`: a pool that may hold `n_blocks` blocks of
        `cache.BLOCK_SIZE` positions, for at most `max_slots` live sequences."""
        raise NotImplementedError


@dataclass(frozen=True)
class KVNeed(CacheNeed):
    """Keys and values per position: `kv_heads` x `head_dim` each; window = 0 keeps all positions,
    window = w keeps the last w (older blocks go back to the pool)."""

    kv_heads: int
    head_dim: int
    window: int = 0

    def make_group(self, runs, n_blocks, max_slots, dtype, device):
        from ..cache.manager import KVGroup
        return KVGroup(self, runs, n_blocks, max_slots, dtype, device)


@dataclass(frozen=True)
class StateNeed(CacheNeed):
    """A block of fixed size per sequence, zeroed when a slot is taken."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32

    def make_group(self, runs, n_blocks, max_slots, dtype, device):
        from ..cache.manager import StateGroup
        return StateGroup(self, runs, max_slots, device)


# ---- build-time and step-time context ---------------------------------------------


@dataclass
class BuildEnv:
    """What parts get when their tensors are bound."""

    dtype: torch.dtype  # activation / cache dtype: torch.bfloat16 or torch.float32
    device: torch.device
    kernels: Any  # HipKernels, or a test's stand-in with the same methods


class _Arena:
    """Bump allocator over one device buffer."""

    ALIGN = 256

    def __init__(self, device: torch.device, nbytes: int) -> None:
        self.device = device
        self.off = 0
        self.high = 0
        self._spill: List[torch.Tensor] = []
        self._set_buffer(nbytes)

    def _set_buffer(self, nbytes: int) -> None:
        nbytes = (int(nbytes) + self.ALIGN - 1) // self.ALIGN * self.ALIGN
        self.buf = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        self._typed = {}  # dtype -> the whole buffer seen as that dtype: a piece of it is one view away

    def rewind(self) -> None:
        self.off = 0
        self._spill = []  # (freed in stream order: later kernels of the step may take the memory)

    def reset(self, grow: bool) -> None:
        if self.high > self.buf.numel() and grow:
            self._set_buffer(int(self.high * 1.25) + self.ALIGN)
        self.off = 0
        self.high = 0
        self._spill = []

    def alloc(self, shape, dtype: torch.dtype, frozen: bool) -> torch.Tensor:
        n = 1
        for s in shape:
            n *= int(s)
        nbytes = n * dtype.itemsize
        start = (self.off + self.ALIGN - 1) // self.ALIGN * self.ALIGN
        end = start + nbytes
        self.off = end
        self.high = max(self.high, end)
        if end > self.buf.numel():
            if frozen:
                raise RuntimeError("workspace of a captured graph is too small for this step")
            t = torch.empty(tuple(shape), dtype=dtype, device=self.device)  # this step only; reset() grows
            self._spill.append(t)
            return t
        base = self._typed.get(dtype)
        if base is None:
            base = self._typed[dtype] = self.buf.view(dtype)
        shape = tuple(shape)
        strides, step = [], 1
        for d in reversed(shape):
            strides.append(step)
            step *= int(d)
        return base.as_strided(shape, strides[::-1], start // dtype.itemsize)


class Workspace:
    """A step's temporary buffers, reset at the start of every step.

    Two lifetimes.  `alloc(..., keep=True)` lasts until the step ends (the residual stream, tables that
    every layer shares).  A plain `alloc` lasts until the end of the *next* run of the schedule: what a
    block leaves for the block after it (a pending delta, row statistics) is still there when that block
    reads it, and the memory is used again two runs later, so a step's footprint is that of two layers,
    not of all of them.  The model calls `next_run()` before each run of the schedule.

    Addresses repeat from step to step for equal shapes, which a captured HIP
    graph relies on.  It grows (outside captures) when a step needs more.
    """

    def __init__(self, device: torch.device, nbytes: int = 1 << 20) -> None:
        self.device = device
        self.step = _Arena(device, nbytes)
        self.runs = [_Arena(device, nbytes), _Arena(device, nbytes)]
        self.cur = 0
        self.frozen = False  # set while a graph that uses these buffers is alive

    def reset(self) -> None:
        for arena in (self.step, *self.runs):
            arena.reset(grow=not self.frozen)
        self.cur = 0

    def next_run(self) -> None:
        """What the run before the last one allocated is given up."""
        self.cur ^= 1
        self.runs[self.cur].rewind()

    def alloc(self, shape, dtype: torch.dtype, keep: bool = False) -> torch.Tensor:
        arena = self.step if keep else self.runs[self.cur]
        return arena.alloc(shape, dtype, self.frozen)

    @property
    def high(self) -> int:
        """Bytes this step has needed so far."""
        return self.step.high + self.runs[0].high + self.runs[1].high

    def fits(self) -> bool:
        """Whether what this step has needed so far lay inside the buffers (else the next `reset` moves them)."""
        return all(a.high <= a.buf.numel() for a in (self.step, *self.runs))


@dataclass
class StepContext:
    """One step's batch as the parts see it.  Device arrays are int32."""

    kernels: Any
    dtype: torch.dtype
    device: torch.device
    ws: Workspace
    rows: int  # tokens in this step, all sequences together (packed, no padding)
    batch: int  # sequences in this step
    tokens: torch.Tensor  # [rows]
    row_seq: torch.Tensor  # [rows] index of the row's sequence within the batch
    row_pos: torch.Tensor  # [rows] absolute position of the row in its sequence
    seq_slot: torch.Tensor  # [batch] slot of each sequence
    seq_start: torch.Tensor  # [batch] length before this step
    seq_len: torch.Tensor  # [batch] length after this step
    cu_rows: torch.Tensor  # [batch + 1] prefix sums of the rows per sequence
    # host copies of the same (lists of ints), for launch shapes and for parts written with torch
    host_slots: List[int] = field(default_factory=list)
    host_start: List[int] = field(default_factory=list)
    host_new: List[int] = field(default_factory=list)
    max_new: int = 0
    max_len: int = 0
    decode: bool = False  # every sequence brings exactly one token
    # a decoding step whose sequences differ much in length (`Mixer.lengths_uneven`): a hint, which changes how the
    # attention kernel shares its work out and nothing in the result beyond the order of its sums
    uneven: bool = False
    want_all: bool = False  # the logits of every row of the step are wanted, in the rows' order
    logits_out: Optional[torch.Tensor] = None  # where the logits go (a captured step's fixed buffer)
    # True while a step is only walked through to learn its workspace size: `kernels` then answers
    # size questions and launches nothing; a part that launches kernels of its own must not either
    dry: bool = False
    shared: Dict[Any, Any] = field(default_factory=dict)  # what parts compute once a step and share
    # debugging: called with ("embed" | "run <i>", x, pending) after the embedding and after every run of the
    # schedule; the residual stream at that point is x plus what is pending (a delta, pieces of one, or
    # nothing when the product has added it already)
    observe: Optional[Any] = None


@dataclass
class LayerCache:
    """The cache as one layer sees it."""

    write: bool = True  # False when the layer reads the cache another layer filled
    # keys/values (KVNeed)
    k: Optional[torch.Tensor] = None  # [blocks, kv_heads, block_size, head_dim]
    v: Optional[torch.Tensor] = None  # [blocks, kv_heads, head_dim, block_size]
    block_table: Optional[torch.Tensor] = None  # int32 [slots, blocks per slot]
    block_size: int = 0
    # fixed-size state (StateNeed)
    state: Optional[torch.Tensor] = None  # [slots, *shape]

    def read_only(self) -> "LayerCache":
        """The same storage for a run of the schedule that reads what another run wrote."""
        return replace(self, write=False)


# ---- the parts -----------------------------------------------------------------------


class Part:
    """Declares the tensors it binds; receives them in `bind`."""

    #: True if forward() does nothing but launch the library's kernels on buffers from ctx.ws:
    #: no allocation, no host synchronisation, no other library's operators.  Only then may a
    #: step that contains the part be captured into a HIP graph.
    graph_safe = False

    def tensor_specs(self) -> List[TensorSpec]:
        return []

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        """`tensors` holds every declared name that the file had, already on the device
        and in the dtype its kind asks for."""
        self.env = env


class Embedding(Part):
    """forward(ctx) -> the float32 residual stream [rows, width] of the step's tokens (`ctx.tokens`, with
    `ctx.row_pos` for an encoding that adds positions here), in a buffer from
    `ctx.ws.alloc(..., keep=True)`.  `table` is the [vocab, width] matrix that a tied output head uses
    (None if the embedding has none of that shape)."""

    table: Optional[torch.Tensor] = None

    def forward(self, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError


class LogitsStep(Part):
    """forward(logits, ctx): changes the float32 logits [wanted, vocab] in place, after the head (a
    scale, a soft cap)."""

    def forward(self, logits: torch.Tensor, ctx: StepContext) -> None:
        raise NotImplementedError


class Norm(Part):
    """forward(x, ctx, delta=None) -> normalised activations [rows, width] in ctx.dtype.

    x is the float32 residual stream; when `delta` is given it is first added
    to x in place (the residual add of the sub-layer before, folded in)."""

    def forward(self, x: torch.Tensor, ctx: StepContext, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    """Either exposes `rotary_frequencies` (float64 [rot/2], half-split pairs) that the
    attention kernel fuses with the cache write, or overrides `apply` to change q and k itself."""

    rotary_frequencies: Optional[torch.Tensor] = None

    def apply(self, q: torch.Tensor, k: torch.Tensor, ctx: StepContext) -> None:
        """Encode positions into q [rows, heads*hd] and k [rows, kv_heads*hd] in place."""
        raise NotImplementedError


class RowStats:
    """The residual stream is up to date and these are its rows' sums of squares, in parts
    [rows, parts]: what a projection leaves that added its result into the stream itself.  If it
    knew the norm that comes next, `scaled` holds x * that norm's gain in the run's dtype."""

    def __init__(self, sq_parts: torch.Tensor, norm=None, scaled: Optional[torch.Tensor] = None) -> None:
        self.sq_parts, self.norm, self.scaled = sq_parts, norm, scaled


class NormedRows:
    """Rows that are not normalised yet: the stream x, the norm that is due, x * gain (`scaled`) and
    the rows' sums of squares.  A consumer whose first projection can divide its output rows by the
    root mean square takes `scaled`, `sq_parts` and `eps`; anyone else calls tensor(ctx) and gets the
    normalised rows."""

    def __init__(self, x: torch.Tensor, norm, stats: RowStats) -> None:
        self.x, self.norm = x, norm
        self.scaled, self.sq_parts, self.eps = stats.scaled, stats.sq_parts, norm.eps

    @property
    def shape(self):
        return self.x.shape

    def tensor(self, ctx: "StepContext") -> torch.Tensor:
        return self.norm.forward(self.x, ctx)


class ResidualSink:
    """Offered to a mixer or feed-forward that sets `takes_residual_sink`: it may add its result into
    x itself (then it sets `stats` and returns None) instead of returning a delta.  `next_norm` is the
    norm that the stream meets next, if the block knows it."""

    def __init__(self, x: torch.Tensor, next_norm=None) -> None:
        self.x, self.next_norm = x, next_norm
        self.stats: Optional[RowStats] = None


class Mixer(Part):
    """forward(h, ctx, cache) -> [rows, width], what the block adds to the residual stream.

    h are the normalised activations of the step's rows (packed; row r belongs
    to sequence ctx.row_seq[r] at position ctx.row_pos[r]).  A mixer must give
    the same result however a sequence's tokens are cut into steps."""

    # Two optional shortcuts, both off unless a part sets the flag.  takes_normed_rows: h may be a
    # NormedRows instead of a tensor.  takes_residual_sink: forward has a keyword `sink`.
    takes_normed_rows = False
    takes_residual_sink = False

    def cache_need(self):
        """KVNeed, StateNeed or None."""
        return None

    # What a decoding step's launches depend on beside its batch size.  The engine asks every mixer and
    # keeps a captured step for as long as the answers stay the same; `ctx.max_len` and `ctx.uneven` carry
    # them (the largest bound and any yes over the model's mixers) into `forward`.
    def length_bound(self, kernels, longest: int) -> int:
        """An upper bound of the sequence lengths for a decoding step whose longest sequence holds
        `longest` tokens.  Steps with one bound must be the same launches: the coarser the bound, the fewer
        captured steps.  Default: the next power of two (at least 64), for a mixer whose launches do not
        depend on the lengths at all or that reads `ctx.max_len` without a rule of its own."""
        bound = 64
        while bound < longest:
            bound *= 2
        return bound

    def lengths_uneven(self, kernels, lengths) -> bool:
        """Whether the mixer wants a decoding step with these lengths (after the step) marked `ctx.uneven`:
        a hint that may change how its launches share out their work and nothing in the result beyond the
        order of its sums."""
        return False

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: Optional[LayerCache]) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """forward(h, ctx) -> [rows, width]; row-independent."""

    takes_normed_rows = False    # as for Mixer
    takes_residual_sink = False

    def forward(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """Arranges norm(s), mixer and feed-forward around the residual stream.

    forward(x, pending, ctx, cache) -> pending': x is the float32 residual
    stream [rows, width], updated in place; `pending` is a delta that still has
    to be added to x (it lets the add ride on the next norm kernel): the true
    stream is x + pending.  Or `pending` is a RowStats: x is up to date and its
    rows' sums of squares are known.  A block that sets `takes_next_norm` is
    also given `next_norm`, the first norm of the block that runs after it (or
    None), and exposes its own as `first_norm`."""

    takes_next_norm = False
    first_norm = None

    mixer: Mixer

    def forward(self, x: torch.Tensor, pending: Optional[torch.Tensor], ctx: StepContext,
                cache: Optional[LayerCache]) -> Optional[torch.Tensor]:
        raise NotImplementedError


def build_part(registry: Registry, spec: PartSpec, **extra):
    cls = registry.get(spec.kind)
    return cls(**dict(spec.params), **extra)


def project_normed(kn, ctx: StepContext, h, w: torch.Tensor, out: torch.Tensor, swiglu: bool = False) -> bool:
    """out = rmsnorm(x) . w^T from a NormedRows without a norm kernel, if the kernels take the size."""
    if not isinstance(h, NormedRows) or h.scaled is None or w.dtype != h.scaled.dtype:
        return False
    fused_parts = getattr(kn, "linear_fused_parts", None)
    if fused_parts is None or fused_parts(w.dtype, h.scaled.shape[0], w.shape[0], w.shape[1]) <= 0:
        return False
    kn.linear_scaled(h.scaled, h.sq_parts, h.eps, w, out, swiglu=swiglu)
    return True


def project_into(kn, ctx: StepContext, act: torch.Tensor, w: torch.Tensor, sink: Optional[ResidualSink]):
    """The last projection of a mixer or feed-forward: into the sink (-> None) where one is offered and
    the kernels take the size, else as a delta (-> tensor)."""
    if sink is not None and w.dtype == act.dtype:
        fused_parts = getattr(kn, "linear_fused_parts", None)
        rows = act.shape[0]
        parts = fused_parts(act.dtype, rows, w.shape[0], w.shape[1]) if fused_parts else 0
        if parts > 0:
            sq = ctx.ws.alloc((rows, parts), torch.float32)
            norm = sink.next_norm if getattr(sink.next_norm, "deferrable", False) else None
            scaled = ctx.ws.alloc((rows, w.shape[0]), act.dtype) if norm is not None else None
            kn.linear_residual(act, w, sink.x, sq, gain=norm.weight if norm is not None else None, scaled=scaled)
            sink.stats = RowStats(sq, norm, scaled)
            return None
    return project_delta(kn, ctx, act, w)


def project_delta(kn, ctx: StepContext, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x . w^T as a float32 delta for the residual stream: [rows, N], or [pieces, rows, N] where the
    kernels prefer to leave partial sums (whoever adds the delta adds the pieces, in order)."""
    rows, n = x.shape[0], w.shape[0]
    pieces = kn.linear_pieces(x.dtype, rows, n, x.shape[1]) if w.dtype == x.dtype else 1
    out = ctx.ws.alloc((pieces, rows, n) if pieces > 1 else (rows, n), torch.float32)
    project(kn, ctx, x, w, out)
    return out


def product_weight(env: BuildEnv, w: torch.Tensor):
    """A weight [N, K] as the kernels' products like to hold it, asked once when weights are bound: what
    `kernels.pack_weight` makes of it (something that `linear` and its siblings take in a tensor's place and that
    still answers `.shape` and `.dtype`), or the dense tensor where the kernel object has no such method."""
    w = w.contiguous()
    pack = getattr(env.kernels, "pack_weight", None)
    return pack(w) if pack is not None else w


def project(kn, ctx: StepContext, x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> None:
    """out = x . w^T.  A weight stored in 32-bit is used in 32-bit: bfloat16
    activations are widened for it rather than the weight narrowed."""
    if w.dtype == x.dtype:
        kn.linear(x, w, out)
        return
    if w.dtype != torch.float32:
        raise RuntimeError(f"a {w.dtype} weight cannot meet {x.dtype} activations")
    wide = ctx.ws.alloc(x.shape, torch.float32)
    kn.cast(x, wide)
    kn.linear(wide, w, out)
