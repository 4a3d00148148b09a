"""The step function: a batch of sequences, each bringing its next tokens.

`Engine.step` runs only the tokens it is given, as one packed batch without
padding, from the cache that earlier steps left, and returns the logits at the
wanted places.  A sequence's first step may bring its whole prompt; later steps
usually bring one token.  Row r of a sequence that already holds n tokens has
position n + r, writes its key and value first and then attends to positions
0..n+r of its own sequence only; that is the reference's per-row contract
(internal/device/metal.go:1384-1424: row r at pos + r, store then attend)
generalised from one sequence to a batch.

The reference validates its input the same way (empty input, ids outside the
vocabulary: internal/engine/engine.go:1300-1331).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..cache import CacheManager
from ..model import DecoderModel
from ..parts.base import BuildEnv, StepContext, Workspace


@dataclass
class StepEntry:
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()  # indices into `tokens` whose logits are asked for


def _pad4(n: int) -> int:
    return (n + 3) // 4 * 4


class StepMeta:
    """Packs a step's integer arrays into one host buffer and one upload."""

    def __init__(self, device: torch.device) -> None:
        self.device = device
        self.cap = 0
        self.host: Optional[torch.Tensor] = None
        self.dev: Optional[torch.Tensor] = None

    def _grow(self, n: int) -> None:
        if n <= self.cap:
            return
        self.cap = max(1024, int(n * 1.5))
        pin = self.device.type == "cuda"
        self.host = torch.empty(self.cap, dtype=torch.int32, pin_memory=pin)
        self.dev = torch.empty(self.cap, dtype=torch.int32, device=self.device)

    def upload(self, sections: Sequence[Sequence[int]]) -> List[torch.Tensor]:
        sizes = [len(s) for s in sections]
        total = sum(_pad4(max(1, n)) for n in sizes)
        self._grow(total)
        flat: List[int] = []
        offsets = []
        for s, n in zip(sections, sizes):
            offsets.append(len(flat))
            flat.extend(s)
            flat.extend([0] * (_pad4(max(1, n)) - n))
        self.host[:total] = torch.tensor(flat, dtype=torch.int32)
        self.dev[:total].copy_(self.host[:total])
        return [self.dev[o : o + max(1, n)] for o, n in zip(offsets, sizes)]


class Engine:
    """A model bound to a device, its cache and its step function."""

    def __init__(self, model: DecoderModel, env: BuildEnv, max_tokens: int, max_slots: int = 256) -> None:
        self.model = model
        self.env = env
        self.kernels = env.kernels
        self.device = env.device
        self.dtype = env.dtype
        self.vocab_size = model.spec.vocab_size
        self.cache = CacheManager(model.cache_needs(), max_tokens, max_slots, env.dtype, env.device)
        self.ws = Workspace(env.device)
        self.meta = StepMeta(env.device)
        self.stream = torch.cuda.Stream(device=env.device) if env.device.type == "cuda" else None
        self.steps_run = 0
        #: whether every part only launches library kernels (then decoding steps can be captured)
        self.graph_safe = all(getattr(b, "graph_safe", False) for b in model.blocks)

    # ---- sequences ---------------------------------------------------------------------
    def new_sequence(self) -> int:
        """Takes a free slot (its length is 0 and its fixed-size state is cleared)."""
        return self.cache.acquire()

    def release(self, slot: int) -> None:
        """Gives the slot and everything it holds back."""
        self.cache.release(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    # ---- the step --------------------------------------------------------------------------
    def _validate(self, entries: Sequence[StepEntry]) -> None:
        if not entries:
            raise ValueError("a step needs at least one sequence")
        seen = set()
        for e in entries:
            if e.slot in seen:
                raise ValueError(f"slot {e.slot} appears twice in one step")
            seen.add(e.slot)
            self.cache.length(e.slot)  # raises if the slot is not in use
            if len(e.tokens) == 0:
                raise ValueError(f"slot {e.slot}: a step entry needs at least one token")
            for t in e.tokens:
                if not 0 <= int(t) < self.vocab_size:
                    raise ValueError(f"slot {e.slot}: token id {t} is outside the vocabulary [0, {self.vocab_size})")
            for w in e.want:
                if not 0 <= int(w) < len(e.tokens):
                    raise ValueError(f"slot {e.slot}: wanted place {w} is outside its {len(e.tokens)} tokens")

    def run_on_stream(self, fn):
        """Runs fn() with the engine's stream current, ordered after what the caller has queued and
        before what it queues next."""
        if self.stream is None:
            return fn()
        self.stream.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(self.stream):
            self.kernels.use_stream(self.stream)
            try:
                out = fn()
            finally:
                self.kernels.use_stream(None)
        torch.cuda.current_stream(self.device).wait_stream(self.stream)
        return out

    def step(self, entries: Sequence[StepEntry], observe=None) -> Optional[torch.Tensor]:
        """Runs the entries' tokens; returns float32 logits [wanted, vocab] in the order of the
        entries and of each entry's `want` (None if nothing is wanted).  `observe(name, x, pending)`, for
        debugging, sees the residual stream after the embedding and after every run of the schedule."""
        self._validate(entries)
        return self.run_on_stream(lambda: self._step(entries, observe))

    def _step(self, entries: Sequence[StepEntry], observe=None) -> Optional[torch.Tensor]:
        cache = self.cache
        growth = {e.slot: len(e.tokens) for e in entries}
        cache.reserve(growth)  # CacheFull leaves everything as it was

        tokens: List[int] = []
        row_seq: List[int] = []
        row_pos: List[int] = []
        want_rows: List[int] = []
        slots, starts, lens, cu = [], [], [], [0]
        for b, e in enumerate(entries):
            n0 = cache.length(e.slot)
            n = len(e.tokens)
            base = len(tokens)
            tokens.extend(int(t) for t in e.tokens)
            row_seq.extend([b] * n)
            row_pos.extend(range(n0, n0 + n))
            want_rows.extend(base + int(w) for w in e.want)
            slots.append(e.slot)
            starts.append(n0)
            lens.append(n0 + n)
            cu.append(len(tokens))
        d_tokens, d_row_seq, d_row_pos, d_slot, d_start, d_len, d_cu, d_want = self.meta.upload(
            [tokens, row_seq, row_pos, slots, starts, lens, cu, want_rows])

        self.ws.reset()
        ctx = StepContext(
            kernels=self.kernels, dtype=self.dtype, device=self.device, ws=self.ws,
            rows=len(tokens), batch=len(entries), tokens=d_tokens, row_seq=d_row_seq, row_pos=d_row_pos,
            seq_slot=d_slot, seq_start=d_start, seq_len=d_len, cu_rows=d_cu,
            host_slots=slots, host_start=starts, host_new=[len(e.tokens) for e in entries],
            max_new=max(len(e.tokens) for e in entries), max_len=max(lens),
            decode=all(len(e.tokens) == 1 for e in entries), observe=observe,
        )
        logits = self.model.forward(ctx, cache.layer_views(), d_want, len(want_rows))
        cache.advance(growth)
        self.steps_run += 1
        return logits
