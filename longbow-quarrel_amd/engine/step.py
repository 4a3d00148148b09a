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
vocabulary: internal/engine/engine.go:1300-1331), and refuses a position at or past
the length its cache was made for (internal/engine/kv_cache.go:121-124); here that
length is `max_sequence_tokens`: the caller's explicit figure if there is one, else
what the configuration allows (the reference sizes its cache in that order too:
internal/engine/kv_cache_sliding_window.go:38-60).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache import CacheManager
from ..model import DecoderModel
from ..parts.base import BuildEnv, StepContext, Workspace


class SequenceTooLong(ValueError):
    """A step would take a sequence past `Engine.max_sequence_tokens`."""


@dataclass
class StepEntry:
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()  # indices into `tokens` whose logits are asked for


def _pad4(n: int) -> int:
    return (n + 3) // 4 * 4


class StepMeta:
    """Packs a step's integer arrays into one pinned host buffer and one upload.  Two host buffers take
    turns, each with an event behind its copy, so that the upload does not wait for the device and a
    buffer is not written again before its last copy has been taken."""

    def __init__(self, device: torch.device) -> None:
        self.device = device
        self.cap = 0
        self.hosts: List[torch.Tensor] = []
        self.events: List[Optional["torch.cuda.Event"]] = [None, None]
        self.turn = 0
        self.dev: Optional[torch.Tensor] = None

    def _grow(self, n: int) -> None:
        if n <= self.cap:
            return
        self.cap = max(1024, int(n * 1.5))
        pin = self.device.type == "cuda"
        for ev in self.events:
            if ev is not None:
                ev.synchronize()
        self.events = [None, None]
        self.hosts = [torch.empty(self.cap, dtype=torch.int32, pin_memory=pin) for _ in range(2)]
        self.dev = torch.empty(self.cap, dtype=torch.int32, device=self.device)

    def upload(self, sections: Sequence[np.ndarray]) -> List[torch.Tensor]:
        """`sections`: integer arrays; each gets a run of the device buffer (16-byte aligned, at least
        one entry long).  -> the device views, in order."""
        sizes = [int(s.size) for s in sections]
        offsets, total = [], 0
        for n in sizes:
            offsets.append(total)
            total += _pad4(max(1, n))
        self._grow(total)
        self.turn ^= 1
        if self.events[self.turn] is not None:
            self.events[self.turn].synchronize()
        host = self.hosts[self.turn]
        flat = host.numpy()
        for s, o, n in zip(sections, offsets, sizes):
            flat[o : o + n] = s
            flat[o + n : o + _pad4(max(1, n))] = 0
        if self.device.type == "cuda":
            self.dev[:total].copy_(host[:total], non_blocking=True)
            ev = torch.cuda.Event()
            ev.record()
            self.events[self.turn] = ev
        else:
            self.dev[:total].copy_(host[:total])
        return [self.dev[o : o + max(1, n)] for o, n in zip(offsets, sizes)]


class Engine:
    """A model bound to a device, its cache and its step function."""

    def __init__(self, model: DecoderModel, env: BuildEnv, max_tokens: int, max_slots: int = 256,
                 max_sequence_tokens: Optional[int] = None) -> None:
        """`max_tokens` sizes the cache's pool (all live sequences together); `max_sequence_tokens` bounds
        one sequence (default: the longest the model's configuration allows; None there: the pool)."""
        self.model = model
        self.env = env
        self.kernels = env.kernels
        self.device = env.device
        prepare = getattr(env.kernels, "prepare", None)
        if prepare is not None:
            prepare(env.device)
        self.dtype = env.dtype
        self.vocab_size = model.spec.vocab_size
        self.cache = CacheManager(model.cache_needs(), max_tokens, max_slots, env.dtype, env.device)
        if max_sequence_tokens is None:
            max_sequence_tokens = model.spec.max_positions
        if max_sequence_tokens is not None and max_sequence_tokens <= 0:
            raise ValueError(f"max_sequence_tokens must be positive, found {max_sequence_tokens}")
        self.max_sequence_tokens: Optional[int] = max_sequence_tokens
        self.ws = Workspace(env.device)
        self.meta = StepMeta(env.device)
        self.stream = torch.cuda.Stream(device=env.device) if env.device.type == "cuda" else None
        self.steps_run = 0
        #: whether every part only launches library kernels (then decoding steps can be captured)
        self.graph_safe = model.graph_safe

    # ---- sequences ---------------------------------------------------------------------
    def new_sequence(self) -> int:
        """Takes a free slot (its length is 0 and its fixed-size state is cleared)."""
        return self.cache.acquire()

    def release(self, slot: int) -> None:
        """Gives the slot and everything it holds back."""
        self.cache.release(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    # ---- what a decoding step's launches depend on beside its batch size ----------------------
    def length_bound(self, longest: int) -> int:
        """The bound of the lengths that a decoding step is shaped for when its longest sequence holds
        `longest` tokens (the mixers' answer: `Mixer.length_bound`)."""
        return self.model.length_bound(self.kernels, longest)

    def lengths_uneven(self, lengths: Sequence[int]) -> bool:
        """Whether a decoding step with these lengths is to be marked `uneven` (the mixers' answer:
        `Mixer.lengths_uneven`); asked here for direct and for captured steps alike, so that both sum
        in the same order."""
        return self.model.lengths_uneven(self.kernels, lengths)

    # ---- the step --------------------------------------------------------------------------
    def _validate(self, entries: Sequence[StepEntry]) -> List[np.ndarray]:
        """Refuses a step that cannot run, before anything changes.  -> each entry's tokens as an array."""
        if not entries:
            raise ValueError("a step needs at least one sequence")
        seen = set()
        arrays: List[np.ndarray] = []
        for e in entries:
            if e.slot in seen:
                raise ValueError(f"slot {e.slot} appears twice in one step")
            seen.add(e.slot)
            held = self.cache.length(e.slot)  # raises if the slot is not in use
            try:
                t = np.asarray(e.tokens, dtype=np.int64).reshape(-1)
            except (TypeError, ValueError, OverflowError):
                raise ValueError(f"slot {e.slot}: token ids must be integers") from None
            if t.size == 0:
                raise ValueError(f"slot {e.slot}: a step entry needs at least one token")
            self.check_room(e.slot, held, int(t.size))
            low, high = int(t.min()), int(t.max())
            if low < 0 or high >= self.vocab_size:
                bad = low if low < 0 else high
                raise ValueError(f"slot {e.slot}: token id {bad} is outside the vocabulary [0, {self.vocab_size})")
            for w in e.want:
                if not 0 <= int(w) < t.size:
                    raise ValueError(f"slot {e.slot}: wanted place {w} is outside its {t.size} tokens")
            arrays.append(t)
        return arrays

    def check_room(self, slot: int, held: int, new: int) -> None:
        limit = self.max_sequence_tokens
        if limit is not None and held + new > limit:
            raise SequenceTooLong(f"slot {slot}: {held} tokens held and {new} more would pass the "
                                  f"{limit} tokens a sequence may have (max_sequence_tokens)")

    def run_on_stream(self, fn, handshake: bool = True):
        """Runs fn() with the engine's stream current, ordered after what the caller has queued and
        before what it queues next.  Without `handshake` the two waits between the caller's stream and
        the engine's are left out: for work that follows other work on the engine's stream and whose
        results the host waits for itself (a wait on each side of every replayed step keeps the device
        idle for a tenth of a millisecond a step)."""
        if self.stream is None:
            return fn()
        if handshake:
            self.stream.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(self.stream):
            self.kernels.use_stream(self.stream)
            try:
                out = fn()
            finally:
                self.kernels.use_stream(None)
        if handshake:
            torch.cuda.current_stream(self.device).wait_stream(self.stream)
        return out

    def step(self, entries: Sequence[StepEntry], observe=None) -> Optional[torch.Tensor]:
        """Runs the entries' tokens; returns float32 logits [wanted, vocab] in the order of the
        entries and of each entry's `want` (None if nothing is wanted).  `observe(name, x, pending)`, for
        debugging, sees the residual stream after the embedding and after every run of the schedule."""
        arrays = self._validate(entries)
        return self.run_on_stream(lambda: self._step(entries, arrays, observe))

    def make_context(self, ws: Workspace, arrays: Sequence[torch.Tensor], slots: Sequence[int],
                     starts: Sequence[int], new: Sequence[int], max_len: int, logits_out=None, observe=None,
                     kernels=None, dry: bool = False, uneven: bool = False, want_all: bool = False) -> StepContext:
        """The one place where a step's `StepContext` is put together, for direct and for captured steps.
        `arrays`: the device arrays tokens, row_seq, row_pos, seq_slot, seq_start, seq_len, cu_rows;
        `slots`, `starts`, `new`: per sequence, on the host (`starts` may be empty where the lengths
        live on the device only, as in a captured step); `max_len`: an upper bound of the lengths after
        the step; `uneven`: whether a decoding step's sequences differ much in length (`Engine.lengths_uneven`);
        `want_all`: the logits of all the step's rows are wanted, in the rows' order."""
        tokens, row_seq, row_pos, seq_slot, seq_start, seq_len, cu_rows = arrays
        return StepContext(
            kernels=kernels if kernels is not None else self.kernels, dtype=self.dtype, device=self.device, ws=ws,
            rows=sum(new), batch=len(new), tokens=tokens, row_seq=row_seq, row_pos=row_pos, seq_slot=seq_slot,
            seq_start=seq_start, seq_len=seq_len, cu_rows=cu_rows, host_slots=list(slots), host_start=list(starts),
            host_new=list(new), max_new=max(new), max_len=max_len, decode=all(n == 1 for n in new),
            logits_out=logits_out, observe=observe, dry=dry, uneven=uneven and all(n == 1 for n in new),
            want_all=want_all)

    def forward(self, ctx: StepContext, want_rows: torch.Tensor, n_want: int) -> Optional[torch.Tensor]:
        """The model over one step's rows, from this engine's cache."""
        return self.model.forward(ctx, self.cache.layer_views(), want_rows, n_want)

    def _step(self, entries: Sequence[StepEntry], arrays: Sequence[np.ndarray], observe=None) -> Optional[torch.Tensor]:
        cache = self.cache
        new = [int(a.size) for a in arrays]
        growth = {e.slot: n for e, n in zip(entries, new)}
        cache.reserve(growth)  # CacheFull leaves everything as it was

        # the step's arrays, whole vectors at a time: no work per token on the host
        batch = len(entries)
        slots = [e.slot for e in entries]
        starts = [cache.length(s) for s in slots]
        counts = np.asarray(new, dtype=np.int64)
        cu = np.zeros(batch + 1, dtype=np.int64)
        np.cumsum(counts, out=cu[1:])
        rows = int(cu[-1])
        first = np.asarray(starts, dtype=np.int64)
        row_seq = np.repeat(np.arange(batch, dtype=np.int64), counts)
        row_pos = np.arange(rows, dtype=np.int64) + np.repeat(first - cu[:-1], counts)
        tokens = arrays[0] if batch == 1 else np.concatenate(arrays)
        want_rows = np.asarray([int(cu[b]) + int(w) for b, e in enumerate(entries) for w in e.want], dtype=np.int64)
        lens = [a + n for a, n in zip(starts, new)]
        d_tokens, d_row_seq, d_row_pos, d_slot, d_start, d_len, d_cu, d_want = self.meta.upload(
            [tokens, row_seq, row_pos, np.asarray(slots), first, np.asarray(lens), cu, want_rows])

        self.ws.reset()
        ctx = self.make_context(self.ws, (d_tokens, d_row_seq, d_row_pos, d_slot, d_start, d_len, d_cu), slots,
                                starts, new, max(lens), observe=observe, uneven=self.lengths_uneven(lens),
                                want_all=want_rows.size == rows and bool((want_rows == np.arange(rows)).all()))
        logits = self.forward(ctx, d_want, int(want_rows.size))
        cache.advance(growth)
        self.steps_run += 1
        return logits
