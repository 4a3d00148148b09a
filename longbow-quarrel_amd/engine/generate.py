"""The generation loop above the step function.

Requests are served in batches of sequences that start together: a batch's
prompts, of unequal lengths, run in one step; then every live sequence advances
by one token a step.  A sequence ends on a stop token or at its token limit, leaves
the batch and gives its slot back; the others go on with a smaller batch.  When a
batch is done the next requests form the next batch on the same slots.

The reference's loop is the single-sequence form of this (prefill, first token from
the last prompt position, then count-1 decode iterations, stop on the end-of-text
id, generated ids only: internal/engine/engine.go:1504-1600, 1611-1772).  Two of
its habits are not kept: the stop id is hard-coded and the first sampled token is
never checked against it (:1744-1747); here stop ids come from the configuration
or the caller and every sampled token is checked.

`GenerationLoop` holds the decisions only and talks to a backend with a handful of
methods, so that the decisions can be tested without a GPU; `EngineBackend` is the
real one.  It feeds a batch's prompts in portions of at most `max_prefill_rows` rows
(the step's workspace grows with its rows, not with the batch).  A row of logits that holds a
NaN or an infinity is not sampled from, where the reference takes the first finite index
(internal/engine/sampler.go:72-75, 107-123): that request ends there (finish "error"), the
others of its batch and the batches after it run to their ends, and then the call raises
`NonFiniteLogits`, which names the requests and carries everybody's tokens as `result`.  Replayed decoding steps
are queued one ahead of the host (`_Launched`, `EngineBackend.ahead`): the device goes from one
step to the next without waiting for the loop's decisions, which arrive a step late and are
applied to the step that is already there.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence

import torch

from ..cache import BLOCK_SIZE, CacheFull
from ..sampling.params import SamplingParams
from ..sampling.sampler import NonFiniteLogits, Sampler
from ..sampling.state import RECENT, SamplerState, sequence_key
from .decode import DecodeGraphs
from .step import Engine, SequenceTooLong, StepEntry


@dataclass
class GenerationResult:
    tokens: List[List[int]]  # generated ids per request, in the order of the prompts (prompts not included)
    finish: List[str]  # "stop" | "length" for each request ("error": its logits held a NaN or an infinity)
    prefill_seconds: float = 0.0
    decode_seconds: float = 0.0
    prefill_tokens: int = 0
    decode_steps: int = 0
    batches: int = 0


class _Launched:
    """A decoding step that has been queued: its sequences, and its sampled tokens once they are asked
    for.  On the GPU the tokens are copied to pinned host memory behind the step, with an event after the
    copy, so that reading them waits for this step only and not for what was queued after it."""

    def __init__(self, slots: List[int], device_tokens: torch.Tensor, host: Optional[torch.Tensor]) -> None:
        self.slots = slots
        n = len(slots)
        if host is None:
            self.host = device_tokens[:n].clone()
            self.event = None
        else:
            self.host = host[:n]
            self.host.copy_(device_tokens[:n], non_blocking=True)
            self.event = torch.cuda.Event()
            self.event.record()

    def wait(self) -> None:
        if self.event is not None:
            self.event.synchronize()
            self.event = None

    def tokens(self, slots: List[int]) -> List[int]:
        """The tokens of `slots`, all or some of the step's sequences, in that order."""
        self.wait()
        got = self.host.tolist()
        if slots == self.slots:
            return got
        at = {s: i for i, s in enumerate(self.slots)}
        return [got[at[s]] for s in slots]


class GenerationLoop:
    """Which requests run together, when a sequence ends, what is returned."""

    def __init__(self, backend, max_batch: int = 64) -> None:
        if max_batch <= 0:
            raise ValueError("max_batch must be positive")
        self.backend = backend
        self.max_batch = max_batch

    def _next_batch(self, pending: List[int], prompts: Sequence[Sequence[int]], limit: Sequence[int]) -> List[int]:
        """The longest prefix of the pending requests that fits the batch size and the cache.  A request
        caches its prompt and every token it is given but the last, which is sampled and never fed back."""
        budget = self.backend.free_blocks()
        chosen: List[int] = []
        for r in pending:
            need = self.backend.blocks_needed(self._cached_tokens(prompts[r], limit[r]))
            if len(chosen) >= self.max_batch or need > budget:
                break
            chosen.append(r)
            budget -= need
        if not chosen:
            r = pending[0]
            raise CacheFull(f"request {r} needs room for {self._cached_tokens(prompts[r], limit[r])} tokens, "
                            "more than the cache can hold")
        return chosen

    @staticmethod
    def _cached_tokens(prompt: Sequence[int], limit: int) -> int:
        return len(prompt) + max(limit, 1) - 1

    def _token_limits(self, prompts: Sequence[Sequence[int]], max_new_tokens: int) -> List[int]:
        """How many tokens each request may get: `max_new_tokens`, or fewer where the sequence would
        pass the length a sequence may have (the last sampled token is never fed back, so a sequence
        that holds n tokens has produced n - prompt + 1)."""
        room = getattr(self.backend, "token_room", None)
        limits = []
        for r, p in enumerate(prompts):
            k = room(len(p)) if room is not None else None
            if k is not None and k <= 0:
                raise SequenceTooLong(f"request {r}: its prompt of {len(p)} tokens is longer than a sequence may be")
            limits.append(max_new_tokens if k is None else min(max_new_tokens, k))
        return limits

    def run(self, prompts: Sequence[Sequence[int]], max_new_tokens: int, stop_ids: Sequence[int] = (),
            include_stop: bool = False, callback: Optional[Callable[[int, int], None]] = None) -> GenerationResult:
        for r, p in enumerate(prompts):
            if len(p) == 0:
                raise ValueError(f"request {r}: empty prompt")  # internal/engine/engine.go:1300-1303
        stops = set(int(s) for s in stop_ids)
        n = len(prompts)
        result = GenerationResult(tokens=[[] for _ in range(n)], finish=["length"] * n)
        if max_new_tokens <= 0 or n == 0:
            return result
        limit = self._token_limits(prompts, max_new_tokens)
        pending = list(range(n))
        be = self.backend
        faulty: List[str] = []
        while pending:
            batch = self._next_batch(pending, prompts, limit)
            pending = pending[len(batch):]
            result.batches += 1
            slots: Dict[int, int] = {}
            try:
                for r in batch:
                    slots[r] = be.new_sequence(r, prompts[r])
                t0 = time.perf_counter()
                sampled = be.prefill([slots[r] for r in batch], [prompts[r] for r in batch])
                result.prefill_seconds += time.perf_counter() - t0
                result.prefill_tokens += sum(len(prompts[r]) for r in batch)
                live = list(batch)
                first = True  # a batch's first decoding step always brings new sequences
                t0 = time.perf_counter()
                while True:
                    survivors: List[int] = []
                    for r, tok in zip(live, sampled):
                        tok = int(tok)
                        if tok < 0:  # no token: the row's logits were not finite
                            result.finish[r] = "error"
                            faulty.append(f"request {r} (slot {slots[r]})")
                            be.release(slots.pop(r))
                            continue
                        if tok in stops:
                            result.finish[r] = "stop"
                            if include_stop:
                                result.tokens[r].append(tok)
                                if callback:
                                    callback(r, tok)
                            be.release(slots.pop(r))
                            continue
                        result.tokens[r].append(tok)
                        if callback:
                            callback(r, tok)
                        if len(result.tokens[r]) >= limit[r]:
                            result.finish[r] = "length"
                            be.release(slots.pop(r))
                            continue
                        survivors.append(r)
                    if not survivors:
                        break
                    changed = first or survivors != live
                    first = False
                    live = survivors
                    # whether a step can follow this one, whatever it samples (a backend may run ahead then)
                    expect = getattr(be, "expect_more", None)
                    if expect is not None:
                        expect(any(len(result.tokens[r]) + 1 < limit[r] for r in live))
                    sampled = be.decode([slots[r] for r in live],
                                        [result.tokens[r][-1] for r in live], changed)
                    result.decode_steps += 1
                result.decode_seconds += time.perf_counter() - t0
            finally:
                for s in slots.values():
                    be.release(s)
        if faulty:
            raise NonFiniteLogits(f"the logits of {', '.join(faulty)} hold a NaN or an infinity; nothing was sampled "
                                  "from them (the other requests ran on: see .result)", result)
        return result


class EngineBackend:
    """Drives an `Engine` for the loop: prompts through `Engine.step`, single-token steps through
    captured graphs (or through `Engine.step` when graphs are off), sampling on the device."""

    def __init__(self, engine: Engine, params: SamplingParams, use_graphs: bool = True,
                 max_prefill_rows: int = 8192, graphs_cls=DecodeGraphs) -> None:
        if max_prefill_rows <= 0:
            raise ValueError("max_prefill_rows must be positive")
        self.engine = engine
        self.params = params
        self.max_prefill_rows = int(max_prefill_rows)
        if not hasattr(engine, "sampler_state"):
            engine.sampler_state = SamplerState(engine.cache.max_slots, engine.device,
                                                window=getattr(engine.kernels, "penalty_window", RECENT))
        self.sampler = Sampler(engine.kernels, engine.sampler_state, params)
        self.use_graphs = use_graphs and engine.graph_safe and \
            (engine.device.type == "cuda" or graphs_cls is not DecodeGraphs)
        self.graphs = graphs_cls(engine, self.sampler) if self.use_graphs else None
        self.current = None  # the graph whose arrays hold the live batch, as the last step left them
        # a copy of each step's logits: before sampling where steps run directly, as the sampler left them
        # (with the repetition penalty applied, if there is one) where they are replayed from a graph
        self.keep_logits = False
        self.last_logits: Optional[torch.Tensor] = None
        self.prefill_steps = 0
        # Running ahead: a replayed step takes its tokens from where the step before left them, on the
        # device, so the step after the one that the loop is asking for can be queued before the host has
        # seen any token: the device then never waits for the host between steps.  `ahead` is that step
        # (launched, not yet read); `more` is what the loop said about a step following (`expect_more`).
        self.run_ahead = True
        self.ahead: Optional[_Launched] = None
        self.more = True
        self.steps_ahead = 0  # steps that were queued before their turn (for tests and curiosity)
        self._token_buffers: List[torch.Tensor] = []

    # ---- what the loop asks ------------------------------------------------------------
    def free_blocks(self) -> int:
        return self.engine.cache.free_blocks()

    def blocks_needed(self, tokens: int) -> int:
        return self.engine.cache.blocks_for(tokens)

    def token_room(self, prompt_tokens: int) -> Optional[int]:
        """How many tokens a request with such a prompt can get before its sequence is as long as
        one may be (None: no bound)."""
        limit = self.engine.max_sequence_tokens
        return None if limit is None else limit - prompt_tokens + 1

    def expect_more(self, more: bool) -> None:
        """The loop's word on whether a step can follow the next `decode`, whatever it samples."""
        self.more = bool(more)

    def new_sequence(self, request_index: int, prompt: Sequence[int]) -> int:
        self._drop_ahead()
        slot = self.engine.new_sequence()
        self.engine.sampler_state.start(slot, sequence_key(self.params.seed, request_index), prompt)
        self.current = None  # whatever a graph's arrays hold is of an earlier batch
        return slot

    def release(self, slot: int) -> None:
        self.engine.release(slot)

    def prefill(self, slots: Sequence[int], prompts: Sequence[Sequence[int]]) -> List[int]:
        """Runs the prompts, in as many steps as `max_prefill_rows` asks for (a step takes the next
        tokens of as many sequences as fit, a long prompt goes on in the next step), and samples each
        sequence's first token from the logits at its last place."""
        e = self.engine
        self._drop_ahead()
        self.current = None
        rows_out: List[Optional[torch.Tensor]] = [None] * len(slots)
        at = [0] * len(slots)  # tokens of each prompt that have run
        steps = 0
        i = 0
        while i < len(slots):
            entries, owners, room = [], [], self.max_prefill_rows
            while i < len(slots) and room > 0:
                n = min(room, len(prompts[i]) - at[i])
                last = at[i] + n == len(prompts[i])
                entries.append(StepEntry(slots[i], prompts[i][at[i] : at[i] + n], [n - 1] if last else []))
                at[i] += n
                room -= n
                if not last:
                    break  # the step is full; this prompt goes on in the next one
                owners.append(i)
                i += 1
            logits = e.step(entries)
            steps += 1
            for k, owner in enumerate(owners):
                rows_out[owner] = logits[k : k + 1]
        self.prefill_steps += steps
        if steps > 1:
            logits = torch.cat(rows_out)  # each sequence's row, side by side for the sampler
        return self._sample_eager(logits, slots)

    def decode(self, slots: Sequence[int], last_tokens: Sequence[int], changed: bool) -> List[int]:
        e = self.engine
        if not self.use_graphs:
            logits = e.step([StepEntry(s, [t], [0]) for s, t in zip(slots, last_tokens)])
            return self._sample_eager(logits, slots)
        # A replayed step follows the prompt step or the step before it on the engine's stream, and the host
        # waits for its tokens before it does anything else with the sequences: no waits between streams.
        # (What is queued ahead is waited for in `_drop_ahead` before other work may touch its slots.)
        step = e.run_on_stream(lambda: self._decode_graph(list(slots), list(last_tokens), changed), handshake=False)
        return step.tokens(list(slots))  # (-1 where a row's logits were not finite: the loop ends that request)

    # ---- internals ------------------------------------------------------------------------
    def _sample_eager(self, logits: torch.Tensor, slots: Sequence[int]) -> List[int]:
        e = self.engine

        def body():
            if self.keep_logits:
                self.last_logits = logits.clone()
            seq_slot = torch.tensor(list(slots), dtype=torch.int32).to(e.device)
            out = torch.empty(len(slots), dtype=torch.int32, device=e.device)
            self.sampler.sample(logits, seq_slot, out)
            return out.cpu().tolist()

        return e.run_on_stream(body)

    def _decode_graph(self, slots: List[int], last_tokens: List[int], changed: bool) -> "_Launched":
        """The launched step whose tokens answer this call: the one queued ahead if it is the step asked
        for (the same sequences, or some of them: a step's results do not depend on who else was in it beyond
        rounding, so a survivor's tokens can differ from a run without steps ahead where two candidates tie),
        else a step launched now.  Queues the step after it while the device still works on this one."""
        step, self.ahead = self.ahead, None
        if step is not None and not (set(slots) <= set(step.slots)):
            step.wait()  # not what is asked for (the loop never does this): its tokens are dropped
            step = None
        if step is None:
            step = self._launch(slots, last_tokens, changed)
        elif step.slots != slots:
            self.current = None  # the batch shrank: its next step starts from arrays written anew
        if self.run_ahead and self.more and not self.keep_logits and step.slots == slots:
            self.ahead = self._launch_next(step)
        return step

    def _launch(self, slots: List[int], last_tokens: Optional[List[int]], changed: bool,
                same_graph=None) -> Optional["_Launched"]:
        """Queues one decoding step.  With `same_graph` (running ahead) only if that very graph takes the
        step as its arrays stand: None otherwise, and nothing has changed."""
        e = self.engine
        cache = e.cache
        starts = [cache.length(s) for s in slots]
        longest = max(starts) + 1
        bound = e.length_bound(longest)
        growth = {s: 1 for s in slots}
        uneven = e.lengths_uneven([n + 1 for n in starts])
        if same_graph is not None:
            if bound != same_graph.bound or uneven != same_graph.uneven:
                return None
            try:
                for s, n in zip(slots, starts):
                    e.check_room(s, n, 1)
                cache.reserve(growth)
            except (SequenceTooLong, CacheFull):
                return None  # the loop meets the same error when (and if) it asks for this step
            g = same_graph
        else:
            for s, n in zip(slots, starts):
                e.check_room(s, n, 1)
            cache.reserve(growth)
            g, fresh = self.graphs.get(len(slots), bound, uneven)
            # a graph's arrays carry on from its own last step only: anything else in between (another graph,
            # a prompt step, a batch whose members changed) means they are written anew
            if fresh or changed or g is not self.current or g.slots != slots:
                g.load(slots, last_tokens, starts)
            if fresh:
                g.capture(self.sampler)
        self.current = g
        g.launch()
        cache.advance(growth)
        e.steps_run += 1
        if self.keep_logits:
            self.last_logits = g.logits.clone()
        return _Launched(list(slots), g.views[0], self._token_buffer(len(slots)))

    def _launch_next(self, step: "_Launched") -> Optional["_Launched"]:
        nxt = self._launch(step.slots, None, False, same_graph=self.current)
        if nxt is not None:
            self.steps_ahead += 1
        return nxt

    def _token_buffer(self, n: int) -> Optional[torch.Tensor]:
        """Pinned host memory for a step's tokens; two buffers take turns (the step ahead and the one
        before it).  None off the GPU, where a copy is taken at once."""
        if self.engine.device.type != "cuda":
            return None
        if not self._token_buffers or self._token_buffers[0].numel() < n:
            self._token_buffers = [torch.empty(max(n, 64), dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self._token_buffers.reverse()
        return self._token_buffers[0]

    def _drop_ahead(self) -> None:
        """A step queued ahead that nobody will ask for (its batch ended, or other work comes first): it has
        run or will run before anything queued after it, and what it wrote belongs to slots that are
        given back or written anew."""
        if self.ahead is not None:
            self.ahead.wait()
            self.ahead = None
            self.current = None

    def close(self) -> None:
        self._drop_ahead()
        if self.graphs is not None:
            self.graphs.close()
        self.current = None


def generate(engine: Engine, prompts: Sequence[Sequence[int]], max_new_tokens: int,
             params: Optional[SamplingParams] = None, stop_ids: Optional[Sequence[int]] = None,
             include_stop: bool = False, max_batch: int = 64, use_graphs: bool = True,
             callback: Optional[Callable[[int, int], None]] = None, max_prefill_rows: int = 8192,
             extra_stop_ids: Sequence[int] = ()) -> GenerationResult:
    """Generates up to `max_new_tokens` ids for every prompt.  `stop_ids` defaults to the
    configuration's end-of-sequence ids (an explicit list stands in their place; `extra_stop_ids`
    are added to whichever it is)."""
    params = params or SamplingParams()
    if stop_ids is None:
        stop_ids = tuple(engine.model.spec.stop_ids)
    stop_ids = tuple(stop_ids) + tuple(extra_stop_ids)
    backend = EngineBackend(engine, params, use_graphs=use_graphs, max_prefill_rows=max_prefill_rows)
    try:
        return GenerationLoop(backend, max_batch=max_batch).run(prompts, max_new_tokens, stop_ids,
                                                                include_stop, callback)
    finally:
        backend.close()
