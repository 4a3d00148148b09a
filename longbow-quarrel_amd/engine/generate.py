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

`GenerationLoop` holds the decisions only and talks to a backend with five
methods, so that the decisions can be tested without a GPU; `EngineBackend` is the
real one.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence

import torch

from ..cache import BLOCK_SIZE, CacheFull
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from ..sampling.state import SamplerState, sequence_key
from .decode import LEN_BUCKET, DecodeGraph
from .step import Engine, StepEntry


@dataclass
class GenerationResult:
    tokens: List[List[int]]  # generated ids per request, in the order of the prompts (prompts not included)
    finish: List[str]  # "stop" | "length" for each request
    prefill_seconds: float = 0.0
    decode_seconds: float = 0.0
    prefill_tokens: int = 0
    decode_steps: int = 0
    batches: int = 0


class GenerationLoop:
    """Which requests run together, when a sequence ends, what is returned."""

    def __init__(self, backend, max_batch: int = 64) -> None:
        if max_batch <= 0:
            raise ValueError("max_batch must be positive")
        self.backend = backend
        self.max_batch = max_batch

    def _next_batch(self, pending: List[int], prompts: Sequence[Sequence[int]], max_new: int) -> List[int]:
        """The longest prefix of the pending requests that fits the batch size and the cache."""
        budget = self.backend.free_blocks()
        chosen: List[int] = []
        for r in pending:
            need = self.backend.blocks_needed(len(prompts[r]) + max_new)
            if len(chosen) >= self.max_batch or need > budget:
                break
            chosen.append(r)
            budget -= need
        if not chosen:
            r = pending[0]
            raise CacheFull(
                f"request {r} needs room for {len(prompts[r]) + max_new} tokens, more than the cache can hold")
        return chosen

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
        pending = list(range(n))
        be = self.backend
        while pending:
            batch = self._next_batch(pending, prompts, max_new_tokens)
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
                t0 = time.perf_counter()
                while True:
                    survivors: List[int] = []
                    for r, tok in zip(live, sampled):
                        tok = int(tok)
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
                        if len(result.tokens[r]) >= max_new_tokens:
                            result.finish[r] = "length"
                            be.release(slots.pop(r))
                            continue
                        survivors.append(r)
                    if not survivors:
                        break
                    changed = survivors != live
                    live = survivors
                    sampled = be.decode([slots[r] for r in live],
                                        [result.tokens[r][-1] for r in live], changed)
                    result.decode_steps += 1
                result.decode_seconds += time.perf_counter() - t0
            finally:
                for s in slots.values():
                    be.release(s)
        return result


class EngineBackend:
    """Drives an `Engine` for the loop: prompts through `Engine.step`, single-token steps through
    captured graphs (or through `Engine.step` when graphs are off), sampling on the device."""

    def __init__(self, engine: Engine, params: SamplingParams, use_graphs: bool = True) -> None:
        self.engine = engine
        self.params = params
        if not hasattr(engine, "sampler_state"):
            engine.sampler_state = SamplerState(engine.cache.max_slots, engine.device)
        self.sampler = Sampler(engine.kernels, engine.sampler_state, params)
        self.use_graphs = use_graphs and engine.device.type == "cuda" and engine.graph_safe
        self.graphs: Dict[tuple, DecodeGraph] = {}
        self.current: Optional[DecodeGraph] = None
        self.keep_logits = False  # direct steps only: a copy of each step's logits before sampling changes them
        self.last_logits: Optional[torch.Tensor] = None

    # ---- what the loop asks ------------------------------------------------------------
    def free_blocks(self) -> int:
        return min((g.blocks.free_count for g in self.engine.cache.kv_groups), default=1 << 30)

    def blocks_needed(self, tokens: int) -> int:
        return (tokens + BLOCK_SIZE - 1) // BLOCK_SIZE

    def new_sequence(self, request_index: int, prompt: Sequence[int]) -> int:
        slot = self.engine.new_sequence()
        self.engine.sampler_state.start(slot, sequence_key(self.params.seed, request_index), prompt)
        return slot

    def release(self, slot: int) -> None:
        self.engine.release(slot)

    def prefill(self, slots: Sequence[int], prompts: Sequence[Sequence[int]]) -> List[int]:
        e = self.engine
        logits = e.step([StepEntry(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)])
        return self._sample_eager(logits, slots)

    def decode(self, slots: Sequence[int], last_tokens: Sequence[int], changed: bool) -> List[int]:
        e = self.engine
        if not self.use_graphs:
            logits = e.step([StepEntry(s, [t], [0]) for s, t in zip(slots, last_tokens)])
            return self._sample_eager(logits, slots)
        return e.run_on_stream(lambda: self._decode_graph(list(slots), list(last_tokens), changed))

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

    def _decode_graph(self, slots: List[int], last_tokens: List[int], changed: bool) -> List[int]:
        e = self.engine
        cache = e.cache
        starts = [cache.length(s) for s in slots]
        growth = {s: 1 for s in slots}
        cache.reserve(growth)
        longest = max(starts) + 1
        bound = (longest + LEN_BUCKET - 1) // LEN_BUCKET * LEN_BUCKET
        key = (len(slots), bound)
        g = self.graphs.get(key)
        fresh = g is None
        if fresh:
            g = DecodeGraph(e, len(slots), bound)
            self.graphs[key] = g
        if fresh or changed or g is not self.current or g.slots != slots:
            g.load(slots, last_tokens, starts)
        if fresh:
            g.capture(self.sampler)
        self.current = g
        g.launch()
        cache.advance(growth)
        e.steps_run += 1
        return g.views[0].cpu().tolist()

    def close(self) -> None:
        for g in self.graphs.values():
            g.destroy()
        self.graphs.clear()


def generate(engine: Engine, prompts: Sequence[Sequence[int]], max_new_tokens: int,
             params: Optional[SamplingParams] = None, stop_ids: Optional[Sequence[int]] = None,
             include_stop: bool = False, max_batch: int = 64, use_graphs: bool = True,
             callback: Optional[Callable[[int, int], None]] = None) -> GenerationResult:
    """Generates up to `max_new_tokens` ids for every prompt.  `stop_ids` defaults to the
    configuration's end-of-sequence ids."""
    params = params or SamplingParams()
    if stop_ids is None:
        stop_ids = tuple(engine.model.spec.stop_ids)
    backend = EngineBackend(engine, params, use_graphs=use_graphs)
    try:
        return GenerationLoop(backend, max_batch=max_batch).run(prompts, max_new_tokens, stop_ids,
                                                                include_stop, callback)
    finally:
        backend.close()
