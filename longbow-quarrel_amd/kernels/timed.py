"""Per-operation device times, measured with HIP events around every kernel call.

`TimedKernels(real)` stands in for a kernel object: every method that launches is bracketed by two
events on the stream it launches on, and `report()` adds the elapsed times up by operation.  The
reference keeps wall clocks per operation of its layer loop in the same way
(internal/device/metal.go:1348-1355).  Steps have to run directly for this (a captured step is one
launch for the host); `bench.py --profile` does that.  Times include the gap that the event pair itself
adds around a kernel (a few microseconds), so they are for comparing operations with each other; a
profiler's kernel trace gives the kernels' own durations.
"""
from __future__ import annotations

from typing import Any, Dict, List, Tuple

import torch

#: methods that do not launch a kernel of their own (plumbing, captures, allocations)
_UNTIMED = {"use_stream", "prepare", "tickets", "graph_begin", "graph_end", "graph_launch", "graph_destroy",
            "interleave_gate_up"}


class TimedKernels:
    def __init__(self, real: Any) -> None:
        self._real = real
        self._pending: List[Tuple[str, "torch.cuda.Event", "torch.cuda.Event"]] = []
        self._total: Dict[str, List[float]] = {}  # operation -> [calls, milliseconds]

    def __getattr__(self, name: str):
        attr = getattr(self._real, name)
        if not callable(attr) or getattr(attr, "is_query", False) or name in _UNTIMED or name.startswith("_"):
            return attr

        def timed(*args, **kwargs):
            # (the stream that the call launches on is the current one: `Engine.run_on_stream` makes it so)
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            try:
                return attr(*args, **kwargs)
            finally:
                end.record()
                self._pending.append((self._label(name, args), start, end))

        return timed

    @staticmethod
    def _label(name: str, args) -> str:
        """The operation, and for products their sizes (rows x columns x K), which is what tells a layer's
        products apart."""
        if name.startswith("linear"):
            x = args[0]
            w = args[3] if name == "linear_scaled" else args[1]
            return f"{name} {x.shape[0]} x {w.shape[0]} x {w.shape[1]}"
        return name

    def reset(self) -> None:
        torch.cuda.synchronize()
        self._pending.clear()
        self._total.clear()

    def report(self) -> Dict[str, Tuple[int, float]]:
        """operation -> (calls, milliseconds in all), waiting for what is still queued."""
        torch.cuda.synchronize()
        for label, start, end in self._pending:
            t = self._total.setdefault(label, [0, 0.0])
            t[0] += 1
            t[1] += start.elapsed_time(end)
        self._pending.clear()
        return {k: (int(v[0]), v[1]) for k, v in sorted(self._total.items(), key=lambda kv: -kv[1][1])}
