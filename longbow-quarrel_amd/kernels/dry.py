"""Walking through a step without launching anything, to learn how much workspace it needs.

A kernel object marks the methods that only answer a question about sizes or capabilities with
`@query`.  `DryKernels(real)` stands in for it during the walk: marked methods answer truthfully,
every other method does nothing, plain attributes pass through.  A part that launches kernels of its
own (not through the kernel object) looks at `ctx.dry` instead.
"""
from __future__ import annotations

from typing import Any, Callable


def query(fn: Callable) -> Callable:
    """Marks a method of a kernel object as a question about sizes or capabilities."""
    fn.is_query = True
    return fn


class DryKernels:
    def __init__(self, real: Any) -> None:
        self._real = real

    def __getattr__(self, name: str):
        attr = getattr(self._real, name)
        if getattr(attr, "is_query", False) or not callable(attr):
            return attr
        return lambda *args, **kwargs: None
