"""Host-side bookkeeping of the cache: which slots and which blocks are free.

A slot stands for one live sequence; a block holds the keys and values of
BLOCK_SIZE consecutive positions.  Both come from free lists and go back to
them when a sequence ends.  Taking what is taken, or giving back what is free,
is an error: nothing is ever lost, held twice or freed twice.
"""
from __future__ import annotations

from typing import List

BLOCK_SIZE = 64


class CacheFull(RuntimeError):
    """No free slot or not enough free blocks."""


class FreeList:
    """Integers 0..n-1; lowest free id first, so reuse is immediate and predictable."""

    def __init__(self, n: int, what: str) -> None:
        self.n = int(n)
        self.what = what
        self._free: List[int] = list(range(self.n - 1, -1, -1))  # pop() gives the lowest
        self._taken = [False] * self.n

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def taken_count(self) -> int:
        return self.n - len(self._free)

    def is_taken(self, i: int) -> bool:
        return 0 <= i < self.n and self._taken[i]

    def take(self) -> int:
        if not self._free:
            raise CacheFull(f"no free {self.what} (all {self.n} are in use)")
        i = self._free.pop()
        self._taken[i] = True
        return i

    def take_many(self, count: int) -> List[int]:
        if count > len(self._free):
            raise CacheFull(f"{count} {self.what}s wanted, {len(self._free)} of {self.n} are free")
        return [self.take() for _ in range(count)]

    def give(self, i: int) -> None:
        if not 0 <= i < self.n:
            raise ValueError(f"{self.what} {i} does not exist (there are {self.n})")
        if not self._taken[i]:
            raise ValueError(f"{self.what} {i} is given back but is not in use")
        self._taken[i] = False
        self._free.append(i)
        # keep "lowest id first" cheaply: the list is small and mostly sorted
        if len(self._free) > 1 and self._free[-2] < i:
            self._free.sort(reverse=True)
