"""Free lists that refuse misuse: the page pool and the slot table.

The reference has one cache per sequence and re-uses it by setting `pos = 0`
(src/model/mod.rs:235-238); its batching sketch keeps a deque of free blocks,
taken from the front and given back at the end (src/model/batching.rs:190,
227-234, 549-555).  Here ids are handed out from a free list, an id is never
held twice, and giving back an id that is not held is an error.
"""
from __future__ import annotations

from typing import List


class CacheFull(RuntimeError):
    """No free page or slot is left."""


class CacheMisuse(RuntimeError):
    """An id was given back that is not held, or used while not held."""


class FreeList:
    """Ids 0..n-1.  `take` returns the id that was given back last (so that a
    freed id is used again at once and re-use is exercised), else the lowest
    id that was never taken."""

    def __init__(self, n: int, what: str):
        self.n = int(n)
        self.what = what
        self._free: List[int] = list(range(self.n - 1, -1, -1))
        self._held = [False] * self.n

    @property
    def n_free(self) -> int:
        return len(self._free)

    @property
    def n_held(self) -> int:
        return self.n - len(self._free)

    def holds(self, i: int) -> bool:
        return 0 <= i < self.n and self._held[i]

    def take(self) -> int:
        if not self._free:
            raise CacheFull(f"no free {self.what} (all {self.n} are held)")
        i = self._free.pop()
        assert not self._held[i]
        self._held[i] = True
        return i

    def give_back(self, i: int) -> None:
        if not (0 <= i < self.n):
            raise CacheMisuse(f"{self.what} {i} does not exist (there are {self.n})")
        if not self._held[i]:
            raise CacheMisuse(f"{self.what} {i} is given back but is not held")
        self._held[i] = False
        self._free.append(i)

    def check(self) -> None:
        """Every id is either free or held, exactly once."""
        assert len(set(self._free)) == len(self._free), f"{self.what}: an id is free twice"
        for i in self._free:
            assert not self._held[i], f"{self.what} {i} is both free and held"
        assert sum(self._held) + len(self._free) == self.n, f"{self.what}: an id is lost"
