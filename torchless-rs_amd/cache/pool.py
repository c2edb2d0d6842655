"""Free lists that refuse misuse: the page pool and the slot table.

The reference has one cache per sequence and re-uses it by setting `pos = 0`
(src/model/mod.rs:235-238); its batching sketch keeps a deque of free blocks,
taken from the front and given back at the end (src/model/batching.rs:190,
227-234, 549-555).  Here ids are handed out from a free list, an id is never
held twice, and giving back an id that is not held is an error.  The lists
themselves live in the host library (csrc/host/books.cpp); the pages' list
there starts in a fixed shuffled order, so that a sequence's pages lie
scattered over the pool.
"""
from __future__ import annotations

import ctypes

from . import native
from .native import CacheFull, CacheMisuse      # noqa: F401  (this module is where callers look for them)


class FreeList:
    """Ids 0..n-1.  `take` returns the id that was given back last (so that a
    freed id is used again at once and re-use is exercised), else the lowest
    id that was never taken."""

    def __init__(self, n: int, what: str):
        self.n = int(n)
        self.what = what
        self._h = ctypes.c_void_p(native.lib().tl_freelist_new(self.n, what.encode()))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            native.lib().tl_freelist_delete(h)

    @property
    def n_free(self) -> int:
        return native.lib().tl_freelist_n_free(self._h)

    @property
    def n_held(self) -> int:
        return self.n - self.n_free

    def holds(self, i: int) -> bool:
        return bool(native.lib().tl_freelist_holds(self._h, int(i)))

    def take(self) -> int:
        out = ctypes.c_int(-1)
        native.check(native.lib().tl_freelist_take(self._h, ctypes.byref(out)))
        return out.value

    def give_back(self, i: int) -> None:
        native.check(native.lib().tl_freelist_give_back(self._h, int(i)))

    def check(self) -> None:
        """Every id is either free or held, exactly once."""
        native.check(native.lib().tl_freelist_check(self._h))
