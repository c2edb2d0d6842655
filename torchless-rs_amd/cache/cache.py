"""The cache: a slot for each live sequence, pages of keys and values for each
group of layers, and per-sequence state of fixed size beside them.

The reference keeps keys and values of ONE sequence as dense arrays
`[layers, kv_heads, max_seq, head_dim]` (src/model/kv_cache.rs:23-63) and
writes row `pos` of every layer as it goes (src/model/mod.rs:201-209).  Here

* storage is cut into pages of `PAGE` positions; a sequence holds a list of
  pages per group and gives them back when its slot is freed;
* mixers with the same needs (all keys, or a window of them; heads; head
  size) form a *group* with storage of its own.  In a windowed group a
  sequence never holds more than `ceil(W / PAGE)` pages: position p lives in
  the sequence's page `(p // PAGE) % ring_pages`, row `p % PAGE`, so old
  positions are overwritten once they have left the window;
* a mixer may ask for a block of fixed size per sequence (`StateRequest`);
  it is zeroed when a slot is taken.

Stale rows are never cleared: what a query may see is decided by the
sequence's length and the window, as in the reference, where a reset only
sets `pos = 0`.

The books are kept in C++ by the host library; the classes here are its
face and own the device storage.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

import ctypes

import numpy as np

from ..kernels.page import PAGE                  # noqa: F401  (positions in a page: csrc/page.h)
from . import native
from .native import CacheFull, CacheMisuse      # noqa: F401

NO_RING = 1 << 24          # "ring" of a group that keeps every position: never wraps


@dataclass(frozen=True)
class KVRequest:
    """Keys and values per position.  `window` None: all positions are kept.  `v_head_dim`
    None: values are as wide as keys (`head_dim`)."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    v_head_dim: Optional[int] = None

    @property
    def value_dim(self) -> int:
        return self.head_dim if self.v_head_dim is None else self.v_head_dim


@dataclass(frozen=True)
class StateRequest:
    """A block of fixed size per sequence."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


def pages_for(n_tokens: int) -> int:
    return (n_tokens + PAGE - 1) // PAGE


def _ints(values) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(values, dtype=np.int32))


class _Books:
    """Owner of the host library's books of one cache.  The views below hold this object and
    never the cache itself, so that a dropped cache is freed at once, without the cycle collector."""

    def __init__(self, max_slots: int, n_pages: int, rings, pages):
        self.max_slots, self.n_pages = int(max_slots), int(n_pages)
        rings, pages = _ints(rings), _ints(pages)
        self._handle = ctypes.c_void_p(native.lib().tl_books_new(self.max_slots, len(rings), rings.ctypes.data,
                                                                 pages.ctypes.data))

    @property
    def h(self):
        """The handle of the books in the host library, for every call into it: the cache and all
        its views (slots, lengths, pools, pages of a slot) come through here, so that none of
        them hands the library a null handle once the cache is closed."""
        h = getattr(self, "_handle", None)
        if h is None:
            raise CacheMisuse("the cache is closed")
        return h

    def close(self) -> None:
        h, self._handle = getattr(self, "_handle", None), None
        if h:
            try:
                native.lib().tl_books_delete(h)
            except (TypeError, AttributeError):         # the interpreter is shutting down: the library is gone with it
                pass

    __del__ = close

    def held_slots(self) -> List[int]:
        buf = np.empty(self.max_slots, dtype=np.int32)
        n = native.lib().tl_books_held_slots(self.h, buf.ctypes.data, buf.size)
        return buf[:n].tolist()

    def holds(self, slot: int) -> bool:
        return bool(native.lib().tl_books_holds(self.h, int(slot)))

    @property
    def free_slots(self) -> int:
        return native.lib().tl_books_free_slots(self.h)


class _Pool:
    """What is free and held of a group's pages (the books are the host library's)."""

    def __init__(self, books: _Books, group: int, n: int):
        self._b, self._g, self.n = books, group, n

    @property
    def n_free(self) -> int:
        return native.lib().tl_books_free_pages(self._b.h, self._g)

    @property
    def n_held(self) -> int:
        return self.n - self.n_free

    def holds(self, page: int) -> bool:
        return bool(native.lib().tl_books_page_held(self._b.h, self._g, int(page)))


class _Slots:
    def __init__(self, books: _Books):
        self._b, self.n = books, books.max_slots

    @property
    def n_free(self) -> int:
        return self._b.free_slots

    @property
    def n_held(self) -> int:
        return self.n - self.n_free

    def holds(self, slot: int) -> bool:
        return self._b.holds(slot)


class _PagesOfSlot:
    """group.pages_of_slot[slot] -> the slot's pages, in the order of the ring (a copy)."""

    def __init__(self, books: _Books, group: int):
        self._b, self._g = books, group

    def __getitem__(self, slot: int) -> List[int]:
        buf = np.empty(self._b.n_pages, dtype=np.int32)
        n = native.lib().tl_books_pages(self._b.h, self._g, int(slot), buf.ctypes.data, buf.size)
        if n < 0:
            raise KeyError(slot)
        return buf[:n].tolist()

    def __contains__(self, slot: int) -> bool:
        return self._b.holds(slot)

    def __iter__(self):
        return iter(self._b.held_slots())

    def __len__(self) -> int:
        return len(self._b.held_slots())


class _Lengths:
    """cache.length[slot] -> positions the slot holds; behaves as a read-only dict."""

    def __init__(self, books: _Books):
        self._b = books

    def __getitem__(self, slot: int) -> int:
        n = native.lib().tl_books_length(self._b.h, int(slot))
        if n < 0:
            raise KeyError(slot)
        return n

    def __contains__(self, slot: int) -> bool:
        return self._b.holds(slot)

    def __iter__(self):
        return iter(self._b.held_slots())

    def __len__(self) -> int:
        return self._b.max_slots - self._b.free_slots

    def values(self):
        return [self[s] for s in self._b.held_slots()]


class KVGroup:
    """Storage of the runs that share one `KVRequest`."""

    def __init__(self, index: int, request: KVRequest, runs: List[int], n_pages: int, dtype, device,
                 allocate: bool):
        self.request = request
        self.runs = list(runs)
        self.layer_of_run = {r: i for i, r in enumerate(self.runs)}
        self.n_pages = n_pages
        # pages one sequence can hold: a ring for a window, else without bound (the pool is the limit)
        self.ring_pages = pages_for(request.window) if request.window else NO_RING
        self.index = index
        self.pool = self.pages_of_slot = None        # views of the books, tied by the cache
        self.storage = None
        if allocate:
            # A page holds the keys of its 64 positions, [kv_head, row, head_dim], and behind them the
            # values transposed, [kv_head, value_dim, row].  With values as wide as keys that is
            # [layer, page, K|V, kv_head, 64, head_dim], the shape the attention kernels take.
            nkv, dk, dv = request.n_kv_heads, request.head_dim, request.value_dim
            if dk == dv:
                self.storage = torch.empty((len(self.runs), n_pages, 2, nkv, PAGE, dk), dtype=dtype, device=device)
            else:
                self.storage = torch.empty((len(self.runs), n_pages, nkv * PAGE * (dk + dv)), dtype=dtype,
                                           device=device)

    def keys(self, layer: int) -> torch.Tensor:
        """A view of one layer's keys: [page, kv_head, row, head_dim]."""
        r = self.request
        flat = self.storage[layer].reshape(self.n_pages, -1)
        return flat[:, :r.n_kv_heads * PAGE * r.head_dim].view(self.n_pages, r.n_kv_heads, PAGE, r.head_dim)

    def values_t(self, layer: int) -> torch.Tensor:
        """A view of one layer's values, transposed as they are kept: [page, kv_head, value_dim, row]."""
        r = self.request
        flat = self.storage[layer].reshape(self.n_pages, -1)
        return flat[:, r.n_kv_heads * PAGE * r.head_dim:].view(self.n_pages, r.n_kv_heads, r.value_dim, PAGE)

    def pages_needed(self, length: int) -> int:
        return min(pages_for(length), self.ring_pages)


class Cache:
    """Slots, pages and state.  The books (who holds what) are kept by the host
    library (csrc/host/books.cpp) and can be used without a device
    (`allocate=False`)."""

    def __init__(self, kv_requests: Dict[int, KVRequest], state_requests: Dict[int, StateRequest],
                 max_tokens: int, dtype=torch.bfloat16, device="cpu", max_slots: Optional[int] = None,
                 allocate: bool = True):
        if max_tokens < 1:
            raise ValueError("max_tokens must be positive")
        self.n_pages = pages_for(max_tokens)
        self.max_slots = int(max_slots) if max_slots else self.n_pages
        self.dtype = dtype
        self.device = device
        by_req: Dict[KVRequest, List[int]] = {}
        for run in sorted(kv_requests):
            by_req.setdefault(kv_requests[run], []).append(run)
        self.groups: List[KVGroup] = [
            KVGroup(gi, req, runs, self.n_pages, dtype, device, allocate)
            for gi, (req, runs) in enumerate(by_req.items())]
        self._books = _Books(self.max_slots, self.n_pages, [g.ring_pages for g in self.groups],
                             [g.n_pages for g in self.groups])
        for g in self.groups:
            g.pool = _Pool(self._books, g.index, g.n_pages)
            g.pages_of_slot = _PagesOfSlot(self._books, g.index)
        self.slots = _Slots(self._books)
        self.length = _Lengths(self._books)
        self.group_of_run: Dict[int, int] = {
            r: gi for gi, g in enumerate(self.groups) for r in g.runs}
        self.state: Dict[int, Optional[torch.Tensor]] = {}
        self.state_requests = dict(state_requests)
        for run, req in state_requests.items():
            self.state[run] = torch.zeros((self.max_slots,) + tuple(req.shape), dtype=req.dtype,
                                          device=device) if allocate else None

    @property
    def _h(self):
        """The handle of the books in the host library (`CacheMisuse` once the cache is closed)."""
        return self._books.h

    def close(self) -> None:
        """Give the device storage and the books back now (the cache cannot be used afterwards).
        Dropping the last reference does the same."""
        for g in self.groups:
            g.storage = None
        self.state = {run: None for run in self.state}
        self._books.close()

    # ---- slots -----------------------------------------------------------
    def alloc_slot(self) -> int:
        out = ctypes.c_int(-1)
        native.check(native.lib().tl_books_alloc_slot(self._h, ctypes.byref(out)))
        s = out.value
        for run, t in self.state.items():
            if t is not None:
                t[s].zero_()
        return s

    def free_slot(self, slot: int) -> None:
        native.check(native.lib().tl_books_free_slot(self._h, int(slot)))

    def held_slots(self) -> List[int]:
        return self._books.held_slots()

    # ---- growth ----------------------------------------------------------
    def prepare(self, growth: List[Tuple[int, int]]) -> None:
        """Make room for `n_new` more positions in each `(slot, n_new)`.
        Either every sequence gets its pages or none is changed."""
        slots, n_new = _ints([g[0] for g in growth]), _ints([g[1] for g in growth])
        native.check(native.lib().tl_books_prepare(self._h, len(growth), slots.ctypes.data, n_new.ctypes.data))

    def fits(self, lengths: List[int]) -> bool:
        """Would new sequences of these final lengths find slots and pages now?"""
        ls = np.ascontiguousarray(np.asarray(lengths, dtype=np.int64))
        return bool(native.lib().tl_books_fits(self._h, len(lengths), ls.ctypes.data))

    def commit(self, growth: List[Tuple[int, int]]) -> None:
        slots, n_new = _ints([g[0] for g in growth]), _ints([g[1] for g in growth])
        native.check(native.lib().tl_books_commit(self._h, len(growth), slots.ctypes.data, n_new.ctypes.data))

    # ---- views for kernels -------------------------------------------------
    def kv_layer(self, run: int) -> Tuple[KVGroup, int]:
        gi = self.group_of_run[run]
        g = self.groups[gi]
        return g, g.layer_of_run[run]

    def tokens_held(self) -> int:
        """Positions held by live sequences, each rounded up to whole pages."""
        return sum(pages_for(n) * PAGE for n in self.length.values())

    def check(self) -> None:
        """Invariants: no page or slot lost, held twice, or both free and held."""
        native.check(native.lib().tl_books_check(self._h))
