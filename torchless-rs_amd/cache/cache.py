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
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from .pool import CacheFull, CacheMisuse, FreeList

PAGE = 64
NO_RING = 1 << 24          # "ring" of a group that keeps every position: never wraps


@dataclass(frozen=True)
class KVRequest:
    """Keys and values per position.  `window` None: all positions are kept."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateRequest:
    """A block of fixed size per sequence."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


def pages_for(n_tokens: int) -> int:
    return (n_tokens + PAGE - 1) // PAGE


class KVGroup:
    """Storage of the runs that share one `KVRequest`."""

    def __init__(self, request: KVRequest, runs: List[int], n_pages: int, dtype, device,
                 allocate: bool):
        self.request = request
        self.runs = list(runs)
        self.layer_of_run = {r: i for i, r in enumerate(self.runs)}
        self.n_pages = n_pages
        # pages one sequence can hold: a ring for a window, else without bound (the pool is the limit)
        self.ring_pages = pages_for(request.window) if request.window else NO_RING
        self.pool = FreeList(n_pages, "page")
        self.pages_of_slot: Dict[int, List[int]] = {}
        self.storage = None
        if allocate:
            # [layer, page, K|V, kv_head, row, head_dim]
            self.storage = torch.empty(
                (len(self.runs), n_pages, 2, request.n_kv_heads, PAGE, request.head_dim),
                dtype=dtype, device=device)

    def pages_needed(self, length: int) -> int:
        return min(pages_for(length), self.ring_pages)


class Cache:
    """Slots, pages and state.  All bookkeeping is on the host and can be used
    without a device (`allocate=False`)."""

    def __init__(self, kv_requests: Dict[int, KVRequest], state_requests: Dict[int, StateRequest],
                 max_tokens: int, dtype=torch.bfloat16, device="cpu", max_slots: Optional[int] = None,
                 allocate: bool = True):
        if max_tokens < 1:
            raise ValueError("max_tokens must be positive")
        self.n_pages = pages_for(max_tokens)
        self.max_slots = int(max_slots) if max_slots else self.n_pages
        self.dtype = dtype
        self.device = device
        self.slots = FreeList(self.max_slots, "slot")
        self.length: Dict[int, int] = {}
        by_req: Dict[KVRequest, List[int]] = {}
        for run in sorted(kv_requests):
            by_req.setdefault(kv_requests[run], []).append(run)
        self.groups: List[KVGroup] = [
            KVGroup(req, runs, self.n_pages, dtype, device, allocate) for req, runs in by_req.items()]
        self.group_of_run: Dict[int, int] = {
            r: gi for gi, g in enumerate(self.groups) for r in g.runs}
        self.state: Dict[int, Optional[torch.Tensor]] = {}
        self.state_requests = dict(state_requests)
        for run, req in state_requests.items():
            self.state[run] = torch.zeros((self.max_slots,) + tuple(req.shape), dtype=req.dtype,
                                          device=device) if allocate else None

    # ---- slots -----------------------------------------------------------
    def alloc_slot(self) -> int:
        s = self.slots.take()
        self.length[s] = 0
        for g in self.groups:
            g.pages_of_slot[s] = []
        for run, t in self.state.items():
            if t is not None:
                t[s].zero_()
        return s

    def free_slot(self, slot: int) -> None:
        self.slots.give_back(slot)
        for g in self.groups:
            for p in g.pages_of_slot.pop(slot):
                g.pool.give_back(p)
        del self.length[slot]

    def _held(self, slot: int) -> None:
        if not self.slots.holds(slot):
            raise CacheMisuse(f"slot {slot} is not held")

    # ---- growth ----------------------------------------------------------
    def prepare(self, growth: List[Tuple[int, int]]) -> None:
        """Make room for `n_new` more positions in each `(slot, n_new)`.
        Either every sequence gets its pages or none is changed."""
        need = [0] * len(self.groups)
        seen = set()
        for slot, n_new in growth:
            self._held(slot)
            if slot in seen:
                raise CacheMisuse(f"slot {slot} appears twice in one step")
            seen.add(slot)
            if n_new < 1:
                raise ValueError(f"slot {slot}: a step must bring at least one token")
            for gi, g in enumerate(self.groups):
                need[gi] += g.pages_needed(self.length[slot] + n_new) - len(g.pages_of_slot[slot])
        for gi, g in enumerate(self.groups):
            if need[gi] > g.pool.n_free:
                raise CacheFull(
                    f"the step needs {need[gi]} more pages of {PAGE} positions, {g.pool.n_free} of "
                    f"{g.n_pages} are free; raise max_tokens")
        for slot, n_new in growth:
            for g in self.groups:
                pages = g.pages_of_slot[slot]
                while len(pages) < g.pages_needed(self.length[slot] + n_new):
                    pages.append(g.pool.take())

    def fits(self, lengths: List[int]) -> bool:
        """Would new sequences of these final lengths find slots and pages now?"""
        if len(lengths) > self.slots.n_free:
            return False
        return all(sum(g.pages_needed(n) for n in lengths) <= g.pool.n_free for g in self.groups)

    def commit(self, growth: List[Tuple[int, int]]) -> None:
        for slot, n_new in growth:
            self.length[slot] += n_new

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
        self.slots.check()
        for g in self.groups:
            g.pool.check()
            held = [p for pages in g.pages_of_slot.values() for p in pages]
            assert len(held) == len(set(held)), "a page is held by two sequences"
            assert len(held) == g.pool.n_held, "a page is held by no sequence"
            for p in held:
                assert g.pool.holds(p)
            assert set(g.pages_of_slot) == set(self.length), "slots and page lists differ"
            for s, pages in g.pages_of_slot.items():
                assert len(pages) == g.pages_needed(self.length[s]) or \
                    len(pages) >= g.pages_needed(self.length[s])
