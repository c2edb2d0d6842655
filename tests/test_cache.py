"""The cache's bookkeeping (no GPU): no slot or page lost, held twice or freed
twice; windows hold a ring of pages; a step gets all its pages or none."""
import ctypes
import random

import pytest
import torch

from torchless_rs_amd.cache import PAGE, Cache, CacheFull, CacheMisuse, KVRequest, StateRequest, pages_for
from torchless_rs_amd.cache import native


class FreeList:
    """The host library's free list (the one its books of slots and pages are made of), by itself."""

    def __init__(self, n, what):
        self.h = ctypes.c_void_p(native.lib().tl_freelist_new(n, what.encode()))

    def __del__(self):
        native.lib().tl_freelist_delete(self.h)

    @property
    def n_free(self):
        return native.lib().tl_freelist_n_free(self.h)

    def take(self):
        out = ctypes.c_int(-1)
        native.check(native.lib().tl_freelist_take(self.h, ctypes.byref(out)))
        return out.value

    def give_back(self, i):
        native.check(native.lib().tl_freelist_give_back(self.h, int(i)))

    def check(self):
        native.check(native.lib().tl_freelist_check(self.h))


def test_free_list():
    f = FreeList(3, "slot")
    a, b, c = f.take(), f.take(), f.take()
    assert sorted([a, b, c]) == [0, 1, 2] and f.n_free == 0
    with pytest.raises(CacheFull):
        f.take()
    f.give_back(b)
    with pytest.raises(CacheMisuse, match="not held"):
        f.give_back(b)                                      # freed twice
    with pytest.raises(CacheMisuse, match="does not exist"):
        f.give_back(7)
    assert f.take() == b                                    # the freed id is used again at once
    f.check()


def make(max_tokens=64 * 6, window=None, slots=None, two_groups=False):
    kv = {0: KVRequest(2, 16, window), 1: KVRequest(2, 16, window)}
    if two_groups:
        kv[2] = KVRequest(2, 16, None)
    return Cache(kv, {1: StateRequest((4,), torch.float32)}, max_tokens, torch.float32, "cpu", slots,
                 allocate=False)


def test_groups_follow_requests():
    c = make(window=100, two_groups=True)
    assert len(c.groups) == 2
    assert c.groups[0].runs == [0, 1] and c.groups[1].runs == [2]
    assert c.groups[0].ring_pages == 2 and c.groups[1].ring_pages > c.n_pages
    assert c.kv_layer(1) == (c.groups[0], 1) and c.kv_layer(2) == (c.groups[1], 0)


def test_growth_and_release():
    c = make()
    a, b = c.alloc_slot(), c.alloc_slot()
    c.prepare([(a, 65), (b, 1)])
    c.commit([(a, 65), (b, 1)])
    g = c.groups[0]
    assert len(g.pages_of_slot[a]) == 2 and len(g.pages_of_slot[b]) == 1 and c.length[a] == 65
    assert c.tokens_held() == 3 * PAGE
    c.prepare([(a, 1), (b, 63)])                            # neither crosses a page
    c.commit([(a, 1), (b, 63)])
    assert g.pool.n_held == 3
    c.prepare([(b, 1)])
    c.commit([(b, 1)])
    assert len(g.pages_of_slot[b]) == 2
    c.check()
    c.free_slot(a)
    with pytest.raises(CacheMisuse):
        c.free_slot(a)
    with pytest.raises(CacheMisuse):
        c.prepare([(a, 1)])
    c.free_slot(b)
    assert g.pool.n_free == c.n_pages and c.slots.n_free == c.max_slots and c.tokens_held() == 0
    c.check()


def test_all_or_nothing():
    c = make(max_tokens=64 * 3)
    a, b = c.alloc_slot(), c.alloc_slot()
    with pytest.raises(CacheFull, match="max_tokens"):
        c.prepare([(a, 100), (b, 100)])                     # 4 pages wanted, 3 there
    assert c.groups[0].pool.n_free == 3 and c.groups[0].pages_of_slot[a] == []
    with pytest.raises(CacheMisuse, match="twice"):
        c.prepare([(a, 1), (a, 1)])
    with pytest.raises(ValueError):
        c.prepare([(a, 0)])
    c.prepare([(a, 100), (b, 64)])
    c.check()


def test_window_holds_a_ring():
    c = make(max_tokens=64 * 8, window=70)                  # ring of 2 pages
    s = c.alloc_slot()
    for n in (10, 60, 500, 1):
        c.prepare([(s, n)])
        c.commit([(s, n)])
    assert len(c.groups[0].pages_of_slot[s]) == 2 and c.length[s] == 571
    assert c.fits([10 ** 6] * 3) and not c.fits([10 ** 6] * 4)          # 3 more rings of 2 fit in 6 pages
    c.check()


def test_fits():
    c = make(max_tokens=64 * 4, slots=3)
    assert c.fits([64, 64, 128]) and not c.fits([64, 64, 129]) and not c.fits([1, 1, 1, 1])
    s = c.alloc_slot()
    c.prepare([(s, 65)])
    assert c.fits([128]) and not c.fits([129])


def test_random_traffic_keeps_the_books():
    rnd = random.Random(0)
    c = make(max_tokens=64 * 40, window=130, two_groups=True, slots=12)
    live = []
    for _ in range(2000):
        r = rnd.random()
        if r < 0.25 and c.slots.n_free:
            live.append(c.alloc_slot())
        elif r < 0.4 and live:
            c.free_slot(live.pop(rnd.randrange(len(live))))
        elif live:
            batch = rnd.sample(live, rnd.randint(1, len(live)))
            growth = [(s, rnd.choice([1, 1, 1, 7, 64, 200])) for s in batch]
            before = {s: (c.length[s], [list(g.pages_of_slot[s]) for g in c.groups]) for s in batch}
            try:
                c.prepare(growth)
                c.commit(growth)
            except CacheFull:
                for s in batch:
                    assert (c.length[s], [list(g.pages_of_slot[s]) for g in c.groups]) == before[s]
        c.check()
    for s in live:
        c.free_slot(s)
    c.check()
    assert all(g.pool.n_free == g.n_pages for g in c.groups)


def test_state_is_zeroed_when_a_slot_is_taken():
    c = Cache({}, {0: StateRequest((3,), torch.float32)}, 64 * 2, torch.float32, "cpu", 2)
    s = c.alloc_slot()
    c.state[0][s] += 5
    c.free_slot(s)
    assert c.alloc_slot() == s and float(c.state[0][s].abs().sum()) == 0


def test_a_dropped_cache_is_freed_without_the_cycle_collector():
    """Nothing in the cache points back at it: dropping the last reference frees its storage at
    once, also when the collector is switched off or the objects are frozen out of its sight."""
    import gc
    import weakref
    gc.collect()
    gc.disable()
    try:
        c = Cache({0: KVRequest(2, 16, None)}, {0: StateRequest((4,))}, 64 * 4, torch.float32, "cpu",
                  max_slots=2, allocate=True)
        s = c.alloc_slot()
        c.prepare([(s, 70)])
        c.commit([(s, 70)])
        storage, state, books = weakref.ref(c.groups[0].storage), weakref.ref(c.state[0]), weakref.ref(c._books)
        del c
        assert storage() is None and state() is None and books() is None
    finally:
        gc.enable()


def test_a_closed_cache_gives_its_storage_back_and_refuses_use():
    import weakref
    c = Cache({0: KVRequest(2, 16, None)}, {}, 64 * 4, torch.float32, "cpu", allocate=True)
    storage = weakref.ref(c.groups[0].storage)
    c.close()
    assert storage() is None
    with pytest.raises(CacheMisuse, match="closed"):
        c.alloc_slot()
    c.close()                                               # twice is harmless


def test_every_view_of_a_closed_cache_refuses_use():
    """The views kept on a cache (slots, lengths, a group's pool and its pages by slot) reach the host
    library through the same checked handle as the cache: after `close` each raises, none hands the
    library a null handle."""
    c = make(two_groups=True)
    s = c.alloc_slot()
    c.prepare([(s, 70)])
    c.commit([(s, 70)])
    slots, length, group = c.slots, c.length, c.groups[0]
    c.close()
    touches = [
        lambda: slots.n_free, lambda: slots.n_held, lambda: slots.holds(s),
        lambda: length[s], lambda: len(length), lambda: s in length, lambda: list(length), lambda: length.values(),
        lambda: group.pool.n_free, lambda: group.pool.n_held, lambda: group.pool.holds(0),
        lambda: group.pages_of_slot[s], lambda: s in group.pages_of_slot, lambda: len(group.pages_of_slot),
        lambda: list(group.pages_of_slot),
        lambda: c.held_slots(), lambda: c.fits([10]), lambda: c.prepare([(s, 1)]), lambda: c.commit([(s, 1)]),
        lambda: c.free_slot(s), lambda: c.check(), lambda: c.tokens_held(),
    ]
    for i, touch in enumerate(touches):
        with pytest.raises(CacheMisuse, match="closed"):
            touch()
            pytest.fail(f"touch {i} went through")
