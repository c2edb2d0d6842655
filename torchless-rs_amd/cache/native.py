"""ctypes face of the host library: free lists, the books of slots and pages, and the packer of a
step's batch.  Return codes become the exceptions of this package."""
from __future__ import annotations

import ctypes
from typing import Optional

from ..kernels.build import load_host

OK, FULL, MISUSE, BAD_VALUE, BAD_STEP = 0, 1, 2, 3, 4


class CacheFull(RuntimeError):
    """No free page or slot is left."""


class CacheMisuse(RuntimeError):
    """An id was given back that is not held, or used while not held."""


class StepError(ValueError):
    """A step that cannot be run as asked (unknown slot, token id outside the
    vocabulary, empty batch, ...)."""


_lib: Optional[ctypes.CDLL] = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        l = load_host()
        l.tl_host_last_error.restype = ctypes.c_char_p
        for name in ("tl_freelist_new", "tl_books_new"):
            getattr(l, name).restype = ctypes.c_void_p
        l.tl_freelist_new.argtypes = [ctypes.c_int, ctypes.c_char_p]
        l.tl_books_new.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        for name in ("tl_freelist_delete", "tl_books_delete"):
            getattr(l, name).argtypes = [ctypes.c_void_p]
            getattr(l, name).restype = None
        l.tl_freelist_take.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        for name in ("tl_freelist_give_back", "tl_freelist_holds", "tl_books_free_slot", "tl_books_holds"):
            getattr(l, name).argtypes = [ctypes.c_void_p, ctypes.c_long]
        for name in ("tl_freelist_n_free", "tl_freelist_check", "tl_books_free_slots", "tl_books_check"):
            getattr(l, name).argtypes = [ctypes.c_void_p]
        l.tl_books_alloc_slot.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        l.tl_books_length.argtypes = [ctypes.c_void_p, ctypes.c_long]
        l.tl_books_length.restype = ctypes.c_long
        l.tl_books_free_pages.argtypes = [ctypes.c_void_p, ctypes.c_int]
        l.tl_books_page_held.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_long]
        l.tl_books_held_slots.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
        l.tl_books_pages.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_void_p, ctypes.c_int]
        for name in ("tl_books_prepare", "tl_books_commit"):
            getattr(l, name).argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        l.tl_books_fits.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
        l.tl_aligned_columns.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        l.tl_aligned_columns.restype = ctypes.c_long
        l.tl_pack_step.argtypes = [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 5 + [ctypes.c_int] + \
            [ctypes.c_void_p] * 2 + [ctypes.c_long] + [ctypes.c_void_p] * 3
        from ..kernels.page import require_same
        require_same(l.tl_host_page(), "the host library")
        _lib = l
    return _lib


def check(rc: int) -> None:
    """Raise what a return code of the host library stands for."""
    if rc == OK:
        return
    msg = (lib().tl_host_last_error() or b"").decode()
    if rc == FULL:
        raise CacheFull(msg)
    if rc == MISUSE:
        raise CacheMisuse(msg)
    if rc == BAD_STEP:
        raise StepError(msg)
    raise ValueError(msg)
