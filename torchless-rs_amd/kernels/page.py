"""Positions in a page of the cache.  The number is written once, in csrc/page.h; this module
reads it from there, and a library whose code was compiled with another is refused when loaded."""
from __future__ import annotations

import os
import re

_HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc", "page.h")


def _read() -> int:
    with open(_HEADER) as f:
        m = re.search(r"^#define\s+TL_PAGE\s+(\d+)\s*$", f.read(), re.M)
    if not m:
        raise RuntimeError(f"{_HEADER} does not define TL_PAGE")
    return int(m.group(1))


PAGE = _read()


def round_up(n_tokens: int) -> int:
    """`n_tokens` rounded up to whole pages."""
    return -(-int(n_tokens) // PAGE) * PAGE


def require_same(compiled: int, what: str) -> None:
    if int(compiled) != PAGE:
        raise RuntimeError(f"{what} was compiled for pages of {compiled} positions, csrc/page.h says {PAGE}; "
                           "build the libraries again")
