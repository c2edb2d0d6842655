"""Binding tensors to a model by name, with one error for everything wrong.

The reference looks names up one by one and stops at the first that is
missing ("Tensor '<name>' not found", src/loader/parameters.rs:913, 1225);
a wrong shape only shows later as an assertion inside a product
(src/loader/parameters.rs:554-555).  Here the whole table is checked first:
missing names, names nobody asked for, and shapes that differ are collected
and raised together.

Storage rule: a tensor keeps the width it is stored in.  bfloat16 stays
bfloat16, float16 becomes bfloat16, a tensor stored in 32 bits (or 64) stays
float32, integer tables become int32.  With `compute_dtype=float32`
every floating tensor is widened to float32.
"""
from __future__ import annotations

import re
from dataclasses import dataclass
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import torch


@dataclass(frozen=True)
class WeightSpec:
    """What a part expects under one name."""
    shape: Tuple[int, ...]
    integer: bool = False
    init: str = "normal"      # how random weights fill it: "normal" or "ones" (norm weights)


class WeightBindingError(ValueError):
    """The checkpoint does not fit the model.  `missing`, `unexpected` and
    `mismatched` (name, found shape, wanted shape) hold the details."""

    def __init__(self, missing, unexpected, mismatched, bad_dtype=()):
        self.missing: List[str] = list(missing)
        self.unexpected: List[str] = list(unexpected)
        self.mismatched: List[Tuple[str, Tuple[int, ...], Tuple[int, ...]]] = list(mismatched)
        self.bad_dtype: List[Tuple[str, str]] = list(bad_dtype)
        lines = ["checkpoint does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.mismatched:
            lines.append(f"  wrong shapes ({len(self.mismatched)}): " + "; ".join(
                f"{n}: found {list(g)}, model needs {list(w)}" for n, g, w in self.mismatched))
        if self.bad_dtype:
            lines.append(f"  wrong dtypes ({len(self.bad_dtype)}): " + "; ".join(
                f"{n}: {why}" for n, why in self.bad_dtype))
        super().__init__("\n".join(lines))


def stored_to_resident(t: torch.Tensor, compute_dtype: torch.dtype) -> torch.Tensor:
    """Apply the storage rule to one tensor."""
    if not t.dtype.is_floating_point:
        return t.to(torch.int32)
    if compute_dtype == torch.float32:
        return t.to(torch.float32)
    if t.dtype in (torch.float32, torch.float64):
        return t.to(torch.float32)
    return t.to(torch.bfloat16)


def bind_weights(expected: Dict[str, WeightSpec], source, compute_dtype: torch.dtype,
                 device, ignore: Sequence[str] = ()) -> Dict[str, torch.Tensor]:
    """Check `source` (anything with names/shape/dtype/tensor) against
    `expected` and return the tensors on `device`.  `ignore` holds regular
    expressions of names that may be present without being used."""
    have = set(source.names())
    ign = [re.compile(p) for p in ignore]
    missing = [n for n in expected if n not in have]
    unexpected = sorted(n for n in have if n not in expected and not any(p.fullmatch(n) for p in ign))
    mismatched, bad = [], []
    for n, spec in expected.items():
        if n not in have:
            continue
        got = tuple(source.shape(n))
        if got != tuple(spec.shape):
            mismatched.append((n, got, tuple(spec.shape)))
        dt = source.dtype(n)
        if spec.integer and dt.is_floating_point:
            bad.append((n, f"stored as {dt}, model needs an integer table"))
        if not spec.integer and not dt.is_floating_point:
            bad.append((n, f"stored as {dt}, model needs floating point"))
    if missing or unexpected or mismatched or bad:
        raise WeightBindingError(missing, unexpected, mismatched, bad)
    out: Dict[str, torch.Tensor] = {}
    for n in expected:
        t = source.tensor(n)
        t = stored_to_resident(t, compute_dtype)
        out[n] = t.to(device).contiguous() if device is not None else t.contiguous()
    return out
