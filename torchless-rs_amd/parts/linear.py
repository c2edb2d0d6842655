"""Products with a weight matrix stored [out, in] as the checkpoint has it
(out[r] = sum_c W[r,c] x[c], src/loader/parameters.rs:551-594 of the
reference).  The kernel is chosen by what the operands are, never by the
model: float32 anywhere means the plain FMA kernel (true 32-bit)."""
from __future__ import annotations

import torch

import contextlib
import contextvars

from ..kernels import ops

# whether weights loaded now may keep tiled copies: set for the extent of one load
# (`loading_with`), per thread and task, never for the process
_tiled_copies = contextvars.ContextVar("tiled_copies", default=True)


@contextlib.contextmanager
def loading_with(tiled_copies: bool):
    """Within this block `Linear(..., tiled=True)` keeps its tiled copy only if `tiled_copies`."""
    token = _tiled_copies.set(bool(tiled_copies))
    try:
        yield
    finally:
        _tiled_copies.reset(token)


class Linear:
    """A weight [N, K] resident on the device in its stored width.  With `tiled` it
    also keeps the tiled copy (`ops.tile_weights`) that the products of steps of at
    most 16 rows read instead: memory spent for the rate at which decoding streams
    the weights (a load under `loading_with(False)` makes none).  `tile_rows`: the
    copy's own order of rows, for a kernel that wants one; then only that kernel
    reads it (`own_tiles`)."""

    def __init__(self, weight: torch.Tensor, tiled: bool = False, tile_rows: torch.Tensor = None):
        assert weight.dim() == 2
        self.weight = weight.contiguous()
        self.out_features, self.in_features = self.weight.shape
        self.tiles = self.own_tiles = None
        if (tiled and _tiled_copies.get() and self.weight.is_cuda and self.weight.dtype == torch.bfloat16
                and ops.tiles_fit(self.out_features, self.in_features)):
            copy = ops.tile_weights(self.weight, tile_rows)
            if tile_rows is None:
                self.tiles = copy
            else:
                self.own_tiles = copy

    def __call__(self, a: torch.Tensor, out: torch.Tensor, accumulate: bool = False, factor=None) -> None:
        """out[M, N] (+)= a[M, K] @ W^T; out is float32.  `factor` (`ops.RowFactor`): the
        second half of the norm that made `a`, a factor per row (at most 16 rows)."""
        if factor is not None:
            ops.gemm_bf16_norm(a, self.weight, out, accumulate, factor=factor, tiles=self.tiles)
        elif self.mid(a):
            ops.gemm_mid_bf16(a, self.weight, out, 1, accumulate)
        else:
            ops.gemm(a, self.weight, out, accumulate, tiles=self.tiles)

    def own_kernels(self, n_rows: int) -> bool:
        """Does a product of `n_rows` rows launch this package's kernels only (never the BLAS
        library's, which a captured graph must not hold)?"""
        return n_rows <= ops.own_rows(self.in_features) or self.weight.dtype != torch.bfloat16

    def mid(self, a: torch.Tensor) -> bool:
        """17..`ops.own_rows(K)` rows of bfloat16: the kernels that share the activations
        through LDS."""
        return 16 < a.shape[0] <= ops.own_rows(self.in_features) and ops.bf16_gemm_ok(a, self.weight)

    def partial(self, a: torch.Tensor, ctx, name: str):
        """The product as partial sums [S, M, N] (float32) for a reader that adds
        them up, where that pays (17..MID_ROWS rows and K worth cutting); else None."""
        if not self.mid(a):
            return None
        S = ops.mid_splits(a.shape[0], self.out_features, self.in_features, ops.compute_units(a.device))
        if S == 1:
            return None
        parts = ctx.workspace.get(name, (S, a.shape[0], self.out_features), torch.float32)
        ops.gemm_mid_bf16(a, self.weight, parts, S)
        return parts

    def add_into(self, a: torch.Tensor, x: torch.Tensor, ctx, name: str) -> None:
        """x += a @ W^T, now or as partial sums left in `ctx.pending`."""
        from .base import flush_pending
        flush_pending(ctx, x)
        norm = ctx.norm_ahead
        form = norm.rms_form() if norm is not None and ops.norm_split_ok(a, self.weight) else None
        if (form is not None and form.size == self.out_features and form.weight is not None
                and form.weight.dtype == torch.float32):
            # the next norm's first half rides on this product
            xt = ctx.workspace.get("prenormed_y", (a.shape[0], self.out_features), torch.bfloat16)
            ssq = ctx.workspace.get(name + "_ssq", (16, -(-self.out_features // 16)), torch.float32)
            groups = ops.gemm_bf16_norm(a, self.weight, x, accumulate=True, norm_weight=form.weight, xt=xt,
                                        ssq_out=ssq, tiles=self.tiles)
            ctx.prenormed = (norm, xt, ops.RowFactor(ssq, groups, form.size, form.eps))
            return
        parts = self.partial(a, ctx, name)
        if parts is None:
            self(a, x, accumulate=True)
        else:
            ctx.pending = parts


def interleave_pairs(gate: torch.Tensor, up: torch.Tensor, block: int = 32) -> torch.Tensor:
    """Rows in groups of 2*block: `block` rows of gate, then the `block` rows of
    up that belong to them: the layout of the products' paired epilogue."""
    I, K = gate.shape
    g = gate.view(I // block, block, K)
    u = up.view(I // block, block, K)
    return torch.stack([g, u], dim=1).reshape(2 * I, K).contiguous()
