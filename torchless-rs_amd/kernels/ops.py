"""Python faces of the HIP kernels.

Every function checks on the host that its operands are on the GPU,
contiguous, of the type and shape that the kernel and its grid assume, and
launches on torch's current stream.  A failure of the launcher raises
`KernelError` with the library's message.  There is no fallback: without the
library nothing here runs.
"""
from __future__ import annotations

import ctypes
import functools
from typing import Optional

import torch

from .build import load, load_measure
from .page import PAGE, require_same

DT_F32, DT_BF16 = 0, 1
_CODES = {torch.float32: DT_F32, torch.bfloat16: DT_BF16}


class KernelError(RuntimeError):
    pass


_configured = False


def lib() -> ctypes.CDLL:
    global _configured
    L = load()
    if not _configured:
        L.tl_last_error.restype = ctypes.c_char_p
        require_same(L.tl_page_size(), "the kernels' library")
        _configured = True
    return L


def _check(rc: int) -> None:
    if rc != 0:
        raise KernelError(lib().tl_last_error().decode())


def _code(dt: torch.dtype) -> int:
    if dt not in _CODES:
        raise KernelError(f"dtype {dt} is not served by the kernels (float32 and bfloat16 are)")
    return _CODES[dt]


def _p(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> ctypes.c_void_p:
    """The current stream's handle (the short way where torch has it: a stream object for every launch
    costs the host a fifth of a step that is not a captured graph)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _req(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    # one test on the usual way (every launch asks several times); what is wrong is named below
    if (t.is_cuda and t.is_contiguous() and (dtype is None or t.dtype == dtype)
            and (shape is None or t.shape == tuple(shape))):
        return
    if not t.is_cuda:
        raise KernelError(f"{name}: must be on the GPU")
    if not t.is_contiguous():
        raise KernelError(f"{name}: must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: dtype {t.dtype}, kernel needs {dtype}")
    raise KernelError(f"{name}: shape {tuple(t.shape)}, kernel needs {tuple(shape)}")


def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
    """out[n, :] = table[ids[n], :] widened to float32."""
    n, H = ids.shape[0], table.shape[1]
    _req(table, "embed.table")
    _req(ids, "embed.ids", torch.int32, (n,))
    _req(out, "embed.out", torch.float32, (n, H))
    _check(lib().tl_embed(_p(table), _code(table.dtype), _p(ids), n, H, _p(out), _stream()))


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    """out = x / sqrt(mean(x^2) + eps) * w, x float32 [n, H], w float32 [H]."""
    n, H = x.shape
    _req(x, "rmsnorm.x", torch.float32)
    _req(w, "rmsnorm.w", torch.float32, (H,))
    _req(out, "rmsnorm.out", None, (n, H))
    _check(lib().tl_rmsnorm(_p(x), _p(w), ctypes.c_float(eps), _p(out), _code(out.dtype), n, H,
                            _stream()))


class Rotation:
    """How q and k are rotated by position: the first `rotary_dim` channels of a head in pairs,
    pair i by the angle pos * inv_freq[i] (float32 [rotary_dim / 2] on the device); pairs are
    (i, i + rotary_dim/2), or (2i, 2i+1) when `interleaved`; the channels behind them pass
    through.  rotary_dim 0 (inv_freq None): nothing is rotated."""

    def __init__(self, inv_freq: Optional[torch.Tensor], rotary_dim: int, interleaved: bool = False):
        self.inv_freq, self.rotary_dim, self.interleaved = inv_freq, int(rotary_dim), bool(interleaved)


NO_ROTATION = Rotation(None, 0)


def _rotation(rot, d: int, what: str) -> Rotation:
    """A `Rotation` checked against the head size `d`.  A bare tensor of d/2 frequencies stands
    for the rotation of the whole head in halves; None for no rotation."""
    if rot is None:
        return NO_ROTATION
    if isinstance(rot, torch.Tensor):
        rot = Rotation(rot, d)
    if rot.rotary_dim % 2 or not (0 <= rot.rotary_dim <= d):
        raise KernelError(f"{what}: {rot.rotary_dim} rotated channels of a head of {d} (even, at most the head)")
    if rot.rotary_dim:
        _req(rot.inv_freq, what + ".inv_freq", torch.float32, (rot.rotary_dim // 2,))
    return rot


def rope_split(qkv: torch.Tensor, row_pos: torch.Tensor, rotation, nq: int, nkv: int,
               d: int, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, vt: Optional[torch.Tensor] = None,
               row_seq=None, tile_off=None, n_cached=None) -> None:
    """Rotate q and k of the fused projection by their rows' positions (`rotation`: a
    `Rotation`, or the d/2 frequencies of a whole head rotated in halves) and
    write q [n,nq,d], k, v [n,nkv,d] (v may be None: the values are taken by
    `v_tiles` then).  With `vt` [nkv, d, cols] the values are
    also written transposed, row n into column tile_off[b] + pos - 64 *
    (n_cached[b] // 64) of its sequence b = row_seq[n]."""
    n = qkv.shape[0]
    _req(qkv, "rope.qkv", torch.float32, (n, (nq + 2 * nkv) * d))
    _req(row_pos, "rope.row_pos", torch.int32, (n,))
    rot = _rotation(rotation, d, "rope")
    _req(q, "rope.q", None, (n, nq, d))
    if nkv:
        _req(k, "rope.k", q.dtype, (n, nkv, d))
        if v is not None:
            _req(v, "rope.v", q.dtype, (n, nkv, d))
    cols = 0
    if vt is not None:
        _req(vt, "rope.vt", q.dtype)
        if vt.dim() != 3 or tuple(vt.shape[:2]) != (nkv, d):
            raise KernelError(f"rope.vt: shape {tuple(vt.shape)}, kernel needs [{nkv}, {d}, columns]")
        cols = vt.shape[2]
        _req(row_seq, "rope.row_seq", torch.int32, (n,))
        _req(tile_off, "rope.tile_off", torch.int32)
        _req(n_cached, "rope.n_cached", torch.int32, tuple(tile_off.shape))
    _check(lib().tl_rope_split(_p(qkv), _p(row_pos), _p(rot.inv_freq), rot.rotary_dim, int(rot.interleaved),
                               n, nq, nkv, d, _p(q), _p(k), _p(v),
                               _p(vt), cols, _p(row_seq), _p(tile_off), _p(n_cached), _code(q.dtype),
                               _stream()))


def kv_commit(k: torch.Tensor, v: torch.Tensor, row_seq, row_pos, len_after, table: torch.Tensor,
              ring_pages: int, pages: torch.Tensor) -> None:
    """Write this step's keys and values into the pages of one layer.
    pages: [n_pages, 2, nkv, PAGE, d]; table: [B, stride] page ids."""
    n, nkv, d = k.shape
    _req(k, "kv_commit.k", pages.dtype)
    _req(v, "kv_commit.v", pages.dtype, (n, nkv, d))
    _req(row_seq, "kv_commit.row_seq", torch.int32, (n,))
    _req(row_pos, "kv_commit.row_pos", torch.int32, (n,))
    _req(len_after, "kv_commit.len_after", torch.int32)
    _req(table, "kv_commit.table", torch.int32)
    _req(pages, "kv_commit.pages")
    if pages.dim() != 5 or tuple(pages.shape[1:]) != (2, nkv, PAGE, d):
        raise KernelError(f"kv_commit.pages: shape {tuple(pages.shape)}, kernel needs [*, 2, {nkv}, {PAGE}, {d}]")
    if table.dim() != 2 or table.shape[0] != len_after.shape[0]:
        raise KernelError("kv_commit.table: needs one row per sequence")
    _check(lib().tl_kv_commit(_p(k), _p(v), _code(k.dtype), _p(row_seq), _p(row_pos), _p(len_after),
                              _p(table), table.shape[1], ring_pages, n, nkv, d, _p(pages), _stream()))


def _tiles_args(B, cu_seqlens, tile_off, n_cached, len_after, what):
    _req(tile_off, what + ".tile_off", torch.int32, (B,))
    _req(n_cached, what + ".n_cached", torch.int32, (B,))
    _req(len_after, what + ".len_after", torch.int32, (B,))
    if cu_seqlens is not None:
        _req(cu_seqlens, what + ".cu_seqlens", torch.int32, (B + 1,))


def v_tiles(qkv: torch.Tensor, nq: int, nkv: int, d: int, vt: torch.Tensor, cu_seqlens, tile_off, n_cached,
            len_after) -> None:
    """The values of a step transposed, from the fused projection: vt[kv head, dv, column],
    sequence b from column tile_off[b] on (`aligned_columns`), written by tiles of 64
    positions in whole lines.  Columns that hold no position of this step are left alone."""
    n = qkv.shape[0]
    _req(qkv, "v_tiles.qkv", torch.float32, (n, (nq + 2 * nkv) * d))
    _req(vt, "v_tiles.vt")
    if vt.dim() != 3 or tuple(vt.shape[:2]) != (nkv, d) or vt.shape[2] % PAGE:
        raise KernelError(f"v_tiles.vt: shape {tuple(vt.shape)}, kernel needs [{nkv}, {d}, a multiple of {PAGE}]")
    B = tile_off.shape[0]
    _tiles_args(B, cu_seqlens, tile_off, n_cached, len_after, "v_tiles")
    _check(lib().tl_v_tiles(_p(qkv), n, nq, nkv, d, _p(vt), vt.shape[2], _code(vt.dtype), B, _p(cu_seqlens),
                            _p(tile_off), _p(n_cached), _p(len_after), _stream()))


def rope_v_tiles(qkv: torch.Tensor, row_pos, rotation, nq: int, nkv: int, d: int, q: torch.Tensor, k: torch.Tensor,
                 vt: torch.Tensor, cu_seqlens, tile_off, n_cached, len_after) -> None:
    """`rope_split` (q and k) and `v_tiles` in one launch: the same bits as the two."""
    n = qkv.shape[0]
    _req(qkv, "rope_v_tiles.qkv", torch.float32, (n, (nq + 2 * nkv) * d))
    _req(row_pos, "rope_v_tiles.row_pos", torch.int32, (n,))
    rot = _rotation(rotation, d, "rope_v_tiles")
    _req(q, "rope_v_tiles.q", None, (n, nq, d))
    _req(k, "rope_v_tiles.k", q.dtype, (n, nkv, d))
    _req(vt, "rope_v_tiles.vt", q.dtype)
    if vt.dim() != 3 or tuple(vt.shape[:2]) != (nkv, d) or vt.shape[2] % PAGE:
        raise KernelError(f"rope_v_tiles.vt: shape {tuple(vt.shape)}, kernel needs [{nkv}, {d}, a multiple of {PAGE}]")
    B = tile_off.shape[0]
    _tiles_args(B, cu_seqlens, tile_off, n_cached, len_after, "rope_v_tiles")
    if cu_seqlens is None:
        raise KernelError("rope_v_tiles.cu_seqlens: needed")
    _check(lib().tl_rope_v_tiles(_p(qkv), _p(row_pos), _p(rot.inv_freq), rot.rotary_dim, int(rot.interleaved), n, nq,
                                 nkv, d, _p(q), _p(k), _p(vt), vt.shape[2], B, _p(cu_seqlens), _p(tile_off),
                                 _p(n_cached), _p(len_after), _code(q.dtype), _stream()))


def kv_commit_tiles(k: torch.Tensor, vt: torch.Tensor, row_seq, row_pos, tile_off, n_cached, len_after,
                    table: torch.Tensor, ring_pages: int, pages: torch.Tensor) -> None:
    """`kv_commit` for a step whose values lie transposed by tiles (`v_tiles`): keys row by
    row, values a tile [d, 64] at a time in whole lines."""
    n, nkv, d = k.shape
    _req(k, "kv_commit.k", pages.dtype)
    _req(vt, "kv_commit.vt", pages.dtype)
    if vt.dim() != 3 or tuple(vt.shape[:2]) != (nkv, d) or vt.shape[2] % PAGE:
        raise KernelError(f"kv_commit.vt: shape {tuple(vt.shape)}, kernel needs [{nkv}, {d}, a multiple of {PAGE}]")
    _req(row_seq, "kv_commit.row_seq", torch.int32, (n,))
    _req(row_pos, "kv_commit.row_pos", torch.int32, (n,))
    B = tile_off.shape[0]
    _tiles_args(B, None, tile_off, n_cached, len_after, "kv_commit")
    _req(table, "kv_commit.table", torch.int32)
    _req(pages, "kv_commit.pages")
    if pages.dim() != 5 or tuple(pages.shape[1:]) != (2, nkv, PAGE, d):
        raise KernelError(f"kv_commit.pages: shape {tuple(pages.shape)}, kernel needs [*, 2, {nkv}, {PAGE}, {d}]")
    if table.dim() != 2 or table.shape[0] != B:
        raise KernelError("kv_commit.table: needs one row per sequence")
    _check(lib().tl_kv_commit_tiles(_p(k), _p(vt), vt.shape[2], _code(k.dtype), _p(row_seq), _p(row_pos), B,
                                    _p(tile_off), _p(n_cached), _p(len_after), _p(table), table.shape[1],
                                    ring_pages, n, nkv, d, _p(pages), _stream()))


def attn_plain(q, k_new, v_new, pages, table, ring_pages: int, row_seq, row_pos, cu_seqlens, n_cached,
               window: Optional[int], scale: float, out) -> None:
    """Attention of every row over its sequence's cached keys (j < n_cached)
    and this step's keys (k_new/v_new rows), causal, with an optional window."""
    n, nq, d = q.shape
    nkv = pages.shape[2]
    B = n_cached.shape[0]
    _req(q, "attn.q", pages.dtype)
    if k_new is not None:
        _req(k_new, "attn.k_new", pages.dtype, (n, nkv, d))
        _req(v_new, "attn.v_new", pages.dtype, (n, nkv, d))
    _req(pages, "attn.pages")
    if pages.dim() != 5 or tuple(pages.shape[1:]) != (2, nkv, PAGE, d):
        raise KernelError(f"attn.pages: shape {tuple(pages.shape)}, kernel needs [*, 2, nkv, {PAGE}, {d}]")
    _req(table, "attn.table", torch.int32)
    _req(row_seq, "attn.row_seq", torch.int32, (n,))
    _req(row_pos, "attn.row_pos", torch.int32, (n,))
    _req(cu_seqlens, "attn.cu_seqlens", torch.int32, (B + 1,))
    _req(n_cached, "attn.n_cached", torch.int32, (B,))
    _req(out, "attn.out", pages.dtype, (n, nq, d))
    if table.dim() != 2 or table.shape[0] != B:
        raise KernelError("attn.table: needs one row per sequence")
    _check(lib().tl_attn_plain(_p(q), _p(k_new), _p(v_new), _p(pages), _code(q.dtype), _p(table),
                               table.shape[1], ring_pages, _p(row_seq), _p(row_pos), _p(cu_seqlens),
                               _p(n_cached), n, nq, nkv, d, int(window or 0), ctypes.c_float(scale),
                               _p(out), _stream()))


def silu_mul(gu: torch.Tensor, out: torch.Tensor) -> None:
    """out[n, i] = silu(gu[n, i]) * gu[n, I + i]."""
    n, I2 = gu.shape
    _req(gu, "silu_mul.gu", torch.float32)
    _req(out, "silu_mul.out", None, (n, I2 // 2))
    _check(lib().tl_silu_mul(_p(gu), n, I2 // 2, _p(out), _code(out.dtype), _stream()))


def silu_mul_pairs(gu: torch.Tensor, out: torch.Tensor) -> None:
    """The same on bfloat16 gu whose columns come in groups of 64: 32 of gate,
    then the 32 of up that belong to them (`interleave_pairs`)."""
    n, I2 = gu.shape
    _req(gu, "silu_mul_pairs.gu", torch.bfloat16)
    _req(out, "silu_mul_pairs.out", torch.bfloat16, (n, I2 // 2))
    _check(lib().tl_silu_mul_pairs(_p(gu), n, I2 // 2, _p(out), _stream()))


def take_tokens(src: torch.Tensor, idx: torch.Tensor, vocab: int, tokens: torch.Tensor) -> None:
    """tokens[j] = src[idx[j]] (int32, on the device); ids outside [0, vocab) become 0."""
    n = tokens.shape[0]
    _req(src, "take_tokens.src", torch.int32)
    _req(idx, "take_tokens.idx", torch.int32, (n,))
    _req(tokens, "take_tokens.tokens", torch.int32, (n,))
    _check(lib().tl_take_tokens(_p(src), _p(idx), n, src.numel(), int(vocab), _p(tokens), _stream()))


def gather_rows(x: torch.Tensor, idx: torch.Tensor, out: torch.Tensor) -> None:
    m, H = idx.shape[0], x.shape[1]
    _req(x, "gather.x", torch.float32)
    _req(idx, "gather.idx", torch.int32, (m,))
    _req(out, "gather.out", torch.float32, (m, H))
    _check(lib().tl_gather_rows(_p(x), _p(idx), m, H, _p(out), _stream()))


def gemm_plain(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """out[M,N] (+)= a[M,K] @ w[N,K]^T, float32 accumulation in plain FMA."""
    M, K = a.shape
    N = w.shape[0]
    _req(a, "gemm.a")
    _req(w, "gemm.w", None, (N, K))
    _req(out, "gemm.out", torch.float32, (M, N))
    _check(lib().tl_gemm_plain(_p(a), _code(a.dtype), _p(w), _code(w.dtype), _p(out), M, N, K, K, K, N,
                               int(accumulate), _stream()))


def sample(logits: torch.Tensor, temperature: float, top_k: int, top_p: float, seed: int,
           counters: torch.Tensor, probs: torch.Tensor, out: torch.Tensor) -> None:
    """One token per row.  counters[b] = (sequence, step) feeds the generator;
    probs receives the distribution the draw was made from (when T > 0)."""
    B, V = logits.shape
    _req(logits, "sample.logits", torch.float32)
    _req(counters, "sample.counters", torch.int32, (B, 2))
    _req(probs, "sample.probs", torch.float32, (B, V))
    _req(out, "sample.out", torch.int32, (B,))
    _check(lib().tl_sample(_p(logits), B, V, ctypes.c_float(temperature), int(top_k),
                           ctypes.c_float(top_p), ctypes.c_ulonglong(seed & (2 ** 64 - 1)),
                           _p(counters), _p(probs), _p(out), _stream()))


EPI_STORE, EPI_ACCUMULATE, EPI_SILU_PAIR = 0, 1, 2


def tiles_fit(N: int, K: int) -> bool:
    """Can a weight [N, K] have a tiled copy?"""
    return N % 16 == 0 and K % 64 == 0


def tile_height(N: int) -> int:
    """Rows of a tile of the tiled copy of a weight with N rows: the channels that a workgroup of the
    products for at most 16 rows owns (16; more where the device has fewer compute units than the
    weight has tiles of 16, so that the units get equal shares)."""
    return int(lib().tl_tile_height(int(N)))


def tile_weights(w: torch.Tensor, rows: Optional[torch.Tensor] = None, height: Optional[int] = None) -> torch.Tensor:
    """The copy of w [N, K] (bfloat16, N % 16 == 0, K % 64 == 0) that the products for at most
    16 rows stream from: [ceil(N / R), K/64, 2, 4, R, 8] with element (T, s, c, g, r, e) =
    w[rows[R T + r], 64 s + 16 g + 8 c + e], so that what a workgroup reads is one run of memory (and
    with R = 16 what a wave loads at a time, lane after lane).  `rows` (int32 [N], on the device): a
    permutation of the rows; None: none.  `height`: R; None: `tile_height(N)`, or 16 with `rows`
    (the kernel that wants its own order reads tiles of 16).  Places of the last tile behind row N are
    zero."""
    N, K = w.shape
    _req(w, "tile_weights.w", torch.bfloat16)
    if not tiles_fit(N, K):
        raise KernelError(f"tile_weights: N={N} must be a multiple of 16 and K={K} of 64")
    if rows is not None:
        _req(rows, "tile_weights.rows", torch.int32, (N,))
    R = int(height) if height is not None else (16 if rows is not None else tile_height(N))
    if not 16 <= R <= 32:
        raise KernelError(f"tile_weights: tiles of {R} rows (16 to 32)")
    n_tiles = -(-N // R)
    make = torch.empty if n_tiles * R == N else torch.zeros
    out = make((n_tiles, K // 64, 2, 4, R, 8), dtype=torch.bfloat16, device=w.device)
    _check(lib().tl_tile_weights(_p(w), _p(rows), N, K, R, _p(out), _stream()))
    return out


def qkv_tile_rows(nq: int, nkv: int, d: int, device, rotation=None) -> torch.Tensor:
    """The order of the rows of w = q|k|v in the tiled copy that `qkv_rope_commit` reads
    (a tile of a q or k head holds both channels of 8 pairs of `rotation`; None: the whole
    head rotated in halves)."""
    n = (nq + 2 * nkv) * d
    buf = (ctypes.c_int * n)()
    rotary_dim, interleaved = (d, False) if rotation is None else (rotation.rotary_dim, rotation.interleaved)
    _check(lib().tl_qkv_tile_rows(int(nq), int(nkv), int(d), int(rotary_dim), int(interleaved), buf))
    return torch.tensor(list(buf), dtype=torch.int32, device=device)


def _req_tiles(tiles: Optional[torch.Tensor], N: int, K: int, height: Optional[int] = None) -> int:
    """Check a tiled copy of a weight [N, K] (`height`: the only tile height the caller reads) and
    return its tile height (16 where there is no copy)."""
    if tiles is None:
        return 16
    if not tiles_fit(N, K):
        raise KernelError(f"gemm.tiles: a weight [{N}, {K}] has no tiled copy")
    R = int(tiles.shape[4]) if tiles.dim() == 6 else 0
    if R < 16 or (height is not None and R != height):
        raise KernelError(f"gemm.tiles: shape {tuple(tiles.shape)} is no tiled copy"
                          + (f" with tiles of {height} rows" if height is not None else ""))
    _req(tiles, "gemm.tiles", torch.bfloat16, (-(-N // R), K // 64, 2, 4, R, 8))
    return R


def gemm_bf16(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False,
              variant: Optional[int] = None, silu_pair: bool = False,
              tiles: Optional[torch.Tensor] = None) -> None:
    """out[M,N] (+)= a[M,K] @ w[N,K]^T on the matrix cores: bfloat16 operands,
    float32 accumulation.  K must be a multiple of 8.  With `silu_pair`, w's
    rows come in groups of 64 (32 gate rows and the 32 up rows that belong to
    them) and out is bfloat16 [M, N/2] = silu(gate) * up.  `variant` (tests
    and tuning) forces one kernel.  `tiles`: `tile_weights(w)`, read instead of
    w by the kernel for at most 16 rows and 16 to 32 channels a workgroup."""
    M, K = a.shape
    N = w.shape[0]
    _req(a, "gemm.a", torch.bfloat16)
    _req(w, "gemm.w", torch.bfloat16, (N, K))
    th = _req_tiles(tiles, N, K)
    if silu_pair:
        if accumulate or N % 64:
            raise KernelError("gemm: the paired epilogue stores, and needs N to be a multiple of 64")
        _req(out, "gemm.out", torch.bfloat16, (M, N // 2))
        epi = EPI_SILU_PAIR
    else:
        _req(out, "gemm.out", torch.float32, (M, N))
        epi = EPI_ACCUMULATE if accumulate else EPI_STORE
    if variant is None:
        _check(lib().tl_gemm_bf16(_p(a), _p(w), _p(tiles), th, _p(out), M, N, K, epi, _stream()))
    else:
        _check(lib().tl_gemm_bf16_variant(_p(a), _p(w), _p(out), M, N, K, epi, int(variant), _stream()))


class RowFactor:
    """The second half of an RMSNorm cut in two around a product: sums of x^2 per
    workgroup of the product that wrote the stream (`ssq` [16, n_part], float32), from
    which the reading product makes rsqrt(sum / size + eps) per row."""

    def __init__(self, ssq: torch.Tensor, n_part: int, size: int, eps: float):
        self.ssq, self.n_part, self.size, self.eps = ssq, int(n_part), int(size), float(eps)


def norm_split_ok(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Can `gemm_bf16_norm` take this product (bfloat16, at most 16 rows)?"""
    return bf16_gemm_ok(a, w) and a.shape[0] <= 16


def gemm_bf16_norm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False,
                   silu_pair: bool = False, factor: Optional[RowFactor] = None,
                   norm_weight: Optional[torch.Tensor] = None, xt: Optional[torch.Tensor] = None,
                   ssq_out: Optional[torch.Tensor] = None, tiles: Optional[torch.Tensor] = None) -> int:
    """`gemm_bf16` for at most 16 rows with the halves of an RMSNorm around it.
    `factor`: every row of the result is multiplied by its rsqrt(mean(x^2) + eps).
    `norm_weight`, `xt`, `ssq_out` (with `accumulate`): out += product, xt =
    bfloat16(out * norm_weight), ssq_out[m, g] = the sum of out[m, :]^2 over workgroup g's
    channels.  `tiles`: see `gemm_bf16`.  Returns the number of workgroups (the reader's n_part)."""
    M, K = a.shape
    N = w.shape[0]
    _req(a, "gemm.a", torch.bfloat16)
    _req(w, "gemm.w", torch.bfloat16, (N, K))
    th = _req_tiles(tiles, N, K)
    if silu_pair:
        if accumulate or N % 64:
            raise KernelError("gemm: the paired epilogue stores, and needs N to be a multiple of 64")
        _req(out, "gemm.out", torch.bfloat16, (M, N // 2))
        epi = EPI_SILU_PAIR
    else:
        _req(out, "gemm.out", torch.float32, (M, N))
        epi = EPI_ACCUMULATE if accumulate else EPI_STORE
    ssq_in, n_part, inv_h, eps = None, 0, 0.0, 0.0
    if factor is not None:
        _req(factor.ssq, "gemm.factor", torch.float32)
        if factor.ssq.numel() < factor.n_part * 16 or factor.n_part < 1:
            raise KernelError(f"gemm.factor: {factor.ssq.numel()} floats for {factor.n_part} workgroups")
        ssq_in, n_part, inv_h, eps = factor.ssq, factor.n_part, 1.0 / factor.size, factor.eps
    cap = 0
    if norm_weight is not None:
        _req(norm_weight, "gemm.norm_weight", torch.float32, (N,))
        _req(xt, "gemm.xt", torch.bfloat16, (M, N))
        _req(ssq_out, "gemm.ssq_out", torch.float32)
        cap = ssq_out.numel()
    groups = ctypes.c_int(0)
    _check(lib().tl_gemm_bf16_norm(_p(a), _p(w), _p(tiles), th, _p(out), M, N, K, epi, _p(ssq_in), n_part,
                                   ctypes.c_float(inv_h), ctypes.c_float(eps), _p(norm_weight), _p(xt),
                                   _p(ssq_out), cap, ctypes.byref(groups), _stream()))
    return groups.value


MID_ROWS = 128      # most rows of the kernels that share a step's activations through LDS
RING_K = 128        # the kernel that brings both operands into a ring of LDS stages takes K in multiples of this
LIBRARY_ROWS = 64   # where K is no such multiple, the BLAS library's product beats ours above this many rows


def own_rows(K: int) -> int:
    """The most rows for which a bfloat16 product over K runs in this package's own kernels (more
    go to the BLAS library)."""
    return MID_ROWS if K % RING_K == 0 else LIBRARY_ROWS


_UNITS: dict = {}


def compute_units(device) -> int:
    """Compute units of the device (256 on an MI355X)."""
    key = str(device)
    if key not in _UNITS:
        _UNITS[key] = int(torch.cuda.get_device_properties(device).multi_processor_count)
    return _UNITS[key]


def mid_splits(M: int, N: int, K: int, units: int) -> int:
    """For 17..MID_ROWS rows: into how many slices K is cut, each a workgroup's own, whose partial
    sums the next kernel adds up; 1 where N alone gives the workgroups.

    K a multiple of RING_K (the ring kernel: 128 channels a workgroup, which holds a compute unit by
    itself): as many slices as make one round of workgroups over the `units` compute units, each
    with four stages of 128 k at least (o and down of the 7B shape at 64 rows: 8 slices, 256
    workgroups, 9.4 and 22.2 us; q|k|v: 5).

    Other K (gemm_mid: 64 channels a workgroup, steps of 256 k): so that some 400 workgroups or more
    are at work, a power of two; twice as many where only that fills the compute units evenly."""
    if K % RING_K == 0:
        blocks = -(-N // 128)
        return max(1, min(units // blocks, (K // RING_K) // 4, 16))
    blocks = -(-N // 64)
    steps = -(-K // 256)
    want = -(-400 // blocks)
    S = 1
    while S < want and S < 16:
        S *= 2
    if 1 < S < 16 and 2 * S <= steps and (blocks * S) % units != 0 and (blocks * 2 * S) % units == 0:
        S *= 2
    while S > steps:
        S //= 2
    return max(1, S)


def gemm_mid_bf16(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, n_split: int = 1,
                  accumulate: bool = False, silu_pair: bool = False) -> None:
    """The product for 17..MID_ROWS rows (the ring kernel where K is a multiple of RING_K, else
    gemm_mid).  n_split == 1: out as in `gemm_bf16`.  n_split > 1: out is float32 [n_split, M, N]
    and receives partial sums that the next kernel adds up (`add_rmsnorm`, `add_partials`,
    `rope_commit`)."""
    M, K = a.shape
    N = w.shape[0]
    _req(a, "gemm.a", torch.bfloat16)
    _req(w, "gemm.w", torch.bfloat16, (N, K))
    if n_split > 1:
        if accumulate or silu_pair:
            raise KernelError("gemm_mid: partial sums cannot be accumulated or paired")
        _req(out, "gemm.out", torch.float32, (n_split, M, N))
        epi = EPI_STORE
    elif silu_pair:
        _req(out, "gemm.out", torch.bfloat16, (M, N // 2))
        epi = EPI_SILU_PAIR
    else:
        _req(out, "gemm.out", torch.float32, (M, N))
        epi = EPI_ACCUMULATE if accumulate else EPI_STORE
    _check(lib().tl_gemm_mid_bf16(_p(a), _p(w), _p(out), M, N, K, int(n_split), epi, _stream()))


def gemm_ring_bf16(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, n_split: int = 1, accumulate: bool = False,
                   silu_pair: bool = False, waves: int = 4, kc: int = 128) -> None:
    """`gemm_mid_bf16` through the kernel that brings both operands into a ring of stages in LDS
    (K a multiple of 128); `waves`: 4, 7 or 8 waves a workgroup with 16 channels each; `kc`: the k
    of a stage, 64 or 128."""
    M, K = a.shape
    N = w.shape[0]
    _req(a, "gemm.a", torch.bfloat16)
    _req(w, "gemm.w", torch.bfloat16, (N, K))
    if n_split > 1:
        if accumulate or silu_pair:
            raise KernelError("gemm_ring: partial sums cannot be accumulated or paired")
        _req(out, "gemm.out", torch.float32, (n_split, M, N))
        epi = EPI_STORE
    elif silu_pair:
        _req(out, "gemm.out", torch.bfloat16, (M, N // 2))
        epi = EPI_SILU_PAIR
    else:
        _req(out, "gemm.out", torch.float32, (M, N))
        epi = EPI_ACCUMULATE if accumulate else EPI_STORE
    _check(lib().tl_gemm_ring_bf16(_p(a), _p(w), _p(out), M, N, K, int(n_split), epi, int(waves), int(kc), _stream()))


def add_rmsnorm(x: torch.Tensor, parts: torch.Tensor, w: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    """x += parts[0] + parts[1] + ... (float32 [S, n, H]); out = rmsnorm(x)."""
    n, H = x.shape
    _req(x, "add_rmsnorm.x", torch.float32)
    _req(parts, "add_rmsnorm.parts", torch.float32)
    if parts.dim() != 3 or tuple(parts.shape[1:]) != (n, H):
        raise KernelError(f"add_rmsnorm.parts: shape {tuple(parts.shape)}, kernel needs [S, {n}, {H}]")
    _req(w, "add_rmsnorm.w", torch.float32, (H,))
    _req(out, "add_rmsnorm.out", None, (n, H))
    _check(lib().tl_add_rmsnorm(_p(x), _p(parts), parts.shape[0], _p(w), ctypes.c_float(eps), _p(out),
                                _code(out.dtype), n, H, _stream()))


def add_partials(x: torch.Tensor, parts: torch.Tensor) -> None:
    """x += parts[0] + parts[1] + ... (float32 [S, n, H])."""
    n, H = x.shape
    _req(x, "add_partials.x", torch.float32)
    _req(parts, "add_partials.parts", torch.float32)
    if parts.dim() != 3 or tuple(parts.shape[1:]) != (n, H):
        raise KernelError(f"add_partials.parts: shape {tuple(parts.shape)}, kernel needs [S, {n}, {H}]")
    _check(lib().tl_add_partials(_p(x), _p(parts), parts.shape[0], n, H, _stream()))


def gemm_library(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """out[M,N] (+)= a[M,K] @ w[N,K]^T through the BLAS library (hipBLASLt below
    torch): bfloat16 operands, float32 accumulation; out is float32, or bfloat16
    when it is only stored.  The reference hands its products to the vendor's
    library likewise (src/kernels/cuda/mod.rs:462-552, src/kernels/rocm/mod.rs)."""
    M, K = a.shape
    N = w.shape[0]
    _req(a, "gemm.a", torch.bfloat16)
    _req(w, "gemm.w", torch.bfloat16, (N, K))
    _req(out, "gemm.out", None, (M, N))
    if out.dtype == torch.float32:
        if accumulate:
            torch.addmm(out, a, w.t(), out_dtype=torch.float32, out=out)
        else:
            torch.mm(a, w.t(), out_dtype=torch.float32, out=out)
    elif out.dtype == torch.bfloat16 and not accumulate:
        torch.mm(a, w.t(), out=out)
    else:
        raise KernelError(f"gemm_library: cannot {'accumulate into' if accumulate else 'store'} {out.dtype}")


def bf16_gemm_ok(a: torch.Tensor, w: torch.Tensor) -> bool:
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.shape[1] % 8 == 0
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False,
         tiles: Optional[torch.Tensor] = None) -> None:
    """out[M,N] (+)= a[M,K] @ w[N,K]^T with float32 accumulation.  The kernel
    follows from the operand types: bfloat16 x bfloat16 goes to the matrix
    cores (our kernels up to `own_rows(K)` rows, the library's above), anything
    with float32 in it to the plain FMA kernel.  `tiles`: see `gemm_bf16`."""
    if bf16_gemm_ok(a, w):
        if a.shape[0] > own_rows(a.shape[1]):
            gemm_library(a, w, out, accumulate)
        elif a.shape[0] > LIBRARY_ROWS:
            gemm_mid_bf16(a, w, out, 1, accumulate)
        else:
            gemm_bf16(a, w, out, accumulate, tiles=tiles)
    else:
        gemm_plain(a, w, out, accumulate)


def rope_commit(qkv: torch.Tensor, row_pos, rotation, table, ring_pages: int, nq: int, nkv: int, d: int,
                q: torch.Tensor, pages: torch.Tensor) -> None:
    """Single-token steps: rotate q and k (`rotation`: see `rope_split`), write q [n,nq,d] and
    put k and v of row n straight into sequence n's page for its position.  qkv may be
    [S, n, width]: partial products that are added up on the way in."""
    n_parts = qkv.shape[0] if qkv.dim() == 3 else 1
    n = qkv.shape[-2]
    _req(qkv, "rope.qkv", torch.float32, ((n_parts,) if qkv.dim() == 3 else ()) + (n, (nq + 2 * nkv) * d))
    _req(row_pos, "rope.row_pos", torch.int32, (n,))
    rot = _rotation(rotation, d, "rope")
    _req(q, "rope.q", pages.dtype, (n, nq, d))
    _req(table, "rope.table", torch.int32)
    _req(pages, "rope.pages")
    if pages.dim() != 5 or tuple(pages.shape[1:]) != (2, nkv, PAGE, d):
        raise KernelError(f"rope.pages: shape {tuple(pages.shape)}, kernel needs [*, 2, {nkv}, {PAGE}, {d}]")
    if table.dim() != 2 or table.shape[0] != n:
        raise KernelError("rope.table: needs one row per sequence")
    _check(lib().tl_rope_commit(_p(qkv), n_parts, _p(row_pos), _p(rot.inv_freq), rot.rotary_dim,
                                int(rot.interleaved), _p(table), table.shape[1], ring_pages,
                                n, nq, nkv, d, _p(q), _p(pages), _code(q.dtype), _stream()))


def qkv_rope_commit_ok(a: torch.Tensor, w: torch.Tensor, d: int, pages: torch.Tensor) -> bool:
    """Whether `qkv_rope_commit` serves this step: bfloat16 all through, at most 16 rows."""
    return bf16_gemm_ok(a, w) and a.shape[0] <= 16 and d % 16 == 0 and pages.dtype == torch.bfloat16


def qkv_rope_commit(a: torch.Tensor, w: torch.Tensor, row_pos, rotation, table, ring_pages: int, nq: int,
                    nkv: int, d: int, q: torch.Tensor, pages: torch.Tensor,
                    factor: Optional[RowFactor] = None, units: int = 0,
                    tiles: Optional[torch.Tensor] = None) -> None:
    """For a step with one token a sequence (at most 16): the product a @ w^T with w = q|k|v,
    the rotation of q and k, q into its buffer and k, v into the pages, in one kernel; the
    same bits as `gemm` and then `rope_commit`.  `factor`: see `gemm_bf16_norm`.  `units`
    (tests): how many units of 8 weight rows a workgroup owns, 1 to 4; 0 leaves it to the launcher.
    `tiles`: `tile_weights(w, qkv_tile_rows(nq, nkv, d, device, rotation))`, read instead of w.
    `rotation`: see `rope_split`."""
    n, K = a.shape
    _req(a, "qkv_rope_commit.a", torch.bfloat16)
    _req(w, "qkv_rope_commit.w", torch.bfloat16, ((nq + 2 * nkv) * d, K))
    _req_tiles(tiles, (nq + 2 * nkv) * d, K, height=16)
    _req(row_pos, "qkv_rope_commit.row_pos", torch.int32, (n,))
    rot = _rotation(rotation, d, "qkv_rope_commit")
    _req(q, "qkv_rope_commit.q", torch.bfloat16, (n, nq, d))
    _req(table, "qkv_rope_commit.table", torch.int32)
    _req(pages, "qkv_rope_commit.pages", torch.bfloat16)
    if pages.dim() != 5 or tuple(pages.shape[1:]) != (2, nkv, PAGE, d):
        raise KernelError(f"qkv_rope_commit.pages: shape {tuple(pages.shape)}, kernel needs [*, 2, {nkv}, {PAGE}, {d}]")
    if table.dim() != 2 or table.shape[0] != n:
        raise KernelError("qkv_rope_commit.table: needs one row per sequence")
    ssq_in, n_part, inv_h, eps = None, 0, 0.0, 0.0
    if factor is not None:
        _req(factor.ssq, "qkv_rope_commit.factor", torch.float32)
        if factor.ssq.numel() < factor.n_part * 16 or factor.n_part < 1:
            raise KernelError(f"qkv_rope_commit.factor: {factor.ssq.numel()} floats for {factor.n_part} workgroups")
        ssq_in, n_part, inv_h, eps = factor.ssq, factor.n_part, 1.0 / factor.size, factor.eps
    _check(lib().tl_gemm_qkv_rope_commit(_p(a), _p(w), _p(tiles), n, K, _p(row_pos), _p(rot.inv_freq),
                                         rot.rotary_dim, int(rot.interleaved), _p(table),
                                         table.shape[1], int(ring_pages), nq, nkv, d, _p(q), _p(pages),
                                         _p(ssq_in), n_part, ctypes.c_float(inv_h), ctypes.c_float(eps),
                                         int(units), _stream()))


def aligned_columns(n_cached, n_new):
    """Column offsets (and their total) at which sequences lie when each is
    given room from the last multiple of 64 below its cached length up to its
    end, rounded up to 64: positions that are multiples of 64 then lie on
    columns that are.  The total is the row length of buffers laid out so (kept
    off multiples of 512: rows a power of two apart would all fall on the same
    memory channels).  The rule is the host library's, which lays out steps."""
    import numpy as np
    from ..cache import native
    c = np.ascontiguousarray(np.asarray(list(n_cached), dtype=np.int64))
    n = np.ascontiguousarray(np.asarray(list(n_new), dtype=np.int64))
    off = np.zeros(len(c), dtype=np.int32)
    total = native.lib().tl_aligned_columns(len(c), c.ctypes.data, n.ctypes.data, off.ctypes.data)
    return off.tolist(), int(total)


PREFILL_BLOCK = 128            # rows of a sequence that one workgroup of the multi-token attention takes
PREFILL_CUT_TILES = 8          # fewest tiles of 64 keys of a run into which a block's keys are cut
PREFILL_MAX_WAYS = 8           # most runs of a block


class PrefillCuts:
    """How the host lays out the work of the multi-token attention for a step with fewer workgroups than
    the device has compute units: `items` int32 [n, 4] on the device, rows (sequence, block, first tile of
    keys, one past the last | slot << 24 | (ways - 1) << 27 | 1 << 30) with the dearest last for one of the
    `ways` runs into which a block's keys are cut, (sequence, block, 0, 0) for a whole block; `blocks` int32 [n_cut, 4], the (sequence,
    block, ways, 0) that are cut; `ways`: the most runs of any block (the places a row has for its sums)."""

    def __init__(self, entries, blocks, n_seqs: int, n_tiles: int, device):
        self.n_items, self.n_cut, self.n_seqs, self.n_tiles = len(entries), len(blocks), n_seqs, n_tiles
        self.ways = max(w for _, _, w in blocks)
        flat = torch.tensor([v for e in entries for v in e] + [v for b in blocks for v in (*b, 0)], dtype=torch.int32)
        dev = flat.to(device)
        self.items = dev[:4 * len(entries)].view(-1, 4)
        self.blocks = dev[4 * len(entries):].view(-1, 4)


def prefill_layout(n_new, len_before, window: Optional[int], nq: int, units: int):
    """The host's side of `prefill_cuts`: (entries, cut blocks, number of blocks), or None where the
    kernel's own order serves.  A launch with fewer workgroups (blocks of 128 rows x heads) than
    compute units leaves units idle while its longest chain of key tiles runs: then a block's keys are cut
    into as many runs as there are units for (`PREFILL_MAX_WAYS` at most, `PREFILL_CUT_TILES` tiles a run at
    least), each run a workgroup of its own, and a second kernel merges their sums.  (A launch that fills the
    device gains nothing: one prompt of 2,048 tokens takes 81 us cut in two against 75.)"""
    global _last_layout
    key = (tuple(int(n) for n in n_new), tuple(int(c) for c in len_before), window, nq, units, PREFILL_CUT_TILES)
    if _last_layout is not None and _last_layout[0] == key:       # every layer of a step asks the same
        return _last_layout[1]
    laid = _prefill_layout(key[0], key[1], window, nq, units)
    _last_layout = (key, laid)
    return laid


_last_layout = None


def _prefill_layout(n_new, len_before, window, nq, units):
    n_blocks = sum(-(-n // PREFILL_BLOCK) for n in n_new)
    if n_blocks == 0 or n_blocks * nq > units:
        return None
    # with a workgroup for more than every other unit only chains twice as long are worth the merge
    # (1,024 tokens alone, 256 workgroups of at most 16 tiles: 43.8 us with the last block cut in two against 40.3)
    run = PREFILL_CUT_TILES * (1 if n_blocks * nq * 2 <= units else 2)
    if max(c + n for c, n in zip(len_before, n_new)) <= (2 * run - 1) * PAGE:
        return None                               # no sequence reaches into the last tile of two runs
    blocks = [(b, t) for b, n in enumerate(n_new) for t in range(-(-n // PREFILL_BLOCK))]
    most = min(PREFILL_MAX_WAYS, 2 * units // (len(blocks) * nq))      # (a compute unit holds two workgroups)
    entries, cut = [], []
    for b, t in blocks:
        first = int(len_before[b])
        p_lo = first + t * PREFILL_BLOCK
        p_hi = first + min((t + 1) * PREFILL_BLOCK, int(n_new[b])) - 1
        j_lo = max(0, p_lo - window + 1) if window else 0
        jt_first, jt_last = j_lo // PAGE, p_hi // PAGE
        tiles = jt_last - jt_first + 1
        ways = min(most, tiles // run)
        if ways < 2:
            entries.append((tiles, (b, t, 0, 0)))
            continue
        cut.append((b, t, ways))
        for w in range(ways):
            lo, hi = jt_first + tiles * w // ways, jt_first + tiles * (w + 1) // ways
            if hi >= 1 << 24:
                return None                   # (a tile index beyond the entry's 24 bits)
            entries.append((hi - lo, (b, t, lo, hi | (w << 24) | ((ways - 1) << 27) | (1 << 30))))
    if not cut:
        return None
    entries.sort(key=lambda e: e[0])
    return [e[1] for e in entries], cut, len(blocks)


def prefill_cuts(n_new, len_before, window: Optional[int], nq: int, units: int, device) -> Optional[PrefillCuts]:
    """The layout (`prefill_layout`) for a step whose sequences bring `n_new` rows after `len_before`
    positions, on the device, or None where the kernel's own order serves."""
    laid = prefill_layout(n_new, len_before, window, nq, units)
    if laid is None:
        return None
    return PrefillCuts(laid[0], laid[1], len(n_new), laid[2], device)


def prefill_serves(dtype: torch.dtype, d: int) -> bool:
    """Does the multi-token attention on the matrix cores serve this dtype and head size?"""
    return dtype == torch.bfloat16 and d % 16 == 0 and 16 <= d <= 256


def attn_prefill_bf16(q, k_new, vt_new, tile_off, pages, table, ring_pages: int, row_pos, cu_seqlens,
                      n_cached, n_tiles: int, window: Optional[int], scale: float, out,
                      cuts: Optional[PrefillCuts] = None, part: Optional[torch.Tensor] = None) -> None:
    """bfloat16 attention for steps with many rows per sequence.  `vt_new`:
    this step's values transposed [nkv, d, cols] at the columns that
    `aligned_columns` gives (`tile_off`).  `n_tiles`: sum over the sequences
    of ceil(rows / 128).  `cuts` (`prefill_cuts` of this step) with `part`, float32 scratch of
    n * nq * cuts.ways * (d + 4) elements: the keys of long blocks go to several workgroups each."""
    n, nq, d = q.shape
    nkv = pages.shape[2]
    B = n_cached.shape[0]
    _req(q, "attn.q", torch.bfloat16)
    _req(k_new, "attn.k_new", torch.bfloat16, (n, nkv, d))
    _req(vt_new, "attn.vt_new", torch.bfloat16)
    if vt_new.dim() != 3 or tuple(vt_new.shape[:2]) != (nkv, d) or vt_new.shape[2] % PAGE:
        raise KernelError(f"attn.vt_new: shape {tuple(vt_new.shape)}, kernel needs [{nkv}, {d}, a multiple of {PAGE}]")
    _req(tile_off, "attn.tile_off", torch.int32, (B,))
    _req(pages, "attn.pages", torch.bfloat16)
    if pages.dim() != 5 or tuple(pages.shape[1:]) != (2, nkv, PAGE, d):
        raise KernelError(f"attn.pages: shape {tuple(pages.shape)}, kernel needs [*, 2, nkv, {PAGE}, {d}]")
    _req(table, "attn.table", torch.int32)
    _req(row_pos, "attn.row_pos", torch.int32, (n,))
    _req(cu_seqlens, "attn.cu_seqlens", torch.int32, (B + 1,))
    _req(n_cached, "attn.n_cached", torch.int32, (B,))
    _req(out, "attn.out", torch.bfloat16, (n, nq, d))
    if table.dim() != 2 or table.shape[0] != B:
        raise KernelError("attn.table: needs one row per sequence")
    if cuts is None:
        _check(lib().tl_attn_prefill_bf16(_p(q), _p(k_new), _p(vt_new), vt_new.shape[2], _p(tile_off), _p(pages),
                                          _p(table), table.shape[1], ring_pages, _p(row_pos), _p(cu_seqlens),
                                          _p(n_cached), B, int(n_tiles), nq, nkv, d, int(window or 0),
                                          ctypes.c_float(scale), _p(out), None, None, 0, None, 0,
                                          ctypes.c_longlong(0), n, _stream()))
        return
    if cuts.n_seqs != B or cuts.n_tiles != int(n_tiles):
        raise KernelError(f"attn.cuts: laid out for {cuts.n_seqs} sequences and {cuts.n_tiles} blocks, "
                          f"the step has {B} and {int(n_tiles)}")
    if part is None:
        raise KernelError("attn.part: blocks cut in halves need room for their sums")
    _req(part, "attn.part", torch.float32)
    _req(cuts.items, "attn.cuts.items", torch.int32, (cuts.n_items, 4))
    _req(cuts.blocks, "attn.cuts.blocks", torch.int32, (cuts.n_cut, 4))
    _check(lib().tl_attn_prefill_bf16(_p(q), _p(k_new), _p(vt_new), vt_new.shape[2], _p(tile_off), _p(pages),
                                      _p(table), table.shape[1], ring_pages, _p(row_pos), _p(cu_seqlens),
                                      _p(n_cached), B, cuts.n_items, nq, nkv, d, int(window or 0),
                                      ctypes.c_float(scale), _p(out), _p(cuts.items), _p(cuts.blocks), cuts.n_cut,
                                      _p(part), cuts.ways, ctypes.c_longlong(part.numel()), n, _stream()))


def attn_decode_bf16(q, pages, table, ring_pages: int, row_pos, window: Optional[int], scale: float,
                     n_splits: int, part, out) -> None:
    """bfloat16 attention of one new token per sequence over its pages (the
    token's own key is already committed).  `part`: float32 scratch of at
    least B * nq * n_splits * (d + 2) elements."""
    B, nq, d = q.shape
    nkv = pages.shape[2]
    _req(q, "attn.q", torch.bfloat16)
    _req(pages, "attn.pages", torch.bfloat16)
    if pages.dim() != 5 or tuple(pages.shape[1:]) != (2, nkv, PAGE, d):
        raise KernelError(f"attn.pages: shape {tuple(pages.shape)}, kernel needs [*, 2, nkv, {PAGE}, {d}]")
    _req(table, "attn.table", torch.int32)
    _req(row_pos, "attn.row_pos", torch.int32, (B,))
    _req(part, "attn.part", torch.float32)
    _req(out, "attn.out", torch.bfloat16, (B, nq, d))
    if table.dim() != 2 or table.shape[0] != B:
        raise KernelError("attn.table: needs one row per sequence")
    if part.numel() < B * nq * n_splits * (d + 2):
        raise KernelError(f"attn.part: {part.numel()} elements, kernel needs {B * nq * n_splits * (d + 2)}")
    _check(lib().tl_attn_decode_bf16(_p(q), _p(pages), _p(table), table.shape[1], ring_pages, _p(row_pos),
                                     B, nq, nkv, d, int(window or 0), ctypes.c_float(scale),
                                     int(n_splits), _p(part), _p(out), _stream()))


def decode_through_lds(on: bool) -> bool:
    """For tests and measurements: whether single-token attention with heads of 64, 128 or 256 goes
    through the kernel that stages the pages in LDS (the default) or, like every other head size,
    through the one that reads them into registers.  Returns the setting before the call."""
    return bool(lib().tl_attn_decode_through_lds(int(bool(on))))


def decode_groups(B: int, nq: int, nkv: int) -> int:
    """Workgroups of a decode step's attention before splitting: one per
    (sequence, KV head, 16 query heads of its group)."""
    return B * nkv * (-(-(nq // nkv) // 16))


SPLIT_PAGES = 4             # fewest pages a part of the keys has
SPLIT_COST = 0.15           # what a part more costs in the merge, in pages of a workgroup's way (8 sequences of
                            # 8 KV heads over 4,096 keys: 4 parts 3.91 ms a step, 8 parts 3.96, 6 parts 4.08)
FULL_UNIT_HEAD = 128        # the kernel that reads the pages into registers: the head size from which one workgroup
                            # has enough bytes under way to keep a compute unit streaming; smaller heads get
                            # FULL_UNIT_HEAD // head_dim workgroups a unit (heads of 48 ...)
LDS_DECODE_PER_UNIT = {64: 2, 128: 2, 256: 1}    # the kernel that stages the pages in LDS (these head sizes): its
                            # workgroups hold 64 KB of LDS each (128 KB with heads of 256), so two share a unit, and
                            # a round of workgroups is twice the units (64 sequences of 8 KV heads of 128 over 4,096
                            # keys, 512 workgroups: 162 us with two a unit, 169 with one holding 128 KB)


def decode_workgroups_per_unit(head_dim: int) -> int:
    """How many workgroups of a decode step's attention a compute unit holds at a time."""
    return LDS_DECODE_PER_UNIT.get(int(head_dim), max(1, FULL_UNIT_HEAD // max(1, int(head_dim))))


@functools.lru_cache(maxsize=4096)
def _decode_splits(groups: int, max_pages: int, units: int) -> int:
    most = max(1, min(-(-max_pages // SPLIT_PAGES), -(-4 * units // groups), 4096))
    # rounds of workgroups over the compute units x pages a workgroup goes through, and the merge
    cost = lambda s: -(-groups * s // units) * -(-max_pages // s) + SPLIT_COST * s
    return min(range(1, most + 1), key=lambda s: (cost(s), s))


def decode_splits(B: int, nq: int, nkv: int, max_pages: int, units: int, head_dim: int) -> int:
    """Into how many parts the keys of a decode step are cut.  A compute unit streams at a rate of
    its own, so the step's attention takes as long as the unit with the most to read: rounds of
    workgroups over the `units` compute units times the pages a workgroup has, plus the merge's
    share for every part; parts have at least four pages.  A round is as many workgroups as the
    units hold at a time (`decode_workgroups_per_unit`): eight sequences with eight KV heads of 128
    are 8 parts, 512 workgroups, two a unit (28.2 us a layer over 4,096 keys against 30.3 in 4 parts).
    With heads of less than 64 the kernel that reads into registers has too few bytes under way to
    keep a unit busy with one workgroup, and a round is 128 // head size a unit (32 sequences of 4 KV
    heads of 32 take 19.2 us in 4 parts, 27.2 in 2)."""
    return _decode_splits(decode_groups(B, nq, nkv), int(max_pages), int(units) * decode_workgroups_per_unit(head_dim))


def uses_transposed_values(dtype: torch.dtype, d: int, all_single: bool) -> bool:
    """Does `attention` take this step's values transposed (`vt_new`)?"""
    return dtype == torch.bfloat16 and d % 16 == 0 and 16 <= d <= 256 and not all_single


def attention(q, k_new, v_new, pages, table, ring_pages: int, ctx, n_cached, window, scale: float,
              out, vt_new=None) -> None:
    """Attention of a step's rows: keys j < n_cached[b] from the pages, later
    ones from this step's rows (`k_new`/`v_new`; None when everything is in
    the pages).  bfloat16 with head sizes in steps of 16 runs on the matrix
    cores, single-token steps and steps with longer rows each in their own
    kernel (the latter takes the values transposed, `vt_new`, see
    `rope_split`); everything else runs in the plain kernel."""
    n, nq, d = q.shape
    fast = q.dtype == torch.bfloat16 and d % 16 == 0 and 16 <= d <= 256
    if fast and k_new is None and ctx.all_single:
        nkv = pages.shape[2]
        splits = decode_splits(n, nq, nkv, table.shape[1], compute_units(q.device), d)   # by the table's width: fixed while a graph lives
        part = ctx.workspace.get("attn_part", (n * nq * splits * (d + 2),), torch.float32)
        attn_decode_bf16(q, pages, table, ring_pages, ctx.row_pos, window, scale, splits, part, out)
    elif fast and k_new is not None and vt_new is not None:
        n_tiles = int(sum(-(-int(x) // PREFILL_BLOCK) for x in ctx.host["n_new"]))
        cuts = part = None
        if not ctx.host.get("fixed_launches"):   # (a captured graph's launches must not be shaped by lengths)
            at = ("prefill_cuts", window, nq)
            if at not in ctx.host:                               # the same for every layer of the step
                ctx.host[at] = prefill_cuts(ctx.host["n_new"], ctx.host["len_before"], window, nq,
                                            compute_units(q.device), q.device)
            cuts = ctx.host[at]
            if cuts is not None:
                part = ctx.workspace.get("attn_prefill_part", (n * nq * cuts.ways * (d + 4),), torch.float32)
        attn_prefill_bf16(q, k_new, vt_new, ctx.tile_off, pages, table, ring_pages, ctx.row_pos,
                          ctx.cu_seqlens, n_cached, n_tiles, window, scale, out, cuts=cuts, part=part)
    else:
        attn_plain(q, k_new, v_new, pages, table, ring_pages, ctx.row_seq, ctx.row_pos, ctx.cu_seqlens,
                   n_cached, window, scale, out)


READ_SHAPES = {0: "8 loads a lane, a grid stride apart", 1: "16 loads a lane", 2: "32 loads a lane",
               3: "8 loads a lane, a contiguous share a workgroup", 4: "16 loads a lane, contiguous",
               5: "8 loads a lane, non-temporal", 6: "16 loads a lane, non-temporal, contiguous",
               7: "8 loads a wave straight into LDS", 8: "16 loads a wave straight into LDS"}


def _measure_lib() -> ctypes.CDLL:
    """The library of the kernels that only measure the machine (built apart from the model's)."""
    L = load_measure()
    L.tl_measure_last_error.restype = ctypes.c_char_p
    return L


def _check_measure(rc: int) -> None:
    if rc != 0:
        raise KernelError(_measure_lib().tl_measure_last_error().decode())


def measure_ceilings(device="cuda:0", gib: float = 8.0, shapes=None) -> dict:
    """What the simplest kernels get on this machine: GB/s of one read of a buffer far larger
    than the caches, in every shape of `READ_SHAPES` (the best is reported with its shape, the
    others beside it), GB/s of a copy (bytes read plus bytes written), and TFLOP/s of independent
    bfloat16 MFMAs on registers (the best of a few runs and launch shapes each)."""
    import time
    units = compute_units(device)
    quantum = units * 32 * 256 * 32 * 16          # whole iterations of every shape at every number of workgroups (1 GiB)
    n_bytes = max(1, round(gib * 2 ** 30 / quantum)) * quantum
    buf = torch.empty(n_bytes // 4, dtype=torch.float32, device=device).normal_()
    sink = torch.zeros(units * 32, dtype=torch.float32, device=device)

    def timed(launch):
        torch.cuda.synchronize()
        t = time.perf_counter()
        _check_measure(launch())
        torch.cuda.synchronize()
        return time.perf_counter() - t

    by_shape = {}
    for shape in (READ_SHAPES if shapes is None else shapes):
        best = 0.0
        for blocks in (units, units * 2, units * 4, units * 8, units * 16, units * 32):
            for _ in range(3):
                dt = timed(lambda: _measure_lib().tl_stream_read_shape(_p(buf), ctypes.c_size_t(n_bytes), _p(sink), blocks,
                                                              shape, _stream()))
                best = max(best, n_bytes / dt / 1e9)
        by_shape[shape] = round(best, 1)
    top = max(by_shape, key=by_shape.get)
    half = n_bytes // 2
    dst = buf.view(-1)[half // 4:]
    best_copy = 0.0
    for blocks in (units, units * 2, units * 4, units * 8):
        for _ in range(3):
            dt = timed(lambda: _measure_lib().tl_stream_copy(_p(buf), _p(dst), ctypes.c_size_t(half), blocks, _stream()))
            best_copy = max(best_copy, 2 * half / dt / 1e9)
    del buf, dst
    best_mfma = 0.0
    for blocks in (units, units * 2, units * 4):
        iters = 8192
        for _ in range(3):
            dt = timed(lambda: _measure_lib().tl_mfma_chain(iters, blocks, _p(sink), _stream()))
            flop = blocks * 4 * iters * 8 * 2 * 32 * 32 * 16
            best_mfma = max(best_mfma, flop / dt / 1e12)
    return {"hbm_read_GBs": by_shape[top], "hbm_read_shape": READ_SHAPES[top],
            "hbm_read_by_shape_GBs": {READ_SHAPES[k]: v for k, v in by_shape.items()},
            "hbm_copy_GBs": round(best_copy, 1), "mfma_bf16_TFLOPs": round(best_mfma, 1)}


def measure_pipes(device="cuda:0", iters: int = 20000) -> dict:
    """Whether a SIMD's matrix pipe and vector pipe work at the same time (`pipes_kernel` in
    csrc/measure/ceilings.hip): nanoseconds an iteration of one workgroup a compute unit, for the same work a
    SIMD laid out in five ways.  `mfma_only`, `vector_only`: one wave a SIMD with one kind of work
    (4 MFMAs 32x32x16, or 32 FMAs and 8 exponentials, an iteration); `both_in_one_wave`: one wave a SIMD
    does both; `both_in_two_waves`: two waves a SIMD, each both, half the iterations (what the prefill
    attention does); `split_roles`: two waves a SIMD, one with the MFMAs and one with the vector work."""
    import time
    units = compute_units(device)
    sink = torch.zeros(16, dtype=torch.float32, device=device)

    def run(role, waves, n):
        best = float("inf")
        for _ in range(3):
            torch.cuda.synchronize()
            t = time.perf_counter()
            _check_measure(_measure_lib().tl_pipes(role, waves, n, units, _p(sink), _stream()))
            torch.cuda.synchronize()
            best = min(best, time.perf_counter() - t)
        return round(best / iters * 1e9, 2)

    return {"mfma_only": run(0, 4, iters), "vector_only": run(1, 4, iters), "both_in_one_wave": run(2, 4, iters),
            "both_in_two_waves": run(2, 8, iters // 2), "split_roles": run(3, 8, iters)}
