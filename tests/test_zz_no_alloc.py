"""The entry point that allocates nothing (`tl_attn_decode_bf16_static`, csrc/no_alloc.h), called
through ctypes: its output against that of `tl_attn_decode_bf16`, which takes the scratch from the
caller, on two calls in a row, the second with a smaller input, and against the plain attention."""
import ctypes
import math

import pytest
import torch

import plain_mistral as plain
from util import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PAGE = 64


def _case(B, nq, nkv, d, window, lens, seed):
    """Sequences whose last position is the new token, everything committed to scattered pages."""
    g = torch.Generator().manual_seed(seed)
    n_pages = sum(-(-n // PAGE) for n in lens) + 3
    ring = -(-window // PAGE) if window else n_pages
    width = min(ring, max(-(-n // PAGE) for n in lens))
    pages = torch.full((n_pages, 2, nkv, PAGE, d), float("nan"), dtype=torch.bfloat16)
    perm = torch.randperm(n_pages, generator=g).tolist()
    table = torch.zeros(B, width, dtype=torch.int32)
    qs, want = [], []
    for b, T in enumerate(lens):
        q = torch.randn(T, nq, d, generator=g).to(torch.bfloat16)
        k = torch.randn(T, nkv, d, generator=g).to(torch.bfloat16)
        v = torch.randn(T, nkv, d, generator=g).to(torch.bfloat16)
        mine = [perm.pop() for _ in range(min(-(-T // PAGE), ring))]
        table[b, :len(mine)] = torch.tensor(mine, dtype=torch.int32)
        for p in range(max(0, T - ring * PAGE), T):
            pg = mine[(p // PAGE) % ring]
            pages[pg, 0, :, p % PAGE] = k[p]
            pages[pg, 1].view(nkv, d, PAGE)[:, :, p % PAGE] = v[p]
        want.append(plain.attention_core(q.double(), k.double(), v.double(), torch.arange(T), window)[-1:])
        qs.append(q[-1:])
    return dict(q=torch.cat(qs).contiguous().to(DEV), pages=pages.to(DEV), table=table.to(DEV), ring=ring,
                row_pos=torch.tensor([T - 1 for T in lens], dtype=torch.int32, device=DEV),
                want=torch.cat(want), B=B, nq=nq, nkv=nkv, d=d, window=window or 0,
                scale=1.0 / math.sqrt(d))


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(lib, c, splits):
    """The same step through the entry point that is given its scratch and the one that has its own."""
    B, nq, d = c["B"], c["nq"], c["d"]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    head = (_ptr(c["q"]), _ptr(c["pages"]), _ptr(c["table"]), c["table"].shape[1], c["ring"], _ptr(c["row_pos"]),
            B, nq, c["nkv"], d, c["window"], ctypes.c_float(c["scale"]), splits)
    part = torch.full((B * nq * splits * (d + 2),), float("nan"), device=DEV)
    given = torch.zeros(B, nq, d, dtype=torch.bfloat16, device=DEV)
    own = torch.zeros(B, nq, d, dtype=torch.bfloat16, device=DEV)
    rc = lib.tl_attn_decode_bf16(*head, _ptr(part), _ptr(given), stream)
    assert rc == 0, lib.tl_last_error().decode()
    rc = lib.tl_attn_decode_bf16_static(*head, _ptr(own), stream)
    assert rc == 0, lib.tl_last_error().decode()
    torch.cuda.synchronize()
    return given, own


def test_static_scratch_entry_point_two_calls_in_a_row():
    from torchless_rs_amd.kernels import ops
    lib = ops.lib()
    lib.tl_static_scratch_bytes.restype = ctypes.c_size_t
    assert lib.tl_static_scratch_bytes() == 8 << 20
    big = _case(6, 8, 2, 128, None, [700, 1, 64, 65, 300, 513], seed=11)
    small = _case(2, 6, 1, 48, 100, [40, 333], seed=12)          # fewer rows, heads, splits; a ring
    for case, splits in ((big, 5), (small, 2), (big, 1)):
        given, own = _both(lib, case, splits)
        assert torch.equal(given, own), "the two entry points run the same kernels"
        assert torch.isfinite(own).all()
        assert rel_err(own, case["want"]) < 6e-3


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    from torchless_rs_amd.kernels import ops
    lib = ops.lib()
    c = _case(1, 4, 1, 64, None, [10], seed=13)
    out = torch.zeros(1, 4, 64, dtype=torch.bfloat16, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # claimed sizes whose partial results would take more than the array holds: refused before any launch
    rc = lib.tl_attn_decode_bf16_static(_ptr(c["q"]), _ptr(c["pages"]), _ptr(c["table"]), 1, c["ring"],
                                        _ptr(c["row_pos"]), 4096, 64, 8, 256, 0, ctypes.c_float(1.0), 64,
                                        _ptr(out), stream)
    assert rc != 0
    assert "static scratch holds" in lib.tl_last_error().decode()
    torch.cuda.synchronize()
    assert (out == 0).all()


def test_static_scratch_entry_point_under_graph_capture():
    """After the set-up call (made outside capture) a call may be captured into a HIP graph: every
    replay, with the program's own eager work and synchronizations between them and with other inputs
    written into the same tensors, gives the bits of the eager call."""
    from torchless_rs_amd.kernels import ops
    lib = ops.lib()
    assert lib.tl_static_scratch_ready() == 0, lib.tl_last_error().decode()
    c = _case(5, 8, 2, 128, None, [130, 700, 64, 65, 1], seed=21)
    other = _case(5, 8, 2, 128, None, [130, 700, 64, 65, 1], seed=22)      # same shapes, other values
    B, nq, d, splits = c["B"], c["nq"], c["d"], 3
    q, pages, table = c["q"].clone(), c["pages"].clone(), c["table"].clone()
    out = torch.zeros(B, nq, d, dtype=torch.bfloat16, device=DEV)

    def call(stream):
        rc = lib.tl_attn_decode_bf16_static(_ptr(q), _ptr(pages), _ptr(table), table.shape[1], c["ring"],
                                            _ptr(c["row_pos"]), B, nq, c["nkv"], d, c["window"],
                                            ctypes.c_float(c["scale"]), splits, _ptr(out),
                                            ctypes.c_void_p(stream.cuda_stream))
        assert rc == 0, lib.tl_last_error().decode()

    eager = {}
    for name, src in (("a", c), ("b", other)):
        q.copy_(src["q"]); pages.copy_(src["pages"]); table.copy_(src["table"])
        call(torch.cuda.current_stream())
        torch.cuda.synchronize()
        eager[name] = out.clone()
    assert not torch.equal(eager["a"], eager["b"])
    graph = torch.cuda.CUDAGraph()
    q.copy_(c["q"]); pages.copy_(c["pages"]); table.copy_(c["table"])
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        call(torch.cuda.current_stream())
    for name in ("a", "b", "b", "a", "a"):
        src = c if name == "a" else other
        q.copy_(src["q"]); pages.copy_(src["pages"]); table.copy_(src["table"])
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager[name]), name
        # the array is shared: an eager call between the replays, with its own output, disturbs nothing
        _both(lib, _case(2, 6, 1, 48, 100, [40, 333], seed=12), 2)
