"""Each kernel alone against a plain float64 computation, at sizes other than
the engine's tests use."""
import math

import numpy as np
import pytest
import torch

import plain_mistral as plain
from util import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# one output rounding of bfloat16 is 2^-9 relative; float32 results differ by summation order only
KTOL = {"float32": 3e-6, "bfloat16": 6e-3}


@pytest.fixture(scope="module")
def ops():
    from torchless_rs_amd.kernels import ops as o
    o.lib()
    return o


def rnd(*shape, seed=0, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_embed(ops, dt):
    table = rnd(77, 130, dtype=DT[dt]).to(DEV)
    ids = torch.tensor([0, 76, 5, 5, 31], dtype=torch.int32, device=DEV)
    out = torch.empty(5, 130, device=DEV)
    ops.embed(table, ids, out)
    assert torch.equal(out.cpu(), table.cpu().float()[ids.cpu().long()])


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,H", [(1, 100), (5, 4097), (3, 64)])
def test_rmsnorm(ops, dt, n, H):
    x = rnd(n, H, seed=1, scale=3.0)
    w = 1 + 0.2 * rnd(H, seed=2)
    out = torch.empty(n, H, dtype=DT[dt], device=DEV)
    ops.rmsnorm(x.to(DEV), w.to(DEV), 1e-3, out)
    assert rel_err(out, plain.rmsnorm(x.double(), w.double(), 1e-3)) < KTOL[dt]
    tiny = x * 1e-3                                      # eps matters here
    ops.rmsnorm(tiny.to(DEV), w.to(DEV), 1e-3, out)
    assert rel_err(out, plain.rmsnorm(tiny.double(), w.double(), 1e-3)) < KTOL[dt]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("nq,nkv,d,theta", [(3, 1, 48, 500.0), (8, 2, 128, 1e6), (2, 2, 16, 1e4)])
def test_rope_split(ops, dt, nq, nkv, d, theta):
    from torchless_rs_amd.parts.position import Rotary
    n = 6
    qkv = rnd(n, (nq + 2 * nkv) * d, seed=3)
    pos = torch.tensor([0, 1, 7, 100, 5000, 40000], dtype=torch.int32)
    q = torch.empty(n, nq, d, dtype=DT[dt], device=DEV)
    k = torch.empty(n, nkv, d, dtype=DT[dt], device=DEV)
    v = torch.empty(n, nkv, d, dtype=DT[dt], device=DEV)
    ops.rope_split(qkv.to(DEV), pos.to(DEV), Rotary(d, theta).inv_freq(DEV), nq, nkv, d, q, k, v)
    x = qkv.double()
    wq = plain.rope(x[:, :nq * d].view(n, nq, d), pos, theta)
    wk = plain.rope(x[:, nq * d:(nq + nkv) * d].view(n, nkv, d), pos, theta)
    wv = x[:, (nq + nkv) * d:].view(n, nkv, d)
    # angles are float32 as the reference's are: pos * inv_freq carries a relative rounding of
    # 2^-24 from each factor, so a row at position p may be off by 1.2e-7 * p radians
    for r, p in enumerate(pos.tolist()):
        tol = KTOL[dt] + 1.2e-7 * p
        assert rel_err(q[r], wq[r]) < tol and rel_err(k[r], wk[r]) < tol, (r, p)
    assert rel_err(v, wv) < KTOL[dt]
    assert torch.equal(q[0].float().cpu(), qkv[0, :nq * d].view(nq, d).to(DT[dt]).float())   # pos 0: identity
    # the values also transposed: two sequences of 2 and 4 rows, the second going on from 70 cached
    pos2 = torch.tensor([0, 1, 70, 71, 72, 73], dtype=torch.int32, device=DEV)
    seq2 = torch.tensor([0, 0, 1, 1, 1, 1], dtype=torch.int32, device=DEV)
    off, cols = ops.aligned_columns([0, 70], [2, 4])
    assert (off, cols) == ([0, 64], 128)
    vt = torch.full((nkv, d, cols), 7.0, dtype=DT[dt], device=DEV)
    ops.rope_split(qkv.to(DEV), pos2, Rotary(d, theta).inv_freq(DEV), nq, nkv, d, q, k, v, vt, seq2,
                   torch.tensor(off, dtype=torch.int32, device=DEV), torch.tensor([0, 70], dtype=torch.int32, device=DEV))
    for r, col in enumerate([0, 1, 64 + 6, 64 + 7, 64 + 8, 64 + 9]):
        assert torch.equal(vt[:, :, col], v[r])
    assert int((vt == 7.0).sum()) == nkv * d * (cols - 6)


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [None, 128])
@pytest.mark.parametrize("nq,nkv,d", [(4, 2, 16), (6, 3, 80), (2, 1, 256)])
def test_values_by_tiles_and_their_commit(ops, dt, window, nq, nkv, d):
    """`v_tiles` writes what `rope_split` writes into vt, and `kv_commit_tiles` commits what
    `kv_commit` commits, for sequences that start inside a page, span pages and wrap a ring."""
    from torchless_rs_amd.cache import PAGE
    from torchless_rs_amd.parts.position import Rotary
    cached, new = [0, 70, 64, 130, 5], [2, 4, 64, 200, 59]
    B, n = len(cached), sum(new)
    i32 = lambda l: torch.tensor(l, dtype=torch.int32, device=DEV)
    qkv = rnd(n, (nq + 2 * nkv) * d, seed=61).to(DEV)
    row_seq = i32([b for b in range(B) for _ in range(new[b])])
    row_pos = i32([cached[b] + i for b in range(B) for i in range(new[b])])
    cu = i32([sum(new[:b]) for b in range(B + 1)])
    after = [c + m for c, m in zip(cached, new)]
    off, cols = ops.aligned_columns(cached, new)
    inv = Rotary(d, 10000.0).inv_freq(DEV)
    q, k, v = (torch.empty(n, h, d, dtype=DT[dt], device=DEV) for h in (nq, nkv, nkv))
    vt_old = torch.full((nkv, d, cols), 7.0, dtype=DT[dt], device=DEV)
    ops.rope_split(qkv, row_pos, inv, nq, nkv, d, q, k, v, vt_old, row_seq, i32(off), i32(cached))
    k2 = torch.empty_like(k)
    q2 = torch.empty_like(q)
    ops.rope_split(qkv, row_pos, inv, nq, nkv, d, q2, k2, None)                 # without the values
    assert torch.equal(q, q2) and torch.equal(k, k2)
    vt_new = torch.full((nkv, d, cols), 7.0, dtype=DT[dt], device=DEV)
    ops.v_tiles(qkv, nq, nkv, d, vt_new, cu, i32(off), i32(cached), i32(after))
    assert torch.equal(vt_old, vt_new)
    assert int((vt_new != 7.0).sum()) >= nkv * d * n - 8                       # (a value may be 7.0 by chance)
    # rotation and transposition in one launch: the same bits
    q3, k3, vt3 = torch.full_like(q, float("nan")), torch.full_like(k, float("nan")), torch.full_like(vt_new, 7.0)
    ops.rope_v_tiles(qkv, row_pos, inv, nq, nkv, d, q3, k3, vt3, cu, i32(off), i32(cached), i32(after))
    assert torch.equal(q3, q2) and torch.equal(k3, k2) and torch.equal(vt3, vt_new)
    # commit: pages of every sequence, rings for the window
    ring = -(-window // PAGE) if window else 1 << 24
    need = [min(-(-a // PAGE), ring) for a in after]
    n_pages = sum(need) + 3
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(5)).tolist()
    table = torch.zeros(B, max(need), dtype=torch.int32)
    for b in range(B):
        table[b, :need[b]] = torch.tensor([perm.pop() for _ in range(need[b])], dtype=torch.int32)
    pages_old = torch.full((n_pages, 2, nkv, PAGE, d), 3.0, dtype=DT[dt], device=DEV)
    pages_new = pages_old.clone()
    ops.kv_commit(k, v, row_seq, row_pos, i32(after), table.to(DEV), ring, pages_old)
    ops.kv_commit_tiles(k, vt_new, row_seq, row_pos, i32(off), i32(cached), i32(after), table.to(DEV), ring, pages_new)
    assert torch.equal(pages_old, pages_new)
    assert not torch.equal(pages_new, torch.full_like(pages_new, 3.0))
    if window:                                    # 330 positions in a ring of 2 pages: the first 202 of the step are skipped
        assert after[3] - ring * PAGE > 131
    with pytest.raises(ops.KernelError, match="multiple of 64"):
        ops.v_tiles(qkv, nq, nkv, d, torch.zeros(nkv, d, 100, dtype=DT[dt], device=DEV), cu, i32(off), i32(cached),
                    i32(after))


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_silu_mul_and_gather(ops, dt):
    n, I = 5, 301
    gu = rnd(n, 2 * I, seed=4, scale=4.0)
    out = torch.empty(n, I, dtype=DT[dt], device=DEV)
    ops.silu_mul(gu.to(DEV), out)
    g, u = gu.double()[:, :I], gu.double()[:, I:]
    assert rel_err(out, plain.silu(g) * u) < KTOL[dt]
    x = rnd(9, 70, seed=5).to(DEV)
    idx = torch.tensor([8, 0, 3, 3], dtype=torch.int32, device=DEV)
    o = torch.empty(4, 70, device=DEV)
    ops.gather_rows(x, idx, o)
    assert torch.equal(o, x[idx.long()])


@pytest.mark.parametrize("adt,wdt", [("float32", "float32"), ("bfloat16", "bfloat16"),
                                     ("bfloat16", "float32"), ("float32", "bfloat16")])
@pytest.mark.parametrize("M,N,K", [(1, 50, 17), (5, 130, 100), (70, 64, 64), (129, 200, 333)])
def test_gemm_plain(ops, adt, wdt, M, N, K):
    a = rnd(M, K, seed=6, dtype=DT[adt])
    w = rnd(N, K, seed=7, dtype=DT[wdt])
    want = a.double() @ w.double().t()
    out = torch.empty(M, N, device=DEV)
    ops.gemm_plain(a.to(DEV), w.to(DEV), out)
    assert rel_err(out, want) < 3e-6
    base = rnd(M, N, seed=8)
    acc = base.clone().to(DEV)
    ops.gemm_plain(a.to(DEV), w.to(DEV), acc, accumulate=True)
    assert rel_err(acc, want + base.double()) < 3e-6
    # [[1,2],[3,4]] . [1,2] = [5,11]  (src/kernels/tests.rs:5-10 of the reference)
    o2 = torch.empty(1, 2, device=DEV)
    ops.gemm_plain(torch.tensor([[1., 2.]], device=DEV), torch.tensor([[1., 2.], [3., 4.]], device=DEV), o2)
    assert o2.tolist() == [[5., 11.]]


def test_gemm_row_does_not_depend_on_the_batch(ops):
    a = rnd(37, 96, seed=9).to(DEV)
    w = rnd(80, 96, seed=10).to(DEV)
    full = torch.empty(37, 80, device=DEV)
    ops.gemm_plain(a, w, full)
    one = torch.empty(1, 80, device=DEV)
    ops.gemm_plain(a[20:21].contiguous(), w, one)
    assert torch.equal(one[0], full[20])


# ---- attention over pages ----------------------------------------------------

def paged_case(ops, dt, nq, nkv, d, window, lens_cached, lens_new, seed=0, n_pages=40):
    """Random sequences with `lens_cached` positions in pages (scattered, rings
    for windows) and `lens_new` new rows; returns the kernel's output and the
    plain result for the new rows."""
    from torchless_rs_amd.cache import PAGE
    tdt = DT[dt]
    B = len(lens_cached)
    ring = -(-window // PAGE) if window else n_pages
    g = torch.Generator().manual_seed(seed)
    pages = torch.full((n_pages, 2, nkv, PAGE, d), float("nan"), dtype=tdt)     # stale rows are poison
    perm = torch.randperm(n_pages, generator=g).tolist()
    table = torch.zeros(B, ring if window else max(1, max(-(-(c + n) // PAGE) for c, n in zip(lens_cached, lens_new))),
                        dtype=torch.int32)
    seqs, q_rows, k_rows, v_rows, want = [], [], [], [], []
    row_seq, row_pos, cu = [], [], [0]
    for b in range(B):
        T = lens_cached[b] + lens_new[b]
        q = torch.randn(T, nq, d, generator=g).to(tdt)
        k = torch.randn(T, nkv, d, generator=g).to(tdt)
        v = torch.randn(T, nkv, d, generator=g).to(tdt)
        need = min(-(-T // PAGE), ring)
        mine = [perm.pop() for _ in range(need)]
        table[b, :need] = torch.tensor(mine, dtype=torch.int32)
        for p in range(max(0, lens_cached[b] - ring * PAGE), lens_cached[b]):
            pg = mine[(p // PAGE) % ring]
            pages[pg, 0, :, p % PAGE] = k[p]
            pages[pg, 1].view(nkv, d, PAGE)[:, :, p % PAGE] = v[p]      # values lie transposed
        full = plain.attention_core(q.double(), k.double(), v.double(), torch.arange(T), window)
        want.append(full[lens_cached[b]:])
        q_rows.append(q[lens_cached[b]:]); k_rows.append(k[lens_cached[b]:]); v_rows.append(v[lens_cached[b]:])
        row_seq += [b] * lens_new[b]
        row_pos += list(range(lens_cached[b], T))
        cu.append(cu[-1] + lens_new[b])
    dev = lambda t: t.contiguous().to(DEV)
    i32 = lambda l: torch.tensor(l, dtype=torch.int32, device=DEV)
    qn, kn, vn = dev(torch.cat(q_rows)), dev(torch.cat(k_rows)), dev(torch.cat(v_rows))
    out = torch.empty_like(qn)
    args = dict(pages=dev(pages), table=dev(table), ring=ring, row_seq=i32(row_seq), row_pos=i32(row_pos),
                cu=i32(cu), cached=i32(lens_cached), after=i32([c + n for c, n in zip(lens_cached, lens_new)]),
                q=qn, k=kn, v=vn, out=out, window=window, scale=1.0 / math.sqrt(d), want=torch.cat(want))
    return args


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("nq,nkv,d,window", [(4, 2, 16, None), (6, 1, 32, 70), (5, 5, 48, 8),
                                             (8, 2, 128, 100), (2, 1, 256, None), (3, 3, 80, 64)])
def test_attention_cached_and_new(ops, dt, nq, nkv, d, window):
    a = paged_case(ops, dt, nq, nkv, d, window, lens_cached=[0, 5, 130, 64, 200], lens_new=[17, 1, 3, 70, 1])
    ops.attn_plain(a["q"], a["k"], a["v"], a["pages"], a["table"], a["ring"], a["row_seq"], a["row_pos"],
                   a["cu"], a["cached"], window, a["scale"], a["out"])
    assert rel_err(a["out"], a["want"]) < KTOL[dt]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [None, 70, 128])
def test_commit_then_decode_reads_the_pages_only(ops, dt, window):
    """One new token per sequence: commit first, then everything comes from
    the pages, also where the ring has wrapped."""
    nq, nkv, d = 4, 2, 32
    a = paged_case(ops, dt, nq, nkv, d, window, lens_cached=[0, 63, 64, 300, 191], lens_new=[1] * 5, seed=3)
    ops.kv_commit(a["k"], a["v"], a["row_seq"], a["row_pos"], a["after"], a["table"], a["ring"], a["pages"])
    ops.attn_plain(a["q"], None, None, a["pages"], a["table"], a["ring"], a["row_seq"], a["row_pos"],
                   a["cu"], a["after"], window, a["scale"], a["out"])
    assert rel_err(a["out"], a["want"]) < KTOL[dt]


def test_commit_of_a_chunk_longer_than_the_ring(ops):
    """A step of 300 rows into a ring of 2 pages keeps the last 128 positions."""
    from torchless_rs_amd.cache import PAGE
    nkv, d, window = 1, 16, 70
    a = paged_case(ops, "float32", 2, nkv, d, window, lens_cached=[10], lens_new=[300], seed=4)
    ops.kv_commit(a["k"], a["v"], a["row_seq"], a["row_pos"], a["after"], a["table"], a["ring"], a["pages"])
    pages, table = a["pages"].cpu(), a["table"].cpu()
    for p in range(310 - 128, 310):
        pg = int(table[0, (p // PAGE) % 2])
        assert torch.equal(pages[pg, 0, 0, p % PAGE], a["k"][p - 10, 0].cpu())
        assert torch.equal(pages[pg, 1].view(nkv, d, PAGE)[0, :, p % PAGE], a["v"][p - 10, 0].cpu())


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds_and_the_windows_edge(ops, dt):
    """One key is made to match the query far better than the rest: the output
    must be its value row iff the key is visible."""
    from torchless_rs_amd.cache import PAGE
    nq, nkv, d, T = 2, 1, 32, 700
    tdt = DT[dt]
    g = torch.Generator().manual_seed(5)
    for window, far, visible in [(None, 3, True), (200, 499, False), (200, 500, True), (200, 699, True)]:
        k = torch.randn(T, nkv, d, generator=g) * 0.1
        v = torch.randn(T, nkv, d, generator=g)
        qv = torch.randn(d, generator=g)
        qv = qv / qv.norm()
        k[far, 0] = qv * 60.0                           # score 60 * |q| / sqrt(d) above all others
        q = (qv * 8.0).view(1, 1, d).repeat(1, nq, 1)
        ring = -(-window // PAGE) if window else 11
        pages = torch.full((11, 2, nkv, PAGE, d), float("nan"), dtype=tdt)
        table = torch.tensor([[7, 2, 9, 0, 5, 1, 10, 3, 8, 4, 6][:ring]], dtype=torch.int32)
        for p in range(max(0, T - ring * PAGE), T):
            pg = int(table[0, (p // PAGE) % ring])
            pages[pg, 0, :, p % PAGE] = k[p].to(tdt)
            pages[pg, 1].view(nkv, d, PAGE)[:, :, p % PAGE] = v[p].to(tdt)
        out = torch.empty(1, nq, d, dtype=tdt, device=DEV)
        i32 = lambda l: torch.tensor(l, dtype=torch.int32, device=DEV)
        ops.attn_plain(q.to(tdt).to(DEV), None, None, pages.to(DEV), table.to(DEV), ring, i32([0]),
                       i32([T - 1]), i32([0, 1]), i32([T]), window, 1.0 / math.sqrt(d), out)
        hit = rel_err(out[0, 0], v[far, 0].to(tdt)) < 1e-2
        assert hit == visible, (window, far)
        assert torch.isfinite(out).all()


# ---- sampling ------------------------------------------------------------------

def philox_uniform(seed: int, step: int, seq: int) -> float:
    """Philox4x32-10, key = seed, counter = (step, seq, 0, 0); first word >> 8 / 2^24."""
    M0, M1, W0, W1, mask = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85, 0xFFFFFFFF
    c = [step & mask, seq & mask, 0, 0]
    k = [seed & mask, (seed >> 32) & mask]
    for r in range(10):
        if r:
            k = [(k[0] + W0) & mask, (k[1] + W1) & mask]
        p0, p1 = M0 * c[0], M1 * c[2]
        c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & mask, (p0 >> 32) ^ c[3] ^ k[1], p0 & mask]
    return (c[0] >> 8) / 16777216.0


def test_philox_known_answer():
    # counter 0, key 0 -> 0x6627e8d5 (the generator's published test vector)
    assert int(philox_uniform(0, 0, 0) * 16777216) == 0x6627e8d5 >> 8


def run_sample(ops, logits, T, k=0, p=0.0, seed=0, counters=None):
    B, V = logits.shape
    counters = counters if counters is not None else [[b, 0] for b in range(B)]
    c = torch.tensor(counters, dtype=torch.int32, device=DEV)
    probs = torch.empty(B, V, device=DEV)
    out = torch.empty(B, dtype=torch.int32, device=DEV)
    ops.sample(logits.to(DEV).contiguous(), T, k, p, seed, c, probs, out)
    return out.tolist(), probs.cpu()


@pytest.mark.parametrize("V", [7, 384, 32000, 50001])
def test_greedy(ops, V):
    logits = rnd(5, V, seed=11)
    logits[1, V // 2] = 50.0
    logits[2, 0] = 50.0
    logits[3, V - 1] = 50.0
    logits[4, 3] = 50.0
    logits[4, V - 2] = 50.0                                 # equal maxima: the last index wins
    ids, _ = run_sample(ops, logits, 0.0)
    assert ids == [plain.greedy(logits[b]) for b in range(5)]
    assert ids[4] == V - 2
    ids, _ = run_sample(ops, logits, 0.0, k=3, p=0.5)       # T = 0 is greedy whatever else is set
    assert ids[1] == V // 2


@pytest.mark.parametrize("V", [13, 384, 32000])
@pytest.mark.parametrize("T,k,p", [(0.8, 0, 0.0), (1.0, 5, 0.0), (0.7, 0, 0.9), (1.3, 50, 0.6), (1.0, 10 ** 6, 1.0)])
def test_distribution_and_draw(ops, V, T, k, p):
    logits = rnd(4, V, seed=12, scale=3.0)
    seed = 1234567891011
    counters = [[3, 0], [3, 1], [9, 0], [0, 77]]
    ids, probs = run_sample(ops, logits, T, k, p, seed, counters)
    for b in range(4):
        want = plain.sample_distribution(logits[b], T, k or None, p or None)
        assert abs(float(probs[b].sum()) - 1) < 1e-4
        assert float((probs[b].double() - want).abs().max()) < 2e-6
        assert int((probs[b] > 0).sum()) == int((want > 0).sum())
        r = philox_uniform(seed, counters[b][1], counters[b][0])
        mine = plain.draw(probs[b].double(), r)
        assert ids[b] == mine or abs(float(probs[b].double().cumsum(0)[min(ids[b], mine)]) - r) < 1e-5


def test_top_k_ties_keep_index_order(ops):
    logits = torch.tensor([[1.0, 3.0, 1.0, 1.0, 2.0, -4.0]])
    _, probs = run_sample(ops, logits, 1.0, k=3)
    want = plain.sample_distribution(logits[0], 1.0, 3, None)
    assert (probs[0] > 0).tolist() == [True, True, False, False, True, False]
    assert float((probs[0].double() - want).abs().max()) < 1e-6


def test_draws_do_not_depend_on_batch_mates_and_follow_the_probabilities(ops):
    V = 8
    z = torch.tensor([[2.0, 1.0, 0.0, -1.0, 0.5, 1.5, -2.0, 0.2]])
    n = 4000
    counters = [[17, t] for t in range(n)]
    ids, probs = run_sample(ops, z.repeat(n, 1), 1.0, seed=5, counters=counters)
    freq = np.bincount(ids, minlength=V) / n
    p = probs[0].double().numpy()
    assert np.all(np.abs(freq - p) < 4 * np.sqrt(p * (1 - p) / n) + 1e-3)
    alone, _ = run_sample(ops, z, 1.0, seed=5, counters=[[17, 123]])
    assert alone[0] == ids[123]
    again, _ = run_sample(ops, z.repeat(n, 1), 1.0, seed=5, counters=counters)
    assert again == ids                                      # the seed decides
    other, _ = run_sample(ops, z.repeat(n, 1), 1.0, seed=6, counters=counters)
    assert other != ids


# ---- bfloat16 products on the matrix cores -----------------------------------------

@pytest.mark.parametrize("variant,M", [(112, 1), (112, 7), (111, 16), (212, 3), (411, 5), (222, 17), (222, 32),
                                       (421, 20), (242, 33), (441, 64), (142, 50)])
@pytest.mark.parametrize("N,K", [(50, 72), (16, 64), (130, 264), (200, 1000), (384, 96)])
def test_gemm_bf16_kernels(ops, variant, M, N, K):
    a = rnd(M, K, seed=21, dtype=torch.bfloat16)
    w = rnd(N, K, seed=22, dtype=torch.bfloat16)
    want = a.double() @ w.double().t()
    out = torch.full((M, N), float("nan"), device=DEV)
    ops.gemm_bf16(a.to(DEV), w.to(DEV), out, variant=variant)
    assert rel_err(out, want) < 3e-6
    base = rnd(M, N, seed=23)
    acc = base.clone().to(DEV)
    ops.gemm_bf16(a.to(DEV), w.to(DEV), acc, accumulate=True, variant=variant)
    assert rel_err(acc, want + base.double()) < 3e-6


@pytest.mark.parametrize("share", [5, 16, 17, 20, 31, 32])
@pytest.mark.parametrize("M,N,K", [(1, 50, 72), (7, 130, 264), (16, 200, 1000), (3, 384, 96)])
def test_gemm_bf16_in_shares_of_any_size(ops, share, M, N, K):
    """The kernel for at most 16 rows with `share` channels a workgroup (the launcher's way of giving
    every compute unit as much to read as the others): the bits of 16 channels a workgroup."""
    a = rnd(M, K, seed=21, dtype=torch.bfloat16).to(DEV)
    w = rnd(N, K, seed=22, dtype=torch.bfloat16).to(DEV)
    want = torch.full((M, N), float("nan"), device=DEV)
    ops.gemm_bf16(a, w, want, variant=112)
    out = torch.full((M, N), float("nan"), device=DEV)
    ops.gemm_bf16(a, w, out, variant=1000 + share)
    assert torch.equal(out, want)
    base = rnd(M, N, seed=23).to(DEV)
    acc, acc_want = base.clone(), base.clone()
    ops.gemm_bf16(a, w, acc, accumulate=True, variant=1000 + share)
    ops.gemm_bf16(a, w, acc_want, accumulate=True, variant=112)
    assert torch.equal(acc, acc_want)
    assert rel_err(out, a.double().cpu() @ w.double().cpu().t()) < 3e-6


def test_gemm_bf16_row_does_not_depend_on_the_batch(ops):
    a = rnd(64, 512, seed=24, dtype=torch.bfloat16).to(DEV)
    w = rnd(96, 512, seed=25, dtype=torch.bfloat16).to(DEV)
    outs = {}
    for M in (1, 9, 16, 17, 40, 64):
        o = torch.empty(M, 96, device=DEV)
        ops.gemm(a[:M].contiguous(), w, o)
        outs[M] = o
    for M in outs:
        assert torch.equal(outs[M][0], outs[64][0])
    assert rel_err(outs[64], a.double().cpu() @ w.double().cpu().t()) < 3e-6
    more = torch.empty(65, 96, device=DEV)
    with pytest.raises(ops.KernelError, match="at most 64"):      # more rows are not this entry point's
        ops.gemm_bf16(torch.cat([a, a[:1]]).contiguous(), w, more)


def test_gemm_dispatch_falls_back_when_k_is_odd(ops):
    a = rnd(3, 52, seed=26, dtype=torch.bfloat16)
    w = rnd(20, 52, seed=27, dtype=torch.bfloat16)
    out = torch.empty(3, 20, device=DEV)
    ops.gemm(a.to(DEV), w.to(DEV), out)                     # 52 % 8 != 0: plain kernel
    assert rel_err(out, a.double() @ w.double().t()) < 3e-6
    with pytest.raises(ops.KernelError, match="multiple of 8"):
        ops.gemm_bf16(a.to(DEV), w.to(DEV), out)


# ---- bfloat16 attention on the matrix cores -----------------------------------------

SHAPES = [(4, 2, 16, None), (6, 1, 32, 70), (5, 5, 48, 8), (8, 2, 128, 100), (2, 1, 256, None),
          (3, 3, 80, 64), (32, 8, 128, 200), (20, 1, 64, None), (4, 4, 160, 130), (6, 2, 96, None),
          (2, 2, 192, 50), (2, 1, 224, None)]


def transposed_values(ops, a, lens_cached, lens_new):
    """The step's values as the prefill kernel takes them: [nkv, d, columns], poisoned elsewhere."""
    off, cols = ops.aligned_columns(lens_cached, lens_new)
    v = a["v"].cpu()
    n, nkv, d = v.shape
    vt = torch.full((nkv, d, cols), float("nan"), dtype=v.dtype)
    r = 0
    for b, (c, nn) in enumerate(zip(lens_cached, lens_new)):
        for i in range(nn):
            vt[:, :, off[b] + (c % 64) + i] = v[r]
            r += 1
    return vt.to(DEV), torch.tensor(off, dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("nq,nkv,d,window", SHAPES)
def test_attention_prefill_bf16(ops, nq, nkv, d, window):
    """Whole prompts, prompts that go on from cached context (page-aligned and not), rows that end
    inside a block of 128, more than one block."""
    a = paged_case(ops, "bfloat16", nq, nkv, d, window, lens_cached=[0, 5, 130, 64, 200, 0],
                   lens_new=[17, 1, 3, 70, 129, 300], n_pages=60)
    n_tiles = sum(-(-n // 128) for n in [17, 1, 3, 70, 129, 300])
    vt, off = transposed_values(ops, a, [0, 5, 130, 64, 200, 0], [17, 1, 3, 70, 129, 300])
    ops.attn_prefill_bf16(a["q"], a["k"], vt, off, a["pages"], a["table"], a["ring"], a["row_pos"], a["cu"],
                          a["cached"], n_tiles, window, a["scale"], a["out"])
    assert rel_err(a["out"], a["want"]) < KTOL["bfloat16"]
    plain_out = torch.empty_like(a["out"])
    ops.attn_plain(a["q"], a["k"], a["v"], a["pages"], a["table"], a["ring"], a["row_seq"], a["row_pos"],
                   a["cu"], a["cached"], window, a["scale"], plain_out)
    assert rel_err(a["out"], plain_out.double()) < KTOL["bfloat16"]


@pytest.mark.parametrize("cut_tiles", [1, 3, 8])
@pytest.mark.parametrize("nq,nkv,d,window", SHAPES)
def test_attention_prefill_with_long_blocks_cut_into_runs(ops, monkeypatch, nq, nkv, d, window, cut_tiles):
    """A launch with fewer workgroups than compute units: the keys of a block with many tiles before it go
    to several workgroups, a run of tiles each, and a merge; the host lays the work out.  With runs of one or
    three tiles most blocks of the usual case are cut (cached context page-aligned and not, rows that end
    inside a block, windows whose edge falls in any run); with the usual eight a long sequence is."""
    lens_cached, lens_new = [0, 5, 130, 64, 200, 0], [17, 1, 3, 70, 129, 300]
    if cut_tiles == 8:
        lens_cached, lens_new = [900, 0, 64], [300, 1200, 5]
    monkeypatch.setattr(ops, "PREFILL_CUT_TILES", cut_tiles)
    a = paged_case(ops, "bfloat16", nq, nkv, d, window, lens_cached=lens_cached, lens_new=lens_new, n_pages=60)
    blocks = [(b, t) for b, n in enumerate(lens_new) for t in range(-(-n // 128))]
    n_tiles = len(blocks)

    def tiles_of(b, t):       # the tiles of 64 keys that the block's rows see: from the window's edge of its first row to its last row
        lo = lens_cached[b] + 128 * t
        hi = lens_cached[b] + min(128 * (t + 1), lens_new[b]) - 1
        first = max(0, lo - window + 1) // 64 if window else 0
        return first, hi // 64

    want_ways = {bt: min(ops.PREFILL_MAX_WAYS, (tiles_of(*bt)[1] - tiles_of(*bt)[0] + 1) // cut_tiles) for bt in blocks}
    vt, off = transposed_values(ops, a, lens_cached, lens_new)
    units = 2 * n_tiles * nq * ops.PREFILL_MAX_WAYS                     # room for every block in eight runs
    cuts = ops.prefill_cuts(lens_new, lens_cached, window, nq, units, DEV)
    if all(w < 2 for w in want_ways.values()):
        assert cuts is None                   # no block has tiles for two runs
        return
    cut_blocks = {bt: w for bt, w in want_ways.items() if w >= 2}
    assert cuts is not None and cuts.ways == max(cut_blocks.values())
    assert {(b, t): w for b, t, w, _ in cuts.blocks.cpu().tolist()} == cut_blocks
    items = cuts.items.cpu().tolist()
    assert cuts.n_items == len(items) == n_tiles + sum(w - 1 for w in cut_blocks.values())
    for bt in blocks:                         # a block's runs follow each other from its first tile to its last
        mine = sorted((lo, w & 0xffffff, (w >> 24) & 7, ((w >> 27) & 7) + 1 if w >> 30 else 0) for b, t, lo, w in items if (b, t) == bt)
        if bt not in cut_blocks:
            assert mine == [(0, 0, 0, 0)]
            continue
        first, last = tiles_of(*bt)
        assert [m[2] for m in mine] == list(range(cut_blocks[bt])) and all(m[3] == cut_blocks[bt] for m in mine)
        assert mine[0][0] == first and mine[-1][1] == last + 1
        assert all(x[1] == y[0] and x[1] - x[0] >= cut_tiles for x, y in zip(mine, mine[1:] + [(last + 1,)]))
    n = a["q"].shape[0]
    part = torch.full((n * nq * cuts.ways * (d + 4),), float("nan"), device=DEV)
    ops.attn_prefill_bf16(a["q"], a["k"], vt, off, a["pages"], a["table"], a["ring"], a["row_pos"], a["cu"],
                          a["cached"], n_tiles, window, a["scale"], a["out"], cuts=cuts, part=part)
    assert rel_err(a["out"], a["want"]) < KTOL["bfloat16"]
    whole = torch.empty_like(a["out"])
    ops.attn_prefill_bf16(a["q"], a["k"], vt, off, a["pages"], a["table"], a["ring"], a["row_pos"], a["cu"],
                          a["cached"], n_tiles, window, a["scale"], whole)
    assert rel_err(a["out"], whole.double()) < 1e-2                 # the runs' sums meet in another order
    cu = a["cu"].tolist()
    rows_whole = [r for (b, t) in blocks if (b, t) not in cut_blocks
                  for r in range(cu[b] + t * 128, cu[b] + min(lens_new[b], (t + 1) * 128))]
    assert torch.equal(a["out"][rows_whole], whole[rows_whole])     # blocks that are not cut keep their bits
    # the layout belongs to one step; too little room for the sums is refused
    with pytest.raises(ops.KernelError, match="laid out for"):
        ops.attn_prefill_bf16(a["q"], a["k"], vt, off, a["pages"], a["table"], a["ring"], a["row_pos"], a["cu"],
                              a["cached"], n_tiles + 1, window, a["scale"], a["out"], cuts=cuts, part=part)
    with pytest.raises(ops.KernelError, match="floats for"):
        ops.attn_prefill_bf16(a["q"], a["k"], vt, off, a["pages"], a["table"], a["ring"], a["row_pos"], a["cu"],
                              a["cached"], n_tiles, window, a["scale"], a["out"], cuts=cuts, part=part[:128])
    # a launch with more workgroups than compute units is left to the kernel's own order; fewer units to
    # spare mean fewer runs (a unit holds two workgroups), and longer ones once every other unit has a workgroup
    assert ops.prefill_cuts(lens_new, lens_cached, window, nq, n_tiles * nq - 1, DEV) is None
    fewer = ops.prefill_cuts(lens_new, lens_cached, window, nq, 2 * n_tiles * nq, DEV)
    assert fewer is None or fewer.ways <= 4
    fuller = ops.prefill_cuts(lens_new, lens_cached, window, nq, n_tiles * nq, DEV)
    assert fuller is None or (fuller.ways == 2 and all((w & 0xffffff) - lo >= 2 * cut_tiles
                                                       for _, _, lo, w in fuller.items.cpu().tolist() if w >> 30))


@pytest.mark.parametrize("through_lds", [True, False])
@pytest.mark.parametrize("splits", [1, 3, 8])
@pytest.mark.parametrize("nq,nkv,d,window", SHAPES)
def test_attention_decode_bf16(ops, nq, nkv, d, window, splits, through_lds):
    """Both decode kernels: the one that stages whole pages in LDS (head sizes 64, 128, 256) and the one that
    reads them into registers (every head size; the switch sends those three through it too)."""
    if not through_lds and d not in (64, 128, 256):
        pytest.skip("this head size has one kernel")
    lens = [0, 63, 64, 300, 191, 31, 32, 700]
    a = paged_case(ops, "bfloat16", nq, nkv, d, window, lens_cached=lens, lens_new=[1] * len(lens), seed=3,
                   n_pages=60)
    ops.kv_commit(a["k"], a["v"], a["row_seq"], a["row_pos"], a["after"], a["table"], a["ring"], a["pages"])
    B = len(lens)
    part = torch.full((B * nq * splits * (d + 2),), float("nan"), device=DEV)
    was = ops.decode_through_lds(through_lds)
    try:
        ops.attn_decode_bf16(a["q"], a["pages"], a["table"], a["ring"], a["row_pos"], window, a["scale"], splits,
                             part, a["out"])
    finally:
        ops.decode_through_lds(was)
    assert was is True                                     # the default
    assert rel_err(a["out"], a["want"]) < KTOL["bfloat16"]


def test_attention_decode_through_lds_over_many_pages(ops):
    """More than 64 pages to one workgroup (its page ids are fetched 64 at a time), a ring that wraps, a window
    that begins inside a page, and stale rows of NaN behind every sequence's end."""
    nq, nkv, d = 8, 2, 128
    for window, lens in ((None, [4500, 64 * 70 - 1, 1]), (2100, [4500, 2099, 2200])):
        a = paged_case(ops, "bfloat16", nq, nkv, d, window, lens_cached=lens, lens_new=[1] * len(lens), seed=9,
                       n_pages=230)
        ops.kv_commit(a["k"], a["v"], a["row_seq"], a["row_pos"], a["after"], a["table"], a["ring"], a["pages"])
        for splits in (1, 2):
            part = torch.full((len(lens) * nq * splits * (d + 2),), float("nan"), device=DEV)
            out = torch.full_like(a["out"], float("nan"))
            ops.attn_decode_bf16(a["q"], a["pages"], a["table"], a["ring"], a["row_pos"], window, a["scale"], splits,
                                 part, out)
            assert rel_err(out, a["want"]) < KTOL["bfloat16"], (window, splits)


def test_attention_bf16_far_key_and_edge(ops):
    """As for the plain kernel: a key that stands out far back, and the two sides of the window's
    edge, through the decode and the prefill kernel."""
    from torchless_rs_amd.cache import PAGE
    nq, nkv, d, T = 4, 1, 64, 700
    g = torch.Generator().manual_seed(5)
    i32 = lambda l: torch.tensor(l, dtype=torch.int32, device=DEV)
    for window, far, visible in [(None, 3, True), (200, 499, False), (200, 500, True), (200, 699, True)]:
        k = torch.randn(T, nkv, d, generator=g) * 0.1
        v = torch.randn(T, nkv, d, generator=g)
        qv = torch.randn(d, generator=g)
        qv = qv / qv.norm()
        k[far, 0] = qv * 60.0
        q = (qv * 8.0).view(1, 1, d).repeat(1, nq, 1).to(torch.bfloat16)
        ring = -(-window // PAGE) if window else 11
        pages = torch.full((11, 2, nkv, PAGE, d), float("nan"), dtype=torch.bfloat16)
        table = torch.tensor([[7, 2, 9, 0, 5, 1, 10, 3, 8, 4, 6][:ring]], dtype=torch.int32)
        for p in range(max(0, T - ring * PAGE), T):
            pg = int(table[0, (p // PAGE) % ring])
            pages[pg, 0, :, p % PAGE] = k[p].to(torch.bfloat16)
            pages[pg, 1].view(nkv, d, PAGE)[:, :, p % PAGE] = v[p].to(torch.bfloat16)
        out = torch.empty(1, nq, d, dtype=torch.bfloat16, device=DEV)
        part = torch.empty(nq * 4 * (d + 2), device=DEV)
        ops.attn_decode_bf16(q.to(DEV), pages.to(DEV), table.to(DEV), ring, i32([T - 1]), window,
                             1.0 / math.sqrt(d), 4, part, out)
        assert (rel_err(out[0, 0], v[far, 0].to(torch.bfloat16)) < 1e-2) == visible, (window, far)
        assert torch.isfinite(out).all()
        # the same through the prefill kernel: the last 2 rows are new, the rest is cached
        pages2 = pages.clone()                            # rows >= n_cached are there but are not read
        kn = k[T - 2:].to(torch.bfloat16).to(DEV)
        vn = v[T - 2:].to(torch.bfloat16).to(DEV)
        q2 = torch.cat([torch.zeros_like(q), q]).to(DEV)
        out2 = torch.empty(2, nq, d, dtype=torch.bfloat16, device=DEV)
        off, cols = ops.aligned_columns([T - 2], [2])
        vt = torch.full((nkv, d, cols), float("nan"), dtype=torch.bfloat16, device=DEV)
        vt[:, :, (T - 2) % 64] = vn[0]
        vt[:, :, (T - 2) % 64 + 1] = vn[1]
        ops.attn_prefill_bf16(q2, kn, vt, i32(off), pages2.to(DEV), table.to(DEV), ring, i32([T - 2, T - 1]),
                              i32([0, 2]), i32([T - 2]), 1, window, 1.0 / math.sqrt(d), out2)
        assert (rel_err(out2[1, 0], v[far, 0].to(torch.bfloat16)) < 1e-2) == visible, (window, far)
        assert torch.isfinite(out2).all()


@pytest.mark.parametrize("variant,M", [(411, 1), (411, 9), (421, 30), (441, 64)])
@pytest.mark.parametrize("I,K", [(64, 72), (160, 64), (96, 200)])
def test_gemm_bf16_paired_silu_epilogue(ops, variant, M, I, K):
    """gate and up rows interleaved in groups of 32: the product writes silu(gate) * up."""
    from torchless_rs_amd.parts.linear import interleave_pairs
    a = rnd(M, K, seed=31, dtype=torch.bfloat16)
    g = rnd(I, K, seed=32, dtype=torch.bfloat16, scale=0.3)
    u = rnd(I, K, seed=33, dtype=torch.bfloat16, scale=0.3)
    w = interleave_pairs(g, u)
    assert torch.equal(w[:32], g[:32]) and torch.equal(w[32:64], u[:32]) and torch.equal(w[64:96], g[32:64])
    want = plain.silu(a.double() @ g.double().t()) * (a.double() @ u.double().t())
    out = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16(a.to(DEV), w.to(DEV), out, variant=variant, silu_pair=True)
    assert rel_err(out, want) < KTOL["bfloat16"]
    out2 = torch.empty_like(out)
    ops.gemm_bf16(a.to(DEV), w.to(DEV), out2, silu_pair=True)           # the kernel the size picks
    assert rel_err(out2, want) < KTOL["bfloat16"]


@pytest.mark.parametrize("M,N,K", [(129, 50, 72), (300, 130, 264), (200, 384, 96)])
def test_gemm_library_products(ops, M, N, K):
    """Above LIBRARY_ROWS rows the dispatcher hands the product to the BLAS library:
    float32 out (stored or accumulated) and bfloat16 out (stored)."""
    a = rnd(M, K, seed=41, dtype=torch.bfloat16)
    w = rnd(N, K, seed=42, dtype=torch.bfloat16)
    want = a.double() @ w.double().t()
    assert M > ops.LIBRARY_ROWS
    out = torch.full((M, N), float("nan"), device=DEV)
    ops.gemm(a.to(DEV), w.to(DEV), out)
    assert rel_err(out, want) < 3e-6
    base = rnd(M, N, seed=43)
    acc = base.clone().to(DEV)
    ops.gemm(a.to(DEV), w.to(DEV), acc, accumulate=True)
    assert rel_err(acc, want + base.double()) < 3e-6
    ours = torch.empty(M, N, device=DEV)
    ops.gemm_plain(a.to(DEV), w.to(DEV), ours)
    assert rel_err(ours, out) < 1e-6                         # the plain kernel agrees up to rounding
    o16 = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.gemm_library(a.to(DEV), w.to(DEV), o16)
    assert rel_err(o16, want) < KTOL["bfloat16"]
    with pytest.raises(ops.KernelError, match="accumulate"):
        ops.gemm_library(a.to(DEV), w.to(DEV), o16, accumulate=True)


@pytest.mark.parametrize("n,I", [(1, 32), (5, 96), (131, 480)])
def test_silu_mul_pairs(ops, n, I):
    from torchless_rs_amd.parts.linear import interleave_pairs
    g = rnd(I, n, seed=44, dtype=torch.bfloat16, scale=3.0)
    u = rnd(I, n, seed=45, dtype=torch.bfloat16, scale=3.0)
    gu = interleave_pairs(g, u).t().contiguous()            # [n, 2I], columns in groups of 64
    out = torch.full((n, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.silu_mul_pairs(gu.to(DEV), out)
    assert rel_err(out, (plain.silu(g.double()) * u.double()).t()) < KTOL["bfloat16"]
    with pytest.raises(ops.KernelError, match="steps of 32"):
        ops.silu_mul_pairs(torch.zeros(2, 80, dtype=torch.bfloat16, device=DEV),
                           torch.zeros(2, 40, dtype=torch.bfloat16, device=DEV))


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [None, 70])
def test_rope_commit_equals_rope_split_then_commit(ops, dt, window):
    from torchless_rs_amd.parts.position import Rotary
    nq, nkv, d = 6, 2, 48
    a = paged_case(ops, dt, nq, nkv, d, window, lens_cached=[0, 63, 64, 300], lens_new=[1] * 4, seed=7)
    n = 4
    qkv = rnd(n, (nq + 2 * nkv) * d, seed=8).to(DEV)
    inv = Rotary(d, 777.0).inv_freq(DEV)
    q1, k1, v1 = (torch.empty(n, h, d, dtype=DT[dt], device=DEV) for h in (nq, nkv, nkv))
    ops.rope_split(qkv, a["row_pos"], inv, nq, nkv, d, q1, k1, v1)
    pages1 = a["pages"].clone()
    ops.kv_commit(k1, v1, a["row_seq"], a["row_pos"], a["after"], a["table"], a["ring"], pages1)
    q2 = torch.empty_like(q1)
    pages2 = a["pages"].clone()
    ops.rope_commit(qkv, a["row_pos"], inv, a["table"], a["ring"], nq, nkv, d, q2, pages2)
    assert torch.equal(q1, q2)
    assert torch.equal(torch.nan_to_num(pages1.float(), nan=-7.0), torch.nan_to_num(pages2.float(), nan=-7.0))
    assert not torch.equal(torch.nan_to_num(pages2.float(), nan=-7.0), torch.nan_to_num(a["pages"].float(), nan=-7.0))


@pytest.mark.parametrize("nq,nkv,d,K,lens", [(6, 2, 48, 72, [0, 63, 64, 300]), (4, 4, 16, 264, [5]),
                                             (8, 2, 128, 1000, [9, 64, 127, 128, 640, 2, 3, 4, 5, 6, 7, 8, 70, 71, 72, 73])])
@pytest.mark.parametrize("window", [None, 70])
def test_qkv_rope_commit_equals_product_then_rope_commit(ops, nq, nkv, d, K, lens, window):
    """The fused kernel of single-token steps gives the bits of the product followed by rope_commit."""
    from torchless_rs_amd.parts.position import Rotary
    n = len(lens)
    c = paged_case(ops, "bfloat16", nq, nkv, d, window, lens_cached=lens, lens_new=[1] * n, seed=9, n_pages=60)
    y = rnd(n, K, seed=10, dtype=torch.bfloat16).to(DEV)
    w = rnd((nq + 2 * nkv) * d, K, seed=11, dtype=torch.bfloat16, scale=0.2).to(DEV)
    inv = Rotary(d, 10000.0).inv_freq(DEV)
    qkv = torch.empty(n, (nq + 2 * nkv) * d, device=DEV)
    ops.gemm(y, w, qkv)
    q1 = torch.empty(n, nq, d, dtype=torch.bfloat16, device=DEV)
    pages1 = c["pages"].clone()
    ops.rope_commit(qkv, c["row_pos"], inv, c["table"], c["ring"], nq, nkv, d, q1, pages1)
    assert ops.qkv_rope_commit_ok(y, w, d, c["pages"])
    for units in (0, 1, 2, 3, 4):                            # the launcher's choice, then 8 to 32 weight rows a workgroup
        q2 = torch.full_like(q1, float("nan"))
        pages2 = c["pages"].clone()
        ops.qkv_rope_commit(y, w, c["row_pos"], inv, c["table"], c["ring"], nq, nkv, d, q2, pages2, units=units)
        assert torch.equal(q1, q2)
        assert torch.equal(torch.nan_to_num(pages1.float(), nan=-7.0), torch.nan_to_num(pages2.float(), nan=-7.0))
    # and against the plain rotation of the plain product
    full = (y.double().cpu() @ w.double().cpu().t()).view(n, nq + 2 * nkv, d)
    pos = c["row_pos"].cpu().long()
    want_q = plain.rope(full[:, :nq], pos, 10000.0)
    assert rel_err(q2, want_q) < KTOL["bfloat16"]
    assert not ops.qkv_rope_commit_ok(torch.zeros(17, K, dtype=torch.bfloat16, device=DEV), w, d, pages2)
    with pytest.raises(ops.KernelError, match="units a workgroup"):
        ops.qkv_rope_commit(y, w, c["row_pos"], inv, c["table"], c["ring"], nq, nkv, d, q2, pages2, units=5)
    with pytest.raises(ops.KernelError, match="steps of 16"):
        ops.qkv_rope_commit(y, w[: (nq + 2 * nkv) * 8].contiguous(), c["row_pos"], inv[: 4].contiguous(), c["table"],
                            c["ring"], nq, nkv, 8, torch.empty(n, nq, 8, dtype=torch.bfloat16, device=DEV),
                            torch.zeros(60, 2, nkv, 64, 8, dtype=torch.bfloat16, device=DEV))


# ---- an RMSNorm cut in two around products of at most 16 rows ----------------------------

@pytest.mark.parametrize("M", [1, 5, 16])
@pytest.mark.parametrize("N,K,N2", [(200, 72, 50), (64, 264, 16384), (1000, 96, 130), (4616, 72, 48), (8296, 40, 48)])   # the last two: more tiles of 16 channels than compute units, in one round of workgroups and in two
def test_gemm_norm_halves(ops, M, N, K, N2):
    """The product that completes the stream writes x * w and its workgroups' sums of x^2;
    the product that reads them applies rsqrt(mean + eps): together the plain norm between."""
    eps = 1e-5
    x0 = rnd(M, N, seed=51, scale=2.0)
    a = rnd(M, K, seed=52, dtype=torch.bfloat16)
    w = rnd(N, K, seed=53, dtype=torch.bfloat16)
    g = (1 + 0.2 * rnd(N, seed=54))
    x = x0.clone().to(DEV)
    xt = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    ssq = torch.full((16, -(-N // 16)), float("nan"), device=DEV)                # [row][workgroup]
    groups = ops.gemm_bf16_norm(a.to(DEV), w.to(DEV), x, accumulate=True, norm_weight=g.to(DEV), xt=xt, ssq_out=ssq)
    want_x = x0.double() + a.double() @ w.double().t()
    assert rel_err(x, want_x) < 3e-6
    plain_x = x0.clone().to(DEV)
    ops.gemm_bf16(a.to(DEV), w.to(DEV), plain_x, accumulate=True)
    assert torch.equal(plain_x, x)                                    # the stream itself is unchanged by the extra
    assert 0 < groups <= -(-N // 16)                                  # workgroups own 16 channels or more
    written = ssq.flatten()[: 16 * groups].view(16, groups)          # [row][workgroup], as many columns as workgroups
    assert rel_err(written[:M].sum(1), (x.double().cpu() ** 2).sum(1)) < 1e-5
    assert rel_err(xt, x.double().cpu() * g.double()) < KTOL["bfloat16"]
    factor = ops.RowFactor(ssq, groups, N, eps)
    normed = plain.rmsnorm(x.double().cpu(), g.double(), eps)
    w2 = rnd(N2, N, seed=55, dtype=torch.bfloat16, scale=0.3)
    out = torch.full((M, N2), float("nan"), device=DEV)
    ops.gemm_bf16_norm(xt, w2.to(DEV), out, factor=factor)
    assert rel_err(out, normed @ w2.double().t()) < KTOL["bfloat16"]
    # exactly: the unscaled product times the factor of the row
    raw = torch.empty(M, N2, device=DEV)
    ops.gemm_bf16(xt, w2.to(DEV), raw)
    r = torch.rsqrt(written[:M].double().sum(1) / N + eps).float()
    assert rel_err(out, raw.double().cpu() * r.double().cpu()[:, None]) < 1e-6
    if N2 % 64 == 0:
        from torchless_rs_amd.parts.linear import interleave_pairs
        h = torch.full((M, N2 // 2), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.gemm_bf16_norm(xt, w2.to(DEV), h, silu_pair=True, factor=factor)
        full = (normed @ w2.double().t()).view(M, N2 // 64, 2, 32)
        assert rel_err(h, (plain.silu(full[:, :, 0]) * full[:, :, 1]).reshape(M, N2 // 2)) < KTOL["bfloat16"]
    with pytest.raises(ops.KernelError, match="at most 16 rows"):
        ops.gemm_bf16_norm(torch.zeros(17, K, dtype=torch.bfloat16, device=DEV), w.to(DEV),
                           torch.zeros(17, N, device=DEV))
    with pytest.raises(ops.KernelError, match="accumulate"):
        ops.gemm_bf16_norm(a.to(DEV), w.to(DEV), x, norm_weight=g.to(DEV), xt=xt, ssq_out=ssq)


def test_qkv_rope_commit_with_row_factor(ops):
    from torchless_rs_amd.parts.position import Rotary
    nq, nkv, d, K, lens, eps = 6, 2, 48, 136, [0, 63, 64, 300, 7], 1e-6
    n = len(lens)
    c = paged_case(ops, "bfloat16", nq, nkv, d, None, lens_cached=lens, lens_new=[1] * n, seed=12, n_pages=60)
    x = rnd(n, K, seed=13, scale=3.0)
    g = (1 + 0.2 * rnd(K, seed=14))
    xt = (x * g).to(torch.bfloat16).to(DEV)
    parts = 5                                                   # the sums of squares, cut into 5 unequal shares
    cuts = [0, 10, 50, 51, 100, K]
    ssq = torch.zeros(16, parts)
    for j in range(parts):
        ssq[:n, j] = (x[:, cuts[j]:cuts[j + 1]] ** 2).sum(1)
    factor = ops.RowFactor(ssq.to(DEV), parts, K, eps)
    w = rnd((nq + 2 * nkv) * d, K, seed=15, dtype=torch.bfloat16, scale=0.2).to(DEV)
    inv = Rotary(d, 10000.0).inv_freq(DEV)
    q = torch.full((n, nq, d), float("nan"), dtype=torch.bfloat16, device=DEV)
    pages = c["pages"].clone()
    ops.qkv_rope_commit(xt, w, c["row_pos"], inv, c["table"], c["ring"], nq, nkv, d, q, pages, factor=factor)
    y = plain.rmsnorm(x.double(), g.double(), eps)
    full = (y @ w.double().cpu().t()).view(n, nq + 2 * nkv, d)
    pos = c["row_pos"].cpu().long()
    assert rel_err(q, plain.rope(full[:, :nq], pos, 10000.0)) < KTOL["bfloat16"]
    want_k = plain.rope(full[:, nq:nq + nkv], pos, 10000.0)
    table = c["table"].cpu()
    for b in range(n):
        p = int(pos[b]); pg = int(table[b, p // 64])
        assert rel_err(pages[pg, 0, :, p % 64], want_k[b]) < KTOL["bfloat16"]
        assert rel_err(pages[pg, 1].reshape(nkv, d, 64)[:, :, p % 64], full[b, nq + nkv:]) < KTOL["bfloat16"]


# ---- the tiled copy of a weight that steps of at most 16 rows stream from ---------------------

def tiled_by_formula(w, rows=None, R=16):
    """[ceil(N/R), K/64, 2, 4, R, 8] with (T, s, c, g, r, e) = w[rows[R T + r], 64 s + 16 g + 8 c + e]; the
    places of the last tile behind row N are zero."""
    N, K = w.shape
    src = w if rows is None else w[rows.long()]
    T = -(-N // R)
    if T * R != N:
        src = torch.cat([src, torch.zeros(T * R - N, K, dtype=w.dtype, device=w.device)])
    return src.view(T, R, K // 64, 4, 2, 8).permute(0, 2, 4, 3, 1, 5).contiguous()


@pytest.mark.parametrize("N,K", [(16, 64), (48, 192), (4112, 320), (5120, 128)])
def test_tile_weights(ops, N, K):
    """Tiles as high as a workgroup's share of the channels (16 while the device has a compute unit for
    every 16 channels, N over the units beyond), 16 for a copy with its own order of rows, any asked for."""
    w = rnd(N, K, seed=61, dtype=torch.bfloat16).to(DEV)
    R = ops.tile_height(N)
    units = ops.compute_units(DEV)
    assert R == (16 if N // 16 <= units else -(-N // (units * -(-N // (32 * units)))))
    assert torch.equal(ops.tile_weights(w), tiled_by_formula(w, R=R))
    rows = torch.randperm(N, generator=torch.Generator().manual_seed(62)).to(torch.int32).to(DEV)
    assert torch.equal(ops.tile_weights(w, rows), tiled_by_formula(w, rows))
    for h in (16, 17, 20, 32):
        assert torch.equal(ops.tile_weights(w, rows, height=h), tiled_by_formula(w, rows, R=h))
    for bad in (w[:, : K - 8].contiguous(), w[: N - 8].contiguous()):
        with pytest.raises(ops.KernelError, match="multiple of 16"):
            ops.tile_weights(bad)
    for h in (8, 15, 33):
        with pytest.raises(ops.KernelError, match="16 to 32"):
            ops.tile_weights(w, height=h)
    assert ops.tiles_fit(N, K) and not ops.tiles_fit(N + 8, K) and not ops.tiles_fit(N, K + 32)


@pytest.mark.parametrize("M", [1, 7, 16])
@pytest.mark.parametrize("N,K", [(16, 64), (48, 192), (4112, 320), (96, 4096), (8208, 128), (5120, 256), (6144, 128)])
def test_products_from_the_tiled_copy_give_the_same_bits(ops, M, N, K):
    """The same values meet in the same MFMAs in the same order, wherever they were read from (the last
    four sizes: more tiles of 16 channels than compute units, so shares and tiles of 17, 17, 20 and 24 rows)."""
    a = rnd(M, K, seed=63, dtype=torch.bfloat16).to(DEV)
    w = rnd(N, K, seed=64, dtype=torch.bfloat16).to(DEV)
    tiles = ops.tile_weights(w)
    x0 = rnd(M, N, seed=65).to(DEV)
    for accumulate in (False, True):
        got, want = x0.clone(), x0.clone()
        ops.gemm_bf16(a, w, want, accumulate=accumulate)
        ops.gemm_bf16(a, w, got, accumulate=accumulate, tiles=tiles)
        assert torch.equal(got, want)
        assert rel_err(got, (x0.double().cpu() if accumulate else 0) + a.double().cpu() @ w.double().cpu().t()) < 1e-5
    # with both halves of a norm around it
    g = (1 + 0.2 * rnd(N, seed=66)).to(DEV)
    res = []
    for t in (None, tiles):
        x = x0.clone()
        xt = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        ssq = torch.full((16, N // 16), float("nan"), device=DEV)
        groups = ops.gemm_bf16_norm(a, w, x, accumulate=True, norm_weight=g, xt=xt, ssq_out=ssq, tiles=t)
        res.append((x, xt, ssq.flatten()[: 16 * groups].view(16, groups)[:M].clone(), groups))
    assert 0 < res[0][3] == res[1][3] <= N // 16
    for u, v in zip(res[0][:3], res[1][:3]):
        assert torch.equal(u, v)
    ssq_in = (torch.rand(16, 3, generator=torch.Generator().manual_seed(67)) * K).to(DEV)
    factor = ops.RowFactor(ssq_in, 3, K, 1e-5)
    o1, o2 = torch.empty(M, N, device=DEV), torch.empty(M, N, device=DEV)
    ops.gemm_bf16_norm(a, w, o1, factor=factor)
    ops.gemm_bf16_norm(a, w, o2, factor=factor, tiles=tiles)
    assert torch.equal(o1, o2)
    # a copy of another weight's shape is refused, and one with tiles of another height than the kernel reads
    with pytest.raises(ops.KernelError, match="tiles"):
        ops.gemm_bf16(a, w, o1, tiles=tiles.view(-1)[: tiles.numel() // 2].clone())
    other = 24 if ops.tile_height(N) != 24 else 16
    with pytest.raises(ops.KernelError, match="tiles of"):
        ops.gemm_bf16(a, w, o1, tiles=ops.tile_weights(w, height=other))


@pytest.mark.parametrize("nq,nkv,d,K,lens", [(6, 2, 48, 64, [0, 63, 64, 300]), (4, 4, 16, 320, [5]), (3, 1, 256, 128, [7, 200]),
                                             (8, 2, 128, 1024, [9, 64, 127, 128, 640, 2, 3, 4, 5, 6, 7, 8, 70, 71, 72, 73])])
def test_qkv_rope_commit_from_the_tiled_copy(ops, nq, nkv, d, K, lens):
    from torchless_rs_amd.parts.position import Rotary
    n = len(lens)
    c = paged_case(ops, "bfloat16", nq, nkv, d, None, lens_cached=lens, lens_new=[1] * n, seed=19, n_pages=60)
    y = rnd(n, K, seed=20, dtype=torch.bfloat16).to(DEV)
    w = rnd((nq + 2 * nkv) * d, K, seed=21, dtype=torch.bfloat16, scale=0.2).to(DEV)
    inv = Rotary(d, 10000.0).inv_freq(DEV)
    rows = ops.qkv_tile_rows(nq, nkv, d, DEV)
    assert sorted(rows.tolist()) == list(range((nq + 2 * nkv) * d))
    head0 = rows[:16].tolist()                       # a tile of a rotated head: 8 channels and their partners
    assert head0 == list(range(8)) + list(range(d // 2, d // 2 + 8))
    v0 = (nq + nkv) * d
    assert rows[v0:v0 + 16].tolist() == list(range(v0, v0 + 16))
    tiles = ops.tile_weights(w, rows)
    ssq_in = (torch.rand(16, 4, generator=torch.Generator().manual_seed(22)) * K).to(DEV)
    for factor in (None, ops.RowFactor(ssq_in, 4, K, 1e-6)):
        for units in (0, 1, 2, 3, 4):
            out = []
            for t in (None, tiles):
                q = torch.full((n, nq, d), float("nan"), dtype=torch.bfloat16, device=DEV)
                pages = c["pages"].clone()
                ops.qkv_rope_commit(y, w, c["row_pos"], inv, c["table"], c["ring"], nq, nkv, d, q, pages,
                                    factor=factor, units=units, tiles=t)
                out.append((q, torch.nan_to_num(pages.float(), nan=-7.0)))
            assert torch.equal(out[0][0], out[1][0])
            assert torch.equal(out[0][1], out[1][1])
    assert not torch.equal(out[1][1], torch.nan_to_num(c["pages"].float(), nan=-7.0))


# ---- many channels against at most 16 rows: whole rows of the weights, 1 KB a load --------------

@pytest.mark.parametrize("M", [1, 5, 16])
@pytest.mark.parametrize("N,K", [(64, 512), (192, 1536), (128, 2560), (320, 1024), (64, 3584)])
def test_gemm_rows_kernel(ops, M, N, K):
    variant = 2
    a = rnd(M, K, seed=71, dtype=torch.bfloat16).to(DEV)
    w = rnd(N, K, seed=72, dtype=torch.bfloat16, scale=0.3).to(DEV)
    want = a.double().cpu() @ w.double().cpu().t()
    out = torch.full((M, N), float("nan"), device=DEV)
    ops.gemm_bf16(a, w, out, variant=variant)
    assert rel_err(out, want) < 1e-5
    x0 = rnd(M, N, seed=73).to(DEV)
    acc = x0.clone()
    ops.gemm_bf16(a, w, acc, accumulate=True, variant=variant)
    assert rel_err(acc, x0.double().cpu() + want) < 1e-5
    # a row's result does not depend on the rows beside it
    alone = torch.empty(1, N, device=DEV)
    ops.gemm_bf16(a[M - 1:].contiguous(), w, alone, variant=variant)
    assert torch.equal(alone[0], out[M - 1])
    h = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16(a, w, h, silu_pair=True, variant=2)
    full = want.view(M, N // 64, 2, 32)
    assert rel_err(h, (plain.silu(full[:, :, 0]) * full[:, :, 1]).reshape(M, N // 2)) < KTOL["bfloat16"]
    with pytest.raises(ops.KernelError, match="gemm_rows"):
        ops.gemm_bf16(a[:, : K - 64].contiguous(), w[:, : K - 64].contiguous(), out, variant=variant)


def test_wide_products_of_few_rows_take_the_rows_kernel(ops):
    """The dispatcher sends gate|up (paired epilogue, with the norm's factor) and a head-sized product
    to the kernel that reads whole rows, and gets what the other kernels get."""
    M, K, N = 6, 1024, 16384 + 64
    a = rnd(M, K, seed=74, dtype=torch.bfloat16).to(DEV)
    w = rnd(N, K, seed=75, dtype=torch.bfloat16, scale=0.2).to(DEV)
    want = a.double().cpu() @ w.double().cpu().t()
    got, forced, other = (torch.empty(M, N, device=DEV) for _ in range(3))
    ops.gemm_bf16(a, w, got)
    ops.gemm_bf16(a, w, forced, variant=2)
    ops.gemm_bf16(a, w, other, variant=411)
    assert torch.equal(got, forced)
    assert rel_err(got, want) < 1e-5 and rel_err(other, want) < 1e-5
    ssq = (torch.rand(16, 5, generator=torch.Generator().manual_seed(76)) * K).to(DEV)
    factor = ops.RowFactor(ssq, 5, K, 1e-5)
    r = torch.rsqrt(ssq[:M].double().sum(1).cpu() / K + 1e-5)
    h = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16_norm(a, w, h, silu_pair=True, factor=factor)
    full = (want * r[:, None]).view(M, N // 64, 2, 32)
    assert rel_err(h, (plain.silu(full[:, :, 0]) * full[:, :, 1]).reshape(M, N // 2)) < KTOL["bfloat16"]
    out = torch.empty(M, N, device=DEV)
    ops.gemm_bf16_norm(a, w, out, factor=factor)
    assert rel_err(out, want * r[:, None]) < 1e-5


# ---- 17..128 rows: shared activations, K cut into partial sums (above 64 rows the k-step is 128) --

@pytest.mark.parametrize("M", [17, 32, 33, 48, 50, 64, 5, 65, 80, 97, 112, 128])
@pytest.mark.parametrize("N,K,S", [(50, 72, 1), (64, 512, 2), (130, 776, 3), (200, 2000, 7), (384, 96, 1), (96, 4096, 16)])
def test_gemm_mid_bf16(ops, M, N, K, S):
    a = rnd(M, K, seed=41, dtype=torch.bfloat16)
    w = rnd(N, K, seed=42, dtype=torch.bfloat16)
    want = a.double() @ w.double().t()
    if S == 1:
        out = torch.full((M, N), float("nan"), device=DEV)
        ops.gemm_mid_bf16(a.to(DEV), w.to(DEV), out)
        assert rel_err(out, want) < 3e-6
        base = rnd(M, N, seed=43)
        acc = base.clone().to(DEV)
        ops.gemm_mid_bf16(a.to(DEV), w.to(DEV), acc, accumulate=True)
        assert rel_err(acc, want + base.double()) < 3e-6
        return
    parts = torch.full((S, M, N), float("nan"), device=DEV)
    ops.gemm_mid_bf16(a.to(DEV), w.to(DEV), parts, S)
    assert rel_err(parts.sum(0), want) < 3e-6
    base = rnd(M, N, seed=44)
    x = base.clone().to(DEV)
    ops.add_partials(x, parts)
    assert rel_err(x, want + base.double()) < 3e-6
    if N % 4 == 0:
        x2 = base.clone().to(DEV)
        g = (1 + 0.1 * rnd(N, seed=45)).to(DEV)
        y = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        ops.add_rmsnorm(x2, parts, g, 1e-5, y)
        assert torch.equal(x2, x)
        assert rel_err(y, plain.rmsnorm(x.double().cpu(), g.double().cpu(), 1e-5)) < KTOL["bfloat16"]


@pytest.mark.parametrize("M", [20, 64, 72, 128])
def test_gemm_mid_paired_silu_and_row_independence(ops, M):
    from torchless_rs_amd.parts.linear import interleave_pairs
    I, K = 160, 200
    a = rnd(M, K, seed=46, dtype=torch.bfloat16)
    g = rnd(I, K, seed=47, dtype=torch.bfloat16, scale=0.3)
    u = rnd(I, K, seed=48, dtype=torch.bfloat16, scale=0.3)
    out = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.gemm_mid_bf16(a.to(DEV), interleave_pairs(g, u).to(DEV), out, silu_pair=True)
    want = plain.silu(a.double() @ g.double().t()) * (a.double() @ u.double().t())
    assert rel_err(out, want) < KTOL["bfloat16"]
    # a row's result does not depend on the other rows of the batch
    w = rnd(96, K, seed=49, dtype=torch.bfloat16).to(DEV)
    full = torch.empty(M, 96, device=DEV)
    ops.gemm_mid_bf16(a.to(DEV), w, full)
    few = torch.empty(17, 96, device=DEV)
    ops.gemm_mid_bf16(a[:17].contiguous().to(DEV), w, few)
    assert torch.equal(few, full[:17])


@pytest.mark.parametrize("waves,kc", [(4, 128), (7, 128), (8, 128), (4, 64), (7, 64), (8, 64)])
@pytest.mark.parametrize("M,N,K,S", [(17, 64, 128, 1), (33, 200, 1024, 2), (64, 256, 512, 1), (100, 336, 1152, 3),
                                     (128, 520, 2048, 4), (5, 40, 384, 1), (96, 130, 256, 2)])
def test_gemm_ring_bf16(ops, waves, kc, M, N, K, S):
    """The product whose operands go from memory straight into a ring of LDS stages: every number of
    waves a workgroup and both stage sizes, rows and channels that fill no tile, K cut into slices
    of unequal numbers of stages; stored, accumulated, and as partial sums."""
    a = rnd(M, K, seed=51, dtype=torch.bfloat16)
    w = rnd(N, K, seed=52, dtype=torch.bfloat16)
    want = a.double() @ w.double().t()
    if S == 1:
        out = torch.full((M, N), float("nan"), device=DEV)
        ops.gemm_ring_bf16(a.to(DEV), w.to(DEV), out, waves=waves, kc=kc)
        assert rel_err(out, want) < 3e-6
        base = rnd(M, N, seed=53)
        acc = base.clone().to(DEV)
        ops.gemm_ring_bf16(a.to(DEV), w.to(DEV), acc, accumulate=True, waves=waves, kc=kc)
        assert rel_err(acc, want + base.double()) < 3e-6
    else:
        parts = torch.full((S, M, N), float("nan"), device=DEV)
        ops.gemm_ring_bf16(a.to(DEV), w.to(DEV), parts, S, waves=waves, kc=kc)
        assert torch.isfinite(parts).all()
        assert rel_err(parts.sum(0), want) < 3e-6
    # a row's result does not depend on the other rows of the batch, nor on how many there are
    full = torch.empty(M, N, device=DEV)
    ops.gemm_ring_bf16(a.to(DEV), w.to(DEV), full, waves=waves, kc=kc)
    few = torch.empty(min(M, 3), N, device=DEV)
    ops.gemm_ring_bf16(a[:min(M, 3)].contiguous().to(DEV), w.to(DEV), few, waves=waves, kc=kc)
    assert torch.equal(few, full[:min(M, 3)])


@pytest.mark.parametrize("waves,kc", [(4, 128), (8, 128), (8, 64)])
@pytest.mark.parametrize("M,I,K", [(64, 128, 512), (40, 192, 256), (128, 64, 384), (20, 160, 128)])
def test_gemm_ring_paired_silu(ops, waves, kc, M, I, K):
    from torchless_rs_amd.parts.linear import interleave_pairs
    a = rnd(M, K, seed=54, dtype=torch.bfloat16)
    g = rnd(I, K, seed=55, dtype=torch.bfloat16, scale=0.3)
    u = rnd(I, K, seed=56, dtype=torch.bfloat16, scale=0.3)
    out = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.gemm_ring_bf16(a.to(DEV), interleave_pairs(g, u).to(DEV), out, silu_pair=True, waves=waves, kc=kc)
    want = plain.silu(a.double() @ g.double().t()) * (a.double() @ u.double().t())
    assert rel_err(out, want) < KTOL["bfloat16"]
    with pytest.raises(ops.KernelError, match="groups of four waves"):
        ops.gemm_ring_bf16(a.to(DEV), interleave_pairs(g, u).to(DEV), out, silu_pair=True, waves=7)


def test_gemm_ring_refuses_what_it_does_not_serve(ops):
    a = torch.zeros(20, 200, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(64, 200, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ops.KernelError, match="multiple of 128"):
        ops.gemm_ring_bf16(a, w, torch.empty(20, 64, device=DEV))
    a, w = torch.zeros(20, 256, dtype=torch.bfloat16, device=DEV), torch.zeros(64, 256, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ops.KernelError, match="waves"):
        ops.gemm_ring_bf16(a, w, torch.empty(20, 64, device=DEV), waves=5)
    with pytest.raises(ops.KernelError, match="splits do not fit"):
        ops.gemm_ring_bf16(a, w, torch.empty(3, 20, 64, device=DEV), n_split=3)
    big = torch.zeros(129, 256, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ops.KernelError, match="M at most"):
        ops.gemm_ring_bf16(big, w, torch.empty(129, 64, device=DEV))


def test_rope_commit_adds_partial_products(ops):
    from torchless_rs_amd.parts.position import Rotary
    nq, nkv, d = 6, 2, 48
    a = paged_case(ops, "bfloat16", nq, nkv, d, None, lens_cached=[0, 63, 64, 300], lens_new=[1] * 4, seed=7)
    qkv = rnd(3, 4, (nq + 2 * nkv) * d, seed=8).to(DEV)
    inv = Rotary(d, 777.0).inv_freq(DEV)
    q1, q2 = (torch.empty(4, nq, d, dtype=torch.bfloat16, device=DEV) for _ in range(2))
    p1, p2 = a["pages"].clone(), a["pages"].clone()
    ops.rope_commit((qkv[0] + qkv[1] + qkv[2]).contiguous(), a["row_pos"], inv, a["table"], a["ring"], nq, nkv, d, q1, p1)
    ops.rope_commit(qkv, a["row_pos"], inv, a["table"], a["ring"], nq, nkv, d, q2, p2)
    assert torch.equal(q1, q2)
    assert torch.equal(torch.nan_to_num(p1.float(), nan=-7.0), torch.nan_to_num(p2.float(), nan=-7.0))


def test_ceilings_are_measured(ops):
    """The plain read (in every shape), the copy and the MFMA chain that bench.py quotes: on an MI355X the
    best read reaches at least 5 of the published 8 TB/s and the chain 1.8 of 2.5 PFLOP/s, and neither
    exceeds the published peak; a figure outside means that the measurement is broken, not the machine."""
    c = ops.measure_ceilings(DEV, gib=2.0)
    assert 5000.0 <= c["hbm_read_GBs"] <= 8000.0, c
    assert c["hbm_read_shape"] in ops.READ_SHAPES.values() and len(c["hbm_read_by_shape_GBs"]) == len(ops.READ_SHAPES)
    assert all(1000.0 < v <= 8000.0 for v in c["hbm_read_by_shape_GBs"].values()), c
    assert 3000.0 <= c["hbm_copy_GBs"] <= 8000.0, c
    assert 1800.0 <= c["mfma_bf16_TFLOPs"] <= 2500.0, c


@pytest.mark.parametrize("window", [None, 4096])
def test_attention_over_a_long_context(ops, window):
    """70,000 cached positions in scattered pages: the new token's query (decode kernel) and a
    chunk of 130 new rows (prefill kernel) against the softmax written out for those rows only.
    One far key is made to stand out, so that a page taken from the wrong place would show."""
    nq, nkv, d, L, n_new = 2, 1, 16, 70000, 130
    PAGE = 64
    ring = -(-window // PAGE) if window else 1 << 24
    T = L + n_new
    g = torch.Generator().manual_seed(3)
    q = torch.randn(T, nq, d, generator=g).to(torch.bfloat16)
    k = torch.randn(T, nkv, d, generator=g).to(torch.bfloat16)
    v = torch.randn(T, nkv, d, generator=g).to(torch.bfloat16)
    far = L - 3000
    q0 = q[L, 0].float()
    k[far] = (q0 * (24.0 * math.sqrt(d) / float(q0 @ q0))).to(torch.bfloat16)   # score 24: row L's head 0 looks at `far`
    held = min(-(-T // PAGE), ring)
    perm = torch.randperm(held + 5, generator=g)
    table = perm[:held].to(torch.int32).view(1, held)

    def fill(upto):
        pages = torch.full((held + 5, 2, nkv, PAGE, d), float("nan"), dtype=torch.bfloat16)
        for p0 in range(max(0, (upto - ring * PAGE) // PAGE * PAGE) if window else 0, upto, PAGE):
            pg = int(table[0, (p0 // PAGE) % ring])
            n = min(PAGE, upto - p0)
            pages[pg, 0, :, :n] = k[p0:p0 + n].transpose(0, 1)
            pages[pg, 1].view(nkv, d, PAGE)[:, :, :n] = v[p0:p0 + n].permute(1, 2, 0)
        return pages

    def want(rows):
        out = torch.empty(len(rows), nq, d, dtype=torch.float64)
        for i, p in enumerate(rows):
            lo = max(0, p - window + 1) if window else 0
            for h in range(nq):
                s = (k[lo:p + 1, 0].double() @ q[p, h].double()) / math.sqrt(d)
                out[i, h] = torch.softmax(s, 0) @ v[lo:p + 1, 0].double()
        return out

    i32 = lambda l: torch.tensor(l, dtype=torch.int32, device=DEV)
    # decode: position L, everything in the pages (the new key committed)
    pages = fill(L + 1).to(DEV)
    out = torch.empty(1, nq, d, dtype=torch.bfloat16, device=DEV)
    for splits in (1, 7, 64):
        part = torch.empty(nq * splits * (d + 2), device=DEV)
        ops.attn_decode_bf16(q[L:L + 1].to(DEV), pages, table.to(DEV), ring, i32([L]), window, 1 / math.sqrt(d),
                             splits, part, out)
        assert rel_err(out, want([L])) < KTOL["bfloat16"], splits
    assert rel_err(out[0, 0], v[far, 0].double()) < 0.05                # head 0 returns the far value
    # prefill: rows L .. L + 129 over the cache of L positions
    pages = fill(L).to(DEV)
    off, cols = ops.aligned_columns([L], [n_new])
    vt = torch.zeros(nkv, d, cols, dtype=torch.bfloat16)
    vt[:, :, L % PAGE:L % PAGE + n_new] = v[L:].permute(1, 2, 0)
    outp = torch.empty(n_new, nq, d, dtype=torch.bfloat16, device=DEV)
    ops.attn_prefill_bf16(q[L:].contiguous().to(DEV), k[L:].contiguous().to(DEV), vt.to(DEV), i32(off), pages,
                          table.to(DEV), ring, i32(list(range(L, T))), i32([0, n_new]), i32([L]), -(-n_new // 128),
                          window, 1 / math.sqrt(d), outp)
    rows = [L, L + 1, L + 63, L + 64, L + 129]
    assert rel_err(outp[[r - L for r in rows]], want(rows)) < KTOL["bfloat16"]
    # and all 70,130 rows in one step, nothing cached
    off, cols = ops.aligned_columns([0], [T])
    vt = torch.zeros(nkv, d, cols, dtype=torch.bfloat16)
    vt[:, :, :T] = v.permute(1, 2, 0)
    outp = torch.empty(T, nq, d, dtype=torch.bfloat16, device=DEV)
    ops.attn_prefill_bf16(q.to(DEV), k.to(DEV), vt.to(DEV), i32(off), pages, table.to(DEV), ring,
                          i32(list(range(T))), i32([0, T]), i32([0]), -(-T // 128), window, 1 / math.sqrt(d), outp)
    rows = [0, 63, 64, 4095, 4096, 4097, 40000, L, T - 1]
    assert rel_err(outp[rows], want(rows)) < KTOL["bfloat16"]
    assert torch.isfinite(outp.float()).all()


# ---- other rotations than the reference's: a share of the head, interleaved pairs, none ----------

ROTATIONS = [(1.0, False), (1.0, True), (0.5, False), (0.5, True), (0.25, True), (0.0, False)]


def rotation_for(ops, d, theta, share, interleaved):
    r = int(d * share) // 2 * 2
    if r == 0:
        return ops.NO_ROTATION, 0
    inv = plain.rope_inv_freq(r, theta).to(torch.float32).to(DEV)
    return ops.Rotation(inv, r, interleaved), r


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("share,interleaved", ROTATIONS)
@pytest.mark.parametrize("nq,nkv,d", [(3, 1, 48), (4, 2, 128), (2, 2, 16)])
def test_rope_split_and_commit_take_any_rotation(ops, dt, share, interleaved, nq, nkv, d):
    """`rope_split` against the plain rotation of the same family, and `rope_commit` bit for bit
    what `rope_split` and `kv_commit` give."""
    theta, lens = 500.0, [0, 63, 300, 5]
    rot, r = rotation_for(ops, d, theta, share, interleaved)
    a = paged_case(ops, dt, nq, nkv, d, None, lens_cached=lens, lens_new=[1] * len(lens), seed=31)
    n = len(lens)
    qkv = rnd(n, (nq + 2 * nkv) * d, seed=32).to(DEV)
    q1, k1, v1 = (torch.empty(n, h, d, dtype=DT[dt], device=DEV) for h in (nq, nkv, nkv))
    ops.rope_split(qkv, a["row_pos"], rot, nq, nkv, d, q1, k1, v1)
    x = qkv.double().cpu().view(n, nq + 2 * nkv, d)
    pos = a["row_pos"].cpu().long()
    wq = plain.rope_variant(x[:, :nq], pos, theta, r, interleaved)
    wk = plain.rope_variant(x[:, nq:nq + nkv], pos, theta, r, interleaved)
    for row, p in enumerate(pos.tolist()):              # float32 angles: off by up to 1.2e-7 * p radians
        tol = KTOL[dt] + 1.2e-7 * p
        assert rel_err(q1[row], wq[row]) < tol and rel_err(k1[row], wk[row]) < tol, (row, p)
    assert torch.equal(v1.cpu(), x[:, nq + nkv:].to(DT[dt]))
    if r < d:                                        # what is not rotated is copied, not computed
        assert torch.equal(q1[..., r:].cpu(), x[:, :nq, r:].to(DT[dt]))
    pages1 = a["pages"].clone()
    ops.kv_commit(k1, v1, a["row_seq"], a["row_pos"], a["after"], a["table"], a["ring"], pages1)
    q2, pages2 = torch.full_like(q1, float("nan")), a["pages"].clone()
    ops.rope_commit(qkv, a["row_pos"], rot, a["table"], a["ring"], nq, nkv, d, q2, pages2)
    assert torch.equal(q1, q2)
    assert torch.equal(torch.nan_to_num(pages1.float(), nan=-7.0), torch.nan_to_num(pages2.float(), nan=-7.0))


@pytest.mark.parametrize("share,interleaved", ROTATIONS[1:])
@pytest.mark.parametrize("nq,nkv,d,K,lens", [(6, 2, 48, 64, [0, 63, 64, 300]), (8, 2, 128, 1024, [9, 64, 640, 2, 3, 70, 71]),
                                             (2, 1, 16, 72, [5, 6])])
def test_qkv_rope_commit_takes_any_rotation(ops, share, interleaved, nq, nkv, d, K, lens):
    """The fused kernel of single-token steps, from the weights as stored and from the tiled copy in
    the order of this rotation's pairs: the bits of the product followed by `rope_commit`."""
    rot, r = rotation_for(ops, d, 10000.0, share, interleaved)
    n = len(lens)
    c = paged_case(ops, "bfloat16", nq, nkv, d, None, lens_cached=lens, lens_new=[1] * n, seed=33, n_pages=60)
    y = rnd(n, K, seed=34, dtype=torch.bfloat16).to(DEV)
    w = rnd((nq + 2 * nkv) * d, K, seed=35, dtype=torch.bfloat16, scale=0.2).to(DEV)
    qkv = torch.empty(n, (nq + 2 * nkv) * d, device=DEV)
    ops.gemm(y, w, qkv)
    q1 = torch.empty(n, nq, d, dtype=torch.bfloat16, device=DEV)
    pages1 = c["pages"].clone()
    ops.rope_commit(qkv, c["row_pos"], rot, c["table"], c["ring"], nq, nkv, d, q1, pages1)
    rows = ops.qkv_tile_rows(nq, nkv, d, DEV, rot)
    assert sorted(rows.tolist()) == list(range((nq + 2 * nkv) * d))
    if interleaved:
        assert rows[:16].tolist() == list(range(0, 16, 2)) + list(range(1, 16, 2))
    tiles = ops.tile_weights(w, rows) if K % 64 == 0 else None
    for t in (None, tiles):
        for units in (1, 2, 3, 4):
            q2, pages2 = torch.full_like(q1, float("nan")), c["pages"].clone()
            ops.qkv_rope_commit(y, w, c["row_pos"], rot, c["table"], c["ring"], nq, nkv, d, q2, pages2,
                                units=units, tiles=t)
            assert torch.equal(q1, q2), (t is not None, units)
            assert torch.equal(torch.nan_to_num(pages1.float(), nan=-7.0), torch.nan_to_num(pages2.float(), nan=-7.0))
    full = (y.double().cpu() @ w.double().cpu().t()).view(n, nq + 2 * nkv, d)
    assert rel_err(q1, plain.rope_variant(full[:, :nq], c["row_pos"].cpu().long(), 10000.0, r, interleaved)) < KTOL["bfloat16"]


def test_rotations_that_cannot_be_are_refused(ops):
    qkv = torch.zeros(2, 4 * 16, device=DEV)
    pos = torch.zeros(2, dtype=torch.int32, device=DEV)
    q, k, v = (torch.empty(2, h, 16, device=DEV) for h in (2, 1, 1))
    inv = torch.ones(9, device=DEV)
    with pytest.raises(ops.KernelError, match="rotated channels"):
        ops.rope_split(qkv, pos, ops.Rotation(inv, 18), 2, 1, 16, q, k, v)           # more than the head
    with pytest.raises(ops.KernelError, match="rotated channels"):
        ops.rope_split(qkv, pos, ops.Rotation(inv[:3].contiguous(), 7), 2, 1, 16, q, k, v)    # odd
    with pytest.raises(ops.KernelError, match="inv_freq"):
        ops.rope_split(qkv, pos, ops.Rotation(inv, 8), 2, 1, 16, q, k, v)            # 9 frequencies for 4 pairs
