"""The layout of a step's batch (no GPU): the host library's packer against the rules written out here."""
import numpy as np
import pytest
import torch

from torchless_rs_amd.cache import PAGE, Cache, CacheFull, KVRequest
from torchless_rs_amd.engine.engine import SeqInput, StepError, pack_step


def make(window=None, two_groups=True, max_tokens=64 * 12, slots=4):
    kv = {0: KVRequest(2, 16, window)}
    if two_groups:
        kv[1] = KVRequest(1, 32, None)
    return Cache(kv, {}, max_tokens, torch.float32, "cpu", slots, allocate=False)


def pieces(p):
    off = np.concatenate([[0], np.cumsum(p.sizes)])
    return [p.flat[off[i]:off[i + 1]] for i in range(len(p.sizes))]


def test_layout_of_a_prompt_step_and_of_a_decode_step():
    c = make(window=100)
    a, b, d = c.alloc_slot(), c.alloc_slot(), c.alloc_slot()
    batch = [SeqInput(a, [5, 6, 7], [0, 2]), SeqInput(b, list(range(70)), []), SeqInput(d, [9], [0])]
    p = pack_step(c, batch, vocab_size=100)
    tok, pos, seq, cu, slots, before, after, want, off, t0, t1 = pieces(p)
    assert tok.tolist() == [5, 6, 7] + list(range(70)) + [9]
    assert pos.tolist() == [0, 1, 2] + list(range(70)) + [0]
    assert seq.tolist() == [0] * 3 + [1] * 70 + [2]
    assert cu.tolist() == [0, 3, 73, 74] and slots.tolist() == [a, b, d]
    assert before.tolist() == [0, 0, 0] and after.tolist() == [3, 70, 1]
    assert want.tolist() == [0, 2, 73]                                  # rows of the packed batch
    assert off.tolist() == [0, 64, 192] and p.host["aligned_cols"] == 256
    assert (p.n_rows, p.n_seqs, p.n_want, p.all_single, p.max_new, p.max_len_after) == (74, 3, 3, False, 70, 70)
    assert p.strides == (2, 2)                                          # two pages for 70 positions
    for t, g in ((t0, c.groups[0]), (t1, c.groups[1])):
        t = t.reshape(3, 2)
        for row, s in enumerate((a, b, d)):
            pg = g.pages_of_slot[s]
            assert t[row, :len(pg)].tolist() == pg and not t[row, len(pg):].any()
    c.commit([(a, 3), (b, 70), (d, 1)])
    # one token each, the tokens on the device: their rows go last, the token section is empty
    q = pack_step(c, [SeqInput(b, [0], [0]), SeqInput(a, [0], [0])], 100, token_rows=[1, 0])
    parts = pieces(q)
    assert parts[0].tolist() == [0, 0] and parts[1].tolist() == [70, 3] and parts[-1].tolist() == [1, 0]
    assert q.all_single and q.strides == (2, 2) and parts[8].tolist() == [0, 64]
    c.commit([(b, 1), (a, 1)])
    c.check()


def test_table_width_is_a_power_of_two_within_the_ring():
    c = make(window=64 * 3, two_groups=True, max_tokens=64 * 40, slots=2)
    s = c.alloc_slot()
    widths = []
    for n in (1, 64, 64, 64, 64 * 2, 64 * 4):
        p = pack_step(c, [SeqInput(s, [1] * n, [])], 10)
        c.commit([(s, n)])
        widths.append(p.strides)
    # windowed group: 1, 2, 3 (the ring, not 4), 3...; full group: 1, 2, 4, 4, 8, 16
    assert widths == [(1, 1), (2, 2), (3, 4), (3, 4), (3, 8), (3, 16)]
    assert len(c.groups[0].pages_of_slot[s]) == 3 and len(c.groups[1].pages_of_slot[s]) == 10


def test_a_sum_of_columns_that_is_a_multiple_of_512_is_padded():
    c = make(two_groups=False, max_tokens=64 * 40)
    s, t = c.alloc_slot(), c.alloc_slot()
    p = pack_step(c, [SeqInput(s, [1] * 500, []), SeqInput(t, [1] * 3, [])], 10)
    assert pieces(p)[8].tolist() == [0, 512] and p.host["aligned_cols"] == 576
    c.commit([(s, 500), (t, 3)])
    p = pack_step(c, [SeqInput(s, [1] * 12, []), SeqInput(t, [1] * 3, [])], 10)       # 500 = 7 * 64 + 52 cached
    assert pieces(p)[8].tolist() == [0, 64] and p.host["aligned_cols"] == 128


def test_errors_leave_the_books_alone():
    c = make(two_groups=False, max_tokens=64 * 2, slots=3)
    s, t = c.alloc_slot(), c.alloc_slot()
    for bad, msg in (([], "at least one sequence"), ([SeqInput(9, [1], [])], "not held"),
                     ([SeqInput(s, [], [])], "at least one token"), ([SeqInput(s, [1, 50], [])], "vocabulary"),
                     ([SeqInput(s, [-1], [])], "vocabulary"), ([SeqInput(s, [1, 2], [2])], "wanted index"),
                     ([SeqInput(s, [1, 2], [0])] * 1 + [SeqInput(s, [3], [])], "twice")):
        with pytest.raises((StepError, Exception), match=msg):
            pack_step(c, bad, vocab_size=50)
    with pytest.raises(StepError, match="one token per entry"):
        pack_step(c, [SeqInput(s, [1, 2], [])], 50, token_rows=[0])
    with pytest.raises(CacheFull, match="more pages"):
        pack_step(c, [SeqInput(s, [1] * 65, []), SeqInput(t, [1] * 65, [])], 50)
    assert c.groups[0].pages_of_slot[s] == [] and c.groups[0].pool.n_free == 2        # all or nothing
    c.check()
    assert PAGE == 64
