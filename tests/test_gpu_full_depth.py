"""The Mistral-7B-v0.1 shape at its full depth of 32 layers, random weights N(0, 0.02): the float32
path against the plain implementation, and bfloat16 against what the format costs, for two short
unequal prompts under every way of cutting the work: each alone and whole; as a batch with the last
tokens one by one, the shorter request ending earlier; and a second batch in the same slots.

The plain implementation is the one the other tests run on the CPU.  Here its tensors lie on the
GPU (float64, a layer at a time), which changes no formula and saves minutes."""
import pytest
import torch

import plain_mistral as plain
from util import TOL, prompts, rel_err, within_the_format

pytestmark = [pytest.mark.gpu, pytest.mark.slow]

SHAPE = dict(architectures=["MistralForCausalLM"], num_hidden_layers=32, hidden_size=4096,
             num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=14336,
             vocab_size=32000, rope_theta=10000.0, sliding_window=4096, rms_norm_eps=1e-5)
LENS, TAILS = [41, 24], [9, 5]


def schedule(eng, ids, tails):
    """One batch: the heads in one step with every row wanted, then one token a step until the
    longest tail is fed.  Returns the logits of every position of every request, and the slots."""
    from torchless_rs_amd.engine import SeqInput
    slots = [eng.alloc() for _ in ids]
    heads = [len(p) - t for p, t in zip(ids, tails)]
    outs = [[] for _ in ids]
    lg = eng.step([SeqInput(s, p[:h], list(range(h))) for s, p, h in zip(slots, ids, heads)]).clone()
    o = 0
    for i, h in enumerate(heads):
        outs[i].append(lg[o:o + h])
        o += h
    for t in range(max(tails)):
        live = [i for i in range(len(ids)) if t < tails[i]]
        lg = eng.step([SeqInput(slots[i], [ids[i][heads[i] + t]], [0]) for i in live]).clone()
        for r, i in enumerate(live):
            outs[i].append(lg[r:r + 1])
        for i in live:
            if t + 1 == tails[i]:
                eng.free(slots[i])                       # the shorter request ends earlier
    for i, tl in enumerate(tails):
        if tl == 0:
            eng.free(slots[i])
    return [torch.cat(o) for o in outs], slots


def test_7b_shape_at_full_depth():
    from torchless_rs_amd import config_from_dict
    from torchless_rs_amd.engine import Engine, model_from_tensors
    from torchless_rs_amd.models import model_spec_for
    from torchless_rs_amd.weights import random_tensors
    cfg = config_from_dict(SHAPE)
    tensors = random_tensors(model_spec_for(cfg).weight_specs(), seed=5, std=0.02, dtype=torch.bfloat16,
                             device="cuda:0")
    ids = prompts(SHAPE["vocab_size"], LENS, seed=21)
    others = prompts(SHAPE["vocab_size"], LENS[::-1], seed=22)          # the second batch: other requests
    exact = plain.forward_many(tensors, SHAPE, ids + others)
    cost32 = max(rel_err(a, b) for a, b in zip(plain.forward_many(tensors, SHAPE, ids + others, dtype=torch.float32), exact))
    got = {}
    for dtype in ("float32", "bfloat16"):
        eng = Engine(model_from_tensors(cfg, tensors, dtype, "cuda:0"), max_tokens=64 * 4, max_slots=2)
        for g in eng.cache.groups:
            g.storage.fill_(float("nan"))                # what no step wrote must never be read
        runs = {}
        runs["whole"] = [schedule(eng, [p], [0])[0][0] for p in ids]
        runs["batch"], first_slots = schedule(eng, ids, TAILS)
        runs["again"], second_slots = schedule(eng, others, TAILS[::-1])
        assert sorted(first_slots) == sorted(second_slots) and not eng.cache.length    # the same slots, all given back
        got[dtype] = runs
        eng.close()
        del eng
    # float32: every cut against the plain float64 logits, and bit for bit alike among themselves
    allowed = max(TOL["float32"], 2 * cost32)
    f = got["float32"]
    worst32 = max(rel_err(g, x) for g, x in zip(f["whole"] + f["batch"] + f["again"], exact[:2] + exact[:2] + exact[2:]))
    print(f"\\n7B shape, 32 layers: float32 {worst32:.2e} of the largest logit (the plain implementation in float32: {cost32:.2e})")
    assert worst32 < allowed
    assert max(rel_err(a, b) for a, b in zip(f["whole"], f["batch"])) < 1e-6
    # bfloat16: against what the format costs the plain implementation with the same roundings
    b = got["bfloat16"]
    heads = [n - t for n, t in zip(LENS, TAILS)]
    rows_whole = [[n] * n for n in LENS]
    rows_batch = [[sum(heads)] * h + [sum(1 for t2 in TAILS if t < t2) for t in range(tl)] for h, tl in zip(heads, TAILS)]
    rows_again = rows_batch[::-1]                  # the second batch: lengths and tails in the other order
    for name, rows, want, reqs in (("whole", rows_whole, exact[:2], ids), ("batch", rows_batch, exact[:2], ids),
                                   ("again", rows_again, exact[2:], others)):
        rounded = [plain.forward_rounded(tensors, SHAPE, p, r) for p, r in zip(reqs, rows)]
        ok, numbers = within_the_format(b[name], rounded, want)
        print(f"   bfloat16 {name}: " + ", ".join(f"{k} {v:.2e}" for k, v in numbers.items()))
        assert ok, (name, numbers)
    # (the second batch, in the slots and pages that the first gave back, is held to the plain rounded
    # implementation of its own requests like the others: a stale row worth the format's cost would show)
