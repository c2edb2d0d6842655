"""Configurations that a Mistral config.json may legally hold and that take another route through
the product than the usual ones: even head sizes that are no multiple of 16 (in bfloat16 the
attention, the rotation with its commit and the q|k|v product then leave the matrix-core kernels
for the plain ones), heads x head size that is no multiple of 8 (the output projection leaves them
too), `tie_word_embeddings: true`, a float16 checkpoint, a width of 5,120.  Each under all three schedules (every
request alone and whole; the last 32 tokens one by one; batches of unequal lengths whose shorter
requests end earlier, a second batch in the same slots), in float32 and bfloat16, against the plain
implementation.  And the default stop ids: config.json's `eos_token_id` ends a sequence through the
library call and the command line unless the caller names other ids or none
(src/sampler/mod.rs:285-299 of the reference is the loop's behaviour)."""
import json
import os
import subprocess

import pytest
import torch

import plain_mistral as plain
from util import TOL, prompts, read_model_dir, rel_err, within_the_format

pytestmark = pytest.mark.gpu
REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

#         name              d   nq nkv  H    I    V   L  window  tie    stored
CASES = [("head6", 6, 4, 2, 40, 96, 130, 2, 7, False, torch.bfloat16),
         ("head6_o18", 6, 3, 3, 48, 64, 257, 2, None, False, torch.bfloat16),     # o reads 18 columns: no multiple of 8
         ("head40", 40, 6, 3, 72, 160, 257, 3, 70, False, torch.bfloat16),
         ("head72", 72, 2, 1, 136, 224, 384, 2, None, False, torch.bfloat16),
         ("head120", 120, 4, 2, 200, 352, 300, 2, 150, False, torch.bfloat16),
         ("tied_head32", 32, 4, 2, 96, 160, 300, 2, 40, True, torch.bfloat16),
         ("tied_head40", 40, 2, 2, 80, 96, 130, 2, None, True, torch.bfloat16),
         ("float16_head64", 64, 4, 1, 128, 192, 384, 2, 100, False, torch.float16),
         ("float16_tied_head6", 6, 4, 4, 40, 64, 130, 1, 7, True, torch.float16),
         # more tiles of 16 channels than the device has compute units: o and down in shares of 20 channels
         # from tiled copies with tiles of 20 rows
         ("wide5120", 64, 8, 2, 5120, 192, 300, 2, 100, False, torch.bfloat16)]
LENS = [70, 9, 33, 1]


def _schedules(eng, ids):
    """The three schedules; for each the logits of every position of every request and, for the
    plain implementation that rounds where the engine does, the number of rows of the step that each
    position came in."""
    from torchless_rs_amd.engine import SeqInput
    out = {}
    # each request alone and whole
    got = []
    for p in ids:
        s = eng.alloc()
        got.append(eng.step([SeqInput(s, p, list(range(len(p))))]).clone())
        eng.free(s)
    out["whole"] = (got, [[len(p)] * len(p) for p in ids])
    # the last 32 tokens one by one
    got, rows = [], []
    for p in ids:
        k = min(32, len(p) - 1)
        s = eng.alloc()
        parts = [eng.step([SeqInput(s, p[:len(p) - k], list(range(len(p) - k)))]).clone()]
        parts += [eng.step([SeqInput(s, [t], [0])]).clone() for t in p[len(p) - k:]]
        eng.free(s)
        got.append(torch.cat(parts))
        rows.append([len(p) - k] * (len(p) - k) + [1] * k)
    out["last32"] = (got, rows)
    # batches of unequal lengths, the shorter requests ending earlier; twice, the second time in the slots
    # and pages that the first gave back, with the requests in the other order
    for name, order in (("batch", list(range(len(ids)))), ("again", list(range(len(ids)))[::-1])):
        reqs = [ids[i] for i in order]
        heads = [max(1, len(p) // 2) for p in reqs]
        tails = [len(p) - h for p, h in zip(reqs, heads)]
        slots = [eng.alloc() for _ in reqs]
        lg = eng.step([SeqInput(s, p[:h], list(range(h))) for s, p, h in zip(slots, reqs, heads)]).clone()
        parts, o = [[] for _ in reqs], 0
        for i, h in enumerate(heads):
            parts[i].append(lg[o:o + h])
            o += h
        for i, tl in enumerate(tails):
            if tl == 0:
                eng.free(slots[i])
        for t in range(max(tails)):
            live = [i for i in range(len(reqs)) if t < tails[i]]
            lg = eng.step([SeqInput(slots[i], [reqs[i][heads[i] + t]], [0]) for i in live]).clone()
            for r, i in enumerate(live):
                parts[i].append(lg[r:r + 1])
                if t + 1 == tails[i]:
                    eng.free(slots[i])
        rows = [[sum(heads)] * h + [sum(1 for t2 in tails if t < t2) for t in range(tl)] for h, tl in zip(heads, tails)]
        back = {i: k for k, i in enumerate(order)}
        out[name] = ([torch.cat(parts[back[i]]) for i in range(len(ids))], [rows[back[i]] for i in range(len(ids))])
        eng.cache.check()
        assert not eng.cache.length
    return out


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_legal_configurations_under_every_schedule(tmp_path, case):
    from torchless_rs_amd import write_random_model
    from torchless_rs_amd.engine import Engine, load_model
    name, d, nq, nkv, H, I, V, L, window, tie, stored = case
    cfg = {"architectures": ["MistralForCausalLM"], "model_type": "mistral", "num_hidden_layers": L,
           "hidden_size": H, "num_attention_heads": nq, "num_key_value_heads": nkv, "head_dim": d,
           "intermediate_size": I, "vocab_size": V, "rope_theta": 10000.0, "sliding_window": window,
           "rms_norm_eps": 1e-5, "max_position_embeddings": 256, "tie_word_embeddings": tie, "hidden_act": "silu"}
    # weights of a size that keeps a layer's gain near one at any width (0.06 up to 600 channels), as real ones are
    std = min(0.06, 1.5 / H ** 0.5)
    mdir = write_random_model(str(tmp_path / "m"), cfg, seed=len(name), std=std, norm_std=0.1, dtype=stored)
    cfgd, stored_w = read_model_dir(mdir)
    assert ("lm_head.weight" in stored_w) == (not tie)
    assert all(t.dtype == stored for t in stored_w.values())
    ids = prompts(V, LENS, seed=50 + len(name))
    for dtype in ("float32", "bfloat16"):
        # float32 widens what is stored; bfloat16 keeps bfloat16 and rounds a float16 checkpoint to it once, at load
        w = stored_w if dtype == "float32" else {k: t.to(torch.bfloat16) for k, t in stored_w.items()}
        exact = [plain.forward(w, cfgd, p) for p in ids]
        model = load_model(mdir, dtype)
        if dtype == "bfloat16":
            assert all(b.mixer.qkv.weight.dtype == torch.bfloat16 for b in model.blocks)
            assert (model.head.proj.weight.data_ptr() == model.embedding.table.data_ptr()) == tie
        eng = Engine(model, max_tokens=64 * 8, max_slots=len(ids))
        for g in eng.cache.groups:
            g.storage.fill_(float("nan"))
        runs = _schedules(eng, ids)
        eng.close()
        for sched, (got, rows) in runs.items():
            if dtype == "float32":
                worst = max(rel_err(g, x) for g, x in zip(got, exact))
                cost = max(rel_err(plain.forward(w, cfgd, p, dtype=torch.float32), x) for p, x in zip(ids, exact))
                assert worst < max(TOL[dtype], 2 * cost), (name, sched, worst, cost)
            else:
                halves = (nq * d) % 8 == 0 and I % 32 == 0 and H % 8 == 0
                rounded = [plain.forward_rounded(w, cfgd, p, r, ffn_norm_in_halves=halves) for p, r in zip(ids, rows)]
                ok, numbers = within_the_format(got, rounded, exact)
                assert ok, (name, sched, numbers)
                assert max(rel_err(g, x) for g, x in zip(got, exact)) < 2 * TOL[dtype], (name, sched)
        # the cuts agree with each other in float32 to the order of summation
        if dtype == "float32":
            for sched in ("last32", "batch", "again"):
                assert max(rel_err(a, b) for a, b in zip(runs[sched][0], runs["whole"][0])) < 1e-5, (name, sched)


# ---- default stop ids ----------------------------------------------------------------------------

def _folder_with_eos(tmp_path, eos):
    """Tiny model A with `eos_token_id` written into its config.json."""
    from util import make_model_dir
    d = make_model_dir(tmp_path, "A", torch.float32)
    with open(os.path.join(d, "config.json")) as f:
        cfg = json.load(f)
    cfg["eos_token_id"] = eos
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    return d


def test_eos_token_id_of_the_configuration_is_the_default_stop_id(tmp_path):
    """Greedy tokens of two prompts are found first with no stop id at all; then a token that the first
    prompt draws at its fourth step or later (and not before) becomes config.json's `eos_token_id`.
    Without `stop_ids` the library call and the command line stop there (the stop id is not part of
    the output, the other prompt goes on to its length); `stop_ids=[]` / `--stop-ids none` run to the
    length; `eos_token_id` as a list works likewise."""
    from torchless_rs_amd.api import generate
    d = _folder_with_eos(tmp_path, None)
    cfg, w = read_model_dir(d)
    ps = [[3, 1, 4, 1, 5], [9, 2, 6]]
    N = 12
    free = [plain.generate_greedy(w, cfg, p, N)[0] for p in ps]
    j = next(j for j in range(3, N) if free[0][j] not in free[0][:j])
    eos = free[0][j]
    want = [plain.generate_greedy(w, cfg, p, N, stop_ids=[eos])[0] for p in ps]
    assert want[0] == free[0][:j] and len(want[0]) < N
    none = generate(d, ps, max_tokens=N, temperature=0.0, dtype="float32")          # no eos in config.json
    assert [r.tokens for r in none] == free and all(r.finish_reason == "length" for r in none)
    for value in (eos, [255, eos]):
        d = _folder_with_eos(tmp_path, value)
        out = generate(d, ps, max_tokens=N, temperature=0.0, dtype="float32")
        assert [r.tokens for r in out] == want
        assert out[0].finish_reason == "stop" and out[0].stopped_at_eos
        assert out[1].finish_reason == ("stop" if len(want[1]) < N else "length")
        out = generate(d, ps, max_tokens=N, temperature=0.0, dtype="float32", stop_ids=[])
        assert [r.tokens for r in out] == free
        other = free[0][1]
        out = generate(d, ps, max_tokens=N, temperature=0.0, dtype="float32", stop_ids=[other])
        assert out[0].tokens == free[0][:free[0].index(other)]                      # the caller's ids replace the default
    exe = os.path.join(REPO, "bin", "torchless")
    common = ["--temperature", "0", "--dtype", "float32", "--max-tokens", str(N)]
    text = "3 1 4 1 5; 9 2 6"
    r = subprocess.run([exe, *common, d, text], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [[int(t) for t in l.split()] for l in r.stdout.rstrip("\n").split("\n")] == want
    assert "finish: stop" in r.stderr
    r = subprocess.run([exe, *common, "--stop-ids", "none", d, text], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [[int(t) for t in l.split()] for l in r.stdout.rstrip("\n").split("\n")] == free
    assert "finish: length, length" in r.stderr
