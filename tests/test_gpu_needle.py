"""Weights made so that a fault of the cache shows in bfloat16 too.

With random weights a key among hundreds carries a few thousandths of an attention's output: a
page, a slot or a window's edge that is off by one would stay below bfloat16's tolerance.  Here a
one-layer model is built (from the framework's own parts, no position encoding) whose last token
asks for exactly one earlier token: the query token's q and the needle token's k point the same
way with a score of 32, every other score is 0.  The logits at the last position then follow the
value of the needle, if and only if the engine finds it: at a page's first and last row, far back,
on both sides of the window's edge, from the cache (the query as a single-token step), beside
another sequence with another needle, and in a slot that held another sequence before."""
import math

import pytest
import torch

import plain_mistral as plain
from util import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
H, D, I, V, EPS = 64, 64, 96, 32, 1e-5
QUERY, NEEDLES, FIRST_FILLER = 0, (1, 2), 3


def build(window):
    """Tensors and the specification.  Token 0 asks, tokens 1 and 2 answer (with different values),
    the others are orthogonal to both directions and score exactly 0."""
    from torchless_rs_amd.parts import LayerSpec, ModelSpec, PartSpec, Run
    g = torch.Generator().manual_seed(40)
    basis = torch.linalg.qr(torch.randn(H, H, generator=g, dtype=torch.float64))[0]
    u_ask, u_answer = basis[0], basis[1]
    emb = torch.zeros(V, H, dtype=torch.float64)
    emb[QUERY] = u_ask
    for n, t in enumerate(NEEDLES):
        emb[t] = u_answer + basis[2 + n]                    # the same key, another value
    coeff = torch.randn(V - FIRST_FILLER, H - 4, generator=g, dtype=torch.float64)
    emb[FIRST_FILLER:] = coeff @ basis[4:] / math.sqrt(H - 4)
    e1 = torch.zeros(D, dtype=torch.float64)
    e1[0] = 1.0
    c = 2.0                                                 # score = c^2 * H / sqrt(D) / (1 + ...) ~ 32 against 0
    w = {"model.embed_tokens.weight": emb,
         "model.layers.0.input_layernorm.weight": torch.ones(H, dtype=torch.float64),
         "model.layers.0.self_attn.q_proj.weight": c * torch.outer(e1, u_ask),
         "model.layers.0.self_attn.k_proj.weight": c * torch.outer(e1, u_answer) * math.sqrt(2.0),
         "model.layers.0.self_attn.v_proj.weight": torch.randn(D, H, generator=g, dtype=torch.float64) * 0.3,
         "model.layers.0.self_attn.o_proj.weight": torch.randn(H, D, generator=g, dtype=torch.float64) * 0.3,
         "model.layers.0.post_attention_layernorm.weight": torch.ones(H, dtype=torch.float64),
         "model.layers.0.mlp.gate_proj.weight": torch.randn(I, H, generator=g, dtype=torch.float64) * 0.2,
         "model.layers.0.mlp.up_proj.weight": torch.randn(I, H, generator=g, dtype=torch.float64) * 0.2,
         "model.layers.0.mlp.down_proj.weight": torch.randn(H, I, generator=g, dtype=torch.float64) * 0.2,
         "model.norm.weight": torch.ones(H, dtype=torch.float64),
         "lm_head.weight": torch.randn(V, H, generator=g, dtype=torch.float64) * 0.3}
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    norm = PartSpec("rmsnorm", {"size": H, "eps": EPS})
    layer = LayerSpec(prefix="model.layers.0.",
                      mixer=PartSpec("attention", {"hidden_size": H, "n_heads": 1, "n_kv_heads": 1, "head_dim": D,
                                                   "window": window, "position": PartSpec("none", {})}),
                      ffn=PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I}), mixer_norm=norm, ffn_norm=norm)
    spec = ModelSpec(hidden_size=H, vocab_size=V, embedding=PartSpec("tokens", {"vocab_size": V, "hidden_size": H}),
                     embedding_prefix="model.", layers=[layer], schedule=[Run(0)], final_norm=norm,
                     final_norm_prefix="model.norm.", head=PartSpec("linear", {"vocab_size": V, "hidden_size": H}),
                     head_prefix="lm_head.")
    return spec, w


def plain_last_logits(w, ids, window):
    """The plain model's logits at the last position (one layer, one head, no rotation)."""
    wd = {k: v.double() for k, v in w.items()}
    T, p = len(ids), "model.layers.0."
    pos = torch.arange(T)
    x = wd["model.embed_tokens.weight"][ids]
    y = plain.rmsnorm(x, wd[p + "input_layernorm.weight"], EPS)
    q, k, v = (plain.linear(y, wd[p + f"self_attn.{n}_proj.weight"]).view(T, 1, D) for n in "qkv")
    a = plain.attention_core(q, k, v, pos, window).reshape(T, D)
    x = x + plain.linear(a, wd[p + "self_attn.o_proj.weight"])
    x = x + plain.swiglu(plain.rmsnorm(x, wd[p + "post_attention_layernorm.weight"], EPS), wd, p)
    return plain.linear(plain.rmsnorm(x, wd["model.norm.weight"], EPS), wd["lm_head.weight"])[-1]


def sequence(T, needle_at, needle, seed):
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(FIRST_FILLER, V, (T,), generator=g).tolist()
    if needle_at is not None:
        ids[needle_at] = needle
    ids[-1] = QUERY
    return ids


@pytest.fixture(scope="module")
def engines():
    from torchless_rs_amd.engine import Engine
    from torchless_rs_amd.engine.model import Model
    from torchless_rs_amd.weights import TensorDict
    made = {}

    def get(window, dtype):
        if (window, dtype) not in made:
            spec, w = build(window)
            model = Model(spec, None, {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype], DEV)
            model.load_weights(TensorDict(w))
            made[(window, dtype)] = (Engine(model, max_tokens=64 * 40, max_slots=4), w)
        return made[(window, dtype)]

    yield get
    for eng, _ in made.values():
        eng.close()


TOL = {"float32": 1e-4, "bfloat16": 3e-2}


def last_logits(eng, ids, decode_last):
    """The engine's logits at the last position: the whole sequence in one step, or all but the
    query in one step and the query as a single-token step that reads everything from the cache."""
    from torchless_rs_amd.engine import SeqInput
    s = eng.alloc()
    if decode_last:
        eng.step([SeqInput(s, ids[:-1], [])])
        lg = eng.step([SeqInput(s, ids[-1:], [0])]).clone()
    else:
        lg = eng.step([SeqInput(s, ids, [len(ids) - 1])]).clone()
    eng.free(s)
    return lg[0]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("decode_last", [False, True])
@pytest.mark.parametrize("T,needle_at", [(130, 0), (130, 63), (130, 64), (130, 128), (300, 5), (700, 1), (700, 448), (700, 511), (700, 512)])
def test_a_needle_is_found_wherever_it_lies(engines, dtype, decode_last, T, needle_at):
    eng, w = engines(None, dtype)
    for g in eng.cache.groups:
        g.storage.fill_(float("nan"))
    ids = sequence(T, needle_at, NEEDLES[0], seed=T + needle_at)
    want = plain_last_logits(w, ids, None)
    without = plain_last_logits(w, sequence(T, None, None, seed=T + needle_at), None)
    other = plain_last_logits(w, sequence(T, needle_at, NEEDLES[1], seed=T + needle_at), None)
    assert rel_err(without, want) > 0.2 and rel_err(other, want) > 0.2          # the needle decides the logits
    assert rel_err(last_logits(eng, ids, decode_last), want) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("decode_last", [False, True])
@pytest.mark.parametrize("window", [70, 128, 200])
def test_the_window_edge_is_where_it_should_be(engines, dtype, decode_last, window):
    """The last key that the query still sees is window - 1 positions back; one further it is gone,
    and the logits are those of a sequence without a needle."""
    eng, w = engines(window, dtype)
    T = 400
    for inside in (True, False):
        at = (T - 1) - (window - 1) - (0 if inside else 1)
        ids = sequence(T, at, NEEDLES[0], seed=window)
        want = plain_last_logits(w, ids, window)
        without = plain_last_logits(w, sequence(T, None, None, seed=window), window)
        assert (rel_err(without, want) > 0.2) == inside
        assert rel_err(last_logits(eng, ids, decode_last), want) < TOL[dtype], (window, inside)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_each_sequence_finds_its_own_needle_and_a_used_slot_holds_no_old_one(engines, dtype):
    """Two sequences side by side with different needles at different places, token by token at the
    end; then, in the slots they gave back, sequences whose needles lie elsewhere (or nowhere): what
    the slots held before must not answer."""
    from torchless_rs_amd.engine import SeqInput
    eng, w = engines(None, dtype)
    first = [sequence(200, 70, NEEDLES[0], seed=1), sequence(131, 64, NEEDLES[1], seed=2)]
    second = [sequence(150, 3, NEEDLES[1], seed=3), sequence(131, None, None, seed=4)]     # the second has no needle at all
    used = []
    for batch in (first, second):
        slots = [eng.alloc() for _ in batch]
        used.append(sorted(slots))
        eng.step([SeqInput(s, ids[:-1], []) for s, ids in zip(slots, batch)])
        lg = eng.step([SeqInput(s, ids[-1:], [0]) for s, ids in zip(slots, batch)]).clone()
        for r, ids in enumerate(batch):
            assert rel_err(lg[r], plain_last_logits(w, ids, None)) < TOL[dtype], r
        for s in slots:
            eng.free(s)
    assert used[0] == used[1]
    # (what a stale needle would have given is far from what is wanted)
    stale = plain_last_logits(w, sequence(131, 64, NEEDLES[1], seed=4), None)
    assert rel_err(stale, plain_last_logits(w, second[1], None)) > 0.2
