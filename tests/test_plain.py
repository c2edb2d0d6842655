"""Pins of the plain implementation: vectors that the reference's own tests
hold, special cases that reduce to a library routine, and invariants, each
chosen so that a plausible mistake fails it."""
import math

import pytest
import torch

import plain_mistral as plain

D = torch.float64


def test_matvec_vectors():
    # src/kernels/tests.rs:5-10 and :106-113
    w = torch.tensor([[1., 2.], [3., 4.]], dtype=D)
    assert plain.linear(torch.tensor([1., 2.], dtype=D), w).tolist() == [5., 11.]
    m = torch.tensor([[1., 2.], [3., 4.], [5., 6.]], dtype=D)            # x @ M = M^T x
    assert plain.linear(torch.tensor([1., 2., 3.], dtype=D), m.t()).tolist() == [22., 28.]


def test_softmax_vectors():
    # src/kernels/tests.rs:13-24, :245-263
    p = plain.softmax(torch.tensor([1., 2., 3.], dtype=D))
    assert abs(float(p.sum()) - 1) < 1e-12 and p[0] < p[1] < p[2]
    big = plain.softmax(torch.tensor([1000., 1001., 1002., 999.], dtype=D))
    assert torch.isfinite(big).all() and abs(float(big.sum()) - 1) < 1e-12
    assert torch.allclose(big, torch.softmax(torch.tensor([1000., 1001., 1002., 999.], dtype=D), 0))
    x = torch.randn(7, dtype=D)
    assert torch.allclose(plain.softmax(x), plain.softmax(x + 3.5))       # shift invariance


def test_silu():
    # src/kernels/tests.rs:27-39
    x = torch.tensor([0., 1., -1., 5.], dtype=D)
    y = plain.silu(x)
    assert y[0] == 0 and y[1] > 0 and y[2] < 0
    assert torch.allclose(y, x * torch.sigmoid(x))


def test_rmsnorm_unit_weight_and_eps_place():
    # src/kernels/tests.rs:42-51: unit weight gives RMS 1
    x = torch.tensor([1., 2., 3.], dtype=D)
    y = plain.rmsnorm(x, torch.ones(3, dtype=D), 1e-5)
    assert abs(float((y * y).mean().sqrt()) - 1) < 1e-4
    # the same by a library's formula
    w = torch.tensor([0.5, 0.6, 0.7], dtype=D)
    assert torch.allclose(plain.rmsnorm(x, w, 1e-5), x * torch.rsqrt((x * x).mean() + 1e-5) * w)
    # eps is inside the root and added to the MEAN: with tiny x it dominates
    t = torch.tensor([1e-3, -1e-3], dtype=D)
    y = plain.rmsnorm(t, torch.ones(2, dtype=D), 1e-2)
    assert torch.allclose(y, t / math.sqrt(1e-6 + 1e-2))
    assert not torch.allclose(y, t / (math.sqrt(1e-6) + 1e-2))            # eps outside the root
    assert not torch.allclose(y, t / math.sqrt((2e-6 + 1e-2) / 2))        # eps added to the sum
    # weight is used as it is, not 1 + w
    assert torch.allclose(plain.rmsnorm(x, torch.zeros(3, dtype=D), 1e-5), torch.zeros(3, dtype=D))


def test_rope_frequencies():
    # src/kernels/tests.rs:54-69
    f = plain.rope_inv_freq(128, 10000.0)
    assert f.shape == (64,) and f[0] == 1.0 and bool((f[1:] < f[:-1]).all())
    assert abs(float(f[32]) - 10000.0 ** -0.5) < 1e-12                   # exponent i / (d/2)


def test_rope_identity_norm_and_pairing():
    x = torch.arange(32, dtype=D).view(1, 2, 16) + 1
    # pos 0 is the identity (src/kernels/tests.rs:72-84, :391-425)
    assert torch.equal(plain.rope(x, torch.tensor([0]), 1e4), x)
    y = plain.rope(x, torch.tensor([5]), 1e4)
    assert not torch.allclose(y, x)
    # each pair (i, i + d/2) keeps its length; neighbours (2i, 2i+1) do not
    h = 8
    assert torch.allclose(x[..., :h] ** 2 + x[..., h:] ** 2, y[..., :h] ** 2 + y[..., h:] ** 2)
    assert not torch.allclose(x[..., 0::2] ** 2 + x[..., 1::2] ** 2, y[..., 0::2] ** 2 + y[..., 1::2] ** 2)
    # pair 0 turns by exactly pos radians (inv_freq[0] = 1), and the sign is that of the reference
    v = torch.zeros(1, 1, 4, dtype=D)
    v[0, 0, 0] = 1.0
    r = plain.rope(v, torch.tensor([1]), 1e4)
    assert abs(float(r[0, 0, 0]) - math.cos(1)) < 1e-12 and abs(float(r[0, 0, 2]) - math.sin(1)) < 1e-12


def test_rope_variants_reduce_to_the_rotation():
    """The toy family: all channels in halves is `rope`; interleaved pairs written out by hand;
    channels behind `rotary_dim` untouched, and the rotated ones as a head of that size."""
    g = torch.Generator().manual_seed(8)
    x = torch.randn(5, 3, 12, generator=g, dtype=D)
    pos = torch.tensor([0, 1, 7, 30, 200])
    assert torch.equal(plain.rope_variant(x, pos, 100.0, 12, False), plain.rope(x, pos, 100.0))
    inter = plain.rope_variant(x, pos, 100.0, 12, True)
    inv = plain.rope_inv_freq(12, 100.0)
    for i in range(6):
        ang = pos.to(D) * inv[i]
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        a, b = x[..., 2 * i], x[..., 2 * i + 1]
        assert torch.allclose(inter[..., 2 * i], a * c - b * s) and torch.allclose(inter[..., 2 * i + 1], a * s + b * c)
    part = plain.rope_variant(x, pos, 100.0, 8, False)
    assert torch.equal(part[..., 8:], x[..., 8:]) and torch.equal(part[..., :8], plain.rope(x[..., :8], pos, 100.0))
    assert torch.equal(plain.rope_variant(x, pos, 100.0, 0, False), x)
    assert not torch.allclose(inter, plain.rope(x, pos, 100.0))


def test_rope_scores_depend_on_distance_only():
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, 1, 16, generator=g, dtype=D)
    k = torch.randn(1, 1, 16, generator=g, dtype=D)
    def score(m, n):
        return float((plain.rope(q, torch.tensor([m]), 1e4) * plain.rope(k, torch.tensor([n]), 1e4)).sum())
    assert abs(score(7, 3) - score(107, 103)) < 1e-9
    assert abs(score(7, 3) - score(3, 7)) > 1e-3


def test_scores_and_weighted_sum_vectors():
    # q=[1,0], K=I -> scores [1,0] before scale (src/kernels/tests.rs:714-728);
    # weights [.5,.5] over rows [2,4],[6,8] -> [4,6] (:698-711)
    q = torch.tensor([[[1., 0.]]], dtype=D)
    k = torch.eye(2, dtype=D).view(2, 1, 2)
    # attention of the second position over both keys with equal scores
    qq = torch.zeros(2, 1, 2, dtype=D)
    v = torch.tensor([[[2., 4.]], [[6., 8.]]], dtype=D)
    out = plain.attention_core(qq, k, v, torch.arange(2), None)
    assert torch.allclose(out[1, 0], torch.tensor([4., 6.], dtype=D))
    assert torch.allclose(out[0, 0], torch.tensor([2., 4.], dtype=D))     # causal: first sees itself


def test_attention_equals_library_without_mask_and_rotation():
    # the last query sees every key: plain softmax(QK^T/sqrt(d))V of a library
    g = torch.Generator().manual_seed(1)
    T, nq, nkv, d = 9, 4, 2, 8
    q = torch.randn(T, nq, d, generator=g, dtype=D)
    k = torch.randn(T, nkv, d, generator=g, dtype=D)
    v = torch.randn(T, nkv, d, generator=g, dtype=D)
    out = plain.attention_core(q, k, v, torch.arange(T), None)
    kk = k.repeat_interleave(nq // nkv, dim=1)          # head h reads KV head h // g
    vv = v.repeat_interleave(nq // nkv, dim=1)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True).transpose(0, 1)
    assert torch.allclose(out, ref, atol=1e-12)
    # scale uses the head size: doubling d by zero padding changes the result
    z = torch.zeros(T, nq, d, dtype=D)
    zk = torch.zeros(T, nkv, d, dtype=D)
    out2 = plain.attention_core(torch.cat([q, z], -1), torch.cat([k, zk], -1), torch.cat([v, zk], -1),
                                torch.arange(T), None)[..., :d]
    assert not torch.allclose(out, out2)


def test_one_head_one_kv_head_reduces_to_library():
    g = torch.Generator().manual_seed(2)
    T, d = 6, 4
    q, k, v = (torch.randn(T, 1, d, generator=g, dtype=D) for _ in range(3))
    out = plain.attention_core(q, k, v, torch.arange(T), None)[:, 0]
    s = (q[:, 0] @ k[:, 0].t()) / math.sqrt(d)
    s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
    assert torch.allclose(out, torch.softmax(s, -1) @ v[:, 0])


def test_window_rule():
    pos = torch.arange(12)
    m = plain.visible(pos, 4)
    # src/model/models/gpt_oss.rs:168-175: exactly min(p+1, W) keys, the newest ones
    assert m.sum(1).tolist() == [min(p + 1, 4) for p in range(12)]
    assert bool(m[10, 7]) and not bool(m[10, 6]) and bool(m[10, 10]) and not bool(m[10, 11])
    assert torch.equal(plain.visible(pos, 12), plain.visible(pos, None))  # W >= T: no window
    # W = 1: every position attends to itself only -> output is its own value row
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(5, 2, 4, generator=g, dtype=D) for _ in range(3))
    assert torch.allclose(plain.attention_core(q, k, v, torch.arange(5), 1), v)


def test_gqa_mapping():
    # zeroing one KV head's values changes exactly its g consecutive query heads
    g = torch.Generator().manual_seed(4)
    T, nq, nkv, d = 5, 6, 3, 4
    q = torch.randn(T, nq, d, generator=g, dtype=D)
    k = torch.randn(T, nkv, d, generator=g, dtype=D)
    v = torch.randn(T, nkv, d, generator=g, dtype=D)
    a = plain.attention_core(q, k, v, torch.arange(T), None)
    v2 = v.clone()
    v2[:, 1] = 0
    b = plain.attention_core(q, k, v2, torch.arange(T), None)
    changed = [(a[:, h] - b[:, h]).abs().max() > 0 for h in range(nq)]
    assert changed == [False, False, True, True, False, False]


def test_online_softmax_vector():
    # src/model/modules/flash_attention.rs:671-706: scores 1,2,3 over value rows 1,2,3
    p = plain.softmax(torch.tensor([1., 2., 3.], dtype=D))
    got = float((p * torch.tensor([1., 2., 3.], dtype=D)).sum())
    want = (math.exp(-2) + 2 * math.exp(-1) + 3) / (math.exp(-2) + math.exp(-1) + 1)
    assert abs(got - want) < 1e-12


def _tiny(seed=0, **over):
    cfg = dict(num_hidden_layers=2, hidden_size=16, num_attention_heads=4, num_key_value_heads=2,
               intermediate_size=24, vocab_size=32, rope_theta=100.0, sliding_window=None,
               rms_norm_eps=1e-5)
    cfg.update(over)
    g = torch.Generator().manual_seed(seed)
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    d = cfg.get("head_dim") or H // cfg["num_attention_heads"]
    nq, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    w = {"model.embed_tokens.weight": torch.randn(V, H, generator=g, dtype=D),
         "model.norm.weight": 1 + 0.1 * torch.randn(H, generator=g, dtype=D),
         "lm_head.weight": torch.randn(V, H, generator=g, dtype=D) * 0.3}
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w[p + "input_layernorm.weight"] = 1 + 0.1 * torch.randn(H, generator=g, dtype=D)
        w[p + "post_attention_layernorm.weight"] = 1 + 0.1 * torch.randn(H, generator=g, dtype=D)
        w[p + "self_attn.q_proj.weight"] = torch.randn(nq * d, H, generator=g, dtype=D) * 0.3
        w[p + "self_attn.k_proj.weight"] = torch.randn(nkv * d, H, generator=g, dtype=D) * 0.3
        w[p + "self_attn.v_proj.weight"] = torch.randn(nkv * d, H, generator=g, dtype=D) * 0.3
        w[p + "self_attn.o_proj.weight"] = torch.randn(H, nq * d, generator=g, dtype=D) * 0.3
        w[p + "mlp.gate_proj.weight"] = torch.randn(I, H, generator=g, dtype=D) * 0.3
        w[p + "mlp.up_proj.weight"] = torch.randn(I, H, generator=g, dtype=D) * 0.3
        w[p + "mlp.down_proj.weight"] = torch.randn(H, I, generator=g, dtype=D) * 0.3
    return cfg, w


def test_model_is_causal_and_untied():
    cfg, w = _tiny()
    ids = [3, 7, 1, 30, 12, 5]
    full = plain.forward(w, cfg, ids)
    assert full.shape == (6, 32)
    assert torch.allclose(plain.forward(w, cfg, ids[:4]), full[:4], atol=1e-12)   # a prefix is a prefix
    w2 = dict(w)
    w2["lm_head.weight"] = w["lm_head.weight"] * 2                         # untied: only the head scales
    assert torch.allclose(plain.forward(w2, cfg, ids), 2 * full, atol=1e-10)


def test_model_norm_placement():
    # pre-norm with a serial residual (src/model/modules/layer.rs:28-56): zero
    # output projections leave the embedding untouched on its way to the head
    cfg, w = _tiny(1)
    for i in range(2):
        w[f"model.layers.{i}.self_attn.o_proj.weight"] *= 0
        w[f"model.layers.{i}.mlp.down_proj.weight"] *= 0
    ids = [4, 9]
    x = w["model.embed_tokens.weight"][ids]
    want = plain.rmsnorm(x, w["model.norm.weight"], 1e-5) @ w["lm_head.weight"].t()
    assert torch.allclose(plain.forward(w, cfg, ids), want, atol=1e-12)


def test_model_window_limits_reach():
    # with L layers and window W a change at position 0 cannot reach positions >= L*(W-1)+1
    cfg, w = _tiny(2, sliding_window=3)
    a = [1, 2, 3, 4, 5, 6, 7, 8]
    b = [9] + a[1:]
    fa, fb = plain.forward(w, cfg, a), plain.forward(w, cfg, b)
    reach = 2 * (3 - 1)
    assert (fa[reach + 1:] - fb[reach + 1:]).abs().max() < 1e-12
    assert (fa[reach] - fb[reach]).abs().max() > 1e-9


def test_explicit_head_dim():
    cfg, w = _tiny(3, head_dim=6)                   # 4 heads * 6 = 24, not the width 16
    out = plain.forward(w, cfg, [1, 2, 3])
    assert out.shape == (3, 32) and torch.isfinite(out).all()


# --- sampling ---------------------------------------------------------------

def test_greedy_and_ties():
    assert plain.greedy(torch.tensor([0.1, 0.9, 0.3])) == 1               # src/sampler/tests.rs:35-50
    assert plain.greedy(torch.tensor([0.5, 0.9, 0.9])) == 2               # of equal maxima the last
    assert plain.sample(torch.tensor([0.1, 0.9, 0.3]), 0.99, 0.0, top_k=2) == 1   # T=0 is greedy


def test_distribution_properties():
    z = torch.tensor([2.0, 1.0, 0.5, 0.1, -1.0])
    p1 = plain.sample_distribution(z, 1.0)
    assert abs(float(p1.sum()) - 1) < 1e-12
    p5 = plain.sample_distribution(z, 5.0)
    assert float(p5.max()) < float(p1.max())                               # higher T flattens
    pk = plain.sample_distribution(z, 1.0, top_k=3)
    assert (pk[3:] == 0).all() and abs(float(pk.sum()) - 1) < 1e-12       # src/sampler/tests.rs:184-203
    assert torch.allclose(plain.sample_distribution(z, 1.0, top_k=5), p1)  # k >= V: no effect
    assert torch.allclose(plain.sample_distribution(z, 1.0, top_p=1.0), p1)
    pp = plain.sample_distribution(torch.tensor([10.0, 0.0, 0.0, 0.0]), 1.0, top_p=0.5)
    assert pp.tolist() == [1.0, 0.0, 0.0, 0.0]                             # src/sampler/tests.rs:259-278
    pkp = plain.sample_distribution(z, 1.0, top_k=3, top_p=0.8)
    assert abs(float(pkp.sum()) - 1) < 1e-12


def test_top_k_ties_in_index_order():
    z = plain.top_k_filter(torch.tensor([1.0, 3.0, 1.0, 1.0, 2.0], dtype=D), 3)
    assert z.tolist() == [1.0, 3.0, float("-inf"), float("-inf"), 2.0]


def test_draw():
    p = torch.tensor([0.2, 0.3, 0.5], dtype=D)
    assert [plain.draw(p, r) for r in (0.0, 0.2, 0.21, 0.5, 0.51, 0.999)] == [0, 0, 1, 1, 2, 2]
    assert plain.draw(torch.tensor([0.2, 0.3], dtype=D), 0.9) == 1         # never reached: last index


# ---- the variant with the engine's bfloat16 roundings --------------------------------

def test_to_bf16_rounds_to_nearest_even():
    one = 1.0
    ulp = 2.0 ** -7                                          # spacing of bfloat16 in [1, 2)
    x = torch.tensor([one + 0.49 * ulp, one + 0.51 * ulp, one + 0.5 * ulp, one + 1.5 * ulp, -3.0, 0.0], dtype=torch.float64)
    want = torch.tensor([one, one + ulp, one, one + 2 * ulp, -3.0, 0.0], dtype=torch.float64)   # ties go to the even mantissa
    assert torch.equal(plain.to_bf16(x), want)


def test_rounded_forward_is_the_plain_forward_when_nothing_is_rounded(monkeypatch):
    """With the rounding taken out, `forward_rounded` must give `forward`'s logits, in both
    forms of the norm and with and without the rounding of gate and up: its formulas are the
    plain ones, only the roundings are its own."""
    cfg, w = _tiny(seed=5, num_hidden_layers=3, head_dim=6, sliding_window=9)
    ids = torch.randint(0, cfg["vocab_size"], (40,), generator=torch.Generator().manual_seed(3)).tolist()
    want = plain.forward(w, cfg, ids)
    monkeypatch.setattr(plain, "to_bf16", lambda t: t)
    for rows in ([40] * 40, [1] * 40, [100] * 30 + [3] * 10):
        got = plain.forward_rounded(w, cfg, ids, rows)
        assert float((got - want).abs().max()) < 1e-10 * float(want.abs().max()), rows


def test_rounded_forward_is_near_and_not_equal():
    cfg, w = _tiny(seed=6)
    ids = torch.randint(0, cfg["vocab_size"], (30,), generator=torch.Generator().manual_seed(4)).tolist()
    want = plain.forward(w, cfg, ids)
    whole, single = plain.forward_rounded(w, cfg, ids, [30] * 30), plain.forward_rounded(w, cfg, ids, [1] * 30)
    err = lambda a: float((a - want).abs().max() / want.abs().max())
    assert 1e-4 < err(whole) < 5e-2 and 1e-4 < err(single) < 5e-2
    assert not torch.equal(whole, single)                   # the norm cut in two rounds elsewhere
    first = plain.forward_rounded(w, cfg, ids[:1], [30])
    assert float((whole[:1] - first).abs().max()) < 1e-9       # a row depends on its prefix only
