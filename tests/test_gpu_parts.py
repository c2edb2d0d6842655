"""Each part alone against the plain implementation; a schedule that names a
layer twice and lets a run read another run's cache; and a toy mixer with
state of its own, defined here, that is registered, built and stepped
without a change to the framework's files."""
import math

import pytest
import torch

import plain_mistral as plain
from util import TOL, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
PTOL = {"float32": 5e-6, "bfloat16": 1.5e-2}


def rnd(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def context(cache, batch, dtype):
    from torchless_rs_amd.engine.engine import build_context
    from torchless_rs_amd.parts import Workspace
    return build_context(cache, batch, 10 ** 6, dtype, torch.device(DEV), Workspace(torch.device(DEV)))[0]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_norm_part(dt):
    from torchless_rs_amd.parts import PartSpec, make_part
    norm = make_part("norm", PartSpec("rmsnorm", {"size": 72, "eps": 1e-4}))
    assert norm.weight_specs()["weight"].shape == (72,)
    w = 1 + 0.3 * rnd(72, seed=1, dtype=DT[dt])
    norm.load({"weight": w.to(DEV)}, DT[dt])
    x = rnd(5, 72, seed=2, scale=2.0)
    out = torch.empty(5, 72, dtype=DT[dt], device=DEV)
    norm.forward(None, x.to(DEV), out)
    assert rel_err(out, plain.rmsnorm(x.double(), w.double(), 1e-4)) < PTOL[dt]


def test_position_part():
    from torchless_rs_amd.parts import PartSpec, make_part
    rot = make_part("position", PartSpec("rotary", {"head_dim": 48, "theta": 500.0}))
    f = rot.inv_freq(DEV).cpu()
    r = rot.rotation(DEV)
    assert (r.rotary_dim, r.interleaved) == (48, False) and r.inv_freq is rot.inv_freq(DEV)
    assert make_part("position", PartSpec("none", {})).rotation(DEV) is None
    part = make_part("position", PartSpec("rotary", {"head_dim": 48, "theta": 500.0, "rotary_dim": 16, "interleaved": True}))
    assert (part.rotation(DEV).rotary_dim, part.rotation(DEV).interleaved) == (16, True)
    assert rel_err(part.inv_freq(DEV).cpu(), plain.rope_inv_freq(16, 500.0)) < 1e-7
    assert f.shape == (24,) and f[0] == 1.0 and bool((f[1:] < f[:-1]).all())     # kernels/tests.rs:54-69
    assert rel_err(f, plain.rope_inv_freq(48, 500.0)) < 1e-7
    with pytest.raises(ValueError):
        make_part("position", PartSpec("rotary", {"head_dim": 7, "theta": 1.0}))


@pytest.mark.parametrize("n", [7, 40])
@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_feed_forward_part(dt, n):
    from torchless_rs_amd.cache import Cache
    from torchless_rs_amd.engine import SeqInput
    from torchless_rs_amd.parts import PartSpec, make_part
    from torchless_rs_amd.parts.base import flush_pending
    H, I = 72, 224
    ffn = make_part("ffn", PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I}))
    w = {"mlp.gate_proj.weight": rnd(I, H, seed=3, scale=0.2, dtype=DT[dt]),
         "mlp.up_proj.weight": rnd(I, H, seed=4, scale=0.2, dtype=DT[dt]),
         "mlp.down_proj.weight": rnd(H, I, seed=5, scale=0.2, dtype=DT[dt])}
    assert {k: v.shape for k, v in ffn.weight_specs().items()} == {k: tuple(v.shape) for k, v in w.items()}
    ffn.load({k: v.to(DEV) for k, v in w.items()}, DT[dt])
    cache = Cache({}, {}, 64, DT[dt], DEV, 1)
    s = cache.alloc_slot()
    ctx = context(cache, [SeqInput(s, [0] * n, [])], DT[dt])
    y = rnd(n, H, seed=6, dtype=DT[dt])
    x0 = rnd(n, H, seed=7)
    x = x0.clone().to(DEV)
    ffn.forward(ctx, y.to(DEV), x)
    flush_pending(ctx, x)
    want = x0.double() + plain.swiglu(y.double(), {k: v.double() for k, v in w.items()}, "")
    assert rel_err(x, want) < PTOL[dt]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("nq,nkv,d,window", [(4, 2, 16, 8), (6, 1, 32, None), (3, 3, 48, 70)])
def test_attention_part_whole_and_in_steps(dt, nq, nkv, d, window):
    """The mixer alone: two sequences, whole, and cut into a head and single tokens."""
    from torchless_rs_amd.cache import Cache
    from torchless_rs_amd.engine import SeqInput
    from torchless_rs_amd.parts import PartSpec, RunBinding, make_part
    from torchless_rs_amd.parts.base import flush_pending
    H, lens = 40, [90, 13]
    mixer = make_part("mixer", PartSpec("attention", {
        "hidden_size": H, "n_heads": nq, "n_kv_heads": nkv, "head_dim": d, "window": window,
        "position": PartSpec("rotary", {"head_dim": d, "theta": 300.0})}))
    w = {"self_attn.q_proj.weight": rnd(nq * d, H, seed=1, scale=0.3, dtype=DT[dt]),
         "self_attn.k_proj.weight": rnd(nkv * d, H, seed=2, scale=0.3, dtype=DT[dt]),
         "self_attn.v_proj.weight": rnd(nkv * d, H, seed=3, scale=0.3, dtype=DT[dt]),
         "self_attn.o_proj.weight": rnd(H, nq * d, seed=4, scale=0.3, dtype=DT[dt])}
    assert {k: v.shape for k, v in mixer.weight_specs().items()} == {k: tuple(v.shape) for k, v in w.items()}
    mixer.load({k: v.to(DEV) for k, v in w.items()}, DT[dt])
    cfg = {"num_attention_heads": nq, "num_key_value_heads": nkv, "head_dim": d, "hidden_size": H,
           "rope_theta": 300.0, "sliding_window": window}
    ys = [rnd(n, H, seed=10 + i, dtype=DT[dt]) for i, n in enumerate(lens)]
    wd = {k: v.double() for k, v in w.items()}
    want = torch.cat([plain.attention(y.double(), wd, "", cfg, torch.arange(y.shape[0])) for y in ys])

    cache = Cache({0: mixer.kv_request()}, {}, 64 * 6, DT[dt], DEV, 2)
    cache.groups[0].storage.fill_(float("nan"))
    g = cache.groups[0]
    run = RunBinding(index=0, kv_group=g, kv_group_index=0, kv_layer=0, kv_source=0)
    # whole
    slots = [cache.alloc_slot() for _ in lens]
    batch = [SeqInput(s, [0] * n, []) for s, n in zip(slots, lens)]
    ctx = context(cache, batch, DT[dt])
    x = torch.zeros(sum(lens), H, device=DEV)
    mixer.forward(ctx, run, torch.cat(ys).to(DEV), x)
    flush_pending(ctx, x)               # a part may leave partial products for the next reader of x
    cache.commit([(s, n) for s, n in zip(slots, lens)])
    assert rel_err(x, want) < PTOL[dt]
    for s in slots:
        cache.free_slot(s)
    # heads of unequal lengths, then one token each until the shorter one ends
    slots = [cache.alloc_slot() for _ in lens]
    heads = [50, 3]
    got = [[], []]
    ctx = context(cache, [SeqInput(s, [0] * h, []) for s, h in zip(slots, heads)], DT[dt])
    x = torch.zeros(sum(heads), H, device=DEV)
    mixer.forward(ctx, run, torch.cat([y[:h] for y, h in zip(ys, heads)]).to(DEV), x)
    flush_pending(ctx, x)
    cache.commit(list(zip(slots, heads)))
    got[0].append(x[:50].clone()); got[1].append(x[50:].clone())
    fed = list(heads)
    while any(f < n for f, n in zip(fed, lens)):
        live = [i for i in range(2) if fed[i] < lens[i]]
        ctx = context(cache, [SeqInput(slots[i], [0], []) for i in live], DT[dt])
        x = torch.zeros(len(live), H, device=DEV)
        mixer.forward(ctx, run, torch.stack([ys[i][fed[i]] for i in live]).to(DEV), x)
        flush_pending(ctx, x)
        cache.commit([(slots[i], 1) for i in live])
        for r, i in enumerate(live):
            got[i].append(x[r:r + 1].clone())
            fed[i] += 1
    assert rel_err(torch.cat(got[0] + got[1]), want) < PTOL[dt]


# ---- the schedule is data ----------------------------------------------------------

def test_a_layer_twice_and_a_run_that_reads_anothers_cache():
    from torchless_rs_amd.engine import Engine, SeqInput
    from torchless_rs_amd.engine.model import Model
    from torchless_rs_amd.parts import LayerSpec, ModelSpec, PartSpec, Run
    from torchless_rs_amd.weights import TensorDict, random_tensors
    H, V, nq, nkv, d, I = 48, 90, 3, 1, 16, 80
    norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-5})
    rot = PartSpec("rotary", {"head_dim": d, "theta": 1000.0})

    def layer(i, own_kv=True, window=None):
        return LayerSpec(prefix=f"model.layers.{i}.",
                         mixer=PartSpec("attention", {"hidden_size": H, "n_heads": nq, "n_kv_heads": nkv,
                                                      "head_dim": d, "window": window, "position": rot,
                                                      "own_kv": own_kv}),
                         ffn=PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I}),
                         mixer_norm=norm, ffn_norm=norm)

    spec = ModelSpec(hidden_size=H, vocab_size=V,
                     embedding=PartSpec("tokens", {"vocab_size": V, "hidden_size": H}), embedding_prefix="model.",
                     layers=[layer(0, window=6), layer(1), layer(2, own_kv=False)],
                     schedule=[Run(0), Run(1), Run(0), Run(2, kv_from=1)],
                     final_norm=norm, final_norm_prefix="model.norm.",
                     head=PartSpec("linear", {"vocab_size": V, "hidden_size": H}), head_prefix="lm_head.")
    names = spec.weight_specs()
    assert "model.layers.2.self_attn.k_proj.weight" not in names and "model.layers.2.self_attn.q_proj.weight" in names
    w = random_tensors(names, seed=3, std=0.15, norm_std=0.1, dtype=torch.float32)
    model = Model(spec, None, torch.float32, DEV)
    model.load_weights(TensorDict(w))
    eng = Engine(model, max_tokens=64 * 4)
    assert len(eng.cache.groups) == 2                       # windowed runs (0 and 2) and the full one
    assert sorted(g.runs for g in eng.cache.groups) == [[0, 2], [1]]

    def plain_forward(ids):
        T = len(ids)
        pos = torch.arange(T)
        wd = {k: v.double() for k, v in w.items()}
        x = wd["model.embed_tokens.weight"][ids]
        cfg0 = {"num_attention_heads": nq, "num_key_value_heads": nkv, "head_dim": d, "hidden_size": H,
                "rope_theta": 1000.0, "rms_norm_eps": 1e-5}
        x = plain.block(x, wd, "model.layers.0.", dict(cfg0, sliding_window=6), pos)
        # layer 1, keeping its rotated keys and its values
        p1 = "model.layers.1."
        y = plain.rmsnorm(x, wd[p1 + "input_layernorm.weight"], 1e-5)
        k1 = plain.rope(plain.linear(y, wd[p1 + "self_attn.k_proj.weight"]).view(T, nkv, d), pos, 1000.0)
        v1 = plain.linear(y, wd[p1 + "self_attn.v_proj.weight"]).view(T, nkv, d)
        x = plain.block(x, wd, p1, dict(cfg0, sliding_window=None), pos)
        x = plain.block(x, wd, "model.layers.0.", dict(cfg0, sliding_window=6), pos)   # the same weights again
        p2 = "model.layers.2."
        y = plain.rmsnorm(x, wd[p2 + "input_layernorm.weight"], 1e-5)
        q = plain.rope(plain.linear(y, wd[p2 + "self_attn.q_proj.weight"]).view(T, nq, d), pos, 1000.0)
        a = plain.attention_core(q, k1, v1, pos, None).reshape(T, nq * d)
        x = x + plain.linear(a, wd[p2 + "self_attn.o_proj.weight"])
        x = x + plain.swiglu(plain.rmsnorm(x, wd[p2 + "post_attention_layernorm.weight"], 1e-5), wd, p2)
        return plain.linear(plain.rmsnorm(x, wd["model.norm.weight"], 1e-5), wd["lm_head.weight"])

    g = torch.Generator().manual_seed(8)
    ids = torch.randint(0, V, (40,), generator=g).tolist()
    want = plain_forward(ids)
    s = eng.alloc()
    whole = eng.step([SeqInput(s, ids, list(range(40)))]).clone()
    eng.free(s)
    assert rel_err(whole, want) < TOL["float32"]
    s = eng.alloc()
    outs = [eng.step([SeqInput(s, ids[:9], list(range(9)))]).clone(),
            eng.step([SeqInput(s, ids[9:25], list(range(16)))]).clone()]
    outs += [eng.step([SeqInput(s, [t], [0])]).clone() for t in ids[25:]]
    eng.free(s)
    assert rel_err(torch.cat(outs), want) < TOL["float32"]


# ---- a toy mixer with state of its own ----------------------------------------------

def test_a_toy_mixer_with_state_registers_builds_and_steps():
    """out_t = W (decay-weighted running sum of the inputs up to t): the sum so
    far is the mixer's state, one row of H floats per sequence, kept in the
    cache's state area.  Library operations are fine for a toy."""
    from torchless_rs_amd.cache import StateRequest
    from torchless_rs_amd.config import config_from_dict, register_architecture, unregister_architecture
    from torchless_rs_amd.config.base import ModelConfig
    from torchless_rs_amd.engine import Engine, SeqInput
    from torchless_rs_amd.engine.model import Model
    from torchless_rs_amd.models import model_spec_for
    from torchless_rs_amd.parts import (LayerSpec, Mixer, ModelSpec, PartSpec, Run, register_part,
                                        unregister_part)
    from torchless_rs_amd.weights import TensorDict, WeightSpec, random_tensors

    class RunningSum(Mixer):
        def __init__(self, hidden_size, decay):
            self.H, self.decay = hidden_size, decay

        def weight_specs(self):
            return {"mix.weight": WeightSpec((self.H, self.H))}

        def state_request(self):
            return StateRequest((self.H,), torch.float32)

        def load(self, tensors, compute_dtype):
            self.w = tensors["mix.weight"].float()

        def forward(self, ctx, run, y, x):
            cu, slots = ctx.host["cu"], ctx.host["slots"]
            for b, slot in enumerate(slots):
                s = run.state[slot].clone()
                for r in range(int(cu[b]), int(cu[b + 1])):
                    s = self.decay * s + y[r].float()
                    x[r] += s @ self.w.t()
                run.state[slot] = s

    class ToyConfig(ModelConfig):
        @classmethod
        def from_dict(cls, d):
            c = cls(architecture="ToyForCausalLM")
            c.d = d
            return c

    def toy_spec(cfg):
        d = cfg.d
        H, V = d["width"], d["vocab"]
        norm = PartSpec("rmsnorm", {"size": H, "eps": d["eps"]})
        layers = [LayerSpec(prefix=f"toy.{i}.", mixer=PartSpec("running_sum", {"hidden_size": H, "decay": d["decay"]}),
                            ffn=PartSpec("swiglu", {"hidden_size": H, "intermediate_size": d["inner"]}),
                            mixer_norm=norm, ffn_norm=norm) for i in range(d["depth"])]
        return ModelSpec(hidden_size=H, vocab_size=V, embedding=PartSpec("tokens", {"vocab_size": V, "hidden_size": H}),
                         embedding_prefix="toy.", layers=layers, schedule=[Run(i) for i in range(d["depth"])],
                         final_norm=norm, final_norm_prefix="toy.norm.",
                         head=PartSpec("linear", {"vocab_size": V, "hidden_size": H, "tied": True}), head_prefix="toy.head.")

    register_part("mixer", "running_sum", RunningSum)
    register_architecture("ToyForCausalLM", ToyConfig, toy_spec)
    try:
        d = {"architectures": ["ToyForCausalLM"], "width": 40, "vocab": 70, "inner": 56, "depth": 2,
             "eps": 1e-5, "decay": 0.9}
        cfg = config_from_dict(d)
        spec = model_spec_for(cfg)
        w = random_tensors(spec.weight_specs(), seed=1, std=0.2, dtype=torch.float32)
        assert "toy.1.mix.weight" in w and "toy.head.weight" not in w
        model = Model(spec, cfg, torch.float32, DEV)
        model.load_weights(TensorDict(w))
        eng = Engine(model, max_tokens=64 * 4, max_slots=3)
        assert not eng.cache.groups and sorted(eng.cache.state) == [0, 1]
        assert eng.cache.state[0].shape == (3, 40)

        def plain_forward(ids):
            wd = {k: v.double() for k, v in w.items()}
            x = wd["toy.embed_tokens.weight"][ids]
            for i in range(2):
                y = plain.rmsnorm(x, wd[f"toy.{i}.input_layernorm.weight"], 1e-5)
                s = torch.zeros(40, dtype=torch.float64)
                add = []
                for t in range(len(ids)):
                    s = 0.9 * s + y[t]
                    add.append(wd[f"toy.{i}.mix.weight"] @ s)
                x = x + torch.stack(add)
                x = x + plain.swiglu(plain.rmsnorm(x, wd[f"toy.{i}.post_attention_layernorm.weight"], 1e-5), wd, f"toy.{i}.")
            return plain.rmsnorm(x, wd["toy.norm.weight"], 1e-5) @ wd["toy.embed_tokens.weight"].t()

        g = torch.Generator().manual_seed(2)
        a = torch.randint(0, 70, (12,), generator=g).tolist()
        b = torch.randint(0, 70, (5,), generator=g).tolist()
        wa, wb = plain_forward(a), plain_forward(b)
        sa, sb = eng.alloc(), eng.alloc()
        lg = eng.step([SeqInput(sa, a[:7], list(range(7))), SeqInput(sb, b[:2], [0, 1])]).clone()
        got_a, got_b = [lg[:7]], [lg[7:]]
        for t in range(3):
            lg = eng.step([SeqInput(sa, [a[7 + t]], [0]), SeqInput(sb, [b[2 + t]], [0])]).clone()
            got_a.append(lg[:1]); got_b.append(lg[1:])
        eng.free(sb)
        lg = eng.step([SeqInput(sa, a[10:], [0, 1])]).clone()
        got_a.append(lg)
        eng.free(sa)
        assert rel_err(torch.cat(got_a), wa) < 1e-5 and rel_err(torch.cat(got_b), wb) < 1e-5
        # the slot that is used again starts from a zeroed state
        s2 = eng.alloc()
        assert s2 in (sa, sb)
        again = eng.step([SeqInput(s2, b, list(range(5)))]).clone()
        eng.free(s2)
        assert rel_err(again, wb) < 1e-5
    finally:
        unregister_part("mixer", "running_sum")
        unregister_architecture("ToyForCausalLM")


# ---- toy parts of other kinds, registered from here ---------------------------------------

def _toy_model(spec_layers, H, V, eps=1e-5):
    from torchless_rs_amd.parts import ModelSpec, PartSpec, Run
    norm = PartSpec("rmsnorm", {"size": H, "eps": eps})
    return ModelSpec(hidden_size=H, vocab_size=V,
                     embedding=PartSpec("tokens", {"vocab_size": V, "hidden_size": H}), embedding_prefix="model.",
                     layers=spec_layers, schedule=[Run(i) for i in range(len(spec_layers))],
                     final_norm=norm, final_norm_prefix="model.norm.",
                     head=PartSpec("linear", {"vocab_size": V, "hidden_size": H}), head_prefix="lm_head.")


def test_a_toy_feed_forward_with_routing():
    """Two experts, each row goes to the one its router prefers (top-1, weight 1): a feed-forward
    with a dispatch stage of its own, built on the framework's products.  It decides on the host,
    so it is not `graph_safe` and its steps are never captured."""
    from torchless_rs_amd.engine import Engine, SeqInput
    from torchless_rs_amd.engine.model import Model
    from torchless_rs_amd.kernels import ops
    from torchless_rs_amd.parts import FeedForward, LayerSpec, PartSpec, register_part, unregister_part
    from torchless_rs_amd.weights import TensorDict, WeightSpec, random_tensors
    H, V, I, E, nq, nkv, d = 48, 60, 64, 2, 3, 1, 16

    class Top1Experts(FeedForward):
        def __init__(self, hidden_size, inner, experts):
            self.H, self.I, self.E = hidden_size, inner, experts

        def weight_specs(self):
            out = {"moe.router.weight": WeightSpec((self.E, self.H))}
            for e in range(self.E):
                out[f"moe.experts.{e}.gate_up.weight"] = WeightSpec((2 * self.I, self.H))
                out[f"moe.experts.{e}.down.weight"] = WeightSpec((self.H, self.I))
            return out

        def load(self, tensors, compute_dtype):
            self.t = tensors

        def forward(self, ctx, y, x):
            n = y.shape[0]
            logits = torch.empty(n, self.E, device=y.device)
            ops.gemm(y, self.t["moe.router.weight"], logits)
            choice = logits.argmax(-1)
            for e in range(self.E):
                rows = (choice == e).nonzero().flatten()
                if not rows.numel():
                    continue
                ye = y[rows].contiguous()
                gu = torch.empty(rows.numel(), 2 * self.I, device=y.device)
                ops.gemm(ye, self.t[f"moe.experts.{e}.gate_up.weight"], gu)
                h = torch.empty(rows.numel(), self.I, dtype=y.dtype, device=y.device)
                ops.silu_mul(gu, h)
                out = torch.empty(rows.numel(), self.H, device=y.device)
                ops.gemm(h, self.t[f"moe.experts.{e}.down.weight"], out)
                x[rows] += out

    register_part("ffn", "top1_experts", Top1Experts)
    try:
        norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-5})
        layers = [LayerSpec(prefix=f"model.layers.{i}.",
                            mixer=PartSpec("attention", {"hidden_size": H, "n_heads": nq, "n_kv_heads": nkv, "head_dim": d,
                                                         "window": None, "position": PartSpec("rotary", {"head_dim": d, "theta": 100.0})}),
                            ffn=PartSpec("top1_experts", {"hidden_size": H, "inner": I, "experts": E}),
                            mixer_norm=norm, ffn_norm=norm) for i in range(2)]
        spec = _toy_model(layers, H, V)
        w = random_tensors(spec.weight_specs(), seed=4, std=0.2, dtype=torch.float32)
        model = Model(spec, None, torch.float32, DEV)
        model.load_weights(TensorDict(w))
        assert not model.graph_safe
        eng = Engine(model, max_tokens=256)

        def plain_forward(ids):
            wd = {k: v.double() for k, v in w.items()}
            T = len(ids)
            pos = torch.arange(T)
            cfg = {"num_attention_heads": nq, "num_key_value_heads": nkv, "head_dim": d, "hidden_size": H, "rope_theta": 100.0}
            x = wd["model.embed_tokens.weight"][ids]
            for i in range(2):
                p = f"model.layers.{i}."
                x = x + plain.attention(plain.rmsnorm(x, wd[p + "input_layernorm.weight"], 1e-5), wd, p, cfg, pos)
                y = plain.rmsnorm(x, wd[p + "post_attention_layernorm.weight"], 1e-5)
                choice = (y @ wd[p + "moe.router.weight"].t()).argmax(-1)
                add = torch.zeros_like(x)
                for t in range(T):
                    e = int(choice[t])
                    gu = wd[p + f"moe.experts.{e}.gate_up.weight"] @ y[t]
                    add[t] = wd[p + f"moe.experts.{e}.down.weight"] @ (plain.silu(gu[:I]) * gu[I:])
                x = x + add
            return plain.rmsnorm(x, wd["model.norm.weight"], 1e-5) @ wd["lm_head.weight"].t()

        g = torch.Generator().manual_seed(3)
        ids = torch.randint(0, V, (30,), generator=g).tolist()
        want = plain_forward(ids)
        s = eng.alloc()
        outs = [eng.step([SeqInput(s, ids[:20], list(range(20)))]).clone()]
        outs += [eng.step([SeqInput(s, [t], [0])]).clone() for t in ids[20:]]
        eng.free(s)
        assert not eng._graphs
        assert rel_err(torch.cat(outs), want) < 1e-5
    finally:
        unregister_part("ffn", "top1_experts")


def test_a_toy_position_encoding():
    """Rotation with every frequency divided by a factor (positions stretched): another position
    encoding, a part of its own kind that the attention mixer takes by name."""
    from torchless_rs_amd.engine import Engine, SeqInput
    from torchless_rs_amd.engine.model import Model
    from torchless_rs_amd.parts import LayerSpec, PartSpec, register_part, unregister_part
    from torchless_rs_amd.parts.position import Rotary
    from torchless_rs_amd.weights import TensorDict, random_tensors
    H, V, I, nq, nkv, d, factor = 40, 50, 56, 5, 5, 8, 4.0

    class StretchedRotary(Rotary):
        def __init__(self, head_dim, theta, factor):
            super().__init__(head_dim, theta)
            self.factor = factor

        def inv_freq_host(self):
            return super().inv_freq_host() / self.factor

    register_part("position", "stretched_rotary", StretchedRotary)
    try:
        norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-5})
        pos_spec = PartSpec("stretched_rotary", {"head_dim": d, "theta": 50.0, "factor": factor})
        layers = [LayerSpec(prefix="model.layers.0.",
                            mixer=PartSpec("attention", {"hidden_size": H, "n_heads": nq, "n_kv_heads": nkv, "head_dim": d,
                                                         "window": 5, "position": pos_spec}),
                            ffn=PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I}),
                            mixer_norm=norm, ffn_norm=norm)]
        spec = _toy_model(layers, H, V)
        w = random_tensors(spec.weight_specs(), seed=6, std=0.3, dtype=torch.float32)
        model = Model(spec, None, torch.float32, DEV)
        model.load_weights(TensorDict(w))
        eng = Engine(model, max_tokens=128)

        def stretched(x, positions):
            # plain.rope at positions / factor is the same angle
            half = d // 2
            inv = plain.rope_inv_freq(d, 50.0, x.dtype) / factor
            ang = positions.to(x.dtype)[:, None] * inv[None, :]
            c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            a, b = x[..., :half], x[..., half:]
            return torch.cat([a * c - b * s, a * s + b * c], -1)

        def plain_forward(ids):
            wd = {k: v.double() for k, v in w.items()}
            T, p = len(ids), "model.layers.0."
            pos = torch.arange(T)
            x = wd["model.embed_tokens.weight"][ids]
            y = plain.rmsnorm(x, wd[p + "input_layernorm.weight"], 1e-5)
            q = stretched(plain.linear(y, wd[p + "self_attn.q_proj.weight"]).view(T, nq, d), pos)
            k = stretched(plain.linear(y, wd[p + "self_attn.k_proj.weight"]).view(T, nkv, d), pos)
            v = plain.linear(y, wd[p + "self_attn.v_proj.weight"]).view(T, nkv, d)
            a = plain.attention_core(q, k, v, pos, 5).reshape(T, nq * d)
            x = x + plain.linear(a, wd[p + "self_attn.o_proj.weight"])
            x = x + plain.swiglu(plain.rmsnorm(x, wd[p + "post_attention_layernorm.weight"], 1e-5), wd, p)
            return plain.rmsnorm(x, wd["model.norm.weight"], 1e-5) @ wd["lm_head.weight"].t()

        g = torch.Generator().manual_seed(7)
        ids = torch.randint(0, V, (24,), generator=g).tolist()
        want = plain_forward(ids)
        s = eng.alloc()
        outs = [eng.step([SeqInput(s, ids[:9], list(range(9)))]).clone()]
        outs += [eng.step([SeqInput(s, [t], [0])]).clone() for t in ids[9:]]
        eng.free(s)
        assert rel_err(torch.cat(outs), want) < 1e-5
        assert rel_err(torch.cat(outs), plain.forward({**w}, {"num_hidden_layers": 1, "hidden_size": H, "num_attention_heads": nq,
                       "num_key_value_heads": nkv, "head_dim": d, "rope_theta": 50.0, "sliding_window": 5,
                       "rms_norm_eps": 1e-5}, ids)) > 1e-3           # and it is not the plain rotation
    finally:
        unregister_part("position", "stretched_rotary")


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("rotary_dim,interleaved", [(16, True), (32, True), (16, False), (None, False)])
def test_other_names_fused_tensors_and_another_rotation_without_a_new_class(dt, rotary_dim, interleaved):
    """What another architecture with the same mathematics may differ in is data: the tensors'
    names (also of the norms), q|k|v and gate|up stored as one tensor each, a rotation of a share
    of the head in interleaved pairs, or no rotation.  The parts are the framework's own, chosen
    and parameterised by the specification; no class is defined here.  Whole prompts, then tokens
    one by one (the fused single-token kernels read tiled copies laid out for this rotation)."""
    from torchless_rs_amd.engine import Engine, SeqInput
    from torchless_rs_amd.engine.model import Model
    from torchless_rs_amd.parts import LayerSpec, ModelSpec, PartSpec, Run
    from torchless_rs_amd.weights import TensorDict, random_tensors
    H, V, I, nq, nkv, d, L, theta, window, eps = 128, 90, 192, 4, 2, 32, 2, 300.0, 40, 1e-5
    if rotary_dim is None:
        position = PartSpec("none", {})
    else:
        position = PartSpec("rotary", {"head_dim": d, "theta": theta, "rotary_dim": rotary_dim, "interleaved": interleaved})
    norm = PartSpec("rmsnorm", {"size": H, "eps": eps})
    layers = [LayerSpec(prefix=f"h.{i}.",
                        mixer=PartSpec("attention", {"hidden_size": H, "n_heads": nq, "n_kv_heads": nkv, "head_dim": d,
                                                     "window": window, "position": position, "prefix": "attn.",
                                                     "names": {"qkv": "qkv_proj.weight", "o": "dense.weight"}}),
                        ffn=PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I, "prefix": "ff.",
                                                "names": {"gate_up": "gate_up_proj.weight", "down": "fc2.weight"}}),
                        mixer_norm=norm, ffn_norm=norm,
                        block=PartSpec("pre_norm", {"mixer_norm_name": "ln_1.", "ffn_norm_name": "ln_2."}))
              for i in range(L)]
    spec = ModelSpec(hidden_size=H, vocab_size=V,
                     embedding=PartSpec("tokens", {"vocab_size": V, "hidden_size": H, "name": "wte.weight"}),
                     embedding_prefix="", layers=layers, schedule=[Run(i) for i in range(L)],
                     final_norm=norm, final_norm_prefix="ln_f.",
                     head=PartSpec("linear", {"vocab_size": V, "hidden_size": H, "name": "out.weight"}), head_prefix="")
    names = set(spec.weight_specs())
    assert names == {"wte.weight", "ln_f.weight", "out.weight"} | {
        f"h.{i}.{n}" for i in range(L) for n in ("ln_1.weight", "ln_2.weight", "attn.qkv_proj.weight", "attn.dense.weight",
                                                   "ff.gate_up_proj.weight", "ff.fc2.weight")}
    w = random_tensors(spec.weight_specs(), seed=12, std=0.08, norm_std=0.1, dtype=torch.bfloat16)
    model = Model(spec, None, DT[dt], DEV)
    model.load_weights(TensorDict(w))
    eng = Engine(model, max_tokens=64 * 6)

    def plain_forward(ids):
        wd = {k: v.double() for k, v in w.items()}
        T, pos = len(ids), torch.arange(len(ids))
        x = wd["wte.weight"][ids]
        for i in range(L):
            p = f"h.{i}."
            y = plain.rmsnorm(x, wd[p + "ln_1.weight"], eps)
            qkv = plain.linear(y, wd[p + "attn.qkv_proj.weight"]).view(T, nq + 2 * nkv, d)
            q, k, v = qkv[:, :nq], qkv[:, nq:nq + nkv], qkv[:, nq + nkv:]
            q = plain.rope_variant(q, pos, theta, rotary_dim or 0, interleaved)
            k = plain.rope_variant(k, pos, theta, rotary_dim or 0, interleaved)
            a = plain.attention_core(q, k, v, pos, window).reshape(T, nq * d)
            x = x + plain.linear(a, wd[p + "attn.dense.weight"])
            gu = plain.linear(plain.rmsnorm(x, wd[p + "ln_2.weight"], eps), wd[p + "ff.gate_up_proj.weight"])
            x = x + plain.linear(plain.silu(gu[:, :I]) * gu[:, I:], wd[p + "ff.fc2.weight"])
        return plain.linear(plain.rmsnorm(x, wd["ln_f.weight"], eps), wd["out.weight"])

    g = torch.Generator().manual_seed(13)
    seqs = [torch.randint(0, V, (n,), generator=g).tolist() for n in (70, 9, 33)]
    wants = [plain_forward(s) for s in seqs]
    tol = {"float32": 2e-5, "bfloat16": 3e-2}[dt]
    for tail in (0, 20):
        slots = [eng.alloc() for _ in seqs]
        heads = [max(1, len(s) - tail) for s in seqs]
        lg = eng.step([SeqInput(sl, s[:h], list(range(h))) for sl, s, h in zip(slots, seqs, heads)]).clone()
        o = 0
        for i, h in enumerate(heads):
            assert rel_err(lg[o:o + h], wants[i][:h]) < tol, (tail, i)
            o += h
        for t in range(tail):
            live = [i for i in range(len(seqs)) if heads[i] + t < len(seqs[i])]
            lg = eng.step([SeqInput(slots[i], [seqs[i][heads[i] + t]], [0]) for i in live]).clone()
            for r, i in enumerate(live):
                assert rel_err(lg[r:r + 1], wants[i][heads[i] + t:heads[i] + t + 1]) < tol, (tail, t, i)
        for sl in slots:
            eng.free(sl)
    if dt == "bfloat16":                       # the single-token steps did run the fused kernel on its tiled copy
        assert all(b.mixer.qkv.own_tiles is not None for b in model.blocks)
    eng.close()


def test_part_parameters_that_cannot_be_are_refused():
    from torchless_rs_amd.parts import PartSpec, make_part
    rot = PartSpec("rotary", {"head_dim": 16, "theta": 10.0})
    base = {"hidden_size": 32, "n_heads": 2, "n_kv_heads": 1, "head_dim": 16, "position": rot}
    with pytest.raises(ValueError, match="no tensors called"):
        make_part("mixer", PartSpec("attention", dict(base, names={"query": "wq"})))
    with pytest.raises(ValueError, match="q alone"):
        make_part("mixer", PartSpec("attention", dict(base, own_kv=False, names={"qkv": "wqkv"})))
    with pytest.raises(ValueError, match="no tensors called"):
        make_part("ffn", PartSpec("swiglu", {"hidden_size": 32, "intermediate_size": 64, "names": {"w1": "x"}}))
    with pytest.raises(ValueError, match="rotated channels"):
        make_part("position", PartSpec("rotary", {"head_dim": 16, "theta": 10.0, "rotary_dim": 18}))
    with pytest.raises(ValueError, match="rotated channels"):
        make_part("position", PartSpec("rotary", {"head_dim": 16, "theta": 10.0, "rotary_dim": 7}))


def test_a_toy_mixer_whose_values_are_wider_than_its_keys():
    """The cache does not assume that keys and values have one size: a mixer asks for keys of 8
    and values of 24 channels (`KVRequest(..., v_head_dim=24)`), gets a group with storage of that
    shape, and writes and reads it through the group's views.  One head, no rotation, all keys
    visible; library operations are fine for a toy."""
    from torchless_rs_amd.cache import KVRequest, PAGE
    from torchless_rs_amd.engine import Engine, SeqInput
    from torchless_rs_amd.engine.model import Model
    from torchless_rs_amd.parts import LayerSpec, Mixer, PartSpec, register_part, unregister_part
    from torchless_rs_amd.weights import TensorDict, WeightSpec, random_tensors
    H, V, I, dk, dv = 32, 40, 48, 8, 24

    class WideValues(Mixer):
        def __init__(self, hidden_size, key_dim, value_dim):
            self.H, self.dk, self.dv = hidden_size, key_dim, value_dim

        def weight_specs(self):
            return {"wq.weight": WeightSpec((self.dk, self.H)), "wk.weight": WeightSpec((self.dk, self.H)),
                    "wv.weight": WeightSpec((self.dv, self.H)), "wo.weight": WeightSpec((self.H, self.dv))}

        def kv_request(self):
            return KVRequest(1, self.dk, None, v_head_dim=self.dv)

        def load(self, tensors, compute_dtype):
            self.w = {k: v.float() for k, v in tensors.items()}

        def forward(self, ctx, run, y, x):
            keys, values = run.kv_group.keys(run.kv_layer), run.kv_group.values_t(run.kv_layer)
            table = ctx.tables[run.kv_group_index].tolist()
            cu, pos = ctx.host["cu"], ctx.row_pos.tolist()
            y = y.float()
            q, k, v = y @ self.w["wq.weight"].t(), y @ self.w["wk.weight"].t(), y @ self.w["wv.weight"].t()
            for b in range(ctx.n_seqs):
                for r in range(int(cu[b]), int(cu[b + 1])):
                    p = pos[r]
                    keys[table[b][p // PAGE], 0, p % PAGE] = k[r]
                    values[table[b][p // PAGE], 0, :, p % PAGE] = v[r]
                    ks = torch.stack([keys[table[b][j // PAGE], 0, j % PAGE] for j in range(p + 1)])
                    vs = torch.stack([values[table[b][j // PAGE], 0, :, j % PAGE] for j in range(p + 1)])
                    a = torch.softmax(ks @ q[r] / math.sqrt(self.dk), 0)
                    x[r] += (a @ vs) @ self.w["wo.weight"].t()

    register_part("mixer", "wide_values", WideValues)
    try:
        norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-5})
        layers = [LayerSpec(prefix=f"model.layers.{i}.", mixer=PartSpec("wide_values", {"hidden_size": H, "key_dim": dk, "value_dim": dv}),
                            ffn=PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I}), mixer_norm=norm, ffn_norm=norm)
                  for i in range(2)]
        spec = _toy_model(layers, H, V)
        w = random_tensors(spec.weight_specs(), seed=14, std=0.3, dtype=torch.float32)
        model = Model(spec, None, torch.float32, DEV)
        model.load_weights(TensorDict(w))
        eng = Engine(model, max_tokens=64 * 6, max_slots=3)
        (group,) = eng.cache.groups
        assert group.keys(1).shape[1:] == (1, PAGE, dk) and group.values_t(1).shape[1:] == (1, dv, PAGE)
        assert group.storage.shape[-1] == PAGE * (dk + dv)
        group.storage.fill_(float("nan"))

        def plain_forward(ids):
            wd = {k_: v_.double() for k_, v_ in w.items()}
            T = len(ids)
            x = wd["model.embed_tokens.weight"][ids]
            for i in range(2):
                p = f"model.layers.{i}."
                y = plain.rmsnorm(x, wd[p + "input_layernorm.weight"], 1e-5)
                q, k, v = (plain.linear(y, wd[p + n + ".weight"]) for n in ("wq", "wk", "wv"))
                s = (q @ k.t()) / math.sqrt(dk)
                s = s.masked_fill(~plain.visible(torch.arange(T), None), float("-inf"))
                x = x + plain.linear(plain.softmax(s) @ v, wd[p + "wo.weight"])
                x = x + plain.swiglu(plain.rmsnorm(x, wd[p + "post_attention_layernorm.weight"], 1e-5), wd, p)
            return plain.linear(plain.rmsnorm(x, wd["model.norm.weight"], 1e-5), wd["lm_head.weight"])

        g = torch.Generator().manual_seed(15)
        a, b = (torch.randint(0, V, (n,), generator=g).tolist() for n in (70, 9))      # the first crosses a page
        wa, wb = plain_forward(a), plain_forward(b)
        sa, sb = eng.alloc(), eng.alloc()
        lg = eng.step([SeqInput(sa, a[:60], list(range(60))), SeqInput(sb, b[:4], list(range(4)))]).clone()
        got_a, got_b = [lg[:60]], [lg[60:]]
        for t in range(5):
            lg = eng.step([SeqInput(sa, [a[60 + t]], [0]), SeqInput(sb, [b[4 + t]], [0])]).clone()
            got_a.append(lg[:1]); got_b.append(lg[1:])
        eng.free(sb)
        got_a.append(eng.step([SeqInput(sa, a[65:], list(range(5)))]).clone())
        eng.free(sa)
        assert rel_err(torch.cat(got_a), wa) < 1e-5 and rel_err(torch.cat(got_b), wb) < 1e-5
        eng.close()
    finally:
        unregister_part("mixer", "wide_values")


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [32, 40])         # on the matrix cores, and on the plain kernels (no multiple of 16)
def test_attention_part_with_a_scale_of_its_own(dt, d):
    """The factor on the scores is a parameter of the mixer (default 1/sqrt(head size)) that reaches all
    three attention kernels: whole rows (prefill), single tokens (decode), and the plain kernel.  The
    factor here is six times the default one, so that taking the default shows far above the tolerance."""
    from torchless_rs_amd.cache import Cache
    from torchless_rs_amd.engine import SeqInput
    from torchless_rs_amd.parts import PartSpec, RunBinding, make_part
    from torchless_rs_amd.parts.base import flush_pending
    H, nq, nkv, n, scale = 48, 4, 2, 70, 6.0 / math.sqrt(d)
    mixer = make_part("mixer", PartSpec("attention", {
        "hidden_size": H, "n_heads": nq, "n_kv_heads": nkv, "head_dim": d, "window": None, "scale": scale,
        "position": PartSpec("rotary", {"head_dim": d, "theta": 300.0})}))
    assert make_part("mixer", PartSpec("attention", {"hidden_size": H, "n_heads": nq, "n_kv_heads": nkv, "head_dim": d,
                                                     "position": PartSpec("none", {})})).scale == 1 / math.sqrt(d)
    w = {"self_attn.q_proj.weight": rnd(nq * d, H, seed=1, scale=0.3, dtype=DT[dt]),
         "self_attn.k_proj.weight": rnd(nkv * d, H, seed=2, scale=0.3, dtype=DT[dt]),
         "self_attn.v_proj.weight": rnd(nkv * d, H, seed=3, scale=0.3, dtype=DT[dt]),
         "self_attn.o_proj.weight": rnd(H, nq * d, seed=4, scale=0.3, dtype=DT[dt])}
    mixer.load({k: v.to(DEV) for k, v in w.items()}, DT[dt])
    y = rnd(n, H, seed=9, dtype=DT[dt])
    wd = {k: v.double() for k, v in w.items()}
    pos = torch.arange(n)
    q = plain.rope(plain.linear(y.double(), wd["self_attn.q_proj.weight"]).view(n, nq, d), pos, 300.0)
    k = plain.rope(plain.linear(y.double(), wd["self_attn.k_proj.weight"]).view(n, nkv, d), pos, 300.0)
    v = plain.linear(y.double(), wd["self_attn.v_proj.weight"]).view(n, nkv, d)
    want = plain.linear(plain.attention_core(q, k, v, pos, None, scale=scale).reshape(n, nq * d), wd["self_attn.o_proj.weight"])
    default = plain.linear(plain.attention_core(q, k, v, pos, None).reshape(n, nq * d), wd["self_attn.o_proj.weight"])
    assert rel_err(default, want) > 0.1
    # scores six times as large cost float32 more than the parts' usual tolerance allows for: the plain
    # formulas run in float32 say how much, and the engine's float32 path is held to twice that
    f = lambda t: t.float()
    w32 = {k_: f(v_) for k_, v_ in w.items()}
    q32 = plain.rope(plain.linear(f(y), w32["self_attn.q_proj.weight"]).view(n, nq, d), pos, 300.0)
    k32 = plain.rope(plain.linear(f(y), w32["self_attn.k_proj.weight"]).view(n, nkv, d), pos, 300.0)
    v32 = plain.linear(f(y), w32["self_attn.v_proj.weight"]).view(n, nkv, d)
    cost = rel_err(plain.linear(plain.attention_core(q32, k32, v32, pos, None, scale=scale).reshape(n, nq * d),
                                w32["self_attn.o_proj.weight"]), want)
    if dt == "bfloat16":
        # ... and amplify the rounding of q and k to bfloat16 sixfold, which is the format's doing: the
        # bfloat16 path is held to the plain formulas on q, k and v rounded as it stores them
        r = plain.to_bf16
        want = plain.linear(plain.attention_core(r(q), r(k), r(v), pos, None, scale=scale).reshape(n, nq * d),
                            wd["self_attn.o_proj.weight"])
    cache = Cache({0: mixer.kv_request()}, {}, 64 * 3, DT[dt], DEV, 1)
    cache.groups[0].storage.fill_(float("nan"))
    run = RunBinding(index=0, kv_group=cache.groups[0], kv_group_index=0, kv_layer=0, kv_source=0)
    s = cache.alloc_slot()
    got = []
    for rows in [40] + [1] * 30:
        o = sum(g.shape[0] for g in got)
        ctx = context(cache, [SeqInput(s, [0] * rows, [])], DT[dt])
        x = torch.zeros(rows, H, device=DEV)
        mixer.forward(ctx, run, y[o:o + rows].to(DEV), x)
        flush_pending(ctx, x)
        cache.commit([(s, rows)])
        got.append(x.clone())
    assert rel_err(torch.cat(got), want) < (max(PTOL[dt], 2 * cost) if dt == "float32" else PTOL[dt])


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_a_block_of_another_arrangement_gets_the_split_norms_from_the_helpers(dt):
    """A layer with three norms and two feed-forwards, x += mixer(n1 x); x += ffn(n2 x); x += ffn_b(n3 x),
    defined here as a block part around the framework's parts with the three helpers of parts/base
    (`read_through_norm`, `expect_norm`, `part_done`).  In bfloat16 single-token steps its norms then run
    cut in two around the products like those of the framework's own block: no norm kernel inside or
    between layers (counted), and the logits are those of the plain composition."""
    from torchless_rs_amd.engine import Engine, SeqInput
    from torchless_rs_amd.engine.model import Model
    from torchless_rs_amd.kernels import ops
    from torchless_rs_amd.parts import LayerSpec, Part, PartSpec, make_part, register_part, unregister_part
    from torchless_rs_amd.parts.base import expect_norm, part_done, read_through_norm, splittable_entry
    from torchless_rs_amd.weights import TensorDict, random_tensors
    H, V, I, Ib, nq, nkv, d, L, eps = 128, 80, 192, 96, 4, 2, 32, 2, 1e-5

    class ThreeNorms(Part):
        def __init__(self, layer, ffn_b, norm_b):
            self.mixer, self.ffn = make_part("mixer", layer.mixer), make_part("ffn", layer.ffn)
            self.n1, self.n2 = make_part("norm", layer.mixer_norm), make_part("norm", layer.ffn_norm)
            self.ffn_b, self.n3 = make_part("ffn", ffn_b), make_part("norm", norm_b)
            self.parts = (self.mixer, self.ffn, self.ffn_b, self.n1, self.n2, self.n3)
            self.graph_safe = all(p.graph_safe for p in self.parts)

        def may_capture(self, n_rows):
            return all(p.may_capture(n_rows) for p in self.parts)

        def weight_specs(self):
            out = {}
            for name, norm in (("ln_a.", self.n1), ("ln_b.", self.n2), ("ln_c.", self.n3)):
                out.update({name + k: v for k, v in norm.weight_specs().items()})
            for part in (self.mixer, self.ffn, self.ffn_b):
                out.update(part.weight_specs())
            return out

        def load(self, tensors, compute_dtype):
            for name, norm in (("ln_a.", self.n1), ("ln_b.", self.n2), ("ln_c.", self.n3)):
                norm.load({k[len(name):]: v for k, v in tensors.items() if k.startswith(name)}, compute_dtype)
            for part in (self.mixer, self.ffn, self.ffn_b):
                part.load(tensors, compute_dtype)

        def entry_norm(self):
            return splittable_entry(self.n1, self.mixer)

        def forward(self, ctx, run, x, norm_after=None):
            y = ctx.workspace.get("block_y", tuple(x.shape), ctx.dtype)
            y1 = read_through_norm(ctx, self.n1, x, y)
            expect_norm(ctx, self.mixer, self.n2, self.ffn)
            self.mixer.forward(ctx, run, y1, x)
            part_done(ctx, self.mixer)
            y2 = read_through_norm(ctx, self.n2, x, y)
            expect_norm(ctx, self.ffn, self.n3, self.ffn_b)
            self.ffn.forward(ctx, y2, x)
            part_done(ctx, self.ffn)
            y3 = read_through_norm(ctx, self.n3, x, y)
            expect_norm(ctx, self.ffn_b, norm_after)
            self.ffn_b.forward(ctx, y3, x)
            part_done(ctx, self.ffn_b)

    register_part("block", "three_norms", ThreeNorms)
    calls = []
    real = {name: getattr(ops, name) for name in ("rmsnorm", "add_rmsnorm")}
    try:
        norm = PartSpec("rmsnorm", {"size": H, "eps": eps})
        block = PartSpec("three_norms", {"ffn_b": PartSpec("swiglu", {"hidden_size": H, "intermediate_size": Ib, "prefix": "mlp_b."}),
                                         "norm_b": norm})
        layers = [LayerSpec(prefix=f"model.layers.{i}.",
                            mixer=PartSpec("attention", {"hidden_size": H, "n_heads": nq, "n_kv_heads": nkv, "head_dim": d,
                                                         "window": 24, "position": PartSpec("rotary", {"head_dim": d, "theta": 100.0})}),
                            ffn=PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I}),
                            mixer_norm=norm, ffn_norm=norm, block=block) for i in range(L)]
        spec = _toy_model(layers, H, V, eps)
        assert "model.layers.1.ln_c.weight" in spec.weight_specs() and "model.layers.1.mlp_b.down_proj.weight" in spec.weight_specs()
        w = random_tensors(spec.weight_specs(), seed=31, std=0.08, norm_std=0.1, dtype=torch.bfloat16)
        model = Model(spec, None, DT[dt], DEV)
        model.load_weights(TensorDict(w))
        eng = Engine(model, max_tokens=64 * 4, use_graphs=False)

        def plain_forward(ids):
            wd = {k: v.double() for k, v in w.items()}
            pos = torch.arange(len(ids))
            cfg = {"num_attention_heads": nq, "num_key_value_heads": nkv, "head_dim": d, "hidden_size": H,
                   "rope_theta": 100.0, "sliding_window": 24}
            x = wd["model.embed_tokens.weight"][ids]
            for i in range(L):
                p = f"model.layers.{i}."
                x = x + plain.attention(plain.rmsnorm(x, wd[p + "ln_a.weight"], eps), wd, p, cfg, pos)
                x = x + plain.swiglu(plain.rmsnorm(x, wd[p + "ln_b.weight"], eps), wd, p)
                wb = {p + "mlp." + k: wd[p + "mlp_b." + k] for k in ("gate_proj.weight", "up_proj.weight", "down_proj.weight")}
                x = x + plain.swiglu(plain.rmsnorm(x, wd[p + "ln_c.weight"], eps), wb, p)
            return plain.linear(plain.rmsnorm(x, wd["model.norm.weight"], eps), wd["lm_head.weight"])

        g = torch.Generator().manual_seed(32)
        seqs = [torch.randint(0, V, (n,), generator=g).tolist() for n in (50, 7)]
        wants = [plain_forward(s) for s in seqs]
        tol = {"float32": 2e-5, "bfloat16": 3e-2}[dt]
        slots = [eng.alloc() for _ in seqs]
        heads = [30, 3]
        lg = eng.step([SeqInput(sl, s[:h], list(range(h))) for sl, s, h in zip(slots, seqs, heads)]).clone()
        assert rel_err(lg[:30], wants[0][:30]) < tol and rel_err(lg[30:], wants[1][:3]) < tol
        for name in real:
            setattr(ops, name, lambda *a, _n=name, **k: (calls.append(_n), real[_n](*a, **k))[1])
        for t in range(20):
            live = [i for i in range(2) if heads[i] + t < len(seqs[i])]
            calls.clear()
            lg = eng.step([SeqInput(slots[i], [seqs[i][heads[i] + t]], [0]) for i in live]).clone()
            for r, i in enumerate(live):
                assert rel_err(lg[r:r + 1], wants[i][heads[i] + t:heads[i] + t + 1]) < tol, (t, i)
            if dt == "bfloat16":
                # the first norm of the first layer (behind the embedding, which is no product) and the
                # last norm on the gathered rows: the 3 L - 1 norms between them ran inside the products
                assert calls == ["rmsnorm", "rmsnorm"], calls
            else:
                assert len(calls) == 3 * L + 1
        eng.close()
    finally:
        for name, fn in real.items():
            setattr(ops, name, fn)
        unregister_part("block", "three_norms")
