"""A plain, slow Mistral: whole sequences, no cache, one function for each part.

Written from the formulas of the reference (paths are relative to the
reference's root).  It shares no code with the engine: it takes a dict of
tensors by their checkpoint names and a dict of the config.json keys, and
works on the CPU in the dtype it is asked for (float64 by default, so that
it can serve as ground truth for the engine's float32 path).
"""
from __future__ import annotations

import math

import torch


def embedding(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """Row copy, no scaling.  src/model/modules/embedding.rs:15-21"""
    return table[ids.long().to(table.device)]


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * w; eps inside the root, weight used as it
    is.  src/kernels/mod.rs:558-568"""
    ss = (x * x).sum(dim=-1, keepdim=True)
    rms = torch.sqrt(ss / x.shape[-1] + eps)
    return (x / rms) * weight


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """out[r] = sum_c W[r, c] x[c], no bias.  src/loader/parameters.rs:551-594"""
    return x @ w.t()


def rope_inv_freq(head_dim: int, theta: float, dtype=torch.float64, device=None) -> torch.Tensor:
    """inv_freq[i] = 1 / theta^(i / (d/2)).  src/kernels/mod.rs:572-579"""
    half = head_dim // 2
    i = torch.arange(half, dtype=dtype, device=device)
    return 1.0 / torch.pow(torch.tensor(theta, dtype=dtype, device=device), i / half)


def rope(x: torch.Tensor, positions: torch.Tensor, theta: float) -> torch.Tensor:
    """Half-split rotation of x[T, heads, d] by the angle pos * inv_freq:
    x'_i = x_i c_i - x_{i+d/2} s_i ; x'_{i+d/2} = x_i s_i + x_{i+d/2} c_i.
    src/kernels/mod.rs:582-608"""
    d = x.shape[-1]
    half = d // 2
    inv = rope_inv_freq(d, theta, x.dtype, x.device)
    ang = positions.to(x.dtype)[:, None] * inv[None, :]          # [T, d/2]
    c = torch.cos(ang)[:, None, :]
    s = torch.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:]
    return torch.cat([a * c - b * s, a * s + b * c], dim=-1)


def rope_variant(x: torch.Tensor, positions: torch.Tensor, theta: float, rotary_dim: int,
                 interleaved: bool) -> torch.Tensor:
    """Not the reference's rotation, but the family around it that the tests' toy position
    encodings use: only the first `rotary_dim` channels of a head are rotated (frequencies
    1 / theta^(i / (rotary_dim/2))), in pairs (i, i + rotary_dim/2), or (2i, 2i+1) when
    `interleaved`; the other channels pass through.  With rotary_dim = d and halves it is `rope`."""
    if rotary_dim == 0:
        return x.clone()
    head, rest = x[..., :rotary_dim], x[..., rotary_dim:]
    if interleaved:                       # bring the pairs (2i, 2i+1) to (i, i + r/2), rotate, bring them back
        order = torch.cat([torch.arange(0, rotary_dim, 2), torch.arange(1, rotary_dim, 2)]).to(x.device)
        back = torch.argsort(order)
        head = rope(head[..., order], positions, theta)[..., back]
    else:
        head = rope(head, positions, theta)
    return torch.cat([head, rest], dim=-1)


def visible(positions: torch.Tensor, window) -> torch.Tensor:
    """mask[p, j]: key j visible to the query at p iff j <= p, and with a
    window W, not (p >= W and j < p - W + 1).  Causality:
    src/model/modules/attention.rs:90 ; window: src/model/models/gpt_oss.rs:168-175"""
    p = positions[:, None]
    j = positions[None, :]
    m = j <= p
    if window:
        m &= ~((p >= window) & (j < p - window + 1))
    return m


def softmax(s: torch.Tensor) -> torch.Tensor:
    """exp(s - max) / sum.  src/kernels/mod.rs:538-543"""
    m = s.max(dim=-1, keepdim=True).values
    e = torch.exp(s - m)
    return e / e.sum(dim=-1, keepdim=True)


def attention_core(q, k, v, positions, window, scale=None) -> torch.Tensor:
    """q[T,nq,d], k,v[T,nkv,d] (already rotated) -> ctx[T,nq,d].
    Query head h reads KV head h // (nq/nkv); score = (k.q) * 1/sqrt(d),
    scale applied after the dot; softmax over the visible keys; weighted sum
    of the value rows.  src/model/modules/attention.rs:82-121 ;
    src/kernels/mod.rs:494-526"""
    T, nq, d = q.shape
    nkv = k.shape[1]
    g = nq // nkv
    if scale is None:           # (another factor: only for parts that tests build with one)
        scale = 1.0 / math.sqrt(d)
    mask = visible(positions, window)
    out = torch.empty_like(q)
    for h in range(nq):
        kvh = h // g
        s = (q[:, h, :] @ k[:, kvh, :].t()) * scale               # [T, T]
        s = s.masked_fill(~mask, float("-inf"))
        p = softmax(s)
        out[:, h, :] = p @ v[:, kvh, :]
    return out


def attention(x, w, prefix, cfg, positions) -> torch.Tensor:
    """Projections, rotation of q and k, attention, output projection.
    src/model/modules/attention.rs:42-135"""
    nq = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads") or nq
    d = cfg.get("head_dim") or cfg["hidden_size"] // nq
    T = x.shape[0]
    q = linear(x, w[prefix + "self_attn.q_proj.weight"]).view(T, nq, d)
    k = linear(x, w[prefix + "self_attn.k_proj.weight"]).view(T, nkv, d)
    v = linear(x, w[prefix + "self_attn.v_proj.weight"]).view(T, nkv, d)
    theta = cfg.get("rope_theta", 10000.0)
    q = rope(q, positions, theta)
    k = rope(k, positions, theta)
    ctx = attention_core(q, k, v, positions, cfg.get("sliding_window"))
    return linear(ctx.reshape(T, nq * d), w[prefix + "self_attn.o_proj.weight"])


def silu(x: torch.Tensor) -> torch.Tensor:
    """x / (1 + exp(-x)).  src/kernels/mod.rs:546-548"""
    return x / (1.0 + torch.exp(-x))


def swiglu(x, w, prefix) -> torch.Tensor:
    """down( silu(gate x) * (up x) ).  src/model/modules/mlp.rs:23-45"""
    g = linear(x, w[prefix + "mlp.gate_proj.weight"])
    u = linear(x, w[prefix + "mlp.up_proj.weight"])
    return linear(silu(g) * u, w[prefix + "mlp.down_proj.weight"])


def block(x, w, prefix, cfg, positions) -> torch.Tensor:
    """x + attn(norm1(x)), then x + mlp(norm2(x)).
    src/model/modules/layer.rs:28-56"""
    eps = cfg["rms_norm_eps"]
    x = x + attention(rmsnorm(x, w[prefix + "input_layernorm.weight"], eps),
                      w, prefix, cfg, positions)
    x = x + swiglu(rmsnorm(x, w[prefix + "post_attention_layernorm.weight"], eps),
                   w, prefix)
    return x


def forward_many(weights, cfg: dict, many_ids, dtype=torch.float64):
    """Logits [T, V] of each of several whole sequences.  `weights` is read name by name, a
    layer at a time (so a large model need not be held in `dtype` at once), and the arithmetic
    runs where its tensors lie.  src/model/mod.rs:430-447"""
    take = lambda name: weights[name].to(dtype)
    table = take("model.embed_tokens.weight")
    xs, positions = [], []
    for ids in many_ids:
        ids = torch.as_tensor(ids)
        xs.append(embedding(table, ids))
        positions.append(torch.arange(ids.shape[0], device=table.device))
    for i in range(cfg["num_hidden_layers"]):
        prefix = f"model.layers.{i}."
        w = {prefix + n: take(prefix + n) for n in LAYER_TENSORS}
        xs = [block(x, w, prefix, cfg, pos) for x, pos in zip(xs, positions)]
    norm = take("model.norm.weight")
    head = table if cfg.get("tie_word_embeddings") else take("lm_head.weight")
    return [linear(rmsnorm(x, norm, cfg["rms_norm_eps"]), head) for x in xs]


LAYER_TENSORS = ("input_layernorm.weight", "post_attention_layernorm.weight", "self_attn.q_proj.weight",
                 "self_attn.k_proj.weight", "self_attn.v_proj.weight", "self_attn.o_proj.weight",
                 "mlp.gate_proj.weight", "mlp.up_proj.weight", "mlp.down_proj.weight")


def forward(weights: dict, cfg: dict, ids, dtype=torch.float64) -> torch.Tensor:
    """Logits [T, V] of one whole sequence.  src/model/mod.rs:430-447"""
    return forward_many(weights, cfg, [ids], dtype)[0]


# --- sampling --------------------------------------------------------------

def greedy(logits: torch.Tensor) -> int:
    """Index of the largest logit; of equal maxima the last, as Rust's
    `max_by` keeps it.  src/sampler/mod.rs:60-68"""
    best, idx = None, 0
    for i, v in enumerate(logits.tolist()):
        if best is None or v >= best:
            best, idx = v, i
    return idx


def top_k_filter(z: torch.Tensor, k: int) -> torch.Tensor:
    """Keep the k largest, others to -inf.  On ties at the threshold: every
    value above it is kept and then values equal to it, in index order, until
    k are kept.  src/sampler/mod.rs:93-119 (the rule is the one its comment at
    :107-109 states; its loop at :110-117 would also drop larger values that
    come after k ties, which no caller can want)."""
    z = z.clone()
    thr = torch.sort(z, descending=True).values[min(k, z.numel()) - 1]
    room = k - int((z > thr).sum())
    for i in range(z.numel()):
        if z[i] < thr:
            z[i] = float("-inf")
        elif z[i] == thr:
            if room > 0:
                room -= 1
            else:
                z[i] = float("-inf")
    return z


def top_p_filter(p: torch.Tensor, top_p: float) -> torch.Tensor:
    """Sort descending, keep the shortest prefix whose sum is >= top_p, zero the
    rest, divide by the new sum.  src/sampler/mod.rs:144-170"""
    p = p.clone()
    order = torch.argsort(p, descending=True, stable=True)
    cum, cutoff = 0.0, p.numel()
    for n, i in enumerate(order.tolist()):
        cum += float(p[i])
        if cum >= top_p:
            cutoff = n + 1
            break
    p[order[cutoff:]] = 0.0
    s = p.sum()
    if s > 0:
        p = p / s
    return p


def sample_distribution(logits, temperature, top_k=None, top_p=None) -> torch.Tensor:
    """Probabilities that the draw is made from: temperature, top-k, softmax,
    top-p, in this order.  src/sampler/mod.rs:194-222"""
    z = logits.to(torch.float64) / temperature
    if top_k is not None and 0 < top_k < z.numel():
        z = top_k_filter(z, top_k)
    p = softmax(z)
    if top_p is not None and 0.0 < top_p < 1.0:
        p = top_p_filter(p, top_p)
    return p


def draw(p: torch.Tensor, r: float) -> int:
    """First index whose running sum reaches r, else the last index.
    src/sampler/mod.rs:225-238"""
    cum = 0.0
    for i, v in enumerate(p.tolist()):
        cum += v
        if cum >= r:
            return i
    return p.numel() - 1


def sample(logits, r, temperature, top_k=None, top_p=None) -> int:
    """src/sampler/mod.rs:194-222"""
    if temperature <= 0.0:
        return greedy(logits)
    return draw(sample_distribution(logits, temperature, top_k, top_p), r)


def generate_greedy(weights, cfg, prompt, max_tokens, stop_ids=(), dtype=torch.float64):
    """Feed the prompt, then the argmax of the last row again and again; a stop
    id ends the sequence and is not part of the output.
    src/sampler/mod.rs:269-305 ; src/main.rs:557-597"""
    ids = list(prompt)
    out = []
    for _ in range(max_tokens):
        logits = forward(weights, cfg, ids, dtype)[-1]
        t = greedy(logits)
        if t in stop_ids:
            return out, "stop"
        out.append(t)
        ids.append(t)
    return out, "length"


# --- the same model with the engine's bfloat16 roundings ------------------------

def to_bf16(t: torch.Tensor) -> torch.Tensor:
    """Round as a float32 value is rounded when it is stored in bfloat16 (nearest even)."""
    return t.to(torch.float32).to(torch.bfloat16).to(t.dtype)


def forward_rounded(weights: dict, cfg: dict, ids, step_rows, library_rows="auto", matrix_core_heads=None,
                    ffn_norm_in_halves=True) -> torch.Tensor:
    """`forward` in float64 with a rounding to bfloat16 at every place where the engine's
    bfloat16 path stores one, and nowhere else: the output of a norm, q and k after the rotation,
    v, the probabilities as they enter the product with the values (their sum is taken
    unrounded), the attention's output, silu(gate) * up.  The residual stream, all sums and the
    softmax are not rounded (the engine keeps them in float32).

    Two roundings depend on how many rows the step had that a row came in (`step_rows[t]`):
    * up to 16 rows, a norm that follows a product is cut in two around the products next to
      it: bfloat16(x * w) goes into the product and the results are multiplied by
      rsqrt(mean(x^2) + eps) (all but the first layer's first norm and the last norm);
    * above `library_rows` rows, gate and up are themselves stored in bfloat16 before the
      activation (None: never; "auto": the engine's rule, 128 rows where the hidden size is a multiple
      of 128, else 64).
    (The kernels round a probability against the running maximum of the keys seen so far and
    scale float32 sums afterwards; here it is rounded against the row's maximum: another
    realisation of the same rounding.)
    `matrix_core_heads` (default: the head size is a multiple of 16): with other head sizes the
    engine's attention runs in its plain kernels, which keep the probabilities in float32, and
    its q|k|v product cannot take a norm in halves, so the norm before it is stored whole.
    `ffn_norm_in_halves`: false where the output projection or gate|up cannot do the halves
    (heads x head size no multiple of 8, an inner size no multiple of 32).
    The formulas are those of the functions above; only the roundings are added."""
    f64 = torch.float64
    take = lambda name: weights[name].to(f64)            # a layer at a time, where the tensors lie
    table = take("model.embed_tokens.weight")
    dev = table.device
    ids = torch.as_tensor(ids)
    T = ids.shape[0]
    step_rows = torch.as_tensor(step_rows, device=dev)
    if library_rows == "auto":
        library_rows = 128 if cfg["hidden_size"] % 128 == 0 else 64
    split = (step_rows <= 16)[:, None]
    pre_round = (step_rows > library_rows)[:, None] if library_rows else torch.zeros(T, 1, dtype=torch.bool, device=dev)
    positions = torch.arange(T, device=dev)
    eps = cfg["rms_norm_eps"]
    nq = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads") or nq
    d = cfg.get("head_dim") or cfg["hidden_size"] // nq
    theta = cfg.get("rope_theta", 10000.0)
    if matrix_core_heads is None:
        matrix_core_heads = d % 16 == 0
    round_p = to_bf16 if matrix_core_heads else (lambda t: t)

    def normed(x, weight, may_split):
        """(input of the products, factor on their results)"""
        whole = to_bf16(rmsnorm(x, weight, eps))
        if not may_split:
            return whole, torch.ones(T, 1, dtype=f64, device=dev)
        r = 1.0 / torch.sqrt((x * x).sum(-1, keepdim=True) / x.shape[-1] + eps)
        return torch.where(split, to_bf16(x * weight), whole), torch.where(split, r, torch.ones_like(r))

    x = embedding(table, ids)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w = {p + n: take(p + n) for n in LAYER_TENSORS}
        y, r = normed(x, w[p + "input_layernorm.weight"], i > 0 and matrix_core_heads)
        q = (linear(y, w[p + "self_attn.q_proj.weight"]) * r).view(T, nq, d)
        k = (linear(y, w[p + "self_attn.k_proj.weight"]) * r).view(T, nkv, d)
        v = (linear(y, w[p + "self_attn.v_proj.weight"]) * r).view(T, nkv, d)
        q, k, v = to_bf16(rope(q, positions, theta)), to_bf16(rope(k, positions, theta)), to_bf16(v)
        mask = visible(positions, cfg.get("sliding_window"))
        ctx = torch.empty_like(q)
        for h in range(nq):
            kvh = h // (nq // nkv)
            s = (q[:, h, :] @ k[:, kvh, :].t()) * (1.0 / math.sqrt(d))
            s = s.masked_fill(~mask, float("-inf"))
            e = torch.exp(s - s.max(dim=-1, keepdim=True).values)
            ctx[:, h, :] = (round_p(e) @ v[:, kvh, :]) / e.sum(dim=-1, keepdim=True)
        x = x + linear(to_bf16(ctx).reshape(T, nq * d), w[p + "self_attn.o_proj.weight"])
        y, r = normed(x, w[p + "post_attention_layernorm.weight"], ffn_norm_in_halves)
        g = linear(y, w[p + "mlp.gate_proj.weight"]) * r
        u = linear(y, w[p + "mlp.up_proj.weight"]) * r
        g, u = torch.where(pre_round, to_bf16(g), g), torch.where(pre_round, to_bf16(u), u)
        x = x + linear(to_bf16(silu(g) * u), w[p + "mlp.down_proj.weight"])
    y = to_bf16(rmsnorm(x, take("model.norm.weight"), eps))
    return linear(y, table if cfg.get("tie_word_embeddings") else take("lm_head.weight"))
