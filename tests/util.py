"""Shared by the tests: tiny configurations, model folders in temporary
places, and the measure by which logits are compared."""
from __future__ import annotations

import json
import os

import torch

# Two tiny configurations that differ in every size and option, and a third
# whose window is no multiple of the cache's page and is exceeded many times.
TINY_A = {
    "architectures": ["MistralForCausalLM"], "model_type": "mistral",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "intermediate_size": 160, "vocab_size": 256, "rope_theta": 10000.0, "sliding_window": 8,
    "rms_norm_eps": 1e-5, "max_position_embeddings": 64, "tie_word_embeddings": False,
    "hidden_act": "silu",
}
TINY_B = {
    "architectures": ["MistralForCausalLM"], "model_type": "mistral",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 6, "num_key_value_heads": 1,
    "head_dim": 32, "intermediate_size": 224, "vocab_size": 384, "rope_theta": 1000000.0,
    "sliding_window": None, "rms_norm_eps": 1e-6, "max_position_embeddings": 128,
    "tie_word_embeddings": False, "hidden_act": "silu",
}
TINY_C = {
    "architectures": ["MistralForCausalLM"], "model_type": "mistral",
    "num_hidden_layers": 2, "hidden_size": 80, "num_attention_heads": 5, "num_key_value_heads": 5,
    "head_dim": 48, "intermediate_size": 112, "vocab_size": 300, "rope_theta": 500.0,
    "sliding_window": 70, "rms_norm_eps": 1e-4, "max_position_embeddings": 512,
    "tie_word_embeddings": False, "hidden_act": "silu",
}
INIT = {"A": dict(seed=0, std=0.02, norm_std=0.0), "B": dict(seed=2, std=0.05, norm_std=0.1),
        "C": dict(seed=9, std=0.06, norm_std=0.2)}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C}

# Largest difference of logits as a share of the largest logit.  Fixed before
# the first run: float32 leaves only the order of summation, bfloat16 rounds
# activations to 8 bits of mantissa at each product's input.
TOL = {"float32": 2e-5, "bfloat16": 3e-2}


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    got, want = got.double().cpu(), want.double().cpu()
    assert got.shape == want.shape, (got.shape, want.shape)
    return float((got - want).abs().max() / (want.abs().max() + 1e-30))


def rms_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """Root mean square of the difference as a share of the root mean square of `want`: a far
    steadier measure of rounding noise than the largest difference."""
    got, want = got.double().cpu(), want.double().cpu()
    assert got.shape == want.shape, (got.shape, want.shape)
    return float(((got - want) ** 2).mean().sqrt() / ((want ** 2).mean().sqrt() + 1e-30))


def within_the_format(got, rounded, exact):
    """Is the engine's bfloat16 result `got` as far from the float64 logits `exact` as the format
    makes it, and no further?  `rounded`: the plain implementation with the same roundings.
    (Lists of tensors, one a request.)  The root mean square over all logits may exceed the plain
    implementation's by a quarter, the largest difference (the maximum of as many draws, which
    scatters more, most at small widths) by a factor of two.  Returns (ok, the four numbers)."""
    g, r, x = torch.cat(list(got)), torch.cat(list(rounded)), torch.cat(list(exact))
    rms, rms_cost = rms_err(g, x), rms_err(r, x)
    top, top_cost = rel_err(g, x), rel_err(r, x)
    ok = rms < 1.25 * rms_cost + 1e-4 and top < 2.0 * top_cost + 1e-3
    return ok, dict(rms=rms, rms_of_roundings=rms_cost, largest=top, largest_of_roundings=top_cost)


def held_to_the_format(dtype, got, exact, w, cfg, ids, step_rows, what=""):
    """The stricter of the measures for a schedule's logits (lists, one tensor a request): float32
    within the fixed tolerance; bfloat16 within what the format costs the plain implementation that
    rounds where the engine does, on these very requests cut into these very steps (`step_rows`:
    for every position the number of rows of the step it came in), so that a stale or misplaced row
    of little weight, far below the fixed tolerance, still shows."""
    import plain_mistral as plain
    if dtype == "float32":
        worst = max(rel_err(g, x) for g, x in zip(got, exact))
        assert worst < TOL[dtype], (what, worst)
        return
    rounded = [plain.forward_rounded(w, cfg, p, r) for p, r in zip(ids, step_rows)]
    ok, numbers = within_the_format(got, rounded, exact)
    assert ok, (what, numbers)


def make_model_dir(tmp, name: str, dtype=torch.bfloat16) -> str:
    from torchless_rs_amd import write_random_model
    d = os.path.join(str(tmp), f"tiny_{name}_{str(dtype).split('.')[-1]}")
    if not os.path.isdir(d):
        write_random_model(d, dict(CONFIGS[name]), dtype=dtype, **INIT[name])
    return d


def read_model_dir(d: str):
    """config dict and tensors by name, read with the test's own reader."""
    import struct
    with open(os.path.join(d, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with open(os.path.join(d, "model.safetensors"), "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    dts = {"F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16}
    for k, e in header.items():
        if k == "__metadata__":
            continue
        b, en = e["data_offsets"]
        tensors[k] = torch.frombuffer(bytearray(data[b:en]), dtype=dts[e["dtype"]]).view(e["shape"]).clone()
    return cfg, tensors


def prompts(vocab: int, lengths, seed: int):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (n,), generator=g).tolist() for n in lengths]
