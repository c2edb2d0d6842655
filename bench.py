"""Decode and prefill throughput of the Mistral-7B-v0.1 shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 8192] [--layers L]
                    [--shape 7b-v0.1|7b-v0.3|nemo-12b] [--only decode|prefill] [--prefill-tokens T]
                    [--no-points] [--no-tiled-copies]

One JSON line: decoded tokens a second of the default run (batch 8 at the
context length of the configuration), the prefill of one 2,048-token prompt,
the decode step's share of the HBM roofline, decoding at batch 1 and 64, and
what a plain read and a chain of MFMAs reach on the machine ("ceilings").
Weights are random (seeded), token ids synthetic.  The context is built by a
real prefill of synthetic prompts.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

HBM_PEAK_GBS = 8000.0                 # MI355X, published
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}

# Mistral-7B-v0.1 shape: the third configuration of the baseline, and the default
SHAPE = dict(num_hidden_layers=32, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
             head_dim=128, intermediate_size=14336, vocab_size=32000, rope_theta=10000.0,
             sliding_window=4096, rms_norm_eps=1e-5)
# the baseline's other shapes of the same architecture, for --shape
SHAPES = {
    "7b-v0.1": ("Mistral-7B-v0.1 shape", SHAPE),
    "7b-v0.3": ("Mistral-7B-v0.3 shape", dict(SHAPE, vocab_size=32768, rope_theta=1e6, sliding_window=None)),
    "nemo-12b": ("Mistral-NeMo-12B shape", dict(SHAPE, num_hidden_layers=40, hidden_size=5120, vocab_size=131072,
                                                 rope_theta=1e6, sliding_window=None)),
}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--shape", choices=sorted(SHAPES), default="7b-v0.1")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64")
    ap.add_argument("--no-tiled-copies", action="store_true",
                    help="keep no second copies of q|k|v, o and down in the layout that single-token steps stream")
    ap.add_argument("--only", choices=["prefill", "decode"], default=None,
                    help="measure one phase only and print its line to stderr (for profiling)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not served")
        return 2

    import torch
    from torchless_rs_amd import SamplingConfig, config_from_dict
    from torchless_rs_amd.engine import Engine, SeqInput, model_from_tensors
    from torchless_rs_amd.models import model_spec_for
    from torchless_rs_amd.sampling.sampler import Sampler
    from torchless_rs_amd.weights import random_tensors

    shape_name, shape = SHAPES[args.shape]
    if args.layers is None:
        args.layers = shape["num_hidden_layers"]
    cfgd = dict(shape, architectures=["MistralForCausalLM"], num_hidden_layers=args.layers)
    cfg = config_from_dict(cfgd)
    dev = "cuda:0"
    t0 = time.time()
    tensors = random_tensors(model_spec_for(cfg).weight_specs(), seed=5, std=0.02,
                             dtype=torch.bfloat16, device=dev)
    model = model_from_tensors(cfg, tensors, "bfloat16", dev, tiled_copies=not args.no_tiled_copies)
    del tensors
    torch.cuda.synchronize()
    resident_gib = round(torch.cuda.memory_allocated() / 2 ** 30, 2)     # weights and their tiled copies
    print(f"[bench] weights ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)

    L, H, I, V = args.layers, cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    nq, nkv, d, W = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.sliding_window
    per_layer = (nq + 2 * nkv) * d * H + H * nq * d + 3 * I * H
    weight_bytes = 2 * (L * per_layer + V * H)          # every matrix once; one embedding row is noise
    kv_per_token = 2 * nkv * d * 2 * L                  # K and V, bf16, all layers
    sampler = Sampler(SamplingConfig.greedy(), dev)
    gen = torch.Generator().manual_seed(11)

    def run_decode(batch: int, context: int, steps: int, warmup: int, engine=None):
        """Prefill `batch` prompts of `context - steps - warmup` tokens, then time `steps` decode
        steps (model step + greedy sampling)."""
        held = min(context, W) if W else context
        eng = engine or Engine(model, max_tokens=batch * (-(-held // 64) * 64 + 64), max_slots=batch)
        plen = max(1, context - steps - warmup - 1)
        slots = [eng.alloc() for _ in range(batch)]
        chunk = 2048
        for s in slots:                                  # prompt by prompt, in chunks
            ids = torch.randint(0, V, (plen,), generator=gen).tolist()
            for c0 in range(0, plen, chunk):
                part = ids[c0:c0 + chunk]
                last = c0 + chunk >= plen
                lg = eng.step([SeqInput(s, part, [len(part) - 1] if last else [])])
        first = sampler.sample(lg, [0], [0]) * batch
        lg = eng.step([SeqInput(s, [t], [0]) for s, t in zip(slots, first)])
        drawn = sampler.draw(lg, list(range(batch)), [0] * batch)
        entries = [SeqInput(s, [0], [0]) for s in slots]

        def one():
            # as the generation loop runs: the next step is launched with the drawn tokens still on
            # the device, then the host reads the tokens of the step before
            nonlocal drawn
            lg = eng.step(entries, device_tokens=drawn.device)
            ahead = sampler.draw(lg, list(range(batch)), [0] * batch)
            drawn.tokens()
            drawn = ahead

        for _ in range(warmup):
            one()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            one()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        ctx_mid = plen + warmup + steps // 2
        for s in slots:
            eng.free(s)
        return dt / steps, ctx_mid

    if args.only == "decode":
        sec, _ = run_decode(args.batch, args.context, args.steps, args.warmup)
        print(f"[bench] decode b{args.batch}: {args.batch / sec:.1f} tok/s, {sec * 1e3:.3f} ms/step",
              file=sys.stderr, flush=True)
        return 0

    # prefill of one prompt
    T = args.prefill_tokens
    eng = Engine(model, max_tokens=T + 64, max_slots=1)
    ids = torch.randint(0, V, (T,), generator=gen).tolist()
    pre_ms = []
    for it in range(2):
        s = eng.alloc()
        torch.cuda.synchronize()
        t = time.perf_counter()
        eng.step([SeqInput(s, ids, [T - 1])])
        torch.cuda.synchronize()
        pre_ms.append((time.perf_counter() - t) * 1e3)
        eng.free(s)
    del eng
    pre = min(pre_ms)
    attn_flops = sum(4 * nq * d * min(p + 1, W or (p + 1)) for p in range(T)) * L
    pre_flops = 2 * T * (L * per_layer) + 2 * V * H + attn_flops
    prefill = {"value": round(T / (pre / 1e3), 1), "tokens": T, "ms": round(pre, 3),
               "frac": round(pre_flops / (pre / 1e3) / (PEAK_TFLOPS["bf16"] * 1e12), 4)}
    print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)
    if args.only == "prefill":
        return 0

    sec, ctx_mid = run_decode(args.batch, args.context, args.steps, args.warmup)
    held = min(ctx_mid, W) if W else ctx_mid
    step_bytes = weight_bytes + args.batch * held * kv_per_token
    achieved = step_bytes / sec / 1e9
    value = args.batch / sec
    print(f"[bench] decode b{args.batch}: {value:.1f} tok/s, {sec * 1e3:.3f} ms/step", file=sys.stderr,
          flush=True)
    points = {}
    if not args.no_points:
        for b in (1, 64):
            s_b, _ = run_decode(b, args.context, max(8, args.steps // 2), 2)
            points[f"decode_b{b}"] = round(b / s_b, 1)
            print(f"[bench] decode b{b}: {b / s_b:.1f} tok/s", file=sys.stderr, flush=True)

    # what the simplest kernels get here: a plain read of 8 GiB, independent MFMAs on registers
    from torchless_rs_amd.kernels import ops as _ops
    del model
    torch.cuda.empty_cache()
    ceilings = _ops.measure_ceilings(dev)
    print(f"[bench] measured ceilings {ceilings}", file=sys.stderr, flush=True)
    ceilings["decode_frac_of_read"] = round(achieved / ceilings["hbm_read_GBs"], 4)
    ceilings["prefill_frac_of_mfma"] = round(pre_flops / (pre / 1e3) / (ceilings["mfma_bf16_TFLOPs"] * 1e12), 4)
    out = {
        "metric": f"decode tok/s at batch {args.batch} ({shape_name}), with prefill tok/s at "
                  f"{args.prefill_tokens:,} tokens",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic: random weights N(0,0.02) seed 5, uniform random token ids",
        "config": {"model": shape_name, "layers": L, "layers_of_config": shape["num_hidden_layers"],
                   "hidden_size": H, "heads": nq, "kv_heads": nkv, "head_dim": d,
                   "intermediate_size": I, "vocab_size": V, "sliding_window": W,
                   "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_norm_eps,
                   "global_batch": args.batch, "seq_len": args.context, "parallelism": "none",
                   "sampling": "greedy", "tiled_weight_copies": not args.no_tiled_copies,
                   "weights_resident_gib": resident_gib},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
        "ceilings": ceilings,
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
