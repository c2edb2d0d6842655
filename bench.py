"""Decode and prefill throughput of the Mistral-7B-v0.1 shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 8192] [--layers L]
                    [--shape 7b-v0.1|7b-v0.3|nemo-12b] [--only decode|prefill] [--prefill-tokens T]
                    [--no-points] [--no-kernels] [--no-workloads] [--no-tiled-copies]

One JSON line: decoded tokens a second of the default run (batch 8 at the
context length of the configuration), the prefill of one 2,048-token prompt,
the decode step's share of the HBM roofline, decoding at batch 1 and 64
("points"), the step's kernels one by one with their own shares of the HBM
roofline ("kernels"), the baseline's configurations as it words them, run
through the generation loop ("workloads"), and what a plain read and a chain
of MFMAs reach on the machine ("ceilings").  Weights are random (seeded),
token ids synthetic.  The context is built by a real prefill of synthetic
prompts.
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
    ap.add_argument("--no-kernels", action="store_true", help="skip the timing of the step's kernels one by one")
    ap.add_argument("--no-workloads", action="store_true", help="skip the baseline's configurations as it words them")
    ap.add_argument("--no-tiled-copies", action="store_true",
                    help="keep no second copies of q|k|v, o and down in the layout that single-token steps stream")
    ap.add_argument("--workload", choices=["baseline"], default="baseline",
                    help="the baseline's configurations as it words them (unequal prompt lengths drawn from a seed, "
                         "256/128/128 new tokens, temperature 0.7 for the NeMo shape) run through the generation "
                         "loop, under 'workloads' (the default; --no-workloads skips them)")
    ap.add_argument("--only", choices=["prefill", "decode", "pipes"], default=None,
                    help="measure one phase only and print its line to stderr (for profiling); pipes: whether a "
                         "SIMD's matrix and vector pipes overlap (ops.measure_pipes)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not served")
        return 2

    import torch
    if args.only == "pipes":
        from torchless_rs_amd.kernels import ops as _o
        print(json.dumps({"pipes_ns_per_iteration": _o.measure_pipes("cuda:0")}), flush=True)
        return 0
    from torchless_rs_amd import SamplingConfig, config_from_dict
    from torchless_rs_amd.engine import Engine, SeqInput, model_from_tensors
    from torchless_rs_amd.engine.generate import BatchRun
    from torchless_rs_amd.kernels.page import PAGE, round_up
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

    def run_decode(batch: int, context: int, steps: int, warmup: int, engine=None, then=None):
        """Prefill `batch` prompts of `context - steps - warmup` tokens, then time `steps` decode
        steps (model step + greedy sampling).  `then(engine, slots)`: called after the timed steps
        while the sequences are still held."""
        held = min(context, W) if W else context
        eng = engine or Engine(model, max_tokens=batch * (round_up(held) + PAGE), max_slots=batch, freeze_gc=True)
        plen = max(1, context - steps - warmup - 1)
        slots = [eng.alloc() for _ in range(batch)]
        chunk = 2048
        for s in slots:                                  # prompt by prompt, in chunks
            ids = torch.randint(0, V, (plen,), generator=gen).tolist()
            for c0 in range(0, plen, chunk):
                part = ids[c0:c0 + chunk]
                last = c0 + chunk >= plen
                lg = eng.step([SeqInput(s, part, [len(part) - 1] if last else [])])
        # every sequence goes on with the same first token; from here the steps are the generation
        # loop's own (`BatchRun.advance`: the next step is launched with the drawn tokens still on
        # the device, then the host reads the tokens of the step before)
        first = sampler.sample(lg, [0], [0]) * batch
        lg = eng.step([SeqInput(s, [t], [0]) for s, t in zip(slots, first)])
        run = BatchRun(eng, sampler, accept=lambda i, t: False, max_tokens=1 << 30, run_ahead=True)
        run.resume(list(range(batch)), lg, slots=slots)
        for _ in range(warmup):
            run.advance()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            run.advance()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        ctx_mid = plen + warmup + steps // 2
        extra = then(eng, [run.slots[i] for i in range(batch)]) if then is not None else None
        run.release()
        if engine is None:
            eng.close()
        return (dt / steps, ctx_mid) if then is None else (dt / steps, ctx_mid, extra)

    def kernels_one_by_one(eng, slots):
        """The kernels of one decode step, each kind by itself: one more step is run with every call
        into the kernels' Python face noted (function and arguments, layer after layer), then the calls
        of each kind are captured as a graph of their own (every layer's launch of that kernel, each on
        its own weights and cache, so that nothing is warm that the step would not find warm) and the
        graph is timed with events.  Bytes are what the kernel has to read once: its weight, or the
        keys and values of the live sequences."""
        from torchless_rs_amd.kernels import ops as K
        names = ("embed", "rmsnorm", "add_rmsnorm", "qkv_rope_commit", "rope_commit", "attention", "gemm_bf16_norm",
                 "gemm_bf16", "gemm_mid_bf16", "gemm", "gemm_library", "add_partials", "gather_rows", "silu_mul_pairs")
        real = {n: getattr(K, n) for n in names}
        tape = []
        depth = [0]

        def noted(name):
            def call(*a, **k):
                if depth[0] == 0:               # (a face that calls another face counts once)
                    tape.append((name, a, k))
                depth[0] += 1
                try:
                    return real[name](*a, **k)
                finally:
                    depth[0] -= 1
            return call

        use_graphs, eng.use_graphs = eng.use_graphs, False
        for n in names:
            setattr(K, n, noted(n))
        try:
            ctx, want_rows, n_want = eng.build_context([SeqInput(s, [0], [0]) for s in slots])
            eng.model.forward(ctx, eng.runs, want_rows, n_want)
        finally:
            for n, f in real.items():
                setattr(K, n, f)
            eng.use_graphs = use_graphs
        torch.cuda.synchronize()
        held_rows = sum(min(int(n), W) if W else int(n) for n in ctx.host["len_after"])

        def kind_and_bytes(name, a, k):
            if name == "attention":
                return "attention", held_rows * 2 * nkv * d * 2
            w = next((t for t in a[:3] if isinstance(t, torch.Tensor) and t.dim() == 2 and t.dtype == torch.bfloat16
                      and t.shape[0] > 64), None)
            if name in ("qkv_rope_commit", "gemm_bf16_norm", "gemm_bf16", "gemm_mid_bf16", "gemm", "gemm_library") and w is not None:
                label = {(nq + 2 * nkv) * d: "qkv", 2 * I: "gate_up", V: "head"}.get(w.shape[0])
                if label is None:
                    label = "o" if w.shape[1] == nq * d else "down"
                if name == "qkv_rope_commit":
                    label = "qkv_rope_commit"
                return label, w.numel() * 2
            return name, 0

        kinds = {}
        for name, a, k in tape:
            kind, nbytes = kind_and_bytes(name, a, k)
            kinds.setdefault(kind, {"calls": [], "bytes": 0})
            kinds[kind]["calls"].append((real[name], a, k))
            kinds[kind]["bytes"] += nbytes
        out, total = {}, 0.0
        side = torch.cuda.Stream()
        for kind, rec in kinds.items():
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for f, a, k in rec["calls"]:
                    f(*a, **k)
            torch.cuda.synchronize()
            best = float("inf")
            for _ in range(5):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                graph.replay()
                e1.record()
                e1.synchronize()
                best = min(best, e0.elapsed_time(e1) * 1e3)
            n = len(rec["calls"])
            out[f"{kind}_us"] = round(best / n, 2)
            out[f"{kind}_calls"] = n
            if rec["bytes"]:
                out[f"{kind}_frac"] = round(rec["bytes"] / (best * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)
            total += best
            del graph
        out["sum_us"] = round(total, 1)
        return out

    def run_workload(mdl, mcfg, n_layers, batch, lo, hi, new_tokens, temperature, seed):
        """`batch` requests with prompt lengths uniform in [lo, hi] and `new_tokens` new tokens each,
        through `generate_until_eos` as a user would call it: prompts in one step, then one token a
        step.  The prefill ends and decoding begins when the host holds the first token."""
        from torchless_rs_amd import generate_until_eos
        g = torch.Generator().manual_seed(seed)
        lens = torch.randint(lo, hi + 1, (batch,), generator=g).tolist()
        prompts = [torch.randint(0, mcfg.vocab_size, (n,), generator=g).tolist() for n in lens]
        win = mcfg.sliding_window
        held = [min(n + new_tokens, win) if win else n + new_tokens for n in lens]
        eng = Engine(mdl, max_tokens=sum(round_up(h) + PAGE for h in held), max_slots=batch, freeze_gc=True)
        scfg = SamplingConfig(temperature=temperature, seed=seed) if temperature > 0 else SamplingConfig.greedy()
        stamps = []

        def on_token(i, t):
            if not stamps:
                torch.cuda.synchronize()
                stamps.append(time.perf_counter())

        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = generate_until_eos(eng, prompts, scfg, max_tokens=new_tokens, on_token=on_token)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        eng.close()
        assert all(len(r.tokens) == new_tokens for r in out)
        t_pre, t_dec = stamps[0] - t0, t2 - stamps[0]
        per_l = ((mcfg.num_attention_heads + 2 * mcfg.num_key_value_heads) * mcfg.head_dim * mcfg.hidden_size
                 + mcfg.hidden_size * mcfg.num_attention_heads * mcfg.head_dim
                 + 3 * mcfg.intermediate_size * mcfg.hidden_size)
        w_bytes = 2 * (n_layers * per_l + mcfg.vocab_size * mcfg.hidden_size)
        kv_tok = 2 * mcfg.num_key_value_heads * mcfg.head_dim * 2 * n_layers
        steps = new_tokens - 1                           # the first token comes out of the prompts' step
        ctx = [n + new_tokens / 2 for n in lens]
        step_bytes = w_bytes + sum((min(c, win) if win else c) for c in ctx) * kv_tok
        gbs = step_bytes * steps / t_dec / 1e9
        return {"batch": batch, "prompt_tokens": sum(lens), "new_tokens": new_tokens, "temperature": temperature,
                "prefill_tok_s": round(sum(lens) / t_pre, 1), "prefill_ms": round(t_pre * 1e3, 1),
                "decode_tok_s": round(batch * steps / t_dec, 1), "decode_ms_per_step": round(t_dec / steps * 1e3, 3),
                "roofline_frac": round(gbs / HBM_PEAK_GBS, 4), "achieved_GBs": round(gbs, 1)}

    if args.only == "decode":
        sec, _ = run_decode(args.batch, args.context, args.steps, args.warmup)
        print(f"[bench] decode b{args.batch}: {args.batch / sec:.1f} tok/s, {sec * 1e3:.3f} ms/step",
              file=sys.stderr, flush=True)
        return 0

    # prefill of one prompt
    T = args.prefill_tokens
    eng = Engine(model, max_tokens=T + PAGE, max_slots=1, freeze_gc=True)
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
    eng.close()
    pre = min(pre_ms)
    attn_flops = sum(4 * nq * d * min(p + 1, W or (p + 1)) for p in range(T)) * L
    pre_flops = 2 * T * (L * per_layer) + 2 * V * H + attn_flops
    prefill = {"value": round(T / (pre / 1e3), 1), "tokens": T, "ms": round(pre, 3),
               "frac": round(pre_flops / (pre / 1e3) / (PEAK_TFLOPS["bf16"] * 1e12), 4)}
    print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)
    if args.only == "prefill":
        return 0

    if args.no_kernels:
        (sec, ctx_mid), kernels = run_decode(args.batch, args.context, args.steps, args.warmup), {}
    else:
        sec, ctx_mid, kernels = run_decode(args.batch, args.context, args.steps, args.warmup, then=kernels_one_by_one)
        kernels["step_us"] = round(sec * 1e6, 1)
        print(f"[bench] kernels of the step one by one {kernels}", file=sys.stderr, flush=True)
    held = min(ctx_mid, W) if W else ctx_mid
    step_bytes = weight_bytes + args.batch * held * kv_per_token
    achieved = step_bytes / sec / 1e9
    value = args.batch / sec
    print(f"[bench] decode b{args.batch}: {value:.1f} tok/s, {sec * 1e3:.3f} ms/step", file=sys.stderr,
          flush=True)
    points = {}
    if not args.no_points:
        for b in (1, 64):
            s_b, _ = run_decode(b, args.context, max(32, args.steps), 4)
            points[f"decode_b{b}"] = round(b / s_b, 1)
            print(f"[bench] decode b{b}: {b / s_b:.1f} tok/s", file=sys.stderr, flush=True)

    workloads = {}
    if args.workload == "baseline" and not args.no_workloads:
        if args.shape == "7b-v0.1":                     # the model that is loaded: prompts U[128, 2048], 256 new tokens
            for b in (1, 8, 64):
                workloads[f"7b-v0.1_b{b}"] = run_workload(model, cfg, L, b, 128, 2048, 256, 0.0, seed=5)
                print(f"[bench] workload 7b-v0.1 b{b}: {workloads[f'7b-v0.1_b{b}']}", file=sys.stderr, flush=True)
        del model
        torch.cuda.empty_cache()
        for key, b, lo, hi, new, temp, seed in (("7b-v0.3", 8, 1024, 16384, 128, 0.0, 6),
                                                ("nemo-12b", 16, 256, 8192, 128, 0.7, 7)):
            wcfg = config_from_dict(dict(SHAPES[key][1], architectures=["MistralForCausalLM"]))
            wt = random_tensors(model_spec_for(wcfg).weight_specs(), seed=seed, std=0.02, dtype=torch.bfloat16, device=dev)
            wm = model_from_tensors(wcfg, wt, "bfloat16", dev, tiled_copies=not args.no_tiled_copies)
            del wt
            workloads[f"{key}_b{b}"] = run_workload(wm, wcfg, wcfg.num_hidden_layers, b, lo, hi, new, temp, seed)
            print(f"[bench] workload {key} b{b}: {workloads[f'{key}_b{b}']}", file=sys.stderr, flush=True)
            del wm
            torch.cuda.empty_cache()
        model = None

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
    if kernels:
        out["kernels"] = kernels
    if workloads:
        # flat: decoded and prefilled tokens a second and the decode steps' share of the HBM roofline
        out["workloads"] = {f"{k}_{f}": v[f] for k, v in workloads.items()
                            for f in ("decode_tok_s", "prefill_tok_s", "roofline_frac")}
        out["workload_details"] = workloads
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
