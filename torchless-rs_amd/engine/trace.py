"""Trace replay: feed given token ids through the model step by step and write
the logits.  Nothing is sampled.  It drives the same model, step function,
cache and kernels as generation does.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input carries one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

A request is given a slot when its id is first seen and gives it back when
the id appears in `end`.  For a step in which logits are wanted,
`<out>/<step>.f32` receives them as little-endian float32 [wanted, vocab], in
the order of the entries and of their `want` lists.  After every step the
line `done <step>` is printed and flushed.  When the input ends (or the run
fails) `<out>/index.json` lists, for every step that wrote logits, which row
of its file belongs to which request and position:

    {"vocab": V, "steps": {"0": [{"id": "a", "position": 0, "row": 0}, ...]}}
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Dict

import numpy as np


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder that receives <step>.f32")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to whole pages of the cache, 64)")
    args = ap.parse_args(argv)

    print("[trace_run] loading torch and the kernels", file=sys.stderr, flush=True)
    from .engine import Engine, load_model

    os.makedirs(args.out, exist_ok=True)
    model = load_model(args.model, args.dtype, "cuda:0")
    from ..kernels.page import PAGE
    engine = Engine(model, max_tokens=max(args.max_tokens, PAGE))
    print("[trace_run] ready", file=sys.stderr, flush=True)

    slot_of: Dict[str, int] = {}
    index: Dict[str, list] = {}
    try:
        _replay(engine, args.out, slot_of, index)
    finally:
        with open(os.path.join(args.out, "index.json"), "w") as f:
            json.dump({"vocab": engine.vocab_size, "steps": index}, f)
    return 0


def _replay(engine, out_dir: str, slot_of: Dict[str, int], index: Dict[str, list]) -> None:
    import torch
    from .engine import SeqInput
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        batch, rows = [], []
        for e in rec.get("entries", []):
            rid = str(e["id"])
            if rid not in slot_of:
                slot_of[rid] = engine.alloc()
            batch.append(SeqInput(slot_of[rid], e["tokens"], e.get("want", [])))
            held = engine.length(slot_of[rid])
            rows += [{"id": rid, "position": held + int(w), "row": len(rows) + k}
                     for k, w in enumerate(e.get("want", []))]
        if batch:
            logits = engine.step(batch)
            if logits.shape[0]:
                arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                with open(os.path.join(out_dir, f"{step}.f32"), "wb") as f:
                    f.write(np.ascontiguousarray(arr).tobytes())
                index[str(step)] = rows
            else:
                torch.cuda.synchronize()
        for rid in rec.get("end", []):
            rid = str(rid)
            if rid in slot_of:
                engine.free(slot_of.pop(rid))
        print(f"done {step}", flush=True)


if __name__ == "__main__":
    sys.exit(main())
