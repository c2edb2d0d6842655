"""The command line, in the manner of the reference's `torchless`
(src/main.rs:28-91 for the options, :179-345 for how they are read):

    torchless [OPTIONS] <model_path> [prompt]

The prompt is a list of token ids ("1 5 17" or "1,5,17"); several prompts are
separated by ';' and are served as batches.  Options with the reference's
names and meanings: --max-tokens N, --max-seq-len N, --temperature T (default
0.7; 0 = greedy), --top-k K, --top-p P, --debug, --help/-h.  Ours: --seed S,
--dtype bfloat16|float32, --stop-ids "a,b" (default: config.json's
eos_token_id; "none" disables), --random-weights with --config FILE, --std,
--norm-std: write a randomly initialised model folder at <model_path> first.
An unknown option or a missing value is an error with exit code 1.
"""
from __future__ import annotations

import json
import sys
import time
from typing import List, Optional

USAGE = """Usage: {prog} [OPTIONS] <model_path> [prompt]

Options:
  --max-tokens <N>      Maximum tokens to generate per prompt (default: a quarter of
                        --max-seq-len, from 1024 to 32768, within the context's room)
  --max-seq-len <N>     Maximum sequence length / context window
                        (default: the model's max_position_embeddings)
  --temperature <T>     Sampling temperature (default: 0.7)
                        0.0 = greedy/deterministic, 0.7 = balanced, 1.0+ = creative
  --top-k <K>           Top-k sampling: only consider the top K tokens
  --top-p <P>           Nucleus sampling: keep smallest set of tokens with
                        cumulative probability >= P
  --seed <S>            Seed of the sampler (default: 0)
  --dtype <TYPE>        bfloat16 (default) or float32
  --stop-ids <IDS>      Token ids that end a sequence (default: config.json's eos_token_id;
                        "none" for no stop ids)
  --random-weights      Write a randomly initialised model into <model_path> first
  --config <FILE>       config.json to use with --random-weights
  --std <S>             Standard deviation of random matrices (default: 0.02)
  --norm-std <S>        Standard deviation of random norm weights around 1 (default: 0)
  --debug               Enable debug output
  --help                Show this help message

The prompt is a list of token ids: "1 5 17" or "1,5,17"; ';' separates prompts.

Examples:
  {prog} model_dir "1 733 4123"
  {prog} --temperature 0 --max-tokens 32 model_dir "1,733,4123;1,28705"
  {prog} --random-weights --config config.json --seed 5 new_dir "1 2 3"
"""

_VALUE_OPTS = {"--max-tokens": int, "--max-seq-len": int, "--temperature": float, "--top-k": int,
               "--top-p": float, "--seed": int, "--dtype": str, "--stop-ids": str, "--config": str,
               "--std": float, "--norm-std": float}
_FLAGS = {"--debug", "--random-weights"}


def parse_ids(text: str) -> List[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def parse_args(argv: List[str], prog: str = "torchless"):
    """Returns (options, positionals) or exits as the reference does."""
    opts = {"--max-tokens": None, "--max-seq-len": None, "--temperature": 0.7, "--top-k": None,
            "--top-p": None, "--seed": 0, "--dtype": "bfloat16", "--stop-ids": None, "--config": None,
            "--std": 0.02, "--norm-std": 0.0, "--debug": False, "--random-weights": False}
    pos: List[str] = []
    i = 0
    while i < len(argv):
        a = argv[i]
        if a in ("--help", "-h"):
            sys.stderr.write(USAGE.format(prog=prog))
            raise SystemExit(0)
        if a in _FLAGS:
            opts[a] = True
            i += 1
        elif a in _VALUE_OPTS:
            if i + 1 >= len(argv):
                sys.stderr.write(f"Error: {a} requires a value\n")
                raise SystemExit(1)
            try:
                opts[a] = _VALUE_OPTS[a](argv[i + 1])
            except ValueError:
                sys.stderr.write(f"Error: invalid {a} value '{argv[i + 1]}'\n")
                raise SystemExit(1)
            i += 2
        elif a.startswith("-"):
            sys.stderr.write(f"Error: unknown option '{a}'\nUse --help for usage information.\n")
            raise SystemExit(1)
        else:
            pos.append(a)
            i += 1
    return opts, pos


def main(argv: Optional[List[str]] = None, prog: str = "torchless") -> int:
    opts, pos = parse_args(list(sys.argv[1:] if argv is None else argv), prog)
    if not pos:
        sys.stderr.write(USAGE.format(prog=prog))
        return 1
    model_path = pos[0]
    prompt_text = " ".join(pos[1:])
    if opts["--dtype"] not in ("bfloat16", "bf16", "float32", "fp32", "f32"):
        sys.stderr.write(f"Error: invalid --dtype value '{opts['--dtype']}'. Use bfloat16 or float32\n")
        return 1
    if opts["--random-weights"]:
        if not opts["--config"]:
            sys.stderr.write("Error: --random-weights requires --config <FILE>\n")
            return 1
        import torch
        from .weights.random_init import write_random_model
        with open(opts["--config"]) as f:
            cfg = json.load(f)
        st = torch.float32 if opts["--dtype"] in ("float32", "fp32", "f32") else torch.bfloat16
        write_random_model(model_path, cfg, opts["--seed"], opts["--std"], opts["--norm-std"], st)
        sys.stderr.write(f"Wrote random weights (seed {opts['--seed']}) to {model_path}\n")
        if not prompt_text:
            return 0
    if not prompt_text:
        sys.stderr.write("Error: no prompt given (a list of token ids)\n")
        return 1
    try:
        prompts = [parse_ids(p) for p in prompt_text.split(";") if p.strip()]
    except ValueError:
        sys.stderr.write("Error: the prompt must be token ids, e.g. \"1 5 17\"\n")
        return 1
    if not prompts or any(not p for p in prompts):
        sys.stderr.write("Error: empty prompt\n")
        return 1
    stop = opts["--stop-ids"]
    stop_ids = None if stop is None else ([] if stop.strip().lower() == "none" else parse_ids(stop))
    max_tokens = opts["--max-tokens"]            # None: the default follows the context (api.default_max_tokens)

    from .api import generate
    t0 = time.time()
    if opts["--debug"]:
        sys.stderr.write(f"Loading {model_path} ({opts['--dtype']})\n")
    try:
        results = generate(model_path, prompts, max_tokens=max_tokens, temperature=opts["--temperature"],
                           top_k=opts["--top-k"], top_p=opts["--top-p"], seed=opts["--seed"],
                           stop_ids=stop_ids, dtype=opts["--dtype"], max_seq_len=opts["--max-seq-len"],
                           freeze_gc=True)
    except (ValueError, OSError, RuntimeError, KeyError) as e:
        # a request beyond --max-seq-len or the cache, a token id outside the vocabulary, a folder
        # that is not a model, weights that do not fit the configuration, no GPU
        if opts["--debug"]:
            raise
        sys.stderr.write(f"Error: {e}\n")
        return 1
    dt = time.time() - t0
    for r in results:
        print(" ".join(str(t) for t in r.tokens))
    n = sum(len(r.tokens) for r in results)
    sys.stderr.write(f"{n} tokens for {len(results)} prompt(s) in {dt:.2f} s "
                     f"(finish: {', '.join(r.finish_reason for r in results)})\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
