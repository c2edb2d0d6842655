"""The library's entry point in Python.

The reference's library use is load -> model -> state -> generate
(src/lib.rs:28-91): `Parameters::load(path)`, `Mistral::load(params)`,
`InferenceState::new(config)`, `generate(&model, &mut state, token, &cfg)`,
`generate_until_eos(...)`.  The same steps here:

    model  = load_model("dir", dtype="bfloat16")           # config.json picks the class
    engine = Engine(model, max_tokens=8192)                 # cache sized in positions
    out    = generate_until_eos(engine, prompts, SamplingConfig.greedy(), max_tokens=32,
                                eos_token_ids=[2])
    out[0].tokens, out[0].stopped_at_eos
"""
from __future__ import annotations

from typing import Callable, List, Optional, Sequence

from .engine.engine import Engine, SeqInput, load_model, model_from_tensors
from .engine.generate import GenerationResult, generate as _generate
from .sampling.config import SamplingConfig


def generate_until_eos(engine: Engine, prompts: Sequence[Sequence[int]], config: SamplingConfig,
                       max_tokens: int, eos_token_ids: Sequence[int] = (),
                       on_token: Optional[Callable[[int, int], None]] = None,
                       max_batch: Optional[int] = None) -> List[GenerationResult]:
    """Generate for each prompt (a list of token ids) until `max_tokens` tokens
    are out or one of `eos_token_ids` is drawn; the stop id is not returned."""
    from .sampling.sampler import Sampler
    return _generate(engine, Sampler(config, engine.device), prompts, max_tokens, eos_token_ids,
                     max_batch, on_token)


def default_max_tokens(max_seq_len: int) -> int:
    """The tokens to generate when the caller names no number: a quarter of the context, at
    least 1024 (2048 from a context of 4096 on) and at most 32768 (`resolve_max_tokens`,
    src/main.rs:140-153 of the reference)."""
    low = 2048 if max_seq_len >= 4096 else 1024
    return min(max(max_seq_len // 4, low), 32768)


def generate(model_dir: str, prompts: Sequence[Sequence[int]], max_tokens: Optional[int] = None,
             temperature: float = 0.7, top_k: Optional[int] = None, top_p: Optional[float] = None,
             seed: int = 0, stop_ids: Optional[Sequence[int]] = None, dtype: str = "bfloat16",
             max_seq_len: Optional[int] = None, device: str = "cuda:0",
             freeze_gc: bool = False) -> List[GenerationResult]:
    """Load the model folder and generate for every prompt.  `stop_ids` None
    means config.json's eos_token_id, if it has one; `max_tokens` None means `default_max_tokens`
    of the context, cut to the room behind the longest prompt.  The engine made for the call is closed
    when it ends, its cache given back.  `freeze_gc`: see `Engine`."""
    model = load_model(model_dir, dtype, device)
    if stop_ids is None:
        stop_ids = list(getattr(model.config, "eos_token_ids", []) or [])
    if max_tokens is None:
        # the reference's default, and no more than the context has room for behind the longest prompt
        context = max_seq_len or getattr(model.config, "max_position_embeddings", None) or 4096
        max_tokens = max(1, min(default_max_tokens(context), context - max(len(p) for p in prompts)))
    longest = max(len(p) for p in prompts) + max_tokens
    # the longest sequence allowed: the model's max_position_embeddings unless the caller sets
    # another limit, which may exceed it with a warning (src/main.rs:111-137 of the reference)
    trained = getattr(model.config, "max_position_embeddings", None)
    if max_seq_len is not None and trained and max_seq_len > trained:
        import sys
        sys.stderr.write(f"WARNING: --max-seq-len {max_seq_len} exceeds the model's trained context "
                         f"length ({trained}).\n")
    limit = max_seq_len if max_seq_len is not None else trained
    if limit is not None and longest > limit:
        raise ValueError(f"a request needs {longest} positions, " +
                         (f"--max-seq-len allows {limit}" if max_seq_len is not None else
                          f"the model's max_position_embeddings is {limit}; raise --max-seq-len to go beyond"))
    from .kernels.page import round_up
    per_seq = round_up(longest)
    engine = Engine(model, max_tokens=per_seq * len(prompts), max_slots=len(prompts), freeze_gc=freeze_gc)
    try:
        cfg = SamplingConfig(temperature=temperature, top_k=top_k, top_p=top_p, seed=seed)
        return generate_until_eos(engine, prompts, cfg, max_tokens, stop_ids)
    finally:
        engine.close()
